// Row gathers: device-side materialised gather of selected K/V rows, and the
// host-side staging of selected rows from pinned memory for the offload tier.
#include <string.h>

#include <thread>
#include <vector>

#include "okv_internal.h"

namespace okv {

// One thread moves 16 bytes at a time, grid-stride.  grid (blocks, batch).
__global__ __launch_bounds__(256) void gather_rows_kernel(RowList rows, int hkv, int esize,
                                                          char* __restrict__ dst,
                                                          int64_t dst_token_stride,
                                                          int64_t dst_head_stride,
                                                          int64_t dst_batch_stride) {
  const int b = blockIdx.y;
  const int n = rl_main_len(rows, b);
  const int upr = kHeadDimBytes16(esize);
  const int per_token = hkv * upr;
  const int64_t units = (int64_t)n * per_token;
  for (int64_t u = (int64_t)blockIdx.x * 256 + threadIdx.x; u < units; u += (int64_t)gridDim.x * 256) {
    const int64_t j = u / per_token;
    const int rem = (int)(u % per_token);
    const int g = rem / upr, x = rem % upr;
    bool in_tail;
    int64_t so = rl_row_offset(rows, b, (int)j, n, &in_tail) + (int64_t)g * rows.head_stride;
    int64_t dofs = (int64_t)b * dst_batch_stride + j * dst_token_stride + (int64_t)g * dst_head_stride;
    const uint4* sp = reinterpret_cast<const uint4*>((const char*)rows.k_base + so * esize) + x;
    uint4* dp = reinterpret_cast<uint4*>(dst + dofs * esize) + x;
    *dp = *sp;
  }
}

}  // namespace okv

using namespace okv;

extern "C" {

int okv_gather_rows(const void* src_base, const okv_kv_layout_t* layout, const int32_t* idx,
                    int64_t idx_stride, const int32_t* sel_lens, int32_t max_sel_len,
                    int32_t batch, void* dst, int64_t dst_token_stride, int64_t dst_head_stride,
                    int64_t dst_batch_stride, okv_stream_t stream) {
  int rc = validate_layout(layout, src_base, src_base);
  if (rc) return rc;
  OKV_REQUIRE(idx && dst, OKV_ERR_INVALID, "idx or dst is NULL");
  OKV_REQUIRE(batch >= 1 && max_sel_len >= 0, OKV_ERR_INVALID, "bad batch or length");
  OKV_REQUIRE(idx_stride >= max_sel_len, OKV_ERR_INVALID, "idx_stride < max_sel_len");
  OKV_REQUIRE(((uintptr_t)dst & 15) == 0 && dst_token_stride % 8 == 0 &&
                  dst_head_stride % 8 == 0 && dst_batch_stride % 8 == 0,
              OKV_ERR_INVALID, "dst must be 16-byte aligned with strides multiple of 8");
  if (max_sel_len == 0) return OKV_OK;
  const int esize = layout->dtype == OKV_F32 ? 4 : 2;
  RowList r;
  memset(&r, 0, sizeof(r));
  r.k_base = src_base;
  r.token_stride = layout->token_stride;
  r.head_stride = layout->head_stride;
  r.batch_stride = layout->batch_stride;
  rl_set_pages(&r, layout->page_table, layout->page_size, layout->page_table_stride, layout->page_stride);
  r.idx = idx;
  r.idx_stride = idx_stride;
  r.main_lens = sel_lens;
  r.max_main_len = max_sel_len;
  const int64_t units = (int64_t)max_sel_len * layout->num_kv_heads * kHeadDimBytes16(esize);
  int64_t blocks = (units + 255) / 256;
  // A source in host memory (the zero-copy offload tier) is read over the host link: a few
  // waves with loads in flight saturate it, and a grid of the usual size would sit on every
  // CU's wave slots waiting for the link while the kernels of the other streams starve.
  hipPointerAttribute_t attr;
  if (hipPointerGetAttributes(&attr, src_base) == hipSuccess) {
    if (attr.type == hipMemoryTypeHost && blocks > 64) blocks = 64;
  } else {
    (void)hipGetLastError();  // unregistered pointer: not ours to judge
  }
  dim3 grid((unsigned)blocks, batch);
  hipLaunchKernelGGL(gather_rows_kernel, grid, dim3(256), 0, (hipStream_t)stream, r,
                     layout->num_kv_heads, esize, (char*)dst, dst_token_stride, dst_head_stride,
                     dst_batch_stride);
  OKV_HIP_CHECK(hipGetLastError());
  return OKV_OK;
}

int okv_offload_stage(const void* host_src, int64_t row_bytes, const int32_t* host_idx,
                      int32_t n_rows, void* host_staging, int32_t host_threads, void* dev_dst,
                      okv_stream_t copy_stream, void* done_event) {
  OKV_REQUIRE(host_src && host_idx && host_staging && dev_dst, OKV_ERR_INVALID, "NULL argument");
  OKV_REQUIRE(row_bytes > 0 && n_rows >= 0, OKV_ERR_INVALID, "bad row_bytes or n_rows");
  OKV_REQUIRE(host_threads >= 1 && host_threads <= 64, OKV_ERR_INVALID, "host_threads out of range");
  if (n_rows > 0) {
    const char* src = (const char*)host_src;
    char* stg = (char*)host_staging;
    auto pack = [&](int lo, int hi) {
      // runs of consecutive indices become one memcpy
      int i = lo;
      while (i < hi) {
        int j = i + 1;
        while (j < hi && host_idx[j] == host_idx[j - 1] + 1) ++j;
        memcpy(stg + (int64_t)i * row_bytes, src + (int64_t)host_idx[i] * row_bytes,
               (size_t)(j - i) * row_bytes);
        i = j;
      }
    };
    int nt = host_threads;
    if ((int64_t)n_rows * row_bytes < (1 << 20)) nt = 1;
    if (nt == 1) {
      pack(0, n_rows);
    } else {
      std::vector<std::thread> th;
      int per = (n_rows + nt - 1) / nt;
      for (int t = 0; t < nt; ++t) {
        int lo = t * per, hi = lo + per < n_rows ? lo + per : n_rows;
        if (lo >= hi) break;
        th.emplace_back(pack, lo, hi);
      }
      for (auto& x : th) x.join();
    }
    OKV_HIP_CHECK(hipMemcpyAsync(dev_dst, host_staging, (size_t)n_rows * row_bytes,
                                 hipMemcpyHostToDevice, (hipStream_t)copy_stream));
  }
  if (done_event) OKV_HIP_CHECK(hipEventRecord((hipEvent_t)done_event, (hipStream_t)copy_stream));
  return OKV_OK;
}

}  // extern "C"
