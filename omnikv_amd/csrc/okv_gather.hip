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

// ---------------------------------------------------------------------------
// Incremental staging of the host tier.  The rows staged on the device for a group of sparse
// layers are a SET (attention does not care about row order): a new selection keeps the rows it
// shares with the previous one where they are and fetches only the others into the slots the
// dropped rows free.  One workgroup plans the exchange for the whole group:
//   slot_tok[s]  token whose row sits in slot s (-1: empty)        k entries, in / out
//   slot_of[t]   slot of token t (-1: not staged)                  num_tokens entries, in / out
//   fetch_tok / fetch_slot / fetch_count   the rows to copy and where to, in ascending token order
// Phases are separated by workgroup barriers; pairing the r-th new token with the r-th free slot
// makes the result independent of timing.
__global__ __launch_bounds__(1024) void offload_plan_kernel(const int32_t* __restrict__ idx_new, int k,
                                                            int32_t* __restrict__ slot_tok,
                                                            int32_t* __restrict__ slot_of, int num_tokens,
                                                            int32_t* __restrict__ fetch_tok,
                                                            int32_t* __restrict__ fetch_slot,
                                                            int32_t* __restrict__ fetch_count) {
  extern __shared__ uint32_t plan_lds[];  // [ceil(k/32)] slots that stay, then two 1024-entry scans
  const int words = (k + 31) / 32;
  uint32_t* kept = plan_lds;
  int* scan_a = reinterpret_cast<int*>(plan_lds + words);
  int* scan_b = scan_a + 1024;
  const int tid = threadIdx.x;
  for (int w = tid; w < words; w += 1024) kept[w] = 0u;
  __syncthreads();
  const int per = (k + 1023) / 1024;
  const int lo = min(tid * per, k), hi = min(lo + per, k);
  int n_fetch = 0;
  for (int j = lo; j < hi; ++j) {
    const int t = idx_new[j];
    const int s = (unsigned)t < (unsigned)num_tokens ? slot_of[t] : -1;
    if (s >= 0 && s < k) atomicOr(&kept[s >> 5], 1u << (s & 31));
    else if ((unsigned)t < (unsigned)num_tokens) ++n_fetch;
  }
  __syncthreads();
  int n_free = 0;
  for (int s = lo; s < hi; ++s) n_free += !((kept[s >> 5] >> (s & 31)) & 1u);
  scan_a[tid] = n_fetch;
  scan_b[tid] = n_free;
  __syncthreads();
  for (int o = 1; o < 1024; o <<= 1) {  // inclusive scans of both counts
    const int a = tid >= o ? scan_a[tid - o] : 0, b = tid >= o ? scan_b[tid - o] : 0;
    __syncthreads();
    scan_a[tid] += a;
    scan_b[tid] += b;
    __syncthreads();
  }
  const int m = min(scan_a[1023], scan_b[1023]);  // equal unless the caller's state is inconsistent
  int pa = scan_a[tid] - n_fetch, pb = scan_b[tid] - n_free;
  for (int j = lo; j < hi; ++j) {
    const int t = idx_new[j];
    if ((unsigned)t < (unsigned)num_tokens) {
      const int s = slot_of[t];
      if (!(s >= 0 && s < k)) {
        if (pa < m) fetch_tok[pa] = t;
        ++pa;
      }
    }
  }
  for (int s = lo; s < hi; ++s)
    if (!((kept[s >> 5] >> (s & 31)) & 1u)) {
      if (pb < m) fetch_slot[pb] = s;
      ++pb;
    }
  __syncthreads();  // both lists are complete (and nobody reads slot_of any more) before the maps change
  for (int r = tid; r < m; r += 1024) {
    const int s = fetch_slot[r], t_new = fetch_tok[r], t_old = slot_tok[s];
    if ((unsigned)t_old < (unsigned)num_tokens) slot_of[t_old] = -1;  // dropped tokens and fetched ones are disjoint
    slot_of[t_new] = s;
    slot_tok[s] = t_new;
  }
  if (tid == 0) fetch_count[0] = m;
}

// dst row fetch_slot[r] = src row fetch_tok[r] for r < fetch_count[0]; rows of row_bytes bytes (a
// multiple of 16), 16 bytes per thread.  The source is usually pinned host memory read over the
// host link, so the grid is small: a few waves with loads in flight saturate the link, and the
// CUs stay free for the kernels of the other streams.
__global__ __launch_bounds__(256) void fetch_rows_kernel(const char* __restrict__ src, int64_t row_bytes,
                                                         const int32_t* __restrict__ fetch_tok,
                                                         const int32_t* __restrict__ fetch_slot,
                                                         const int32_t* __restrict__ fetch_count, int max_rows,
                                                         char* __restrict__ dst) {
  const int n = min(fetch_count[0], max_rows);
  const int upr = (int)(row_bytes / 16);
  const int64_t units = (int64_t)n * upr;
  for (int64_t u = (int64_t)blockIdx.x * 256 + threadIdx.x; u < units; u += (int64_t)gridDim.x * 256) {
    const int r = (int)(u / upr), x = (int)(u % upr);
    const uint4* sp = reinterpret_cast<const uint4*>(src + (int64_t)fetch_tok[r] * row_bytes) + x;
    uint4* dp = reinterpret_cast<uint4*>(dst + (int64_t)fetch_slot[r] * row_bytes) + x;
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

int okv_offload_plan(const int32_t* idx_new, int32_t k, int32_t* slot_tok, int32_t* slot_of,
                     int32_t num_tokens, int32_t* fetch_tok, int32_t* fetch_slot, int32_t* fetch_count,
                     okv_stream_t stream) {
  OKV_REQUIRE(idx_new && slot_tok && slot_of && fetch_tok && fetch_slot && fetch_count, OKV_ERR_INVALID,
              "NULL argument");
  OKV_REQUIRE(k >= 1 && num_tokens >= 1, OKV_ERR_INVALID, "k and num_tokens must be >= 1");
  OKV_REQUIRE(k <= (1 << 18), OKV_ERR_UNSUPPORTED, "at most %d staged rows per group", 1 << 18);
  const size_t lds = (size_t)((k + 31) / 32) * 4 + 2 * 1024 * sizeof(int);
  hipLaunchKernelGGL(offload_plan_kernel, dim3(1), dim3(1024), lds, (hipStream_t)stream, idx_new, k, slot_tok,
                     slot_of, num_tokens, fetch_tok, fetch_slot, fetch_count);
  OKV_HIP_CHECK(hipGetLastError());
  return OKV_OK;
}

int okv_offload_fetch(const void* src, int64_t row_bytes, const int32_t* fetch_tok, const int32_t* fetch_slot,
                      const int32_t* fetch_count, int32_t max_rows, void* dev_dst, okv_stream_t stream) {
  OKV_REQUIRE(src && fetch_tok && fetch_slot && fetch_count && dev_dst, OKV_ERR_INVALID, "NULL argument");
  OKV_REQUIRE(row_bytes > 0 && row_bytes % 16 == 0, OKV_ERR_INVALID, "row_bytes must be a positive multiple of 16");
  OKV_REQUIRE(((uintptr_t)src & 15) == 0 && ((uintptr_t)dev_dst & 15) == 0, OKV_ERR_INVALID,
              "src and dev_dst must be 16-byte aligned");
  OKV_REQUIRE(max_rows >= 0, OKV_ERR_INVALID, "max_rows must be >= 0");
  if (max_rows == 0) return OKV_OK;
  int64_t blocks = ((int64_t)max_rows * (row_bytes / 16) + 255) / 256;
  if (blocks > 64) blocks = 64;
  hipLaunchKernelGGL(fetch_rows_kernel, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream, (const char*)src,
                     row_bytes, fetch_tok, fetch_slot, fetch_count, max_rows, (char*)dev_dst);
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
