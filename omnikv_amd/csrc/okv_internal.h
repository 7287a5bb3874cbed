// Shared declarations of libomnikv_hip.so (gfx950 only).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>

#include <atomic>

#include "../../include/omnikv_hip.h"

namespace okv {

// ---------------------------------------------------------------- errors
void set_error(const char* fmt, ...);

#define OKV_REQUIRE(cond, code, ...) \
  do {                               \
    if (!(cond)) {                   \
      okv::set_error(__VA_ARGS__);   \
      return (code);                 \
    }                                \
  } while (0)

#define OKV_HIP_CHECK(expr)                                                      \
  do {                                                                           \
    hipError_t e_ = (expr);                                                      \
    if (e_ != hipSuccess) {                                                      \
      okv::set_error("%s failed: %s (%s:%d)", #expr, hipGetErrorString(e_),      \
                     __FILE__, __LINE__);                                        \
      return OKV_ERR_HIP;                                                        \
    }                                                                            \
  } while (0)

// ---------------------------------------------------------------- row lists
// One request's rows as the attention / scoring kernels see them: a main
// segment (all cached tokens, or the selected ones through idx) followed by an
// optional tail segment held in a separate buffer.
struct RowList {
  const void* k_base;
  const void* v_base;
  int64_t token_stride, head_stride, batch_stride;  // elements
  const int32_t* page_table;
  int32_t page_size, page_table_stride;
  int32_t page_shift;  // log2(page_size) when it is a power of two, else -1 (set by rl_set_pages)
  int64_t page_stride;
  const int32_t* idx;  // optional indirection of the main segment
  int64_t idx_stride;
  const int32_t* main_lens;  // optional per-request lengths
  int32_t max_main_len;
  const void* tail_k;
  const void* tail_v;
  int64_t tail_token_stride, tail_head_stride, tail_batch_stride;
  const int32_t* tail_lens;
  int32_t max_tail_len;
  const int32_t* score_lens;  // rows [0, score_len) are scored; 0 = no scoring
  int32_t max_score_len;
};

// token -> (page slot of its request's table, slot inside the page); shifts when page_size = 2^n
__device__ __forceinline__ int rl_page_of(const RowList& r, int t) {
  return r.page_shift >= 0 ? t >> r.page_shift : t / r.page_size;
}
__device__ __forceinline__ int rl_slot_of(const RowList& r, int t) {
  return r.page_shift >= 0 ? t & (r.page_size - 1) : t % r.page_size;
}
inline void rl_set_pages(RowList* r, const int32_t* table, int page_size, int table_stride, int64_t page_stride) {
  r->page_table = table;
  r->page_size = page_size;
  r->page_table_stride = table_stride;
  r->page_stride = page_stride;
  r->page_shift = -1;
  if (page_size > 0 && (page_size & (page_size - 1)) == 0) {
    int sh = 0;
    while ((1 << sh) < page_size) ++sh;
    r->page_shift = sh;
  }
}

__device__ __forceinline__ int rl_main_len(const RowList& r, int b) {
  return r.main_lens ? r.main_lens[b] : r.max_main_len;
}
__device__ __forceinline__ int rl_tail_len(const RowList& r, int b) {
  return r.tail_lens ? r.tail_lens[b] : r.max_tail_len;
}
__device__ __forceinline__ int rl_score_len(const RowList& r, int b) {
  int s = r.score_lens ? r.score_lens[b] : r.max_score_len;
  int m = rl_main_len(r, b);
  return s < m ? s : m;
}

// Splits tile the scored rows [0, A) and the remaining rows [A, L) separately so
// that no split straddles the scoring boundary.
__device__ __forceinline__ void rl_split_range(int split, int split_rows, int A, int L,
                                               int* begin, int* end) {
  int nA = (A + split_rows - 1) / split_rows;
  if (split < nA) {
    *begin = split * split_rows;
    int e = *begin + split_rows;
    *end = e < A ? e : A;
  } else {
    *begin = A + (split - nA) * split_rows;
    int e = *begin + split_rows;
    *end = e < L ? e : L;
  }
}
__host__ __device__ __forceinline__ int rl_num_splits(int split_rows, int A, int L) {
  return (A + split_rows - 1) / split_rows + (L - A + split_rows - 1) / split_rows;
}

// Element offset of logical row `row` (kv head 0, d 0) and which buffer it is in.
__device__ __forceinline__ int64_t rl_row_offset(const RowList& r, int b, int row,
                                                 int main_len, bool* in_tail) {
  if (row >= main_len) {
    *in_tail = true;
    return (int64_t)b * r.tail_batch_stride + (int64_t)(row - main_len) * r.tail_token_stride;
  }
  *in_tail = false;
  int t = r.idx ? r.idx[(int64_t)b * r.idx_stride + row] : row;
  if (r.page_table) {
    int page = r.page_table[(int64_t)b * r.page_table_stride + rl_page_of(r, t)];
    return (int64_t)page * r.page_stride + (int64_t)rl_slot_of(r, t) * r.token_stride;
  }
  return (int64_t)b * r.batch_stride + (int64_t)t * r.token_stride;
}

// 16-byte units in one 128-element row of `esize`-byte elements.
__host__ __device__ __forceinline__ int kHeadDimBytes16(int esize) { return 128 * esize / 16; }

// ---------------------------------------------------------------- workspace
// Partial results of the split pass, carved from the caller's workspace.
struct AttnWorkspace {
  float* part_o;    // [batch][Hq][splits][D]   normalised partial outputs
  float* part_lse;  // [batch][Hq][splits]      log2-domain log-sum-exp
  float* logits;    // [batch][Hq][score_stride] scaled logits (natural units)
  float* score_lse; // [batch][Hq]              log2-domain lse over scored rows
  int32_t max_splits;
  int32_t split_rows;
  int64_t logits_stride;
  // Raw scores need no per-head normaliser, so the split pass may fold the q heads of a kv
  // head itself and leave one logits row per kv head: a quarter of the bytes at group 4.
  int32_t group_reduce;  // 0 = one row per q head, 1 = max over the group, 2 = sum over the group
  int32_t logit_heads;   // rows of `logits` per request: Hq, or Hkv when group_reduce
};

// Kernel arguments are fetched by scalar loads that the compiler places next to their first use: a
// chain of round trips through the scalar cache at the start of a pass that lasts a few microseconds.
// Naming every field in an empty asm statement at the top makes all of them one batch of loads.
template <typename X>
__device__ __forceinline__ void fetch_now(const X& x) {
  asm volatile("" ::"s"(x));
}
__device__ __forceinline__ void fetch_args_now(const RowList& r, const AttnWorkspace& w) {
  fetch_now(r.k_base); fetch_now(r.v_base); fetch_now(r.token_stride); fetch_now(r.head_stride);
  fetch_now(r.batch_stride); fetch_now(r.page_table); fetch_now(r.page_size); fetch_now(r.page_table_stride);
  fetch_now(r.page_shift); fetch_now(r.page_stride); fetch_now(r.idx); fetch_now(r.idx_stride);
  fetch_now(r.main_lens); fetch_now(r.max_main_len); fetch_now(r.tail_k); fetch_now(r.tail_v);
  fetch_now(r.tail_token_stride); fetch_now(r.tail_head_stride); fetch_now(r.tail_batch_stride);
  fetch_now(r.tail_lens); fetch_now(r.max_tail_len); fetch_now(r.score_lens); fetch_now(r.max_score_len);
  fetch_now(w.part_o); fetch_now(w.part_lse); fetch_now(w.logits); fetch_now(w.max_splits);
  fetch_now(w.split_rows); fetch_now(w.logits_stride); fetch_now(w.group_reduce); fetch_now(w.logit_heads);
}

// Device timestamps inside the gather-mode split pass and the merge, for the timeline build only
// (-DOKV_STAMPS, libomnikv_hip_stamps.so: `build.py --stamps`; neither the product nor the measurement
// build contains them).  Thread 0 of every workgroup stores the 100 MHz wall clock at up to eight
// points; okv_stamps_read copies them out.
#ifdef OKV_STAMPS
constexpr int kStampSlots = 8, kStampBlocks = 4096;
// `arr`: a __device__ unsigned long long[kStampBlocks * kStampSlots] of the translation unit (device symbols
// are not shared between them)
#define OKV_STAMP(arr, block, i)                                                                        \
  do {                                                                                                  \
    if (threadIdx.x == 0 && (block) < okv::kStampBlocks) arr[(block) * okv::kStampSlots + (i)] = wall_clock64(); \
  } while (0)
int stamps_read_split(unsigned long long* dst, int clear);  // okv_attn_mfma.hip
#else
#define OKV_STAMP(arr, block, i) \
  do {                           \
  } while (0)
#endif

// The last W query positions of every q head riding along a dense pass (window selectors): the
// pass then also leaves, per scored split, the log-sum-exp of every (position, head) column's
// logits, which is what the first of the window selector's two passes over K computes.
constexpr int kWinCols = 64;  // columns (positions x q heads of one kv head) per kv head
struct WindowFuse {
  const void* wq;  // element (b, h, w, d) at wq + b*q_batch_stride + h*q_head_stride + w*q_pos_stride + d
  int64_t q_batch_stride, q_head_stride, q_pos_stride;
  int32_t window;
  float* part;  // [batch][Hkv][kWinCols][max_splits]  log2-domain partial log-sum-exp
  float* lse;   // [batch][Hkv][kWinCols]  the partials merged (the pass's merge launch does it)
};

#ifdef __HIPCC__
// One (request, kv head) of the window columns: the splits' partial log-sum-exps of each of the 64
// columns folded into one.  256 threads: 64 columns x 4 split lanes, independent loads.
__device__ __forceinline__ void window_lse_merge_body(const float* __restrict__ part, float* __restrict__ lse,
                                                      int bg, int num_splits, int max_splits) {
  __shared__ float sM[4][kWinCols], sD[4][kWinCols];
  const int c = threadIdx.x & 63, sl = threadIdx.x >> 6;
  const float* p = part + ((int64_t)bg * kWinCols + c) * max_splits;
  float M = -INFINITY, den = 0.f;
  constexpr int U = 8;
  for (int s0 = sl; s0 < num_splits; s0 += 4 * U) {
    float x[U];
#pragma unroll
    for (int u = 0; u < U; ++u) x[u] = s0 + 4 * u < num_splits ? p[s0 + 4 * u] : -INFINITY;
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const float mn = fmaxf(M, x[u]);
      if (mn != -INFINITY) {
        den = fmaf(den, exp2f(M - mn), exp2f(x[u] - mn));
        M = mn;
      }
    }
  }
  sM[sl][c] = M;
  sD[sl][c] = den;
  __syncthreads();
  if (sl == 0) {
    float Mt = fmaxf(fmaxf(sM[0][c], sM[1][c]), fmaxf(sM[2][c], sM[3][c]));
    float d = 0.f;
#pragma unroll
    for (int x = 0; x < 4; ++x) d += sM[x][c] == -INFINITY ? 0.f : sD[x][c] * exp2f(sM[x][c] - Mt);
    lse[(int64_t)bg * kWinCols + c] = Mt + log2f(d);
  }
}
#endif

size_t attn_workspace_bytes(int batch, int hq, int hkv, int d, int max_main, int max_tail,
                            int max_score, bool with_v, bool with_logits,
                            int* split_rows, int* max_splits,
                            int kind = 0);  // kind: 0 plain, 1 gather, 2 with a query window, 3 logits folded per kv head
int lds_bytes_per_workgroup();
int carve_attn_workspace(void* ws, size_t ws_bytes, int batch, int hq, int hkv, int d,
                         int max_main, int max_tail, int max_score, bool with_v,
                         bool with_logits, AttnWorkspace* out, int kind = 0);

extern std::atomic<int> g_split_rows_override;  // 0 = automatic

// Tokens per score-finishing block.  Every block recomputes the per-head normalisers from the
// splits' partials, work that grows with blocks x splits: short blocks (more CUs pulling the
// logits) while that stays small next to the logits themselves.
inline int finish_tokens_for(int split_rows, int max_score_len) {
  const int64_t splits = split_rows > 0 ? (max_score_len + split_rows - 1) / split_rows : 0;
  return splits * ((max_score_len + 511) / 512) <= 65536 ? 512 : 1024;
}

size_t topk_mb_workspace_bytes(int batch, int max_seq_len);  // okv_topk_mb.hip
static constexpr int kMultiBlockMinLen = 14336;  // top-k of shorter vectors: one workgroup per request is faster

int validate_layout(const okv_kv_layout_t* layout, const void* k_base, const void* v_base);

// Implemented in okv_attn.hip.
int launch_attention(const void* q, const RowList& rows, const okv_kv_layout_t* layout,
                     int batch, float scale, void* out, bool with_v, int head_reduce,
                     int normalise, float* scores, int64_t score_stride,
                     const AttnWorkspace& w, hipStream_t stream);

int launch_attention_window(const void* q, const RowList& rows, const okv_kv_layout_t* layout, int batch,
                            float scale, void* out, const AttnWorkspace& w, const WindowFuse& wf,
                            hipStream_t stream);
void fill_main(RowList* r, const void* k, const void* v, const okv_kv_layout_t* layout);

}  // namespace okv
