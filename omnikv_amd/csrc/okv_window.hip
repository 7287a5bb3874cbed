// Window selectors (`uniform`, `exp`): the score of a token is a sum over the last W
// query positions of the head-max of each position's softmax over the tokens
// (modeling/omnikv.py:59-105).  The reference runs W separate q.K^T / softmax / max
// passes; here the W x Hq query rows ride together through the matrix cores, so K is
// read twice in total instead of W times:
//
//   pass 1  window_lse_mfma    per (position, head): log-sum-exp of its logits over the
//                              tokens, split-context partials + a small merge
//   pass 2  window_score_mfma  logits again, max over the q heads of a kv head of
//                              logit - lse (DPP), one exponential per position and row,
//                              max over the kv heads by LDS atomics, then the sum over
//                              the positions in the reference's order of additions
//
// The B operand of a kv head g holds its W*G query rows as columns: column c is
// position c/G, q head g*G + c%G; up to four 16-column blocks (W*G <= 64).
#include <math.h>

#include "okv_device.h"
#include "okv_internal.h"

namespace okv {

struct WindowArgs {
  const void* q;
  int64_t q_batch_stride, q_head_stride, q_pos_stride;  // elements
  const void* k_base;
  int64_t token_stride, head_stride, batch_stride;
  const int32_t* score_lens;
  int32_t max_score_len;
  int32_t window, group, hkv;
  float scale;
  int32_t split_rows, max_splits;
  float* part;  // [batch][hkv][kWinCols][max_splits]  log2-domain partial lse
  float* lse;   // [batch][hkv][kWinCols]              log2-domain lse
};

__device__ __forceinline__ int win_len(const WindowArgs& a, int b) {
  return a.score_lens ? min(a.score_lens[b], a.max_score_len) : a.max_score_len;
}

// q fragments of kv head g: qf[cb][s] = elements 32s + 8(l/16) .. +8 of column 16cb + l%16
template <typename T, int NCB>
__device__ __forceinline__ void load_window_q(const WindowArgs& a, int b, int g, int r16, int j4,
                                              uint4 (&qf)[NCB][4]) {
#pragma unroll
  for (int cb = 0; cb < NCB; ++cb) {
    const int c = 16 * cb + r16;
    const int w = c / a.group, hg = c % a.group;
    const bool valid = w < a.window;
    const T* qp = reinterpret_cast<const T*>(a.q) + (int64_t)b * a.q_batch_stride +
                  (int64_t)(g * a.group + hg) * a.q_head_stride +
                  (int64_t)(valid ? w : 0) * a.q_pos_stride + 8 * j4;
#pragma unroll
    for (int s = 0; s < 4; ++s) {
      const uint4 v = *reinterpret_cast<const uint4*>(qp + 32 * s);
      qf[cb][s] = valid ? v : make_uint4(0, 0, 0, 0);
    }
  }
}

// ------------------------------------------------------------------ pass 1
// grid (kv heads, splits, batch), 256 threads; wave w of the block takes the 16-row
// tiles begin + 16(w + 4n) of its split.
template <typename T, int NCB>
__global__ __launch_bounds__(256) void window_lse_mfma(WindowArgs a) {
  __shared__ float sm[16][16 * NCB], sl[16][16 * NCB];
  const int g = blockIdx.x, split = blockIdx.y, b = blockIdx.z;
  const int A = win_len(a, b);
  const int begin = split * a.split_rows;
  const int end = min(begin + a.split_rows, A);
  if (begin >= end) return;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int r16 = lane & 15, j4 = lane >> 4;

  uint4 qf[NCB][4];
  load_window_q<T, NCB>(a, b, g, r16, j4, qf);
  const T* kb = reinterpret_cast<const T*>(a.k_base) + (int64_t)b * a.batch_stride +
                (int64_t)g * a.head_stride + 8 * j4;
  const uint32_t ts = (uint32_t)a.token_stride;
  const int last = end - 1;
  // K straight into the A-operand layout with ordinary (cached) loads in both passes.  Measured
  // alternatives: whole rows streamed (non-temporal) and transposed through LDS make pass 1 no
  // faster and pass 2 slower (78 vs 69 us: streamed lines do not stay in the memory-side cache
  // for the second reading); in pass 2 the LDS detour waits on the LDS atomics (128 us).
  auto load_tile = [&](int tbase, uint4 (&kf)[4]) {
    int r = tbase + r16;
    r = r < last ? r : last;
    const T* kp = kb + (uint64_t)(uint32_t)r * ts;
#pragma unroll
    for (int s = 0; s < 4; ++s) kf[s] = *reinterpret_cast<const uint4*>(kp + 32 * s);
  };
  const float sl2 = a.scale * kLog2e;
  float m[NCB], l[NCB];  // per column block: state of (column r16, lane row j4), m in raw units
#pragma unroll
  for (int cb = 0; cb < NCB; ++cb) {
    m[cb] = -INFINITY;
    l[cb] = 0.f;
  }
  auto compute = [&](int tbase, const uint4 (&kf)[4]) {
    const int row0 = tbase + 4 * j4;
    const bool ragged = tbase + 16 > end;  // wave-uniform: only a split's last tile has rows to mask
#pragma unroll
    for (int cb = 0; cb < NCB; ++cb) {
      f32x4_t S = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int s = 0; s < 4; ++s) S = mfma16((const T*)nullptr, kf[s], qf[cb][s], S);
      float sv[4] = {S[0], S[1], S[2], S[3]};
      if (ragged) {
#pragma unroll
        for (int i = 0; i < 4; ++i)
          if (row0 + i >= end) sv[i] = -INFINITY;
      }
      const float mn = fmaxf(fmaxf(fmaxf(sv[0], sv[1]), fmaxf(sv[2], sv[3])), m[cb]);
      const float ms = (mn == -INFINITY ? 0.f : mn) * sl2;
      const float alpha = __builtin_amdgcn_exp2f(fmaf(m[cb], sl2, -ms));
      float p = 0.f;
#pragma unroll
      for (int i = 0; i < 4; ++i) p += __builtin_amdgcn_exp2f(fmaf(sv[i], sl2, -ms));
      l[cb] = fmaf(l[cb], alpha, p);
      m[cb] = mn;
    }
  };
  {
    uint4 kA[4], kB[4];
    int t = begin + wave * 16;
    if (t < end) {
      const int t_last = t + ((last - t) >> 6 << 6);
      load_tile(t, kA);
      if (t == t_last) {
        compute(t, kA);
      } else {
        while (true) {  // every load unconditional (clamped): the next tile stays in flight
          load_tile(min(t + 64, t_last), kB);
          compute(t, kA);
          t += 64;
          load_tile(min(t + 64, t_last), kA);
          compute(t, kB);
          if (t == t_last) break;
          t += 64;
          if (t == t_last) {
            compute(t, kA);
            break;
          }
        }
      }
    }
  }
  const int grp = wave * 4 + j4;
#pragma unroll
  for (int cb = 0; cb < NCB; ++cb) {
    sm[grp][16 * cb + r16] = m[cb];
    sl[grp][16 * cb + r16] = l[cb];
  }
  __syncthreads();
  if (threadIdx.x < 16 * NCB) {
    const int c = threadIdx.x;
    float M = -INFINITY;
#pragma unroll
    for (int x = 0; x < 16; ++x) M = fmaxf(M, sm[x][c]);
    float den = 0.f;
#pragma unroll
    for (int x = 0; x < 16; ++x) {
      const float mm = sm[x][c];
      den = fmaf(sl[x][c], mm == -INFINITY ? 0.f : __builtin_amdgcn_exp2f((mm - M) * sl2), den);
    }
    a.part[((int64_t)(b * a.hkv + g) * kWinCols + c) * a.max_splits + split] =
        M == -INFINITY ? -INFINITY : M * sl2 + log2f(den);
  }
}

// grid (batch * kv heads), 256 threads
__global__ __launch_bounds__(256) void window_lse_merge(WindowArgs a) {
  const int bg = blockIdx.x;
  const int A = win_len(a, bg / a.hkv);
  window_lse_merge_body(a.part, a.lse, bg, (A + a.split_rows - 1) / a.split_rows, a.max_splits);
}

// Max over the G neighbouring lanes (G = 1, 2, 4 or 8) of four values at once, each step one
// v_max_f32 with a DPP operand: xor 1 and xor 2 inside the quad, then the mirrored lane of the half
// row (any lane of the other quad holds that quad's max by then).  Written out because fmaxf() on
// a DPP-moved value makes the compiler quiet every operand with a v_max x, x of its own.  The
// leading s_nop covers the two wait states between a VALU write and a DPP read of the same
// register; inside the block three other instructions separate every write from its DPP read.
#define OKV_DPP_MAX4(CTRL)                                                        \
  "v_max_f32_dpp %0, %0, %0 " CTRL " row_mask:0xf bank_mask:0xf\n\t"              \
  "v_max_f32_dpp %1, %1, %1 " CTRL " row_mask:0xf bank_mask:0xf\n\t"              \
  "v_max_f32_dpp %2, %2, %2 " CTRL " row_mask:0xf bank_mask:0xf\n\t"              \
  "v_max_f32_dpp %3, %3, %3 " CTRL " row_mask:0xf bank_mask:0xf\n\t"
template <int G>
__device__ __forceinline__ void group_max4(float& a, float& b, float& c, float& d) {
  if (G == 2)
    asm volatile("s_nop 1\n\t" OKV_DPP_MAX4("quad_perm:[1,0,3,2]") : "+v"(a), "+v"(b), "+v"(c), "+v"(d));
  else if (G == 4)
    asm volatile("s_nop 1\n\t" OKV_DPP_MAX4("quad_perm:[1,0,3,2]") OKV_DPP_MAX4("quad_perm:[2,3,0,1]")
                 : "+v"(a), "+v"(b), "+v"(c), "+v"(d));
  else if (G == 8)
    asm volatile("s_nop 1\n\t" OKV_DPP_MAX4("quad_perm:[1,0,3,2]") OKV_DPP_MAX4("quad_perm:[2,3,0,1]")
                     OKV_DPP_MAX4("row_half_mirror")
                 : "+v"(a), "+v"(b), "+v"(c), "+v"(d));
}
#undef OKV_DPP_MAX4

// ------------------------------------------------------------------ pass 2
// words between two positions' rows in LDS: 8 mod 32, so that the 4 positions x 8 rows which half a
// wave's lanes touch in one atomic instruction fall into the 32 different banks
__host__ __device__ inline int window_row_stride(int rows_per_block) { return (rows_per_block + 23) / 32 * 32 + 8; }

// grid (row blocks, batch), one wave per kv head; LDS: [window][window_row_stride] bit
// patterns of non-negative floats (their unsigned order is their numeric order).
template <typename T, int NCB, int G>
__global__ __launch_bounds__(512, 4) void window_score_mfma(WindowArgs a, int rows_per_block, int exp_decay,
                                                         float* __restrict__ scores,
                                                         int64_t score_stride) {
  extern __shared__ uint32_t wmax[];
  const int b = blockIdx.y;
  const int A = win_len(a, b);
  const int begin = blockIdx.x * rows_per_block;
  const int end = min(begin + rows_per_block, A);
  if (begin >= end) return;
  const int lane = threadIdx.x & 63, g = threadIdx.x >> 6;
  const int r16 = lane & 15, j4 = lane >> 4;
  const int nrows = end - begin;

  const int wstride = window_row_stride(rows_per_block);
  for (int i = threadIdx.x; i < a.window * wstride; i += blockDim.x) wmax[i] = 0u;

  uint4 qf[NCB][4];
  load_window_q<T, NCB>(a, b, g, r16, j4, qf);
  // The q heads of a kv head sit in G neighbouring columns.  After the max
  // over them every lane of the group holds the group's four rows; lane `sub` of the group
  // reports row `sub`, so one atomic instruction carries min(G, 4) rows of every position.
  const int sub = r16 & (G - 1);
  float lse[NCB];
  int wrow[NCB];  // first word of this lane's position's row of maxima, or -1 when the lane reports nothing
#pragma unroll
  for (int cb = 0; cb < NCB; ++cb) {
    const int c = 16 * cb + r16;
    lse[cb] = a.lse[(int64_t)(b * a.hkv + g) * kWinCols + c];
    wrow[cb] = (sub < 4 && c / G < a.window) ? (c / G) * wstride : -1;
  }
  const T* kb = reinterpret_cast<const T*>(a.k_base) + (int64_t)b * a.batch_stride +
                (int64_t)g * a.head_stride + 8 * j4;
  const uint32_t ts = (uint32_t)a.token_stride;
  const int last = end - 1;
  auto load_tile = [&](int tbase, uint4 (&kf)[4]) {
    int r = tbase + r16;
    r = r < last ? r : last;
    const T* kp = kb + (uint64_t)(uint32_t)r * ts;
#pragma unroll
    for (int s = 0; s < 4; ++s) kf[s] = *reinterpret_cast<const uint4*>(kp + 32 * s);
  };
  const float sl2 = a.scale * kLog2e;
  // exp2 is applied after the max over the heads (it is monotonic: the largest exponent gives the
  // largest probability), once per reported row instead of once per logit
  auto report = [&](int cb, float x, int row) {
    if (wrow[cb] >= 0 && row < nrows) atomicMax(&wmax[wrow[cb] + row], __float_as_uint(__builtin_amdgcn_exp2f(x)));
  };
  auto compute = [&](int tbase, const uint4 (&kf)[4]) {
    const int row0 = tbase + 4 * j4 - begin;
#pragma unroll
    for (int cb = 0; cb < NCB; ++cb) {
      f32x4_t S = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int s = 0; s < 4; ++s) S = mfma16((const T*)nullptr, kf[s], qf[cb][s], S);
      float x[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) x[i] = fmaf(S[i], sl2, -lse[cb]);
      group_max4<G>(x[0], x[1], x[2], x[3]);
      if (G >= 4) {
        const float lo = sub & 1 ? x[1] : x[0], hi = sub & 1 ? x[3] : x[2];
        report(cb, sub & 2 ? hi : lo, row0 + sub);
      } else if (G == 2) {
        report(cb, sub ? x[1] : x[0], row0 + sub);
        report(cb, sub ? x[3] : x[2], row0 + 2 + sub);
      } else {
#pragma unroll
        for (int i = 0; i < 4; ++i) report(cb, x[i], row0 + i);
      }
    }
  };
  __syncthreads();  // the zero fill is complete
  {
    // two tiles in flight per wave, two workgroups per CU (four waves per SIMD): one workgroup
    // with four tiles in flight is slower, and so are three or four workgroups of shorter row
    // blocks (every wave first loads its kv head's query fragments); every load is
    // unconditional, past the end it repeats the last tile
    uint4 kf[2][4];
    const int t_last = begin + ((last - begin) >> 4 << 4);
#pragma unroll
    for (int u = 0; u < 2; ++u) load_tile(min(begin + 16 * u, t_last), kf[u]);
    for (int t = begin; t <= t_last; t += 32) {
#pragma unroll
      for (int u = 0; u < 2; ++u) {
        const int tt = t + 16 * u;
        if (tt <= t_last) compute(tt, kf[u]);
        load_tile(min(tt + 32, t_last), kf[u]);
      }
    }
  }
  __syncthreads();
  for (int r = threadIdx.x; r < nrows; r += blockDim.x) {
    // the reference's order: positions oldest first, running sum (uniform) or
    // running sum halved before each addition (exp)
    float acc = __uint_as_float(wmax[r]);
    for (int w = 1; w < a.window; ++w) {
      const float v = __uint_as_float(wmax[w * wstride + r]);
      acc = exp_decay ? acc * 0.5f + v : acc + v;
    }
    scores[(int64_t)b * score_stride + begin + r] = acc;
  }
}

// ------------------------------------------------------------------ host
static int window_split_rows(int batch, int hkv, int max_len, int cus) {
  const int64_t capacity = (int64_t)cus * 3;
  const int64_t work = (int64_t)max_len * hkv * batch;
  int64_t rows = (work + capacity - 1) / capacity;
  rows = (rows + 63) / 64 * 64;
  return (int)(rows < 64 ? 64 : rows);
}

static int num_cus() {
  int dev = 0, n = 0;
  if (hipGetDevice(&dev) == hipSuccess &&
      hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && n > 0)
    return n;
  return 256;
}

static size_t window_part_bytes(int batch, int hkv, int splits);

size_t window_workspace_bytes(int batch, int hkv, int max_len) {
  const int sr = window_split_rows(batch, hkv, max_len, num_cus());
  const int splits = (max_len + sr - 1) / sr;
  return window_part_bytes(batch, hkv, splits);
}

template <typename T, int NCB, int G>
static void launch_window(WindowArgs a, int batch, int exp_decay, float* scores, int64_t score_stride,
                          int cus, hipStream_t stream, bool lse_ready) {
  if (!lse_ready) {  // otherwise the dense pass of the same call and its merge launch have left them
    hipLaunchKernelGGL((window_lse_mfma<T, NCB>), dim3(a.hkv, a.max_splits, batch), dim3(256), 0, stream, a);
    hipLaunchKernelGGL(window_lse_merge, dim3(batch * a.hkv), dim3(256), 0, stream, a);
  }
  // one round of row blocks, two blocks of `hkv` waves per CU; LDS bounds the rows
  int64_t per = ((int64_t)a.max_score_len * batch + 2 * cus - 1) / (2 * cus);
  int rpb = (int)((per + 15) / 16 * 16);
  if (rpb < 64) rpb = 64;
  const int cap = (48 * 1024 / 4 / a.window - 8) / 32 * 32;  // window_row_stride(cap) == cap + 8: 48 KB of LDS at most
  if (rpb > cap) {  // several rounds of one block per CU: equal ones
    const int64_t rounds = (per + cap - 1) / cap;
    rpb = (int)(((per + rounds - 1) / rounds + 15) / 16 * 16);
  }
  dim3 grid((a.max_score_len + rpb - 1) / rpb, batch);
  hipLaunchKernelGGL((window_score_mfma<T, NCB, G>), grid, dim3(64 * a.hkv),
                     (size_t)a.window * window_row_stride(rpb) * sizeof(uint32_t), stream, a, rpb, exp_decay, scores,
                     score_stride);
}

template <typename T, int G>
static void launch_window_g(const WindowArgs& a, int batch, int exp_decay, float* scores, int64_t score_stride,
                            int cus, hipStream_t stream, bool lse_ready) {
  const int ncb = (a.window * G + 15) / 16;
  switch (ncb) {
    case 1: launch_window<T, 1, G>(a, batch, exp_decay, scores, score_stride, cus, stream, lse_ready); break;
    case 2: launch_window<T, 2, G>(a, batch, exp_decay, scores, score_stride, cus, stream, lse_ready); break;
    case 3: launch_window<T, 3, G>(a, batch, exp_decay, scores, score_stride, cus, stream, lse_ready); break;
    default: launch_window<T, 4, G>(a, batch, exp_decay, scores, score_stride, cus, stream, lse_ready); break;
  }
}

// the q heads per kv head: 1, 2, 4 or 8 (window_group_supported)
template <typename T>
static void launch_window_t(const WindowArgs& a, int batch, int exp_decay, float* scores,
                            int64_t score_stride, int cus, hipStream_t stream, bool lse_ready = false) {
  switch (a.group) {
    case 1: launch_window_g<T, 1>(a, batch, exp_decay, scores, score_stride, cus, stream, lse_ready); break;
    case 2: launch_window_g<T, 2>(a, batch, exp_decay, scores, score_stride, cus, stream, lse_ready); break;
    case 4: launch_window_g<T, 4>(a, batch, exp_decay, scores, score_stride, cus, stream, lse_ready); break;
    case 8: launch_window_g<T, 8>(a, batch, exp_decay, scores, score_stride, cus, stream, lse_ready); break;
    default: break;  // refused by the entry points
  }
}

static bool window_group_supported(int group) { return group == 1 || group == 2 || group == 4 || group == 8; }

// bytes of the window columns' partials and merged log-sum-exps for `splits` splits per request
static size_t window_part_bytes(int batch, int hkv, int splits) {
  return (size_t)batch * hkv * kWinCols * ((size_t)(splits > 0 ? splits : 1) + 1) * sizeof(float) + 512;
}

size_t dense_window_workspace_bytes(int batch, int hq, int hkv, int d, int max_seq_len, int max_score_len) {
  int splits = 0;
  const size_t attn = attn_workspace_bytes(batch, hq, hkv, d, max_seq_len, 0, max_score_len, true, false, nullptr,
                                           &splits, 2);
  return ((attn + 255) & ~(size_t)255) + window_part_bytes(batch, hkv, splits);
}

}  // namespace okv

using namespace okv;

extern "C" int okv_score_window(const void* q, int64_t q_batch_stride, int64_t q_head_stride,
                                int64_t q_pos_stride, int32_t window, int32_t exp_decay,
                                const void* k_base, const okv_kv_layout_t* layout,
                                const int32_t* score_lens, int32_t max_score_len, int32_t batch,
                                float scale, float* scores, int64_t score_stride, void* ws,
                                size_t ws_bytes, okv_stream_t stream) {
  int rc = validate_layout(layout, k_base, k_base);
  if (rc) return rc;
  OKV_REQUIRE(q && scores, OKV_ERR_INVALID, "q or scores is NULL");
  OKV_REQUIRE(batch >= 1 && max_score_len >= 0 && window >= 1, OKV_ERR_INVALID,
              "bad batch, length or window");
  OKV_REQUIRE(score_stride >= max_score_len, OKV_ERR_INVALID, "score_stride < max_score_len");
  OKV_REQUIRE(((uintptr_t)q & 15) == 0 && q_batch_stride % 8 == 0 && q_head_stride % 8 == 0 &&
                  q_pos_stride % 8 == 0,
              OKV_ERR_INVALID, "q must be 16-byte aligned with strides that are multiples of 8");
  const int hkv = layout->num_kv_heads, group = layout->num_q_heads / hkv;
  OKV_REQUIRE(layout->dtype == OKV_BF16 || layout->dtype == OKV_F16, OKV_ERR_UNSUPPORTED,
              "window scoring runs on the matrix cores: 16-bit K only");
  OKV_REQUIRE(layout->page_table == nullptr, OKV_ERR_UNSUPPORTED, "window scoring reads contiguous K only");
  OKV_REQUIRE(window * group <= kWinCols, OKV_ERR_UNSUPPORTED,
              "window %d x group %d exceeds %d query rows per kv head", window, group, kWinCols);
  OKV_REQUIRE(window_group_supported(group), OKV_ERR_UNSUPPORTED,
              "window scoring takes 1, 2, 4 or 8 q heads per kv head, not %d", group);
  OKV_REQUIRE(hkv <= 8, OKV_ERR_UNSUPPORTED, "more than 8 kv heads");
  OKV_REQUIRE(layout->token_stride < (1ll << 31), OKV_ERR_UNSUPPORTED, "token stride too large");
  if (max_score_len == 0) return OKV_OK;
  OKV_REQUIRE(ws != nullptr && ws_bytes >= window_workspace_bytes(batch, hkv, max_score_len),
              OKV_ERR_WORKSPACE, "workspace too small: have %zu, need %zu", ws_bytes,
              window_workspace_bytes(batch, hkv, max_score_len));
  const int cus = num_cus();
  WindowArgs a;
  a.q = q;
  a.q_batch_stride = q_batch_stride;
  a.q_head_stride = q_head_stride;
  a.q_pos_stride = q_pos_stride;
  a.k_base = k_base;
  a.token_stride = layout->token_stride;
  a.head_stride = layout->head_stride;
  a.batch_stride = layout->batch_stride;
  a.score_lens = score_lens;
  a.max_score_len = max_score_len;
  a.window = window;
  a.group = group;
  a.hkv = hkv;
  a.scale = scale;
  a.split_rows = window_split_rows(batch, hkv, max_score_len, cus);
  a.max_splits = (max_score_len + a.split_rows - 1) / a.split_rows;
  char* p = (char*)(((uintptr_t)ws + 255) & ~(uintptr_t)255);
  a.part = (float*)p;
  a.lse = a.part + (size_t)batch * hkv * kWinCols * a.max_splits;
  if (layout->dtype == OKV_BF16)
    launch_window_t<BF16>(a, batch, exp_decay != 0, scores, score_stride, cus, (hipStream_t)stream);
  else
    launch_window_t<F16>(a, batch, exp_decay != 0, scores, score_stride, cus, (hipStream_t)stream);
  OKV_HIP_CHECK(hipGetLastError());
  return OKV_OK;
}

extern "C" int okv_dense_attn_window(const void* q, const void* q_window, int64_t q_batch_stride,
                                     int64_t q_head_stride, int64_t q_pos_stride, int32_t window,
                                     int32_t exp_decay, const void* k_base, const void* v_base,
                                     const okv_kv_layout_t* layout, const int32_t* seq_lens, int32_t max_seq_len,
                                     int32_t batch, float scale, void* out, const int32_t* score_lens,
                                     int32_t max_score_len, float* scores, int64_t score_stride, void* ws,
                                     size_t ws_bytes, okv_stream_t stream) {
  int rc = validate_layout(layout, k_base, v_base);
  if (rc) return rc;
  OKV_REQUIRE(q && q_window && scores && out && v_base, OKV_ERR_INVALID, "q, q_window, v_base, out or scores is NULL");
  OKV_REQUIRE(batch >= 1 && max_seq_len >= 1 && window >= 1, OKV_ERR_INVALID, "bad batch, length or window");
  OKV_REQUIRE(max_score_len >= 1 && max_score_len <= max_seq_len, OKV_ERR_INVALID, "max_score_len out of range");
  OKV_REQUIRE(score_stride >= max_score_len, OKV_ERR_INVALID, "score_stride < max_score_len");
  OKV_REQUIRE(((uintptr_t)q_window & 15) == 0 && ((uintptr_t)q & 15) == 0 && q_batch_stride % 8 == 0 &&
                  q_head_stride % 8 == 0 && q_pos_stride % 8 == 0,
              OKV_ERR_INVALID, "q and q_window must be 16-byte aligned with strides that are multiples of 8");
  const int hq = layout->num_q_heads, hkv = layout->num_kv_heads, group = hq / hkv;
  OKV_REQUIRE(layout->dtype == OKV_BF16 || layout->dtype == OKV_F16, OKV_ERR_UNSUPPORTED,
              "window scoring runs on the matrix cores: 16-bit K only");
  OKV_REQUIRE(layout->page_table == nullptr, OKV_ERR_UNSUPPORTED, "window scoring reads contiguous K only");
  OKV_REQUIRE(window * group <= kWinCols, OKV_ERR_UNSUPPORTED,
              "window %d x group %d exceeds %d query rows per kv head", window, group, kWinCols);
  OKV_REQUIRE(window_group_supported(group), OKV_ERR_UNSUPPORTED,
              "window scoring takes 1, 2, 4 or 8 q heads per kv head, not %d", group);
  OKV_REQUIRE(hkv <= 8, OKV_ERR_UNSUPPORTED, "more than 8 kv heads");
  OKV_REQUIRE(layout->token_stride < (1ll << 31), OKV_ERR_UNSUPPORTED, "token stride too large");
  const size_t need = dense_window_workspace_bytes(batch, hq, hkv, layout->head_dim, max_seq_len, max_score_len);
  OKV_REQUIRE(ws != nullptr && ws_bytes >= need, OKV_ERR_WORKSPACE, "workspace too small: have %zu, need %zu",
              ws_bytes, need);
  const size_t attn_bytes = (attn_workspace_bytes(batch, hq, hkv, layout->head_dim, max_seq_len, 0, max_score_len,
                                                  true, false, nullptr, nullptr, 2) + 255) & ~(size_t)255;
  AttnWorkspace w;
  rc = carve_attn_workspace(ws, attn_bytes, batch, hq, hkv, layout->head_dim, max_seq_len, 0, max_score_len, true,
                            false, &w, 2);
  if (rc) return rc;
  WindowArgs a;
  a.q = q_window;
  a.q_batch_stride = q_batch_stride;
  a.q_head_stride = q_head_stride;
  a.q_pos_stride = q_pos_stride;
  a.k_base = k_base;
  a.token_stride = layout->token_stride;
  a.head_stride = layout->head_stride;
  a.batch_stride = layout->batch_stride;
  a.score_lens = score_lens;
  a.max_score_len = max_score_len;
  a.window = window;
  a.group = group;
  a.hkv = hkv;
  a.scale = scale;
  a.split_rows = w.split_rows;  // the dense pass's splits: its scored ones tile [0, score_len)
  a.max_splits = w.max_splits;
  char* p = (char*)(((uintptr_t)ws + attn_bytes + 255) & ~(uintptr_t)255);
  a.part = (float*)p;
  a.lse = a.part + (size_t)batch * hkv * kWinCols * a.max_splits;
  WindowFuse wf;
  wf.wq = q_window;
  wf.q_batch_stride = q_batch_stride;
  wf.q_head_stride = q_head_stride;
  wf.q_pos_stride = q_pos_stride;
  wf.window = window;
  wf.part = a.part;
  wf.lse = a.lse;
  RowList r;
  fill_main(&r, k_base, v_base, layout);
  r.main_lens = seq_lens;
  r.max_main_len = max_seq_len;
  r.score_lens = score_lens;
  r.max_score_len = max_score_len;
  rc = launch_attention_window(q, r, layout, batch, scale, out, w, wf, (hipStream_t)stream);
  if (rc) return rc;
  const int cus = num_cus();
  if (layout->dtype == OKV_BF16)
    launch_window_t<BF16>(a, batch, exp_decay != 0, scores, score_stride, cus, (hipStream_t)stream, true);
  else
    launch_window_t<F16>(a, batch, exp_decay != 0, scores, score_stride, cus, (hipStream_t)stream, true);
  OKV_HIP_CHECK(hipGetLastError());
  return OKV_OK;
}
