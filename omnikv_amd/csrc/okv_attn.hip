// Split-context GQA decode attention and filter-layer scoring for gfx950.
//
// One pass over the rows of a request (stage 1) produces, per (q head, split),
// a normalised partial output and its log-sum-exp, and optionally the scaled
// logits of the scored rows.  A merge kernel combines the splits; a finishing
// kernel turns logits into one score per token.
//
// This file holds the portable wave64 VALU formulation (any of f32 / bf16 / f16,
// GQA group 1..8): sixteen lanes share a 128-element row, eight elements each.
#include <math.h>
#include <string.h>

#include <atomic>
#include <mutex>

#include "okv_internal.h"
#include "okv_device.h"

namespace okv {

// ----------------------------------------------------------------- stage 1
// grid (kv heads, splits, batch), 256 threads.  Each group of 16 lanes walks
// every 16th row of the split, keeping a private online-softmax state for the G
// q heads of the kv head; the 16 groups of the block are merged at the end.
template <typename T, int G, bool WITH_V>
__global__ __launch_bounds__(256) void attn_stage1_generic(const T* __restrict__ q, RowList rows,
                                                           int hq, float scale, AttnWorkspace w,
                                                           int write_logits) {
  const int g = blockIdx.x, split = blockIdx.y, b = blockIdx.z;
  const int main_len = rl_main_len(rows, b);
  const int L = main_len + rl_tail_len(rows, b);
  const int A = rl_score_len(rows, b);
  int begin, end;
  rl_split_range(split, w.split_rows, A, L, &begin, &end);
  if (begin >= end) return;

  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int c = lane & 15;
  const int grp = wave * 4 + (lane >> 4);

  float qr[G][8];
#pragma unroll
  for (int h = 0; h < G; ++h) load8(q + ((int64_t)(b * hq + g * G + h) * kD + c * 8), qr[h]);

  float m[G], l[G], acc[G][8];
#pragma unroll
  for (int h = 0; h < G; ++h) {
    m[h] = -INFINITY;
    l[h] = 0.f;
#pragma unroll
    for (int i = 0; i < 8; ++i) acc[h][i] = 0.f;
  }
  const float sl2 = scale * kLog2e;
  const T* kb = reinterpret_cast<const T*>(rows.k_base);
  const T* vb = reinterpret_cast<const T*>(rows.v_base);
  const T* tkb = reinterpret_cast<const T*>(rows.tail_k);
  const T* tvb = reinterpret_cast<const T*>(rows.tail_v);

  for (int row = begin + grp; row < end; row += 16) {
    bool in_tail;
    int64_t off = rl_row_offset(rows, b, row, main_len, &in_tail);
    off += (int64_t)g * (in_tail ? rows.tail_head_stride : rows.head_stride) + c * 8;
    float kf[8];
    load8((in_tail ? tkb : kb) + off, kf);
    float s[G];
#pragma unroll
    for (int h = 0; h < G; ++h) {
      float a = 0.f;
#pragma unroll
      for (int i = 0; i < 8; ++i) a = fmaf(qr[h][i], kf[i], a);
      a += __shfl_xor(a, 8);
      a += __shfl_xor(a, 4);
      a += __shfl_xor(a, 2);
      a += __shfl_xor(a, 1);
      s[h] = a;
    }
    if (write_logits && row < A) {
#pragma unroll
      for (int h = 0; h < G; ++h)
        if (c == h) w.logits[(int64_t)(b * hq + g * G + h) * w.logits_stride + row] = s[h] * scale;
    }
    float vf[8];
    if (WITH_V) load8((in_tail ? tvb : vb) + off, vf);
#pragma unroll
    for (int h = 0; h < G; ++h) {
      float s2 = s[h] * sl2;
      float mn = fmaxf(m[h], s2);
      float alpha = __builtin_amdgcn_exp2f(m[h] - mn);
      float p = __builtin_amdgcn_exp2f(s2 - mn);
      l[h] = l[h] * alpha + p;
      m[h] = mn;
      if (WITH_V) {
#pragma unroll
        for (int i = 0; i < 8; ++i) acc[h][i] = acc[h][i] * alpha + p * vf[i];
      }
    }
  }

  // merge the four 16-lane groups of the wave (lanes l, l^16, l^32, l^48)
#pragma unroll
  for (int h = 0; h < G; ++h) {
    float M = fmaxf(m[h], __shfl_xor(m[h], 16));
    M = fmaxf(M, __shfl_xor(M, 32));
    float f = (m[h] == -INFINITY) ? 0.f : exp2f(m[h] - M);
    float ll = l[h] * f;
    ll += __shfl_xor(ll, 16);
    ll += __shfl_xor(ll, 32);
    l[h] = ll;
    m[h] = M;
    if (WITH_V) {
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        float a = acc[h][i] * f;
        a += __shfl_xor(a, 16);
        a += __shfl_xor(a, 32);
        acc[h][i] = a;
      }
    }
  }

  __shared__ float sm[4][G];
  __shared__ float sl[4][G];
  __shared__ float sacc[WITH_V ? 4 : 1][G][kD];
  if (lane < 16) {
#pragma unroll
    for (int h = 0; h < G; ++h) {
      if (c == 0) {
        sm[wave][h] = m[h];
        sl[wave][h] = l[h];
      }
      if (WITH_V) {
#pragma unroll
        for (int i = 0; i < 8; ++i) sacc[wave][h][c * 8 + i] = acc[h][i];
      }
    }
  }
  __syncthreads();
  for (int o = threadIdx.x; o < G * kD; o += 256) {
    const int h = o / kD, d = o % kD;
    float M = fmaxf(fmaxf(sm[0][h], sm[1][h]), fmaxf(sm[2][h], sm[3][h]));
    float den = 0.f, num = 0.f;
#pragma unroll
    for (int x = 0; x < 4; ++x) {
      float f = (sm[x][h] == -INFINITY) ? 0.f : exp2f(sm[x][h] - M);
      den += sl[x][h] * f;
      if (WITH_V) num += sacc[x][h][d] * f;
    }
    const int64_t ph = (int64_t)(b * hq + g * G + h) * w.max_splits + split;
    if (WITH_V) w.part_o[ph * kD + d] = num / den;
    if (d == 0) w.part_lse[ph] = M + log2f(den);
  }
}

// ------------------------------------------------------------------- merge
#ifdef OKV_STAMPS
__device__ unsigned long long g_merge_stamps[kStampBlocks * kStampSlots];
#endif
// grid (q heads, batch), 256 threads: 32 float4 columns x 8 split lanes.  Every
// thread folds its splits with a running max (all loads independent, one trip to
// memory), then the 8 split lanes of a column meet in LDS.
template <typename T>
__device__ __forceinline__ void merge_body(const RowList& rows, int hq, const AttnWorkspace& w,
                                           T* __restrict__ out, int with_v, int with_score_lse, int h,
                                           int b) {
  __shared__ float4 snum[8][32];
  OKV_STAMP(g_merge_stamps, h, 0);  // merge timeline: 0 entry, 1 arguments and lengths there, 2 own splits folded, 3 after the barrier, 4 end
  __shared__ float sm[8], sden[8], smA[8], sdenA[8];
  const int tid = threadIdx.x;
  const int main_len = rl_main_len(rows, b);
  const int L = main_len + rl_tail_len(rows, b);
  const int A = rl_score_len(rows, b);
  const int ns = rl_num_splits(w.split_rows, A, L);
  const int nA = with_score_lse ? (A + w.split_rows - 1) / w.split_rows : 0;
  const int64_t ph = (int64_t)(b * hq + h) * w.max_splits;
  const float* lse = w.part_lse + ph;
  const int dq = tid & 31, sl = tid >> 5;
  const float4* po = reinterpret_cast<const float4*>(w.part_o + ph * kD) + dq;

  OKV_STAMP(g_merge_stamps, h, 1);
  float m = -INFINITY, den = 0.f, mA = -INFINITY, denA = 0.f;
  float4 num = make_float4(0.f, 0.f, 0.f, 0.f);
  constexpr int U = 8;  // splits in flight per thread: all loads of a batch leave before any is used
  for (int s0 = sl; s0 < ns; s0 += 8 * U) {
    float xs[U];
    float4 os[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int s = s0 + 8 * u;
      xs[u] = s < ns ? lse[s] : -INFINITY;
      os[u] = make_float4(0.f, 0.f, 0.f, 0.f);
      if (with_v && s < ns) os[u] = po[(int64_t)s * 32];
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int s = s0 + 8 * u;
      if (s >= ns) break;
      const float x = xs[u];
      const float mn = fmaxf(m, x);
      const float a = __builtin_amdgcn_exp2f(m - mn), f = __builtin_amdgcn_exp2f(x - mn);
      den = fmaf(den, a, f);
      num.x = fmaf(num.x, a, f * os[u].x);
      num.y = fmaf(num.y, a, f * os[u].y);
      num.z = fmaf(num.z, a, f * os[u].z);
      num.w = fmaf(num.w, a, f * os[u].w);
      m = mn;
      if (s < nA) {
        const float mnA = fmaxf(mA, x);
        denA = fmaf(denA, __builtin_amdgcn_exp2f(mA - mnA), __builtin_amdgcn_exp2f(x - mnA));
        mA = mnA;
      }
    }
  }
  OKV_STAMP(g_merge_stamps, h, 2);
  snum[sl][dq] = num;
  if (dq == 0) {
    sm[sl] = m;
    sden[sl] = den;
    smA[sl] = mA;
    sdenA[sl] = denA;
  }
  __syncthreads();
  OKV_STAMP(g_merge_stamps, h, 3);
  if (with_v && tid < kD) {
    float M = -INFINITY;
#pragma unroll
    for (int x = 0; x < 8; ++x) M = fmaxf(M, sm[x]);
    const float* sn = reinterpret_cast<const float*>(&snum[0][0]);
    float a = 0.f, d = 0.f;
#pragma unroll
    for (int x = 0; x < 8; ++x) {
      const float f = (sm[x] == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f(sm[x] - M);
      a = fmaf(sn[x * kD + tid], f, a);
      d = fmaf(sden[x], f, d);
    }
    store1(out + (int64_t)(b * hq + h) * kD + tid, ns > 0 ? a / d : 0.f);
  }
  if (with_score_lse && tid == 0) {
    float M = -INFINITY;
#pragma unroll
    for (int x = 0; x < 8; ++x) M = fmaxf(M, smA[x]);
    float d = 0.f;
#pragma unroll
    for (int x = 0; x < 8; ++x) d += (smA[x] == -INFINITY) ? 0.f : sdenA[x] * __builtin_amdgcn_exp2f(smA[x] - M);
    w.score_lse[b * hq + h] = M + log2f(d);
  }
  OKV_STAMP(g_merge_stamps, h, 4);
}

template <typename T>
__global__ __launch_bounds__(256) void attn_merge(RowList rows, int hq, AttnWorkspace w,
                                                  T* __restrict__ out, int with_v,
                                                  int with_score_lse) {
  fetch_now(out);
  fetch_args_now(rows, w);
  merge_body<T>(rows, hq, w, out, with_v, with_score_lse, blockIdx.x, blockIdx.y);
}

// The merge launch behind a dense pass with window columns: blocks [0, Hq) of a request merge the
// attention partials, blocks [Hq, Hq + Hkv) the window columns' log-sum-exps -- one launch, not two.
template <typename T>
__global__ __launch_bounds__(256) void attn_window_merge(RowList rows, int hq, int hkv, AttnWorkspace w,
                                                         T* __restrict__ out, WindowFuse wf) {
  const int b = blockIdx.y;
  if ((int)blockIdx.x < hq) {
    merge_body<T>(rows, hq, w, out, 1, 0, blockIdx.x, b);
  } else {
    const int A = rl_score_len(rows, b);
    window_lse_merge_body(wf.part, wf.lse, b * hkv + (int)blockIdx.x - hq, (A + w.split_rows - 1) / w.split_rows,
                          w.max_splits);
  }
}

// ------------------------------------------------------------ score finish
// 256 threads, TPT consecutive tokens each, block `bx` of request `b`.  With own_lse the
// block works out the per-head score normalisers itself from the splits' partial
// log-sum-exps (a few KB from L2) instead of reading what a merge launch left, so that it
// does not have to run after one.  Blocks of 512 tokens put twice as many CUs to pulling the
// logits as blocks of 1024 (6.0 against 6.9 us at 128K), but each block's normalisers cost
// Hq x splits loads, so long contexts keep the larger block.
constexpr int kMaxFinishHeads = 256;
template <int TPT>
__device__ __forceinline__ void finish_body(const RowList& rows, int hq, const AttnWorkspace& w,
                                            int head_reduce, int normalise, float* __restrict__ scores,
                                            int64_t score_stride, int bx, int b, bool own_lse) {
  __shared__ float s_lse[kMaxFinishHeads];
  const int tid = threadIdx.x;
  const int t0 = (bx * 256 + tid) * TPT;
  const int A = rl_score_len(rows, b);
  if (bx * 256 * TPT >= A) return;  // the whole block: nothing below depends on the thread
  const bool is_max = head_reduce == OKV_REDUCE_MAX;
  const bool soft = normalise == OKV_NORM_SOFTMAX;
  if (soft && own_lse) {  // 8 threads per head, 32 heads per trip
    const int nA = (A + w.split_rows - 1) / w.split_rows;
    const int sub = tid & 7;
    for (int h0 = 0; h0 < hq; h0 += 32) {
      const int h = h0 + (tid >> 3);
      float M = -INFINITY, d = 0.f;
      if (h < hq) {
        const float* pl = w.part_lse + (int64_t)(b * hq + h) * w.max_splits;
        constexpr int U = 8;  // loads of a batch leave together
        for (int s2 = sub; s2 < nA; s2 += 8 * U) {
          float xs[U];
#pragma unroll
          for (int u = 0; u < U; ++u) xs[u] = s2 + 8 * u < nA ? pl[s2 + 8 * u] : -INFINITY;
#pragma unroll
          for (int u = 0; u < U; ++u) {
            const float mn = fmaxf(M, xs[u]);
            if (mn != -INFINITY) {
              d = fmaf(d, __builtin_amdgcn_exp2f(M - mn), __builtin_amdgcn_exp2f(xs[u] - mn));
              M = mn;
            }
          }
        }
      }
#pragma unroll
      for (int o = 1; o < 8; o <<= 1) {
        const float M2 = __shfl_xor(M, o), d2 = __shfl_xor(d, o);
        const float mn = fmaxf(M, M2);
        if (mn != -INFINITY) d = d * __builtin_amdgcn_exp2f(M - mn) + d2 * __builtin_amdgcn_exp2f(M2 - mn);
        M = mn;
      }
      if (h < hq && sub == 0) s_lse[h] = M + log2f(d);
    }
  }
  if (soft && own_lse) __syncthreads();
  const float init = is_max ? -INFINITY : 0.f;
  float acc[TPT];
#pragma unroll
  for (int i = 0; i < TPT; ++i) acc[i] = init;
  if (t0 < A) {
    const int nh = w.logit_heads;  // Hq, or Hkv when the split pass has folded each group already
    const float* lg = w.logits + (int64_t)b * nh * w.logits_stride + t0;
#pragma unroll 16
    for (int h = 0; h < nh; ++h) {
      float v[TPT];
      if constexpr (TPT == 4) {
        const float4 v4 = *reinterpret_cast<const float4*>(lg + (int64_t)h * w.logits_stride);
        v[0] = v4.x; v[1] = v4.y; v[2] = v4.z; v[3] = v4.w;
      } else {
        const float2 v2 = *reinterpret_cast<const float2*>(lg + (int64_t)h * w.logits_stride);
        v[0] = v2.x; v[1] = v2.y;
      }
      const float lse = soft ? (own_lse ? s_lse[h] : w.score_lse[b * hq + h]) : 0.f;
#pragma unroll
      for (int i = 0; i < TPT; ++i) {
        // one v_exp_f32 (a probability below 2^-126 counts as zero): with Hq exponentials per token
        // the block's time was its arithmetic, not its loads
        float x = soft ? __builtin_amdgcn_exp2f(fmaf(v[i], kLog2e, -lse)) : v[i];
        acc[i] = is_max ? fmaxf(acc[i], x) : acc[i] + x;
      }
    }
    float* sp = scores + (int64_t)b * score_stride + t0;
    if (t0 + TPT - 1 < A && (((uintptr_t)sp) & (4 * TPT - 1)) == 0) {
      if constexpr (TPT == 4) *reinterpret_cast<float4*>(sp) = make_float4(acc[0], acc[1], acc[2], acc[3]);
      else *reinterpret_cast<float2*>(sp) = make_float2(acc[0], acc[1]);
    } else {
#pragma unroll
      for (int i = 0; i < TPT; ++i)
        if (t0 + i < A) sp[i] = acc[i];
    }
  }
}

// grid (ceil(max_score / (256 TPT)), batch)
template <int TPT>
__global__ __launch_bounds__(256) void score_finish(RowList rows, int hq, AttnWorkspace w,
                                                    int head_reduce, int normalise,
                                                    float* __restrict__ scores,
                                                    int64_t score_stride) {
  finish_body<TPT>(rows, hq, w, head_reduce, normalise, scores, score_stride, blockIdx.x, blockIdx.y, false);
}

// Both in one launch: blocks [0, merge_blocks) fold the splits of one q head each, the rest
// finish the scores (with their own normalisers: nothing here waits for another block).
// grid (merge_blocks + ceil(max_score / (256 TPT)), batch)
template <typename T, int TPT>
__global__ __launch_bounds__(256) void merge_and_finish(RowList rows, int hq, AttnWorkspace w,
                                                        T* __restrict__ out, int merge_blocks,
                                                        int head_reduce, int normalise,
                                                        float* __restrict__ scores,
                                                        int64_t score_stride) {
  fetch_now(out);
  fetch_now(scores);
  fetch_args_now(rows, w);
  if ((int)blockIdx.x < merge_blocks)
    merge_body<T>(rows, hq, w, out, 1, 0, blockIdx.x, blockIdx.y);
  else
    finish_body<TPT>(rows, hq, w, head_reduce, normalise, scores, score_stride, blockIdx.x - merge_blocks,
                     blockIdx.y, true);
}

// ----------------------------------------------------------------- launch
std::atomic<int> g_attn_variant{0};  // 0 = pick per dtype, 1 = portable VALU stage 1 everywhere
#ifdef OKV_DIAG
std::atomic<int> g_split_pass_only{0};  // measurement build only (okv_diag_split_pass_only): no merge / finish launch
#endif

bool launch_stage1_mfma(int dtype, const void* q, const RowList& rows, int hq, int hkv, int batch,
                        float scale, const AttnWorkspace& w, bool with_v, bool write_logits,
                        hipStream_t stream);
bool launch_score_raw_mfma(int dtype, const void* q, const RowList& rows, int hq, int hkv, int batch,
                           float scale, int head_reduce, float* scores, int64_t score_stride,
                           hipStream_t stream);

template <typename T, int G>
static void launch_stage1(const void* q, const RowList& rows, int hq, int hkv, int batch,
                          float scale, const AttnWorkspace& w, bool with_v, bool write_logits,
                          hipStream_t stream) {
  dim3 grid(hkv, w.max_splits, batch);  // kv head fastest: co-resident blocks cover whole token rows
  if (with_v)
    hipLaunchKernelGGL((attn_stage1_generic<T, G, true>), grid, dim3(256), 0, stream,
                       (const T*)q, rows, hq, scale, w, (int)write_logits);
  else
    hipLaunchKernelGGL((attn_stage1_generic<T, G, false>), grid, dim3(256), 0, stream,
                       (const T*)q, rows, hq, scale, w, (int)write_logits);
}

template <typename T>
static int launch_typed(const void* q, const RowList& rows, const okv_kv_layout_t* lay,
                        int batch, float scale, void* out, bool with_v, int head_reduce,
                        int normalise, float* scores, int64_t score_stride,
                        const AttnWorkspace& w, hipStream_t stream) {
  const int hq = lay->num_q_heads, hkv = lay->num_kv_heads, G = hq / hkv;
  const bool want_scores = scores != nullptr;
  // raw scores alone need no normaliser: one launch that reduces the heads in the workgroup
  if (g_attn_variant.load(std::memory_order_relaxed) != 1 && !with_v && want_scores && normalise == OKV_NORM_RAW &&
      launch_score_raw_mfma(lay->dtype, q, rows, hq, hkv, batch, scale, head_reduce, scores, score_stride,
                            stream)) {
    OKV_HIP_CHECK(hipGetLastError());
    return OKV_OK;
  }
  AttnWorkspace wm = w;  // what the matrix-core kernel may do on top: fold the group for raw scores
  if (want_scores && normalise == OKV_NORM_RAW && G > 1) {
    wm.group_reduce = head_reduce == OKV_REDUCE_MAX ? 1 : 2;
    wm.logit_heads = hkv;
  }
  const AttnWorkspace* used = &w;
  if (g_attn_variant.load(std::memory_order_relaxed) != 1 &&
      launch_stage1_mfma(lay->dtype, q, rows, hq, hkv, batch, scale, wm, with_v, want_scores, stream)) {
    used = &wm;  // 16-bit K/V: stage 1 ran on the matrix-core kernel
  } else
  switch (G) {
    case 1: launch_stage1<T, 1>(q, rows, hq, hkv, batch, scale, w, with_v, want_scores, stream); break;
    case 2: launch_stage1<T, 2>(q, rows, hq, hkv, batch, scale, w, with_v, want_scores, stream); break;
    case 4: launch_stage1<T, 4>(q, rows, hq, hkv, batch, scale, w, with_v, want_scores, stream); break;
    case 8: launch_stage1<T, 8>(q, rows, hq, hkv, batch, scale, w, with_v, want_scores, stream); break;
    default: set_error("GQA group %d not supported", G); return OKV_ERR_UNSUPPORTED;
  }
  const bool need_score_lse = want_scores && normalise == OKV_NORM_SOFTMAX;
  const int ftok = finish_tokens_for(w.split_rows, rows.max_score_len);
  const int finish_blocks = want_scores ? (rows.max_score_len + ftok - 1) / ftok : 0;
  const AttnWorkspace& uw = *used;
#ifdef OKV_DIAG
  if (g_split_pass_only.load(std::memory_order_relaxed)) return OKV_OK;  // measurement hook: the split pass alone
#endif
  if (finish_blocks > 0 && hq <= kMaxFinishHeads) {
    // one launch: the merge of the outputs next to the finishing of the scores
    const dim3 grid((with_v ? hq : 0) + finish_blocks, batch);
    if (ftok == 512)
      hipLaunchKernelGGL((merge_and_finish<T, 2>), grid, dim3(256), 0, stream, rows, hq, uw, (T*)out,
                         with_v ? hq : 0, head_reduce, normalise, scores, score_stride);
    else
      hipLaunchKernelGGL((merge_and_finish<T, 4>), grid, dim3(256), 0, stream, rows, hq, uw, (T*)out,
                         with_v ? hq : 0, head_reduce, normalise, scores, score_stride);
  } else {
    if (with_v || need_score_lse)
      hipLaunchKernelGGL((attn_merge<T>), dim3(hq, batch), dim3(256), 0, stream, rows, hq, uw,
                         (T*)out, (int)with_v, (int)need_score_lse);
    if (finish_blocks > 0) {
      if (ftok == 512)
        hipLaunchKernelGGL(score_finish<2>, dim3(finish_blocks, batch), dim3(256), 0, stream, rows, hq, uw,
                           head_reduce, normalise, scores, score_stride);
      else
        hipLaunchKernelGGL(score_finish<4>, dim3(finish_blocks, batch), dim3(256), 0, stream, rows, hq, uw,
                           head_reduce, normalise, scores, score_stride);
    }
  }
  OKV_HIP_CHECK(hipGetLastError());
  return OKV_OK;
}

int launch_attention(const void* q, const RowList& rows, const okv_kv_layout_t* lay, int batch,
                     float scale, void* out, bool with_v, int head_reduce, int normalise,
                     float* scores, int64_t score_stride, const AttnWorkspace& w,
                     hipStream_t stream) {
  switch (lay->dtype) {
    case OKV_F32:
      return launch_typed<float>(q, rows, lay, batch, scale, out, with_v, head_reduce, normalise,
                                 scores, score_stride, w, stream);
    case OKV_BF16:
      return launch_typed<BF16>(q, rows, lay, batch, scale, out, with_v, head_reduce, normalise,
                                scores, score_stride, w, stream);
    case OKV_F16:
      return launch_typed<F16>(q, rows, lay, batch, scale, out, with_v, head_reduce, normalise,
                               scores, score_stride, w, stream);
  }
  set_error("dtype %d not supported", lay->dtype);
  return OKV_ERR_UNSUPPORTED;
}

bool launch_stage1_window(int dtype, const void* q, const RowList& rows, int hq, int hkv, int batch, float scale,
                          const AttnWorkspace& w, const WindowFuse& wf, hipStream_t stream);

// Dense attention of 16-bit contiguous K/V whose split pass also leaves the window columns'
// partial log-sum-exps (see WindowFuse); the merge of the attention output follows.
int launch_attention_window(const void* q, const RowList& rows, const okv_kv_layout_t* lay, int batch, float scale,
                            void* out, const AttnWorkspace& w, const WindowFuse& wf, hipStream_t stream) {
  const int hq = lay->num_q_heads, hkv = lay->num_kv_heads;
  if (!launch_stage1_window(lay->dtype, q, rows, hq, hkv, batch, scale, w, wf, stream)) {
    set_error("window scoring inside the dense pass needs 16-bit contiguous K/V and window x group <= %d", kWinCols);
    return OKV_ERR_UNSUPPORTED;
  }
  if (lay->dtype == OKV_BF16)
    hipLaunchKernelGGL((attn_window_merge<BF16>), dim3(hq + hkv, batch), dim3(256), 0, stream, rows, hq, hkv, w,
                       (BF16*)out, wf);
  else
    hipLaunchKernelGGL((attn_window_merge<F16>), dim3(hq + hkv, batch), dim3(256), 0, stream, rows, hq, hkv, w,
                       (F16*)out, wf);
  OKV_HIP_CHECK(hipGetLastError());
  return OKV_OK;
}

void fill_main(RowList* r, const void* k, const void* v, const okv_kv_layout_t* lay) {
  memset(r, 0, sizeof(*r));
  r->k_base = k;
  r->v_base = v;
  r->token_stride = lay->token_stride;
  r->head_stride = lay->head_stride;
  r->batch_stride = lay->batch_stride;
  rl_set_pages(r, lay->page_table, lay->page_size, lay->page_table_stride, lay->page_stride);
}

}  // namespace okv

using namespace okv;

extern "C" {

int okv_set_option(const char* name, int value) {
  OKV_REQUIRE(name != nullptr, OKV_ERR_INVALID, "option name is NULL");
  if (strcmp(name, "attn_variant") == 0) {
    OKV_REQUIRE(value == 0 || value == 1, OKV_ERR_INVALID, "attn_variant must be 0 or 1");
    g_attn_variant = value;
    return OKV_OK;
  }
  if (strcmp(name, "split_rows") == 0) {
    OKV_REQUIRE(value == 0 || (value >= 64 && value <= 8192 && value % 16 == 0), OKV_ERR_INVALID,
                "split_rows must be 0 (automatic) or a multiple of 16 in [64, 8192]");
    g_split_rows_override = value;
    return OKV_OK;
  }
  set_error("unknown option %s", name);
  return OKV_ERR_INVALID;
}

#ifdef OKV_STAMPS
// Timeline build only: copies the device timestamps of the last launches out (which: 0 split pass, 1 merge);
// dst holds okv::kStampBlocks * okv::kStampSlots 64-bit values, 10 ns units, 0 where nothing was stamped.
int okv_stamps_read(int which, unsigned long long* dst, int clear) {
  OKV_REQUIRE(dst && (which == 0 || which == 1), OKV_ERR_INVALID, "which must be 0 or 1");
  if (which == 0) return stamps_read_split(dst, clear);
  const size_t bytes = sizeof(unsigned long long) * kStampBlocks * kStampSlots;
  OKV_HIP_CHECK(hipMemcpyFromSymbol(dst, HIP_SYMBOL(g_merge_stamps), bytes));
  if (clear) {
    void* p = nullptr;
    OKV_HIP_CHECK(hipGetSymbolAddress(&p, HIP_SYMBOL(g_merge_stamps)));
    OKV_HIP_CHECK(hipMemset(p, 0, bytes));
  }
  return OKV_OK;
}
#endif

#ifdef OKV_DIAG
// Measurement hook of the measurement build (compiled with -DOKV_DIAG into libomnikv_hip_diag.so; the
// product library does not contain it): with 1 the attention / scoring entry points launch their
// split pass alone (outputs are then not produced), so that a timer around the call measures that
// kernel.  Process-wide.
int okv_diag_split_pass_only(int on) {
  g_split_pass_only.store(on ? 1 : 0, std::memory_order_relaxed);
  return OKV_OK;
}
#endif

int okv_score(const void* q, const void* k_base, const okv_kv_layout_t* layout,
              const int32_t* score_lens, int32_t max_score_len, int32_t batch,
              int32_t head_reduce, int32_t normalise, float scale, float* scores,
              int64_t score_stride, void* ws, size_t ws_bytes, okv_stream_t stream) {
  int rc = validate_layout(layout, k_base, k_base);
  if (rc) return rc;
  OKV_REQUIRE(q && scores, OKV_ERR_INVALID, "q or scores is NULL");
  OKV_REQUIRE(batch >= 1 && max_score_len >= 0, OKV_ERR_INVALID, "bad batch or length");
  OKV_REQUIRE(score_stride >= max_score_len, OKV_ERR_INVALID, "score_stride < max_score_len");
  OKV_REQUIRE(head_reduce == OKV_REDUCE_MAX || head_reduce == OKV_REDUCE_SUM, OKV_ERR_INVALID,
              "bad head_reduce %d", head_reduce);
  OKV_REQUIRE(normalise == OKV_NORM_RAW || normalise == OKV_NORM_SOFTMAX, OKV_ERR_INVALID,
              "bad normalise %d", normalise);
  if (max_score_len == 0) return OKV_OK;
  AttnWorkspace w;
  rc = carve_attn_workspace(ws, ws_bytes, batch, layout->num_q_heads, layout->num_kv_heads,
                            layout->head_dim, max_score_len, 0, max_score_len, false, true, &w);
  if (rc) return rc;
  RowList r;
  fill_main(&r, k_base, k_base, layout);
  r.main_lens = score_lens;
  r.max_main_len = max_score_len;
  r.score_lens = score_lens;
  r.max_score_len = max_score_len;
  return launch_attention(q, r, layout, batch, scale, nullptr, false, head_reduce, normalise,
                          scores, score_stride, w, (hipStream_t)stream);
}

int okv_dense_attn(const void* q, const void* k_base, const void* v_base,
                   const okv_kv_layout_t* layout, const int32_t* seq_lens, int32_t max_seq_len,
                   int32_t batch, float scale, void* out, const int32_t* score_lens,
                   int32_t max_score_len, int32_t head_reduce, int32_t normalise, float* scores,
                   int64_t score_stride, void* ws, size_t ws_bytes, okv_stream_t stream) {
  int rc = validate_layout(layout, k_base, v_base);
  if (rc) return rc;
  OKV_REQUIRE(q && out && v_base, OKV_ERR_INVALID, "q, v_base or out is NULL");
  OKV_REQUIRE(batch >= 1 && max_seq_len >= 1, OKV_ERR_INVALID, "bad batch or length");
  if (scores) {
    OKV_REQUIRE(max_score_len >= 0 && max_score_len <= max_seq_len, OKV_ERR_INVALID,
                "max_score_len out of range");
    OKV_REQUIRE(score_stride >= max_score_len, OKV_ERR_INVALID, "score_stride < max_score_len");
    OKV_REQUIRE(head_reduce == OKV_REDUCE_MAX || head_reduce == OKV_REDUCE_SUM, OKV_ERR_INVALID,
                "bad head_reduce %d", head_reduce);
    OKV_REQUIRE(normalise == OKV_NORM_RAW || normalise == OKV_NORM_SOFTMAX, OKV_ERR_INVALID,
                "bad normalise %d", normalise);
  } else {
    max_score_len = 0;
    score_lens = nullptr;
  }
  AttnWorkspace w;
  // raw scores of 16-bit K are folded per kv head inside the pass: a quarter of the logits to stage, longer splits
  const bool folds = scores && normalise == OKV_NORM_RAW && layout->dtype != OKV_F32 &&
                     layout->num_q_heads > layout->num_kv_heads;
  rc = carve_attn_workspace(ws, ws_bytes, batch, layout->num_q_heads, layout->num_kv_heads,
                            layout->head_dim, max_seq_len, 0, max_score_len, true,
                            scores != nullptr, &w, folds ? 3 : 0);
  if (rc) return rc;
  RowList r;
  fill_main(&r, k_base, v_base, layout);
  r.main_lens = seq_lens;
  r.max_main_len = max_seq_len;
  r.score_lens = score_lens;
  r.max_score_len = max_score_len;
  return launch_attention(q, r, layout, batch, scale, out, true, head_reduce, normalise, scores,
                          score_stride, w, (hipStream_t)stream);
}

int okv_dense_attn_select(const void* q, const void* k_base, const void* v_base,
                          const okv_kv_layout_t* layout, const int32_t* seq_lens, int32_t max_seq_len,
                          int32_t batch, float scale, void* out, const int32_t* score_lens,
                          int32_t max_score_len, int32_t head_reduce, int32_t normalise, float* scores,
                          int64_t score_stride, const int32_t* k_per_seg, int32_t max_k,
                          int32_t* idx_out, int64_t idx_stride, void* ws, size_t ws_bytes,
                          okv_stream_t stream) {
  OKV_REQUIRE(scores && idx_out, OKV_ERR_INVALID, "scores or idx_out is NULL");
  OKV_REQUIRE(layout != nullptr, OKV_ERR_INVALID, "layout is NULL");
  OKV_REQUIRE(batch >= 1 && max_seq_len >= 1 && max_score_len >= 0 && max_score_len <= max_seq_len,
              OKV_ERR_INVALID, "bad batch or length");
  // the attention's partials first, the selection's histograms and candidates behind them
  const size_t attn_bytes = (attn_workspace_bytes(batch, layout->num_q_heads, layout->num_kv_heads,
                                                  layout->head_dim, max_seq_len, 0, max_score_len, true, true,
                                                  nullptr, nullptr) + 255) & ~(size_t)255;
  // long score vectors are selected by many workgroups, which need their own part of the workspace
  const size_t need = attn_bytes + (max_score_len >= kMultiBlockMinLen ? topk_mb_workspace_bytes(batch, max_score_len) : 0);
  OKV_REQUIRE(ws != nullptr, OKV_ERR_INVALID, "workspace pointer is NULL");
  OKV_REQUIRE(ws_bytes >= need, OKV_ERR_WORKSPACE, "workspace too small: have %zu, need %zu", ws_bytes, need);
  int rc = okv_dense_attn(q, k_base, v_base, layout, seq_lens, max_seq_len, batch, scale, out, score_lens,
                          max_score_len, head_reduce, normalise, scores, score_stride, ws, attn_bytes, stream);
  if (rc) return rc;
  return okv_topk(scores, score_stride, score_lens, max_score_len, k_per_seg, max_k, batch, idx_out, idx_stride,
                  (char*)ws + attn_bytes, ws_bytes - attn_bytes, stream);
}

int okv_sparse_attn(const void* q, const void* k_base, const void* v_base,
                    const okv_kv_layout_t* layout, const int32_t* idx, int64_t idx_stride,
                    const int32_t* sel_lens, int32_t max_sel_len, const void* tail_k,
                    const void* tail_v, int64_t tail_token_stride, int64_t tail_head_stride,
                    int64_t tail_batch_stride, const int32_t* tail_lens, int32_t max_tail_len,
                    int32_t batch, float scale, void* out, void* ws, size_t ws_bytes,
                    okv_stream_t stream) {
  int rc = validate_layout(layout, k_base, v_base);
  if (rc) return rc;
  OKV_REQUIRE(q && out && v_base, OKV_ERR_INVALID, "q, v_base or out is NULL");
  OKV_REQUIRE(batch >= 1 && max_sel_len >= 0 && max_tail_len >= 0, OKV_ERR_INVALID,
              "bad batch or length");
  OKV_REQUIRE(max_sel_len + max_tail_len >= 1, OKV_ERR_INVALID, "no rows to attend to");
  if (idx) OKV_REQUIRE(idx_stride >= max_sel_len, OKV_ERR_INVALID, "idx_stride < max_sel_len");
  if (max_tail_len > 0) {
    OKV_REQUIRE(tail_k && tail_v, OKV_ERR_INVALID, "tail pointers are NULL");
    OKV_REQUIRE(((uintptr_t)tail_k & 15) == 0 && ((uintptr_t)tail_v & 15) == 0, OKV_ERR_INVALID,
                "tail pointers must be 16-byte aligned");
    OKV_REQUIRE(tail_token_stride % 8 == 0 && tail_head_stride % 8 == 0 &&
                    tail_batch_stride % 8 == 0,
                OKV_ERR_INVALID, "tail strides must be multiples of 8 elements");
  }
  AttnWorkspace w;
  rc = carve_attn_workspace(ws, ws_bytes, batch, layout->num_q_heads, layout->num_kv_heads,
                            layout->head_dim, max_sel_len, max_tail_len, 0, true, false, &w, true);
  if (rc) return rc;
  RowList r;
  fill_main(&r, k_base, v_base, layout);
  r.idx = idx;
  r.idx_stride = idx_stride;
  r.main_lens = sel_lens;
  r.max_main_len = max_sel_len;
  r.tail_k = tail_k;
  r.tail_v = tail_v;
  r.tail_token_stride = tail_token_stride;
  r.tail_head_stride = tail_head_stride;
  r.tail_batch_stride = tail_batch_stride;
  r.tail_lens = tail_lens;
  r.max_tail_len = max_tail_len;
  return launch_attention(q, r, layout, batch, scale, out, true, 0, 0, nullptr, 0, w,
                          (hipStream_t)stream);
}

// ---------------------------------------------------------------------------
// Sparse attention for callers that can neither allocate nor bring a workspace: the
// per-(q head, split) partials live in a fixed array of the library's own, one copy per
// GPU.  Host code never passes the array's name to a kernel (on the host it is only a
// stand-in): the device address is asked for once per device and used from then on.
constexpr size_t kScratchBytes = (size_t)4 << 20;
static __device__ __align__(256) unsigned char scratch[kScratchBytes];
constexpr int kMaxScratchDevices = 64;
static void* g_scratch_ptr[kMaxScratchDevices];  // [device] -> that GPU's copy of `scratch`
static std::mutex g_scratch_mutex;

static int scratch_of_current_device(void** out) {
  int dev = -1;
  OKV_HIP_CHECK(hipGetDevice(&dev));
  OKV_REQUIRE(dev >= 0 && dev < kMaxScratchDevices, OKV_ERR_UNSUPPORTED, "device %d: at most %d devices", dev,
              kMaxScratchDevices);
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (g_scratch_ptr[dev] == nullptr) {
    void* p = nullptr;
    OKV_HIP_CHECK(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
    OKV_REQUIRE(p != nullptr, OKV_ERR_HIP, "hipGetSymbolAddress returned a NULL address");
    g_scratch_ptr[dev] = p;
  }
  *out = g_scratch_ptr[dev];
  return OKV_OK;
}

int okv_sparse_attn_noalloc(const void* q, const void* k_base, const void* v_base,
                            const okv_kv_layout_t* layout, const int32_t* idx, int64_t idx_stride,
                            const int32_t* sel_lens, int32_t max_sel_len, const void* tail_k,
                            const void* tail_v, int64_t tail_token_stride, int64_t tail_head_stride,
                            int64_t tail_batch_stride, const int32_t* tail_lens, int32_t max_tail_len,
                            int32_t batch, float scale, void* out, okv_stream_t stream) {
  OKV_REQUIRE(layout != nullptr, OKV_ERR_INVALID, "layout is NULL");
  OKV_REQUIRE(batch >= 1 && max_sel_len >= 0 && max_tail_len >= 0, OKV_ERR_INVALID, "bad batch or length");
  const size_t need = attn_workspace_bytes(batch, layout->num_q_heads, layout->num_kv_heads, layout->head_dim,
                                           max_sel_len, max_tail_len, 0, true, false, nullptr, nullptr, true);
  OKV_REQUIRE(need <= kScratchBytes, OKV_ERR_WORKSPACE,
              "okv_sparse_attn_noalloc: batch %d x (%d selected + %d tail) rows needs %zu bytes of partial "
              "results, the library's fixed scratch holds %zu; use okv_sparse_attn with a workspace",
              batch, max_sel_len, max_tail_len, need, kScratchBytes);
  void* ws = nullptr;
  int rc = scratch_of_current_device(&ws);
  if (rc) return rc;
  // every partial the merge reads is written by the split pass of the same call: nothing to clear
  return okv_sparse_attn(q, k_base, v_base, layout, idx, idx_stride, sel_lens, max_sel_len, tail_k, tail_v,
                         tail_token_stride, tail_head_stride, tail_batch_stride, tail_lens, max_tail_len, batch,
                         scale, out, ws, kScratchBytes, stream);
}

int64_t okv_noalloc_scratch_bytes(void) { return (int64_t)kScratchBytes; }

}  // extern "C"
