// Stage 1 of split-context GQA decode attention for 16-bit K/V on gfx950, with the
// q.K^T contraction on the matrix cores.
//
// A wave owns 16-row tiles of one kv head.  q.K^T for the tile is four
// v_mfma_f32_16x16x32 (K rows are the A operand straight from global memory: lane l
// holds row l%16, elements 32s + 8(l/16) .. +8 of k-step s; the G q heads of the kv
// head are the first G columns of the B operand, the rest zero).  The result leaves
// lane l holding column (head) l%16 of tile rows 4(l/16) .. +4: the lanes of one
// 16-lane row hold all heads of the same four rows, so each row of lanes keeps its
// own online softmax and the probabilities reach the P.V lanes by DPP row
// broadcasts.  P.V is VALU work: lane l owns output elements 8(l%16) .. +8 and
// accumulates the four rows of its lane row, reading V fully coalesced (256 bytes
// per row per 16 lanes).  Next tile's K and V are in flight while the current one
// is consumed.
#include <math.h>

#include "okv_device.h"
#include "okv_internal.h"

namespace okv {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8_t;
typedef __attribute__((ext_vector_type(8))) _Float16 f16x8_t;
typedef __attribute__((ext_vector_type(4))) float f32x4_t;

__device__ __forceinline__ f32x4_t mfma16(const BF16*, const uint4& a, const uint4& b, f32x4_t c) {
  return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, a),
                                                 __builtin_bit_cast(bf16x8_t, b), c, 0, 0, 0);
}
__device__ __forceinline__ f32x4_t mfma16(const F16*, const uint4& a, const uint4& b, f32x4_t c) {
  return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8_t, a),
                                                __builtin_bit_cast(f16x8_t, b), c, 0, 0, 0);
}

// value of lane H of the caller's 16-lane row
template <int H>
__device__ __forceinline__ float row_bcast(float x) {
  return __int_as_float(
      __builtin_amdgcn_update_dpp(0, __float_as_int(x), 0x150 + H, 0xf, 0xf, false));
}

template <int H, int G, bool RESCALE>
struct HeadStep {
  // acc[h][:] (*= alpha_h) += p_h * v[:] for heads H .. G-1
  static __device__ __forceinline__ void fma(float (&acc)[G][8], float p, const float* v) {
    const float ph = row_bcast<H>(p);
#pragma unroll
    for (int d = 0; d < 8; ++d) acc[H][d] = fmaf(ph, v[d], acc[H][d]);
    HeadStep<H + 1, G, RESCALE>::fma(acc, p, v);
  }
  static __device__ __forceinline__ void scale(float (&acc)[G][8], float a) {
    const float ah = row_bcast<H>(a);
#pragma unroll
    for (int d = 0; d < 8; ++d) acc[H][d] *= ah;
    HeadStep<H + 1, G, RESCALE>::scale(acc, a);
  }
};
template <int G, bool R>
struct HeadStep<G, G, R> {
  static __device__ __forceinline__ void fma(float (&)[G][8], float, const float*) {}
  static __device__ __forceinline__ void scale(float (&)[G][8], float) {}
};

struct TileRows {
  int64_t k_off;     // element offset of this lane's K row (kv head and d included)
  int64_t v_off[4];  // element offsets of this lane's four V rows
  bool k_tail, v_tail[4];
};

template <typename T, int G, bool WITH_V, bool SIMPLE>
__global__ __launch_bounds__(256) void attn_stage1_mfma(const T* __restrict__ q, RowList rows,
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
  const int r16 = lane & 15, j4 = lane >> 4;

  // B operand: q heads of this kv head in columns 0..G-1
  uint4 qf[4];
#pragma unroll
  for (int s = 0; s < 4; ++s) {
    qf[s] = make_uint4(0, 0, 0, 0);
    if (r16 < G)
      qf[s] = *reinterpret_cast<const uint4*>(q + ((int64_t)(b * hq + g * G + r16) * kD + 32 * s + 8 * j4));
  }

  const T* kb = reinterpret_cast<const T*>(rows.k_base);
  const T* vb = reinterpret_cast<const T*>(rows.v_base);
  const T* tkb = reinterpret_cast<const T*>(rows.tail_k);
  const T* tvb = reinterpret_cast<const T*>(rows.tail_v);
  const int64_t head_off = (int64_t)g * rows.head_stride;
  const int64_t tail_head_off = (int64_t)g * rows.tail_head_stride;

  auto tile_rows = [&](int tbase, TileRows& tr) {
    const int last = end - 1;
    int kr = tbase + r16;
    kr = kr < last ? kr : last;
    if (SIMPLE) {
      tr.k_tail = false;
      tr.k_off = (int64_t)b * rows.batch_stride + (int64_t)kr * rows.token_stride + head_off + 8 * j4;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        int vr = tbase + 4 * j4 + i;
        vr = vr < last ? vr : last;
        tr.v_tail[i] = false;
        tr.v_off[i] = (int64_t)b * rows.batch_stride + (int64_t)vr * rows.token_stride + head_off + 8 * r16;
      }
    } else {
      tr.k_off = rl_row_offset(rows, b, kr, main_len, &tr.k_tail) +
                 (tr.k_tail ? tail_head_off : head_off) + 8 * j4;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        int vr = tbase + 4 * j4 + i;
        vr = vr < last ? vr : last;
        tr.v_off[i] = rl_row_offset(rows, b, vr, main_len, &tr.v_tail[i]) +
                      (tr.v_tail[i] ? tail_head_off : head_off) + 8 * r16;
      }
    }
  };
  auto load_tile = [&](const TileRows& tr, uint4 (&kf)[4], uint4 (&vf)[4]) {
    const T* kp = (tr.k_tail ? tkb : kb) + tr.k_off;
#pragma unroll
    for (int s = 0; s < 4; ++s) kf[s] = *reinterpret_cast<const uint4*>(kp + 32 * s);
    if (WITH_V) {
#pragma unroll
      for (int i = 0; i < 4; ++i)
        vf[i] = *reinterpret_cast<const uint4*>((tr.v_tail[i] ? tvb : vb) + tr.v_off[i]);
    }
  };

  float m = -INFINITY, l = 0.f;  // softmax state of (head r16, lane row j4)
  float acc[G][8];               // output elements 8*r16.. of the rows of lane row j4
#pragma unroll
  for (int h = 0; h < G; ++h)
#pragma unroll
    for (int d = 0; d < 8; ++d) acc[h][d] = 0.f;
  const float sl2 = scale * kLog2e;

  auto compute = [&](int tbase, const uint4 (&kf)[4], const uint4 (&vf)[4]) {
    f32x4_t S = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int s = 0; s < 4; ++s) S = mfma16((const T*)nullptr, kf[s], qf[s], S);
    const int row0 = tbase + 4 * j4;
    if (write_logits && begin < A && r16 < G && row0 < end) {  // a scored split ends at or before A
      float* lp = w.logits + (int64_t)(b * hq + g * G + r16) * w.logits_stride + row0;
      if (row0 + 3 < end) {
        *reinterpret_cast<float4*>(lp) = make_float4(S[0] * scale, S[1] * scale, S[2] * scale, S[3] * scale);
      } else {
#pragma unroll
        for (int i = 0; i < 4; ++i)
          if (row0 + i < end) lp[i] = S[i] * scale;
      }
    }
    float s2[4];
    float mt = -INFINITY;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      s2[i] = (row0 + i < end) ? S[i] * sl2 : -INFINITY;
      mt = fmaxf(mt, s2[i]);
    }
    const float mn = fmaxf(m, mt);
    const float ms = (mn == -INFINITY) ? 0.f : mn;
    const float alpha = exp2f(m - ms);
    float p[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) p[i] = exp2f(s2[i] - ms);
    l = l * alpha + ((p[0] + p[1]) + (p[2] + p[3]));
    m = mn;
    if (WITH_V) {
      const bool changed = (r16 < G) && (alpha != 1.0f);
      if (__ballot(changed) != 0ull) HeadStep<0, G, true>::scale(acc, alpha);
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        float v[8];
        cvt8((const T*)nullptr, vf[i], v);
        HeadStep<0, G, false>::fma(acc, p[i], v);
      }
    }
  };

  // ---- tiles of this wave: begin + 16*(wave + 4*n), software-pipelined by one tile
  uint4 kA[4], vA[4], kB[4], vB[4];
  TileRows tr;
  int t = begin + wave * 16;
  if (t < end) {
    tile_rows(t, tr);
    load_tile(tr, kA, vA);
    while (true) {
      int tn = t + 64;
      bool more = tn < end;
      if (more) {
        tile_rows(tn, tr);
        load_tile(tr, kB, vB);
      }
      compute(t, kA, vA);
      if (!more) break;
      t = tn;
      tn = t + 64;
      more = tn < end;
      if (more) {
        tile_rows(tn, tr);
        load_tile(tr, kA, vA);
      }
      compute(t, kB, vB);
      if (!more) break;
      t = tn;
    }
  }

  // ---- merge the four lane rows of the wave
  float M = fmaxf(m, __shfl_xor(m, 16));
  M = fmaxf(M, __shfl_xor(M, 32));
  const float f = (m == -INFINITY) ? 0.f : exp2f(m - M);
  float lw = l * f;
  lw += __shfl_xor(lw, 16);
  lw += __shfl_xor(lw, 32);
  if (WITH_V) {
    HeadStep<0, G, true>::scale(acc, f);
#pragma unroll
    for (int h = 0; h < G; ++h)
#pragma unroll
      for (int d = 0; d < 8; ++d) {
        float a = acc[h][d];
        a += __shfl_xor(a, 16);
        a += __shfl_xor(a, 32);
        acc[h][d] = a;
      }
  }

  // ---- merge the four waves through LDS and write the split's partial
  __shared__ float sm[4][G];
  __shared__ float sl[4][G];
  __shared__ float sacc[WITH_V ? 4 : 1][G][kD];
  if (j4 == 0) {
    if (r16 < G) {
      sm[wave][r16] = M;
      sl[wave][r16] = lw;
    }
    if (WITH_V) {
#pragma unroll
      for (int h = 0; h < G; ++h)
#pragma unroll
        for (int d = 0; d < 8; ++d) sacc[wave][h][r16 * 8 + d] = acc[h][d];
    }
  }
  __syncthreads();
  for (int o = threadIdx.x; o < G * kD; o += 256) {
    const int h = o / kD, d = o % kD;
    const float Mb = fmaxf(fmaxf(sm[0][h], sm[1][h]), fmaxf(sm[2][h], sm[3][h]));
    float den = 0.f, num = 0.f;
#pragma unroll
    for (int x = 0; x < 4; ++x) {
      const float fx = (sm[x][h] == -INFINITY) ? 0.f : exp2f(sm[x][h] - Mb);
      den += sl[x][h] * fx;
      if (WITH_V) num += sacc[x][h][d] * fx;
    }
    const int64_t ph = (int64_t)(b * hq + g * G + h) * w.max_splits + split;
    if (WITH_V) w.part_o[ph * kD + d] = num / den;
    if (d == 0) w.part_lse[ph] = Mb + log2f(den);
  }
}

template <typename T, int G>
static void launch_g(const void* q, const RowList& rows, int hq, int hkv, int batch, float scale,
                     const AttnWorkspace& w, bool with_v, bool write_logits, hipStream_t stream) {
  dim3 grid(hkv, w.max_splits, batch);  // kv head fastest: co-resident blocks cover whole token rows
  const bool simple = !rows.idx && !rows.page_table && rows.max_tail_len == 0 && !rows.tail_lens;
#define OKV_LAUNCH(WV, SI)                                                                    \
  hipLaunchKernelGGL((attn_stage1_mfma<T, G, WV, SI>), grid, dim3(256), 0, stream, (const T*)q, \
                     rows, hq, scale, w, (int)write_logits)
  if (with_v) {
    if (simple) OKV_LAUNCH(true, true);
    else OKV_LAUNCH(true, false);
  } else {
    if (simple) OKV_LAUNCH(false, true);
    else OKV_LAUNCH(false, false);
  }
#undef OKV_LAUNCH
}

template <typename T>
static bool launch_t(const void* q, const RowList& rows, int hq, int hkv, int batch, float scale,
                     const AttnWorkspace& w, bool with_v, bool write_logits, hipStream_t stream) {
  switch (hq / hkv) {
    case 1: launch_g<T, 1>(q, rows, hq, hkv, batch, scale, w, with_v, write_logits, stream); return true;
    case 2: launch_g<T, 2>(q, rows, hq, hkv, batch, scale, w, with_v, write_logits, stream); return true;
    case 4: launch_g<T, 4>(q, rows, hq, hkv, batch, scale, w, with_v, write_logits, stream); return true;
    case 8: launch_g<T, 8>(q, rows, hq, hkv, batch, scale, w, with_v, write_logits, stream); return true;
  }
  return false;
}

bool launch_stage1_mfma(int dtype, const void* q, const RowList& rows, int hq, int hkv, int batch,
                        float scale, const AttnWorkspace& w, bool with_v, bool write_logits,
                        hipStream_t stream) {
  if (dtype == OKV_BF16)
    return launch_t<BF16>(q, rows, hq, hkv, batch, scale, w, with_v, write_logits, stream);
  if (dtype == OKV_F16)
    return launch_t<F16>(q, rows, hq, hkv, batch, scale, w, with_v, write_logits, stream);
  return false;
}

}  // namespace okv
