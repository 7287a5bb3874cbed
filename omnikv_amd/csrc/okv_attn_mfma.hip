// Stage 1 of split-context GQA decode attention for 16-bit K/V on gfx950, with the
// q.K^T contraction on the matrix cores.
//
// A wave owns 16-row tiles of one kv head.  q.K^T for the tile is four
// v_mfma_f32_16x16x32 (K rows are the A operand: lane l holds row l%16, elements
// 32s + 8(l/16) .. +8 of k-step s -- loaded in that layout by the gather modes, loaded as
// whole streamed rows and turned into it through LDS by the streaming modes; the G q
// heads of the kv head are the first G columns of the B operand, the rest zero).  The result leaves
// lane l holding column (head) l%16 of tile rows 4(l/16) .. +4 -- which is the A-operand
// layout of v_mfma_f32_16x16x16 with the heads as rows and the tile's 16 rows as the
// contraction.  So P.V runs on the matrix cores too: the probabilities, rounded to the K/V
// element type, are the A operand as they stand, and V, read fully coalesced as whole rows
// (256 bytes per row per 16 lanes: lane l holds elements 8(l%16) .. +8 of rows 4(l/16) .. +4),
// gives eight B operands, one per element position e (column n of block e is output element
// 8n + e), after sixteen v_perm that pair the rows.  The wave keeps ONE running maximum per
// head (a tile whose logits stay below it costs a compare and a ballot; one that raises it,
// two lane-row exchanges and a rescale of the accumulators), so the four waves of the block,
// not sixteen lane rows, meet in LDS at the end.
// The rows of tile t+2 are looked up and the K/V of tile t+1 are in flight while
// tile t is consumed.
#include <math.h>

#include <atomic>

#include "okv_device.h"
#include "okv_internal.h"

namespace okv {

#ifdef OKV_STAMPS
__device__ unsigned long long g_split_stamps[kStampBlocks * kStampSlots];
int stamps_read_split(unsigned long long* dst, int clear) {
  const size_t bytes = sizeof(unsigned long long) * kStampBlocks * kStampSlots;
  OKV_HIP_CHECK(hipMemcpyFromSymbol(dst, HIP_SYMBOL(g_split_stamps), bytes));
  if (clear) {
    void* p = nullptr;
    OKV_HIP_CHECK(hipGetSymbolAddress(&p, HIP_SYMBOL(g_split_stamps)));
    OKV_HIP_CHECK(hipMemset(p, 0, bytes));
  }
  return OKV_OK;
}
#endif
// split pass timeline (gather mode, three-tile shares): 0 entry, 1 query loads issued, 2 index loads issued,
// 3 first tile's row loads issued, 4 all row loads issued, 5 first tile consumed, 6 last tile consumed, 7 end
#define SPLIT_STAMP(i) do { if (MODE == 1) OKV_STAMP(g_split_stamps, blockIdx.y * gridDim.x + blockIdx.x, i); } while (0)

// two fp32 -> one dword of two 16-bit elements (first argument in the low half)
__device__ __forceinline__ uint32_t pack2(const BF16*, float a, float b) {
  f32x2_t x = {a, b};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(x, bf16x2_t));
}
__device__ __forceinline__ uint32_t pack2(const F16*, float a, float b) {
  f32x2_t x = {a, b};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(x, f16x2_t));
}
// D(16 heads x 16 columns) += A(16 heads x 16 rows) . B(16 rows x 16 columns): lane l holds A row
// l%16 / B column l%16, contraction elements 4(l/16) .. +4, and D column l%16, rows 4(l/16) .. +4.
typedef __attribute__((ext_vector_type(4))) short s16x4_t;
typedef __attribute__((ext_vector_type(4))) _Float16 f16x4_t;
__device__ __forceinline__ f32x4_t mfma16k16(const BF16*, uint32_t a0, uint32_t a1, uint32_t b0, uint32_t b1, f32x4_t c) {
  const uint2 a = make_uint2(a0, a1), b = make_uint2(b0, b1);
  return __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(__builtin_bit_cast(s16x4_t, a), __builtin_bit_cast(s16x4_t, b), c,
                                                   0, 0, 0);
}
__device__ __forceinline__ f32x4_t mfma16k16(const F16*, uint32_t a0, uint32_t a1, uint32_t b0, uint32_t b1, f32x4_t c) {
  const uint2 a = make_uint2(a0, a1), b = make_uint2(b0, b1);
  return __builtin_amdgcn_mfma_f32_16x16x16f16(__builtin_bit_cast(f16x4_t, a), __builtin_bit_cast(f16x4_t, b), c, 0,
                                               0, 0);
}

// value of lane H of the caller's 16-lane row
template <int H>
__device__ __forceinline__ uint32_t row_bcast(uint32_t x) {
  return (uint32_t)__builtin_amdgcn_update_dpp((int)x, (int)x, 0x150 + H, 0xf, 0xf, true);
}
template <int H>
__device__ __forceinline__ float row_bcast_f(float x) {
  return __uint_as_float(row_bcast<H>(__float_as_uint(x)));
}

// max / sum over the four lane rows (lanes l, l^16, l^32, l^48), left in all of them
__device__ __forceinline__ float lane_rows_max(float x) {
  auto a = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
  x = fmaxf(__uint_as_float(a[0]), __uint_as_float(a[1]));
  auto b = __builtin_amdgcn_permlane16_swap(__float_as_uint(x), __float_as_uint(x), false, false);
  return fmaxf(__uint_as_float(b[0]), __uint_as_float(b[1]));
}
__device__ __forceinline__ float lane_rows_sum(float x) {
  auto a = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
  x = __uint_as_float(a[0]) + __uint_as_float(a[1]);
  auto b = __builtin_amdgcn_permlane16_swap(__float_as_uint(x), __float_as_uint(x), false, false);
  return __uint_as_float(b[0]) + __uint_as_float(b[1]);
}

// The P.V accumulators of a wave: acc[e][i] of lane l is output element 8(l%16) + e of head
// 4(l/16) + i.  Heads beyond G (lane rows beyond G/4) accumulate the zero-query columns and are
// never read.
template <int G>
__device__ __forceinline__ void scale_heads(f32x4_t (&acc)[8], float alpha, int j4) {
  float a[4] = {row_bcast_f<0>(alpha), row_bcast_f<1>(alpha), row_bcast_f<2>(alpha), row_bcast_f<3>(alpha)};
  if (G > 4) {
    const float b[4] = {row_bcast_f<4>(alpha), row_bcast_f<5>(alpha), row_bcast_f<6>(alpha), row_bcast_f<7>(alpha)};
#pragma unroll
    for (int i = 0; i < 4; ++i) a[i] = (j4 & 1) ? b[i] : a[i];
  }
#pragma unroll
  for (int e = 0; e < 8; ++e)
#pragma unroll
    for (int i = 0; i < 4; ++i) acc[e][i] *= a[i];
}

// What a lane needs to know about the rows of a tile before it can address them:
// the K row (index 0) and its four V rows (1..4).
struct TileRows {
  int32_t tok[5];  // token (or page) the row maps to; raw load results
  int32_t row[5];  // logical row, clamped into the split
  bool direct;     // wave-uniform: all 16 rows are selected rows of the split -- tok[0] is the token of row
                   // r16 (the lane's K row), tok[1] that of row 4*j4 + r16%4 (its quad holds the four V rows)
};

// value of lane I of the caller's quad
template <int I>
__device__ __forceinline__ uint32_t quad_bcast(uint32_t x) {
  return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)x, I * 0x55, 0xf, 0xf, true);
}

template <int G>
__host__ __device__ constexpr int stage1_lds_floats(bool with_v) {
  return 2 * 4 * G + 8 + (with_v ? 4 * G * kD : 0);  // per wave and head: max, sum, partial output
}
constexpr int kWindowLdsFloats = 2 * 16 * kWinCols;  // [16 lane rows][64 columns] running max and sum

// The streaming modes (0, 3) load K as whole rows and transpose the tile in LDS (see
// k_rows_to_a_operand); the gather modes keep the direct A-operand loads: their pass is a
// chain of latencies and the detour adds to it (measured: 13.5 vs 13.1 us at 8781 rows).
__host__ __device__ constexpr bool stage1_k_through_lds(int mode) { return mode == 0 || mode == 3; }
__host__ __device__ constexpr bool stage1_gathers(int mode) { return mode == 1 || mode == 4; }  // main rows + tail, two "tokens" per lane

// MODE 0: contiguous rows, no index, no tail.  MODE 1: rows through idx (no page table),
// optional tail.  MODE 2: anything (page tables, idx or not, tail or not).  MODE 3: page
// table with pages of 2^n >= 16 rows, no index, no tail (a tile never straddles a page).
// MODE 4: contiguous rows followed by a tail (selected rows staged from the host tier): MODE 1
// with the row number in place of the index lookup.
// WINDOW: the tiles of the scored splits also meet the W x G window query rows of the kv head
// (four more 16-column B operands: column c is position c / G, q head g*G + c % G) and every
// column keeps the running max and sum of its logits; nothing else changes.
template <typename T, int G, bool WITH_V, int MODE, bool LOGITS, bool WINDOW>
__device__ __forceinline__ void stage1_mfma_body(const T* __restrict__ q, const RowList& rows, int hq, float scale,
                                                 const AttnWorkspace& w, const WindowFuse& wf) {
  extern __shared__ float lds[];
  SPLIT_STAMP(0);
  constexpr bool KLDS = stage1_k_through_lds(MODE);
  const int g = blockIdx.x, split = blockIdx.y, b = blockIdx.z;
  const int main_len = rl_main_len(rows, b);
  const int L = main_len + rl_tail_len(rows, b);
  const int A = rl_score_len(rows, b);
  int begin, end;
  rl_split_range(split, w.split_rows, A, L, &begin, &end);
  if (begin >= end) return;

  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);  // scalar: tile bases and the paths below are wave-uniform
  const int r16 = lane & 15, j4 = lane >> 4;

  // B operand: q heads of this kv head in columns 0..G-1; the columns beyond repeat head G-1 (their
  // results are never read, and unconditional loads keep the prologue free of branches)
  uint4 qf[4];
  {
    const int hcol = r16 < G ? r16 : G - 1;
    const T* qp = q + ((int64_t)(b * hq + g * G + hcol) * kD + 8 * j4);
#pragma unroll
    for (int s = 0; s < 4; ++s) qf[s] = *reinterpret_cast<const uint4*>(qp + 32 * s);
  }

  SPLIT_STAMP(1);
  constexpr int WCB = WINDOW ? kWinCols / 16 : 1;
  uint4 wqf[WCB][4];
  float wm[WCB], wl[WCB];  // per column block: state of (column r16, lane row j4), max in raw units
  const bool wscored = WINDOW && begin < A;  // a scored split ends at or before A
  if (WINDOW) {
#pragma unroll
    for (int cb = 0; cb < WCB; ++cb) {
      const int c = 16 * cb + r16;
      const int wpos = c / G, hg = c % G;
      const bool valid = wpos < wf.window;
      const T* qp = reinterpret_cast<const T*>(wf.wq) + (int64_t)b * wf.q_batch_stride +
                    (int64_t)(g * G + hg) * wf.q_head_stride + (int64_t)(valid ? wpos : 0) * wf.q_pos_stride + 8 * j4;
#pragma unroll
      for (int s = 0; s < 4; ++s) {
        const uint4 v = *reinterpret_cast<const uint4*>(qp + 32 * s);
        wqf[cb][s] = valid ? v : make_uint4(0, 0, 0, 0);
      }
      wm[cb] = -INFINITY;
      wl[cb] = 0.f;
    }
  }

  const T* kb = reinterpret_cast<const T*>(rows.k_base) + (int64_t)b * rows.batch_stride +
                (int64_t)g * rows.head_stride;
  const T* vb = reinterpret_cast<const T*>(rows.v_base) + (int64_t)b * rows.batch_stride +
                (int64_t)g * rows.head_stride;
  const T* tkb = reinterpret_cast<const T*>(rows.tail_k) + (int64_t)b * rows.tail_batch_stride +
                 (int64_t)g * rows.tail_head_stride;
  const T* tvb = reinterpret_cast<const T*>(rows.tail_v) + (int64_t)b * rows.tail_batch_stride +
                 (int64_t)g * rows.tail_head_stride;
  const T* pkb = reinterpret_cast<const T*>(rows.k_base) + (int64_t)g * rows.head_stride;  // paged
  const T* pvb = reinterpret_cast<const T*>(rows.v_base) + (int64_t)g * rows.head_stride;
  const uint32_t ts = (uint32_t)rows.token_stride, tts = (uint32_t)rows.tail_token_stride;
  const int last = end - 1;
  const bool tiles_aligned = (begin & 15) == 0;  // block-uniform; every tile base is begin + 16*i

  // ---- which rows a tile touches (issues the index / page-table loads)
  const int32_t* idx_row = rows.idx + (int64_t)b * rows.idx_stride;
  // Gather mode: two index loads per lane and tile -- the lane's K row (tile row r16) and one of its lane
  // row's four V rows (tile row 4*j4 + r16%4; a quad holds the four between its lanes).  Both are always
  // issued from clamped positions, so every tile has the same loads in flight; a row of the tail
  // segment is carried as the complement of its position there (negative).  Tiles that lie wholly
  // inside the selected rows of the split take the short address arithmetic.
  constexpr bool GATHERS = stage1_gathers(MODE);
  const int direct_end = GATHERS ? min(main_len, end) : 0;
  auto gather_tok = [&](int r) -> int32_t {
    r = r < last ? r : last;
    int ri = r < main_len ? r : main_len - 1;
    ri = ri < 0 ? 0 : ri;  // a request with tail rows only: the index still holds one entry
    const int32_t t = MODE == 1 ? idx_row[ri] : ri;
    const int32_t in_tail = (main_len - 1 - r) >> 31;  // all ones for a tail row
    return t ^ ((t ^ ~(r - main_len)) & in_tail);
  };
  auto tile_rows = [&](int tbase, TileRows& tr) {
    if (GATHERS) {
      tr.direct = __builtin_amdgcn_readfirstlane(tbase) + 16 <= direct_end;
      tr.tok[0] = gather_tok(tbase + r16);
      tr.tok[1] = gather_tok(tbase + 4 * j4 + (r16 & 3));
      return;
    }
#pragma unroll
    for (int x = 0; x < 5; ++x) {
      int r = x == 0 ? tbase + r16 : tbase + 4 * j4 + (x - 1);
      r = r < last ? r : last;
      tr.row[x] = r;
      if (MODE == 0) {
        tr.tok[x] = r;
      } else if (MODE == 3) {
        // pages of 16k rows: a tile that starts on a multiple of 16 lies in one page, looked up
        // once through the scalar unit.  The splits behind a scoring boundary that is not a
        // multiple of 16 start wherever it is: their tiles straddle pages, one lookup per row.
        if (tiles_aligned) {
          const int tb = __builtin_amdgcn_readfirstlane(tbase);
          tr.tok[x] = rows.page_table[(int64_t)b * rows.page_table_stride + (tb >> rows.page_shift)];
        } else {
          tr.tok[x] = rows.page_table[(int64_t)b * rows.page_table_stride + (r >> rows.page_shift)];
        }
      } else if (r >= main_len) {
        tr.tok[x] = r - main_len;
      } else {
        int t = rows.idx ? idx_row[r] : r;
        if (rows.page_table) {
          tr.row[x] = -1 - rl_slot_of(rows, t);  // slot in page, tagged as paged
          t = rows.page_table[(int64_t)b * rows.page_table_stride + rl_page_of(rows, t)];
        }
        tr.tok[x] = t;
      }
    }
  };
  auto row_ptr = [&](const TileRows& tr, int x, bool is_v) -> const T* {
    if (MODE == 0) return (is_v ? vb : kb) + (uint64_t)(uint32_t)tr.tok[x] * ts;
    if (MODE == 3)
      return (is_v ? pvb : pkb) + (int64_t)tr.tok[x] * rows.page_stride +
             (uint64_t)(uint32_t)(tr.row[x] & (rows.page_size - 1)) * ts;
    if (tr.row[x] >= main_len) return (is_v ? tvb : tkb) + (uint64_t)(uint32_t)tr.tok[x] * tts;
    if (tr.row[x] < 0)
      return (is_v ? pvb : pkb) + (int64_t)tr.tok[x] * rows.page_stride +
             (uint64_t)(uint32_t)(-1 - tr.row[x]) * ts;
    return (is_v ? vb : kb) + (uint64_t)(uint32_t)tr.tok[x] * ts;
  };
  auto load_tile = [&](const TileRows& tr, uint4 (&kf)[4], uint4 (&vf)[4]) {
    if (GATHERS) {
      // a row's address from its (possibly complemented) token: selected rows of K / V, or rows of the tail
      auto addr = [&](int32_t e, bool is_v) -> const T* {
        const bool in_tail = e < 0;
        const uint32_t t = in_tail ? ~e : e;
        return (in_tail ? (is_v ? tvb : tkb) : (is_v ? vb : kb)) + (uint64_t)t * (in_tail ? tts : ts);
      };
      const int32_t e4[4] = {(int32_t)quad_bcast<0>(tr.tok[1]), (int32_t)quad_bcast<1>(tr.tok[1]),
                             (int32_t)quad_bcast<2>(tr.tok[1]), (int32_t)quad_bcast<3>(tr.tok[1])};
      if (tr.direct) {  // wave-uniform: no tail row in the tile
        const T* kp = kb + (uint64_t)(uint32_t)tr.tok[0] * ts + 8 * j4;
#pragma unroll
        for (int s = 0; s < 4; ++s) kf[s] = *reinterpret_cast<const uint4*>(kp + 32 * s);
        if (WITH_V) {
#pragma unroll
          for (int i = 0; i < 4; ++i) vf[i] = load_stream16(vb + (uint64_t)(uint32_t)e4[i] * ts + 8 * r16);
        }
      } else {
        const T* kp = addr(tr.tok[0], false) + 8 * j4;
#pragma unroll
        for (int s = 0; s < 4; ++s) kf[s] = *reinterpret_cast<const uint4*>(kp + 32 * s);
        if (WITH_V) {
#pragma unroll
          for (int i = 0; i < 4; ++i) vf[i] = load_stream16(addr(e4[i], true) + 8 * r16);
        }
      }
      return;
    }
    if (KLDS) {
      // whole rows, like V; compute() turns the tile into the A-operand layout through LDS
#pragma unroll
      for (int i = 0; i < 4; ++i) kf[i] = load_stream16(row_ptr(tr, 1 + i, false) + 8 * r16);
    } else {
      const T* kp = row_ptr(tr, 0, false) + 8 * j4;
#pragma unroll
      for (int s = 0; s < 4; ++s) kf[s] = *reinterpret_cast<const uint4*>(kp + 32 * s);
    }
    if (WITH_V) {
      // V rows are consumed whole (256 bytes per 16 lanes) and never read again in this launch:
      // streamed.  K in the direct layout is not: a row's 128-byte lines are consumed by two
      // consecutive loads, and a streamed line can leave L1 between them (measured: slower).
#pragma unroll
      for (int i = 0; i < 4; ++i)
        vf[i] = load_stream16(row_ptr(tr, 1 + i, true) + 8 * r16);
    }
  };

  float m = -INFINITY;  // running max of head r16 over the wave's rows so far (the same in all four lane rows); raw q.k units
  float l = 0.f;        // sum of exp over the rows of lane row j4, relative to m
  f32x4_t acc[8];       // acc[e][i]: output element 8*r16 + e of head 4*j4 + i, summed over the wave's rows
#pragma unroll
  for (int e = 0; e < 8; ++e) acc[e] = f32x4_t{0.f, 0.f, 0.f, 0.f};
  const float sl2 = scale * kLog2e;
  const bool scored = LOGITS && begin < A;  // a scored split ends at or before A
  float* slog = lds;  // [G or 1][split_rows] scaled logits of the split; flushed before LDS is reused below

  // K staging of the streaming modes: 4 KB per wave behind everything else the block keeps in LDS
  int kst_off = stage1_lds_floats<G>(WITH_V);
  const int staged = (w.group_reduce ? 1 : G) * w.split_rows;  // one logits row per q head, or per kv head when folded
  if (LOGITS && staged > kst_off) kst_off = staged;
  float* wlds = lds + kst_off;  // the window columns' states meet here at the end
  if (WINDOW) kst_off += kWindowLdsFloats;
  char* kstage = reinterpret_cast<char*>(lds + kst_off) + wave * 4096;
  auto compute = [&](int tbase, const uint4 (&kf_in)[4], const uint4 (&vf)[4]) {
    float s[4];
    uint4 kf[4];
    if (KLDS) {
      k_rows_to_a_operand(kstage, r16, j4, kf_in, kf);
    } else {
#pragma unroll
      for (int s = 0; s < 4; ++s) kf[s] = kf_in[s];
    }
    f32x4_t S = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int s = 0; s < 4; ++s) S = mfma16((const T*)nullptr, kf[s], qf[s], S);
    const int row0 = tbase + 4 * j4;
    const bool partial = tbase + 16 > end;  // wave-uniform
    if (WINDOW) {
      if (wscored) {
#pragma unroll
        for (int cb = 0; cb < WCB; ++cb) {
          f32x4_t W = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
          for (int s = 0; s < 4; ++s) W = mfma16((const T*)nullptr, kf[s], wqf[cb][s], W);
          float sv[4] = {W[0], W[1], W[2], W[3]};
          if (partial) {
#pragma unroll
            for (int i = 0; i < 4; ++i)
              if (row0 + i >= end) sv[i] = -INFINITY;
          }
          const float mn = fmaxf(fmaxf(fmaxf(sv[0], sv[1]), fmaxf(sv[2], sv[3])), wm[cb]);
          const float ms = mn == -INFINITY ? 0.f : mn;
          const float neg = -ms * sl2;
          const float alpha = __builtin_amdgcn_exp2f((wm[cb] - ms) * sl2);
          float pw = 0.f;
#pragma unroll
          for (int i = 0; i < 4; ++i) pw += __builtin_amdgcn_exp2f(fmaf(sv[i], sl2, neg));
          wl[cb] = fmaf(wl[cb], alpha, pw);
          wm[cb] = mn;
        }
      }
    }
    if (scored) {  // staged in LDS, flushed after the loop: no global store in the loop
      float v[4] = {S[0] * scale, S[1] * scale, S[2] * scale, S[3] * scale};
      if (w.group_reduce) {  // raw scores: fold the G q heads (lanes 0..G-1 of the lane row) here
#pragma unroll
        for (int i = 0; i < 4; ++i) {
#pragma unroll
          for (int o = 1; o < G; o <<= 1) {
            const float x = __shfl_xor(v[i], o);
            v[i] = w.group_reduce == 1 ? fmaxf(v[i], x) : v[i] + x;
          }
        }
      }
      if (r16 < (w.group_reduce ? 1 : G))
        *reinterpret_cast<float4*>(slog + r16 * w.split_rows + (row0 - begin)) =
            make_float4(v[0], v[1], v[2], v[3]);
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) s[i] = S[i];
    if (partial) {
#pragma unroll
      for (int i = 0; i < 4; ++i)
        if (row0 + i >= end) s[i] = -INFINITY;
    }
    const float ml = fmaxf(fmaxf(s[0], s[1]), fmaxf(s[2], s[3]));
    if (__ballot(ml > m) != 0ull) {  // some head's max moves (always on the wave's first tile)
      const float mn = lane_rows_max(fmaxf(ml, m));
      const float alpha = __builtin_amdgcn_exp2f((m - (mn == -INFINITY ? 0.f : mn)) * sl2);  // 1 for a head whose max stands
      l *= alpha;
      if (WITH_V) scale_heads<G>(acc, alpha, j4);  // nothing accumulated yet on the first tile
      m = mn;
    }
    const float neg = (m == -INFINITY ? 0.f : -m) * sl2;
    float p[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) p[i] = __builtin_amdgcn_exp2f(fmaf(s[i], sl2, neg));
    l += (p[0] + p[1]) + (p[2] + p[3]);
    if (WITH_V) {
    // A operand: P of head r16, rows 4*j4 .. +4, as it stands.  B operand of block e: element e of
    // the lane's four V rows.
    const uint32_t p01 = pack2((const T*)nullptr, p[0], p[1]);
    const uint32_t p23 = pack2((const T*)nullptr, p[2], p[3]);
    const uint32_t a[4] = {vf[0].x, vf[0].y, vf[0].z, vf[0].w};
    const uint32_t c[4] = {vf[1].x, vf[1].y, vf[1].z, vf[1].w};
    const uint32_t x[4] = {vf[2].x, vf[2].y, vf[2].z, vf[2].w};
    const uint32_t y[4] = {vf[3].x, vf[3].y, vf[3].z, vf[3].w};
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const uint32_t lo01 = __builtin_amdgcn_perm(c[j], a[j], 0x05040100u);
      const uint32_t hi01 = __builtin_amdgcn_perm(c[j], a[j], 0x07060302u);
      const uint32_t lo23 = __builtin_amdgcn_perm(y[j], x[j], 0x05040100u);
      const uint32_t hi23 = __builtin_amdgcn_perm(y[j], x[j], 0x07060302u);
      acc[2 * j] = mfma16k16((const T*)nullptr, p01, p23, lo01, lo23, acc[2 * j]);
      acc[2 * j + 1] = mfma16k16((const T*)nullptr, p01, p23, hi01, hi23, acc[2 * j + 1]);
    }
    }
  };
  // ---- tiles of this wave: begin + 16*(wave + 4*n).  Inside the loop every load is
  // unconditional (a tile index past the wave's last tile is clamped to it), so the
  // number of loads in flight is the same on every path and the wait before a tile's
  // first use leaves the next tile's loads outstanding.
  {
    int t = begin + wave * 16;
    if (t < end) {
      const int t_last = t + ((last - t) >> 6 << 6);
      // every path issues all its first lookups before it waits for any of them
      if (t == t_last) {  // one tile
        uint4 kA[4], vA[4];
        TileRows tr0;
        tile_rows(t, tr0);
        load_tile(tr0, kA, vA);
        compute(t, kA, vA);
      } else if (t + 64 == t_last) {  // two tiles: everything in flight at once, nothing extra
        uint4 kA[4], vA[4], kB[4], vB[4];
        TileRows tr, tr0;
        tile_rows(t, tr0);
        tile_rows(t + 64, tr);
        load_tile(tr0, kA, vA);
        load_tile(tr, kB, vB);
        compute(t, kA, vA);
        compute(t + 64, kB, vB);
      } else if (!KLDS && t + 128 == t_last) {
        // three tiles (a sparse layer's usual share): a third set of registers keeps all of them in
        // flight behind one index round trip, instead of the third tile waiting for the first
        uint4 kA[4], vA[4], kB[4], vB[4], kC[4], vC[4];
        TileRows tr, tr0, tr2;
        tile_rows(t, tr0);
        tile_rows(t + 64, tr);
        tile_rows(t + 128, tr2);
        SPLIT_STAMP(2);
        load_tile(tr0, kA, vA);
        SPLIT_STAMP(3);
        load_tile(tr, kB, vB);
        load_tile(tr2, kC, vC);
        SPLIT_STAMP(4);
        compute(t, kA, vA);
        SPLIT_STAMP(5);
        compute(t + 64, kB, vB);
        compute(t + 128, kC, vC);
        SPLIT_STAMP(6);
      } else {
        uint4 kA[4], vA[4], kB[4], vB[4];
        TileRows tr, tr0;
        tile_rows(t, tr0);
        tile_rows(t + 64, tr);  // both lookups leave before the first one is awaited
        load_tile(tr0, kA, vA);
        while (true) {
          load_tile(tr, kB, vB);
          tile_rows(min(t + 128, t_last), tr);
          compute(t, kA, vA);
          t += 64;
          load_tile(tr, kA, vA);
          tile_rows(min(t + 128, t_last), tr);
          compute(t, kB, vB);
          if (t == t_last) break;
          t += 64;
          if (t == t_last) {
            compute(t, kA, vA);
            break;
          }
        }
      }
    }
  }

  // ---- a scored split hands its logits over, then LDS changes hands
  if (scored) {
    __syncthreads();
    const int quads = (end - begin + 3) >> 2;
    const int nh = w.group_reduce ? 1 : G;  // logits rows this kv head contributes
    for (int h = 0; h < nh; ++h) {
      float* lrow = w.logits + (int64_t)(b * w.logit_heads + g * nh + h) * w.logits_stride + begin;
      const float* srow = slog + h * w.split_rows;
#pragma unroll 2
      for (int qd = threadIdx.x; qd < quads; qd += 256) {
        const int rr = 4 * qd;
        const float4 v = *reinterpret_cast<const float4*>(srow + rr);
        if (begin + rr + 3 < end) {
          *reinterpret_cast<float4*>(lrow + rr) = v;
        } else {
          lrow[rr] = v.x;
          if (begin + rr + 1 < end) lrow[rr + 1] = v.y;
          if (begin + rr + 2 < end) lrow[rr + 2] = v.z;
        }
      }
    }
    // LDS changes hands once every thread has READ its logits; the stores themselves carry registers
    // and need not have landed, so the block meets over LDS only
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
  }

  // ---- the four waves of the block meet in LDS
  float* sm = lds;                 // [4][G] running max (raw units)
  float* sl = lds + 4 * G;         // [4][G] sum of exp
  float* sacc = lds + 8 * G + 8;   // [4][G][128]
  const int grp = wave * 4 + j4;
  l = lane_rows_sum(l);
  if (r16 < G && j4 == 0) {
    sm[wave * G + r16] = m;
    sl[wave * G + r16] = l;
  }
  if (WITH_V) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int h = 4 * j4 + i;
      if (h < G) {
        float4* dst = reinterpret_cast<float4*>(sacc + (wave * G + h) * kD + r16 * 8);
        dst[0] = make_float4(acc[0][i], acc[1][i], acc[2][i], acc[3][i]);
        dst[1] = make_float4(acc[4][i], acc[5][i], acc[6][i], acc[7][i]);
      }
    }
  }
  if (WINDOW) {
    if (wscored) {
#pragma unroll
      for (int cb = 0; cb < WCB; ++cb) {
        wlds[grp * kWinCols + 16 * cb + r16] = wm[cb];
        wlds[16 * kWinCols + grp * kWinCols + 16 * cb + r16] = wl[cb];
      }
    }
  }
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");  // over LDS only: the logits' stores may still be on their way
  __builtin_amdgcn_s_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
  if (WINDOW) {
    if (wscored && threadIdx.x < kWinCols) {
      const int c = threadIdx.x;
      float M = -INFINITY;
#pragma unroll
      for (int x = 0; x < 16; ++x) M = fmaxf(M, wlds[x * kWinCols + c]);
      float den = 0.f;
#pragma unroll
      for (int x = 0; x < 16; ++x) {
        const float mm = wlds[x * kWinCols + c];
        den = fmaf(wlds[16 * kWinCols + x * kWinCols + c], mm == -INFINITY ? 0.f : __builtin_amdgcn_exp2f((mm - M) * sl2),
                   den);
      }
      wf.part[((int64_t)(b * (hq / G) + g) * kWinCols + c) * w.max_splits + split] =
          M == -INFINITY ? -INFINITY : M * sl2 + log2f(den);
    }
  }
  for (int o = threadIdx.x; o < G * kD; o += 256) {
    const int h = o / kD, d = o % kD;
    float M = -INFINITY;
#pragma unroll
    for (int x = 0; x < 4; ++x) M = fmaxf(M, sm[x * G + h]);
    float den = 0.f, num = 0.f;
#pragma unroll
    for (int x = 0; x < 4; ++x) {
      const float mm = sm[x * G + h];
      const float fx = (mm == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f((mm - M) * sl2);
      den = fmaf(sl[x * G + h], fx, den);
      if (WITH_V) num = fmaf(sacc[(x * G + h) * kD + d], fx, num);
    }
    const int64_t ph = (int64_t)(b * hq + g * G + h) * w.max_splits + split;
    if (WITH_V) w.part_o[ph * kD + d] = num / den;
    if (d == 0) w.part_lse[ph] = M * sl2 + log2f(den);
  }
  SPLIT_STAMP(7);
}

template <typename T, int G, bool WITH_V, int MODE, bool LOGITS>
__global__ __launch_bounds__(256) void attn_stage1_mfma(const T* __restrict__ q, RowList rows,
                                                        int hq, float scale, AttnWorkspace w) {
  fetch_now(q);
  fetch_args_now(rows, w);
  stage1_mfma_body<T, G, WITH_V, MODE, LOGITS, false>(q, rows, hq, scale, w, WindowFuse{});
}

// The dense pass with the window columns.  The 64 registers of window query fragments put a wave
// beyond half a SIMD's register file, so one workgroup is resident per CU and the splits are sized
// for that (capping the registers for two per CU spills and is slower).
template <typename T, int G>
__global__ __launch_bounds__(256) void attn_stage1_window_mfma(const T* __restrict__ q, RowList rows,
                                                                  int hq, float scale, AttnWorkspace w,
                                                                  WindowFuse wf) {
  stage1_mfma_body<T, G, true, 0, false, true>(q, rows, hq, scale, w, wf);
}

template <typename T, int G, bool WITH_V, int MODE, bool LOGITS, bool WINDOW = false>
static void launch_one(const void* q, const RowList& rows, int hq, int hkv, int batch, float scale,
                       const AttnWorkspace& w, hipStream_t stream, const WindowFuse& wf = WindowFuse{}) {
  const void* kern_ptr;
  if constexpr (WINDOW) kern_ptr = reinterpret_cast<const void*>(attn_stage1_window_mfma<T, G>);
  else kern_ptr = reinterpret_cast<const void*>(attn_stage1_mfma<T, G, WITH_V, MODE, LOGITS>);
  size_t lds_floats = stage1_lds_floats<G>(WITH_V);  // the logits staging aliases the merge buffers
  const size_t staged = (size_t)(w.group_reduce ? 1 : G) * w.split_rows;
  if (LOGITS && staged > lds_floats) lds_floats = staged;
  if (WINDOW) lds_floats += kWindowLdsFloats;
  if (stage1_k_through_lds(MODE)) lds_floats += 4 * 1024;  // 4 KB of K staging per wave
  const size_t lds_bytes = lds_floats * sizeof(float);
  static std::atomic<size_t> configured{0};  // per instantiation; two threads raising it at once both succeed
  if (lds_bytes > configured.load(std::memory_order_relaxed)) {
    (void)hipFuncSetAttribute(kern_ptr, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes);
    size_t seen = configured.load(std::memory_order_relaxed);
    while (seen < lds_bytes && !configured.compare_exchange_weak(seen, lds_bytes, std::memory_order_relaxed)) {
    }
  }
  dim3 grid(hkv, w.max_splits, batch);  // kv head fastest: co-resident blocks cover whole token rows
  if constexpr (WINDOW)
    hipLaunchKernelGGL((attn_stage1_window_mfma<T, G>), grid, dim3(256), lds_bytes, stream, (const T*)q, rows, hq,
                       scale, w, wf);
  else
    hipLaunchKernelGGL((attn_stage1_mfma<T, G, WITH_V, MODE, LOGITS>), grid, dim3(256), lds_bytes, stream,
                       (const T*)q, rows, hq, scale, w);
}

template <typename T, int G>
static void launch_g(const void* q, const RowList& rows, int hq, int hkv, int batch, float scale,
                     const AttnWorkspace& w, bool with_v, bool write_logits, hipStream_t stream) {
  const bool no_tail = rows.max_tail_len == 0 && !rows.tail_lens;
  int mode = 2;
  if (!rows.idx && !rows.page_table && no_tail) mode = 0;
  else if (rows.idx && !rows.page_table && rows.max_main_len >= 1) mode = 1;
  else if (rows.page_table && !rows.idx && no_tail && rows.page_shift >= 4) mode = 3;
  else if (!rows.idx && !rows.page_table && with_v && !write_logits) mode = 4;  // contiguous rows + tail
#define OKV_MODES(WV, LG)                                                                  \
  do {                                                                                     \
    if (mode == 0) launch_one<T, G, WV, 0, LG>(q, rows, hq, hkv, batch, scale, w, stream); \
    else if (mode == 1) launch_one<T, G, WV, 1, LG>(q, rows, hq, hkv, batch, scale, w, stream); \
    else if (mode == 3) launch_one<T, G, WV, 3, LG>(q, rows, hq, hkv, batch, scale, w, stream); \
    else launch_one<T, G, WV, 2, LG>(q, rows, hq, hkv, batch, scale, w, stream);           \
  } while (0)
  if (mode == 4) launch_one<T, G, true, 4, false>(q, rows, hq, hkv, batch, scale, w, stream);
  else if (!with_v) OKV_MODES(false, true);  // scoring only
  else if (write_logits) OKV_MODES(true, true);
  else OKV_MODES(true, false);
#undef OKV_MODES
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

// ---------------------------------------------------------------------------
// Raw (un-normalised) scores in ONE launch.  A workgroup owns a range of rows and ALL
// kv heads, one wave per kv head: every wave streams its head's K rows through the
// same MFMA tiles as above, reduces its G q heads with lane swaps, and leaves one
// value per row in LDS; the workgroup then reduces over kv heads and writes the scores.
// No logits round trip, no merge, no finishing launch.
template <typename T, int G, bool PAGED>
__global__ __launch_bounds__(1024) void score_raw_mfma(const T* __restrict__ q, RowList rows, int hq,
                                                       float scale, int head_reduce,
                                                       int rows_per_block, float* __restrict__ scores,
                                                       int64_t score_stride) {
  extern __shared__ float lds[];  // [kv heads][rows_per_block] scores, then 4 KB of K staging per wave
  const int b = blockIdx.y;
  const int A = rl_score_len(rows, b);
  const int begin = blockIdx.x * rows_per_block;
  const int end = min(begin + rows_per_block, A);
  if (begin >= end) return;
  const int lane = threadIdx.x & 63, g = threadIdx.x >> 6;
  const int r16 = lane & 15, j4 = lane >> 4;
  const bool is_max = head_reduce == OKV_REDUCE_MAX;

  uint4 qf[4];
  {
    const int hcol = r16 < G ? r16 : G - 1;
    const T* qp = q + ((int64_t)(b * hq + g * G + hcol) * kD + 8 * j4);
#pragma unroll
    for (int s = 0; s < 4; ++s) qf[s] = *reinterpret_cast<const uint4*>(qp + 32 * s);  // columns beyond G repeat head G-1
  }
  const T* kb = reinterpret_cast<const T*>(rows.k_base) + (int64_t)g * rows.head_stride + 8 * r16 +
                (PAGED ? 0 : (int64_t)b * rows.batch_stride);
  const uint32_t ts = (uint32_t)rows.token_stride;
  const int last = end - 1;
  // whole rows (instruction i: rows 4*(l/16) + i), transposed for the matrix cores in compute()
  auto load_tile = [&](int tbase, uint4 (&kf)[4]) {
    int page = 0;
    if (PAGED && rows.page_shift >= 4)  // pages of 2^n >= 16 rows hold the whole tile: one scalar lookup
      page = rows.page_table[(int64_t)b * rows.page_table_stride +
                             (__builtin_amdgcn_readfirstlane(tbase) >> rows.page_shift)];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      int r = tbase + 4 * j4 + i;
      r = r < last ? r : last;
      const T* kp;
      if (PAGED) {
        if (rows.page_shift < 4) page = rows.page_table[(int64_t)b * rows.page_table_stride + rl_page_of(rows, r)];
        kp = kb + (int64_t)page * rows.page_stride + (uint64_t)(uint32_t)rl_slot_of(rows, r) * ts;
      } else {
        kp = kb + (uint64_t)(uint32_t)r * ts;
      }
      kf[i] = load_stream16(kp);
    }
  };
  char* kstage = reinterpret_cast<char*>(lds + (blockDim.x >> 6) * rows_per_block) + g * 4096;
  float* mine = lds + g * rows_per_block;
  auto compute = [&](int tbase, const uint4 (&kf_in)[4]) {
    uint4 kf[4];
    k_rows_to_a_operand(kstage, r16, j4, kf_in, kf);
    f32x4_t S = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int s = 0; s < 4; ++s) S = mfma16((const T*)nullptr, kf[s], qf[s], S);
    float v[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      v[i] = S[i] * scale;
#pragma unroll
      for (int o = 1; o < G; o <<= 1) {  // lanes 0..G-1 of the lane row hold the G heads
        const float x = __shfl_xor(v[i], o);
        v[i] = is_max ? fmaxf(v[i], x) : v[i] + x;
      }
    }
    if (r16 == 0)
      *reinterpret_cast<float4*>(mine + (tbase - begin) + 4 * j4) = make_float4(v[0], v[1], v[2], v[3]);
  };
  {
    uint4 kA[4], kB[4];
    const int t_last = begin + ((last - begin) >> 4 << 4);
    int t = begin;
    load_tile(t, kA);
    if (t == t_last) {
      compute(t, kA);
    } else {
      while (true) {
        load_tile(min(t + 16, t_last), kB);
        compute(t, kA);
        t += 16;
        load_tile(min(t + 16, t_last), kA);
        compute(t, kB);
        if (t == t_last) break;
        t += 16;
        if (t == t_last) {
          compute(t, kA);
          break;
        }
      }
    }
  }
  __syncthreads();
  const int nheads = blockDim.x >> 6;
  for (int r = threadIdx.x; r < end - begin; r += blockDim.x) {
    float acc = lds[r];
    for (int x = 1; x < nheads; ++x) {
      const float y = lds[x * rows_per_block + r];
      acc = is_max ? fmaxf(acc, y) : acc + y;
    }
    scores[(int64_t)b * score_stride + begin + r] = acc;
  }
}

template <typename T, int G>
static void launch_score_raw_g(const void* q, const RowList& rows, int hq, int hkv, int batch,
                               float scale, int head_reduce, float* scores, int64_t score_stride,
                               hipStream_t stream) {
  int cus = 256, dev = 0;
  if (hipGetDevice(&dev) == hipSuccess) {
    int n = 0;
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && n > 0) cus = n;
  }
  // one round of workgroups, three resident per CU, equal shares of the rows; a batch may be
  // ragged (short requests leave their blocks empty), so it gets blocks half the size
  const int64_t slots = (int64_t)cus * (batch > 1 ? 6 : 3);
  int64_t per = ((int64_t)rows.max_score_len * batch + slots - 1) / slots;
  int rpb = (int)((per + 15) / 16 * 16);
  if (rpb < 64) rpb = 64;
  if (rpb > 1024) rpb = 1024;
  dim3 grid((rows.max_score_len + rpb - 1) / rpb, batch), block(64 * hkv);
  const size_t lds_bytes = (size_t)hkv * rpb * sizeof(float) + (size_t)hkv * 4096;  // scores + K staging
  if (rows.page_table) {
    auto kern = score_raw_mfma<T, G, true>;
    if (lds_bytes > 48 * 1024)
      (void)hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                (int)lds_bytes);
    hipLaunchKernelGGL(kern, grid, block, lds_bytes, stream, (const T*)q, rows, hq, scale, head_reduce, rpb,
                       scores, score_stride);
  } else {
    auto kern = score_raw_mfma<T, G, false>;
    if (lds_bytes > 48 * 1024)
      (void)hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                (int)lds_bytes);
    hipLaunchKernelGGL(kern, grid, block, lds_bytes, stream, (const T*)q, rows, hq, scale, head_reduce, rpb,
                       scores, score_stride);
  }
}

template <typename T>
static bool launch_score_raw_t(const void* q, const RowList& rows, int hq, int hkv, int batch, float scale,
                               int head_reduce, float* scores, int64_t score_stride, hipStream_t stream) {
  switch (hq / hkv) {
    case 1: launch_score_raw_g<T, 1>(q, rows, hq, hkv, batch, scale, head_reduce, scores, score_stride, stream); return true;
    case 2: launch_score_raw_g<T, 2>(q, rows, hq, hkv, batch, scale, head_reduce, scores, score_stride, stream); return true;
    case 4: launch_score_raw_g<T, 4>(q, rows, hq, hkv, batch, scale, head_reduce, scores, score_stride, stream); return true;
    case 8: launch_score_raw_g<T, 8>(q, rows, hq, hkv, batch, scale, head_reduce, scores, score_stride, stream); return true;
  }
  return false;
}

// Stand-alone raw scoring (no V, no softmax) of 16-bit K with at most 16 kv heads.
bool launch_score_raw_mfma(int dtype, const void* q, const RowList& rows, int hq, int hkv, int batch,
                           float scale, int head_reduce, float* scores, int64_t score_stride,
                           hipStream_t stream) {
  if (hkv > 16 || rows.idx || rows.token_stride >= (1ll << 31)) return false;
  if (dtype == OKV_BF16)
    return launch_score_raw_t<BF16>(q, rows, hq, hkv, batch, scale, head_reduce, scores, score_stride, stream);
  if (dtype == OKV_F16)
    return launch_score_raw_t<F16>(q, rows, hq, hkv, batch, scale, head_reduce, scores, score_stride, stream);
  return false;
}

// The dense pass (contiguous 16-bit K/V, no index, no tail) with the query window riding along.
bool launch_stage1_window(int dtype, const void* q, const RowList& rows, int hq, int hkv, int batch, float scale,
                          const AttnWorkspace& w, const WindowFuse& wf, hipStream_t stream) {
  if (rows.token_stride >= (1ll << 31) || rows.idx || rows.page_table || rows.max_tail_len != 0 || rows.tail_lens)
    return false;
  const int G = hq / hkv;
  if (wf.window < 1 || wf.window * G > kWinCols) return false;
#define OKV_WIN(T, GG) launch_one<T, GG, true, 0, false, true>(q, rows, hq, hkv, batch, scale, w, stream, wf)
  if (dtype == OKV_BF16) {
    switch (G) {
      case 1: OKV_WIN(BF16, 1); return true;
      case 2: OKV_WIN(BF16, 2); return true;
      case 4: OKV_WIN(BF16, 4); return true;
      case 8: OKV_WIN(BF16, 8); return true;
    }
  } else if (dtype == OKV_F16) {
    switch (G) {
      case 1: OKV_WIN(F16, 1); return true;
      case 2: OKV_WIN(F16, 2); return true;
      case 4: OKV_WIN(F16, 4); return true;
      case 8: OKV_WIN(F16, 8); return true;
    }
  }
#undef OKV_WIN
  return false;
}

bool launch_stage1_mfma(int dtype, const void* q, const RowList& rows, int hq, int hkv, int batch,
                        float scale, const AttnWorkspace& w, bool with_v, bool write_logits,
                        hipStream_t stream) {
  // token strides are used as 32-bit multipliers
  if (rows.token_stride >= (1ll << 31) || rows.tail_token_stride >= (1ll << 31)) return false;
  // the split's logits (one row per q head of the group, or one per kv head when the pass folds the
  // group) are staged in LDS next to the K staging
  const size_t logit_rows = w.group_reduce ? 1 : hq / hkv;
  if (write_logits && logit_rows * w.split_rows * sizeof(float) + 20 * 1024 > (size_t)lds_bytes_per_workgroup())
    return false;
  if (dtype == OKV_BF16)
    return launch_t<BF16>(q, rows, hq, hkv, batch, scale, w, with_v, write_logits, stream);
  if (dtype == OKV_F16)
    return launch_t<F16>(q, rows, hq, hkv, batch, scale, w, with_v, write_logits, stream);
  return false;
}

}  // namespace okv
