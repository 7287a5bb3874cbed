// Top-k of long score vectors across many workgroups: a fill launch and four passes
// over 4096-element chunks (one workgroup per chunk, the scores stay in L2).
//
//   pass 0  zero the two shared histograms (a fill kernel, safe to capture in a graph)
//   pass 1  histogram of the top 12 key bits            (LDS per chunk -> global atomics)
//   pass 2  every workgroup scans that histogram, finds the bin of the k-th largest key,
//           histograms the next 12 bits inside it, counts its keys above the bin
//   pass 3  the same one level down; the low 8 bits inside the 24-bit prefix are
//           histogrammed per chunk, privately
//   pass 4  every workgroup sums the per-chunk low-bit histograms (all chunks: the exact
//           threshold T and how many keys equal to T are taken; chunks before it: its
//           output offset), then writes the indices of its chunk in order
//
// Grid-wide dependencies are kernel boundaries; no workgroup waits for another and
// the workspace needs no preparation by the caller.
#include "okv_internal.h"

namespace okv {

static constexpr int kChunk = 4096;
static constexpr int kMbThreads = 256;
static constexpr int kBins12 = 4096;

__device__ __forceinline__ uint32_t mb_key(float s) {
  uint32_t u = __float_as_uint(s);
  if ((u & 0x7fffffffu) > 0x7f800000u) return 0xffffffffu;  // NaN ranks first
  if (u == 0x80000000u) u = 0;                              // -0.0 == +0.0
  return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}

struct TopkMbState {  // per request, written by workgroup 0 of a pass for the later ones
  uint32_t bin0, want1, bin1, want2;
};

struct TopkMbWs {
  uint32_t* hist0;       // [batch][4096]
  uint32_t* hist1;       // [batch][4096]
  TopkMbState* state;    // [batch]
  uint32_t* chunk_gt;    // [batch][max_chunks] keys above the 24-bit prefix, per chunk
  uint16_t* chunk_low;   // [batch][max_chunks][256] low-byte histogram inside the prefix
  int max_chunks;
};

size_t topk_mb_workspace_bytes(int batch, int max_seq_len) {
  const size_t chunks = (size_t)(max_seq_len + kChunk - 1) / kChunk;
  size_t b = 0;
  b += (size_t)batch * kBins12 * 4 * 2;
  b += (size_t)batch * sizeof(TopkMbState);
  b += (size_t)batch * chunks * 4;
  b += (size_t)batch * chunks * 256 * 2;
  return b + 1024;
}

static TopkMbWs carve_topk(void* ws, int batch, int max_seq_len) {
  TopkMbWs w;
  const size_t chunks = (size_t)(max_seq_len + kChunk - 1) / kChunk;
  char* p = (char*)(((uintptr_t)ws + 255) & ~(uintptr_t)255);
  w.hist0 = (uint32_t*)p;
  p += (size_t)batch * kBins12 * 4;
  w.hist1 = (uint32_t*)p;
  p += (size_t)batch * kBins12 * 4;
  w.state = (TopkMbState*)p;
  p += ((size_t)batch * sizeof(TopkMbState) + 255) & ~(size_t)255;
  w.chunk_gt = (uint32_t*)p;
  p += ((size_t)batch * chunks * 4 + 255) & ~(size_t)255;
  w.chunk_low = (uint16_t*)p;
  w.max_chunks = (int)chunks;
  return w;
}

// 16 keys per thread of chunk `c`; element j of thread t is chunk element 4*(j/4*256 + t) + j%4
// (coalesced float4s) or, with ORDERED, element 16*t + j (consecutive, for the final pass).
template <bool ORDERED>
__device__ __forceinline__ void load_chunk_keys(const float* __restrict__ s, int n, int c,
                                                uint32_t (&key)[16], uint32_t& valid_mask) {
  const int t = threadIdx.x;
  const int base = c * kChunk;
  const bool vec = (((uintptr_t)s) & 15) == 0;
  valid_mask = 0;
#pragma unroll
  for (int q = 0; q < 4; ++q) {
    const int e = ORDERED ? base + 16 * t + 4 * q : base + 4 * (q * kMbThreads + t);
    float x[4];
    if (vec && e + 3 < n) {
      const float4 a = *reinterpret_cast<const float4*>(s + e);
      x[0] = a.x; x[1] = a.y; x[2] = a.z; x[3] = a.w;
      valid_mask |= 0xfu << (4 * q);
    } else {
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        x[j] = (e + j < n) ? s[e + j] : 0.f;
        if (e + j < n) valid_mask |= 1u << (4 * q + j);
      }
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) key[4 * q + j] = mb_key(x[j]);
  }
}

// Every thread learns the bin (counted from the top) holding the `want`-th largest
// element of a 4096-bin histogram in global memory, and the rank wanted inside it.
__device__ void scan_hist12(const uint32_t* __restrict__ hist, uint32_t want, uint32_t* bin,
                            uint32_t* want_in, uint32_t* sm /* >= 8 words of LDS */) {
  const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
  // thread t owns bins 4095-16t .. 4080-16t (descending keys)
  uint32_t h[16];
  const uint4* hp = reinterpret_cast<const uint4*>(hist + (kBins12 - 16 * (t + 1)));
#pragma unroll
  for (int q = 0; q < 4; ++q) {
    const uint4 v = hp[q];
    h[4 * q] = v.x; h[4 * q + 1] = v.y; h[4 * q + 2] = v.z; h[4 * q + 3] = v.w;
  }
  uint32_t mine = 0;
#pragma unroll
  for (int i = 0; i < 16; ++i) mine += h[i];
  uint32_t inc = mine;
#pragma unroll
  for (int o = 1; o < 64; o <<= 1) {
    const uint32_t v = __shfl_up(inc, o);
    if (lane >= o) inc += v;
  }
  __syncthreads();
  if (lane == 63) sm[wave] = inc;
  __syncthreads();
  uint32_t off = 0;
  for (int x = 0; x < wave; ++x) off += sm[x];
  inc += off;
  const uint32_t exc = inc - mine;
  __syncthreads();
  if (exc < want && want <= inc) {  // exactly one thread
    uint32_t run = exc;
#pragma unroll
    for (int i = 15; i >= 0; --i) {  // h[15] is the thread's highest bin
      if (run < want && want <= run + h[i]) {
        sm[4] = (uint32_t)(kBins12 - 16 * (t + 1) + i);
        sm[5] = want - run;
      }
      run += h[i];
    }
  }
  __syncthreads();
  *bin = sm[4];
  *want_in = sm[5];
}

__device__ __forceinline__ int req_len(const int32_t* seq_lens, int max_seq_len, int b) {
  return seq_lens ? seq_lens[b] : max_seq_len;
}
__device__ __forceinline__ int req_k(const int32_t* k_per_seg, int max_k, int b, int n) {
  int k = k_per_seg ? k_per_seg[b] : max_k;
  return k < n ? k : n;
}

// LDS histogram of `bits` -> global atomics for the non-empty bins
template <int NB>
__device__ __forceinline__ void flush_hist(uint32_t* lh, uint32_t* __restrict__ gh) {
  __syncthreads();
  for (int i = threadIdx.x; i < NB; i += kMbThreads) {
    const uint32_t v = lh[i];
    if (v) atomicAdd(gh + i, v);
  }
}

__global__ __launch_bounds__(kMbThreads) void topk_mb_pass0(uint4* __restrict__ p, int n16) {
  const int i = blockIdx.x * kMbThreads + threadIdx.x;
  if (i < n16) p[i] = make_uint4(0, 0, 0, 0);
}

__global__ __launch_bounds__(kMbThreads) void topk_mb_pass1(const float* __restrict__ scores,
                                                            int64_t score_stride,
                                                            const int32_t* __restrict__ seq_lens,
                                                            int max_seq_len,
                                                            const int32_t* __restrict__ k_per_seg,
                                                            int max_k, TopkMbWs w) {
  __shared__ uint32_t lh[kBins12];
  const int c = blockIdx.x, b = blockIdx.y;
  const int n = req_len(seq_lens, max_seq_len, b);
  const int k = req_k(k_per_seg, max_k, b, n);
  if (c * kChunk >= n || k <= 0 || k == n) return;
  for (int i = threadIdx.x; i < kBins12; i += kMbThreads) lh[i] = 0;
  __syncthreads();
  uint32_t key[16], valid;
  load_chunk_keys<false>(scores + (int64_t)b * score_stride, n, c, key, valid);
#pragma unroll
  for (int j = 0; j < 16; ++j)
    if (valid >> j & 1) atomicAdd(&lh[key[j] >> 20], 1u);
  flush_hist<kBins12>(lh, w.hist0 + (int64_t)b * kBins12);
}

__global__ __launch_bounds__(kMbThreads) void topk_mb_pass2(const float* __restrict__ scores,
                                                            int64_t score_stride,
                                                            const int32_t* __restrict__ seq_lens,
                                                            int max_seq_len,
                                                            const int32_t* __restrict__ k_per_seg,
                                                            int max_k, TopkMbWs w) {
  __shared__ uint32_t lh[kBins12];
  __shared__ uint32_t sm[8];
  const int c = blockIdx.x, b = blockIdx.y;
  const int n = req_len(seq_lens, max_seq_len, b);
  const int k = req_k(k_per_seg, max_k, b, n);
  if (c * kChunk >= n || k <= 0 || k == n) return;
  for (int i = threadIdx.x; i < kBins12; i += kMbThreads) lh[i] = 0;
  uint32_t bin0, want1;
  scan_hist12(w.hist0 + (int64_t)b * kBins12, (uint32_t)k, &bin0, &want1, sm);
  if (c == 0 && threadIdx.x == 0) {
    w.state[b].bin0 = bin0;
    w.state[b].want1 = want1;
  }
  uint32_t key[16], valid;
  load_chunk_keys<false>(scores + (int64_t)b * score_stride, n, c, key, valid);
  uint32_t gt = 0;
#pragma unroll
  for (int j = 0; j < 16; ++j) {
    if (!(valid >> j & 1)) continue;
    const uint32_t top = key[j] >> 20;
    if (top > bin0) ++gt;
    else if (top == bin0) atomicAdd(&lh[(key[j] >> 8) & 0xfffu], 1u);
  }
  // keys of this chunk above the level-0 bin
#pragma unroll
  for (int o = 32; o >= 1; o >>= 1) gt += __shfl_xor(gt, o);
  __syncthreads();
  if ((threadIdx.x & 63) == 0) sm[threadIdx.x >> 6] = gt;
  __syncthreads();
  if (threadIdx.x == 0) w.chunk_gt[(int64_t)b * w.max_chunks + c] = sm[0] + sm[1] + sm[2] + sm[3];
  flush_hist<kBins12>(lh, w.hist1 + (int64_t)b * kBins12);
}

__global__ __launch_bounds__(kMbThreads) void topk_mb_pass3(const float* __restrict__ scores,
                                                            int64_t score_stride,
                                                            const int32_t* __restrict__ seq_lens,
                                                            int max_seq_len,
                                                            const int32_t* __restrict__ k_per_seg,
                                                            int max_k, TopkMbWs w) {
  __shared__ uint32_t low[256];
  __shared__ uint32_t sm[8];
  const int c = blockIdx.x, b = blockIdx.y;
  const int n = req_len(seq_lens, max_seq_len, b);
  const int k = req_k(k_per_seg, max_k, b, n);
  if (c * kChunk >= n || k <= 0 || k == n) return;
  low[threadIdx.x] = 0;
  const uint32_t bin0 = w.state[b].bin0, want1 = w.state[b].want1;
  uint32_t bin1, want2;
  scan_hist12(w.hist1 + (int64_t)b * kBins12, want1, &bin1, &want2, sm);
  if (c == 0 && threadIdx.x == 0) {
    w.state[b].bin1 = bin1;
    w.state[b].want2 = want2;
  }
  const uint32_t prefix = (bin0 << 12) | bin1;
  uint32_t key[16], valid;
  load_chunk_keys<false>(scores + (int64_t)b * score_stride, n, c, key, valid);
  uint32_t gt = 0;
#pragma unroll
  for (int j = 0; j < 16; ++j) {
    if (!(valid >> j & 1)) continue;
    const uint32_t hi = key[j] >> 8;
    if ((hi >> 12) == bin0 && hi > prefix) ++gt;
    else if (hi == prefix) atomicAdd(&low[key[j] & 0xffu], 1u);
  }
#pragma unroll
  for (int o = 32; o >= 1; o >>= 1) gt += __shfl_xor(gt, o);
  __syncthreads();
  if ((threadIdx.x & 63) == 0) sm[threadIdx.x >> 6] = gt;
  __syncthreads();
  if (threadIdx.x == 0) w.chunk_gt[(int64_t)b * w.max_chunks + c] += sm[0] + sm[1] + sm[2] + sm[3];
  w.chunk_low[((int64_t)b * w.max_chunks + c) * 256 + threadIdx.x] = (uint16_t)low[threadIdx.x];
}

__global__ __launch_bounds__(kMbThreads) void topk_mb_pass4(const float* __restrict__ scores,
                                                            int64_t score_stride,
                                                            const int32_t* __restrict__ seq_lens,
                                                            int max_seq_len,
                                                            const int32_t* __restrict__ k_per_seg,
                                                            int max_k, TopkMbWs w,
                                                            int32_t* __restrict__ idx_out,
                                                            int64_t idx_stride) {
  __shared__ uint32_t sm[16];
  const int c = blockIdx.x, b = blockIdx.y, t = threadIdx.x, lane = t & 63, wave = t >> 6;
  const int n = req_len(seq_lens, max_seq_len, b);
  const int k = req_k(k_per_seg, max_k, b, n);
  if (c * kChunk >= n || k <= 0) return;
  int32_t* out = idx_out + (int64_t)b * idx_stride;
  if (k == n) {  // everything is selected
    for (int i = c * kChunk + t; i < n && i < (c + 1) * kChunk; i += kMbThreads) out[i] = i;
    return;
  }
  const int chunks = (n + kChunk - 1) / kChunk;
  const TopkMbState st = w.state[b];
  // column t of the per-chunk low-byte histograms: over all chunks, and over those before c
  uint32_t total = 0, before = 0;
  const uint16_t* col = w.chunk_low + (int64_t)b * w.max_chunks * 256 + t;
#pragma unroll 4
  for (int x = 0; x < chunks; ++x) {
    const uint32_t v = col[(int64_t)x * 256];
    total += v;
    if (x < c) before += v;
  }
  // suffix scan over the 256 low-byte values (thread t holds value t): rank from the top
  uint32_t inc = total;  // inclusive sum over values >= t within the wave, built from the high end
#pragma unroll
  for (int o = 1; o < 64; o <<= 1) {
    const uint32_t v = __shfl_down(inc, o);
    if (lane + o < 64) inc += v;
  }
  if (lane == 0) sm[wave] = inc;
  __syncthreads();
  uint32_t above_waves = 0;
  for (int x = wave + 1; x < 4; ++x) above_waves += sm[x];
  inc += above_waves;                  // keys of the prefix with low byte >= t
  const uint32_t exc = inc - total;    // ... with low byte > t
  __syncthreads();
  if (exc < st.want2 && st.want2 <= inc) {  // exactly one thread: its value is T's low byte
    sm[8] = (uint32_t)t;
    sm[9] = st.want2 - exc;  // how many keys == T are taken
  }
  __syncthreads();
  const uint32_t low_t = sm[8], need_eq = sm[9];
  const uint32_t T = (st.bin0 << 20) | (st.bin1 << 8) | low_t;
  // selected keys in the chunks before this one: above the prefix, inside it above T, equal to T
  uint32_t gt_before = (t > (int)low_t) ? before : 0u;
  for (int x = t; x < c; x += kMbThreads) gt_before += w.chunk_gt[(int64_t)b * w.max_chunks + x];
  uint32_t eq_before = (t == (int)low_t) ? before : 0u;
#pragma unroll
  for (int o = 32; o >= 1; o >>= 1) {
    gt_before += __shfl_xor(gt_before, o);
    eq_before += __shfl_xor(eq_before, o);
  }
  __syncthreads();
  if (lane == 0) {
    sm[wave] = gt_before;
    sm[4 + wave] = eq_before;
  }
  __syncthreads();
  gt_before = sm[0] + sm[1] + sm[2] + sm[3];
  eq_before = sm[4] + sm[5] + sm[6] + sm[7];
  __syncthreads();

  // ordered compaction of this chunk: 16 consecutive tokens per thread
  uint32_t key[16], valid;
  load_chunk_keys<true>(scores + (int64_t)b * score_stride, n, c, key, valid);
  uint32_t gmask = 0, emask = 0;
#pragma unroll
  for (int j = 0; j < 16; ++j) {
    if (!(valid >> j & 1)) continue;
    if (key[j] > T) gmask |= 1u << j;
    else if (key[j] == T) emask |= 1u << j;
  }
  const uint32_t packed = __popc(gmask) | (__popc(emask) << 16);  // <= 4096 each per chunk
  uint32_t pinc = packed;
#pragma unroll
  for (int o = 1; o < 64; o <<= 1) {
    const uint32_t v = __shfl_up(pinc, o);
    if (lane >= o) pinc += v;
  }
  if (lane == 63) sm[wave] = pinc;
  __syncthreads();
  uint32_t woff = 0;
  for (int x = 0; x < wave; ++x) woff += sm[x];
  const uint32_t pexc = pinc - packed + woff;
  uint32_t pgt = gt_before + (pexc & 0xffffu);
  uint32_t peq = eq_before + (pexc >> 16);
  const int i0 = c * kChunk + 16 * t;
#pragma unroll
  for (int j = 0; j < 16; ++j) {
    if (gmask >> j & 1) {
      const uint32_t pos = pgt + (peq < need_eq ? peq : need_eq);
      if (pos < (uint32_t)k) out[pos] = i0 + j;  // the bound only matters if the counts were corrupted
      ++pgt;
    } else if (emask >> j & 1) {
      if (peq < need_eq && pgt + peq < (uint32_t)k) out[pgt + peq] = i0 + j;
      ++peq;
    }
  }
}

int launch_topk_mb(const float* scores, int64_t score_stride, const int32_t* seq_lens,
                   int32_t max_seq_len, const int32_t* k_per_seg, int32_t max_k, int32_t batch,
                   int32_t* idx_out, int64_t idx_stride, void* ws, hipStream_t stream) {
  const TopkMbWs w = carve_topk(ws, batch, max_seq_len);
  dim3 grid(w.max_chunks, batch), block(kMbThreads);
  const int n16 = batch * kBins12 * 2 * 4 / 16;  // hist0 and hist1 are adjacent
  hipLaunchKernelGGL(topk_mb_pass0, dim3((n16 + kMbThreads - 1) / kMbThreads), block, 0, stream,
                     reinterpret_cast<uint4*>(w.hist0), n16);
  hipLaunchKernelGGL(topk_mb_pass1, grid, block, 0, stream, scores, score_stride, seq_lens,
                     max_seq_len, k_per_seg, max_k, w);
  hipLaunchKernelGGL(topk_mb_pass2, grid, block, 0, stream, scores, score_stride, seq_lens,
                     max_seq_len, k_per_seg, max_k, w);
  hipLaunchKernelGGL(topk_mb_pass3, grid, block, 0, stream, scores, score_stride, seq_lens,
                     max_seq_len, k_per_seg, max_k, w);
  hipLaunchKernelGGL(topk_mb_pass4, grid, block, 0, stream, scores, score_stride, seq_lens,
                     max_seq_len, k_per_seg, max_k, w, idx_out, idx_stride);
  OKV_HIP_CHECK(hipGetLastError());
  return OKV_OK;
}

}  // namespace okv
