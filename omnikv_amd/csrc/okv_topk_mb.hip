// Top-k of long score vectors across many workgroups, in three launches.  A request's scores
// are cut into chunks of one or more 4096-key tiles, one workgroup of 1024 threads per chunk
// (four keys per thread and tile: the work is chains of short dependent steps, and sixteen
// waves per CU hide each other's latencies); the scores stay in L2 between the launches.
//
//   hist   every chunk histograms the top 12 bits of its keys in LDS and stores the histogram
//          (16-bit counts) and its 256-bin summary in its own slot of the workspace
//   cand   every workgroup sums the chunks' summaries, then the 16 bins inside the summary bin
//          that holds the k-th largest key, which gives the bin B0 of that key; it copies the
//          keys of its chunk that fall into B0 -- the candidates, a few percent of the chunk
//          for smooth scores -- behind those of the chunks before it (their number is in the
//          histograms it has just read), and counts its keys above B0
//   write  every workgroup reads all candidates (kept in LDS when they fit), finds the exact
//          threshold T among them over the remaining 20 bits in two 10-bit levels, counts what
//          the chunks before its own hold above T and equal to T, and writes the selected
//          indices of its chunk in order
//
// Nothing is accumulated across workgroups: no atomics on global memory, nothing to clear before
// a call, no workgroup waits for another, and every count is an integer sum whose value does not
// depend on the order of execution.
#include "okv_internal.h"

namespace okv {

static constexpr int kTile = 4096;         // keys per tile: 1024 threads x 4
static constexpr int kMbThreads = 1024;
static constexpr int kMbWaves = kMbThreads / 64;
static constexpr int kBins12 = 4096;
static constexpr int kMaxChunkTiles = 15;  // 61440 keys: a 16-bit count per bin cannot overflow
static constexpr int kTargetChunks = 64;   // histograms every workgroup of `cand` sums
static constexpr int kCandCache = 8192;    // candidates `write` keeps in LDS

__device__ __forceinline__ uint32_t mb_key(float s) {
  uint32_t u = __float_as_uint(s);
  if ((u & 0x7fffffffu) > 0x7f800000u) return 0xffffffffu;  // NaN ranks first
  if (u == 0x80000000u) u = 0;                              // -0.0 == +0.0
  return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}

struct TopkMbState {  // per request, written by chunk 0 of `cand` for `write`
  uint32_t bin0, want1, num_cand, pad;
};

struct TopkMbWs {
  uint16_t* hist0;      // [batch][max_chunks][4096]
  uint16_t* coarse;     // [batch][max_chunks][256]  sums of 16 adjacent bins of hist0
  uint32_t* cand;       // [batch][max_chunks * chunk_keys]  candidates, chunk after chunk, no gaps
  uint32_t* cand_base;  // [batch][max_chunks]  where a chunk's candidates start
  uint32_t* chunk_gt;   // [batch][max_chunks][16]  keys above the level-0 bin, per wave of the chunk's workgroup
  TopkMbState* state;   // [batch]
  int max_chunks;
  int chunk_tiles;
};

// all arguments of a launch in one batch of scalar loads at the top (see fetch_now)
__device__ __forceinline__ void fetch_topk_args_now(const float* scores, int64_t score_stride, const int32_t* seq_lens,
                                                    int max_seq_len, const int32_t* k_per_seg, int max_k,
                                                    const TopkMbWs& w) {
  fetch_now(scores); fetch_now(score_stride); fetch_now(seq_lens); fetch_now(max_seq_len); fetch_now(k_per_seg);
  fetch_now(max_k); fetch_now(w.hist0); fetch_now(w.coarse); fetch_now(w.cand); fetch_now(w.cand_base);
  fetch_now(w.chunk_gt); fetch_now(w.state); fetch_now(w.max_chunks); fetch_now(w.chunk_tiles);
}

static void chunking(int max_seq_len, int* chunk_tiles, int* chunks) {
  const int tiles = (max_seq_len + kTile - 1) / kTile;
  int ct = (tiles + kTargetChunks - 1) / kTargetChunks;
  if (ct < 1) ct = 1;
  if (ct > kMaxChunkTiles) ct = kMaxChunkTiles;
  *chunk_tiles = ct;
  *chunks = (tiles + ct - 1) / ct;
}

static inline size_t up256(size_t x) { return (x + 255) & ~(size_t)255; }

// An upper bound of what carve_topk() lays out that never shrinks when max_seq_len grows (the
// exact layout does, where one more tile makes the chunks twice as long and half as many), so
// that a workspace sized for a length also serves every shorter one.
size_t topk_mb_workspace_bytes(int batch, int max_seq_len) {
  const int tiles = (max_seq_len + kTile - 1) / kTile;
  int chunks = tiles < kTargetChunks ? tiles : kTargetChunks;            // chunks of up to kMaxChunkTiles tiles: at most
  const int long_chunks = (tiles + kMaxChunkTiles - 1) / kMaxChunkTiles;  // this many, or that many once they are full
  if (long_chunks > chunks) chunks = long_chunks;
  if (chunks < 1) chunks = 1;
  const size_t cand_tiles = (size_t)tiles + kMaxChunkTiles;  // chunks * tiles per chunk < tiles + tiles per chunk
  size_t b = 0;
  b += up256((size_t)batch * chunks * kBins12 * 2);
  b += up256((size_t)batch * chunks * 256 * 2);
  b += up256((size_t)batch * cand_tiles * kTile * 4);
  b += up256((size_t)batch * chunks * 4);
  b += up256((size_t)batch * chunks * kMbWaves * 4);
  b += up256((size_t)batch * sizeof(TopkMbState));
  return b + 256;
}

static TopkMbWs carve_topk(void* ws, int batch, int max_seq_len) {
  TopkMbWs w;
  int ct, chunks;
  chunking(max_seq_len, &ct, &chunks);
  char* p = (char*)(((uintptr_t)ws + 255) & ~(uintptr_t)255);
  w.hist0 = (uint16_t*)p;
  p += up256((size_t)batch * chunks * kBins12 * 2);
  w.coarse = (uint16_t*)p;
  p += up256((size_t)batch * chunks * 256 * 2);
  w.cand = (uint32_t*)p;
  p += up256((size_t)batch * chunks * ct * kTile * 4);
  w.cand_base = (uint32_t*)p;
  p += up256((size_t)batch * chunks * 4);
  w.chunk_gt = (uint32_t*)p;
  p += up256((size_t)batch * chunks * kMbWaves * 4);
  w.state = (TopkMbState*)p;
  w.max_chunks = chunks;
  w.chunk_tiles = ct;
  return w;
}

// Scores 4t .. 4t+3 of tile `tile` for thread t (one 16-byte load when aligned and in range).
// Loading and key conversion are separate so that a kernel can issue the load first and wait
// for it after its other memory round trips.
__device__ __forceinline__ void load_tile_raw(const float* __restrict__ s, int n, int tile,
                                              float (&x)[4], uint32_t& valid_mask) {
  const int e = tile * kTile + 4 * threadIdx.x;
  if ((((uintptr_t)s) & 15) == 0 && e + 3 < n) {
    const float4 a = *reinterpret_cast<const float4*>(s + e);
    x[0] = a.x; x[1] = a.y; x[2] = a.z; x[3] = a.w;
    valid_mask = 0xfu;
    return;
  }
  valid_mask = 0;
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    x[j] = (e + j < n) ? s[e + j] : 0.f;
    if (e + j < n) valid_mask |= 1u << j;
  }
}
__device__ __forceinline__ void keys_of(const float (&x)[4], uint32_t (&key)[4]) {
#pragma unroll
  for (int j = 0; j < 4; ++j) key[j] = mb_key(x[j]);
}

// Inclusive prefix sum over the 64 lanes of a wave.
__device__ __forceinline__ uint32_t wave_scan(uint32_t v) {
  const int lane = threadIdx.x & 63;
#pragma unroll
  for (int o = 1; o < 64; o <<= 1) {
    const uint32_t u = __shfl_up(v, o);
    if (lane >= o) v += u;
  }
  return v;
}

// Sum over the 64 lanes of a wave, in every lane.
__device__ __forceinline__ uint32_t wave_sum(uint32_t v) {
#pragma unroll
  for (int o = 32; o >= 1; o >>= 1) v += __shfl_xor(v, o);
  return v;
}

// For ONE wave: the bin of an NB-bin histogram in LDS (16-byte aligned, complete) that holds the
// `want`-th largest key, and the rank wanted inside it, in every lane.  Lane l takes bins
// [NB - PER*(l+1), NB - PER*l): ascending lanes are descending keys.  A workgroup-wide scan
// would cost three barriers of sixteen waves; this costs the callers one.
template <int NB>
__device__ __forceinline__ void wave_find_bin(const uint32_t* hist, uint32_t want, uint32_t& bin,
                                              uint32_t& want_in) {
  constexpr int PER = NB / 64;
  const int lane = threadIdx.x & 63;
  const int first = NB - PER * (lane + 1);
  uint32_t h[PER];
#pragma unroll
  for (int q = 0; q < PER / 4; ++q) {
    const uint4 v = reinterpret_cast<const uint4*>(hist + first)[q];
    h[4 * q] = v.x; h[4 * q + 1] = v.y; h[4 * q + 2] = v.z; h[4 * q + 3] = v.w;
  }
  uint32_t mine = 0;
#pragma unroll
  for (int i = 0; i < PER; ++i) mine += h[i];
  const uint32_t inc = wave_scan(mine);
  uint32_t run = inc - mine, fb = 0, fw = 1;
  const bool found = run < want && want <= inc;  // at most one lane
  if (found) {
#pragma unroll
    for (int i = PER - 1; i >= 0; --i) {  // h[PER-1] is the lane's highest bin
      if (run < want && want <= run + h[i]) {
        fb = (uint32_t)(first + i);
        fw = want - run;
      }
      run += h[i];
    }
  }
  const unsigned long long m = __ballot(found);
  const int src = m ? __ffsll((long long)m) - 1 : 0;  // lane 0's defaults if the counts fell short
  bin = __shfl(fb, src);
  want_in = __shfl(fw, src);
}

__device__ __forceinline__ int req_len(const int32_t* seq_lens, int max_seq_len, int b) {
  return seq_lens ? seq_lens[b] : max_seq_len;
}
__device__ __forceinline__ int req_k(const int32_t* k_per_seg, int max_k, int b, int n) {
  int k = k_per_seg ? k_per_seg[b] : max_k;
  return k < n ? k : n;
}

__global__ __launch_bounds__(kMbThreads) void topk_mb_hist(const float* __restrict__ scores,
                                                           int64_t score_stride,
                                                           const int32_t* __restrict__ seq_lens,
                                                           int max_seq_len,
                                                           const int32_t* __restrict__ k_per_seg,
                                                           int max_k, TopkMbWs w) {
  fetch_topk_args_now(scores, score_stride, seq_lens, max_seq_len, k_per_seg, max_k, w);
  __shared__ __attribute__((aligned(16))) uint32_t lh[kBins12];
  const int c = blockIdx.x, b = blockIdx.y, t = threadIdx.x;
  const int n = req_len(seq_lens, max_seq_len, b);
  const int k = req_k(k_per_seg, max_k, b, n);
  const int tile0 = c * w.chunk_tiles;
  if ((int64_t)tile0 * kTile >= n || k <= 0 || k == n) return;
  const float* s = scores + (int64_t)b * score_stride;
  float x[4];
  uint32_t valid;
  load_tile_raw(s, n, tile0, x, valid);
  reinterpret_cast<uint4*>(lh)[t] = make_uint4(0, 0, 0, 0);
  __syncthreads();
  for (int i = 0;;) {
    uint32_t key[4];
    keys_of(x, key);
#pragma unroll
    for (int j = 0; j < 4; ++j)
      if (valid >> j & 1) atomicAdd(&lh[key[j] >> 20], 1u);
    if (++i >= w.chunk_tiles || (int64_t)(tile0 + i) * kTile >= n) break;
    load_tile_raw(s, n, tile0 + i, x, valid);
  }
  __syncthreads();
  // bins 4t .. 4t+3 as 16-bit counts, and the sum of 16 adjacent bins from four adjacent lanes
  const uint4 a = reinterpret_cast<const uint4*>(lh)[t];
  uint16_t* hp = w.hist0 + ((int64_t)b * w.max_chunks + c) * kBins12;
  reinterpret_cast<uint2*>(hp)[t] = make_uint2(a.x | a.y << 16, a.z | a.w << 16);
  uint32_t s16 = a.x + a.y + a.z + a.w;
  s16 += __shfl_xor(s16, 1);
  s16 += __shfl_xor(s16, 2);
  if ((t & 3) == 0) w.coarse[((int64_t)b * w.max_chunks + c) * 256 + (t >> 2)] = (uint16_t)s16;
}

// the 16-bit halves of the four words of v, added to h[0..8)
__device__ __forceinline__ void add_counts8(uint32_t* h, const uint4& v) {
  const uint32_t e[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    if (e[j] & 0xffffu) atomicAdd(&h[2 * j], e[j] & 0xffffu);
    if (e[j] >> 16) atomicAdd(&h[2 * j + 1], e[j] >> 16);
  }
}

__global__ __launch_bounds__(kMbThreads) void topk_mb_cand(const float* __restrict__ scores,
                                                           int64_t score_stride,
                                                           const int32_t* __restrict__ seq_lens,
                                                           int max_seq_len,
                                                           const int32_t* __restrict__ k_per_seg,
                                                           int max_k, TopkMbWs w) {
  fetch_topk_args_now(scores, score_stride, seq_lens, max_seq_len, k_per_seg, max_k, w);
  __shared__ __attribute__((aligned(16))) uint32_t ch[256];  // the request's 256-bin summary
  __shared__ uint32_t fh[16];   // its 16 fine bins inside the summary bin of the k-th key
  __shared__ uint32_t fhb[16];  // the same over the chunks before this one
  __shared__ uint32_t sm[4];
  __shared__ uint32_t cnt;
  const int c = blockIdx.x, b = blockIdx.y, t = threadIdx.x, lane = t & 63, wave = t >> 6;
  const int n = req_len(seq_lens, max_seq_len, b);
  const int k = req_k(k_per_seg, max_k, b, n);
  const int tile0 = c * w.chunk_tiles;
  if ((int64_t)tile0 * kTile >= n || k <= 0 || k == n) return;
  const int chunk_keys = w.chunk_tiles * kTile;
  const int chunks = (n + chunk_keys - 1) / chunk_keys;
  const float* s = scores + (int64_t)b * score_stride;
  // the chunk's first tile is requested now and used after the two histogram round trips
  float x[4];
  uint32_t valid;
  load_tile_raw(s, n, tile0, x, valid);
  if (t < 256) ch[t] = 0;
  if (t < 16) fh[t] = fhb[t] = 0;
  if (t == 0) cnt = 0;
  __syncthreads();
  // summaries of all chunks: chunks*32 16-byte pieces, piece l = chunk l/32, bins 8*(l%32) ..
  {
    const uint4* cp = reinterpret_cast<const uint4*>(w.coarse + (int64_t)b * w.max_chunks * 256);
    const int pieces = chunks * 32;
    for (int base = 0; base < pieces; base += 2 * kMbThreads) {
      const int l0 = base + t, l1 = base + kMbThreads + t;
      const uint4 v0 = l0 < pieces ? cp[l0] : make_uint4(0, 0, 0, 0);
      const uint4 v1 = l1 < pieces ? cp[l1] : make_uint4(0, 0, 0, 0);
      add_counts8(&ch[8 * (t & 31)], v0);  // kMbThreads is a multiple of 32: l % 32 == t % 32
      add_counts8(&ch[8 * (t & 31)], v1);
    }
  }
  __syncthreads();
  if (wave == 0) {
    uint32_t cb, wc;
    wave_find_bin<256>(ch, (uint32_t)k, cb, wc);
    if (lane == 0) {
      sm[0] = cb;
      sm[1] = wc;
    }
  }
  __syncthreads();
  const uint32_t cbin = sm[0], wantc = sm[1];
  // the 16 fine bins inside it: two 16-byte pieces per chunk
  {
    const uint16_t* hp = w.hist0 + (int64_t)b * w.max_chunks * kBins12 + 16 * cbin;
    for (int l = t; l < 2 * chunks; l += kMbThreads) {
      const uint4 v = *reinterpret_cast<const uint4*>(hp + (int64_t)(l >> 1) * kBins12 + 8 * (l & 1));
      add_counts8(&fh[8 * (l & 1)], v);
      if ((l >> 1) < c) add_counts8(&fhb[8 * (l & 1)], v);
    }
  }
  __syncthreads();
  // the 16 bins from the top, one per lane (every wave does the same): lane j looks at bin 15-j
  uint32_t bin0, want1;
  {
    const uint32_t v = fh[15 - (lane & 15)];
    uint32_t inc = v;
#pragma unroll
    for (int o = 1; o < 16; o <<= 1) {
      const uint32_t u = __shfl_up(inc, o, 16);
      if ((lane & 15) >= o) inc += u;
    }
    const bool found = lane < 16 && inc - v < wantc && wantc <= inc;
    const unsigned long long m = __ballot(found);
    const int src = m ? __ffsll((long long)m) - 1 : 0;
    bin0 = 16 * cbin + 15 - src;
    want1 = m ? wantc - __shfl(inc - v, src) : 1u;
  }
  // the candidates of a chunk are its keys in bin0, and every chunk's count of those is in the
  // histograms just read: this chunk's candidates go right behind those of the chunks before it
  const uint32_t base = fhb[bin0 & 15];
  if (t == 0) {
    w.cand_base[(int64_t)b * w.max_chunks + c] = base;
    if (c == 0) {
      w.state[b].bin0 = bin0;
      w.state[b].want1 = want1;
      w.state[b].num_cand = fh[bin0 & 15];
    }
  }
  uint32_t* cand = w.cand + (int64_t)b * w.max_chunks * chunk_keys + base;
  uint32_t gt = 0;
  for (int i = 0;;) {
    uint32_t key[4];
    keys_of(x, key);
    uint32_t cmask = 0;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      if (!(valid >> j & 1)) continue;
      const uint32_t top = key[j] >> 20;
      if (top > bin0) ++gt;
      else if (top == bin0) cmask |= 1u << j;
    }
    // one LDS atomic per wave reserves room for the wave's candidates; their order is free
    const uint32_t pc = __popc(cmask);
    const uint32_t inc = wave_scan(pc);
    const uint32_t wave_total = __shfl(inc, 63);
    if (wave_total) {
      uint32_t at = 0;
      if (lane == 63) at = atomicAdd(&cnt, wave_total);
      at = __shfl(at, 63) + inc - pc;
#pragma unroll
      for (int j = 0; j < 4; ++j)
        if (cmask >> j & 1) cand[at++] = key[j];
    }
    if (++i >= w.chunk_tiles || (int64_t)(tile0 + i) * kTile >= n) break;
    load_tile_raw(s, n, tile0 + i, x, valid);
  }
  gt = wave_sum(gt);
  if (lane == 0) w.chunk_gt[((int64_t)b * w.max_chunks + c) * kMbWaves + wave] = gt;
}

__global__ __launch_bounds__(kMbThreads) void topk_mb_write(const float* __restrict__ scores,
                                                            int64_t score_stride,
                                                            const int32_t* __restrict__ seq_lens,
                                                            int max_seq_len,
                                                            const int32_t* __restrict__ k_per_seg,
                                                            int max_k, TopkMbWs w,
                                                            int32_t* __restrict__ idx_out,
                                                            int64_t idx_stride) {
  fetch_topk_args_now(scores, score_stride, seq_lens, max_seq_len, k_per_seg, max_k, w);
  fetch_now(idx_out);
  fetch_now(idx_stride);
  __shared__ __attribute__((aligned(16))) uint32_t hA[1024], hB[1024], hBb[1024];
  __shared__ uint32_t cache[kCandCache];
  __shared__ uint32_t sm[8];
  __shared__ uint32_t acc;                 // selected keys of the chunks before this one, above T
  __shared__ uint32_t part[2][kMbWaves];   // wave totals of the compaction, alternating per tile
  const int c = blockIdx.x, b = blockIdx.y, t = threadIdx.x, lane = t & 63, wave = t >> 6;
  const int n = req_len(seq_lens, max_seq_len, b);
  const int k = req_k(k_per_seg, max_k, b, n);
  const int tile0 = c * w.chunk_tiles;
  if ((int64_t)tile0 * kTile >= n || k <= 0) return;
  const int chunk_keys = w.chunk_tiles * kTile;
  int32_t* out = idx_out + (int64_t)b * idx_stride;
  if (k == n) {  // everything is selected
    const int hi = (c + 1) * chunk_keys < n ? (c + 1) * chunk_keys : n;
    for (int i = c * chunk_keys + t; i < hi; i += kMbThreads) out[i] = i;
    return;
  }
  const TopkMbState st = w.state[b];
  // the chunk's first tile is requested now and used once the threshold is known
  const float* s = scores + (int64_t)b * score_stride;
  float x[4];
  uint32_t valid;
  load_tile_raw(s, n, tile0, x, valid);
  const uint32_t M = st.num_cand < (uint32_t)n ? st.num_cand : (uint32_t)n;  // candidates of the request
  const uint32_t Mb = w.cand_base[(int64_t)b * w.max_chunks + c];            // ... of the chunks before this one
  uint32_t gt_before = 0;  // this thread's share of the keys above T in the chunks before this one
  for (int i = t; i < c * kMbWaves; i += kMbThreads) gt_before += w.chunk_gt[(int64_t)b * w.max_chunks * kMbWaves + i];
  hA[t] = hB[t] = hBb[t] = 0;
  if (t == 0) acc = 0;
  __syncthreads();
  const bool cached = M <= (uint32_t)kCandCache;
  const uint32_t* cand = w.cand + (int64_t)b * w.max_chunks * chunk_keys;

  // level A: bits 19..10 of all candidates, four loads per thread in flight
  for (uint32_t base = 0; base < M; base += 4 * kMbThreads) {
    uint32_t kk[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const uint32_t i = base + u * kMbThreads + t;
      kk[u] = i < M ? cand[i] : 0u;
    }
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const uint32_t i = base + u * kMbThreads + t;
      if (i < M) {
        if (cached) cache[i] = kk[u];
        atomicAdd(&hA[(kk[u] >> 10) & 1023u], 1u);
      }
    }
  }
  __syncthreads();
  if (wave == 0) {
    uint32_t ba, wb;
    wave_find_bin<1024>(hA, st.want1, ba, wb);
    if (lane == 0) {
      sm[0] = ba;
      sm[1] = wb;
    }
  }
  __syncthreads();
  const uint32_t binA = sm[0], wantB = sm[1];

  // level B: bits 9..0 of the candidates inside bin A, over all chunks and over the chunks before
  // this one; candidates of earlier chunks in higher A bins are above T whatever T's low bits
  {
    auto visit = [&](uint32_t i, uint32_t kk) {
      const uint32_t a = (kk >> 10) & 1023u;
      if (a == binA) {
        atomicAdd(&hB[kk & 1023u], 1u);
        if (i < Mb) atomicAdd(&hBb[kk & 1023u], 1u);
      } else if (a > binA && i < Mb) {
        ++gt_before;
      }
    };
    if (cached) {
      for (uint32_t i = t; i < M; i += kMbThreads) visit(i, cache[i]);
    } else {
      for (uint32_t base = 0; base < M; base += 4 * kMbThreads) {
        uint32_t kk[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
          const uint32_t i = base + u * kMbThreads + t;
          kk[u] = i < M ? cand[i] : 0u;
        }
#pragma unroll
        for (int u = 0; u < 4; ++u) {
          const uint32_t i = base + u * kMbThreads + t;
          if (i < M) visit(i, kk[u]);
        }
      }
    }
  }
  gt_before = wave_sum(gt_before);
  if (lane == 0 && gt_before) atomicAdd(&acc, gt_before);
  __syncthreads();
  if (wave == 0) {
    uint32_t bb, ne;
    wave_find_bin<1024>(hB, wantB, bb, ne);
    // keys of the earlier chunks inside bin A: above T's low bits, and equal to them
    uint32_t g = 0;
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const int first = 1024 - 16 * (lane + 1) + 4 * q;
      const uint4 v = *reinterpret_cast<const uint4*>(hBb + first);
      if ((uint32_t)first > bb) g += v.x;
      if ((uint32_t)first + 1 > bb) g += v.y;
      if ((uint32_t)first + 2 > bb) g += v.z;
      if ((uint32_t)first + 3 > bb) g += v.w;
    }
    g = wave_sum(g);
    if (lane == 0) {
      sm[2] = bb;
      sm[3] = ne;
      sm[4] = hBb[bb];
      sm[5] = acc + g;
    }
  }
  __syncthreads();
  const uint32_t binB = sm[2], need_eq = sm[3], eq_before = sm[4];
  gt_before = sm[5];
  const uint32_t T = (st.bin0 << 20) | (binA << 10) | binB;

  // ordered compaction of this chunk, tile after tile: 4 consecutive tokens per thread
  uint32_t run_gt = gt_before, run_eq = eq_before;
  for (int i = 0;;) {
    uint32_t key[4];
    keys_of(x, key);
    uint32_t gmask = 0, emask = 0;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      if (!(valid >> j & 1)) continue;
      if (key[j] > T) gmask |= 1u << j;
      else if (key[j] == T) emask |= 1u << j;
    }
    const uint32_t packed = __popc(gmask) | (__popc(emask) << 16);  // <= 4096 each per tile
    const uint32_t pinc = wave_scan(packed);
    if (lane == 63) part[i & 1][wave] = pinc;
    __syncthreads();
    // wave totals -> offsets: lanes 0..15 of every wave scan the sixteen totals
    uint32_t tinc = part[i & 1][lane & 15];
    const uint32_t tmine = tinc;
#pragma unroll
    for (int o = 1; o < 16; o <<= 1) {
      const uint32_t u = __shfl_up(tinc, o, 16);
      if ((lane & 15) >= o) tinc += u;
    }
    const uint32_t woff = __shfl(tinc - tmine, wave), total = __shfl(tinc, 15);
    const uint32_t pexc = pinc - packed + woff;
    uint32_t pgt = run_gt + (pexc & 0xffffu);
    uint32_t peq = run_eq + (pexc >> 16);
    const int i0 = (tile0 + i) * kTile + 4 * t;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      if (gmask >> j & 1) {
        const uint32_t pos = pgt + (peq < need_eq ? peq : need_eq);
        if (pos < (uint32_t)k) out[pos] = i0 + j;  // the bound only matters if the counts were corrupted
        ++pgt;
      } else if (emask >> j & 1) {
        if (peq < need_eq && pgt + peq < (uint32_t)k) out[pgt + peq] = i0 + j;
        ++peq;
      }
    }
    run_gt += total & 0xffffu;
    run_eq += total >> 16;
    if (++i >= w.chunk_tiles || (int64_t)(tile0 + i) * kTile >= n) break;
    load_tile_raw(s, n, tile0 + i, x, valid);
  }
}

int launch_topk_mb(const float* scores, int64_t score_stride, const int32_t* seq_lens,
                   int32_t max_seq_len, const int32_t* k_per_seg, int32_t max_k, int32_t batch,
                   int32_t* idx_out, int64_t idx_stride, void* ws, hipStream_t stream) {
  const TopkMbWs w = carve_topk(ws, batch, max_seq_len);
  dim3 grid(w.max_chunks, batch), block(kMbThreads);
  hipLaunchKernelGGL(topk_mb_hist, grid, block, 0, stream, scores, score_stride, seq_lens,
                     max_seq_len, k_per_seg, max_k, w);
  hipLaunchKernelGGL(topk_mb_cand, grid, block, 0, stream, scores, score_stride, seq_lens,
                     max_seq_len, k_per_seg, max_k, w);
  hipLaunchKernelGGL(topk_mb_write, grid, block, 0, stream, scores, score_stride, seq_lens,
                     max_seq_len, k_per_seg, max_k, w, idx_out, idx_stride);
  OKV_HIP_CHECK(hipGetLastError());
  return OKV_OK;
}

}  // namespace okv
