// Per-request top-k of fp32 scores by radix select, with ordered compaction.
//
// One 1024-thread workgroup per request.  Scores map to order-preserving 32-bit
// keys (-0.0 == +0.0, NaN largest).  The k-th largest key T is found with an
// 11/11/10-bit radix descent whose first level bins the key range actually
// present (min..max) so that narrow score distributions still spread over the
// LDS histogram; the candidates of the first level's bin are pulled into LDS so
// the lower levels never touch global memory again.  A final ordered pass emits
// the indices of keys > T, and of the lowest-index keys == T until k are out,
// using wave ballots and popcount prefixes; the output is ascending by
// construction.
#include "okv_internal.h"

namespace okv {

static constexpr int kThreads = 1024;
static constexpr int kWaves = kThreads / 64;
static constexpr int kBins = 2048;
static constexpr int kCandCap = 8192;  // candidate keys held in LDS (32 KB)

__device__ __forceinline__ uint32_t score_key(float s) {
  uint32_t u = __float_as_uint(s);
  if ((u & 0x7fffffffu) > 0x7f800000u) return 0xffffffffu;  // NaN ranks first
  if (u == 0x80000000u) u = 0;                              // -0.0 == +0.0
  return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}

struct TopkShared {
  uint32_t hist[kBins];
  uint32_t cand[kCandCap];
  uint32_t wave_tmp[kWaves];
  uint32_t wave_tmp2[kWaves];
  uint32_t bcast[8];
};

// Finds the bin holding the `want`-th largest element of a histogram of `nbins`
// bins (bin 0 = smallest keys).  Returns the bin in *bin and the rank still wanted
// inside it (1-based) in *want_in_bin.  Every thread receives the result.
__device__ void find_bin(TopkShared& sh, int nbins, uint32_t want, uint32_t* bin,
                         uint32_t* want_in_bin, uint32_t* bin_count) {
  __syncthreads();
  // thread t owns bins [t*per, t*per+per) counted from the TOP
  const int per = (nbins + kThreads - 1) / kThreads;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  uint32_t mine = 0;
  for (int i = 0; i < per; ++i) {
    int bi = nbins - 1 - (tid * per + i);
    if (bi >= 0) mine += sh.hist[bi];
  }
  // inclusive scan over threads (descending key order)
  uint32_t inc = mine;
#pragma unroll
  for (int o = 1; o < 64; o <<= 1) {
    uint32_t v = __shfl_up(inc, o);
    if (lane >= o) inc += v;
  }
  if (lane == 63) sh.wave_tmp[wave] = inc;
  __syncthreads();
  uint32_t wave_off = 0;
  for (int x = 0; x < wave; ++x) wave_off += sh.wave_tmp[x];
  inc += wave_off;
  uint32_t exc = inc - mine;
  if (exc < want && want <= inc) {  // exactly one thread
    uint32_t run = exc;
    for (int i = 0; i < per; ++i) {
      int bi = nbins - 1 - (tid * per + i);
      uint32_t hcount = bi >= 0 ? sh.hist[bi] : 0;
      if (run < want && want <= run + hcount) {
        sh.bcast[0] = (uint32_t)bi;
        sh.bcast[1] = want - run;
        sh.bcast[2] = hcount;
        break;
      }
      run += hcount;
    }
  }
  __syncthreads();
  *bin = sh.bcast[0];
  *want_in_bin = sh.bcast[1];
  *bin_count = sh.bcast[2];
  __syncthreads();
}

// Calls fn(key) for every score of the request, sixteen loads in flight per thread.
template <typename F>
__device__ __forceinline__ void for_each_key(const float* __restrict__ s, int n, F fn) {
  const int tid = threadIdx.x;
  int done = 0;
  if ((((uintptr_t)s) & 15) == 0) {
    const float4* s4 = reinterpret_cast<const float4*>(s);
    const int nvec = n >> 2;
    int i = tid;
    for (; i + 3 * kThreads < nvec; i += 4 * kThreads) {
      const float4 a = s4[i], b = s4[i + kThreads], c = s4[i + 2 * kThreads], d = s4[i + 3 * kThreads];
      fn(score_key(a.x)); fn(score_key(a.y)); fn(score_key(a.z)); fn(score_key(a.w));
      fn(score_key(b.x)); fn(score_key(b.y)); fn(score_key(b.z)); fn(score_key(b.w));
      fn(score_key(c.x)); fn(score_key(c.y)); fn(score_key(c.z)); fn(score_key(c.w));
      fn(score_key(d.x)); fn(score_key(d.y)); fn(score_key(d.z)); fn(score_key(d.w));
    }
    for (; i < nvec; i += kThreads) {
      const float4 a = s4[i];
      fn(score_key(a.x)); fn(score_key(a.y)); fn(score_key(a.z)); fn(score_key(a.w));
    }
    done = nvec << 2;
  }
  for (int i = done + tid; i < n; i += kThreads) fn(score_key(s[i]));
}

__device__ __forceinline__ void clear_hist(TopkShared& sh, int nbins) {
  for (int i = threadIdx.x; i < nbins; i += kThreads) sh.hist[i] = 0;
  __syncthreads();
}

__global__ __launch_bounds__(kThreads) void topk_select(const float* __restrict__ scores,
                                                        int64_t score_stride,
                                                        const int32_t* __restrict__ seq_lens,
                                                        int32_t max_seq_len,
                                                        const int32_t* __restrict__ k_per_seg,
                                                        int32_t max_k, int32_t* __restrict__ idx_out,
                                                        int64_t idx_stride) {
  __shared__ TopkShared sh;
  const int b = blockIdx.x;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int n = seq_lens ? seq_lens[b] : max_seq_len;
  int k = k_per_seg ? k_per_seg[b] : max_k;
  if (k > n) k = n;
  if (k <= 0) return;
  const float* s = scores + (int64_t)b * score_stride;
  int32_t* out = idx_out + (int64_t)b * idx_stride;
  if (k == n) {
    for (int i = tid; i < n; i += kThreads) out[i] = i;
    return;
  }

  // ---- pass 0: key range
  uint32_t kmin = 0xffffffffu, kmax = 0;
  for_each_key(s, n, [&](uint32_t key) {
    kmin = key < kmin ? key : kmin;
    kmax = key > kmax ? key : kmax;
  });
#pragma unroll
  for (int o = 32; o >= 1; o >>= 1) {
    uint32_t a = __shfl_xor(kmin, o), c = __shfl_xor(kmax, o);
    kmin = a < kmin ? a : kmin;
    kmax = c > kmax ? c : kmax;
  }
  if (lane == 0) {
    sh.wave_tmp[wave] = kmin;
    sh.wave_tmp2[wave] = kmax;
  }
  __syncthreads();
  kmin = sh.wave_tmp[0];
  kmax = sh.wave_tmp2[0];
  for (int x = 1; x < kWaves; ++x) {
    kmin = sh.wave_tmp[x] < kmin ? sh.wave_tmp[x] : kmin;
    kmax = sh.wave_tmp2[x] > kmax ? sh.wave_tmp2[x] : kmax;
  }
  __syncthreads();

  uint32_t T;        // k-th largest key
  uint32_t need_eq;  // how many keys == T belong to the selection
  if (kmin == kmax) {
    T = kmin;
    need_eq = (uint32_t)k;
  } else {
    // ---- level 0: bins over (key - kmin) >> shift0, at most 2048 bins
    const uint32_t range = kmax - kmin;
    int shift0 = 0;
    while ((range >> shift0) >= (uint32_t)kBins) ++shift0;
    clear_hist(sh, kBins);
    for_each_key(s, n, [&](uint32_t key) { atomicAdd(&sh.hist[(key - kmin) >> shift0], 1u); });
    uint32_t bin0, want, cnt;
    find_bin(sh, kBins, (uint32_t)k, &bin0, &want, &cnt);
    // keys of bin0 are kmin + [bin0 << shift0, (bin0+1) << shift0)
    const uint32_t base0 = kmin + (bin0 << shift0);
    if (shift0 == 0) {
      T = base0;
      need_eq = want;
    } else if (cnt <= (uint32_t)kCandCap) {
      // ---- pull the candidates (low bits only) into LDS
      if (tid == 0) sh.bcast[4] = 0;
      __syncthreads();
      for_each_key(s, n, [&](uint32_t key) {
        const uint32_t rel = key - kmin;
        if ((rel >> shift0) == bin0) {
          uint32_t pos = atomicAdd(&sh.bcast[4], 1u);
          sh.cand[pos] = rel & ((1u << shift0) - 1u);
        }
      });
      __syncthreads();
      const int nc = (int)cnt;
      // descend the remaining shift0 bits, up to 11 at a time
      uint32_t prefix = 0;  // decided high part of the low bits
      int rem = shift0;
      while (rem > 0) {
        const int bits = rem > 11 ? 11 : rem;
        const int sh_r = rem - bits;
        clear_hist(sh, 1 << bits);
        for (int i = tid; i < nc; i += kThreads) {
          uint32_t v = sh.cand[i];
          if ((rem == shift0) || ((v >> rem) == prefix))
            atomicAdd(&sh.hist[(v >> sh_r) & ((1u << bits) - 1u)], 1u);
        }
        uint32_t bsel, cnt2;
        find_bin(sh, 1 << bits, want, &bsel, &want, &cnt2);
        prefix = (prefix << bits) | bsel;
        rem = sh_r;
      }
      T = base0 + prefix;
      need_eq = want;
    } else {
      // ---- too many candidates for LDS: descend over global memory
      uint32_t prefix = bin0;  // decided value of rel >> rem
      int rem = shift0;
      while (rem > 0) {
        const int bits = rem > 11 ? 11 : rem;
        const int sh_r = rem - bits;
        clear_hist(sh, 1 << bits);
        for_each_key(s, n, [&](uint32_t key) {
          const uint32_t rel = key - kmin;
          if ((rel >> rem) == prefix)
            atomicAdd(&sh.hist[(rel >> sh_r) & ((1u << bits) - 1u)], 1u);
        });
        uint32_t bsel, cnt2;
        find_bin(sh, 1 << bits, want, &bsel, &want, &cnt2);
        prefix = (prefix << bits) | bsel;
        rem = sh_r;
      }
      T = kmin + prefix;
      need_eq = want;
    }
  }

  // ---- ordered compaction: 4 consecutive tokens per thread per chunk
  const bool vec = (((uintptr_t)s) & 15) == 0;
  auto load_chunk = [&](int base, float (&x)[4]) {
    const int i0 = base + tid * 4;
    if (vec && i0 + 3 < n) {
      const float4 a = *reinterpret_cast<const float4*>(s + i0);
      x[0] = a.x; x[1] = a.y; x[2] = a.z; x[3] = a.w;
    } else {
#pragma unroll
      for (int j = 0; j < 4; ++j) x[j] = (i0 + j < n) ? s[i0 + j] : 0.f;
    }
  };
  uint32_t run_gt = 0, run_eq = 0;  // selected-so-far counts before this chunk
  float cur[4], nxt[4];
  load_chunk(0, cur);
  for (int base = 0; base < n; base += kThreads * 4) {
    if (base + kThreads * 4 < n) load_chunk(base + kThreads * 4, nxt);
    const int i0 = base + tid * 4;
    uint32_t gt[4], eq[4];
    uint32_t cgt = 0, ceq = 0;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const bool valid = i0 + j < n;
      const uint32_t key = score_key(cur[j]);
      gt[j] = valid && key > T;
      eq[j] = valid && key == T;
      cgt += gt[j];
      ceq += eq[j];
    }
    uint32_t packed = cgt | (ceq << 16);  // both <= 4096 per chunk
    uint32_t inc = packed;
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) {
      uint32_t v = __shfl_up(inc, o);
      if (lane >= o) inc += v;
    }
    if (lane == 63) sh.wave_tmp[wave] = inc;
    __syncthreads();
    uint32_t woff = 0, total = 0;
    for (int x = 0; x < kWaves; ++x) {
      uint32_t v = sh.wave_tmp[x];
      if (x < wave) woff += v;
      total += v;
    }
    __syncthreads();
    uint32_t exc = inc - packed + woff;
    uint32_t pgt = run_gt + (exc & 0xffffu);
    uint32_t peq = run_eq + (exc >> 16);
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      if (gt[j]) {
        out[pgt + (peq < need_eq ? peq : need_eq)] = i0 + j;
        ++pgt;
      } else if (eq[j]) {
        if (peq < need_eq) out[pgt + peq] = i0 + j;
        ++peq;
      }
    }
    run_gt += total & 0xffffu;
    run_eq += total >> 16;
#pragma unroll
    for (int j = 0; j < 4; ++j) cur[j] = nxt[j];
  }
}

int launch_topk_mb(const float* scores, int64_t score_stride, const int32_t* seq_lens,
                   int32_t max_seq_len, const int32_t* k_per_seg, int32_t max_k, int32_t batch,
                   int32_t* idx_out, int64_t idx_stride, void* ws, hipStream_t stream);

}  // namespace okv

using namespace okv;

extern "C" int okv_topk(const float* scores, int64_t score_stride, const int32_t* seq_lens,
                        int32_t max_seq_len, const int32_t* k_per_seg, int32_t max_k,
                        int32_t batch, int32_t* idx_out, int64_t idx_stride, void* ws,
                        size_t ws_bytes, okv_stream_t stream) {
  OKV_REQUIRE(scores && idx_out, OKV_ERR_INVALID, "scores or idx_out is NULL");
  OKV_REQUIRE(batch >= 1, OKV_ERR_INVALID, "batch must be >= 1");
  OKV_REQUIRE(max_seq_len >= 0 && max_k >= 0, OKV_ERR_INVALID, "negative length");
  OKV_REQUIRE(score_stride >= max_seq_len, OKV_ERR_INVALID, "score_stride < max_seq_len");
  int kk = max_k < max_seq_len ? max_k : max_seq_len;
  OKV_REQUIRE(idx_stride >= kk, OKV_ERR_INVALID, "idx_stride < min(max_k, max_seq_len)");
  if (max_seq_len == 0 || max_k == 0) return OKV_OK;
  // long vectors: chunked multi-workgroup passes, if the caller brought the workspace
  if (max_seq_len >= kMultiBlockMinLen && ws != nullptr &&
      ws_bytes >= topk_mb_workspace_bytes(batch, max_seq_len))
    return launch_topk_mb(scores, score_stride, seq_lens, max_seq_len, k_per_seg, max_k, batch,
                          idx_out, idx_stride, ws, (hipStream_t)stream);
  hipLaunchKernelGGL(topk_select, dim3(batch), dim3(kThreads), 0, (hipStream_t)stream, scores,
                     score_stride, seq_lens, max_seq_len, k_per_seg, max_k, idx_out, idx_stride);
  OKV_HIP_CHECK(hipGetLastError());
  return OKV_OK;
}
