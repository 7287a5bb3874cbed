// The small per-token operations around the attention of a decode step: RMSNorm (with the
// residual add in front of it), rotary embedding of q and k, SiLU(gate) * up.  Each is a single
// launch over a handful of rows where a framework's op-by-op chain issues five to ten, and each
// rounds where that chain rounds (every torch op on 16-bit tensors computes in fp32 and rounds
// its result to the tensor type), so that the values match the op-by-op result.
#include <math.h>

#include "okv_device.h"
#include "okv_internal.h"

// Every product and sum below is rounded on its own, as a chain of separate framework ops rounds
// them: no contraction into fused multiply-adds (the compiler would otherwise form 16-bit FMAs).
#pragma clang fp contract(off)

namespace okv {

template <typename T>
__device__ __forceinline__ float ld1(const T* p);
template <>
__device__ __forceinline__ float ld1<float>(const float* p) { return *p; }
template <>
__device__ __forceinline__ float ld1<BF16>(const BF16* p) { return __uint_as_float((uint32_t)p->v << 16); }
template <>
__device__ __forceinline__ float ld1<F16>(const F16* p) {
  return (float)*reinterpret_cast<const _Float16*>(p);
}
// fp32 -> T -> fp32: what storing an intermediate result in a tensor of type T does to it
template <typename T>
__device__ __forceinline__ float rnd(float v) {
  T t;
  store1(&t, v);
  return ld1<T>(&t);
}
template <>
__device__ __forceinline__ float rnd<float>(float v) { return v; }

// Eight consecutive elements of type T as fp32 (one 16- or 32-byte load) and back.
template <typename T>
__device__ __forceinline__ void ld8(const T* p, float (&o)[8]) { load8(p, o); }
template <typename T>
__device__ __forceinline__ void st8(T* p, const float (&v)[8]) {
#pragma unroll
  for (int i = 0; i < 8; ++i) store1(p + i, v[i]);
}

// grid (rows), 256 threads.  h = x (+ residual, rounded to T and written to sum_out when asked for);
// out = T(weight * T(h * rsqrt(mean(h^2) + eps))).  A thread owns up to CH chunks of eight consecutive
// elements and keeps them in registers between the two passes, every load of a pass in flight at once
// (one launch, a handful of rows: the time is the length of the dependent chain, not the bytes);
// rows longer than 256 * 8 * CH elements, or not a multiple of eight, take the element-wise loop.
template <typename T, int CH>
__global__ __launch_bounds__(256) void rmsnorm_kernel(const T* __restrict__ x, const T* __restrict__ residual,
                                                      const T* __restrict__ weight, float eps, int hidden,
                                                      int aligned16, T* __restrict__ sum_out, T* __restrict__ out) {
  __shared__ float part[4];
  const int64_t row = blockIdx.x;
  const T* xr = x + row * hidden;
  const T* rr = residual ? residual + row * hidden : nullptr;
  const bool vec = aligned16 && (hidden & 7) == 0 && hidden <= 256 * 8 * CH;
  float h[CH][8], wgt[CH][8];
  float ss = 0.f;
  if (vec) {
    float r[CH][8];
#pragma unroll
    for (int c = 0; c < CH; ++c) {
      const int i = (c * 256 + (int)threadIdx.x) * 8;
      if (i < hidden) {
        ld8<T>(xr + i, h[c]);
        if (rr) ld8<T>(rr + i, r[c]);
        ld8<T>(weight + i, wgt[c]);  // needed after the reduction only: one round trip instead of two
      }
    }
#pragma unroll
    for (int c = 0; c < CH; ++c) {
      const int i = (c * 256 + (int)threadIdx.x) * 8;
      if (i < hidden) {
        if (rr) {
#pragma unroll
          for (int e = 0; e < 8; ++e) h[c][e] = rnd<T>(h[c][e] + r[c][e]);
          st8<T>(sum_out + row * hidden + i, h[c]);
        }
#pragma unroll
        for (int e = 0; e < 8; ++e) ss = fmaf(h[c][e], h[c][e], ss);
      }
    }
  } else {
    for (int i = threadIdx.x; i < hidden; i += 256) {
      float v = ld1<T>(xr + i);
      if (rr) {
        v = rnd<T>(v + ld1<T>(rr + i));
        store1(sum_out + row * hidden + i, v);
      }
      ss = fmaf(v, v, ss);
    }
  }
#pragma unroll
  for (int o = 32; o >= 1; o >>= 1) ss += __shfl_xor(ss, o);
  if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = ss;
  __syncthreads();
  const float var = ((part[0] + part[1]) + (part[2] + part[3])) / (float)hidden;
  const float rstd = rsqrtf(var + eps);
  if (vec) {
#pragma unroll
    for (int c = 0; c < CH; ++c) {
      const int i = (c * 256 + (int)threadIdx.x) * 8;
      if (i < hidden) {
        float o[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) o[e] = wgt[c][e] * rnd<T>(h[c][e] * rstd);
        st8<T>(out + row * hidden + i, o);
      }
    }
  } else {
    const T* hr = rr ? sum_out + row * hidden : xr;  // this thread re-reads what it wrote itself
    for (int i = threadIdx.x; i < hidden; i += 256)
      store1(out + row * hidden + i, ld1<T>(weight + i) * rnd<T>(ld1<T>(hr + i) * rstd));
  }
}

// grid (rows, heads_q + heads_k [+ heads_k]), 64 threads (D = 128: a lane owns elements l and l + 64).
// x_rot = T(T(x * cos) + T(rotate_half(x) * sin)), rotate_half(x) = (-x[D/2:], x[:D/2]).
// The rotated k row of (request r, kv head h) goes to k_dst + r*dst_batch + h*dst_head + pos*dst_token,
// pos read from device memory when pos_dev is given -- a contiguous (rows, heads, D) output or the
// K store of a cache alike; with v given, its row is copied to the same place of v_dst.
template <typename T>
__global__ __launch_bounds__(64) void rope_kernel(const T* __restrict__ q, const T* __restrict__ k,
                                                  const T* __restrict__ v, const T* __restrict__ cos,
                                                  const T* __restrict__ sin, int hq, int hkv, int64_t q_row_stride,
                                                  int64_t k_row_stride, int64_t v_row_stride, T* __restrict__ q_out,
                                                  T* __restrict__ k_dst, T* __restrict__ v_dst, int64_t dst_token,
                                                  int64_t dst_head, int64_t dst_batch,
                                                  const int64_t* __restrict__ pos_dev, int64_t pos) {
  const int64_t row = blockIdx.x;
  const int head = blockIdx.y, l = threadIdx.x;
  if (head >= hq) {
    if (pos_dev) pos = pos_dev[0];
    if (head >= hq + hkv) {  // the value row: a copy
      const int h = head - hq - hkv;
      const T* src = v + row * v_row_stride + (int64_t)h * kD;
      T* dst = v_dst + row * dst_batch + h * dst_head + pos * dst_token;
      dst[l] = src[l];
      dst[l + 64] = src[l + 64];
      return;
    }
  }
  const bool is_q = head < hq;
  const int h = is_q ? head : head - hq;
  const T* src = (is_q ? q + row * q_row_stride : k + row * k_row_stride) + (int64_t)h * kD;
  T* dst = is_q ? q_out + (row * hq + h) * kD : k_dst + row * dst_batch + h * dst_head + pos * dst_token;
  const float x0 = ld1<T>(src + l), x1 = ld1<T>(src + l + 64);
  const float c0 = ld1<T>(cos + row * kD + l), c1 = ld1<T>(cos + row * kD + l + 64);
  const float s0 = ld1<T>(sin + row * kD + l), s1 = ld1<T>(sin + row * kD + l + 64);
  store1(dst + l, rnd<T>(x0 * c0) + rnd<T>(-x1 * s0));
  store1(dst + l + 64, rnd<T>(x1 * c1) + rnd<T>(x0 * s1));
}

// out = T(T(silu(gate)) * up), silu(g) = g / (1 + exp(-g)); eight consecutive elements per thread
// (n a multiple of 8 and 16-byte aligned operands), else one.
template <typename T, bool VEC>
__global__ __launch_bounds__(256) void silu_mul_kernel(const T* __restrict__ gate, const T* __restrict__ up,
                                                       int64_t n, T* __restrict__ out) {
  if (VEC) {
    for (int64_t i = ((int64_t)blockIdx.x * 256 + threadIdx.x) * 8; i < n; i += (int64_t)gridDim.x * 256 * 8) {
      float g[8], u[8], o[8];
      ld8<T>(gate + i, g);
      ld8<T>(up + i, u);
#pragma unroll
      for (int e = 0; e < 8; ++e) o[e] = rnd<T>(g[e] / (1.0f + expf(-g[e]))) * u[e];
      st8<T>(out + i, o);
    }
  } else {
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (int64_t)gridDim.x * 256) {
      const float g = ld1<T>(gate + i);
      store1(out + i, rnd<T>(g / (1.0f + expf(-g))) * ld1<T>(up + i));
    }
  }
}

template <typename T>
static void launch_rmsnorm(const void* x, const void* residual, const void* weight, float eps, int rows, int hidden,
                           void* sum_out, void* out, hipStream_t stream) {
  const uintptr_t all = (uintptr_t)x | (uintptr_t)residual | (uintptr_t)weight | (uintptr_t)sum_out | (uintptr_t)out;
  hipLaunchKernelGGL((rmsnorm_kernel<T, 4>), dim3(rows), dim3(256), 0, stream, (const T*)x, (const T*)residual,
                     (const T*)weight, eps, hidden, (int)((all & 15) == 0), (T*)sum_out, (T*)out);
}
template <typename T>
static void launch_rope(const void* q, const void* k, const void* v, const void* cos, const void* sin, int rows,
                        int hq, int hkv, int64_t qs, int64_t ks, int64_t vs, void* q_out, void* k_dst, void* v_dst,
                        int64_t dst_token, int64_t dst_head, int64_t dst_batch, const int64_t* pos_dev, int64_t pos,
                        hipStream_t stream) {
  hipLaunchKernelGGL(rope_kernel<T>, dim3(rows, hq + hkv + (v ? hkv : 0)), dim3(64), 0, stream, (const T*)q,
                     (const T*)k, (const T*)v, (const T*)cos, (const T*)sin, hq, hkv, qs, ks, vs, (T*)q_out, (T*)k_dst,
                     (T*)v_dst, dst_token, dst_head, dst_batch, pos_dev, pos);
}
template <typename T>
static void launch_silu_mul(const void* gate, const void* up, int64_t n, void* out, hipStream_t stream) {
  const bool vec = n % 8 == 0 && (((uintptr_t)gate | (uintptr_t)up | (uintptr_t)out) & 15) == 0;
  int64_t blocks = ((vec ? n / 8 : n) + 255) / 256;
  if (blocks > 4096) blocks = 4096;
  if (vec)
    hipLaunchKernelGGL((silu_mul_kernel<T, true>), dim3((unsigned)blocks), dim3(256), 0, stream, (const T*)gate,
                       (const T*)up, n, (T*)out);
  else
    hipLaunchKernelGGL((silu_mul_kernel<T, false>), dim3((unsigned)blocks), dim3(256), 0, stream, (const T*)gate,
                       (const T*)up, n, (T*)out);
}

}  // namespace okv

using namespace okv;

#define OKV_BY_DTYPE(dtype, CALL)                                     \
  switch (dtype) {                                                    \
    case OKV_F32: CALL(float); break;                                 \
    case OKV_BF16: CALL(BF16); break;                                 \
    case OKV_F16: CALL(F16); break;                                   \
    default:                                                          \
      set_error("dtype %d not supported", dtype);                     \
      return OKV_ERR_UNSUPPORTED;                                     \
  }

extern "C" {

int okv_rmsnorm(const void* x, const void* residual, const void* weight, float eps, int32_t rows, int32_t hidden,
                int32_t dtype, void* sum_out, void* out, okv_stream_t stream) {
  OKV_REQUIRE(x && weight && out, OKV_ERR_INVALID, "x, weight or out is NULL");
  OKV_REQUIRE(rows >= 0 && hidden >= 1, OKV_ERR_INVALID, "bad rows or hidden");
  OKV_REQUIRE(!residual || sum_out, OKV_ERR_INVALID, "a residual needs sum_out");
  if (rows == 0) return OKV_OK;
#define CALL(T) launch_rmsnorm<T>(x, residual, weight, eps, rows, hidden, sum_out, out, (hipStream_t)stream)
  OKV_BY_DTYPE(dtype, CALL)
#undef CALL
  OKV_HIP_CHECK(hipGetLastError());
  return OKV_OK;
}

int okv_rope(const void* q, int64_t q_row_stride, const void* k, int64_t k_row_stride, const void* cos,
             const void* sin, int32_t rows, int32_t num_q_heads, int32_t num_kv_heads, int32_t head_dim,
             int32_t dtype, void* q_out, void* k_out, okv_stream_t stream) {
  OKV_REQUIRE(q && k && cos && sin && q_out && k_out, OKV_ERR_INVALID, "NULL argument");
  OKV_REQUIRE(head_dim == kD, OKV_ERR_UNSUPPORTED, "head_dim %d not supported (kernels are built for 128)", head_dim);
  OKV_REQUIRE(rows >= 0 && num_q_heads >= 1 && num_kv_heads >= 1, OKV_ERR_INVALID, "bad rows or head counts");
  if (rows == 0) return OKV_OK;
#define CALL(T)                                                                                                   \
  launch_rope<T>(q, k, nullptr, cos, sin, rows, num_q_heads, num_kv_heads, q_row_stride, k_row_stride, 0, q_out, \
                 k_out, nullptr, 0, kD, (int64_t)num_kv_heads * kD, nullptr, 0, (hipStream_t)stream)
  OKV_BY_DTYPE(dtype, CALL)
#undef CALL
  OKV_HIP_CHECK(hipGetLastError());
  return OKV_OK;
}

int okv_rope_append(const void* q, int64_t q_row_stride, const void* k, int64_t k_row_stride, const void* v,
                    int64_t v_row_stride, const void* cos, const void* sin, int32_t rows, int32_t num_q_heads,
                    int32_t num_kv_heads, int32_t head_dim, int32_t dtype, void* q_out, void* k_store, void* v_store,
                    int64_t store_token_stride, int64_t store_head_stride, int64_t store_batch_stride,
                    const int64_t* pos_dev, int64_t pos, okv_stream_t stream) {
  OKV_REQUIRE(q && k && v && cos && sin && q_out && k_store && v_store, OKV_ERR_INVALID, "NULL argument");
  OKV_REQUIRE(head_dim == kD, OKV_ERR_UNSUPPORTED, "head_dim %d not supported (kernels are built for 128)", head_dim);
  OKV_REQUIRE(rows >= 0 && num_q_heads >= 1 && num_kv_heads >= 1, OKV_ERR_INVALID, "bad rows or head counts");
  OKV_REQUIRE(pos_dev || pos >= 0, OKV_ERR_INVALID, "negative position");
  if (rows == 0) return OKV_OK;
#define CALL(T)                                                                                                    \
  launch_rope<T>(q, k, v, cos, sin, rows, num_q_heads, num_kv_heads, q_row_stride, k_row_stride, v_row_stride,     \
                 q_out, k_store, v_store, store_token_stride, store_head_stride, store_batch_stride, pos_dev, pos, \
                 (hipStream_t)stream)
  OKV_BY_DTYPE(dtype, CALL)
#undef CALL
  OKV_HIP_CHECK(hipGetLastError());
  return OKV_OK;
}

int okv_silu_mul(const void* gate, const void* up, int64_t n, int32_t dtype, void* out, okv_stream_t stream) {
  OKV_REQUIRE(gate && up && out, OKV_ERR_INVALID, "NULL argument");
  OKV_REQUIRE(n >= 0, OKV_ERR_INVALID, "bad element count");
  if (n == 0) return OKV_OK;
#define CALL(T) launch_silu_mul<T>(gate, up, n, out, (hipStream_t)stream)
  OKV_BY_DTYPE(dtype, CALL)
#undef CALL
  OKV_HIP_CHECK(hipGetLastError());
  return OKV_OK;
}

}  // extern "C"
