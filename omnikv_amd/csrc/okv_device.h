// Device-side element types and conversions shared by the attention kernels.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace okv {

static constexpr float kLog2e = 1.4426950408889634f;
static constexpr int kD = 128;

struct BF16 {
  uint16_t v;
};
struct F16 {
  uint16_t v;
};

// ---- eight consecutive elements -> fp32
__device__ __forceinline__ void load8(const float* p, float* o) {
  float4 a = *reinterpret_cast<const float4*>(p);
  float4 b = *reinterpret_cast<const float4*>(p + 4);
  o[0] = a.x; o[1] = a.y; o[2] = a.z; o[3] = a.w;
  o[4] = b.x; o[5] = b.y; o[6] = b.z; o[7] = b.w;
}
__device__ __forceinline__ void load8(const BF16* p, float* o) {
  uint4 u = *reinterpret_cast<const uint4*>(p);
  o[0] = __uint_as_float(u.x << 16); o[1] = __uint_as_float(u.x & 0xffff0000u);
  o[2] = __uint_as_float(u.y << 16); o[3] = __uint_as_float(u.y & 0xffff0000u);
  o[4] = __uint_as_float(u.z << 16); o[5] = __uint_as_float(u.z & 0xffff0000u);
  o[6] = __uint_as_float(u.w << 16); o[7] = __uint_as_float(u.w & 0xffff0000u);
}
__device__ __forceinline__ void load8(const F16* p, float* o) {
  uint4 u = *reinterpret_cast<const uint4*>(p);
  const _Float16* h = reinterpret_cast<const _Float16*>(&u);
#pragma unroll
  for (int i = 0; i < 8; ++i) o[i] = (float)h[i];
}

__device__ __forceinline__ void store1(float* p, float v) { *p = v; }
__device__ __forceinline__ void store1(BF16* p, float v) {
  uint32_t u = __float_as_uint(v);
  uint16_t r;
  if ((u & 0x7fffffffu) > 0x7f800000u) {
    r = 0x7fc0;  // NaN
  } else {
    u += 0x7fffu + ((u >> 16) & 1u);  // round to nearest even
    r = (uint16_t)(u >> 16);
  }
  p->v = r;
}
__device__ __forceinline__ void store1(F16* p, float v) {
  _Float16 h = (_Float16)v;
  p->v = *reinterpret_cast<uint16_t*>(&h);
}


// 16 raw bytes (eight 16-bit elements) -> fp32
__device__ __forceinline__ void cvt8(const BF16*, const uint4& u, float* o) {
  o[0] = __uint_as_float(u.x << 16); o[1] = __uint_as_float(u.x & 0xffff0000u);
  o[2] = __uint_as_float(u.y << 16); o[3] = __uint_as_float(u.y & 0xffff0000u);
  o[4] = __uint_as_float(u.z << 16); o[5] = __uint_as_float(u.z & 0xffff0000u);
  o[6] = __uint_as_float(u.w << 16); o[7] = __uint_as_float(u.w & 0xffff0000u);
}
__device__ __forceinline__ void cvt8(const F16*, const uint4& u, float* o) {
  const _Float16* h = reinterpret_cast<const _Float16*>(&u);
#pragma unroll
  for (int i = 0; i < 8; ++i) o[i] = (float)h[i];
}

// ---- matrix cores: D(16x16 fp32) += A(16 rows x 32) . B(32 x 16 cols) of 16-bit elements.
// Lane l holds A row l%16 / B column l%16, elements 8(l/16) .. +8 of the k-step, and
// D column l%16, rows 4(l/16) .. +4.
typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8_t;
typedef __attribute__((ext_vector_type(8))) _Float16 f16x8_t;
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2_t;
typedef __attribute__((ext_vector_type(2))) _Float16 f16x2_t;
typedef __attribute__((ext_vector_type(2))) float f32x2_t;
typedef __attribute__((ext_vector_type(4))) float f32x4_t;

__device__ __forceinline__ f32x4_t mfma16(const BF16*, const uint4& a, const uint4& b, f32x4_t c) {
  return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, a),
                                                 __builtin_bit_cast(bf16x8_t, b), c, 0, 0, 0);
}
__device__ __forceinline__ f32x4_t mfma16(const F16*, const uint4& a, const uint4& b, f32x4_t c) {
  return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8_t, a),
                                                __builtin_bit_cast(f16x8_t, b), c, 0, 0, 0);
}

// ---- K tiles for the matrix cores, loaded as whole rows.
// A 16-byte load per lane straight into the A-operand layout touches 16 different rows per
// 16 lanes (64 bytes of each); loading like V instead -- instruction i brings rows
// 4*(l/16) + i, lane l%16 its 16-byte chunk, whole 256-byte rows per 16 lanes, marked
// non-temporal -- streams measurably faster, and the tile is turned into the A-operand layout
// through a wave-private 4 KB of LDS: row R at R*256, its chunk c at position c ^ R, so the
// 16 lanes that write a row and the 16 lanes that read one k-chunk of 16 rows both cover all
// banks exactly once.  The LDS operations of one wave execute in order: no s_barrier.
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4_t;
__device__ __forceinline__ uint4 load_stream16(const void* p) {
  const u32x4_t v = __builtin_nontemporal_load(reinterpret_cast<const u32x4_t*>(p));
  return make_uint4(v.x, v.y, v.z, v.w);
}
__device__ __forceinline__ void k_rows_to_a_operand(char* stage, int r16, int j4, const uint4 (&rows_in)[4],
                                                    uint4 (&a)[4]) {
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int R = 4 * j4 + i;
    *reinterpret_cast<uint4*>(stage + R * 256 + 16 * (r16 ^ R)) = rows_in[i];
  }
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
  for (int s = 0; s < 4; ++s)
    a[s] = *reinterpret_cast<const uint4*>(stage + r16 * 256 + 16 * ((4 * s + j4) ^ r16));
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();  // the next tile's writes stay behind these reads
}
}  // namespace okv
