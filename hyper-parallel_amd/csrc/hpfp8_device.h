// Device-side helpers shared by the quantize and GEMM kernels (gfx950 only).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace hpfp8 {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v8i __attribute__((ext_vector_type(8)));
typedef float v2f __attribute__((ext_vector_type(2)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef unsigned short v2u16 __attribute__((ext_vector_type(2)));

typedef unsigned int u32x2 __attribute__((ext_vector_type(2)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));

// Streaming (non-temporal) 64/128-bit accesses for data touched exactly once.
__device__ __forceinline__ uint4 nt_load16(const void* p) {
  u32x4 v = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(p));
  return make_uint4(v.x, v.y, v.z, v.w);
}
__device__ __forceinline__ void nt_store16(void* p, const uint4& v) {
  u32x4 t = {v.x, v.y, v.z, v.w};
  __builtin_nontemporal_store(t, reinterpret_cast<u32x4*>(p));
}
__device__ __forceinline__ void nt_store8(void* p, const uint2& v) {
  u32x2 t = {v.x, v.y};
  __builtin_nontemporal_store(t, reinterpret_cast<u32x2*>(p));
}

constexpr float kFp8Max = 448.0f;
constexpr float kAmaxEps = 1e-12f;
constexpr int kBlock = 128;

// DPP controls (gfx9 encoding)
constexpr int kDppQuadXor1 = 0xB1;      // quad_perm:[1,0,3,2]
constexpr int kDppQuadXor2 = 0x4E;      // quad_perm:[2,3,0,1]
constexpr int kDppRowHalfMirror = 0x141;
constexpr int kDppRowMirror = 0x140;

template <int CTRL>
__device__ __forceinline__ uint32_t dpp_u32(uint32_t v) {
  return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, CTRL, 0xf, 0xf, false);
}

// Packed max of two 16-bit magnitudes per word (bf16 |x| compares like an unsigned integer).
__device__ __forceinline__ uint32_t pk_max_u16(uint32_t a, uint32_t b) {
  v2u16 r = __builtin_elementwise_max(__builtin_bit_cast(v2u16, a), __builtin_bit_cast(v2u16, b));
  return __builtin_bit_cast(uint32_t, r);
}

__device__ __forceinline__ uint32_t umax(uint32_t a, uint32_t b) { return a > b ? a : b; }

// Max over the 16 lanes of a DPP row; every lane of the row ends with the result.
__device__ __forceinline__ uint32_t row16_max_u32(uint32_t v) {
  v = umax(v, dpp_u32<kDppQuadXor1>(v));
  v = umax(v, dpp_u32<kDppQuadXor2>(v));
  v = umax(v, dpp_u32<kDppRowHalfMirror>(v));
  v = umax(v, dpp_u32<kDppRowMirror>(v));
  return v;
}

// |bf16| magnitudes of the 8 values in a uint4, reduced to one 16-bit magnitude (low half).
__device__ __forceinline__ uint32_t mag8(const uint4& v) {
  uint32_t m = pk_max_u16(pk_max_u16(v.x & 0x7FFF7FFFu, v.y & 0x7FFF7FFFu),
                          pk_max_u16(v.z & 0x7FFF7FFFu, v.w & 0x7FFF7FFFu));
  return umax(m & 0xFFFFu, m >> 16);
}

__device__ __forceinline__ float bf16lo(uint32_t w) { return __uint_as_float(w << 16); }
__device__ __forceinline__ float bf16hi(uint32_t w) { return __uint_as_float(w & 0xFFFF0000u); }

// amax -> quantize multiplier and its inverse: two IEEE fp32 divisions, never rcp * x.
// pow2: the inverse is rounded up to the next power of two (its exponent field is then its E8M0 code,
// which the matrix instruction can apply by itself) and the multiplier is its exact reciprocal.
__device__ __forceinline__ void scales_from_amax(float amax, float& scale, float& scale_inv, int pow2 = 0) {
  float amc = amax < kAmaxEps ? kAmaxEps : amax;   // (not fmaxf: a NaN amax must stay NaN, so that the group's scales and codes are NaN)
  scale = kFp8Max / amc;
  scale_inv = amc / kFp8Max;
  if (pow2) {
    uint32_t u = __float_as_uint(scale_inv);
    if ((u & 0x007FFFFFu) && u < 0x7F800000u) u = (u & 0xFF800000u) + 0x00800000u;   // (a NaN stays as it is)
    scale_inv = __uint_as_float(u);
    scale = 1.0f / scale_inv;
  }
}

// Scales of the four groups that the 16 lanes of a row share (m[u] = the row's amax bits of group u, the same
// in all 16 lanes): lane l computes the pair of group l % 4 only, so the divisions run once per lane instead of
// four times, and every lane receives the four quantize multipliers through quad broadcasts.  mine / mine_inv
// are the lane's own pair (lanes 0..3 of a row hold groups 0..3).
__device__ __forceinline__ void scales4_from_amax(const uint32_t m[4], int l16, int pow2, float s[4], float& mine,
                                                  float& mine_inv) {
  const int u = l16 & 3;
  const uint32_t mm = u == 0 ? m[0] : (u == 1 ? m[1] : (u == 2 ? m[2] : m[3]));
  scales_from_amax(__uint_as_float(mm << 16), mine, mine_inv, pow2);
  const uint32_t sb = __float_as_uint(mine);
  s[0] = __uint_as_float(dpp_u32<0x00>(sb));   // quad_perm:[0,0,0,0]
  s[1] = __uint_as_float(dpp_u32<0x55>(sb));   // quad_perm:[1,1,1,1]
  s[2] = __uint_as_float(dpp_u32<0xAA>(sb));   // quad_perm:[2,2,2,2]
  s[3] = __uint_as_float(dpp_u32<0xFF>(sb));   // quad_perm:[3,3,3,3]
}

__device__ __forceinline__ float clamp448(float y) {
  const float c = __builtin_amdgcn_fmed3f(y, -kFp8Max, kFp8Max);   // of a NaN and two numbers the median instruction returns a number
  return y != y ? y : c;                                            // NaN stays NaN (and is cast to the NaN code)
}

// Two bf16 in one word -> two E4M3 codes in the chosen half of `old`.
// CLAMP = false is for kernels whose scale was derived from the amax of the very values being
// cast: then |x * scale| <= 448 * (1 + 2^-23), which rounds to 448 like the clamped value does, so
// the explicit clamp to +-448 cannot change a code for finite inputs and is left out.  With a scale
// that comes from elsewhere (a caller-supplied amax) the clamp is required.
template <bool HI, bool CLAMP>
__device__ __forceinline__ uint32_t cvt2(uint32_t old, uint32_t w, float scale) {
  float a = bf16lo(w) * scale;
  float b = bf16hi(w) * scale;
  if (CLAMP) {
    a = clamp448(a);
    b = clamp448(b);
  }
  return (uint32_t)__builtin_amdgcn_cvt_pk_fp8_f32(a, b, (int)old, HI);
}

// 8 bf16 (uint4) -> 8 E4M3 codes (uint2), element order kept.
template <bool CLAMP>
__device__ __forceinline__ uint2 cvt8(const uint4& v, float scale) {
  uint2 r;
  r.x = cvt2<true, CLAMP>(cvt2<false, CLAMP>(0u, v.x, scale), v.y, scale);
  r.y = cvt2<true, CLAMP>(cvt2<false, CLAMP>(0u, v.z, scale), v.w, scale);
  return r;
}

// ---- SwiGLU arithmetic (shared by the quantizers and the GEMM epilogue) ----
// exp(t), t clamped to [-86, 89], from IEEE fp32 operations only (no fused multiply-add, no hardware
// exp), so that the CPU restatement reproduces it bit for bit: k = rint(t * log2 e),
// r = t - k * ln2 (two constants), degree-6 Taylor polynomial in Horner form, times 2^(k-1), times 2
// (two steps so that results up to the largest float come out finite and larger ones as +inf).
__device__ __forceinline__ float exp_spec(float t) {
  t = fminf(fmaxf(t, -86.0f), 89.0f);
  const float k = __builtin_rintf(t * 1.44269504f);
  float r = t - k * 0.693359375f;
  r = r - k * -2.12194440e-4f;
  float p = 1.0f / 720.0f;
  p = p * r + 1.0f / 120.0f;
  p = p * r + 1.0f / 24.0f;
  p = p * r + 1.0f / 6.0f;
  p = p * r + 0.5f;
  p = p * r + 1.0f;
  p = p * r + 1.0f;
  return (p * __uint_as_float((uint32_t)((int)k + 126) << 23)) * 2.0f;
}

// silu(g) = g / (1 + exp(-g)).  FAST: with the hardware's base-2 exponential and reciprocal (each within one
// unit in the last place of fp32), 4 instructions instead of about 35; the result can differ from the exactly
// specified one in the last bits of fp32, which moves roughly one bf16 rounding in several thousand.
template <bool FAST>
__device__ __forceinline__ float silu_f32(float g) {
  if (FAST) return g * __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(g * -1.44269504f));
  return g / (1.0f + exp_spec(-g));
}

// bf16(bf16(silu(g)) * u) for two (g, u) pairs packed like their sources: the two roundings of the
// unfused bf16 graph (silu, then the product).
template <bool FAST>
__device__ __forceinline__ uint32_t swiglu2(uint32_t gw, uint32_t uw) {
  typedef float f32x2 __attribute__((ext_vector_type(2)));
  typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
  // both values of a pair through one conversion instruction, rounded to nearest even like the scalar cast
  const f32x2 sf = {silu_f32<FAST>(bf16lo(gw)), silu_f32<FAST>(bf16hi(gw))};
  const uint32_t sw = __builtin_bit_cast(uint32_t, __builtin_convertvector(sf, bf16x2));
  const f32x2 af = {bf16lo(sw) * bf16lo(uw), bf16hi(sw) * bf16hi(uw)};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(af, bf16x2));
}

}  // namespace hpfp8
