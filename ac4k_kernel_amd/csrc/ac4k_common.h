// Shared host/device helpers of the gfx950 NVFP4 library.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "ac4k_nvfp4.h"

namespace ac4k {

// ---------------------------------------------------------------------------
// host side: error reporting for the C ABI
// ---------------------------------------------------------------------------
int set_error(const char *fmt, ...) __attribute__((format(printf, 1, 2)));
int check_launch(const char *what);  // hipGetLastError() -> status

#define AC4K_REQUIRE(cond, ...)                      \
  do {                                               \
    if (!(cond)) return ::ac4k::set_error(__VA_ARGS__); \
  } while (0)

__host__ __device__ constexpr inline int64_t ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }
__host__ __device__ constexpr inline int64_t align_up(int64_t a, int64_t b) { return ceil_div(a, b) * b; }

// ---------------------------------------------------------------------------
// device side
// ---------------------------------------------------------------------------
typedef uint16_t u16x2 __attribute__((ext_vector_type(2)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

// streaming (non-temporal) 16-byte load / 4- and 8-byte stores: data touched once
__device__ __forceinline__ uint4 ld_stream_u4(const void *p) {
  u32x4 v = __builtin_nontemporal_load(static_cast<const u32x4 *>(p));
  return make_uint4(v.x, v.y, v.z, v.w);
}
__device__ __forceinline__ void st_stream_u2(void *p, uint2 v) {
  u32x2 w = {v.x, v.y};
  __builtin_nontemporal_store(w, static_cast<u32x2 *>(p));
}
__device__ __forceinline__ void st_stream_u1(void *p, uint32_t v) {
  __builtin_nontemporal_store(v, static_cast<uint32_t *>(p));
}

// DPP controls (lane i of a 16-lane row receives from ...)
constexpr int DPP_QUAD_XOR1 = 0xB1;  // quad_perm:[1,0,3,2]
constexpr int DPP_QUAD_XOR2 = 0x4E;  // quad_perm:[2,3,0,1]
constexpr int DPP_ROW_SHL(int n) { return 0x100 + n; }  // lane i <- lane i+n
constexpr int DPP_ROW_SHR(int n) { return 0x110 + n; }  // lane i <- lane i-n
constexpr int DPP_ROW_MIRROR = 0x140;
constexpr int DPP_ROW_HALF_MIRROR = 0x141;

template <int CTRL>
__device__ __forceinline__ uint32_t dpp_u32(uint32_t v) {
  // bound_ctrl = true: lanes whose source is outside the row read 0
  return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, CTRL, 0xF, 0xF, true);
}

__device__ __forceinline__ uint32_t umax32(uint32_t a, uint32_t b) { return a > b ? a : b; }

// max over groups of 2/4/8/16 adjacent lanes (result in every lane of the group)
template <int GROUP>
__device__ __forceinline__ uint32_t group_umax(uint32_t v) {
  static_assert(GROUP == 1 || GROUP == 2 || GROUP == 4 || GROUP == 8 || GROUP == 16 || GROUP == 32 ||
                GROUP == 64);
  if (GROUP >= 2) v = umax32(v, dpp_u32<DPP_QUAD_XOR1>(v));
  if (GROUP >= 4) v = umax32(v, dpp_u32<DPP_QUAD_XOR2>(v));
  if (GROUP >= 8) v = umax32(v, dpp_u32<DPP_ROW_HALF_MIRROR>(v));
  if (GROUP >= 16) v = umax32(v, dpp_u32<DPP_ROW_MIRROR>(v));
  if (GROUP >= 32) v = umax32(v, (uint32_t)__builtin_amdgcn_ds_swizzle((int)v, 0x401F));  // xor 16
  if (GROUP >= 64) {
    uint32_t lo = (uint32_t)__builtin_amdgcn_readlane((int)v, 0);
    uint32_t hi = (uint32_t)__builtin_amdgcn_readlane((int)v, 32);
    v = umax32(lo, hi);
  }
  return v;
}

// |bf16| maximum of the eight values in a 16-byte vector, as a bf16 bit pattern in bits 0..15.
// Non-negative bf16 patterns order like unsigned integers.
__device__ __forceinline__ uint32_t absmax_bf16x8(uint4 v) {
  u16x2 a = __builtin_bit_cast(u16x2, v.x & 0x7fff7fffu);
  u16x2 b = __builtin_bit_cast(u16x2, v.y & 0x7fff7fffu);
  u16x2 c = __builtin_bit_cast(u16x2, v.z & 0x7fff7fffu);
  u16x2 d = __builtin_bit_cast(u16x2, v.w & 0x7fff7fffu);
  u16x2 m = __builtin_elementwise_max(__builtin_elementwise_max(a, b), __builtin_elementwise_max(c, d));
  uint32_t mm = __builtin_bit_cast(uint32_t, m);
  return umax32(mm & 0xffffu, mm >> 16);
}

__device__ __forceinline__ float bf16_lo(uint32_t w) { return __uint_as_float(w << 16); }
__device__ __forceinline__ float bf16_hi(uint32_t w) { return __uint_as_float(w & 0xffff0000u); }
__device__ __forceinline__ float bf16_bits_to_f32(uint32_t h) { return __uint_as_float(h << 16); }

// cvt.rn.satfinite.e4m3.f32 for a NON-NEGATIVE or NaN input (the nvfp4 block scale).
// v_cvt_pk_fp8_f32 on gfx950 is OCP E4M3 with RNE but turns |x| >= 464 into NaN, so the
// input is clamped to 448 first; NaN is mapped to 0x7F explicitly.
__device__ __forceinline__ uint32_t f32_to_ue4m3_satfinite(float x) {
  float c = __builtin_fminf(x, 448.0f);
  uint32_t code = (uint32_t)__builtin_amdgcn_cvt_pk_fp8_f32(c, c, 0, false) & 0xffu;
  return (x != x) ? 0x7fu : code;
}

__device__ __forceinline__ float e4m3_to_f32(uint32_t code) {
  return __builtin_amdgcn_cvt_f32_fp8((int)code, 0);
}

// cvt.rn.satfinite.e2m1x2.f32 of eight floats -> eight nibbles, element 0 in bits 0..3.
// v_cvt_scalef32_pk_fp4_f32 with scale 1.0 is RNE, ties to the even code, saturating at 6,
// sign of zero kept, first source in the low nibble.
__device__ __forceinline__ uint32_t f32x8_to_e2m1x8(const float (&f)[8]) {
  uint32_t r = 0;
  r = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(r, f[0], f[1], 1.0f, 0);
  r = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(r, f[2], f[3], 1.0f, 1);
  r = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(r, f[4], f[5], 1.0f, 2);
  r = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(r, f[6], f[7], 1.0f, 3);
  return r;
}

// ---------------------------------------------------------------------------
// nvfp4 block arithmetic shared by the quantizers and the linear kernel that quantizes its activation
// ---------------------------------------------------------------------------
// Correctly rounded fp32 reciprocals of the 128 non-negative E4M3 codes (entry 0 is 0, entry
// 0x7F is NaN): the block scale takes one of these values, so the IEEE division of the spec
// (about a dozen VALU instructions) becomes one LDS read.  The table is folded at compile time
// (constant folding of `/` is correctly rounded).
struct RcpE4M3Table {
  float v[128];
  constexpr RcpE4M3Table() : v() {
    for (int c = 0; c < 128; ++c) {
      const int e = c >> 3, m = c & 7;
      float val = 0.0f;
      if (e == 0) {
        val = (float)m * 0.001953125f;  // m * 2^-9
      } else {
        val = 1.0f + (float)m * 0.125f;
        for (int i = 7; i < e; ++i) val *= 2.0f;
        for (int i = e; i < 7; ++i) val *= 0.5f;
      }
      v[c] = c == 0 ? 0.0f : (c == 127 ? __builtin_nanf("") : 1.0f / val);
    }
  }
};
static __constant__ RcpE4M3Table g_rcp_e4m3;  // one copy per translation unit

// Fills the block's LDS copy of the table (every thread must call it; ends with a barrier).
__device__ __forceinline__ void load_rcp_table(float *lut) {
  if (threadIdx.x < 128) lut[threadIdx.x] = g_rcp_e4m3.v[threadIdx.x];
  __syncthreads();
}

// Scale of one 16-block.  Returns the multiplier alpha * (1 / fp32(sf)) and the e4m3 code.
// With code 0 the table gives 0 (alpha is finite then: alpha = inf makes every code 0x7E/0x7F).
__device__ __forceinline__ float nvfp4_block_scale(float amax, float alpha, const float *lut, uint32_t &code) {
  float s32 = alpha * (amax * 0.16666666666666666f);
  code = f32_to_ue4m3_satfinite(s32);
  return alpha * lut[code];
}

__device__ __forceinline__ uint32_t nvfp4_pack8(uint4 v, float o) {
  float f[8] = {bf16_lo(v.x) * o, bf16_hi(v.x) * o, bf16_lo(v.y) * o, bf16_hi(v.y) * o,
                bf16_lo(v.z) * o, bf16_hi(v.z) * o, bf16_lo(v.w) * o, bf16_hi(v.w) * o};
  // A NaN multiplier (global scale 0: inf * 0) makes every product NaN; cvt.satfinite maps NaN
  // to +6 whatever its sign, the gfx950 converter keeps the sign, so this case is spelled out.
  return (o != o) ? 0x77777777u : f32x8_to_e2m1x8(f);
}

}  // namespace ac4k
