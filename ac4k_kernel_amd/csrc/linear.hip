// NVFP4 dot-scale linear for gfx950:  D = (A . B^T) * (gsA*gsB) + bias.
//
// Math contract of the reference kernel (lib/cuda/sm120/linear_nvfp4.cu:337-751, block-scaled
// MMA in lib/cuda/sm120/mma.cuh:13-56): every product e2m1*e2m1 is weighted by the two E4M3
// block scales of its 16-block, accumulated in fp32, then scaled by gsA*gsB, bias added,
// and rounded to the output type (:586-633).
//
// gfx950's scaled MFMA takes power-of-two scales per 32 elements, not E4M3 per 16, so the
// packed tiles are decoded on the fly: v_cvt_scalef32_pk_f16_fp4 expands two nibbles to two
// fp16 values and one v_pk_mul_f16 applies the E4M3 block scale.  e2m1 * e4m3 has at most
// 5 significant bits and lies in [2^-10, 2688], so the fp16 product is exact; the MFMA
// (v_mfma_f32_32x32x16_f16, same rate as bf16) accumulates in fp32.
#include <stdlib.h>
#include <string.h>

#include "ac4k_common.h"

namespace ac4k {

struct LinearArgs {
  void *D;
  const uint8_t *A, *B;
  const uint32_t *A_sf, *B_sf;  // one dword per (64-chunk, row): sf_u32[chunk * rows_padded + row]
  const float *A_gs, *B_gs;
  const void *bias;
  int64_t M, N, K, Mp, Np;
};

// --- output / bias element types -------------------------------------------
template <int DT>
struct Elem;
template <>
struct Elem<AC4K_DTYPE_BF16> {
  using T = uint16_t;
  static __device__ __forceinline__ float load(const void *p, int64_t i) {
    return bf16_bits_to_f32(static_cast<const uint16_t *>(p)[i]);
  }
  static __device__ __forceinline__ T cvt(float f) {  // round to nearest even, NaN kept quiet
    uint32_t u = __float_as_uint(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (T)((u >> 16) | 0x40u);
    return (T)((u + 0x7fffu + ((u >> 16) & 1u)) >> 16);
  }
};
template <>
struct Elem<AC4K_DTYPE_FP16> {
  using T = _Float16;
  static __device__ __forceinline__ float load(const void *p, int64_t i) {
    return (float)static_cast<const _Float16 *>(p)[i];
  }
  static __device__ __forceinline__ T cvt(float f) { return (_Float16)f; }
};
template <>
struct Elem<AC4K_DTYPE_FP32> {
  using T = float;
  static __device__ __forceinline__ float load(const void *p, int64_t i) {
    return static_cast<const float *>(p)[i];
  }
  static __device__ __forceinline__ T cvt(float f) { return f; }
};
constexpr int BIAS_NONE = 3;

// --- decode -------------------------------------------------------------------
// E4M3 scale byte -> fp16x2 pattern worth scale * 2^-8 in both halves (exponent bias 7 vs 15;
// E4M3 subnormals land on fp16 subnormals with the same ratio).  Bit 7 (sign) is dropped: the
// block scale is unsigned.
__device__ __forceinline__ f16x2 scale_pattern(uint32_t byte) {
  return __builtin_bit_cast(f16x2, (byte & 0x7fu) * 0x00800080u);
}

// eight nibbles of `w` times the block scale -> eight fp16 (exact); the converter multiplies
// by 2^8 to undo the 2^-8 carried by the scale pattern.
__device__ __forceinline__ void decode8(uint32_t w, f16x2 sp, f16x2 (&h)[4]) {
  h[0] = __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(w, 256.0f, 0) * sp;
  h[1] = __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(w, 256.0f, 1) * sp;
  h[2] = __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(w, 256.0f, 2) * sp;
  h[3] = __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(w, 256.0f, 3) * sp;
}

// ===========================================================================
// 128x128x64 tile kernel, 4 waves (2x2), each wave 64x64 = 2x2 MFMA 32x32x16 tiles.
// LDS holds the decoded fp16 tiles: row pitch 128 B (64 k), 16-byte chunk index XORed with
// (row & 7) so that both the decode stores and the MFMA fragment loads are conflict-free.
// ===========================================================================
constexpr int T_BM = 128, T_BN = 128, T_BK = 64;

struct PackedRegs {
  uint2 d[2];    // two 16-blocks (8 bytes each) of this thread's row
  uint32_t sf;   // scale bytes of the two blocks in bits 0..7 and 8..15
};

__device__ __forceinline__ PackedRegs load_packed(const uint8_t *base, const uint32_t *sf, int64_t rows,
                                                  int64_t rows_p, int64_t K, int64_t row, int64_t k0,
                                                  int half) {
  PackedRegs r;
  r.d[0] = r.d[1] = make_uint2(0, 0);
  r.sf = 0;
  if (row < rows_p) {
    uint32_t w = sf[(k0 >> 6) * rows_p + row] >> (16 * half);
    const uint8_t *p = base + row * (K >> 1) + (k0 >> 1) + half * 16;
#pragma unroll
    for (int b = 0; b < 2; ++b) {
      if (row < rows && k0 + half * 32 + b * 16 < K) {
        r.d[b] = *reinterpret_cast<const uint2 *>(p + b * 8);
        r.sf |= ((w >> (8 * b)) & 0xffu) << (8 * b);
      }
    }
  }
  return r;
}

__device__ __forceinline__ void decode_to_lds(_Float16 *tile, int row, int half, const PackedRegs &r) {
#pragma unroll
  for (int b = 0; b < 2; ++b) {
    f16x2 sp = scale_pattern(r.sf >> (8 * b));
    f16x2 lo[4], hi[4];
    decode8(r.d[b].x, sp, lo);
    decode8(r.d[b].y, sp, hi);
    const int c0 = half * 4 + b * 2;  // logical 16-byte chunk of elements [c0*8, c0*8+8)
    uint4 v0 = make_uint4(__builtin_bit_cast(uint32_t, lo[0]), __builtin_bit_cast(uint32_t, lo[1]),
                          __builtin_bit_cast(uint32_t, lo[2]), __builtin_bit_cast(uint32_t, lo[3]));
    uint4 v1 = make_uint4(__builtin_bit_cast(uint32_t, hi[0]), __builtin_bit_cast(uint32_t, hi[1]),
                          __builtin_bit_cast(uint32_t, hi[2]), __builtin_bit_cast(uint32_t, hi[3]));
    *reinterpret_cast<uint4 *>(tile + row * 64 + ((c0 ^ (row & 7)) << 3)) = v0;
    *reinterpret_cast<uint4 *>(tile + row * 64 + (((c0 + 1) ^ (row & 7)) << 3)) = v1;
  }
}

__device__ __forceinline__ f16x8 lds_frag(const _Float16 *tile, int row, int chunk) {
  return *reinterpret_cast<const f16x8 *>(tile + row * 64 + ((chunk ^ (row & 7)) << 3));
}

template <int D_DT, int BIAS_DT>
__global__ __launch_bounds__(256) void linear_nvfp4_tile128_kernel(LinearArgs a) {
  __shared__ __attribute__((aligned(16))) _Float16 sA[T_BM * T_BK];
  __shared__ __attribute__((aligned(16))) _Float16 sB[T_BN * T_BK];

  // Workgroups are dealt round-robin to the 8 XCDs; give each XCD a contiguous run of tiles so
  // its L2 sees neighbouring tiles, then walk tiles in groups of 8 tile-rows.
  const int64_t tiles_m = ceil_div(a.M, T_BM), tiles_n = ceil_div(a.N, T_BN);
  const int64_t ntiles = tiles_m * tiles_n;
  int64_t pid = blockIdx.x;
  {
    const int64_t per = ntiles / 8, rem = ntiles % 8;
    const int64_t xcd = pid % 8, idx = pid / 8;
    pid = xcd * per + (xcd < rem ? xcd : rem) + idx;
  }
  constexpr int GROUP_M = 8;
  const int64_t group = pid / (GROUP_M * tiles_n);
  const int64_t first_m = group * GROUP_M;
  const int64_t gsize = (tiles_m - first_m) < GROUP_M ? (tiles_m - first_m) : GROUP_M;
  const int64_t tm = first_m + (pid % (GROUP_M * tiles_n)) % gsize;
  const int64_t tn = (pid % (GROUP_M * tiles_n)) / gsize;

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  const int ld_row = tid >> 1, ld_half = tid & 1;
  const int64_t arow = tm * T_BM + ld_row, brow = tn * T_BN + ld_row;

  f32x16 acc[2][2];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.0f;

  const int64_t nk = ceil_div(a.K, T_BK);
  PackedRegs ra = load_packed(a.A, a.A_sf, a.M, a.Mp, a.K, arow, 0, ld_half);
  PackedRegs rb = load_packed(a.B, a.B_sf, a.N, a.Np, a.K, brow, 0, ld_half);
  for (int64_t kt = 0; kt < nk; ++kt) {
    decode_to_lds(sA, ld_row, ld_half, ra);
    decode_to_lds(sB, ld_row, ld_half, rb);
    __syncthreads();
    if (kt + 1 < nk) {  // prefetch the next packed slices while the MFMAs run
      ra = load_packed(a.A, a.A_sf, a.M, a.Mp, a.K, arow, (kt + 1) * T_BK, ld_half);
      rb = load_packed(a.B, a.B_sf, a.N, a.Np, a.K, brow, (kt + 1) * T_BK, ld_half);
    }
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) {
      const int chunk = ks * 2 + (lane >> 5);
      f16x8 fa[2], fb[2];
#pragma unroll
      for (int i = 0; i < 2; ++i) fa[i] = lds_frag(sA, wm * 64 + i * 32 + (lane & 31), chunk);
#pragma unroll
      for (int j = 0; j < 2; ++j) fb[j] = lds_frag(sB, wn * 64 + j * 32 + (lane & 31), chunk);
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(fa[i], fb[j], acc[i][j], 0, 0, 0);
    }
    __syncthreads();
  }

  // epilogue: * (gsA*gsB), + bias, round, store (linear_nvfp4.cu:586-633)
  const float scale = (*a.A_gs) * (*a.B_gs);
  using DE = Elem<D_DT>;
  typename DE::T *D = static_cast<typename DE::T *>(a.D);
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    const int64_t n = tn * T_BN + wn * 64 + j * 32 + (lane & 31);
    float bv = 0.0f;
    if constexpr (BIAS_DT != BIAS_NONE) {
      if (n < a.N) bv = Elem<BIAS_DT>::load(a.bias, n);
    }
#pragma unroll
    for (int i = 0; i < 2; ++i) {
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        const int64_t m = tm * T_BM + wm * 64 + i * 32 + (e >> 2) * 8 + (lane >> 5) * 4 + (e & 3);
        if (m < a.M && n < a.N) {
          float v = acc[i][j][e] * scale;
          if constexpr (BIAS_DT != BIAS_NONE) v += bv;
          D[m * a.N + n] = DE::cvt(v);
        }
      }
    }
  }
}

// ===========================================================================
// 256x256x64 tile kernel for large problems: 4 waves (2x2), each wave 128x128 = 4x4 MFMA
// 32x32x16 tiles (256 fp32 accumulators per lane).  A wave tile this large halves the LDS
// fragment traffic per flop against 64x64 wave tiles.  LDS is double buffered (2 x 64 KiB):
// while the MFMAs consume K-step kt from one buffer, the packed slice of step kt+1 (already
// in registers) is decoded into the other and the packed slice of step kt+2 is fetched.
// Thread t owns row t of the A tile and row t of the B tile: 32 packed bytes + one scale
// dword per K-step each.  Requires K % 64 == 0.
// ===========================================================================
constexpr int L_BM = 256, L_BN = 256, L_BK = 64;
constexpr int L_TILE_HALVES = L_BM * L_BK;  // fp16 elements per operand tile

struct PackedRow {
  uint4 lo, hi;  // 64 nibbles: four 16-blocks
  uint32_t sf;   // their four scale bytes
};

// `row` is clamped by the caller: rows past the matrix read the last valid row and feed
// accumulators whose outputs are never stored, so the load needs no predicate.
__device__ __forceinline__ PackedRow load_row(const uint8_t *base, const uint32_t *sf, int64_t rows_p,
                                              int64_t K, int64_t row, int64_t kt) {
  PackedRow r;
  const uint4 *p = reinterpret_cast<const uint4 *>(base + row * (K >> 1) + kt * 32);
  r.lo = p[0];
  r.hi = p[1];
  r.sf = sf[kt * rows_p + row];
  return r;
}

// decode 16-block `q` (0..3) of a packed row into its two 16-byte LDS chunks
__device__ __forceinline__ void decode_block_to_lds(_Float16 *tile, int row, int q, uint32_t w0, uint32_t w1,
                                                    uint32_t sfw) {
  f16x2 sp = scale_pattern(sfw >> (8 * q));
  f16x2 lo[4], hi[4];
  decode8(w0, sp, lo);
  decode8(w1, sp, hi);
  uint4 v0 = make_uint4(__builtin_bit_cast(uint32_t, lo[0]), __builtin_bit_cast(uint32_t, lo[1]),
                        __builtin_bit_cast(uint32_t, lo[2]), __builtin_bit_cast(uint32_t, lo[3]));
  uint4 v1 = make_uint4(__builtin_bit_cast(uint32_t, hi[0]), __builtin_bit_cast(uint32_t, hi[1]),
                        __builtin_bit_cast(uint32_t, hi[2]), __builtin_bit_cast(uint32_t, hi[3]));
  *reinterpret_cast<uint4 *>(tile + row * 64 + (((2 * q) ^ (row & 7)) << 3)) = v0;
  *reinterpret_cast<uint4 *>(tile + row * 64 + (((2 * q + 1) ^ (row & 7)) << 3)) = v1;
}

__device__ __forceinline__ void decode_row_quarter(_Float16 *tile, int row, int q, const PackedRow &r) {
#ifdef EXP_NO_DECODE
  return;
#endif
  const uint32_t w[8] = {r.lo.x, r.lo.y, r.lo.z, r.lo.w, r.hi.x, r.hi.y, r.hi.z, r.hi.w};
  decode_block_to_lds(tile, row, q, w[2 * q], w[2 * q + 1], r.sf);
}

struct Frags {
  f16x8 a[4], b[4];
};

__device__ __forceinline__ void load_frags(Frags &f, const _Float16 *cA, const _Float16 *cB, int arow, int brow,
                                           int chunk) {
#ifdef EXP_NO_LDSREAD
  if (chunk >= 0) return;
#endif
#pragma unroll
  for (int i = 0; i < 4; ++i) f.a[i] = lds_frag(cA, arow + i * 32, chunk);
#pragma unroll
  for (int j = 0; j < 4; ++j) f.b[j] = lds_frag(cB, brow + j * 32, chunk);
}

template <int D_DT, int BIAS_DT>
__global__ __launch_bounds__(256, 1) void linear_nvfp4_tile256_kernel(LinearArgs a) {
  extern __shared__ __attribute__((aligned(16))) _Float16 lds[];  // [2 buffers][A tile | B tile]

  const int64_t tiles_m = ceil_div(a.M, L_BM), tiles_n = ceil_div(a.N, L_BN);
  const int64_t ntiles = tiles_m * tiles_n;
  int64_t pid = blockIdx.x;
  {  // contiguous run of tiles per XCD (workgroups are dealt round-robin to the 8 XCDs)
    const int64_t per = ntiles / 8, rem = ntiles % 8;
    const int64_t xcd = pid % 8, idx = pid / 8;
    pid = xcd * per + (xcd < rem ? xcd : rem) + idx;
  }
  constexpr int GROUP_M = 4;
  const int64_t group = pid / (GROUP_M * tiles_n);
  const int64_t first_m = group * GROUP_M;
  const int64_t gsize = (tiles_m - first_m) < GROUP_M ? (tiles_m - first_m) : GROUP_M;
  const int64_t tm = first_m + (pid % (GROUP_M * tiles_n)) % gsize;
  const int64_t tn = (pid % (GROUP_M * tiles_n)) / gsize;

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  int64_t arow = tm * L_BM + tid, brow = tn * L_BN + tid;
  arow = arow < a.M ? arow : a.M - 1;
  brow = brow < a.N ? brow : a.N - 1;
  const int nk = (int)(a.K / L_BK);
  const int fa_row = wm * 128 + (lane & 31), fb_row = wn * 128 + (lane & 31), half = lane >> 5;

  f32x16 acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.0f;

  // Software pipeline.  Step kt multiplies LDS buffer kt&1 while it decodes the packed slice of
  // step kt+1 (held in registers since the previous step) into the other buffer; the packed
  // slices of steps kt+2 / kt+3 are in flight in the second register set.  The decode is done
  // in sub-steps 0..2, the workgroup barrier sits before sub-step 3, and sub-step 3's MFMAs
  // cover the barrier skew, the first fragment loads of step kt+1 and the next global loads.
  PackedRow ra0 = load_row(a.A, a.A_sf, a.Mp, a.K, arow, 0);
  PackedRow rb0 = load_row(a.B, a.B_sf, a.Np, a.K, brow, 0);
#pragma unroll
  for (int q = 0; q < 4; ++q) {
    decode_row_quarter(lds, tid, q, ra0);
    decode_row_quarter(lds + L_TILE_HALVES, tid, q, rb0);
  }
  const int klast = nk - 1;
  ra0 = load_row(a.A, a.A_sf, a.Mp, a.K, arow, 1 < klast ? 1 : klast);
  rb0 = load_row(a.B, a.B_sf, a.Np, a.K, brow, 1 < klast ? 1 : klast);
  PackedRow ra1 = load_row(a.A, a.A_sf, a.Mp, a.K, arow, 2 < klast ? 2 : klast);
  PackedRow rb1 = load_row(a.B, a.B_sf, a.Np, a.K, brow, 2 < klast ? 2 : klast);
  __syncthreads();

  Frags f[2];
  load_frags(f[0], lds, lds + L_TILE_HALVES, fa_row, fb_row, half);

  auto mfma16 = [&](const Frags &c) {
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j)
        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(c.a[i], c.b[j], acc[i][j], 0, 0, 0);
  };
  // one K-step; da/db hold the packed slice of step kt+1 and are refilled with step kt+3
  auto kstep = [&](int kt, PackedRow &da, PackedRow &db) {
    const _Float16 *cA = lds + (kt & 1) * (2 * L_TILE_HALVES);
    const _Float16 *cB = cA + L_TILE_HALVES;
    _Float16 *nA = lds + ((kt + 1) & 1) * (2 * L_TILE_HALVES);
    _Float16 *nB = nA + L_TILE_HALVES;
    // sub-step 0
    load_frags(f[1], cA, cB, fa_row, fb_row, 2 + half);
    decode_row_quarter(nA, tid, 0, da);
    decode_row_quarter(nA, tid, 1, da);
    decode_row_quarter(nA, tid, 2, da);
    mfma16(f[0]);
#pragma unroll
    for (int g = 0; g < 16; ++g) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x002, 4, 0);
      if (g < 8) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
      if (g >= 10) __builtin_amdgcn_sched_group_barrier(0x200, 1, 0);
    }
    __builtin_amdgcn_sched_barrier(0);
    // sub-step 1
    load_frags(f[0], cA, cB, fa_row, fb_row, 4 + half);
    decode_row_quarter(nA, tid, 3, da);
    decode_row_quarter(nB, tid, 0, db);
    decode_row_quarter(nB, tid, 1, db);
    mfma16(f[1]);
#pragma unroll
    for (int g = 0; g < 16; ++g) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x002, 4, 0);
      if (g < 8) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
      if (g >= 10) __builtin_amdgcn_sched_group_barrier(0x200, 1, 0);
    }
    __builtin_amdgcn_sched_barrier(0);
    // sub-step 2
    load_frags(f[1], cA, cB, fa_row, fb_row, 6 + half);
    decode_row_quarter(nB, tid, 2, db);
    decode_row_quarter(nB, tid, 3, db);
    mfma16(f[0]);
#pragma unroll
    for (int g = 0; g < 16; ++g) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x002, 3, 0);
      if (g < 8) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
      if (g >= 12) __builtin_amdgcn_sched_group_barrier(0x200, 1, 0);
    }
    __builtin_amdgcn_sched_barrier(0);
    __syncthreads();  // buffer (kt+1)&1 is complete, buffer kt&1 has been read by everyone
    // sub-step 3
    load_frags(f[0], nA, nB, fa_row, fb_row, half);
    const int kn = kt + 3 < klast ? kt + 3 : klast;
    da = load_row(a.A, a.A_sf, a.Mp, a.K, arow, kn);
    db = load_row(a.B, a.B_sf, a.Np, a.K, brow, kn);
    mfma16(f[1]);
#pragma unroll
    for (int g = 0; g < 16; ++g) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x002, 2, 0);
      if (g < 8) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
      if (g >= 8 && g < 14) __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);
    }
    __builtin_amdgcn_sched_barrier(0);
  };
  for (int kt = 0; kt < nk; ++kt) {
    PackedRow na = ra1, nb = rb1;
    kstep(kt, ra0, rb0);   // consumes ra0/rb0 (step kt+1), refills them with step kt+3
    ra1 = ra0; rb1 = rb0;  // rotate: next step decodes the old ra1/rb1 (step kt+2)
    ra0 = na; rb0 = nb;
  }

  const float scale = (*a.A_gs) * (*a.B_gs);
  using DE = Elem<D_DT>;
  typename DE::T *D = static_cast<typename DE::T *>(a.D);
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int64_t n = tn * L_BN + wn * 128 + j * 32 + (lane & 31);
    float bv = 0.0f;
    if constexpr (BIAS_DT != BIAS_NONE) {
      if (n < a.N) bv = Elem<BIAS_DT>::load(a.bias, n);
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        const int64_t m = tm * L_BM + wm * 128 + i * 32 + (e >> 2) * 8 + (lane >> 5) * 4 + (e & 3);
        if (m < a.M && n < a.N) {
          float v = acc[i][j][e] * scale;
          if constexpr (BIAS_DT != BIAS_NONE) v += bv;
          D[m * a.N + n] = DE::cvt(v);
        }
      }
    }
  }
}

constexpr int L_LDS_BYTES = 2 * 2 * L_TILE_HALVES * (int)sizeof(_Float16);  // 128 KiB

enum class LinearKernel { AUTO, TILE128, TILE256 };

static LinearKernel forced_kernel() {  // benchmarking aid: AC4K_LINEAR_KERNEL=tile128|tile256
  static const LinearKernel k = [] {
    const char *e = getenv("AC4K_LINEAR_KERNEL");
    if (e && !strcmp(e, "tile128")) return LinearKernel::TILE128;
    if (e && !strcmp(e, "tile256")) return LinearKernel::TILE256;
    return LinearKernel::AUTO;
  }();
  return k;
}

template <int D_DT, int BIAS_DT>
static int launch_tile256(const LinearArgs &a, hipStream_t st) {
  auto *kern = linear_nvfp4_tile256_kernel<D_DT, BIAS_DT>;
  static bool attr_set = false;  // per instantiation; the attribute is idempotent
  if (!attr_set) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kern),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, L_LDS_BYTES);
    if (e != hipSuccess) return set_error("hipFuncSetAttribute(LDS=%d): %s", L_LDS_BYTES, hipGetErrorString(e));
    attr_set = true;
  }
  const int64_t ntiles = ceil_div(a.M, L_BM) * ceil_div(a.N, L_BN);
  hipLaunchKernelGGL(kern, dim3((unsigned)ntiles), dim3(256), L_LDS_BYTES, st, a);
  return 0;
}

template <int D_DT, int BIAS_DT>
static int launch_linear(const LinearArgs &a, hipStream_t st) {
  LinearKernel k = forced_kernel();
  const bool big_ok = a.K % L_BK == 0 && (((uintptr_t)a.A | (uintptr_t)a.B) & 15) == 0;
  if (k == LinearKernel::AUTO) k = (big_ok && a.M > 128 && a.N > 128) ? LinearKernel::TILE256 : LinearKernel::TILE128;
  if (k == LinearKernel::TILE256 && big_ok) return launch_tile256<D_DT, BIAS_DT>(a, st);
  const int64_t ntiles = ceil_div(a.M, T_BM) * ceil_div(a.N, T_BN);
  hipLaunchKernelGGL((linear_nvfp4_tile128_kernel<D_DT, BIAS_DT>), dim3((unsigned)ntiles), dim3(256), 0, st, a);
  return 0;
}

template <int D_DT>
static int dispatch_bias(const LinearArgs &a, int bias_dtype, hipStream_t st) {
  if (!a.bias) return launch_linear<D_DT, BIAS_NONE>(a, st);
  switch (bias_dtype) {
    case AC4K_DTYPE_BF16: return launch_linear<D_DT, AC4K_DTYPE_BF16>(a, st);
    case AC4K_DTYPE_FP16: return launch_linear<D_DT, AC4K_DTYPE_FP16>(a, st);
    case AC4K_DTYPE_FP32: return launch_linear<D_DT, AC4K_DTYPE_FP32>(a, st);
  }
  return set_error("bias must be bfloat16, half or float (dtype tag %d)", bias_dtype);
}

}  // namespace ac4k

using namespace ac4k;

extern "C" __attribute__((visibility("default"))) int ac4k_linear_nvfp4(void *D, int d_dtype, const void *A, const void *A_sf, const float *A_gs,
                                 const void *B, const void *B_sf, const float *B_gs, const void *bias,
                                 int bias_dtype, int64_t M, int64_t N, int64_t K, ac4k_stream_t stream) {
  AC4K_REQUIRE(D && A && A_sf && A_gs && B && B_sf && B_gs, "null pointer argument");
  AC4K_REQUIRE(M >= 1 && N >= 1 && K >= 1, "M, N, K must be positive (M=%lld N=%lld K=%lld)", (long long)M,
               (long long)N, (long long)K);
  AC4K_REQUIRE(K % 16 == 0, "A size(1)*2 must be multiple of 16 but see %lld", (long long)K);
  AC4K_REQUIRE(((uintptr_t)A & 7) == 0 && ((uintptr_t)B & 7) == 0 && ((uintptr_t)A_sf & 3) == 0 &&
                   ((uintptr_t)B_sf & 3) == 0,
               "A/B must be 8-byte aligned and the scale tensors 4-byte aligned");
  AC4K_REQUIRE(ceil_div(M, T_BM) * ceil_div(N, T_BN) < (1ll << 31), "problem too large");
  LinearArgs a{D,
               static_cast<const uint8_t *>(A),
               static_cast<const uint8_t *>(B),
               static_cast<const uint32_t *>(A_sf),
               static_cast<const uint32_t *>(B_sf),
               A_gs,
               B_gs,
               bias,
               M,
               N,
               K,
               align_up(M, 16),
               align_up(N, 16)};
  hipStream_t st = (hipStream_t)stream;
  int rc;
  switch (d_dtype) {
    case AC4K_DTYPE_BF16: rc = dispatch_bias<AC4K_DTYPE_BF16>(a, bias_dtype, st); break;
    case AC4K_DTYPE_FP16: rc = dispatch_bias<AC4K_DTYPE_FP16>(a, bias_dtype, st); break;
    case AC4K_DTYPE_FP32: rc = dispatch_bias<AC4K_DTYPE_FP32>(a, bias_dtype, st); break;
    default: return set_error("d must be bfloat16, half or float (dtype tag %d)", d_dtype);
  }
  if (rc) return rc;
  return check_launch("ac4k_linear_nvfp4");
}

extern "C" __attribute__((visibility("default"))) int ac4k_linear_nvfp4_fused_bf16(void *D, int d_dtype, const void *X, void *X_q, void *X_sf,
                                            float *X_gs, const void *B, const void *B_sf, const float *B_gs,
                                            const void *bias, int bias_dtype, int64_t M, int64_t N, int64_t K,
                                            ac4k_stream_t stream) {
  AC4K_REQUIRE(X && X_q && X_sf && X_gs, "null pointer argument");
  AC4K_REQUIRE(K % 64 == 0, "K must be a multiple of 64 (got %lld)", (long long)K);
  AC4K_REQUIRE(M >= 1 && M <= 32, "the fused skinny linear takes 1 <= M <= 32 (got %lld)", (long long)M);
  if (int rc = ac4k_global_scale_bf16(X_gs, X, M * K, 2688.0f, stream)) return rc;
  if (int rc = ac4k_quantize_nvfp4(X_q, X_sf, X, X_gs, 1, 1, M, K, 0, 0, K, 1, 0, stream)) return rc;
  return ac4k_linear_nvfp4(D, d_dtype, X_q, X_sf, X_gs, B, B_sf, B_gs, bias, bias_dtype, M, N, K, stream);
}
