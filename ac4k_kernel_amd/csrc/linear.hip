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
// 6 significant bits and lies in [2^-10, 2688], so the fp16 product is exact; the MFMA
// (v_mfma_f32_32x32x16_f16, same rate as bf16) accumulates in fp32.
#include <stdlib.h>
#include <string.h>

#include <atomic>
#include <mutex>
#include <type_traits>

#include "ac4k_common.h"

namespace ac4k {

struct LinearArgs {
  void *D;
  const uint8_t *A, *B;
  const uint32_t *A_sf, *B_sf;  // one dword per (64-chunk, row): sf_u32[chunk * rows_padded + row]
  const float *A_gs, *B_gs;
  const void *bias;
  int64_t M, N, K, Mp, Np;
  int prepacked = 0;  // B points at a weight image (W_BLOCK_BYTES blocks, see below) and B_sf is unused
};

// --- pre-packed weight image -----------------------------------------------------
// Static weights can be re-laid once into the order the kernels fetch them: one block per
// (128 rows, 128 k), blocks of a 128-row band consecutive along k, bands consecutive along n (N is
// padded with zero rows to a whole band).  A block is the LDS stage picture of those rows: 128 rows x
// 64 packed bytes with the 16-byte piece p of row r at position p ^ ((r >> 1) & 3), followed by the
// scale dwords [2 chunks][128 rows].  Every LDS-DMA transfer of a stage then reads one contiguous
// kilobyte, and a stage of the decode-sized kernel (256 k) is one contiguous run of two blocks.
constexpr int W_BLOCK_ROWS = 128, W_BLOCK_K = 128;
constexpr int W_BLOCK_DATA = W_BLOCK_ROWS * W_BLOCK_K / 2;            // 8192
constexpr int W_BLOCK_BYTES = W_BLOCK_DATA + 2 * W_BLOCK_ROWS * 4;    // 9216

// --- output / bias element types -------------------------------------------
template <int DT>
struct Elem;
template <>
struct Elem<AC4K_DTYPE_BF16> {
  using T = uint16_t;
  static __device__ __forceinline__ float load(const void *p, int64_t i) {
    return bf16_bits_to_f32(static_cast<const uint16_t *>(p)[i]);
  }
  // round to nearest even, NaN stays NaN: v_cvt_pk_bf16_f32
  static __device__ __forceinline__ T cvt(float f) { return __builtin_bit_cast(uint16_t, (__bf16)f); }
  static __device__ __forceinline__ uint32_t cvt2(float lo, float hi) {
    typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
    const f32x2 v = {lo, hi};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2_t));
  }
};
template <>
struct Elem<AC4K_DTYPE_FP16> {
  using T = _Float16;
  static __device__ __forceinline__ float load(const void *p, int64_t i) {
    return (float)static_cast<const _Float16 *>(p)[i];
  }
  static __device__ __forceinline__ T cvt(float f) { return (_Float16)f; }
  static __device__ __forceinline__ uint32_t cvt2(float lo, float hi) {
    const f16x2 v = {(_Float16)lo, (_Float16)hi};
    return __builtin_bit_cast(uint32_t, v);
  }
};
template <>
struct Elem<AC4K_DTYPE_FP32> {
  using T = float;
  static __device__ __forceinline__ float load(const void *p, int64_t i) {
    return static_cast<const float *>(p)[i];
  }
  static __device__ __forceinline__ T cvt(float f) { return f; }
  static __device__ __forceinline__ uint32_t cvt2(float lo, float) { return __float_as_uint(lo); }  // unused: 4-byte outputs are not packed
};
constexpr int BIAS_NONE = 3;

// --- decode -------------------------------------------------------------------
// E4M3 scale byte -> fp16x2 pattern worth scale * 2^-8 in both halves (exponent bias 7 vs 15;
// E4M3 subnormals land on fp16 subnormals with the same ratio).  The scale bytes are read as
// the signed float8_e4m3fn their tensor type says, by every linear kernel (the quantizers only
// produce non-negative scales).
__device__ __forceinline__ f16x2 scale_pattern(uint32_t byte) {
  return __builtin_bit_cast(f16x2, (byte & 0x7fu) * 0x00800080u + (byte & 0x80u) * 0x01000100u);
}

// eight nibbles of `w` times the block scale -> eight fp16 (exact); the converter multiplies
// by 2^8 to undo the 2^-8 carried by the scale pattern.
__device__ __forceinline__ void decode8(uint32_t w, f16x2 sp, f16x2 (&h)[4]) {
  h[0] = __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(w, 256.0f, 0) * sp;
  h[1] = __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(w, 256.0f, 1) * sp;
  h[2] = __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(w, 256.0f, 2) * sp;
  h[3] = __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(w, 256.0f, 3) * sp;
}

// --- workgroup -> output tile ---------------------------------------------------
// Workgroups are dealt round-robin to the 8 XCDs, each with its own L2.  Workgroup `pid` is first
// renumbered so that every XCD owns one contiguous run of the tile sequence, and the sequence walks
// the tiles in bands of GROUP_M tile-rows, column by column inside a band: the workgroups resident
// on one XCD at a time then cover a compact GROUP_M x (CUs / GROUP_M) patch and share its operand
// panels through that L2.
struct TileCoord {
  int64_t m, n;
};
template <int GROUP_M>
__device__ __forceinline__ TileCoord tile_of_workgroup(int64_t pid, int64_t tiles_m, int64_t tiles_n) {
  const int64_t ntiles = tiles_m * tiles_n;
  const int64_t per = ntiles / 8, rem = ntiles % 8;
  const int64_t xcd = pid % 8, idx = pid / 8;
  pid = xcd * per + (xcd < rem ? xcd : rem) + idx;
  const int64_t band = pid / (GROUP_M * tiles_n), in_band = pid % (GROUP_M * tiles_n);
  const int64_t first_m = band * GROUP_M;
  const int64_t rows = (tiles_m - first_m) < GROUP_M ? (tiles_m - first_m) : GROUP_M;
  return {first_m + in_band % rows, in_band / rows};
}

// ===========================================================================
// 128x128x64 tile kernel, 4 waves (2x2), each wave 64x64 = 2x2 MFMA 32x32x16 tiles.
// LDS holds the decoded fp16 tiles: row pitch 128 B (64 k), 16-byte chunk index XORed with
// LDS_SWZ(row) so that both the decode stores and the MFMA fragment loads are conflict-free.
// ===========================================================================
constexpr int T_BM = 128, T_BN = 128, T_BK = 64;
#define LDS_SWZ(row) ((row) & 7)

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
    *reinterpret_cast<uint4 *>(tile + row * 64 + ((c0 ^ LDS_SWZ(row)) << 3)) = v0;
    *reinterpret_cast<uint4 *>(tile + row * 64 + (((c0 + 1) ^ LDS_SWZ(row)) << 3)) = v1;
  }
}

__device__ __forceinline__ f16x8 lds_frag(const _Float16 *tile, int row, int chunk) {
  return *reinterpret_cast<const f16x8 *>(tile + row * 64 + ((chunk ^ LDS_SWZ(row)) << 3));
}

template <int D_DT, int BIAS_DT>
__global__ __launch_bounds__(256) void linear_nvfp4_tile128_kernel(LinearArgs a) {
  __shared__ __attribute__((aligned(16))) _Float16 sA[T_BM * T_BK];
  __shared__ __attribute__((aligned(16))) _Float16 sB[T_BN * T_BK];

  const TileCoord tc = tile_of_workgroup<8>(blockIdx.x, ceil_div(a.M, T_BM), ceil_div(a.N, T_BN));
  const int64_t tm = tc.m, tn = tc.n;

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
// (64 MI) x (64 NJ) tile, packed operands in LDS, decode after the fragment load.
//
// The packed A/B slices and their scale dwords go from global memory straight into LDS with
// LDS-DMA loads (global_load_lds: no VGPR staging, no LDS store instruction), PS stages of
// 128 k each.  A wave (4 waves, 2x2, (32 MI) x (32 NJ) each) reads for every 32-row fragment ONE
// 16-byte word per lane per 64-chunk: lane (row r, half h) owns elements [32h, 32h+32) of the
// chunk; dword s of that word feeds MFMA sub-step s.  The same k-slot assignment is used for A
// and B, so the permutation of k inside a chunk cancels in the dot product.  Decode per dword:
// 4 x v_cvt_scalef32_pk_f16_fp4 + 4 x v_pk_mul_f16 by the block scale (E4M3 -> fp16 with
// v_cvt_scalef32_pk_f16_fp8, splat through op_sel); the decode of a sub-step is interleaved with
// the MFMAs of the previous one.  A single wave per SIMD is bound by instruction issue: the
// 4 decode instructions per MFMA of the 256x256 tile stretch a 32-cycle MFMA slot to about 38
// cycles, the smaller tiles (more decode per MFMA) are decode-bound outright; that, not LDS or
// HBM, bounds the loop.  There is one workgroup barrier per 128 k, placed in the middle of the
// step so that the next stage is readable before the current one ends.
// Split-K: blockIdx.y selects a contiguous range of stages; with more than one range the
// accumulators go to an fp32 partial buffer and a second kernel adds the ranges.
// Requires K % 128 == 0 and 16-byte aligned operands.
// ===========================================================================
constexpr int P_BK = 128;     // k per stage (two 64-chunks)
constexpr int P_ROW = 64;     // packed bytes per row per stage: [chunk][half] x 16 B

template <int BM, int BN, int PS>
struct PLayout {               // byte offsets inside one LDS stage; PS stages
  static constexpr int OFF_B = BM * P_ROW;                 // B rows follow the A rows
  static constexpr int OFF_SFA = OFF_B + BN * P_ROW;       // scale dwords: [chunk][BM rows]
  static constexpr int OFF_SFB = OFF_SFA + 2 * BM * 4;     // [chunk][BN rows]
  static constexpr int STAGE_BYTES = OFF_SFB + 2 * BN * 4;
  static constexpr int LDS_BYTES = PS * STAGE_BYTES;
  static_assert(LDS_BYTES <= 160 * 1024, "stages must fit in the CU's LDS");
};

template <int N>
__device__ __forceinline__ void wait_vmcnt() {
  asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}

// Pins a wave-uniform pointer to scalar registers (the halves are taken as unsigned: readfirstlane
// returns a signed int, and a sign-extended low half would corrupt the high one).
__device__ __forceinline__ const uint8_t *uniform_ptr(const void *p) {
  const uint64_t v = (uint64_t)p;
  const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)v), hi = __builtin_amdgcn_readfirstlane((uint32_t)(v >> 32));
  return reinterpret_cast<const uint8_t *>(((uint64_t)hi << 32) | lo);
}

// LDS-DMA: global_load_lds with a scalar 64-bit base, a 32-bit lane offset and the LDS
// destination of lane 0 in M0 (lane l lands at M0 + size * l).  Issued through inline asm so
// that the compiler's wait-count insertion does not see these loads: with the builtin it puts
// s_waitcnt vmcnt(0) in front of every later LDS read, which serialises the prefetch.  The
// kernel waits with explicit s_waitcnt vmcnt(..) before the barrier that publishes a stage.
__device__ __forceinline__ void dma16(const void *sbase, uint32_t voff, uint32_t lds_stage, uint32_t lds_piece) {
  // (wave-uniform by construction; the read keeps them in scalar registers when the compiler cannot tell)
  lds_stage = (uint32_t)__builtin_amdgcn_readfirstlane((int)lds_stage);
  lds_piece = (uint32_t)__builtin_amdgcn_readfirstlane((int)lds_piece);
  sbase = uniform_ptr(sbase);
  asm volatile("s_add_u32 m0, %0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %2, %3"
               :: "s"(lds_stage), "s"(lds_piece), "v"(voff), "s"(sbase) : "memory", "scc");
}
__device__ __forceinline__ void dma4(const void *sbase, uint32_t voff, uint32_t lds_stage, uint32_t lds_piece) {
  lds_stage = (uint32_t)__builtin_amdgcn_readfirstlane((int)lds_stage);
  lds_piece = (uint32_t)__builtin_amdgcn_readfirstlane((int)lds_piece);
  sbase = uniform_ptr(sbase);
  asm volatile("s_add_u32 m0, %0, %1\n\ts_nop 0\n\tglobal_load_lds_dword %2, %3"
               :: "s"(lds_stage), "s"(lds_piece), "v"(voff), "s"(sbase) : "memory", "scc");
}

template <int MI, int NJ>
struct DecFrags {
  f16x8 a[MI], b[NJ];
};

// dword `w` (8 nibbles) times block scale `sc` (both halves of `sc2` hold candidates, HI picks)
template <bool HI>
__device__ __forceinline__ f16x8 decode_dword(uint32_t w, f16x2 sc2) {
  const f16x2 sc = HI ? (f16x2){sc2.y, sc2.y} : (f16x2){sc2.x, sc2.x};
  f16x2 d0 = __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(w, 1.0f, 0) * sc;
  f16x2 d1 = __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(w, 1.0f, 1) * sc;
  f16x2 d2 = __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(w, 1.0f, 2) * sc;
  f16x2 d3 = __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(w, 1.0f, 3) * sc;
  return (f16x8){d0.x, d0.y, d1.x, d1.y, d2.x, d2.y, d3.x, d3.y};
}

template <int S>
__device__ __forceinline__ uint32_t dword_of(const uint4 &v) {
  return S == 0 ? v.x : S == 1 ? v.y : S == 2 ? v.z : v.w;
}

// Build with -DAC4K_LINEAR_TIMELINE (`build.py --timeline`) to record per workgroup the 100 MHz clock at
// kernel entry, loop entry, loop exit and kernel exit plus the shader cycles spent in the loop of the
// tile kernel and of the K-split-waves kernel; ac4k_debug_linear_timeline copies the stamps out
// (a profiling aid; not compiled into the library).
#ifdef AC4K_LINEAR_TIMELINE
__device__ uint64_t g_linear_timeline[8192][6];
#define AC4K_LTL(i, v)                                                     \
  do {                                                                     \
    if (threadIdx.x == 0 && blockIdx.x + gridDim.x * blockIdx.y < 8192)      \
      g_linear_timeline[blockIdx.x + gridDim.x * blockIdx.y][i] = (v);        \
  } while (0)
#else
#define AC4K_LTL(i, v)
#endif

struct SplitK {
  float *partial;  // [splits][M][N] fp32, or null: convert and store to D
  int splits;
};

// Epilogue of the packed-LDS tile kernel: the accumulators of one wave, (32*MI) x (32*NJ) outputs, to
// `out` (row stride N).  acc[i][j] holds the TRANSPOSED 32x32 block (the MFMAs are issued with the
// operands swapped): lane l, element e <-> n = j*32 + (e>>2)*8 + (l>>5)*4 + (e&3), m = i*32 + (l&31),
// i.e. four consecutive n per lane.  RAW stores the fp32 sums as they are (split-K partials);
// otherwise out = cvt(acc * scale + bias).  Outputs are staged through LDS (`lds`, free at this
// point), one wave-private block of RP rows at a time, so that every lane stores 16 bytes and a
// wave store covers whole row segments; the bias of the tile's columns sits behind the staging
// blocks as fp32.  Callers have passed a workgroup barrier after their last read of `lds`.
template <int OUT_DT, int BIAS_DT, bool RAW, int MI, int NJ, int LDS_BYTES>
__device__ __forceinline__ void store_tile(const f32x16 (&acc)[MI][NJ], char *lds, void *out, const void *bias,
                                           float scale, int64_t M, int64_t N, int64_t m0, int64_t n0,
                                           int64_t tile_n0) {
  using DE = Elem<OUT_DT>;
  using DT = typename DE::T;
  DT *Dp = static_cast<DT *>(out);
  constexpr int S = sizeof(DT);
  constexpr int WN = 32 * NJ;               // columns per wave
  constexpr int RP = S == 2 ? 64 : 32;      // rows per staging pass
  constexpr int PITCH = WN * S + 16;        // bytes per staged row, 16 bytes of padding
  constexpr int STG_BYTES = 4 * RP * PITCH;
  static_assert(STG_BYTES + 2 * WN * 4 <= LDS_BYTES, "epilogue staging and bias must fit in LDS");
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, half = lane >> 5, wn = wave & 1;
  const float *bias_s = reinterpret_cast<const float *>(lds + STG_BYTES) + wn * WN + half * 4;
  if constexpr (BIAS_DT != BIAS_NONE) {
    if (tid < 2 * WN) {
      const int64_t n = tile_n0 + tid;
      reinterpret_cast<float *>(lds + STG_BYTES)[tid] = n < N ? Elem<BIAS_DT>::load(bias, n) : 0.0f;
    }
    __syncthreads();
  }
  // the four outputs acc[i][j][4g .. 4g+3] of a lane, scaled, plus their bias b
  // The 256x256 tile keeps its 256 sums per lane in accumulation registers.  Left alone, the compiler
  // moves all of them to ordinary registers at the top of the epilogue and spills what does not fit;
  // reading them with a volatile move keeps each read inside the pass that stages the value.
  auto sum_of = [&](int i, int j, int e) {
    if constexpr (MI * NJ == 16) {
      float v;
      asm volatile("v_accvgpr_read_b32 %0, %1" : "=v"(v) : "a"(acc[i][j][e]));
      return v;
    } else {
      return acc[i][j][e];
    }
  };
  auto value4 = [&](int i, int j, int g, const float4 &b) {
    float4 v = make_float4(sum_of(i, j, 4 * g), sum_of(i, j, 4 * g + 1), sum_of(i, j, 4 * g + 2), sum_of(i, j, 4 * g + 3));
    if constexpr (!RAW) {
      v.x *= scale; v.y *= scale; v.z *= scale; v.w *= scale;
    }
    if constexpr (BIAS_DT != BIAS_NONE) {
      v.x += b.x; v.y += b.y; v.z += b.z; v.w += b.w;
    }
    return v;
  };
  // bias of column block j: four 16-byte LDS reads in one go (one wait), kept for the rows of a pass
  auto bias_of = [&](int j, float4 (&b)[4]) {
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      b[g] = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
      if constexpr (BIAS_DT != BIAS_NONE) b[g] = *reinterpret_cast<const float4 *>(bias_s + j * 32 + g * 8);
    }
  };
  // 16-byte stores need rows that start on 16-byte boundaries; other shapes leave the staging block
  // element by element (a rolled loop over LDS, so that this rare path costs no registers)
  const bool vec_ok = (N % (16 / S) == 0) && ((uintptr_t)out % 16 == 0);
  char *stg = lds + wave * (RP * PITCH);
  constexpr int CPR = WN * S / 16;   // 16-byte pieces per staged row
  constexpr int RS = 64 / CPR;       // rows covered by one wave store
  const int lrow = lane / CPR, lq = lane % CPR;
  const int64_t row_bytes = N * S;
  const uint32_t lane_off = (uint32_t)(lrow * row_bytes) + lq * 16;
  char *out0 = reinterpret_cast<char *>(Dp) + (m0 * N + n0) * S;  // wave-uniform
  const bool interior = vec_ok && m0 + 32 * MI <= M && n0 + WN <= N;
  const int64_t cl = N - n0 - lq * (16 / S);
  const int cols_left = cl > 16 / S ? 16 / S : (int)cl;  // columns of this lane's piece inside the matrix
  const int64_t rl = M - m0 - lrow;
  const int rows_left = rl > 32 * MI ? 32 * MI : (int)rl;  // rows of the block below this lane's first one
#pragma unroll
  for (int p = 0; p < 32 * MI / RP; ++p) {
    asm volatile("" ::: "memory");  // keeps the bias reads of one pass from being merged with the next one's
#pragma unroll
    for (int j = 0; j < NJ; ++j) {
      float4 b[4];
      bias_of(j, b);
#pragma unroll
      for (int ii = 0; ii < RP / 32; ++ii) {
        const int i = p * (RP / 32) + ii;
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          const float4 v = value4(i, j, g, b[g]);
          char *dst = stg + (ii * 32 + (lane & 31)) * PITCH + (j * 32 + g * 8 + half * 4) * S;
          if constexpr (S == 2) *reinterpret_cast<uint2 *>(dst) = make_uint2(DE::cvt2(v.x, v.y), DE::cvt2(v.z, v.w));
          else *reinterpret_cast<float4 *>(dst) = v;
        }
      }
    }
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // the staging block is private to the wave
    // pass `it` stores rows it*RS .. it*RS+RS-1 of the block: a wave-uniform base that advances by
    // RS rows, plus a fixed 32-bit lane offset; the bounds checks are per lane only on edge tiles
    const char *src = stg + lrow * PITCH + lq * 16;
    char *rowp = out0 + (int64_t)p * RP * row_bytes;
    if (interior) {
#pragma unroll
      for (int it = 0; it < RP / RS; ++it)
        *reinterpret_cast<uint4 *>(rowp + it * RS * row_bytes + lane_off) =
            *reinterpret_cast<const uint4 *>(src + it * RS * PITCH);
    } else if (vec_ok) {
#pragma unroll
      for (int it = 0; it < RP / RS; ++it) {
        const uint4 v = *reinterpret_cast<const uint4 *>(src + it * RS * PITCH);
        if (cols_left > 0 && p * RP + it * RS < rows_left) *reinterpret_cast<uint4 *>(rowp + it * RS * row_bytes + lane_off) = v;
      }
    } else {
#pragma unroll 1
      for (int it = 0; it < RP / RS; ++it) {
        if (p * RP + it * RS >= rows_left) break;
        const DT *se = reinterpret_cast<const DT *>(src + it * RS * PITCH);
        DT *de = reinterpret_cast<DT *>(rowp + it * RS * row_bytes + lane_off);
#pragma unroll 1
        for (int e = 0; e < cols_left; ++e) de[e] = se[e];
      }
    }
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
  }
}

// MI = 32-row fragments per wave along M: 4 (BM = 256) or 2 (BM = 128);
// NJ = 32-column fragments per wave along N: 4 (BN = 256), 2 (BN = 128) or 1 (BN = 64);
// PS = LDS stages: PS - 1 k-steps are in flight ahead of the one being multiplied, which a small
// tile needs because its k-step is much shorter than the memory latency.
template <int D_DT, int BIAS_DT, int MI, int NJ, int PS>
__global__ __launch_bounds__(256, 1) void linear_nvfp4_tile256p_kernel(LinearArgs a, SplitK sk) {
  extern __shared__ __attribute__((aligned(16))) char plds[];
  AC4K_LTL(0, wall_clock64());
  constexpr int BM = 64 * MI, BN = 64 * NJ;  // two waves along M, two along N
  using PL = PLayout<BM, BN, PS>;
  constexpr int NDA = BM / 4 / 16;         // 16-row A transfers per wave per stage
  constexpr int NDB = BN / 4 / 16;         // 16-row B transfers per wave per stage
  constexpr int NSA = 2 * (BM / 64);       // scale transfers of A per stage: chunks x 64-row blocks
  constexpr int NSB = 2 * (BN / 64);
  constexpr int NS = (NSA + NSB + 3) / 4;  // scale transfers per wave (a remainder repeats the last one)
  constexpr int NPIECES = NDA + NDB + NS;

  const TileCoord tc = tile_of_workgroup<4>(blockIdx.x, ceil_div(a.M, BM), ceil_div(a.N, BN));
  const int64_t tm = tc.m, tn = tc.n;

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  const int half = lane >> 5;
  // this workgroup's range of 128-k stages
  const int nkt_all = (int)(a.K / P_BK);
  const int kt0 = (int)((int64_t)nkt_all * blockIdx.y / sk.splits);
  const int nkt = (int)((int64_t)nkt_all * (blockIdx.y + 1) / sk.splits) - kt0;

  // LDS-DMA.  One transfer moves 16 rows x 64 B: the four lanes 4r .. 4r+3 read the four 16-byte
  // pieces of row r (one 64-byte sector) and land at LDS base + 16*l, i.e. row-major 64-byte rows.
  // Piece p of row r sits at position p ^ ((r >> 1) & 3) of its row: a fragment read takes one piece
  // of each of 32 rows, and unswizzled those addresses fall on a quarter of the LDS banks (an
  // eight-way conflict on every ds_read_b128).  The 32-bit lane offset is loop invariant and the
  // 64-bit part is a scalar base that advances by 64 bytes per stage.
  const int dma_piece = (lane & 3) ^ ((lane >> 3) & 3);  // tile rows of a transfer start at a multiple of 16
  const int swave = __builtin_amdgcn_readfirstlane(wave);
  const int64_t kb = a.K >> 1;
  uint32_t offA[NDA], offB[NDB];
#pragma unroll
  for (int q = 0; q < NDA; ++q) {
    int64_t ra = (swave * NDA + q) * 16 + (lane >> 2);
    ra = tm * BM + ra < a.M ? ra : a.M - 1 - tm * BM;  // rows past the matrix read the last valid row
    offA[q] = (uint32_t)(ra * kb + dma_piece * 16);
  }
  // weight image: a transfer's 16 rows are one contiguous kilobyte of a block (the swizzle is part of
  // the image); bands past the last one read the last band, whose outputs are never stored
  const int64_t w_band_bytes = (int64_t)nkt_all * W_BLOCK_BYTES, w_last_band = (a.N - 1) / W_BLOCK_ROWS;
  auto w_band_of = [&](int64_t row, int64_t &within) {
    int64_t band = row / W_BLOCK_ROWS;
    within = row % W_BLOCK_ROWS;
    return band < w_last_band ? band : w_last_band;
  };
#pragma unroll
  for (int q = 0; q < NDB; ++q) {
    if (a.prepacked) {
      int64_t within;
      const int64_t band = w_band_of(tn * BN + (swave * NDB + q) * 16, within);
      offB[q] = (uint32_t)(band * w_band_bytes + within * P_ROW + lane * 16);
    } else {
      int64_t rb = (swave * NDB + q) * 16 + (lane >> 2);
      rb = tn * BN + rb < a.N ? rb : a.N - 1 - tn * BN;
      offB[q] = (uint32_t)(rb * kb + dma_piece * 16);
    }
  }
  const int64_t strideB = a.prepacked ? W_BLOCK_BYTES : P_ROW;  // bytes per stage along k
  const uint8_t *baseA = uniform_ptr(a.A + tm * BM * kb + (int64_t)kt0 * P_ROW);
  const uint8_t *baseB = uniform_ptr(a.prepacked ? a.B + (int64_t)kt0 * W_BLOCK_BYTES : a.B + tn * BN * kb + (int64_t)kt0 * P_ROW);
  // scale transfers: piece g = swave * NS + p (past the last piece: the last piece again, which
  // lands the same bytes in the same place).  g < NSA: operand A, chunk g / (BM/64), 64-row block
  // g % (BM/64); otherwise operand B, chunk (g-NSA) / (BN/64), block (g-NSA) % (BN/64).  Source
  // base, bytes per stage and LDS offset are wave-uniform and fixed, computed here so that the
  // loop body stays free of branches.
  const uint8_t *sfA8 = uniform_ptr(a.A_sf), *sfB8 = uniform_ptr(a.B_sf);
  uint32_t offS[NS], ldsS[NS];
  const uint8_t *baseS[NS];
  int64_t strideS[NS];
#pragma unroll
  for (int p2 = 0; p2 < NS; ++p2) {
    const int gq = swave * NS + p2 < NSA + NSB ? swave * NS + p2 : NSA + NSB - 1;
    const bool isB = gq >= NSA;
    const int gl = isB ? gq - NSA : gq, nb = isB ? BN / 64 : BM / 64;
    const int c = gl / nb, rb = gl % nb;
    const int64_t rows = isB ? a.Np : a.Mp;
    if (isB && a.prepacked) {  // the scale dwords follow the packed rows of the block
      int64_t within;
      const int64_t band = w_band_of(tn * BN + rb * 64, within);
      offS[p2] = (uint32_t)(band * w_band_bytes + W_BLOCK_DATA + c * (W_BLOCK_ROWS * 4) + (within + lane) * 4);
      strideS[p2] = W_BLOCK_BYTES;
      baseS[p2] = uniform_ptr(a.B + (int64_t)kt0 * W_BLOCK_BYTES);
    } else {
      int64_t sr = (isB ? tn * BN : tm * BM) + rb * 64 + lane;
      sr = sr < rows ? sr : rows - 1;
      offS[p2] = (uint32_t)sr * 4u;  // byte offset inside a scale plane
      strideS[p2] = 2 * rows * 4;    // two planes (chunks) per stage
      baseS[p2] = uniform_ptr((isB ? sfB8 : sfA8) + c * rows * 4 + kt0 * strideS[p2]);
    }
    ldsS[p2] = (uint32_t)__builtin_amdgcn_readfirstlane((isB ? PL::OFF_SFB + c * BN * 4 : PL::OFF_SFA + c * BM * 4) + rb * 256);
  }
  const uint32_t lds_base = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) char *)plds;
  // LDS destinations of this wave's transfers inside a stage (wave-uniform, loop invariant)
  uint32_t ldsA[NDA], ldsB[NDB];
#pragma unroll
  for (int q = 0; q < NDA; ++q) ldsA[q] = (uint32_t)__builtin_amdgcn_readfirstlane((swave * NDA + q) * 1024);
#pragma unroll
  for (int q = 0; q < NDB; ++q) ldsB[q] = (uint32_t)__builtin_amdgcn_readfirstlane(PL::OFF_B + (swave * NDB + q) * 1024);
  // Source pointers of the k-step being fetched.  They advance by one step per iteration and stop
  // at the last step of the range: fetches past the end re-read the last slice into a stage buffer
  // nobody reads again, which keeps the main loop free of branches.
  struct Src {
    const uint8_t *a, *b, *s[NS];
  };
  auto src_at = [&](int kt) {
    Src p;
    p.a = baseA + (int64_t)kt * P_ROW;
    p.b = baseB + (int64_t)kt * strideB;
#pragma unroll
    for (int p2 = 0; p2 < NS; ++p2) p.s[p2] = baseS[p2] + kt * strideS[p2];
    return p;
  };
  auto issue_piece = [&](uint32_t stage_lds, const Src &p, int q) {
    if (q < NDA) {
      dma16(p.a, offA[q], stage_lds, ldsA[q]);
    } else if (q < NDA + NDB) {
      dma16(p.b, offB[q - NDA], stage_lds, ldsB[q - NDA]);
    } else {
      const int p2 = q - NDA - NDB;
      dma4(p.s[p2], offS[p2], stage_lds, ldsS[p2]);
    }
  };
  auto issue_stage = [&](uint32_t stage_lds, const Src &p) {
#pragma unroll
    for (int q = 0; q < NPIECES; ++q) issue_piece(stage_lds, p, q);
  };
  // pieces issued in quarter `qr` (0..3) of the second half of a step
  auto issue_quarter = [&](uint32_t stage_lds, const Src &p, int qr) {
#pragma unroll
    for (int q = 0; q < NDA; ++q)
      if (q * 4 / NDA == qr) issue_piece(stage_lds, p, q);
#pragma unroll
    for (int q = 0; q < NDB; ++q)
      if (q * 4 / NDB == qr) issue_piece(stage_lds, p, NDA + q);
#pragma unroll
    for (int q = 0; q < NS; ++q)
      if (q * 4 / NS == qr) issue_piece(stage_lds, p, NDA + NDB + q);
  };

  f32x16 acc[MI][NJ];
#pragma unroll
  for (int i = 0; i < MI; ++i)
#pragma unroll
    for (int j = 0; j < NJ; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.0f;

  // fragment addresses inside a stage (bytes)
  // (a lane's rows differ by multiples of 32, so the swizzle term of its row is (lane >> 1) & 3 for all of them)
  const int fa_off = (wm * (32 * MI) + (lane & 31)) * P_ROW;
  const int fb_off = PL::OFF_B + (wn * (32 * NJ) + (lane & 31)) * P_ROW;
  const int piece_off[2] = {((0 + half) ^ ((lane >> 1) & 3)) * 16, ((2 + half) ^ ((lane >> 1) & 3)) * 16};  // chunk 0, chunk 1
  // a lane needs the two scale bytes of its half of the chunk: blocks 2*half, 2*half+1
  const int sa_off = PL::OFF_SFA + (wm * (32 * MI) + (lane & 31)) * 4 + half * 2;
  const int sb_off = PL::OFF_SFB + (wn * (32 * NJ) + (lane & 31)) * 4 + half * 2;

  uint4 PA[2][MI], PB[2][NJ];  // packed fragments of a 64-chunk, double buffered by chunk parity
  f16x2 SA[2][MI], SB[2][NJ];  // their two block scales (blocks 2*half, 2*half+1) as fp16
  auto load_chunk = [&](uint32_t stage_off, int c) {
    const char *st = plds + stage_off;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      if (i < MI) PA[c][i] = *reinterpret_cast<const uint4 *>(st + fa_off + piece_off[c] + i * 32 * P_ROW);
      if (i < NJ) PB[c][i] = *reinterpret_cast<const uint4 *>(st + fb_off + piece_off[c] + i * 32 * P_ROW);
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      if (i < MI) {
        const uint32_t wa = *reinterpret_cast<const uint16_t *>(st + sa_off + c * (BM * 4) + i * 128);
        SA[c][i] = __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(wa, 1.0f, false);
      }
      if (i < NJ) {
        const uint32_t wb = *reinterpret_cast<const uint16_t *>(st + sb_off + c * (BN * 4) + i * 128);
        SB[c][i] = __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(wb, 1.0f, false);
      }
    }
  };

  DecFrags<MI, NJ> D[2];
  auto decode = [&](DecFrags<MI, NJ> &d, int c, auto S) {
    constexpr int s = decltype(S)::value;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      if (i < MI) d.a[i] = decode_dword<(s >= 2)>(dword_of<s>(PA[c][i]), SA[c][i]);
      if (i < NJ) d.b[i] = decode_dword<(s >= 2)>(dword_of<s>(PB[c][i]), SB[c][i]);
    }
  };
  auto mfma16 = [&](const DecFrags<MI, NJ> &d) {
#pragma unroll
    for (int i = 0; i < MI; ++i)
#pragma unroll
      for (int jj = 0; jj < NJ; ++jj) {
        // boustrophedon order: every MFMA shares one operand with the one before it (measured 0.6 %
        // faster than row by row on the power-limited 8192^3 problem: less operand switching)
        const int j = (i & 1) ? NJ - 1 - jj : jj;
        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(d.b[j], d.a[i], acc[i][j], 0, 0, 0);  // D^T block
      }
  };
  auto interleave = [&]() {  // the decode of the next sub-step rides in the shadow of the MFMAs
    constexpr int NMFMA = MI * NJ, NVALU = 8 * (MI + NJ);
    constexpr int PER = (NVALU + NMFMA - 1) / NMFMA;  // 4 for 4x4, 6 for 2x4 and 4x2, 8 for 2x2, ...
#pragma unroll
    for (int g = 0; g < NMFMA; ++g) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x002, PER, 0);
    }
    __builtin_amdgcn_sched_barrier(0);
  };
  using I0 = std::integral_constant<int, 0>;
  using I1 = std::integral_constant<int, 1>;
  using I2 = std::integral_constant<int, 2>;
  using I3 = std::integral_constant<int, 3>;

  // prologue: stages 0 .. PS-2 in flight (past the last k-step: the last one again), stage 0
  // visible, chunk 0 fragments and first decode
  static_assert(PS >= 3 && (PS - 2) * NPIECES <= 63, "the wait counts below must fit the 6-bit counter");
  const int last = nkt - 1;
#pragma unroll
  for (int d = 0; d < PS - 1; ++d) issue_stage(lds_base + d * PL::STAGE_BYTES, src_at(d < last ? d : last));
  wait_vmcnt<(PS - 2) * NPIECES>();  // everything of stage 0 has landed, later stages may be in flight
  __syncthreads();
  load_chunk(0, 0);
  decode(D[0], 0, I0{});

  // loop-carried, wave-uniform: LDS offsets of the stages holding k-steps kt, kt+1 and of the one
  // being filled with kt+PS-1 (a ring of PS), and the source pointers of k-step min(kt+PS-1, last)
  uint32_t st_cur = 0, st_nxt = PL::STAGE_BYTES, st_dma = (PS - 1) * PL::STAGE_BYTES;
  auto ring_next = [](uint32_t o) { return o + PL::STAGE_BYTES == (uint32_t)PL::LDS_BYTES ? 0u : o + PL::STAGE_BYTES; };
  Src src = src_at(last < PS - 1 ? last : PS - 1);
#ifdef AC4K_LINEAR_TIMELINE
  const uint64_t tl_c0 = __builtin_readcyclecounter();
#endif
  AC4K_LTL(1, wall_clock64());
  for (int kt = 0; kt < nkt; ++kt) {
    // chunk 0: sub-steps 0..3 (fragments of chunk 1 are fetched meanwhile)
    load_chunk(st_cur, 1);
    decode(D[1], 0, I1{});
    mfma16(D[0]);
    interleave();
    decode(D[0], 0, I2{});
    mfma16(D[1]);
    interleave();
    decode(D[1], 0, I3{});
    mfma16(D[0]);
    interleave();
    decode(D[0], 1, I0{});
    mfma16(D[1]);
    interleave();
    // stage kt+1 must be complete (own DMA done, then everybody's; stages kt+2 .. kt+PS-2 may still
    // be in flight); stage kt-1 is free after this
    wait_vmcnt<(PS - 3) * NPIECES>();
    __syncthreads();
    // chunk 1: sub-steps 4..7 (chunk 0 of the next stage is fetched meanwhile); the DMA of stage
    // kt+PS-1 is spread over these sub-steps
    const uint32_t dma_lds = lds_base + st_dma;
    decode(D[1], 1, I1{});
    issue_quarter(dma_lds, src, 0);
    mfma16(D[0]);
    interleave();
    load_chunk(st_nxt, 0);  // past the end this reads a stale stage; the result is never used
    decode(D[0], 1, I2{});
    issue_quarter(dma_lds, src, 1);
    mfma16(D[1]);
    interleave();
    decode(D[1], 1, I3{});
    issue_quarter(dma_lds, src, 2);
    mfma16(D[0]);
    interleave();
    decode(D[0], 0, I0{});  // first sub-step of the next stage (unused after the last step)
    issue_quarter(dma_lds, src, 3);
    mfma16(D[1]);
    interleave();
    // rotate the stages; advance the sources unless they already sit on the last k-step
    st_cur = st_nxt;
    st_nxt = ring_next(st_nxt);
    st_dma = ring_next(st_dma);
    const bool adv = kt + PS <= last;
    src.a += adv ? P_ROW : 0;
    src.b += adv ? strideB : 0;
#pragma unroll
    for (int p2 = 0; p2 < NS; ++p2) src.s[p2] += adv ? strideS[p2] : 0;
  }
  AC4K_LTL(2, wall_clock64());
#ifdef AC4K_LINEAR_TIMELINE
  AC4K_LTL(4, __builtin_readcyclecounter() - tl_c0);
  {
    uint32_t xcc, hwid;
    asm volatile("s_getreg_b32 %0, hwreg(HW_REG_XCC_ID)" : "=s"(xcc));
    asm volatile("s_getreg_b32 %0, hwreg(HW_REG_HW_ID)" : "=s"(hwid));
    AC4K_LTL(5, (xcc & 0xf) | (hwid << 8));
  }
#endif

  // ---- epilogue.  The MFMAs were issued with the operands swapped, so acc[i][j] holds the
  // TRANSPOSED 32x32 block: lane l, element e <-> n = j*32 + (e>>2)*8 + (l>>5)*4 + (e&3),
  // m = i*32 + (l&31): four consecutive n per lane.
  const int64_t m0 = tm * BM + (swave >> 1) * (32 * MI), n0 = tn * BN + (swave & 1) * (32 * NJ);
  // the last iterations' LDS-DMA fetches (into a stage nobody reads) must have landed before the
  // stages are reused, and every wave must be done reading them
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();
  if (sk.partial) {  // split-K: raw fp32 sums of this K range; the reduce kernel scales and converts
    store_tile<AC4K_DTYPE_FP32, BIAS_NONE, true, MI, NJ, PL::LDS_BYTES>(
        acc, plds, sk.partial + (int64_t)blockIdx.y * a.M * a.N, nullptr, 1.0f, a.M, a.N, m0, n0, tn * BN);
  } else {
    store_tile<D_DT, BIAS_DT, false, MI, NJ, PL::LDS_BYTES>(acc, plds, a.D, a.bias, (*a.A_gs) * (*a.B_gs), a.M, a.N,
                                                           m0, n0, tn * BN);
  }
  AC4K_LTL(3, wall_clock64());
}

// Raises a kernel's dynamic LDS limit once per (kernel instantiation, device): the attribute belongs
// to the device the call is made on.
template <typename Kernel>
static int allow_dynamic_lds(Kernel *kern, std::atomic<uint32_t> &done_mask, int bytes) {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) dev = 0;
  const uint32_t bit = 1u << (dev & 31);
  if (done_mask.load(std::memory_order_relaxed) & bit) return 0;
  hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
  if (e != hipSuccess) return set_error("hipFuncSetAttribute(LDS=%d): %s", bytes, hipGetErrorString(e));
  done_mask.fetch_or(bit, std::memory_order_relaxed);
  return 0;
}

// LDS stages per tile shape: enough k-steps in flight to cover the memory latency
constexpr int tile_stages(int mi, int nj) { return mi * nj >= 16 ? 3 : mi * nj >= 8 ? 4 : mi * nj >= 4 ? 6 : 8; }

template <int D_DT, int BIAS_DT, int MI, int NJ>
static int launch_tile_p(const LinearArgs &a, const SplitK &sk, hipStream_t st) {
  constexpr int PS = tile_stages(MI, NJ);
  auto *kern = linear_nvfp4_tile256p_kernel<D_DT, BIAS_DT, MI, NJ, PS>;
  using PL = PLayout<64 * MI, 64 * NJ, PS>;
  static std::atomic<uint32_t> lds_ok{0};
  if (int rc = allow_dynamic_lds(kern, lds_ok, PL::LDS_BYTES)) return rc;
  const int64_t ntiles = ceil_div(a.M, 64 * MI) * ceil_div(a.N, 64 * NJ);
  hipLaunchKernelGGL(kern, dim3((unsigned)ntiles, (unsigned)sk.splits), dim3(256), PL::LDS_BYTES, st, a, sk);
  return 0;
}

// Tile shape and K split of the packed-LDS kernel for one problem.
struct TilePlan {
  int mi, nj;              // tile = (64 mi) x (64 nj)
  int splits;              // K ranges per tile; > 1 needs `partial_bytes` of fp32 scratch
  int64_t partial_bytes;
};

// Picks the tile and the split by a rough cost model in microseconds on 256 CUs: rounds of
// workgroups x stages per range x time per 128-k stage of that tile, a fixed prologue/epilogue,
// and for more than one range the partial sums written and read back at about 4.5 TB/s plus the
// second launch.  Big problems (192 or more of the largest tiles) take the largest tile as is.
// The time per stage is a fit to measured loops of the five tile shapes: per 16-k sub-step about
// 14 cycles per MFMA plus 5 per decode instruction, 400 cycles per stage on top, at 2.1 GHz.
// Tuning overrides (ac4k_set_linear_tuning): a forced tile plan packed as mi | nj << 8 | splits << 16
// (0 = the cost model decides) and a forced K slice of the decode-sized kernel (0 = automatic).
static std::atomic<uint32_t> g_forced_tile_plan{0};
static std::atomic<int> g_forced_skinny_ks{0};

static TilePlan tile_plan(int64_t M, int64_t N, int64_t K, bool allow_split) {
  TilePlan best{M <= 128 ? 2 : 4, 4, 1, 0};
  if (const uint32_t f = g_forced_tile_plan.load(std::memory_order_relaxed)) {
    const int mi = f & 0xff, nj = (f >> 8) & 0xff, sp = (int)(f >> 16);
    if (sp <= K / P_BK && (sp == 1 || allow_split)) return TilePlan{mi, nj, sp, sp > 1 ? (int64_t)sp * M * N * 4 : 0};
  }
  const int64_t stages = K / P_BK;
  if (ceil_div(M, 64 * best.mi) * ceil_div(N, 256) >= 192) return best;
  double best_t = 0.0;
  bool first = true;
  for (int mi = 2; mi <= 4; mi += 2) {
    if (mi == 4 && M <= 128) continue;
    for (int nj = 4; nj >= 1; nj >>= 1) {
      if (mi == 4 && nj == 1) continue;  // not instantiated
      if (nj < 4 && N < 64 * nj * 2) continue;
      const int nm = mi * nj, nv = 8 * (mi + nj);
      const double stage_us = (8.0 * (14.0 * nm + 5.0 * nv) + 400.0) / 2100.0;
      const double fixed_us = 5.0 + 0.1 * nm;
      const int64_t tiles = ceil_div(M, 64 * mi) * ceil_div(N, 64 * nj);
      for (int64_t sp = 1; sp <= 32 && (sp == 1 || (allow_split && sp * 2 <= stages)); ++sp) {
        const double rounds = (double)ceil_div(tiles * sp, 256);
        double t = rounds * (double)ceil_div(stages, sp) * stage_us + fixed_us;
        if (sp > 1) t += (double)sp * (double)(M * N) * 8.0 / 4.5e6 + 2.5;
        if (first || t < best_t) {
          first = false;
          best_t = t;
          best = TilePlan{mi, nj, (int)sp, sp > 1 ? sp * M * N * 4 : 0};
        }
      }
    }
  }
  return best;
}

template <int D_DT, int BIAS_DT>
static int launch_tile_plan(const LinearArgs &a, const TilePlan &p, const SplitK &sk, hipStream_t st) {
  if (p.mi == 4) return p.nj == 4 ? launch_tile_p<D_DT, BIAS_DT, 4, 4>(a, sk, st) : launch_tile_p<D_DT, BIAS_DT, 4, 2>(a, sk, st);
  if (p.nj == 4) return launch_tile_p<D_DT, BIAS_DT, 2, 4>(a, sk, st);
  return p.nj == 2 ? launch_tile_p<D_DT, BIAS_DT, 2, 2>(a, sk, st) : launch_tile_p<D_DT, BIAS_DT, 2, 1>(a, sk, st);
}

// the packed-LDS kernel with the tile that suits the shape; no split-K (one K range, output to D)
template <int D_DT, int BIAS_DT>
static int launch_tile256p(const LinearArgs &a, hipStream_t st) {
  const SplitK one{nullptr, 1};
  return launch_tile_plan<D_DT, BIAS_DT>(a, tile_plan(a.M, a.N, a.K, false), one, st);
}

// ===========================================================================
// Mid-sized M (33 .. 128): every weight byte is used by at most four 32-row activation fragments, so
// the problem is bound by streaming the weights and by decode instructions, not by the MFMA rate, and
// there are too few 256-wide tiles to fill the GPU.  Tile (32 MI) x (32 NJ) with ALL of M in one tile
// (MI = 4, NJ = 2: 128 x 64) and the four waves of the workgroup splitting K, not the tile: a stage is
// 256 k = four 64-chunks, wave w multiplies the whole tile over chunk w.  Every packed fragment of the
// stage is then decoded exactly once per workgroup (the 2 x 2 wave grid of the tile kernel decodes each
// one twice): (MI + NJ) * 8 decode instructions per MI * NJ MFMAs, 6 per MFMA for 128 x 64, with one
// wave per SIMD.  Packed rows and scale dwords of a stage travel by LDS-DMA into a ring (128-byte rows,
// 16-byte pieces at position piece ^ (row & 7), scales as [chunk][row] dwords); one workgroup barrier
// per stage.  The four k parts of the tile meet through LDS at the end: wave w receives the sums of a
// quarter of the tile from the other three, adds them in wave order, and stores its quarter
// (times gsA * gsB, plus bias), or the raw fp32 sums of this K range when K is split over workgroups.
// Requires K % 256 == 0 and 16-byte aligned operands and scale tensors.
// ===========================================================================
constexpr int KW_BK = 256;          // k per stage
constexpr int KW_ROW = KW_BK / 2;   // packed bytes per row per stage

template <int MI, int NJ>
struct KWLayout {
  static constexpr int BM = 32 * MI, BN = 32 * NJ;
  static_assert(BM % 64 == 0 && BN % 64 == 0, "a scale transfer covers 64-row blocks");
  static constexpr int OFF_W = 0;                         // BN weight rows, then BM activation rows
  static constexpr int OFF_A = BN * KW_ROW;
  static constexpr int OFF_SFW = OFF_A + BM * KW_ROW;     // scale dwords [4 chunks][BN rows]
  static constexpr int OFF_SFA = OFF_SFW + 4 * BN * 4;    // [4 chunks][BM rows]
  static constexpr int STAGE_BYTES = OFF_SFA + 4 * BM * 4;
  static constexpr int PS = (160 * 1024) / STAGE_BYTES < 8 ? (160 * 1024) / STAGE_BYTES : 8;  // ring slots
  static constexpr int LDS_BYTES = PS * STAGE_BYTES;
  static constexpr int NROW = (BM + BN) / 8 / 4;          // 8-row transfers per wave per stage
  static constexpr int NSCW = BN / 64, NSCA = BM / 64;    // scale transfers per stage (1 KB each)
  static constexpr int NPIECES = NROW + 1;                // every wave issues the same count
  static constexpr int PPW = MI * NJ / 4;                 // 32 x 32 output blocks a wave finishes
  static_assert((BM + BN) % 32 == 0 && NSCW + NSCA <= 4 && MI * NJ % 4 == 0, "transfers are dealt evenly to four waves");
  static_assert(PS >= 3 && (PS - 2) * NPIECES <= 63, "the wait counts must fit the 6-bit counter");
  static_assert(LDS_BYTES >= 16 * PPW * 4096, "the ring doubles as the exchange buffer of the four k parts");
};

template <int D_DT, int BIAS_DT, int MI, int NJ>
__global__ __launch_bounds__(256, 1) void linear_nvfp4_ksplit_kernel(LinearArgs a, SplitK sk) {
  using L = KWLayout<MI, NJ>;
  constexpr int BM = L::BM, BN = L::BN, PS = L::PS, NP = L::NPIECES;
  extern __shared__ __attribute__((aligned(16))) char kwlds[];
  AC4K_LTL(0, wall_clock64());
  const int tid = threadIdx.x, lane = tid & 63, half = lane >> 5, r32 = lane & 31;
  const int swave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int64_t tiles_n = ceil_div(a.N, BN);
  const int64_t tm = blockIdx.x / tiles_n, tn = blockIdx.x % tiles_n;
  const int64_t m0 = tm * BM, n0 = tn * BN;
  const int nst_all = (int)(a.K / KW_BK);
  const int s0 = (int)((int64_t)nst_all * blockIdx.y / sk.splits);
  const int nst = (int)((int64_t)nst_all * (blockIdx.y + 1) / sk.splits) - s0;  // >= 1: splits <= stages
  const int64_t kb = a.K >> 1;
  // workgroup b starts at stage b % nst of its range and wraps around, so that the workgroups of a
  // launch do not all ask for the same column of their rows at the same time (memory channels)
  const int rot = (int)(blockIdx.x % (unsigned)nst);
  const int last = nst - 1;
  auto stage_of = [&](int step) {
    const int p = (step < last ? step : last) + rot;
    return p >= nst ? p - nst : p;
  };

  // --- this wave's transfers of a stage
  const uint32_t lds_base = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) char *)kwlds;
  // rows: transfer t = swave * NROW + q moves rows 8 t .. 8 t + 7 of the stage (weight rows first), lane l
  // the piece of row l / 8 that belongs at position l % 8
  // On a weight image (a.prepacked) a stage is two blocks of the row's 128-row band, 64 bytes of the row in
  // each, pieces at p ^ ((row >> 1) & 3), and the four chunk planes of scale dwords sit behind the blocks' data.
  const int64_t img_band_bytes = (a.K / W_BLOCK_K) * (int64_t)W_BLOCK_BYTES;
  uint32_t offR[L::NROW], ldsR[L::NROW];
  const uint8_t *srcR[L::NROW];
  int strR[L::NROW];  // bytes per stage along k
#pragma unroll
  for (int q = 0; q < L::NROW; ++q) {
    const int t = swave * L::NROW + q;
    const bool isW = t < BN / 8;
    const int loc = (isW ? t : t - BN / 8) * 8 + (lane >> 3);
    const int pp = (lane & 7) ^ (loc & 7);  // the piece of the stage row that belongs at this lane's position
    if (isW && a.prepacked) {
      const int64_t wrow = n0 + loc;  // rows past N exist in the image (zeros)
      const int64_t band = wrow / W_BLOCK_ROWS, within = wrow % W_BLOCK_ROWS;
      offR[q] = (uint32_t)(band * img_band_bytes + (pp >> 2) * W_BLOCK_BYTES + within * 64 + (((pp & 3) ^ ((within >> 1) & 3)) * 16));
      srcR[q] = uniform_ptr(a.B + (int64_t)s0 * (2 * W_BLOCK_BYTES));
      strR[q] = 2 * W_BLOCK_BYTES;
    } else {
      const int64_t rows = isW ? a.N : a.M, first = isW ? n0 : m0;
      const int64_t row = first + loc < rows ? loc : rows - 1 - first;  // rows past the matrix read its last row
      offR[q] = (uint32_t)(row * kb + pp * 16);
      srcR[q] = uniform_ptr((isW ? a.B + n0 * kb : a.A + m0 * kb) + (int64_t)s0 * KW_ROW);
      strR[q] = KW_ROW;
    }
    strR[q] = __builtin_amdgcn_readfirstlane(strR[q]);
    ldsR[q] = (uint32_t)__builtin_amdgcn_readfirstlane(t * 1024);
  }
  // scales: one transfer is 256 dwords of the [chunk][row] picture, a lane the four dwords of rows
  // 4 g .. 4 g + 3 of one chunk (16 bytes of the scale tensor).  Transfers 0 .. NSCW - 1 are the weights',
  // the others the activation's; a wave past the last transfer repeats the last one.
  uint32_t offS, ldsS;
  const uint8_t *srcS;
  int64_t strideS;
  {
    const int t = swave < L::NSCW + L::NSCA ? swave : L::NSCW + L::NSCA - 1;
    const bool isW = t < L::NSCW;
    const int tt = isW ? t : t - L::NSCW;
    const int bx = isW ? BN : BM;                         // rows of the operand's tile
    const int cpt = 256 / bx;                             // chunks per transfer (4 or 2)
    const int chunk = tt * cpt + lane / (bx / 4), grp = lane % (bx / 4);
    const int64_t rows_p = isW ? a.Np : a.Mp, first = isW ? n0 : m0;
    int64_t row = first + 4 * grp;
    if (isW && a.prepacked) {
      const int64_t band = row / W_BLOCK_ROWS, within = row % W_BLOCK_ROWS;
      offS = (uint32_t)(band * img_band_bytes + (chunk >> 1) * W_BLOCK_BYTES + W_BLOCK_DATA + (chunk & 1) * (W_BLOCK_ROWS * 4) + within * 4);
      strideS = 2 * W_BLOCK_BYTES;
      srcS = uniform_ptr(a.B + s0 * strideS);
    } else {
      row = row + 4 <= rows_p ? row : rows_p - 4;         // groups past the padded rows read the last group
      offS = (uint32_t)((chunk * rows_p + row) * 4);
      strideS = 4 * rows_p * 4;                           // bytes per stage: four chunk planes
      srcS = uniform_ptr(reinterpret_cast<const uint8_t *>(isW ? a.B_sf : a.A_sf) + s0 * strideS);
    }
    ldsS = (uint32_t)__builtin_amdgcn_readfirstlane((isW ? L::OFF_SFW : L::OFF_SFA) + tt * 1024);
  }
  // Transfer q of this wave's NPIECES for stage `st` into the ring slot at `base`.  Past the end of the range
  // the loop keeps issuing, so that it stays free of branches and its wait counts stay fixed: those transfers
  // read the last stage again (cache hits) into slots nobody reads any more.
  auto issue_piece = [&](uint32_t base, int st, int q) {
    if (q < L::NROW)
      dma16(srcR[q] + (int64_t)st * strR[q], offR[q], base, ldsR[q]);
    else
      dma16(srcS + st * strideS, offS, base, ldsS);
  };
  // the transfers of a stage are issued in four parts, one per 16-k sub-step
  auto issue_part = [&](uint32_t base, int st, int part) {
#pragma unroll
    for (int q = 0; q < NP; ++q)
      if (q * 4 / NP == part) issue_piece(base, st, q);
  };

  // --- this wave's fragments of a stage: chunk swave; lane (r32, half) holds elements [32 half, 32 half + 32)
  // of the chunk of one row per fragment (16 packed bytes) and the two block scales that go with them
  struct Frags {
    uint4 x[MI], w[NJ];
    uint32_t xs[MI], ws[NJ];
  };
  const int piece = swave * 2 + half;
  const int f_off = r32 * KW_ROW + ((piece ^ (r32 & 7)) * 16);  // rows 32 apart share the swizzle term
  const int ws_off = L::OFF_SFW + (swave * BN + r32) * 4 + half * 2;
  const int xs_off = L::OFF_SFA + (swave * BM + r32) * 4 + half * 2;
  auto load_frags = [&](int slot) {
    const char *st = kwlds + slot * L::STAGE_BYTES;
    Frags f;
#pragma unroll
    for (int j = 0; j < NJ; ++j) {
      f.w[j] = *reinterpret_cast<const uint4 *>(st + L::OFF_W + f_off + j * 32 * KW_ROW);
      f.ws[j] = *reinterpret_cast<const uint16_t *>(st + ws_off + j * 128);
    }
#pragma unroll
    for (int i = 0; i < MI; ++i) {
      f.x[i] = *reinterpret_cast<const uint4 *>(st + L::OFF_A + f_off + i * 32 * KW_ROW);
      f.xs[i] = *reinterpret_cast<const uint16_t *>(st + xs_off + i * 128);
    }
    return f;
  };

  f32x16 acc[MI][NJ];
#pragma unroll
  for (int i = 0; i < MI; ++i)
#pragma unroll
    for (int j = 0; j < NJ; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.0f;

  DecFrags<MI, NJ> D[2];
  auto decode = [&](DecFrags<MI, NJ> &d, const Frags &f, auto S) {
    constexpr int s = decltype(S)::value;
#pragma unroll
    for (int j = 0; j < NJ; ++j)
      d.b[j] = decode_dword<(s >= 2)>(dword_of<s>(f.w[j]), __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(f.ws[j], 1.0f, false));
#pragma unroll
    for (int i = 0; i < MI; ++i)
      d.a[i] = decode_dword<(s >= 2)>(dword_of<s>(f.x[i]), __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(f.xs[i], 1.0f, false));
  };
  auto mfma_all = [&](const DecFrags<MI, NJ> &d) {
#pragma unroll
    for (int i = 0; i < MI; ++i)
#pragma unroll
      for (int jj = 0; jj < NJ; ++jj) {
        const int j = (i & 1) ? NJ - 1 - jj : jj;  // neighbours share an operand
        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(d.b[j], d.a[i], acc[i][j], 0, 0, 0);  // D^T block
      }
  };
  auto interleave = [&]() {  // the decode of the next sub-step rides in the shadow of the MFMAs
    constexpr int NMFMA = MI * NJ, NVALU = 8 * (MI + NJ) + (MI + NJ);
    constexpr int PER = (NVALU + NMFMA - 1) / NMFMA;
#pragma unroll
    for (int g = 0; g < NMFMA; ++g) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x002, PER, 0);
    }
    __builtin_amdgcn_sched_barrier(0);
  };
  using I0 = std::integral_constant<int, 0>;
  using I1 = std::integral_constant<int, 1>;
  using I2 = std::integral_constant<int, 2>;
  using I3 = std::integral_constant<int, 3>;

  // prologue: the first PS stages in flight, stage 0 landed and its fragments in registers (every wave's,
  // before slot 0 is refilled), then stage 1 landed
#pragma unroll
  for (int d = 0; d < PS; ++d) {
#pragma unroll
    for (int q = 0; q < NP; ++q) issue_piece(lds_base + d * L::STAGE_BYTES, stage_of(d), q);
  }
  wait_vmcnt<(PS - 1) * NP>();
  __syncthreads();
  Frags F0 = load_frags(0), F1;
  decode(D[0], F0, I0{});
  wait_vmcnt<(PS - 2) * NP>();
  asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
  __syncthreads();

  int slot_cur = 0, slot_next = 1;
#ifdef AC4K_LINEAR_TIMELINE
  const uint64_t tl_c0 = __builtin_readcyclecounter();
#endif
  AC4K_LTL(1, wall_clock64());
  // one stage: `cur` holds its fragments, `nxt` receives those of the next one (two named sets that swap
  // roles, so that no register is copied between stages)
  auto stage_step = [&](const Frags &cur, Frags &nxt, int s) {
    // The slot of this stage is free (every wave had its fragments in registers before the previous
    // barrier): stage s + PS goes there.
    const int st_new = stage_of(s + PS);
    const uint32_t base_new = lds_base + slot_cur * L::STAGE_BYTES;
    // fragments of the next stage (it landed before the previous barrier) travel from LDS while this
    // one is decoded and multiplied (past the range: a stage nobody uses)
    nxt = load_frags(slot_next);
    decode(D[1], cur, I1{});
    issue_part(base_new, st_new, 0);
    mfma_all(D[0]);
    interleave();
    decode(D[0], cur, I2{});
    issue_part(base_new, st_new, 1);
    mfma_all(D[1]);
    interleave();
    decode(D[1], cur, I3{});
    issue_part(base_new, st_new, 2);
    mfma_all(D[0]);
    interleave();
    decode(D[0], nxt, I0{});
    issue_part(base_new, st_new, 3);
    mfma_all(D[1]);
    interleave();
    wait_vmcnt<(PS - 2) * NP>();                        // own transfers of stage s + 2 have landed
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // and the fragments of stage s + 1 are in registers
    __syncthreads();
    slot_cur = slot_next;
    slot_next = slot_next + 1 == PS ? 0 : slot_next + 1;
  };
  for (int s = 0; s < nst; s += 2) {
    stage_step(F0, F1, s);
    if (s + 1 < nst) stage_step(F1, F0, s + 1);
  }
  AC4K_LTL(2, wall_clock64());
#ifdef AC4K_LINEAR_TIMELINE
  AC4K_LTL(4, __builtin_readcyclecounter() - tl_c0);
#endif
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // no LDS-DMA may land after this point: the ring is reused
  __syncthreads();

  // --- the four k parts meet: wave d finishes blocks p = d * PPW + q (i = p / NJ, j = p % NJ).
  // acc[i][j]: lane l, element e <-> m = 32 i + (l & 31), n = 32 j + (e >> 2) * 8 + (l >> 5) * 4 + (e & 3)
  constexpr int PPW = L::PPW;
  float4 *xch = reinterpret_cast<float4 *>(kwlds);
  auto xch_at = [&](int d, int src, int q, int g) { return xch + ((((d * 4 + src) * PPW + q) * 4 + g) * 64 + lane); };
#pragma unroll
  for (int d = 0; d < 4; ++d) {
    if (d == swave) continue;
#pragma unroll
    for (int q = 0; q < PPW; ++q) {
      const int p = d * PPW + q, i = p / NJ, j = p % NJ;
#pragma unroll
      for (int g = 0; g < 4; ++g)
        *xch_at(d, swave, q, g) = make_float4(acc[i][j][4 * g], acc[i][j][4 * g + 1], acc[i][j][4 * g + 2], acc[i][j][4 * g + 3]);
    }
  }
  __syncthreads();
  const float scale = sk.partial ? 1.0f : (*a.A_gs) * (*a.B_gs);
  using DE = Elem<D_DT>;
  const bool vec_ok = (a.N & 3) == 0 && (((uintptr_t)a.D | (uintptr_t)sk.partial) & 15) == 0;
#pragma unroll
  for (int d = 0; d < 4; ++d) {
    if (d != swave) continue;
#pragma unroll
    for (int q = 0; q < PPW; ++q) {
      const int p = d * PPW + q, i = p / NJ, j = p % NJ;
      const int64_t m = m0 + 32 * i + r32;
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        float4 sum = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
#pragma unroll
        for (int src = 0; src < 4; ++src) {  // always in wave order
          const float4 t = src == d ? make_float4(acc[i][j][4 * g], acc[i][j][4 * g + 1], acc[i][j][4 * g + 2], acc[i][j][4 * g + 3])
                                    : *xch_at(d, src, q, g);
          if (src == 0) sum = t;
          else { sum.x += t.x; sum.y += t.y; sum.z += t.z; sum.w += t.w; }
        }
        const int64_t n = n0 + 32 * j + g * 8 + half * 4;
        if (m >= a.M || n >= a.N) continue;
        if (sk.partial) {  // raw fp32 sums of this K range; the reduce kernel scales and converts
          float *pp = sk.partial + ((int64_t)blockIdx.y * a.M + m) * a.N + n;
          if (vec_ok && n + 3 < a.N) *reinterpret_cast<float4 *>(pp) = sum;
          else {
            const float v[4] = {sum.x, sum.y, sum.z, sum.w};
#pragma unroll
            for (int c = 0; c < 4; ++c)
              if (n + c < a.N) pp[c] = v[c];
          }
          continue;
        }
        float v[4] = {sum.x * scale, sum.y * scale, sum.z * scale, sum.w * scale};
        if constexpr (BIAS_DT != BIAS_NONE) {
#pragma unroll
          for (int c = 0; c < 4; ++c) v[c] += n + c < a.N ? Elem<BIAS_DT>::load(a.bias, n + c) : 0.0f;
        }
        typename DE::T *dst = static_cast<typename DE::T *>(a.D) + m * a.N + n;
        if (vec_ok && n + 3 < a.N) {
          if constexpr (sizeof(typename DE::T) == 2)
            *reinterpret_cast<uint2 *>(dst) = make_uint2(DE::cvt2(v[0], v[1]), DE::cvt2(v[2], v[3]));
          else
            *reinterpret_cast<float4 *>(dst) = make_float4(v[0], v[1], v[2], v[3]);
        } else {
#pragma unroll
          for (int c = 0; c < 4; ++c)
            if (n + c < a.N) dst[c] = DE::cvt(v[c]);
        }
      }
    }
  }
  AC4K_LTL(3, wall_clock64());
}

template <int D_DT, int BIAS_DT, int MI, int NJ>
static int launch_ksplit_t(const LinearArgs &a, const SplitK &sk, hipStream_t st) {
  using L = KWLayout<MI, NJ>;
  auto *kern = linear_nvfp4_ksplit_kernel<D_DT, BIAS_DT, MI, NJ>;
  static std::atomic<uint32_t> lds_ok{0};
  if (int rc = allow_dynamic_lds(kern, lds_ok, L::LDS_BYTES)) return rc;
  const int64_t ntiles = ceil_div(a.M, L::BM) * ceil_div(a.N, L::BN);
  hipLaunchKernelGGL(kern, dim3((unsigned)ntiles, (unsigned)sk.splits), dim3(256), L::LDS_BYTES, st, a, sk);
  return 0;
}

// Tile and K split of the K-split-waves kernel.
struct KsplitPlan {
  int mi, nj;
  int splits;              // K ranges per tile; > 1 needs `partial_bytes` of fp32 scratch
  int64_t partial_bytes;
};

// shapes the K-split-waves kernel takes (its pointer conditions are in ksplit_aligned)
static bool ksplit_shape(int64_t M, int64_t N, int64_t K) {
  return M > 32 && M <= 128 && N >= 64 && K >= KW_BK && K % KW_BK == 0 && (K >> 1) * 128 < (1ll << 31) && N < (1ll << 27) &&
         g_forced_tile_plan.load(std::memory_order_relaxed) == 0;
}
static bool ksplit_aligned(const LinearArgs &a) {
  return (((uintptr_t)a.A | (uintptr_t)a.B | (uintptr_t)a.A_sf | (uintptr_t)a.B_sf) & 15) == 0;
}

// All of M in one tile: 128 x 64 above 64 rows, 64 x 64 below (64 x 128 when even those fill the GPU).
// Fewer than 192 tiles: as many K ranges as make about 256 workgroups, each at least two stages long.
static KsplitPlan ksplit_plan(int64_t M, int64_t N, int64_t K, bool allow_split) {
  KsplitPlan p{M <= 64 ? 2 : 4, 2, 1, 0};
  if (M <= 64 && ceil_div(N, 128) >= 192) p.nj = 4;
  const int64_t tiles = ceil_div(M, 32 * p.mi) * ceil_div(N, 32 * p.nj), stages = K / KW_BK;
  int64_t splits = 1;
  if (allow_split) {
    if (const int f = g_forced_skinny_ks.load(std::memory_order_relaxed)) {  // forced length of a K range
      splits = K / f;
    } else if (tiles < 192) {
      splits = 256 / tiles;
      if (splits > stages / 2) splits = stages / 2;
      if (splits > 32) splits = 32;
    }
    if (splits < 1) splits = 1;
    if (splits > stages) splits = stages;
  }
  p.splits = (int)splits;
  p.partial_bytes = splits > 1 ? splits * M * N * 4 : 0;
  return p;
}

template <int D_DT, int BIAS_DT>
static int launch_ksplit(const LinearArgs &a, const KsplitPlan &p, const SplitK &sk, hipStream_t st) {
  if (p.mi == 4) return launch_ksplit_t<D_DT, BIAS_DT, 4, 2>(a, sk, st);
  return p.nj == 4 ? launch_ksplit_t<D_DT, BIAS_DT, 2, 4>(a, sk, st) : launch_ksplit_t<D_DT, BIAS_DT, 2, 2>(a, sk, st);
}

// ===========================================================================
// Decode-sized linear (1 <= M <= 32): bound by streaming the weights once.  Two kernels; this one
// streams the weights into registers, linear_nvfp4_stream_kernel below through an LDS ring, and
// skinny_plan chooses between them by shape.
//
// A workgroup (4 waves) owns 128 weight rows and one K-slice; every wave one 32-row tile.  It
// first decodes its slice of the packed activation to fp16 (exact, without the global scale)
// into LDS, shared by the four waves (with more than 16 activation rows, 512 k at a time, so that
// the LDS footprint stays at 33 KB).  Lane (row r, half h) streams 64 contiguous bytes of its weight row per 256-k step
// (elements [128h, 128h+128) of the step) and decodes them dword by dword into MFMA operands; the
// MFMA is issued as D^T = W . Ahat^T so a lane ends up with 4 consecutive n for one m.  K-slices of one row
// group meet through fp32 partial tiles in a caller-provided workspace; a small second kernel
// adds them in slice order (deterministic), applies gsA*gsB and the bias, converts and stores.
// (A last-arriver reduction inside the kernel needs device-scope fences, which write back the
// XCD's L2 and cost far more than the second launch.)
// Requires K % 256 == 0 and 16-byte aligned weights.
// ===========================================================================
struct SkinnyArgs {
  void *D;
  const uint8_t *Aq;         // packed activation [M, K/2] and its scale bytes [K/64, Mp, 4]
  const uint8_t *A_sf;
  int64_t Mp;
  const uint8_t *B;
  const uint32_t *B_sf;
  const float *A_gs, *B_gs;
  const void *bias;
  float *partial;      // [splitK][M][N]
  int64_t M, N, K, Np;
  int ks_len, split_k;
  int prepacked = 0;  // B is a weight image (LDS-ring kernel only), B_sf unused
};

constexpr int SK_ROWS = 128;   // weight rows per workgroup
constexpr int SK_STEP = 256;   // k per step

// MAX_IT: 16-byte activation vectors a lane may have to fetch (M * 32 / 256 rounded up): 1 for M <= 8, 2 for
// M <= 16, 4 for M <= 32.  With one accumulator tile (the MFMAs of a lane then queue behind each other, which a
// kernel that waits for memory does not notice) the two smaller variants fit four workgroups on a CU.
template <int D_DT, int BIAS_DT, int MAX_IT>
__global__ __launch_bounds__(256, MAX_IT <= 2 ? 4 : 3) void linear_nvfp4_skinny_kernel(SkinnyArgs a) {
  extern __shared__ __attribute__((aligned(16))) char slds[];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int r = lane & 31, h = lane >> 5;
  // K-slice is the fast grid index: workgroups that run together then read neighbouring pieces of the
  // same rows (all HBM channels), not the same 512-byte column of different rows (a few channels)
  const int ksl = blockIdx.x;
  const int64_t ng = blockIdx.y, n0 = ng * SK_ROWS + wave * 32;
  const int64_t kbeg = (int64_t)ksl * a.ks_len;
  const int nsteps = a.ks_len / SK_STEP;  // 1..4
  // With more than 16 activation rows a 1024-k slice goes through LDS in two halves of 512 k, which
  // keeps the slice at 33 KB and three workgroups on a CU.
  const bool halves = a.M > 16 && nsteps == 4;
  const int lds_k = halves ? 512 : a.ks_len;  // k positions held in LDS at a time
  const int pitch = lds_k * 2 + 16;       // LDS row pitch in bytes (16 bytes of padding: no bank conflicts)

  // activation slice -> LDS as its exact fp16 dequantization (without the global scale).  A thread
  // takes 32 elements (16 packed bytes, two 16-blocks) at a time; every load of the slice is issued
  // before the first decode, so the slice costs one memory latency whatever M is.
  // (the activation loads go out before the weight stream: the memory counter is in order, so loads
  // issued behind the stream could only be waited for together with all of it)
  const int vec_per_row = a.ks_len / 32;
  const int total = (int)a.M * vec_per_row;
  uint4 aw[MAX_IT];
  uint32_t ac[MAX_IT];
#pragma unroll
  for (int it = 0; it < MAX_IT; ++it) {
    const int i = it * 256 + tid;
    if (i < total) {
      const int m = i / vec_per_row, v = i % vec_per_row;
      const int64_t k = kbeg + v * 32;
      aw[it] = *reinterpret_cast<const uint4 *>(a.Aq + (int64_t)m * (a.K >> 1) + (k >> 1));
      // scale bytes of blocks (k/16) % 4 and the next one: k % 32 == 0, so an aligned pair
      ac[it] = *reinterpret_cast<const uint16_t *>(a.A_sf + (((k >> 6) * a.Mp + m) << 2) + ((k >> 4) & 3));
    }
  }
  // weight stream of this lane: all steps of the slice are requested up front
  int64_t wrow = n0 + r;
  wrow = wrow < a.N ? wrow : a.N - 1;  // rows past N feed outputs that are never stored
  const uint8_t *wp = a.B + wrow * (a.K >> 1) + (kbeg >> 1) + h * 64;
  const uint32_t *sp = a.B_sf + ((kbeg >> 6) + 2 * h) * a.Np + wrow;
  uint4 W[4][4];
  uint32_t S[4][2];
#pragma unroll
  for (int t = 0; t < 4; ++t) {
    if (t < nsteps) {
#pragma unroll
      for (int q = 0; q < 4; ++q) W[t][q] = *reinterpret_cast<const uint4 *>(wp + t * 128 + q * 16);  // cached: the four words share a line
      S[t][0] = sp[(int64_t)(t * 4) * a.Np];
      S[t][1] = sp[(int64_t)(t * 4 + 1) * a.Np];
    }
  }
  // decode of the activation slice (or of its half `part`), in the shadow of the weight loads
  auto decode_activation = [&](int part) {
#pragma unroll
    for (int it = 0; it < MAX_IT; ++it) {
      const int i = it * 256 + tid;
      if (i < total) {
        const int m = i / vec_per_row, v = i % vec_per_row;
        if (halves && (v >> 4) != part) continue;
        const f16x2 sc = __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(ac[it], 1.0f, false);
        f16x8 *dst = reinterpret_cast<f16x8 *>(slds + m * pitch + (halves ? v & 15 : v) * 64);
        dst[0] = decode_dword<false>(aw[it].x, sc);
        dst[1] = decode_dword<false>(aw[it].y, sc);
        dst[2] = decode_dword<true>(aw[it].z, sc);
        dst[3] = decode_dword<true>(aw[it].w, sc);
      }
    }
  };
  decode_activation(0);
  __syncthreads();

  f32x16 acc0;
#pragma unroll
  for (int e = 0; e < 16; ++e) acc0[e] = 0.0f;
  const int am = r < (int)a.M ? r : (int)a.M - 1;  // lanes past M read a valid row; their outputs are dropped
  const char *arow = slds + am * pitch + h * 256;
#pragma unroll
  for (int t = 0; t < 4; ++t) {
    if (t == 2 && halves) {  // second half of the slice replaces the first in LDS
      __syncthreads();
      decode_activation(1);
      __syncthreads();
    }
    if (t < nsteps) {
      f16x2 sc[2][2];  // [chunk][block pair] -> scales of blocks (0,1) and (2,3) of each 64-chunk
#pragma unroll
      for (int c = 0; c < 2; ++c) {
        sc[c][0] = __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(S[t][c], 1.0f, false);
        sc[c][1] = __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(S[t][c], 1.0f, true);
      }
#pragma unroll
      for (int q = 0; q < 4; ++q) {       // 16-byte word q: elements [32q, 32q+32) of the lane's 128
        const uint32_t w[4] = {W[t][q].x, W[t][q].y, W[t][q].z, W[t][q].w};
#pragma unroll
        for (int d = 0; d < 4; ++d) {     // dword d: elements [32q + 8d, +8): block (4q + d) / 2 of the lane
          const int blk = (4 * q + d) >> 1;   // 0..7: chunk blk/4, block blk%4
          const f16x2 pair = sc[blk >> 2][(blk & 3) >> 1];
          f16x8 wdec = (blk & 1) ? decode_dword<true>(w[d], pair) : decode_dword<false>(w[d], pair);
          const f16x8 afrag = *reinterpret_cast<const f16x8 *>(arow + (halves ? t & 1 : t) * 512 + (q * 4 + d) * 16);
          acc0 = __builtin_amdgcn_mfma_f32_32x32x16_f16(wdec, afrag, acc0, 0, 0, 0);
        }
      }
    }
  }

  // acc0: lane <-> m = r, element e <-> n = n0 + (e>>2)*8 + h*4 + (e&3): 4 consecutive n per group
  const int m = r;
  if (m >= (int)a.M) return;
  if (a.split_k > 1) {  // fp32 partial tile of this K-slice; skinny_reduce_kernel adds the slices
    float *pp = a.partial + ((int64_t)ksl * a.M + m) * a.N;
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      const int64_t n = n0 + g * 8 + h * 4;
      if (n + 3 < a.N && (a.N & 3) == 0) {
        *reinterpret_cast<float4 *>(pp + n) = make_float4(acc0[4 * g], acc0[4 * g + 1], acc0[4 * g + 2], acc0[4 * g + 3]);
      } else {
#pragma unroll
        for (int q = 0; q < 4; ++q)
          if (n + q < a.N) pp[n + q] = acc0[4 * g + q];
      }
    }
    return;
  }
  using DE = Elem<D_DT>;
  typename DE::T *Dp = static_cast<typename DE::T *>(a.D);
  const float scale = (*a.A_gs) * (*a.B_gs);
#pragma unroll
  for (int e = 0; e < 16; ++e) {
    const int64_t n = n0 + (e >> 2) * 8 + h * 4 + (e & 3);
    if (n < a.N) {
      float v = acc0[e] * scale;
      if constexpr (BIAS_DT != BIAS_NONE) v += Elem<BIAS_DT>::load(a.bias, n);
      Dp[(int64_t)m * a.N + n] = DE::cvt(v);
    }
  }
}

// D[m, n] = cvt( (sum over K-slices of partial[s][m][n]) * gsA*gsB + bias[n] ), slices added in order.
// V outputs per thread (V = 4: 16-byte loads; needs N % 4 == 0); the loads of eight slices are in
// flight together, the additions stay in slice order.
template <int D_DT, int BIAS_DT, int V>
__global__ __launch_bounds__(256) void skinny_reduce_kernel(SkinnyArgs a) {
  const int64_t i = ((int64_t)blockIdx.x * 256 + threadIdx.x) * V;
  const int64_t total = a.M * a.N;
  if (i >= total) return;
  float v[V];
#pragma unroll
  for (int q = 0; q < V; ++q) v[q] = 0.0f;
  const float *p = a.partial + i;
  int sidx = 0;
  for (; sidx + 8 <= a.split_k; sidx += 8) {
    float t[8][V];
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      if constexpr (V == 4) {
        const float4 f = *reinterpret_cast<const float4 *>(p + (int64_t)(sidx + u) * total);
        t[u][0] = f.x; t[u][1] = f.y; t[u][2] = f.z; t[u][3] = f.w;
      } else {
        t[u][0] = p[(int64_t)(sidx + u) * total];
      }
    }
#pragma unroll
    for (int u = 0; u < 8; ++u)
#pragma unroll
      for (int q = 0; q < V; ++q) v[q] += t[u][q];
  }
  for (; sidx < a.split_k; ++sidx) {
    if constexpr (V == 4) {
      const float4 f = *reinterpret_cast<const float4 *>(p + (int64_t)sidx * total);
      v[0] += f.x; v[1] += f.y; v[2] += f.z; v[3] += f.w;
    } else {
      v[0] += p[(int64_t)sidx * total];
    }
  }
  const float scale = (*a.A_gs) * (*a.B_gs);
  using DE = Elem<D_DT>;
  typename DE::T *D = static_cast<typename DE::T *>(a.D);
  const int64_t n = i % a.N;  // V consecutive outputs share a row (N % V == 0)
#pragma unroll
  for (int q = 0; q < V; ++q) {
    v[q] *= scale;
    if constexpr (BIAS_DT != BIAS_NONE) v[q] += Elem<BIAS_DT>::load(a.bias, n + q);
  }
  if constexpr (V == 4 && sizeof(typename DE::T) == 2) {
    *reinterpret_cast<uint2 *>(D + i) = make_uint2(DE::cvt2(v[0], v[1]), DE::cvt2(v[2], v[3]));
  } else if constexpr (V == 4) {
    *reinterpret_cast<float4 *>(D + i) = make_float4(v[0], v[1], v[2], v[3]);
  } else {
    D[i] = DE::cvt(v[0]);
  }
}

template <int D_DT, int BIAS_DT>
static void launch_reduce(const SkinnyArgs &a, hipStream_t st) {
  const int64_t total = a.M * a.N;
  const bool v4 = a.N % 4 == 0 && ((uintptr_t)a.D & 15) == 0 && ((uintptr_t)a.partial & 15) == 0;
  if (v4)
    hipLaunchKernelGGL((skinny_reduce_kernel<D_DT, BIAS_DT, 4>), dim3((unsigned)ceil_div(total / 4, 256)), dim3(256), 0, st, a);
  else
    hipLaunchKernelGGL((skinny_reduce_kernel<D_DT, BIAS_DT, 1>), dim3((unsigned)ceil_div(total, 256)), dim3(256), 0, st, a);
}

// ===========================================================================
// Decode-sized linear (1 <= M <= 32, K % 256 == 0): the weights are streamed once, through LDS.
//
// A workgroup (8 waves) owns 128 weight rows and a contiguous range of 256-k stages.  Weights, weight
// scales, the packed activation rows and their scales go from global memory straight into an LDS ring
// of six or seven stages with LDS-DMA loads: lane l of a transfer fetches piece l % 8 of row l / 8, so eight
// lanes read one 128-byte run of a row, and every request is a full 64-byte line.  (With loads into
// registers in the MFMA operand layout every lane reads from a different row: four times the address
// work per byte, and the partial sums of a K split on top; the same pattern with 16 bytes per lane, as a
// wave's fragment of one stage would need, measured 2 TB/s.)  Wave (wn, kh) = (wave % 4, wave / 4) takes
// weight rows 32 wn .. 32 wn + 31 and the 64-chunks 2 kh, 2 kh + 1 of every stage: its packed
// fragments of the NEXT stage travel from LDS to registers while it decodes the current ones in
// registers (weights and activation alike: 4 converts + 4 packed multiplies per 8 elements) and
// issues D^T += W . Xhat^T with v_mfma_f32_32x32x16_f16, so a lane ends up with four consecutive n for
// one m.  One workgroup barrier per stage: a stage costs about 0.45 us of barrier, transfer issue and
// waits whatever its size, which is why it is 256 k long (128-k stages: 40 us on N = 28672, K = 8192).
// The two k halves meet through LDS at the end, always added in the same order.  Activation rows past
// M read row M - 1 and feed outputs that are never stored.  With one K range per tile the epilogue
// applies gsA*gsB and the bias and stores D; with several (too few tiles to fill the GPU) the fp32
// sums go to the caller's workspace and skinny_reduce_kernel adds the ranges in order.
// ===========================================================================
constexpr int ST_BN = 128;        // weight rows per workgroup
constexpr int ST_THREADS = 512;
constexpr int ST_BK = 256;        // k per stage (four 64-chunks)
constexpr int ST_ROW = ST_BK / 2; // packed bytes per row per stage
constexpr int ST_NPIECES = 4;     // LDS-DMA instructions per wave per stage (three from a weight image)
// A stage: the weight rows, their scale dwords [chunk][128 rows], MR packed activation rows and their scale
// dwords [chunk][MR rows].  MR is 32, or 16 when M <= 16: the smaller stage leaves room for a seventh one
// in the ring, i.e. one more stage of weights in flight.
constexpr int ST_OFF_B = 0;
constexpr int ST_OFF_SFB = ST_OFF_B + ST_BN * ST_ROW;
constexpr int ST_OFF_A = ST_OFF_SFB + 4 * ST_BN * 4;  // 18432
__host__ __device__ constexpr int st_off_sfa(int mr) { return ST_OFF_A + mr * ST_ROW; }
__host__ __device__ constexpr int st_stage_bytes(int mr) { return st_off_sfa(mr) + 4 * mr * 4; }
__host__ __device__ constexpr int st_stages(int mr) { return mr == 32 ? 6 : 7; }
__host__ __device__ constexpr int st_lds_bytes(int mr) { return st_stages(mr) * st_stage_bytes(mr); }
static_assert(st_lds_bytes(32) <= 160 * 1024 && st_lds_bytes(16) <= 160 * 1024, "the ring must fit in the CU's LDS");
static_assert((st_stages(16) - 3) * ST_NPIECES <= 63, "the wait counts must fit the 6-bit counter");
static_assert(st_lds_bytes(16) >= 4 * 64 * 16 * 4, "the ring doubles as the exchange buffer of the two k halves");
// From a weight image (PRE) the weights and weight scales of a stage are ONE contiguous run of two blocks,
// copied as it lies to the head of the LDS stage by 18 one-kilobyte transfers; with the transfers of the
// activation rows and of their scales that is three per wave.  The activation part of the stage is the same.
constexpr int ST_PRE_W_BYTES = 2 * W_BLOCK_BYTES;  // 18432
static_assert(ST_PRE_W_BYTES == ST_OFF_A, "both layouts put the activation behind 18 KB of weights and scales");
constexpr int ST_PRE_NPIECES = 3;

// a wave's fragments of one stage: for each of its two 64-chunks (2 kh, 2 kh + 1) 32 packed elements
// of a weight row and of an activation row (the lane's half of the chunk) and the two block scales of each
struct StageFrags {
  uint4 w[2], x[2];
  uint32_t ws[2], xs[2];
};

// acc[c] += W . Xhat^T over the wave's two chunks of a stage (decode in registers)
__device__ __forceinline__ void stream_multiply(const StageFrags &cur, f32x16 (&acc)[2]) {
#pragma unroll
  for (int c = 0; c < 2; ++c) {
    const f16x2 wsc = __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(cur.ws[c], 1.0f, false);
    const f16x2 xsc = __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(cur.xs[c], 1.0f, false);
    acc[c] = __builtin_amdgcn_mfma_f32_32x32x16_f16(decode_dword<false>(cur.w[c].x, wsc), decode_dword<false>(cur.x[c].x, xsc), acc[c], 0, 0, 0);
    acc[c] = __builtin_amdgcn_mfma_f32_32x32x16_f16(decode_dword<false>(cur.w[c].y, wsc), decode_dword<false>(cur.x[c].y, xsc), acc[c], 0, 0, 0);
    acc[c] = __builtin_amdgcn_mfma_f32_32x32x16_f16(decode_dword<true>(cur.w[c].z, wsc), decode_dword<true>(cur.x[c].z, xsc), acc[c], 0, 0, 0);
    acc[c] = __builtin_amdgcn_mfma_f32_32x32x16_f16(decode_dword<true>(cur.w[c].w, wsc), decode_dword<true>(cur.x[c].w, xsc), acc[c], 0, 0, 0);
  }
}

// End of the LDS-ring kernels, after the last LDS-DMA has landed and every wave has passed a barrier:
// the two chunk sums of a wave, then the NK k parts of each of the NWN row groups (through `xch_base`,
// always in this order), then either the fp32 partial sums of this K range or the finished outputs
// (times gsA * gsB, plus bias).
template <int D_DT, int BIAS_DT, int NK = 2, int NWN = 4>
__device__ __forceinline__ void stream_finish(f32x16 (&acc)[2], const SkinnyArgs &a, char *xch_base, float gs_a, int wn, int kh,
                                              int lane, int64_t n0) {
  const int half = lane >> 5, r32 = lane & 31;
#pragma unroll
  for (int e = 0; e < 16; ++e) acc[0][e] += acc[1][e];
  // the NK k parts of a row group meet in the waves of part 0, added in the order of the parts
  if (kh != 0) {
    float4 *xch = reinterpret_cast<float4 *>(xch_base) + (((kh - 1) * NWN + wn) * 64 + lane) * 4;
#pragma unroll
    for (int g = 0; g < 4; ++g) xch[g] = make_float4(acc[0][4 * g], acc[0][4 * g + 1], acc[0][4 * g + 2], acc[0][4 * g + 3]);
  }
  __syncthreads();
  if (kh != 0) return;
#pragma unroll
  for (int k = 1; k < NK; ++k) {
    const float4 *xch = reinterpret_cast<const float4 *>(xch_base) + (((k - 1) * NWN + wn) * 64 + lane) * 4;
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      const float4 o = xch[g];
      acc[0][4 * g] += o.x; acc[0][4 * g + 1] += o.y; acc[0][4 * g + 2] += o.z; acc[0][4 * g + 3] += o.w;
    }
  }

  // acc: lane <-> m = r32, element e <-> n = (e >> 2) * 8 + half * 4 + (e & 3): four consecutive n per group
  const int m = r32;
  if (m >= (int)a.M) return;
  const int64_t nw = n0 + wn * 32;
  if (a.split_k > 1) {
    float *pp = a.partial + ((int64_t)blockIdx.y * a.M + m) * a.N;
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      const int64_t n = nw + g * 8 + half * 4;
      if (n + 3 < a.N && (a.N & 3) == 0) {
        *reinterpret_cast<float4 *>(pp + n) = make_float4(acc[0][4 * g], acc[0][4 * g + 1], acc[0][4 * g + 2], acc[0][4 * g + 3]);
      } else {
#pragma unroll
        for (int q = 0; q < 4; ++q)
          if (n + q < a.N) pp[n + q] = acc[0][4 * g + q];
      }
    }
    return;
  }
  using DE = Elem<D_DT>;
  typename DE::T *Dp = static_cast<typename DE::T *>(a.D);
  const float scale = gs_a * (*a.B_gs);
  // a lane's four consecutive outputs of a group leave as one 8- or 16-byte store where the rows allow it
  const bool vec_ok = (a.N & 3) == 0 && ((uintptr_t)a.D & 15) == 0;
#pragma unroll
  for (int g = 0; g < 4; ++g) {
    const int64_t n = nw + g * 8 + half * 4;
    float v[4];
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      v[q] = acc[0][4 * g + q] * scale;
      if constexpr (BIAS_DT != BIAS_NONE) v[q] += n + q < a.N ? Elem<BIAS_DT>::load(a.bias, n + q) : 0.0f;
    }
    typename DE::T *dst = Dp + (int64_t)m * a.N + n;
    if (vec_ok && n + 3 < a.N) {
      if constexpr (sizeof(typename DE::T) == 2)
        *reinterpret_cast<uint2 *>(dst) = make_uint2(DE::cvt2(v[0], v[1]), DE::cvt2(v[2], v[3]));
      else
        *reinterpret_cast<float4 *>(dst) = make_float4(v[0], v[1], v[2], v[3]);
    } else {
#pragma unroll
      for (int q = 0; q < 4; ++q)
        if (n + q < a.N) dst[q] = DE::cvt(v[q]);
    }
  }
}

template <int D_DT, int BIAS_DT, bool PRE, int MR>
__global__ __launch_bounds__(ST_THREADS, 1) void linear_nvfp4_stream_kernel(SkinnyArgs a) {
  static_assert(MR == 32 || MR == 16, "activation rows per stage");
  constexpr int NPIECES = PRE ? ST_PRE_NPIECES : ST_NPIECES;
  constexpr int OFF_A = ST_OFF_A, OFF_SFA = st_off_sfa(MR);
  constexpr int ST_PS = st_stages(MR), ST_STAGE_BYTES = st_stage_bytes(MR);
  extern __shared__ __attribute__((aligned(16))) char stlds[];
  const int tid = threadIdx.x, lane = tid & 63, half = lane >> 5, r32 = lane & 31;
  const int swave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wn = swave & 3, kh = swave >> 2;
  const int64_t n0 = (int64_t)blockIdx.x * ST_BN;
  const int nst_all = (int)(a.K / ST_BK);
  const int s0 = (int)((int64_t)nst_all * blockIdx.y / a.split_k);
  const int nst = (int)((int64_t)nst_all * (blockIdx.y + 1) / a.split_k) - s0;  // >= 1: split_k <= stages
  const int64_t kb = a.K >> 1;
  // Workgroup b walks its stages starting at stage b % nst and wraps around.  In step, every workgroup
  // would ask for the same 128-byte column of its rows at the same time; with a row pitch that is a
  // power of two (K = 8192: 4096 bytes) all those addresses fall on the same few memory channels.
  const int rot = (int)(blockIdx.x % (unsigned)nst);
  auto stage_of = [&](int step) {
    const int p = step + rot;
    return p >= nst ? p - nst : p;
  };

  // LDS holds row-major 128-byte rows (lane l of a transfer lands at 16 l: eight rows per transfer);
  // the eight 16-byte pieces of row r sit at positions piece ^ (r & 7), which spreads a fragment read
  // (one piece of each of 32 rows) over all LDS banks.  Unswizzled those reads fall on a quarter of the
  // banks and, issued by eight waves every stage, held the transfers back (40 us against 31 us on
  // N = 28672, K = 8192).
  // --- this wave's transfers of a stage: lane offsets (loop invariant), LDS destinations, sources
  const uint32_t lds_base = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) char *)stlds;
  // weights (and, from an image, their scales)
  uint32_t offW[3];
  const uint8_t *srcW;
  int64_t strideW;
  uint32_t ldsW;
  if constexpr (PRE) {
    // transfers 2 swave, 2 swave + 1 of the stage's 18 contiguous kilobytes; waves 0 and 1 also 16, 17
    offW[0] = (uint32_t)(swave * 2048 + lane * 16);
    offW[1] = offW[0] + 1024;
    offW[2] = (uint32_t)((16 + swave) * 1024 + lane * 16);
    strideW = ST_PRE_W_BYTES;
    srcW = uniform_ptr(a.B + ((int64_t)blockIdx.x * (a.K / W_BLOCK_K) + 2 * (int64_t)s0) * W_BLOCK_BYTES);
    ldsW = (uint32_t)__builtin_amdgcn_readfirstlane(swave * 2048);
  } else {
    // weight rows swave * 16 + {0..7}, {8..15}, 128 B each
#pragma unroll
    for (int q = 0; q < 2; ++q) {
      const int loc = swave * 16 + q * 8 + (lane >> 3);
      int64_t row = n0 + loc;
      row = row < a.N ? row : a.N - 1;  // rows past N read the last row; their outputs are never stored
      offW[q] = (uint32_t)((row - n0) * kb + ((lane & 7) ^ (loc & 7)) * 16);
    }
    offW[2] = 0;
    strideW = ST_ROW;
    srcW = uniform_ptr(a.B + n0 * kb + (int64_t)s0 * ST_ROW);
    ldsW = (uint32_t)__builtin_amdgcn_readfirstlane(ST_OFF_B + swave * 2048);
  }
  // weight scales from the scale tensor: chunk swave / 2, rows (swave % 2) * 64 + lane of the tile
  uint32_t offS = 0, ldsS = 0;
  int64_t strideS = 0;
  const uint8_t *srcS = nullptr;
  if constexpr (!PRE) {
    int64_t srow = n0 + (swave & 1) * 64 + lane;
    srow = srow < a.Np ? srow : a.Np - 1;
    offS = (uint32_t)(srow * 4);
    strideS = 4 * a.Np * 4;  // bytes per stage (four chunk planes)
    srcS = uniform_ptr(reinterpret_cast<const uint8_t *>(a.B_sf) + (int64_t)(swave >> 1) * a.Np * 4 + s0 * strideS);
    ldsS = (uint32_t)__builtin_amdgcn_readfirstlane(ST_OFF_SFB + (swave >> 1) * (ST_BN * 4) + (swave & 1) * 256);
  }
  // activation: MR / 8 waves take the packed rows w * 8 + {0..7}; the scale dwords are one transfer for
  // MR = 16 (lane = chunk x row) and two for MR = 32 (chunks 2 p + {0, 1}, p = 0, 1).  From an image waves
  // 0 and 1 have their third weight transfer first.  The waves left over repeat a scale transfer: every wave
  // issues the same count.
  constexpr int A_FIRST = PRE ? 2 : 0;  // first wave of those that move the rows
  constexpr int A_WAVES = MR / 8;
  const bool moves_rows = swave >= A_FIRST && swave < A_FIRST + A_WAVES;
  uint32_t off4 = 0, lds4 = 0;
  const uint8_t *src4 = nullptr;
  int64_t stride4 = 0;
  if (moves_rows) {
    const int loc = (swave - A_FIRST) * 8 + (lane >> 3);
    const int64_t row = loc < a.M ? loc : a.M - 1;  // rows past M read row M - 1; their outputs are never stored
    off4 = (uint32_t)(row * kb + ((lane & 7) ^ (loc & 7)) * 16);
    stride4 = ST_ROW;
    src4 = uniform_ptr(a.Aq + (int64_t)s0 * ST_ROW);
    lds4 = (uint32_t)__builtin_amdgcn_readfirstlane(OFF_A + (swave - A_FIRST) * 1024);
  } else if (!PRE || swave >= 2) {
    stride4 = 4 * a.Mp * 4;
    src4 = uniform_ptr(a.A_sf + s0 * stride4);
    if constexpr (MR == 32) {
      const int pair = swave & 1;  // chunks 2 pair, 2 pair + 1
      const int64_t row = r32 < a.Mp ? r32 : a.Mp - 1;
      off4 = (uint32_t)(((2 * pair + half) * a.Mp + row) * 4);
      lds4 = (uint32_t)__builtin_amdgcn_readfirstlane(OFF_SFA + pair * 256);
    } else {
      off4 = (uint32_t)(((lane >> 4) * a.Mp + (lane & 15)) * 4);  // Mp >= 16
      lds4 = (uint32_t)__builtin_amdgcn_readfirstlane(OFF_SFA);
    }
  }
  auto issue_stage = [&](int slot, int step) {  // step: position in this workgroup's order of stages
    const int st = stage_of(step);
    const uint32_t base = lds_base + slot * ST_STAGE_BYTES;
    const uint8_t *pw = srcW + (int64_t)st * strideW;
    dma16(pw, offW[0], base, ldsW);
    dma16(pw, offW[1], base, ldsW + 1024);
    if constexpr (PRE) {
      if (swave < 2)
        dma16(pw, offW[2], base, (uint32_t)__builtin_amdgcn_readfirstlane((16 + swave) * 1024));
      else if (moves_rows)
        dma16(src4 + st * stride4, off4, base, lds4);
      else
        dma4(src4 + st * stride4, off4, base, lds4);
    } else {
      dma4(srcS + st * strideS, offS, base, ldsS);
      if (moves_rows)
        dma16(src4 + st * stride4, off4, base, lds4);
      else
        dma4(src4 + st * stride4, off4, base, lds4);
    }
  };

  const int wrow_l = wn * 32 + r32;
  const int xrow = r32 & (MR - 1);  // lanes of rows past MR read a staged row; their outputs are never stored
  int wf_off[2], xf_off[2];
#pragma unroll
  for (int c = 0; c < 2; ++c) {
    const int piece = kh * 4 + c * 2 + half;
    if constexpr (PRE)  // block kh of the stage; 64-byte rows, piece p of a chunk pair at p ^ ((r >> 1) & 3)
      wf_off[c] = kh * W_BLOCK_BYTES + wrow_l * 64 + (((c * 2 + half) ^ ((wrow_l >> 1) & 3)) * 16);
    else
      wf_off[c] = ST_OFF_B + wrow_l * ST_ROW + ((piece ^ (wrow_l & 7)) * 16);
    xf_off[c] = OFF_A + xrow * ST_ROW + ((piece ^ (xrow & 7)) * 16);
  }
  // scale planes of the wave's two chunks: `ws_pitch` bytes apart
  constexpr int ws_pitch = PRE ? W_BLOCK_ROWS * 4 : ST_BN * 4;
  const int ws_off = (PRE ? kh * W_BLOCK_BYTES + W_BLOCK_DATA : ST_OFF_SFB + (kh * 2) * (ST_BN * 4)) + wrow_l * 4 + half * 2;
  const int xs_off = OFF_SFA + (kh * 2) * (MR * 4) + xrow * 4 + half * 2;
  auto load_frags = [&](int slot) {
    const char *st = stlds + slot * ST_STAGE_BYTES;
    StageFrags f;
#pragma unroll
    for (int c = 0; c < 2; ++c) {
      f.w[c] = *reinterpret_cast<const uint4 *>(st + wf_off[c]);
      f.x[c] = *reinterpret_cast<const uint4 *>(st + xf_off[c]);
      f.ws[c] = *reinterpret_cast<const uint16_t *>(st + ws_off + c * ws_pitch);
      f.xs[c] = *reinterpret_cast<const uint16_t *>(st + xs_off + c * (MR * 4));
    }
    return f;
  };

  f32x16 acc[2];  // one per chunk of the pair: two independent accumulation chains
#pragma unroll
  for (int c = 0; c < 2; ++c)
#pragma unroll
    for (int e = 0; e < 16; ++e) acc[c][e] = 0.0f;

  // prologue: stages 0 .. PS-2 in flight (past the range: the last stage again, into slots nobody
  // reads), stages 0 and 1 landed, fragments of stage 0 in registers
  const int last = nst - 1;
#pragma unroll
  for (int d = 0; d < ST_PS - 1; ++d) issue_stage(d, d < last ? d : last);
  wait_vmcnt<(ST_PS - 3) * NPIECES>();
  __syncthreads();
  StageFrags cur = load_frags(0);

  int slot_next = 1, slot_dma = ST_PS - 1;
  for (int s = 0; s < nst; ++s) {
    // fragments of the next stage (it landed before the previous barrier) travel from LDS while this
    // stage is decoded and multiplied (past the range: a stage nobody uses)
    const StageFrags nxt = load_frags(slot_next);
    stream_multiply(cur, acc);
    // refill the slot of the stage before this one (everybody read it before the previous barrier)
    const int sd = s + ST_PS - 1;
    issue_stage(slot_dma, sd < last ? sd : last);
    wait_vmcnt<(ST_PS - 3) * NPIECES>();  // own transfers of stage s + 2 have landed
    __syncthreads();
    cur = nxt;
    slot_next = slot_next + 1 == ST_PS ? 0 : slot_next + 1;
    slot_dma = slot_dma + 1 == ST_PS ? 0 : slot_dma + 1;
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // no LDS-DMA may land after this point: the ring is reused
  __syncthreads();
  stream_finish<D_DT, BIAS_DT>(acc, a, stlds, *a.A_gs, wn, kh, lane, n0);
}

// ===========================================================================
// The LDS-ring kernel with 64 weight rows per workgroup, for weights with so few rows that 128-row
// tiles leave CUs idle or force a K split with partial sums and a second launch (N = 14336: 112
// tiles of 128 rows, 224 of 64).  Same ring, swizzle, stage order and arithmetic; wave (wn, kq) =
// (wave % 2, wave / 2) takes weight rows 32 wn .. 32 wn + 31 and chunk kq of every stage, and the four
// k parts of a row group meet through LDS at the end.  A stage is 13.5 KB (64 weight rows, 32
// activation rows, their scales), ten of them make the ring; three transfers per wave per stage.
// Plain layout only.
// ===========================================================================
constexpr int S6_BN = 64;
constexpr int S6_PS = 10;
constexpr int S6_NPIECES = 3;
constexpr int S6_OFF_B = 0;
constexpr int S6_OFF_A = S6_OFF_B + S6_BN * ST_ROW;      // 32 packed activation rows
constexpr int S6_OFF_SFB = S6_OFF_A + 32 * ST_ROW;       // weight scale dwords [chunk][64 rows]
constexpr int S6_OFF_SFA = S6_OFF_SFB + 4 * S6_BN * 4;   // activation scale dwords [chunk][32 rows]
constexpr int S6_STAGE_BYTES = S6_OFF_SFA + 4 * 32 * 4;  // 13824
constexpr int S6_LDS_BYTES = S6_PS * S6_STAGE_BYTES;
static_assert(S6_LDS_BYTES <= 160 * 1024, "the ring must fit in the CU's LDS");
static_assert((S6_PS - 3) * S6_NPIECES <= 63, "the wait counts must fit the 6-bit counter");
static_assert(S6_LDS_BYTES >= 3 * 2 * 64 * 16 * 4, "the ring doubles as the exchange buffer of the four k parts");

template <int D_DT, int BIAS_DT>
__global__ __launch_bounds__(ST_THREADS, 1) void linear_nvfp4_stream64_kernel(SkinnyArgs a) {
  extern __shared__ __attribute__((aligned(16))) char stlds[];
  const int tid = threadIdx.x, lane = tid & 63, half = lane >> 5, r32 = lane & 31;
  const int swave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wn = swave & 1, kq = swave >> 1;
  const int64_t n0 = (int64_t)blockIdx.x * S6_BN;
  const int nst_all = (int)(a.K / ST_BK);
  const int s0 = (int)((int64_t)nst_all * blockIdx.y / a.split_k);
  const int nst = (int)((int64_t)nst_all * (blockIdx.y + 1) / a.split_k) - s0;  // >= 1: split_k <= stages
  const int64_t kb = a.K >> 1;
  const int rot = (int)(blockIdx.x % (unsigned)nst);  // stages are walked from stage b % nst on (see linear_nvfp4_stream_kernel)
  auto stage_of = [&](int step) {
    const int p = step + rot;
    return p >= nst ? p - nst : p;
  };
  const uint32_t lds_base = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) char *)stlds;
  // (1) weight rows swave * 8 + {0..7}, 128 B each, piece p of row r at position p ^ (r & 7)
  uint32_t offW;
  {
    const int loc = swave * 8 + (lane >> 3);
    int64_t row = n0 + loc;
    row = row < a.N ? row : a.N - 1;  // rows past N read the last row; their outputs are never stored
    offW = (uint32_t)((row - n0) * kb + ((lane & 7) ^ (loc & 7)) * 16);
  }
  const uint8_t *srcW = uniform_ptr(a.B + n0 * kb + (int64_t)s0 * ST_ROW);
  const uint32_t ldsW = (uint32_t)__builtin_amdgcn_readfirstlane(S6_OFF_B + swave * 1024);
  // (2) waves 0..3: weight scale dwords of chunk swave, rows n0 + lane; waves 4..7: packed activation
  //     rows (swave - 4) * 8 + {0..7}
  uint32_t off2, lds2;
  const uint8_t *src2;
  int64_t stride2;
  if (swave < 4) {
    int64_t srow = n0 + lane;
    srow = srow < a.Np ? srow : a.Np - 1;
    off2 = (uint32_t)(srow * 4);
    stride2 = 4 * a.Np * 4;  // bytes per stage (four chunk planes)
    src2 = uniform_ptr(reinterpret_cast<const uint8_t *>(a.B_sf) + (int64_t)swave * a.Np * 4 + s0 * stride2);
    lds2 = (uint32_t)__builtin_amdgcn_readfirstlane(S6_OFF_SFB + swave * (S6_BN * 4));
  } else {
    const int loc = (swave - 4) * 8 + (lane >> 3);
    const int64_t row = loc < a.M ? loc : a.M - 1;  // rows past M read row M - 1; their outputs are never stored
    off2 = (uint32_t)(row * kb + ((lane & 7) ^ (loc & 7)) * 16);
    stride2 = ST_ROW;
    src2 = uniform_ptr(a.Aq + (int64_t)s0 * ST_ROW);
    lds2 = (uint32_t)__builtin_amdgcn_readfirstlane(S6_OFF_A + (swave - 4) * 1024);
  }
  // (3) activation scales of chunks 2 p + {0, 1}, p = swave % 2 (waves 2..7 repeat the transfers of waves
  //     0 and 1: every wave issues the same count)
  const int pair = swave & 1;
  const int64_t arow = r32 < a.Mp ? r32 : a.Mp - 1;
  const uint32_t off3 = (uint32_t)(((2 * pair + half) * a.Mp + arow) * 4);
  const int64_t stride3 = 4 * a.Mp * 4;
  const uint8_t *src3 = uniform_ptr(a.A_sf + s0 * stride3);
  const uint32_t lds3 = (uint32_t)__builtin_amdgcn_readfirstlane(S6_OFF_SFA + pair * 256);
  auto issue_stage = [&](int slot, int step) {  // step: position in this workgroup's order of stages
    const int st = stage_of(step);
    const uint32_t base = lds_base + slot * S6_STAGE_BYTES;
    dma16(srcW + (int64_t)st * ST_ROW, offW, base, ldsW);
    if (swave < 4)
      dma4(src2 + st * stride2, off2, base, lds2);
    else
      dma16(src2 + st * stride2, off2, base, lds2);
    dma4(src3 + st * stride3, off3, base, lds3);
  };

  // this wave's fragments of a stage: chunk kq, 32 packed elements of a weight row and of an activation
  // row (the lane's half of the chunk) and the two block scales of each
  struct Frags {
    uint4 w, x;
    uint32_t ws, xs;
  };
  const int wrow_l = wn * 32 + r32;
  const int piece = kq * 2 + half;
  const int wf_off = S6_OFF_B + wrow_l * ST_ROW + ((piece ^ (wrow_l & 7)) * 16);
  const int xf_off = S6_OFF_A + r32 * ST_ROW + ((piece ^ (r32 & 7)) * 16);
  const int ws_off = S6_OFF_SFB + kq * (S6_BN * 4) + wrow_l * 4 + half * 2;
  const int xs_off = S6_OFF_SFA + kq * (32 * 4) + r32 * 4 + half * 2;
  auto load_frags = [&](int slot) {
    const char *st = stlds + slot * S6_STAGE_BYTES;
    Frags f;
    f.w = *reinterpret_cast<const uint4 *>(st + wf_off);
    f.x = *reinterpret_cast<const uint4 *>(st + xf_off);
    f.ws = *reinterpret_cast<const uint16_t *>(st + ws_off);
    f.xs = *reinterpret_cast<const uint16_t *>(st + xs_off);
    return f;
  };

  f32x16 acc[2];  // two independent accumulation chains: the first and the second half of the chunk
#pragma unroll
  for (int c = 0; c < 2; ++c)
#pragma unroll
    for (int e = 0; e < 16; ++e) acc[c][e] = 0.0f;

  const int last = nst - 1;
#pragma unroll
  for (int d = 0; d < S6_PS - 1; ++d) issue_stage(d, d < last ? d : last);
  wait_vmcnt<(S6_PS - 3) * S6_NPIECES>();
  __syncthreads();
  Frags cur = load_frags(0);

  int slot_next = 1, slot_dma = S6_PS - 1;
  for (int s = 0; s < nst; ++s) {
    const Frags nxt = load_frags(slot_next);  // it landed before the previous barrier
    const f16x2 wsc = __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(cur.ws, 1.0f, false);
    const f16x2 xsc = __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(cur.xs, 1.0f, false);
    acc[0] = __builtin_amdgcn_mfma_f32_32x32x16_f16(decode_dword<false>(cur.w.x, wsc), decode_dword<false>(cur.x.x, xsc), acc[0], 0, 0, 0);
    acc[0] = __builtin_amdgcn_mfma_f32_32x32x16_f16(decode_dword<false>(cur.w.y, wsc), decode_dword<false>(cur.x.y, xsc), acc[0], 0, 0, 0);
    acc[1] = __builtin_amdgcn_mfma_f32_32x32x16_f16(decode_dword<true>(cur.w.z, wsc), decode_dword<true>(cur.x.z, xsc), acc[1], 0, 0, 0);
    acc[1] = __builtin_amdgcn_mfma_f32_32x32x16_f16(decode_dword<true>(cur.w.w, wsc), decode_dword<true>(cur.x.w, xsc), acc[1], 0, 0, 0);
    const int sd = s + S6_PS - 1;
    issue_stage(slot_dma, sd < last ? sd : last);
    wait_vmcnt<(S6_PS - 3) * S6_NPIECES>();  // own transfers of stage s + 2 have landed
    __syncthreads();
    cur = nxt;
    slot_next = slot_next + 1 == S6_PS ? 0 : slot_next + 1;
    slot_dma = slot_dma + 1 == S6_PS ? 0 : slot_dma + 1;
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // no LDS-DMA may land after this point: the ring is reused
  __syncthreads();
  stream_finish<D_DT, BIAS_DT, 4, 2>(acc, a, stlds, *a.A_gs, wn, kq, lane, n0);
}

// Plan of a decode-sized linear: which of the two kernels, its K split and the fp32 scratch it needs.
enum { DECODE_REGISTERS = 1, DECODE_LDS_RING = 2, DECODE_LDS_RING64 = 3 };
struct SkinnyPlan {
  int kind;                // DECODE_REGISTERS: linear_nvfp4_skinny_kernel; DECODE_LDS_RING: linear_nvfp4_stream_kernel;
                           // DECODE_LDS_RING64: linear_nvfp4_stream64_kernel
  int ks_len;              // register kernel: k per workgroup (256, 512 or 1024)
  int split_k;             // K ranges; > 1 needs `partial_bytes` of fp32 scratch
  int64_t partial_bytes, groups;
  int lds_bytes;
};
static std::atomic<int> g_forced_decode_kernel{0};  // ac4k_set_linear_tuning: 0 = by shape

// Register kernel: K slices of up to 1024, halved until about 768 workgroups are in flight.
static void plan_registers(int64_t M, int64_t N, int64_t K, SkinnyPlan &p) {
  int ks = 1024;
  const int f = g_forced_skinny_ks.load(std::memory_order_relaxed);
  if (f == 256 || f == 512 || f == 1024) ks = f;
  while (ks > SK_STEP && K % ks != 0) ks >>= 1;
  p.kind = DECODE_REGISTERS;
  p.groups = ceil_div(N, SK_ROWS);
  // short problems: use smaller slices to get enough workgroups in flight
  while (ks > SK_STEP && p.groups * (K / ks) < 768) ks >>= 1;
  p.ks_len = ks;
  p.split_k = (int)(K / ks);
  p.partial_bytes = p.split_k > 1 ? (int64_t)p.split_k * M * N * 4 : 0;
  p.lds_bytes = (int)M * ((M > 16 && ks == 1024 ? 512 : ks) * 2 + 16);
}

// LDS-ring kernel: one K range per 128-row tile when the tiles alone fill the GPU; otherwise the
// smallest number of ranges that gives about 200 workgroups, each range at least two stages long.
static void plan_lds_ring(int64_t M, int64_t N, int64_t K, SkinnyPlan &p, int rows = ST_BN) {
  p.kind = rows == ST_BN ? DECODE_LDS_RING : DECODE_LDS_RING64;
  p.groups = ceil_div(N, rows);
  const int64_t stages = K / ST_BK;
  int64_t splits = 1;
  if (const int f = g_forced_skinny_ks.load(std::memory_order_relaxed)) {  // forced length of a K range
    splits = K / f;
  } else if (p.groups < 192) {
    splits = ceil_div(200, p.groups);
    if (splits > stages / 2) splits = stages / 2;
    if (splits > 32) splits = 32;
  }
  if (splits < 1) splits = 1;
  if (splits > stages) splits = stages;
  p.ks_len = 0;
  p.split_k = (int)splits;
  p.partial_bytes = splits > 1 ? splits * M * N * 4 : 0;
  p.lds_bytes = rows == ST_BN ? st_lds_bytes(M <= 16 ? 16 : 32) : S6_LDS_BYTES;
}

// Shapes of the decode-sized kernels (all need K % 256 == 0) and the choice between them.  The
// register kernel has all its loads in flight at once and four workgroups per CU, which wins while M
// is small and the problem needs a K split anyway (few row tiles, long K); it pays for partial sums
// and a second launch, and its registers run out as M grows.  The LDS-ring kernels take nearly the
// same time for every M <= 32 and need no second launch when their row tiles alone fill the GPU:
// 128-row tiles when there are 192 of them, 64-row tiles for narrower weights.
// Measured on one box, linear alone, weights from HBM, register / ring 128 / ring 64 in us:
//   N = 28672, K = 8192 (224 / 448 tiles):  M = 1 31.0 / 32.4 / 41.3, M = 8 35.1 / 33.6 / 41.6, M = 16 40.4 / 35.5 / 42.7, M = 32 45.5 / 37.3 / 44.3
//   N = 14336, K = 4096 (112 / 224 tiles):  M = 1 14.0 / 15.5 / 13.8, M = 8 14.5 / 15.8 / 14.2, M = 16 17.6 / 16.4 / 13.9, M = 32 22.1 / 17.2 / 14.9
//   N = 4096, K = 14336 (32 / 64 tiles):    M = 1 15.1 / 16.8 / 16.2, M = 8 16.3 / 17.3 / 16.3, M = 16 18.7 / 17.5 / 16.9, M = 32 22.9 / 17.8 / 17.1
// Hence: with 192 tiles of 128 rows and more, 128-row tiles from M = 8 on; otherwise 64-row tiles when
// there are 192 of those, or from M = 8 on; the register kernel in the remaining cases.
static bool skinny_plan(int64_t M, int64_t N, int64_t K, SkinnyPlan &p) {
  if (M < 1 || M > 32 || K < SK_STEP || K % SK_STEP != 0 || N < 1) return false;
  const bool ring_ok = (K >> 1) * ST_BN < (1ll << 31) && N < (1ll << 27);  // 32-bit lane offsets
  int kind = g_forced_decode_kernel.load(std::memory_order_relaxed);
  if (kind == 0) {
    if (ceil_div(N, ST_BN) >= 192)
      kind = M >= 8 ? DECODE_LDS_RING : DECODE_REGISTERS;
    else
      kind = (M >= 8 || ceil_div(N, S6_BN) >= 192) ? DECODE_LDS_RING64 : DECODE_REGISTERS;
  }
  if (kind == DECODE_LDS_RING64 && ring_ok)
    plan_lds_ring(M, N, K, p, S6_BN);
  else if (kind == DECODE_LDS_RING && ring_ok)
    plan_lds_ring(M, N, K, p);
  else
    plan_registers(M, N, K, p);
  return true;
}

template <int D_DT, int BIAS_DT, int MAX_IT>
static int launch_skinny_it(const SkinnyArgs &a, const SkinnyPlan &p, hipStream_t st) {
  auto *kern = linear_nvfp4_skinny_kernel<D_DT, BIAS_DT, MAX_IT>;
  static std::atomic<uint32_t> lds_ok{0};
  if (int rc = allow_dynamic_lds(kern, lds_ok, 32 * (1024 * 2 + 16))) return rc;
  hipLaunchKernelGGL(kern, dim3((unsigned)p.split_k, (unsigned)p.groups), dim3(256), p.lds_bytes, st, a);
  return 0;
}

template <int D_DT, int BIAS_DT, bool PRE, int MR>
static int launch_ring(const SkinnyArgs &a, const SkinnyPlan &p, hipStream_t st) {
  auto *kern = linear_nvfp4_stream_kernel<D_DT, BIAS_DT, PRE, MR>;
  static std::atomic<uint32_t> lds_ok{0};
  if (int rc = allow_dynamic_lds(kern, lds_ok, st_lds_bytes(MR))) return rc;
  hipLaunchKernelGGL(kern, dim3((unsigned)p.groups, (unsigned)p.split_k), dim3(ST_THREADS), st_lds_bytes(MR), st, a);
  return 0;
}

template <int D_DT, int BIAS_DT>
static int launch_skinny(const SkinnyArgs &a, const SkinnyPlan &p, hipStream_t st) {
  if (p.kind == DECODE_LDS_RING) {
    int rc;
    if (a.M <= 16)
      rc = a.prepacked ? launch_ring<D_DT, BIAS_DT, true, 16>(a, p, st) : launch_ring<D_DT, BIAS_DT, false, 16>(a, p, st);
    else
      rc = a.prepacked ? launch_ring<D_DT, BIAS_DT, true, 32>(a, p, st) : launch_ring<D_DT, BIAS_DT, false, 32>(a, p, st);
    if (rc) return rc;
  } else if (p.kind == DECODE_LDS_RING64) {
    auto *kern = linear_nvfp4_stream64_kernel<D_DT, BIAS_DT>;
    static std::atomic<uint32_t> lds_ok{0};
    if (int rc = allow_dynamic_lds(kern, lds_ok, S6_LDS_BYTES)) return rc;
    hipLaunchKernelGGL(kern, dim3((unsigned)p.groups, (unsigned)p.split_k), dim3(ST_THREADS), S6_LDS_BYTES, st, a);
  } else {
    int rc;
    if (a.M <= 8) rc = launch_skinny_it<D_DT, BIAS_DT, 1>(a, p, st);
    else if (a.M <= 16) rc = launch_skinny_it<D_DT, BIAS_DT, 2>(a, p, st);
    else rc = launch_skinny_it<D_DT, BIAS_DT, 4>(a, p, st);
    if (rc) return rc;
  }
  if (p.split_k > 1) launch_reduce<D_DT, BIAS_DT>(a, st);
  return 0;
}

template <int D_DT>
static int dispatch_skinny_bias(const SkinnyArgs &a, const SkinnyPlan &p, int bias_dtype, hipStream_t st) {
  if (!a.bias) return launch_skinny<D_DT, BIAS_NONE>(a, p, st);
  switch (bias_dtype) {
    case AC4K_DTYPE_BF16: return launch_skinny<D_DT, AC4K_DTYPE_BF16>(a, p, st);
    case AC4K_DTYPE_FP16: return launch_skinny<D_DT, AC4K_DTYPE_FP16>(a, p, st);
    case AC4K_DTYPE_FP32: return launch_skinny<D_DT, AC4K_DTYPE_FP32>(a, p, st);
  }
  return set_error("bias must be bfloat16, half or float (dtype tag %d)", bias_dtype);
}

static int dispatch_skinny(const SkinnyArgs &a, const SkinnyPlan &p, int d_dtype, int bias_dtype, hipStream_t st) {
  switch (d_dtype) {
    case AC4K_DTYPE_BF16: return dispatch_skinny_bias<AC4K_DTYPE_BF16>(a, p, bias_dtype, st);
    case AC4K_DTYPE_FP16: return dispatch_skinny_bias<AC4K_DTYPE_FP16>(a, p, bias_dtype, st);
    case AC4K_DTYPE_FP32: return dispatch_skinny_bias<AC4K_DTYPE_FP32>(a, p, bias_dtype, st);
  }
  return set_error("d must be bfloat16, half or float (dtype tag %d)", d_dtype);
}

// shapes the packed-LDS kernel takes: whole 128-k stages, 16-byte aligned rows, 32-bit lane offsets
// (256 operand rows in the loop, 4 output rows of up to 4-byte elements in the epilogue)
static bool packed_kernel_ok(const LinearArgs &a) {
  return a.K % P_BK == 0 && (((uintptr_t)a.A | (uintptr_t)a.B) & 15) == 0 && (a.K >> 1) * 256 < (1ll << 31) &&
         a.N < (1ll << 27);
}

// Decode-sized shapes through the entry point that has no scratch: the plan of the workspace entry point
// when it needs none (one K range), otherwise the LDS-ring kernel with one K range per tile - fewer
// workgroups than the split plan, still the weights streamed once instead of the 128x128 tile kernel.
static bool noscratch_skinny_plan(const LinearArgs &a, SkinnyPlan &p) {
  if (!skinny_plan(a.M, a.N, a.K, p) || (((uintptr_t)a.A | (uintptr_t)a.B) & 15) != 0) return false;
  if (p.partial_bytes == 0) return true;
  if (!((a.K >> 1) * ST_BN < (1ll << 31) && a.N < (1ll << 27))) return false;  // the ring kernels' 32-bit lane offsets
  p.kind = ceil_div(a.N, ST_BN) >= 192 ? DECODE_LDS_RING : DECODE_LDS_RING64;
  p.groups = ceil_div(a.N, p.kind == DECODE_LDS_RING ? ST_BN : S6_BN);
  p.ks_len = 0;
  p.split_k = 1;
  p.partial_bytes = 0;
  p.lds_bytes = p.kind == DECODE_LDS_RING ? st_lds_bytes(a.M <= 16 ? 16 : 32) : S6_LDS_BYTES;
  return true;
}

// Decode-sized M goes to the weight-streaming kernels, 32 < M <= 128 to the K-split-waves kernel, larger
// M to the packed-operand tile kernel, each whenever its layout conditions hold; the 128x128 kernel,
// which has no condition beyond K % 64 == 0, takes everything else.
template <int D_DT, int BIAS_DT>
static int launch_linear(const LinearArgs &a, hipStream_t st) {
  SkinnyPlan sp;
  if (noscratch_skinny_plan(a, sp)) {
    const SkinnyArgs sa{a.D, a.A, reinterpret_cast<const uint8_t *>(a.A_sf), a.Mp, a.B, a.B_sf, a.A_gs, a.B_gs, a.bias, nullptr,
                        a.M, a.N, a.K, a.Np, sp.ks_len, sp.split_k};
    return launch_skinny<D_DT, BIAS_DT>(sa, sp, st);
  }
  if (ksplit_shape(a.M, a.N, a.K) && ksplit_aligned(a))  // all of M in one tile, one K range (no scratch here)
    return launch_ksplit<D_DT, BIAS_DT>(a, ksplit_plan(a.M, a.N, a.K, false), SplitK{nullptr, 1}, st);
  if (a.M > 32 && a.N >= 128 && packed_kernel_ok(a)) return launch_tile256p<D_DT, BIAS_DT>(a, st);
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

namespace ac4k {

// Split-K for problems with too few output tiles to fill the GPU (32 < M, few tiles, long K): the
// K-split-waves kernel (M <= 128) or the packed-LDS tile kernel runs `splits` K ranges per tile into
// fp32 partial buffers in the workspace and skinny_reduce_kernel adds them.
struct MidPlan {
  bool has_ksplit;   // the shape suits the K-split-waves kernel (taken when the pointers are aligned for it)
  KsplitPlan kp;
  TilePlan tp;       // what the tile kernel does with the shape otherwise (given enough scratch)
  int64_t bytes;     // scratch of the preferred choice
};
// shapes the workspace entry point takes with 32 < M
static bool mid_plan(int64_t M, int64_t N, int64_t K, MidPlan &p) {
  if (M <= 32 || N < 128 || K % P_BK != 0 || (K >> 1) * 256 >= (1ll << 31) || N >= (1ll << 27)) return false;
  p.tp = tile_plan(M, N, K, true);
  p.has_ksplit = ksplit_shape(M, N, K);
  p.kp = p.has_ksplit ? ksplit_plan(M, N, K, true) : KsplitPlan{0, 0, 1, 0};
  p.bytes = p.has_ksplit ? p.kp.partial_bytes : p.tp.partial_bytes;
  return p.has_ksplit || p.tp.splits > 1;
}

// `partial_bytes` of scratch at `partial` (possibly none): the K-split-waves kernel when the shape and the
// pointers suit it, else the tile kernel, split along K when the scratch holds its partial sums
template <int D_DT, int BIAS_DT>
static int launch_mid(const LinearArgs &a, const MidPlan &p, float *partial, int64_t partial_bytes, hipStream_t st) {
  int splits;
  if (p.has_ksplit && ksplit_aligned(a)) {
    splits = p.kp.splits;
    if (int rc = launch_ksplit<D_DT, BIAS_DT>(a, p.kp, SplitK{splits > 1 ? partial : nullptr, splits}, st)) return rc;
  } else {
    const TilePlan tp = p.tp.partial_bytes <= partial_bytes ? p.tp : tile_plan(a.M, a.N, a.K, false);
    splits = tp.splits;
    if (int rc = launch_tile_plan<D_DT, BIAS_DT>(a, tp, SplitK{splits > 1 ? partial : nullptr, splits}, st)) return rc;
  }
  if (splits > 1) {
    SkinnyArgs r{a.D, nullptr, nullptr, 0, nullptr, nullptr, a.A_gs, a.B_gs, a.bias, partial, a.M, a.N, a.K, a.Np, 0, splits};
    launch_reduce<D_DT, BIAS_DT>(r, st);
  }
  return 0;
}

template <int D_DT>
static int dispatch_mid_bias(const LinearArgs &a, const MidPlan &p, float *partial, int64_t partial_bytes, int bias_dtype,
                             hipStream_t st) {
  if (!a.bias) return launch_mid<D_DT, BIAS_NONE>(a, p, partial, partial_bytes, st);
  switch (bias_dtype) {
    case AC4K_DTYPE_BF16: return launch_mid<D_DT, AC4K_DTYPE_BF16>(a, p, partial, partial_bytes, st);
    case AC4K_DTYPE_FP16: return launch_mid<D_DT, AC4K_DTYPE_FP16>(a, p, partial, partial_bytes, st);
    case AC4K_DTYPE_FP32: return launch_mid<D_DT, AC4K_DTYPE_FP32>(a, p, partial, partial_bytes, st);
  }
  return set_error("bias must be bfloat16, half or float (dtype tag %d)", bias_dtype);
}

static int dispatch_mid(const LinearArgs &a, const MidPlan &p, float *partial, int64_t partial_bytes, int d_dtype,
                        int bias_dtype, hipStream_t st) {
  switch (d_dtype) {
    case AC4K_DTYPE_BF16: return dispatch_mid_bias<AC4K_DTYPE_BF16>(a, p, partial, partial_bytes, bias_dtype, st);
    case AC4K_DTYPE_FP16: return dispatch_mid_bias<AC4K_DTYPE_FP16>(a, p, partial, partial_bytes, bias_dtype, st);
    case AC4K_DTYPE_FP32: return dispatch_mid_bias<AC4K_DTYPE_FP32>(a, p, partial, partial_bytes, bias_dtype, st);
  }
  return set_error("d must be bfloat16, half or float (dtype tag %d)", d_dtype);
}

// one K range of the tile kernel with a given plan (the entry point of the weight image)
template <int D_DT>
static int dispatch_prepacked_bias(const LinearArgs &a, const TilePlan &p, int bias_dtype, hipStream_t st) {
  const SplitK one{nullptr, 1};
  if (!a.bias) return launch_tile_plan<D_DT, BIAS_NONE>(a, p, one, st);
  switch (bias_dtype) {
    case AC4K_DTYPE_BF16: return launch_tile_plan<D_DT, AC4K_DTYPE_BF16>(a, p, one, st);
    case AC4K_DTYPE_FP16: return launch_tile_plan<D_DT, AC4K_DTYPE_FP16>(a, p, one, st);
    case AC4K_DTYPE_FP32: return launch_tile_plan<D_DT, AC4K_DTYPE_FP32>(a, p, one, st);
  }
  return set_error("bias must be bfloat16, half or float (dtype tag %d)", bias_dtype);
}

// shared tail of the two decode-sized entry points: packed activation in, partial sums in the workspace
static int run_skinny(void *D, int d_dtype, const void *Aq, const void *A_sf, const float *A_gs, const void *B,
                      const void *B_sf, const float *B_gs, const void *bias, int bias_dtype, int64_t M, int64_t N,
                      int64_t K, const SkinnyPlan &p, void *workspace, hipStream_t st) {
  SkinnyArgs a{D,
               static_cast<const uint8_t *>(Aq),
               static_cast<const uint8_t *>(A_sf),
               align_up(M, 16),
               static_cast<const uint8_t *>(B),
               static_cast<const uint32_t *>(B_sf),
               A_gs,
               B_gs,
               bias,
               static_cast<float *>(workspace),
               M,
               N,
               K,
               align_up(N, 16),
               p.ks_len,
               p.split_k};
  return dispatch_skinny(a, p, d_dtype, bias_dtype, st);
}

static int check_skinny(const SkinnyPlan &p, bool ok, const void *B, void *workspace, int64_t workspace_bytes) {
  AC4K_REQUIRE(ok, "no workspace-assisted path for this shape: decode-sized shapes need 1 <= M <= 32 and K a multiple of 256");
  AC4K_REQUIRE(((uintptr_t)B & 15) == 0, "weights must be 16-byte aligned");
  if (p.partial_bytes > 0) {  // one K range per tile needs no scratch
    AC4K_REQUIRE(workspace && ((uintptr_t)workspace & 255) == 0, "workspace must be 256-byte aligned");
    AC4K_REQUIRE(workspace_bytes >= p.partial_bytes, "workspace too small: %lld bytes needed", (long long)p.partial_bytes);
  }
  return 0;
}

}  // namespace ac4k

extern "C" __attribute__((visibility("default"))) int64_t ac4k_linear_nvfp4_skinny_workspace_bytes(int64_t M, int64_t N, int64_t K) {
  SkinnyPlan p;
  if (skinny_plan(M, N, K, p)) return p.partial_bytes;
  MidPlan mp;
  if (mid_plan(M, N, K, mp)) return mp.bytes;
  return 0;
}

namespace ac4k {

// body of the two workspace-assisted entry points (caller's workspace / the library's static array)
static int linear_skinny_impl(void *D, int d_dtype, const void *A, const void *A_sf, const float *A_gs, const void *B,
                              const void *B_sf, const float *B_gs, const void *bias, int bias_dtype, int64_t M,
                              int64_t N, int64_t K, void *workspace, int64_t workspace_bytes, hipStream_t st,
                              const char *what) {
  AC4K_REQUIRE(D && A && A_sf && A_gs && B && B_sf && B_gs, "null pointer argument");
  AC4K_REQUIRE(M >= 1 && N >= 1 && K >= 1, "M, N, K must be positive (M=%lld N=%lld K=%lld)", (long long)M,
               (long long)N, (long long)K);
  MidPlan mp;
  if (M > 32 && mid_plan(M, N, K, mp)) {  // few tiles, long K: split-K
    AC4K_REQUIRE((((uintptr_t)A | (uintptr_t)B) & 15) == 0 && (((uintptr_t)A_sf | (uintptr_t)B_sf) & 3) == 0,
                 "A and B must be 16-byte aligned and the scale tensors 4-byte aligned");
    if (mp.bytes > 0) {  // one K range per tile needs no scratch
      AC4K_REQUIRE(workspace && ((uintptr_t)workspace & 255) == 0, "workspace must be 256-byte aligned");
      AC4K_REQUIRE(workspace_bytes >= mp.bytes, "workspace too small: %lld bytes needed", (long long)mp.bytes);
    }
    LinearArgs la{D, static_cast<const uint8_t *>(A), static_cast<const uint8_t *>(B),
                  static_cast<const uint32_t *>(A_sf), static_cast<const uint32_t *>(B_sf), A_gs, B_gs, bias,
                  M, N, K, align_up(M, 16), align_up(N, 16)};
    if (int rc = dispatch_mid(la, mp, static_cast<float *>(workspace), workspace ? workspace_bytes : 0, d_dtype, bias_dtype, st))
      return rc;
    return check_launch(what);
  }
  SkinnyPlan p;
  const bool ok = skinny_plan(M, N, K, p);
  if (int rc = check_skinny(p, ok, B, workspace, workspace_bytes)) return rc;
  AC4K_REQUIRE(((uintptr_t)A & 15) == 0, "A must be 16-byte aligned");
  if (int rc = run_skinny(D, d_dtype, A, A_sf, A_gs, B, B_sf, B_gs, bias, bias_dtype, M, N, K, p, workspace, st))
    return rc;
  return check_launch(what);
}

// ---------------------------------------------------------------------------
// Scratch of the entry point that allocates nothing: one array per GPU, held until the process ends.
// In host code the array's name is only a handle: its device address comes from hipGetSymbolAddress,
// once per device with that device current, and that pointer is what the kernels are given.
// ---------------------------------------------------------------------------
constexpr int64_t STATIC_SCRATCH_BYTES = AC4K_STATIC_SCRATCH_BYTES;
static __device__ __align__(256) unsigned char scratch[STATIC_SCRATCH_BYTES];

static int static_scratch(void **ptr_out) {
  constexpr int MAX_DEV = 64;
  static void *ptrs[MAX_DEV] = {};
  static std::mutex mu;
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return set_error("hipGetDevice: %s", hipGetErrorString(e));
  AC4K_REQUIRE(dev >= 0 && dev < MAX_DEV, "device index %d out of range", dev);
  std::lock_guard<std::mutex> lock(mu);
  if (!ptrs[dev]) {
    void *p = nullptr;
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess || !p) return set_error("hipGetSymbolAddress(scratch): %s", hipGetErrorString(e));
    ptrs[dev] = p;
  }
  *ptr_out = ptrs[dev];
  return 0;
}

}  // namespace ac4k

extern "C" __attribute__((visibility("default"))) int ac4k_linear_nvfp4_skinny(void *D, int d_dtype, const void *A, const void *A_sf, const float *A_gs,
                                        const void *B, const void *B_sf, const float *B_gs, const void *bias,
                                        int bias_dtype, int64_t M, int64_t N, int64_t K, void *workspace,
                                        int64_t workspace_bytes, ac4k_stream_t stream) {
  return linear_skinny_impl(D, d_dtype, A, A_sf, A_gs, B, B_sf, B_gs, bias, bias_dtype, M, N, K, workspace,
                            workspace_bytes, (hipStream_t)stream, "ac4k_linear_nvfp4_skinny");
}

extern "C" __attribute__((visibility("default"))) int ac4k_linear_nvfp4_skinny_static(void *D, int d_dtype, const void *A, const void *A_sf,
                                               const float *A_gs, const void *B, const void *B_sf,
                                               const float *B_gs, const void *bias, int bias_dtype, int64_t M,
                                               int64_t N, int64_t K, ac4k_stream_t stream) {
  AC4K_REQUIRE(M >= 1 && N >= 1 && K >= 1, "M, N, K must be positive (M=%lld N=%lld K=%lld)", (long long)M,
               (long long)N, (long long)K);
  const int64_t need = ac4k_linear_nvfp4_skinny_workspace_bytes(M, N, K);
  AC4K_REQUIRE(need <= STATIC_SCRATCH_BYTES,
               "shape needs %lld bytes of scratch, the static scratch holds %lld: use ac4k_linear_nvfp4_skinny with a "
               "workspace of the caller",
               (long long)need, (long long)STATIC_SCRATCH_BYTES);
  void *ws = nullptr;
  if (int rc = static_scratch(&ws)) return rc;
  // the partial sums are written before they are read: nothing in the array has to start at zero
  return linear_skinny_impl(D, d_dtype, A, A_sf, A_gs, B, B_sf, B_gs, bias, bias_dtype, M, N, K, ws,
                            STATIC_SCRATCH_BYTES, (hipStream_t)stream, "ac4k_linear_nvfp4_skinny_static");
}

namespace ac4k {

// One workgroup writes one block of the weight image: 128 rows x 64 packed bytes (rows past N zero),
// piece p of row r at position p ^ ((r >> 1) & 3), then the scale dwords [2 chunks][128 rows].
__global__ __launch_bounds__(256) void prepack_weight_kernel(uint8_t *image, const uint8_t *B, const uint32_t *B_sf,
                                                             int64_t N, int64_t K, int64_t Np) {
  const int64_t kt = blockIdx.x, band = blockIdx.y;
  uint8_t *blk = image + (band * gridDim.x + kt) * W_BLOCK_BYTES;
  const int t = threadIdx.x;
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const int r = (t + i * 256) >> 2, pc = t & 3;
    const int64_t row = band * W_BLOCK_ROWS + r;
    uint4 v = make_uint4(0, 0, 0, 0);
    if (row < N) v = *reinterpret_cast<const uint4 *>(B + row * (K >> 1) + kt * (W_BLOCK_K / 2) + pc * 16);
    *reinterpret_cast<uint4 *>(blk + r * (W_BLOCK_K / 2) + ((pc ^ ((r >> 1) & 3)) * 16)) = v;
  }
  const int c = t >> 7, r = t & 127;
  const int64_t row = band * W_BLOCK_ROWS + r;
  reinterpret_cast<uint32_t *>(blk + W_BLOCK_DATA)[c * W_BLOCK_ROWS + r] = row < N ? B_sf[(kt * 2 + c) * Np + row] : 0u;
}

static int64_t weight_image_bytes(int64_t N, int64_t K) {
  if (N < 1 || K < W_BLOCK_K || K % W_BLOCK_K != 0) return 0;
  return ceil_div(N, W_BLOCK_ROWS) * (K / W_BLOCK_K) * W_BLOCK_BYTES;
}

// How a linear on a weight image runs: the LDS-ring kernel for decode-sized M (K % 256 == 0), the K-split-waves
// kernel for 32 < M <= 128, the tile kernel otherwise, split along K when the workspace entry point of the plain
// layout would split too.
struct PrepackedPlan {
  bool ring, mid;
  SkinnyPlan sp;
  KsplitPlan kp;
  TilePlan tp;
  int64_t partial_bytes;
};
static bool prepacked_plan(int64_t M, int64_t N, int64_t K, PrepackedPlan &p) {
  const int64_t bytes = weight_image_bytes(N, K);
  if (M < 1 || bytes == 0 || bytes >= (1ll << 32) || (K >> 1) * 256 >= (1ll << 31) || N >= (1ll << 27)) return false;
  p.ring = M <= 32 && K % ST_BK == 0;
  p.mid = !p.ring && ksplit_shape(M, N, K);
  if (p.ring) {
    plan_lds_ring(M, N, K, p.sp);
    p.partial_bytes = p.sp.partial_bytes;
  } else {
    p.tp = tile_plan(M, N, K, true);
    p.partial_bytes = p.tp.partial_bytes;
    if (p.mid) {
      p.kp = ksplit_plan(M, N, K, true);
      p.partial_bytes = p.kp.partial_bytes;
    }
  }
  return true;
}

}  // namespace ac4k

extern "C" __attribute__((visibility("default"))) int64_t ac4k_prepack_weight_nvfp4_bytes(int64_t N, int64_t K) {
  const int64_t bytes = weight_image_bytes(N, K);
  return bytes < (1ll << 32) ? bytes : 0;
}

extern "C" __attribute__((visibility("default"))) int ac4k_prepack_weight_nvfp4(void *image, const void *B, const void *B_sf, int64_t N, int64_t K,
                                                                                ac4k_stream_t stream) {
  AC4K_REQUIRE(image && B && B_sf, "null pointer argument");
  const int64_t bytes = ac4k_prepack_weight_nvfp4_bytes(N, K);
  AC4K_REQUIRE(bytes > 0, "no weight image for N = %lld, K = %lld: K must be a multiple of 128 and the image smaller than 4 GiB",
               (long long)N, (long long)K);
  AC4K_REQUIRE((((uintptr_t)image | (uintptr_t)B) & 15) == 0 && ((uintptr_t)B_sf & 3) == 0,
               "image and B must be 16-byte aligned, B_sf 4-byte aligned");
  hipLaunchKernelGGL(prepack_weight_kernel, dim3((unsigned)(K / W_BLOCK_K), (unsigned)ceil_div(N, W_BLOCK_ROWS)), dim3(256), 0,
                     (hipStream_t)stream, static_cast<uint8_t *>(image), static_cast<const uint8_t *>(B),
                     static_cast<const uint32_t *>(B_sf), N, K, align_up(N, 16));
  return check_launch("ac4k_prepack_weight_nvfp4");
}

extern "C" __attribute__((visibility("default"))) int64_t ac4k_linear_nvfp4_prepacked_workspace_bytes(int64_t M, int64_t N, int64_t K) {
  PrepackedPlan p;
  return prepacked_plan(M, N, K, p) ? p.partial_bytes : 0;
}

extern "C" __attribute__((visibility("default"))) int ac4k_linear_nvfp4_prepacked(void *D, int d_dtype, const void *A, const void *A_sf, const float *A_gs,
                                                                                  const void *W_image, const float *B_gs, const void *bias,
                                                                                  int bias_dtype, int64_t M, int64_t N, int64_t K, void *workspace,
                                                                                  int64_t workspace_bytes, ac4k_stream_t stream) {
  AC4K_REQUIRE(D && A && A_sf && A_gs && W_image && B_gs, "null pointer argument");
  AC4K_REQUIRE(M >= 1 && N >= 1, "M and N must be positive (M = %lld, N = %lld)", (long long)M, (long long)N);
  PrepackedPlan p;
  AC4K_REQUIRE(prepacked_plan(M, N, K, p), "no weight image for N = %lld, K = %lld (ac4k_prepack_weight_nvfp4_bytes returns 0)",
               (long long)N, (long long)K);
  AC4K_REQUIRE((((uintptr_t)A | (uintptr_t)W_image) & 15) == 0 && ((uintptr_t)A_sf & 3) == 0,
               "A and the weight image must be 16-byte aligned, A_sf 4-byte aligned");
  AC4K_REQUIRE(ceil_div(M, 128) * ceil_div(N, 64) < (1ll << 31), "problem too large");
  if (p.partial_bytes > 0) {
    AC4K_REQUIRE(workspace && ((uintptr_t)workspace & 255) == 0, "workspace must be 256-byte aligned");
    AC4K_REQUIRE(workspace_bytes >= p.partial_bytes, "workspace too small: %lld bytes needed", (long long)p.partial_bytes);
  }
  hipStream_t st = (hipStream_t)stream;
  if (p.ring) {
    SkinnyArgs a{D, static_cast<const uint8_t *>(A), static_cast<const uint8_t *>(A_sf), align_up(M, 16),
                 static_cast<const uint8_t *>(W_image), nullptr, A_gs, B_gs, bias, static_cast<float *>(workspace),
                 M, N, K, align_up(N, 16), 0, p.sp.split_k, 1};
    if (int rc = dispatch_skinny(a, p.sp, d_dtype, bias_dtype, st)) return rc;
    return check_launch("ac4k_linear_nvfp4_prepacked");
  }
  LinearArgs la{D, static_cast<const uint8_t *>(A), static_cast<const uint8_t *>(W_image),
                static_cast<const uint32_t *>(A_sf), nullptr, A_gs, B_gs, bias,
                M, N, K, align_up(M, 16), align_up(N, 16), 1};
  int rc;
  if (p.mid || p.tp.splits > 1) {
    rc = dispatch_mid(la, MidPlan{p.mid, p.mid ? p.kp : KsplitPlan{0, 0, 1, 0}, p.tp, p.partial_bytes},
                      static_cast<float *>(workspace), workspace_bytes, d_dtype, bias_dtype, st);
  } else {
    switch (d_dtype) {
      case AC4K_DTYPE_BF16: rc = dispatch_prepacked_bias<AC4K_DTYPE_BF16>(la, p.tp, bias_dtype, st); break;
      case AC4K_DTYPE_FP16: rc = dispatch_prepacked_bias<AC4K_DTYPE_FP16>(la, p.tp, bias_dtype, st); break;
      case AC4K_DTYPE_FP32: rc = dispatch_prepacked_bias<AC4K_DTYPE_FP32>(la, p.tp, bias_dtype, st); break;
      default: return set_error("d must be bfloat16, half or float (dtype tag %d)", d_dtype);
    }
  }
  if (rc) return rc;
  return check_launch("ac4k_linear_nvfp4_prepacked");
}

extern "C" __attribute__((visibility("default"))) int ac4k_linear_nvfp4_fused_bf16(void *D, int d_dtype, const void *X, void *X_q, void *X_sf,
                                            float *X_gs, const void *B, const void *B_sf, const float *B_gs,
                                            const void *bias, int bias_dtype, int64_t M, int64_t N, int64_t K,
                                            void *workspace, int64_t workspace_bytes, ac4k_stream_t stream) {
  AC4K_REQUIRE(D && X && X_q && X_sf && X_gs && B && B_sf && B_gs, "null pointer argument");
  AC4K_REQUIRE(M >= 1 && M <= 32, "the fused skinny linear takes 1 <= M <= 32 (got %lld)", (long long)M);
  AC4K_REQUIRE(N >= 1 && K >= 1, "N and K must be positive (N=%lld K=%lld)", (long long)N, (long long)K);
  SkinnyPlan p;
  const bool ok = skinny_plan(M, N, K, p);
  if (int rc = check_skinny(p, ok, B, workspace, workspace_bytes)) return rc;
  hipStream_t st = (hipStream_t)stream;
  AC4K_REQUIRE(((uintptr_t)X & 15) == 0, "activation must be 16-byte aligned");
  if (int rc = ac4k_quantize_nvfp4_bf16(X_q, X_sf, X_gs, X, 1, 1, M, K, 0, 0, K, 1, 0, 2688.0f, stream)) return rc;
  if (int rc = run_skinny(D, d_dtype, X_q, X_sf, X_gs, B, B_sf, B_gs, bias, bias_dtype, M, N, K, p, workspace,
                          st))
    return rc;
  return check_launch("ac4k_linear_nvfp4_fused_bf16");
}

extern "C" __attribute__((visibility("default"))) int ac4k_set_linear_tuning(int mi, int nj, int splits, int skinny_ks,
                                                                          int decode_kernel) {
  // every argument is checked before any is stored: a rejected call changes nothing
  AC4K_REQUIRE(decode_kernel >= 0 && decode_kernel <= 3,
               "decode_kernel must be 0 (by shape), 1 (register kernel), 2 (LDS-ring kernel) or 3 (LDS-ring kernel with "
               "64-row tiles) (got %d)", decode_kernel);
  const bool no_plan = mi == 0 && nj == 0 && splits == 0;
  AC4K_REQUIRE(no_plan || ((mi == 2 || mi == 4) && (nj == 1 || nj == 2 || nj == 4) && !(mi == 4 && nj == 1) && splits >= 1 &&
                           splits <= 0xffff),
               "tile plan must be mi in {2,4}, nj in {1,2,4} (not 4,1), 1 <= splits (got %d,%d,%d)", mi, nj, splits);
  AC4K_REQUIRE(skinny_ks >= 0 && skinny_ks % 256 == 0, "skinny_ks must be 0 (automatic) or a multiple of 256 (got %d)",
               skinny_ks);
  ac4k::g_forced_decode_kernel.store(decode_kernel);
  ac4k::g_forced_tile_plan.store(no_plan ? 0u : (uint32_t)mi | ((uint32_t)nj << 8) | ((uint32_t)splits << 16));
  ac4k::g_forced_skinny_ks.store(skinny_ks);
  return 0;
}

#ifdef AC4K_LINEAR_TIMELINE
// Timeline build only: copies the per-workgroup stamps of the last tile / K-split-waves launch to host
// memory ([8192][6]: 100 MHz ticks at kernel entry, loop entry, loop exit, kernel exit; shader cycles in
// the loop; XCC and hardware id for the tile kernel).  Synchronises the device.
extern "C" __attribute__((visibility("default"))) int ac4k_debug_linear_timeline(uint64_t *host_out) {
  hipError_t e = hipDeviceSynchronize();
  if (e == hipSuccess) e = hipMemcpyFromSymbol(host_out, HIP_SYMBOL(ac4k::g_linear_timeline), sizeof(uint64_t) * 8192 * 6);
  return e == hipSuccess ? 0 : ac4k::set_error("ac4k_debug_linear_timeline: %s", hipGetErrorString(e));
}
#endif
