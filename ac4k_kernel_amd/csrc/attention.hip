// NVFP4 attention forward for gfx950, head dims up to 128:  O = softmax(Q K^T * sm_scale) V on NVFP4 operands.
//
// Math contract of the reference kernel (lib/cuda/sm120/mha_nvfp4.cu:336-905, host checks :911-1077,
// interface include/ac4k_kernel/ops.h:12-16):
//   S = (Qhat . Khat^T) * (q_gs * k_gs * sm_scale), accumulated in fp32                          :586-598
//   online softmax over kv tiles of 128; kv positions past Nkv inside the last tile have S = 0,
//   enter the row maximum and P, and are taken out of the row sum again                          :600-700
//   P is quantized to NVFP4 on the fly with the global scale 1/2688; its 16-blocks are the kv
//   positions {8g + 4h + j} (g, j = 0..3) of a 32-group, h = 0, 1 - the sets that the swizzle of
//   quantize(v, 3, N_dim, swizzle=True) makes contiguous in V                                    :248-319
//   O = (sum over tiles of Phat . Vhat^T, rescaled) * ((1/l) * (1/2688) * v_gs) -> bf16          :705-830
// A workgroup (four waves) owns 128 query rows, a wave 32 of them.  Per kv tile of 128 the packed K rows and
// the packed V rows (V is stored [d][kv]) are fetched once per workgroup - every thread two 16-byte pieces of
// each plus one scale dword, issued a whole tile ahead -, decoded once to exact fp16 and written to LDS, from
// where all four waves read their MFMA operands.  Two LDS buffers alternate, one barrier per tile.  Decoded rows
// are 256 bytes at a pitch of 272, so that the 16-byte fragment reads of 16 lanes fall on 64 different banks.
//
// The MFMAs are issued so that a lane owns ONE query row: S^T = Khat . Qhat^T and O^T = Vhat . Phat^T
// (v_mfma_f32_32x32x16_f16, exact fp16 decode as in the linear).  Lane (r, h) of a wave then holds, per
// 32-row kv fragment, the 16 values S[r][8g + 4h + j]: exactly one P block, so its maximum, scale and
// nibbles are formed inside the lane, and the row maximum and row sum need one exchange between the two
// halves of the wave.  The k slots of the second product are paired through the stored (swizzled) order
// of V: slot s of step t holds kv position 8 (2t + (s>>1 & 1)) + 4h + 2 (s>>2) + (s & 1).
#include "ac4k_common.h"

#include <atomic>
#include <type_traits>

namespace ac4k {

struct MhaArgs {
  uint16_t *O;
  int64_t o_b, o_h, o_n, o_d;  // element strides of O [B, H, Nq, 128]
  const uint8_t *q, *k, *v, *q_sf, *k_sf, *v_sf;
  const float *q_gs, *k_gs, *v_gs;
  int64_t H, Nq, Nkv, Nqp, Nkvp, Nkv64;  // padded: rows of the Q / K scale planes (16), stored kv length of V (64)
  int chunks, Dv, Dvp;                   // 64-chunks of a Q / K row (1 or 2), rows of V, rows of a V scale plane (16)
  float sm_scale;
  int o_vec;  // O rows are contiguous along d, 16-byte aligned, Dv % 8 == 0: rows leave as 16-byte pieces
};

constexpr float MHA_LOG2E = 1.4426950408889634f;
constexpr float MHA_P_ALPHA = 2688.0f;  // 1 / (global scale of P)

// eight nibbles times the block scale -> eight fp16 (exact)
__device__ __forceinline__ f16x8 mha_decode8(uint32_t w, f16x2 sc) {
  const f16x2 d0 = __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(w, 1.0f, 0) * sc;
  const f16x2 d1 = __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(w, 1.0f, 1) * sc;
  const f16x2 d2 = __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(w, 1.0f, 2) * sc;
  const f16x2 d3 = __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(w, 1.0f, 3) * sc;
  return (f16x8){d0.x, d0.y, d1.x, d1.y, d2.x, d2.y, d3.x, d3.y};
}

// A row-major packed row of Q: the lane's 32 elements [32 h, 32 h + 32) of 64-chunk c, and the two block
// scales that go with them, decoded into the four 16-k operands of that chunk.
__device__ __forceinline__ void mha_load_row_chunk(const uint8_t *row, const uint8_t *sf_chunk_row, int c, int h,
                                                   f16x8 (&out)[4]) {
  const uint4 w = *reinterpret_cast<const uint4 *>(row + c * 32 + h * 16);
  const uint32_t sc = *reinterpret_cast<const uint16_t *>(sf_chunk_row + 2 * h);
  const f16x2 s2 = __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(sc, 1.0f, false);
  const f16x2 lo = {s2.x, s2.x}, hi = {s2.y, s2.y};
  out[0] = mha_decode8(w.x, lo);
  out[1] = mha_decode8(w.y, lo);
  out[2] = mha_decode8(w.z, hi);
  out[3] = mha_decode8(w.w, hi);
}

// dword i (0..7) of two 16-byte pieces; i is a constant after unrolling
__device__ __forceinline__ uint32_t mha_dword(const uint4 &a, const uint4 &b, int i) {
  switch (i) {
    case 0: return a.x;
    case 1: return a.y;
    case 2: return a.z;
    case 3: return a.w;
    case 4: return b.x;
    case 5: return b.y;
    case 6: return b.z;
    default: return b.w;
  }
}

// both halves of the wave (lanes 0-31 and 32-63) receive op(x of the lower half, x of the upper half)
__device__ __forceinline__ float mha_halves_max(float x) { return __builtin_fmaxf(x, __shfl_xor(x, 32, 64)); }
__device__ __forceinline__ float mha_halves_sum(float x) { return x + __shfl_xor(x, 32, 64); }

// Output of one wave: O^T in the MFMA accumulator layout (lane (r, h) owns query row r of the wave: OT[fd][e] is head
// dim 32 fd + 8 (e >> 2) + 4 h + (e & 3)), already scaled, as bf16 bits in ob[fd][e].  Vector path (rows of O
// contiguous along d, 16-byte aligned, Dv % 8 == 0): the wave's 32 x 128 tile goes through LDS (8448 bytes at
// `stage`, free to use: every wave has passed the last barrier of the loop) and leaves as 16-byte pieces of
// adjacent lanes, whole 256-byte rows; otherwise element by element.
constexpr int MHA_OUT_PITCH = 264;  // bytes per row of the staged tile (256 + 8: bank spread)
constexpr int MHA_OUT_LDS = 32 * MHA_OUT_PITCH;
__device__ __forceinline__ void mha_store_rows(uint16_t *o_base, int64_t o_n, int64_t o_d, int o_vec, int64_t row0,
                                               int64_t Nq, int Dv, int lane, uint8_t *stage,
                                               const uint16_t (&ob)[4][16]) {
  const int r = lane & 31, h = lane >> 5;
  if (o_vec) {
#pragma unroll
    for (int fd = 0; fd < 4; ++fd)
#pragma unroll
      for (int q4 = 0; q4 < 4; ++q4) {
        const int d = fd * 32 + q4 * 8 + h * 4;
        *reinterpret_cast<uint2 *>(stage + r * MHA_OUT_PITCH + d * 2) =
            make_uint2(ob[fd][4 * q4] | ((uint32_t)ob[fd][4 * q4 + 1] << 16), ob[fd][4 * q4 + 2] | ((uint32_t)ob[fd][4 * q4 + 3] << 16));
      }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
    for (int p = 0; p < 8; ++p) {
      const int row = p * 4 + (lane >> 4), d = (lane & 15) * 8;
      const uint4 w = *reinterpret_cast<const uint4 *>(stage + row * MHA_OUT_PITCH + d * 2);
      if (row0 + row < Nq && d < Dv) *reinterpret_cast<uint4 *>(o_base + (row0 + row) * o_n + d) = w;
    }
  } else if (row0 + r < Nq) {
    uint16_t *orow = o_base + (row0 + r) * o_n;
#pragma unroll
    for (int fd = 0; fd < 4; ++fd)
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        const int d = fd * 32 + (e >> 2) * 8 + h * 4 + (e & 3);
        if (d < Dv) orow[d * o_d] = ob[fd][e];
      }
  }
}

constexpr int MHA_PITCH = 272;                   // bytes per decoded row in LDS: 128 fp16 + 16 (bank spread)
constexpr int MHA_TILE_LDS = 128 * MHA_PITCH;    // one decoded operand tile: K 128 kv rows, V 128 d rows
constexpr int MHA_LDS_BYTES = 4 * MHA_TILE_LDS;  // K tiles j & 1 at 0 and MHA_TILE_LDS, V tiles j & 1 behind them

// what one thread fetches per kv tile: a quarter of a packed K row (two 16-blocks), a quarter of a packed V row of
// the tile (one 32-group of kv positions), and the two scale bytes of each
struct MhaFetch {
  uint4 k, v;
  uint32_t ksc, vsc;
};

// WAVES = 8 (256 query rows per workgroup, two waves per SIMD: one wave's MFMAs run under the other's vector work)
// or 4 (128 query rows, for problems with too few workgroups of 256 rows to fill the GPU).  Both are compiled for 256
// registers per lane (the launch bounds ask for two 4-wave workgroups per CU, which the LDS tile buffers do not
// allow anyway): with 512, the compiler keeps S^T and O^T in accumulation registers and copies all of them to
// ordinary registers and back around the softmax of every tile.
template <int WAVES>
__global__ __launch_bounds__(64 * WAVES, 8 / WAVES) void mha_nvfp4_fwd_kernel(MhaArgs a) {
  constexpr int PARTS = 8 / WAVES;  // staging shares per thread: a tile is 512 quarter rows of K and of V
  extern __shared__ __attribute__((aligned(16))) uint8_t mha_lds[];
  __shared__ float lut[128];  // exact reciprocals of the e4m3 values, as in the quantizer
  load_rcp_table(lut);
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, r = lane & 31, h = lane >> 5;
  // staging role of share p: row srow + p * (128 / PARTS) of the tile, 64-chunk sc, half sh of the chunk (K:
  // elements 32 sh.. of the chunk, V: 32-group 2 sc + sh)
  const int srow = threadIdx.x >> 2, sc = (threadIdx.x >> 1) & 1, sh = threadIdx.x & 1;
  constexpr int PROWS = 128 / PARTS;
  const int64_t b = blockIdx.z, head = blockIdx.y, bh = b * a.H + head;
  const int64_t m = (int64_t)blockIdx.x * (32 * WAVES) + wave * 32 + r;   // this lane's query row
  const int64_t mq = m < a.Nq ? m : a.Nq - 1;                         // rows past Nq read the last row; never stored
  const int64_t v_row_bytes = a.Nkv64 / 2, v_chunks = a.Nkv64 / 64;

  // head dims below 128: the missing chunk of Q and K and the missing rows of V are zeros
  const int64_t qk_row = a.chunks * 32;  // packed bytes of a Q / K row
  const uint8_t *k_src = a.k + bh * a.Nkv * qk_row + sc * 32 + sh * 16;
  const uint8_t *ksf_src = a.k_sf + (bh * a.chunks + sc) * a.Nkvp * 4 + sh * 2;
  const uint8_t *v_src = a.v + (bh * a.Dv + srow) * v_row_bytes + sc * 32 + sh * 16;
  const uint8_t *vsf_src = a.v_sf + ((bh * v_chunks + sc) * a.Dvp + srow) * 4 + sh * 2;
  // rows past Nkv and chunks past the stored length of V are zeros
  auto fetch = [&](int64_t n0, MhaFetch (&fs)[PARTS]) {
#pragma unroll
    for (int p = 0; p < PARTS; ++p) {
      MhaFetch &f = fs[p];
      const int64_t n = n0 + srow + p * PROWS;
      f.k = f.v = make_uint4(0, 0, 0, 0);
      f.ksc = f.vsc = 0;
      if (n < a.Nkv && sc < a.chunks) {
        f.k = *reinterpret_cast<const uint4 *>(k_src + n * qk_row);
        f.ksc = *reinterpret_cast<const uint16_t *>(ksf_src + n * 4);
      }
      if (n0 + 64 * sc < a.Nkv64 && srow + p * PROWS < a.Dv) {
        f.v = *reinterpret_cast<const uint4 *>(v_src + p * PROWS * v_row_bytes + n0 / 2);
        f.vsc = *reinterpret_cast<const uint16_t *>(vsf_src + p * PROWS * 4 + (n0 / 64) * (a.Dvp * 4));
      }
    }
  };
  // the same for a tile that lies inside Nkv as a whole, head dims of 128: nothing to test, nothing to zero
  auto fetch_whole = [&](int64_t n0, MhaFetch (&fs)[PARTS]) {
#pragma unroll
    for (int p = 0; p < PARTS; ++p) {
      MhaFetch &f = fs[p];
      const int64_t n = n0 + srow + p * PROWS;
      f.k = *reinterpret_cast<const uint4 *>(k_src + n * qk_row);
      f.ksc = *reinterpret_cast<const uint16_t *>(ksf_src + n * 4);
      f.v = *reinterpret_cast<const uint4 *>(v_src + p * PROWS * v_row_bytes + n0 / 2);
      f.vsc = *reinterpret_cast<const uint16_t *>(vsf_src + p * PROWS * 4 + (n0 / 64) * (a.Dvp * 4));
    }
  };
  // decode once per workgroup, into LDS tile buffers `buf`.  V: the thread's 32-group holds 16 stored bytes; operand
  // piece (t, hh) takes the t-th 16-bit halves of its dwords 2 hh and 2 hh + 1, and the scale of stored block hh.
  auto stage = [&](int buf, const MhaFetch (&fs)[PARTS]) {
#pragma unroll
    for (int p = 0; p < PARTS; ++p) {
    const MhaFetch &f = fs[p];
    uint8_t *kd = mha_lds + buf * MHA_TILE_LDS + (srow + p * PROWS) * MHA_PITCH + sc * 128 + sh * 64;
    const f16x2 ks = __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(f.ksc, 1.0f, false);
    const f16x2 kb0 = {ks.x, ks.x}, kb1 = {ks.y, ks.y};
    *reinterpret_cast<f16x8 *>(kd + 0) = mha_decode8(f.k.x, kb0);
    *reinterpret_cast<f16x8 *>(kd + 16) = mha_decode8(f.k.y, kb0);
    *reinterpret_cast<f16x8 *>(kd + 32) = mha_decode8(f.k.z, kb1);
    *reinterpret_cast<f16x8 *>(kd + 48) = mha_decode8(f.k.w, kb1);
    uint8_t *vd = mha_lds + (2 + buf) * MHA_TILE_LDS + (srow + p * PROWS) * MHA_PITCH + sc * 128 + sh * 64;
    const f16x2 vs = __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(f.vsc, 1.0f, false);
    const f16x2 vb0 = {vs.x, vs.x}, vb1 = {vs.y, vs.y};
    *reinterpret_cast<f16x8 *>(vd + 0) = mha_decode8((f.v.x & 0xffffu) | (f.v.y << 16), vb0);           // t 0, hh 0
    *reinterpret_cast<f16x8 *>(vd + 16) = mha_decode8((f.v.z & 0xffffu) | (f.v.w << 16), vb1);          // t 0, hh 1
    *reinterpret_cast<f16x8 *>(vd + 32) = mha_decode8((f.v.x >> 16) | (f.v.y & 0xffff0000u), vb0);      // t 1, hh 0
    *reinterpret_cast<f16x8 *>(vd + 48) = mha_decode8((f.v.z >> 16) | (f.v.w & 0xffff0000u), vb1);      // t 1, hh 1
    }
  };

  // Qhat of the lane's row: 8 operands of 16 k (chunk c, sub-step s), kept for the whole kernel
  f16x8 QF[2][4];
#pragma unroll
  for (int c = 0; c < 2; ++c) {
#pragma unroll
    for (int s = 0; s < 4; ++s) QF[c][s] = (f16x8)((_Float16)0);
    if (c < a.chunks)
      mha_load_row_chunk(a.q + (bh * a.Nq + mq) * qk_row, a.q_sf + ((bh * a.chunks + c) * a.Nqp + mq) * 4, c, h, QF[c]);
  }

  // exp2 argument = S * cs - (row maximum of S) * cs with cs = q_gs * k_gs * sm_scale * log2(e); a negative cs is
  // moved into Q so that the row maximum can be taken over the raw dot products
  float cs = (*a.q_gs) * (*a.k_gs) * a.sm_scale * MHA_LOG2E;
  if (cs < 0.0f) {
    cs = -cs;
#pragma unroll
    for (int c = 0; c < 2; ++c)
#pragma unroll
      for (int s = 0; s < 4; ++s) QF[c][s] = -QF[c][s];
  }
  float ml_run = -__builtin_inff(), l_run = 0.0f;  // running row maximum (in log2 units) and row sum
  f32x16 OT[4];  // O^T: d = 32 fd + 8 (e >> 2) + 4 h + (e & 3), for the lane's query row
#pragma unroll
  for (int fd = 0; fd < 4; ++fd)
#pragma unroll
    for (int e = 0; e < 16; ++e) OT[fd][e] = 0.0f;

  MhaFetch nxt[PARTS];
  fetch(0, nxt);
  stage(0, nxt);
  __syncthreads();
  int buf = 0;
  auto tile_step = [&](auto whole_next_tag, int64_t n0) {
    // the next tile's packed bytes travel while this one is multiplied (zeros past the end)
    if constexpr (decltype(whole_next_tag)::value) fetch_whole(n0 + 128, nxt);
    else fetch(n0 + 128, nxt);
    const uint8_t *kb = mha_lds + buf * MHA_TILE_LDS + r * MHA_PITCH + h * 64;
    const uint8_t *vb = mha_lds + (2 + buf) * MHA_TILE_LDS + r * MHA_PITCH + h * 16;
    // ---- S^T = Khat . Qhat^T for the 128 kv positions of the tile (four 32-row fragments)
    f32x16 ST[4];
#pragma unroll
    for (int c = 0; c < 2; ++c)
#pragma unroll
      for (int s = 0; s < 4; ++s)
#pragma unroll
        for (int f = 0; f < 4; ++f) {  // consecutive MFMAs go to different accumulators
          const f16x8 KF = *reinterpret_cast<const f16x8 *>(kb + f * 32 * MHA_PITCH + c * 128 + s * 16);
          if (c == 0 && s == 0)
            ST[f] = __builtin_amdgcn_mfma_f32_32x32x16_f16(KF, QF[c][s], (f32x16)(0.0f), 0, 0, 0);
          else
            ST[f] = __builtin_amdgcn_mfma_f32_32x32x16_f16(KF, QF[c][s], ST[f], 0, 0, 0);
        }
    // ---- online softmax of the lane's row: its 64 values here, the other 64 in the lane 32 away
    // maxima of the raw values per fragment = per P block: exp2 and the scaling are monotonic, so the largest p of
    // a block is the p of its largest raw value, bit for bit
    float bmax[4];
#pragma unroll
    for (int f = 0; f < 4; ++f) {
      bmax[f] = ST[f][0];
#pragma unroll
      for (int e = 1; e < 16; ++e) bmax[f] = __builtin_fmaxf(bmax[f], ST[f][e]);
    }
    const float mx = __builtin_fmaxf(__builtin_fmaxf(bmax[0], bmax[1]), __builtin_fmaxf(bmax[2], bmax[3]));
    const float ml = __builtin_fmaxf(ml_run, mha_halves_max(mx) * cs);
#pragma unroll
    for (int f = 0; f < 4; ++f) bmax[f] = __builtin_amdgcn_exp2f(__builtin_fmaf(bmax[f], cs, -ml));
    float lsum = 0.0f;
#pragma unroll
    for (int f = 0; f < 4; ++f)
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        ST[f][e] = __builtin_amdgcn_exp2f(__builtin_fmaf(ST[f][e], cs, -ml));  // p
        lsum += ST[f][e];
      }
    const float l_new = mha_halves_sum(lsum);
    const float alpha = __builtin_amdgcn_exp2f(ml_run - ml);
    l_run = alpha * l_run + l_new;
    ml_run = ml;
    if (__builtin_amdgcn_ballot_w64(alpha != 1.0f)) {  // else no row of this wave raised its maximum
#pragma unroll
      for (int fd = 0; fd < 4; ++fd)
#pragma unroll
        for (int e = 0; e < 16; ++e) OT[fd][e] *= alpha;
    }

    // ---- P -> NVFP4 (the lane's 16 values of a fragment are one block), then O^T += Vhat . Phat^T
#pragma unroll
    for (int f = 0; f < 4; ++f) {
      uint32_t code;
      const float o = nvfp4_block_scale(bmax[f], MHA_P_ALPHA, lut, code);  // 2688 / e4m3(2688 * (bm / 6)), 0 for code 0
      const f16x2 s2 = __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(code, 1.0f, false);
      const f16x2 psc = {s2.x, s2.x};
#pragma unroll
      for (int t = 0; t < 2; ++t) {
        // k slots of this step in the order the stored nibbles of V come in (see the header)
        const float pv[8] = {ST[f][8 * t + 0] * o, ST[f][8 * t + 1] * o, ST[f][8 * t + 4] * o, ST[f][8 * t + 5] * o,
                             ST[f][8 * t + 2] * o, ST[f][8 * t + 3] * o, ST[f][8 * t + 6] * o, ST[f][8 * t + 7] * o};
        const f16x8 PF = mha_decode8(f32x8_to_e2m1x8(pv), psc);
#pragma unroll
        for (int fd = 0; fd < 4; ++fd) {
          const f16x8 VF = *reinterpret_cast<const f16x8 *>(vb + fd * 32 * MHA_PITCH + f * 64 + t * 32);
          OT[fd] = __builtin_amdgcn_mfma_f32_32x32x16_f16(VF, PF, OT[fd], 0, 0, 0);
        }
      }
    }
    stage(buf ^ 1, nxt);
    __syncthreads();
  };
  int64_t n0 = 0;
  // tiles followed by a whole tile: the fetch without tests (worth 2 % with eight waves; with four it loses 5 %)
  if (WAVES == 8 && a.chunks == 2 && a.Dv == 128)
    for (; n0 + 256 <= a.Nkv; n0 += 128, buf ^= 1) tile_step(std::true_type{}, n0);
  for (; n0 < a.Nkv; n0 += 128, buf ^= 1) tile_step(std::false_type{}, n0);

  // the zero-filled kv positions of the last tile each added exp(0 - m) to the row sum
  if (a.Nkv % 128 != 0) l_run -= (float)(128 - a.Nkv % 128) / __builtin_amdgcn_exp2f(ml_run);
  // ---- O = O * ((1/l) * (1/2688) * v_gs) -> bf16
  const float scale = (1.0f / l_run) * (1.0f / MHA_P_ALPHA) * (*a.v_gs);
  uint16_t ob[4][16];
#pragma unroll
  for (int fd = 0; fd < 4; ++fd)
#pragma unroll
    for (int e = 0; e < 16; ++e) ob[fd][e] = __builtin_bit_cast(uint16_t, (__bf16)(OT[fd][e] * scale));
  mha_store_rows(a.O + b * a.o_b + head * a.o_h, a.o_n, a.o_d, a.o_vec, (int64_t)blockIdx.x * (32 * WAVES) + wave * 32, a.Nq,
                 a.Dv, lane, mha_lds + wave * MHA_OUT_LDS, ob);
}

// ---------------------------------------------------------------------------------------------------------------
// INT8 (QK) x FP8 (PV) attention forward, head dims up to 128 (lib/cuda/sm120/mha_int8_x_fp8.cu:346-975; host :979-1137;
// interface include/ac4k_kernel/ops.h:18-21):
//   S = Q . K^T in int32 (exact); s = float(S) * ((sm_scale * log2e) * q_sf[row / q_block] * k_sf[tile])   :476,657-677
//   kv positions past Nkv are -inf                                                                    :679-700
//   m = max(rowmax(s) - 7.5, m_old); p = exp2(s - m); l = l * exp2(m_old - m) + sum(p)                 :702-776
//   P -> e4m3 per element (cvt.rn.satfinite, no scales); O = O * exp2(m_old - m) + Phat . Vhat^T        :323-345,828-880
//   O * ((1 / l) * v_sf[d]) -> bf16                                                                   :886-905
// The product Phat . Vhat^T is accumulated in fp32 here (the reference's MMA accumulates each tile in fp16).
// Same structure as the NVFP4 kernel above: a lane owns one query row (S^T = K . Q^T with v_mfma_i32_32x32x32_i8,
// O^T = Vhat . Phat^T with v_mfma_scale_f32_32x32x64_f8f6f4 on e4m3 operands, scales 2^0), but nothing has to be decoded: the int8 rows of K and the
// e4m3 rows of V go from global memory into LDS as they are, and from there into the MFMAs.  V is stored with the
// 16-group swizzle of quantize(v, 3, N_dim, swizzle=True, precision="fp8e4m3"): stored byte 8 h + 4 (j >> 1) + 2 q
// + (j & 1) of a 16-group holds kv position 8 q + 4 h + j, so the eight positions that lane half h owns in a
// 16-group are the contiguous stored bytes [8 h, 8 h + 8): four such pieces are the lane's share of one MFMA operand.

struct Mha8Args {
  uint16_t *O;
  int64_t o_b, o_h, o_n, o_d;  // element strides of O [B, H, Nq, 128]
  const int8_t *q, *k;
  const uint8_t *v;
  const float *q_sf, *k_sf, *v_sf;
  int64_t H, Nq, Nkv, Nkv16, nqb, nkb;  // stored kv length of V (16), scales per head of Q and K
  int Dp, Dv, Dvp;                      // bytes of a Q / K row (head dim padded to 16), rows of V, scales of V per head (16)
  int q_block;
  float sm_scale;
  int o_vec;
};

typedef int i32x4 __attribute__((ext_vector_type(4)));
typedef int i32x8 __attribute__((ext_vector_type(8)));
typedef int i32x16 __attribute__((ext_vector_type(16)));

constexpr int MHA8_PITCH = 144;                    // bytes per 128-byte row in LDS (bank spread)
constexpr int MHA8_TILE_LDS = 128 * MHA8_PITCH;    // K tile: 128 kv rows; V tile: 128 d rows
constexpr int MHA8_LDS_BYTES = 4 * MHA8_TILE_LDS;  // K tiles j & 1, then V tiles j & 1
constexpr float MHA8_EXP_OFFSET = 7.5f;

template <int WAVES>
__global__ __launch_bounds__(64 * WAVES, 8 / WAVES) void mha_int8_x_fp8_fwd_kernel(Mha8Args a) {
  constexpr int PARTS = 8 / WAVES, PROWS = 128 / PARTS;
  extern __shared__ __attribute__((aligned(16))) uint8_t mha_lds[];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, r = lane & 31, h = lane >> 5;
  const int srow = threadIdx.x >> 2, sq = threadIdx.x & 3;  // staging role: row of the tile, 32-byte quarter of it
  const int64_t b = blockIdx.z, head = blockIdx.y, bh = b * a.H + head;
  const int64_t m = (int64_t)blockIdx.x * (32 * WAVES) + wave * 32 + r;  // this lane's query row
  const int64_t mq = m < a.Nq ? m : a.Nq - 1;                            // rows past Nq read the last row; never stored

  // head dims below 128: the missing columns of Q and K and the missing rows of V are zeros
  const int8_t *k_src = a.k + bh * a.Nkv * a.Dp + sq * 32;
  const uint8_t *v_src = a.v + (bh * a.Dv + srow) * a.Nkv16 + sq * 32;
  const bool kc0 = sq * 32 < a.Dp, kc1 = sq * 32 + 16 < a.Dp;
  struct Fetch {
    uint4 k0, k1, v0, v1;
  };
  // rows of K past Nkv and 16-groups of V past its stored length are zeros
  auto fetch = [&](int64_t n0, Fetch (&fs)[PARTS]) {
#pragma unroll
    for (int p = 0; p < PARTS; ++p) {
      Fetch &f = fs[p];
      const int64_t n = n0 + srow + p * PROWS;
      f.k0 = f.k1 = f.v0 = f.v1 = make_uint4(0, 0, 0, 0);
      if (n < a.Nkv) {
        const uint4 *src = reinterpret_cast<const uint4 *>(k_src + n * a.Dp);
        if (kc0) f.k0 = src[0];
        if (kc1) f.k1 = src[1];
      }
      const uint8_t *vs = v_src + p * PROWS * a.Nkv16 + n0;
      const bool vrow = srow + p * PROWS < a.Dv;
      if (vrow && n0 + sq * 32 < a.Nkv16) f.v0 = *reinterpret_cast<const uint4 *>(vs);
      if (vrow && n0 + sq * 32 + 16 < a.Nkv16) f.v1 = *reinterpret_cast<const uint4 *>(vs + 16);
    }
  };
  // the same for a tile that lies inside Nkv as a whole, head dims of 128: nothing to test, nothing to zero
  auto fetch_whole = [&](int64_t n0, Fetch (&fs)[PARTS]) {
#pragma unroll
    for (int p = 0; p < PARTS; ++p) {
      Fetch &f = fs[p];
      const uint4 *src = reinterpret_cast<const uint4 *>(k_src + (n0 + srow + p * PROWS) * a.Dp);
      f.k0 = src[0];
      f.k1 = src[1];
      const uint8_t *vs = v_src + p * PROWS * a.Nkv16 + n0;
      f.v0 = *reinterpret_cast<const uint4 *>(vs);
      f.v1 = *reinterpret_cast<const uint4 *>(vs + 16);
    }
  };
  // a whole tile with smaller head dims: columns of K and rows of V that do not exist are read from a place that does
  // (column 0, row 0) and zeroed by a mask; places and masks do not change from tile to tile
  const int8_t *k_src0 = kc0 ? k_src : k_src - sq * 32, *k_src1 = kc1 ? k_src + 16 : k_src - sq * 32;
  const uint32_t km0 = kc0 ? ~0u : 0u, km1 = kc1 ? ~0u : 0u;
  auto fetch_whole_masked = [&](int64_t n0, Fetch (&fs)[PARTS]) {
#pragma unroll
    for (int p = 0; p < PARTS; ++p) {
      Fetch &f = fs[p];
      const int64_t n = n0 + srow + p * PROWS;
      const bool vrow = srow + p * PROWS < a.Dv;
      const uint32_t vm = vrow ? ~0u : 0u;
      const uint8_t *vs = (vrow ? v_src + p * PROWS * a.Nkv16 : a.v + bh * a.Dv * a.Nkv16 + sq * 32) + n0;
      const uint4 k0 = *reinterpret_cast<const uint4 *>(k_src0 + n * a.Dp), k1 = *reinterpret_cast<const uint4 *>(k_src1 + n * a.Dp);
      const uint4 v0 = *reinterpret_cast<const uint4 *>(vs), v1 = *reinterpret_cast<const uint4 *>(vs + 16);
      f.k0 = make_uint4(k0.x & km0, k0.y & km0, k0.z & km0, k0.w & km0);
      f.k1 = make_uint4(k1.x & km1, k1.y & km1, k1.z & km1, k1.w & km1);
      f.v0 = make_uint4(v0.x & vm, v0.y & vm, v0.z & vm, v0.w & vm);
      f.v1 = make_uint4(v1.x & vm, v1.y & vm, v1.z & vm, v1.w & vm);
    }
  };
  // K rows as they are; V: the thread's two 16-groups (2 sq, 2 sq + 1) regrouped so that the 8-byte pieces of lane
  // half hh of both are one 16-byte run at 32 sq + 16 hh
  auto stage = [&](int buf, const Fetch (&fs)[PARTS]) {
#pragma unroll
    for (int p = 0; p < PARTS; ++p) {
      const Fetch &f = fs[p];
      uint8_t *kd = mha_lds + buf * MHA8_TILE_LDS + (srow + p * PROWS) * MHA8_PITCH + sq * 32;
      *reinterpret_cast<uint4 *>(kd) = f.k0;
      *reinterpret_cast<uint4 *>(kd + 16) = f.k1;
      uint8_t *vd = mha_lds + (2 + buf) * MHA8_TILE_LDS + (srow + p * PROWS) * MHA8_PITCH + sq * 32;
      *reinterpret_cast<uint4 *>(vd) = make_uint4(f.v0.x, f.v0.y, f.v1.x, f.v1.y);
      *reinterpret_cast<uint4 *>(vd + 16) = make_uint4(f.v0.z, f.v0.w, f.v1.z, f.v1.w);
    }
  };

  // Q of the lane's row: the 16 bytes [32 s + 16 h, +16) of k-step s, kept for the whole kernel
  i32x4 QF[4];
#pragma unroll
  for (int s4 = 0; s4 < 4; ++s4) {
    QF[s4] = (i32x4)(0);
    if (s4 * 32 + h * 16 < a.Dp) QF[s4] = *reinterpret_cast<const i32x4 *>(a.q + (bh * a.Nq + mq) * a.Dp + s4 * 32 + h * 16);
  }
  const float qs = (a.sm_scale * MHA_LOG2E) * a.q_sf[bh * a.nqb + mq / a.q_block];

  float m_run = -__builtin_inff(), l_run = 0.0f;  // running maximum (held 7.5 below the row maximum) and row sum
  f32x16 OT[4];  // O^T: d = 32 fd + 8 (e >> 2) + 4 h + (e & 3), for the lane's query row
#pragma unroll
  for (int fd = 0; fd < 4; ++fd)
#pragma unroll
    for (int e = 0; e < 16; ++e) OT[fd][e] = 0.0f;

  Fetch nxt[PARTS];
  fetch(0, nxt);
  stage(0, nxt);
  __syncthreads();
  // one kv tile; TAIL: the last, partial one, whose positions past Nkv are masked (a copy of the code of its own:
  // as a branch inside one body the masks were turned into selects that every tile paid for)
  // The scale of a K tile is asked for in front of the loads of the next tile: behind them, its wait would be a wait
  // for all of them in the middle of the tile.  With eight waves it is loaded a whole tile ahead (the four-wave
  // kernel has no register left for that).
  constexpr bool KSF_AHEAD = WAVES == 8;
  const float *ksf_src = a.k_sf + bh * a.nkb;
  float ksf_cur = KSF_AHEAD ? ksf_src[0] : 0.0f;
  auto tile_step = [&](auto tail_tag, auto whole_next_tag, int64_t n0, int buf) {
    constexpr bool tail = decltype(tail_tag)::value;
    const int64_t t_next = n0 / 128 + 1 < a.nkb ? n0 / 128 + 1 : a.nkb - 1;
    const float ksf_load = ksf_src[KSF_AHEAD ? t_next : n0 / 128];
    asm volatile("" ::: "memory");  // keeps this load in front of the ones below
    // the next tile travels while this one is multiplied (zeros past the end)
    if constexpr (decltype(whole_next_tag)::value == 1) fetch_whole(n0 + 128, nxt);
    else if constexpr (decltype(whole_next_tag)::value == 2) fetch_whole_masked(n0 + 128, nxt);
    else fetch(n0 + 128, nxt);
    const uint8_t *kb = mha_lds + buf * MHA8_TILE_LDS + r * MHA8_PITCH + h * 16;
    const uint8_t *vb = mha_lds + (2 + buf) * MHA8_TILE_LDS + r * MHA8_PITCH + h * 16;
    const float qk = qs * (KSF_AHEAD ? ksf_cur : ksf_load);
    if (KSF_AHEAD) ksf_cur = ksf_load;
    // ---- S^T = K . Q^T for the 128 kv positions of the tile (four 32-row fragments)
    i32x16 SI[4];
#pragma unroll
    for (int s4 = 0; s4 < 4; ++s4)
#pragma unroll
      for (int f = 0; f < 4; ++f) {
        const i32x4 KF = *reinterpret_cast<const i32x4 *>(kb + f * 32 * MHA8_PITCH + s4 * 32);
        if (s4 == 0)
          SI[f] = __builtin_amdgcn_mfma_i32_32x32x32_i8(KF, QF[s4], (i32x16)(0), 0, 0, 0);
        else
          SI[f] = __builtin_amdgcn_mfma_i32_32x32x32_i8(KF, QF[s4], SI[f], 0, 0, 0);
      }
    // ---- online softmax of the lane's row: its 64 values here, the other 64 in the lane 32 away
    float ST[4][16];
#pragma unroll
    for (int f = 0; f < 4; ++f)
#pragma unroll
      for (int e = 0; e < 16; ++e) ST[f][e] = (float)SI[f][e];
    const int left = (int)(a.Nkv - n0) - h * 4;  // kv positions of this tile that exist, seen from the lane's first one
    if (tail) {  // positions past Nkv take no part in the maximum
#pragma unroll
      for (int f = 0; f < 4; ++f)
#pragma unroll
        for (int e = 0; e < 16; ++e)
          if (f * 32 + (e >> 2) * 8 + (e & 3) >= left) ST[f][e] = -__builtin_inff();
    }
    // the maximum of s = float(S) * qk is taken over float(S): qk >= 0 keeps the order, qk < 0 reverses it
    float hi = -__builtin_inff(), lo = __builtin_inff();
#pragma unroll
    for (int f = 0; f < 4; ++f)
#pragma unroll
      for (int e = 0; e < 16; ++e) hi = __builtin_fmaxf(hi, ST[f][e]);
    if (qk < 0.0f) {
      asm volatile("" ::: "memory");
#pragma unroll
      for (int f = 0; f < 4; ++f)
#pragma unroll
        for (int e = 0; e < 16; ++e)
          lo = __builtin_fminf(lo, ST[f][e] == -__builtin_inff() ? __builtin_inff() : ST[f][e]);
    }
    const float smax = qk < 0.0f ? mha_halves_max(lo * qk) : mha_halves_max(hi * qk);
    const float m_new = __builtin_fmaxf(smax - MHA8_EXP_OFFSET, m_run);
    float lsum = 0.0f;
#pragma unroll
    for (int f = 0; f < 4; ++f)
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        ST[f][e] = __builtin_amdgcn_exp2f(__builtin_fmaf(ST[f][e], qk, -m_new));  // p <= 2^7.5
        lsum += ST[f][e];
      }
    if (tail) {  // p of the masked positions is 0 whatever qk is (-inf * 0 would be NaN)
      lsum = 0.0f;
#pragma unroll
      for (int f = 0; f < 4; ++f)
#pragma unroll
        for (int e = 0; e < 16; ++e) {
          if (f * 32 + (e >> 2) * 8 + (e & 3) >= left) ST[f][e] = 0.0f;
          lsum += ST[f][e];
        }
    }
    const float l_new = mha_halves_sum(lsum);
    const float alpha = __builtin_amdgcn_exp2f(m_run - m_new);
    l_run = __builtin_fmaf(l_run, alpha, l_new);
    m_run = m_new;
    if (__builtin_amdgcn_ballot_w64(alpha != 1.0f)) {  // else no row of this wave raised its maximum
#pragma unroll
      for (int fd = 0; fd < 4; ++fd)
#pragma unroll
        for (int e = 0; e < 16; ++e) OT[fd][e] *= alpha;
    }
    // ---- P -> e4m3, O^T += Vhat . Phat^T: one MFMA (k = 64: v_mfma_scale_f32_32x32x64_f8f6f4 with unit scales; lane
    // half h supplies 32 of the 64 k slots) per 64 kv positions and 32 rows of d
#pragma unroll
    for (int j2 = 0; j2 < 2; ++j2) {
      i32x8 PF;
#pragma unroll
      for (int g4 = 0; g4 < 4; ++g4) {  // the lane's four 16-group halves of these 64 positions, in the stored order of V:
        const float *pe = &ST[2 * j2 + (g4 >> 1)][8 * (g4 & 1)];  // e = 8 (g4 & 1) + {0, 1, 4, 5, 2, 3, 6, 7}
        int w0 = __builtin_amdgcn_cvt_pk_fp8_f32(pe[0], pe[1], 0, false);
        w0 = __builtin_amdgcn_cvt_pk_fp8_f32(pe[4], pe[5], w0, true);
        int w1 = __builtin_amdgcn_cvt_pk_fp8_f32(pe[2], pe[3], 0, false);
        w1 = __builtin_amdgcn_cvt_pk_fp8_f32(pe[6], pe[7], w1, true);
        PF[2 * g4] = w0;
        PF[2 * g4 + 1] = w1;
      }
#pragma unroll
      for (int fd = 0; fd < 4; ++fd) {
        const uint4 va = *reinterpret_cast<const uint4 *>(vb + fd * 32 * MHA8_PITCH + (2 * j2) * 32);
        const uint4 vc = *reinterpret_cast<const uint4 *>(vb + fd * 32 * MHA8_PITCH + (2 * j2 + 1) * 32);
        const i32x8 VF = {(int)va.x, (int)va.y, (int)va.z, (int)va.w, (int)vc.x, (int)vc.y, (int)vc.z, (int)vc.w};
        OT[fd] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(VF, PF, OT[fd], 0, 0, 0, 0x7f7f7f7f, 0, 0x7f7f7f7f);
      }
    }
    stage(buf ^ 1, nxt);
    __syncthreads();
  };
  int buf = 0;
  int64_t n0 = 0;
  using FetchTested = std::integral_constant<int, 0>;
  using FetchWhole = std::integral_constant<int, 1>;
  using FetchWholeMasked = std::integral_constant<int, 2>;
  if (a.Dp == 128 && a.Dv == 128)  // tiles followed by a whole tile: the fetch without tests
    for (; n0 + 256 <= a.Nkv; n0 += 128, buf ^= 1) tile_step(std::false_type{}, FetchWhole{}, n0, buf);
  else if constexpr (WAVES == 8)  // (the four-wave kernel has no registers to spare for a third copy of the loop)
    for (; n0 + 256 <= a.Nkv; n0 += 128, buf ^= 1) tile_step(std::false_type{}, FetchWholeMasked{}, n0, buf);
  for (; n0 + 128 <= a.Nkv; n0 += 128, buf ^= 1) tile_step(std::false_type{}, FetchTested{}, n0, buf);
  if (n0 < a.Nkv) tile_step(std::true_type{}, FetchTested{}, n0, buf);

  // ---- O = O * ((1 / l) * v_sf[d]) -> bf16
  const float rl = 1.0f / l_run;
  const float *vsf = a.v_sf + bh * a.Dvp;
  uint16_t ob[4][16];
#pragma unroll
  for (int fd = 0; fd < 4; ++fd)
#pragma unroll
    for (int q4 = 0; q4 < 4; ++q4) {
      const int d = fd * 32 + q4 * 8 + h * 4;  // four consecutive head dims; the scale row is padded to 16
      const float4 sv = d < a.Dvp ? *reinterpret_cast<const float4 *>(vsf + d) : make_float4(0.f, 0.f, 0.f, 0.f);
      const float sc[4] = {rl * sv.x, rl * sv.y, rl * sv.z, rl * sv.w};
#pragma unroll
      for (int e = 0; e < 4; ++e) ob[fd][4 * q4 + e] = __builtin_bit_cast(uint16_t, (__bf16)(OT[fd][4 * q4 + e] * sc[e]));
    }
  mha_store_rows(a.O + b * a.o_b + head * a.o_h, a.o_n, a.o_d, a.o_vec, (int64_t)blockIdx.x * (32 * WAVES) + wave * 32, a.Nq,
                 a.Dv, lane, mha_lds + wave * MHA_OUT_LDS, ob);
}

// Per-token-block int8 quantizer in front of it (python/ac4k_kernel/ops/attention.py:18-99, a Triton kernel in the
// reference): one scale = max|x| / 127 per block of `block` tokens of a head (all D columns), y = int8(trunc(x /
// scale)), 0 where the scale is 0; y is [B, H, N, Dp] with pad columns 0, the scales [B, H, ceil(N / block)].
__global__ __launch_bounds__(256) void quantize_int8_token_block_kernel(int8_t *__restrict__ y, float *__restrict__ scale,
                                                                        const uint16_t *__restrict__ x, int64_t s_b,
                                                                        int64_t s_h, int64_t s_n, int64_t H, int64_t N,
                                                                        int D, int Dp, int block, int vec) {
  __shared__ uint32_t wmax[4];
  const int64_t nb = gridDim.x, blk = blockIdx.x, head = blockIdx.y, b = blockIdx.z;
  const int64_t n0 = blk * block;
  const int rows = (int)((N - n0) < block ? (N - n0) : block);
  const uint16_t *src = x + b * s_b + head * s_h + n0 * s_n;
  int8_t *dst = y + ((b * H + head) * N + n0) * Dp;
  uint32_t mx = 0;
  // rows of whole 16-byte vectors (D % 8 == 0, aligned), at most eight vectors per thread: the block is read once,
  // into registers
  const int vpr = D / 8, nvec = rows * vpr;
  if (vec && nvec <= 8 * 256) {
    uint4 v[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const int i = threadIdx.x + j * 256;
      v[j] = make_uint4(0, 0, 0, 0);
      if (i < nvec) v[j] = ld_stream_u4(src + (int64_t)(i / vpr) * s_n + (i % vpr) * 8);
      mx = umax32(mx, absmax_bf16x8(v[j]));
    }
    mx = group_umax<64>(mx);
    if ((threadIdx.x & 63) == 0) wmax[threadIdx.x >> 6] = mx;
    __syncthreads();
    mx = umax32(umax32(wmax[0], wmax[1]), umax32(wmax[2], wmax[3]));
    const float sc = bf16_bits_to_f32(mx) / 127.0f;
    if (threadIdx.x == 0) scale[(b * H + head) * nb + blk] = sc;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const int i = threadIdx.x + j * 256;
      if (i >= nvec) continue;
      const uint32_t w[4] = {v[j].x, v[j].y, v[j].z, v[j].w};
      uint32_t o2[2] = {0, 0};
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const float xe = bf16_bits_to_f32((w[e >> 1] >> (16 * (e & 1))) & 0xffffu);
        const int q = sc != 0.0f ? (int)(xe / sc) : 0;  // toward zero; |q| <= 127 up to rounding
        o2[e >> 2] |= ((uint32_t)q & 0xffu) << (8 * (e & 3));
      }
      *reinterpret_cast<uint2 *>(dst + (int64_t)(i / vpr) * Dp + (i % vpr) * 8) = make_uint2(o2[0], o2[1]);
    }
    if (Dp != D) {  // D % 16 == 8: eight pad columns per row
      for (int rr = threadIdx.x; rr < rows; rr += 256) *reinterpret_cast<uint2 *>(dst + (int64_t)rr * Dp + D) = make_uint2(0, 0);
    }
    return;
  }
  for (int i = threadIdx.x; i < rows * D; i += 256) mx = umax32(mx, src[(int64_t)(i / D) * s_n + i % D] & 0x7fffu);
  mx = group_umax<64>(mx);
  if ((threadIdx.x & 63) == 0) wmax[threadIdx.x >> 6] = mx;
  __syncthreads();
  mx = umax32(umax32(wmax[0], wmax[1]), umax32(wmax[2], wmax[3]));
  const float sc = bf16_bits_to_f32(mx) / 127.0f;
  if (threadIdx.x == 0) scale[(b * H + head) * nb + blk] = sc;
  for (int i = threadIdx.x; i < rows * Dp; i += 256) {
    const int rr = i / Dp, c = i % Dp;
    float q = 0.0f;
    if (c < D && sc != 0.0f) q = bf16_bits_to_f32(src[(int64_t)rr * s_n + c]) / sc;
    dst[i] = (int8_t)(int)q;  // toward zero; |q| <= 127 up to rounding
  }
}

}  // namespace ac4k

using namespace ac4k;

extern "C" __attribute__((visibility("default"))) int ac4k_mha_nvfp4_fwd(
    void *O, int64_t o_b_stride, int64_t o_h_stride, int64_t o_n_stride, int64_t o_d_stride, const void *q, const void *q_sf,
    const float *q_gs, const void *k, const void *k_sf, const float *k_gs, const void *v, const void *v_sf, const float *v_gs,
    int64_t B, int64_t H, int64_t Nq, int64_t Nkv, int64_t Dqk, int64_t Dv, float sm_scale, ac4k_stream_t stream) {
  AC4K_REQUIRE(O && q && q_sf && q_gs && k && k_sf && k_gs && v && v_sf && v_gs, "null pointer argument");
  AC4K_REQUIRE(B >= 1 && H >= 1 && Nq >= 1 && Nkv >= 1, "B, H, Nq, Nkv must be positive (B=%lld H=%lld Nq=%lld Nkv=%lld)",
               (long long)B, (long long)H, (long long)Nq, (long long)Nkv);
  AC4K_REQUIRE(Dqk % 16 == 0, "Dqk must be multiple of 16");
  AC4K_REQUIRE(Dqk <= 128 && Dv <= 128, "Dqk and Dv must not exceed 128");
  AC4K_REQUIRE(Dqk % 64 == 0 && Dqk >= 64 && Dv >= 1,
               "Dqk must be 64 or 128 (packed rows of whole 64-chunks, as the quantizer writes them) and Dv positive (Dqk=%lld Dv=%lld)",
               (long long)Dqk, (long long)Dv);
  AC4K_REQUIRE((((uintptr_t)q | (uintptr_t)k | (uintptr_t)v) & 15) == 0 && (((uintptr_t)q_sf | (uintptr_t)k_sf | (uintptr_t)v_sf) & 3) == 0,
               "q, k, v must be 16-byte aligned and the scale tensors 4-byte aligned");
  AC4K_REQUIRE(H <= 65535 && B <= 65535 && ceil_div(Nq, 128) < (1ll << 31), "problem too large");
  AC4K_REQUIRE(o_b_stride >= 0 && o_h_stride >= 0 && o_n_stride >= 1 && o_d_stride >= 1, "strides of O must be positive");
  MhaArgs a{static_cast<uint16_t *>(O), o_b_stride, o_h_stride, o_n_stride, o_d_stride,
            static_cast<const uint8_t *>(q), static_cast<const uint8_t *>(k), static_cast<const uint8_t *>(v),
            static_cast<const uint8_t *>(q_sf), static_cast<const uint8_t *>(k_sf), static_cast<const uint8_t *>(v_sf),
            q_gs, k_gs, v_gs, H, Nq, Nkv, align_up(Nq, 16), align_up(Nkv, 16), align_up(Nkv, 64), (int)(Dqk / 64), (int)Dv,
            (int)align_up(Dv, 16), sm_scale,
            (o_d_stride == 1 && Dv % 8 == 0 && ((uintptr_t)O & 15) == 0 && o_b_stride % 8 == 0 && o_h_stride % 8 == 0 && o_n_stride % 8 == 0) ? 1 : 0};
  // 256 query rows per workgroup unless that leaves most of the GPU's 256 CUs without one
  const bool wide = ceil_div(Nq, 256) * H * B >= 192 || ceil_div(Nq, 128) * H * B <= ceil_div(Nq, 256) * H * B;
  auto kern = wide ? mha_nvfp4_fwd_kernel<8> : mha_nvfp4_fwd_kernel<4>;
  {  // more than 64 KB of dynamic LDS has to be allowed once per device and kernel
    static std::atomic<uint32_t> lds_done[2] = {{0}, {0}};
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) dev = 0;
    const uint32_t bit = 1u << (dev & 31);
    if (!(lds_done[wide].load(std::memory_order_relaxed) & bit)) {
      hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                         MHA_LDS_BYTES);
      if (e != hipSuccess) return set_error("hipFuncSetAttribute(LDS=%d): %s", MHA_LDS_BYTES, hipGetErrorString(e));
      lds_done[wide].fetch_or(bit, std::memory_order_relaxed);
    }
  }
  const int rows = wide ? 256 : 128;
  hipLaunchKernelGGL(kern, dim3((unsigned)ceil_div(Nq, rows), (unsigned)H, (unsigned)B), dim3(rows * 2), MHA_LDS_BYTES,
                     (hipStream_t)stream, a);
  return check_launch("ac4k_mha_nvfp4_fwd");
}

// Replaces ac4k::mha_int8_x_fp8_fwd (lib/cuda/sm120/mha_int8_x_fp8.cu:979-1137).
extern "C" __attribute__((visibility("default"))) int ac4k_mha_int8_x_fp8_fwd(
    void *O, int64_t o_b_stride, int64_t o_h_stride, int64_t o_n_stride, int64_t o_d_stride, const void *q,
    const float *q_sf, int q_quantize_block_size, const void *k, const float *k_sf, int k_quantize_block_size, const void *v,
    const float *v_sf, int64_t B, int64_t H, int64_t Nq, int64_t Nkv, int64_t Dqk, int64_t Dv, float sm_scale,
    ac4k_stream_t stream) {
  AC4K_REQUIRE(O && q && q_sf && k && k_sf && v && v_sf, "null pointer argument");
  AC4K_REQUIRE(B >= 1 && H >= 1 && Nq >= 1 && Nkv >= 1, "B, H, Nq, Nkv must be positive (B=%lld H=%lld Nq=%lld Nkv=%lld)",
               (long long)B, (long long)H, (long long)Nq, (long long)Nkv);
  AC4K_REQUIRE(Dqk % 16 == 0, "Dqk must be multiple of 16");
  AC4K_REQUIRE(Dqk <= 128 && Dv <= 128, "Dqk and Dv must not exceed 128");
  AC4K_REQUIRE(q_quantize_block_size == 32 || q_quantize_block_size == 64, "q_quantize_block_size must be 32 or 64 (got %d)",
               q_quantize_block_size);
  AC4K_REQUIRE(k_quantize_block_size == 128, "k_quantize_block_size must be 128 (got %d)", k_quantize_block_size);
  AC4K_REQUIRE(Dqk >= 16 && Dv >= 1, "Dqk and Dv must be positive");
  AC4K_REQUIRE((((uintptr_t)q | (uintptr_t)k | (uintptr_t)v | (uintptr_t)v_sf) & 15) == 0,
               "q, k, v and v_sf must be 16-byte aligned");
  AC4K_REQUIRE(H <= 65535 && B <= 65535 && ceil_div(Nq, 128) < (1ll << 31), "problem too large");
  AC4K_REQUIRE(o_b_stride >= 0 && o_h_stride >= 0 && o_n_stride >= 1 && o_d_stride >= 1, "strides of O must be positive");
  Mha8Args a{static_cast<uint16_t *>(O), o_b_stride, o_h_stride, o_n_stride, o_d_stride,
             static_cast<const int8_t *>(q), static_cast<const int8_t *>(k), static_cast<const uint8_t *>(v),
             q_sf, k_sf, v_sf, H, Nq, Nkv, align_up(Nkv, 16), ceil_div(Nq, q_quantize_block_size), ceil_div(Nkv, 128),
             (int)Dqk, (int)Dv, (int)align_up(Dv, 16), q_quantize_block_size, sm_scale,
             (o_d_stride == 1 && Dv % 8 == 0 && ((uintptr_t)O & 15) == 0 && o_b_stride % 8 == 0 && o_h_stride % 8 == 0 && o_n_stride % 8 == 0) ? 1 : 0};
  const bool wide = ceil_div(Nq, 256) * H * B >= 192 || ceil_div(Nq, 128) * H * B <= ceil_div(Nq, 256) * H * B;
  auto kern = wide ? mha_int8_x_fp8_fwd_kernel<8> : mha_int8_x_fp8_fwd_kernel<4>;
  {  // more than 64 KB of dynamic LDS has to be allowed once per device and kernel
    static std::atomic<uint32_t> lds_done[2] = {{0}, {0}};
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) dev = 0;
    const uint32_t bit = 1u << (dev & 31);
    if (!(lds_done[wide].load(std::memory_order_relaxed) & bit)) {
      hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                         MHA8_LDS_BYTES);
      if (e != hipSuccess) return set_error("hipFuncSetAttribute(LDS=%d): %s", MHA8_LDS_BYTES, hipGetErrorString(e));
      lds_done[wide].fetch_or(bit, std::memory_order_relaxed);
    }
  }
  const int rows = wide ? 256 : 128;
  hipLaunchKernelGGL(kern, dim3((unsigned)ceil_div(Nq, rows), (unsigned)H, (unsigned)B), dim3(rows * 2), MHA8_LDS_BYTES,
                     (hipStream_t)stream, a);
  return check_launch("ac4k_mha_int8_x_fp8_fwd");
}

// Replaces _int8_quantize / _triton_block_token_quantize (python/ac4k_kernel/ops/attention.py:18-99): x bf16 with element
// strides (s_b, s_h, s_n, 1) over [B, H, N, D] -> y int8 [B, H, N, align_up(D, 16)], scale fp32 [B, H, ceil(N / block)].
extern "C" __attribute__((visibility("default"))) int ac4k_quantize_int8_token_block_bf16(
    void *y, float *scale, const void *x, int64_t B, int64_t H, int64_t N, int64_t D, int64_t s_b, int64_t s_h, int64_t s_n,
    int block, ac4k_stream_t stream) {
  AC4K_REQUIRE(y && scale && x, "null pointer argument");
  AC4K_REQUIRE(B >= 1 && H >= 1 && N >= 1 && D >= 1, "B, H, N, D must be positive");
  AC4K_REQUIRE(block >= 16 && (block & (block - 1)) == 0, "the block size must be a power of two, at least 16 (got %d)", block);
  AC4K_REQUIRE(D <= 1024 && block <= 1024, "D and the block size must not exceed 1024");
  AC4K_REQUIRE(H <= 65535 && B <= 65535 && ceil_div(N, (int64_t)block) < (1ll << 31), "problem too large");
  hipLaunchKernelGGL(quantize_int8_token_block_kernel, dim3((unsigned)ceil_div(N, (int64_t)block), (unsigned)H, (unsigned)B),
                     dim3(256), 0, (hipStream_t)stream, static_cast<int8_t *>(y), scale, static_cast<const uint16_t *>(x), s_b,
                     s_h, s_n, H, N, (int)D, (int)align_up(D, 16), block,
                     (D % 8 == 0 && ((uintptr_t)x & 15) == 0 && s_b % 8 == 0 && s_h % 8 == 0 && s_n % 8 == 0) ? 1 : 0);
  return check_launch("ac4k_quantize_int8_token_block_bf16");
}
