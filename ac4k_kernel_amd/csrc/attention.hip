// NVFP4 attention forward for gfx950, head dim 128:  O = softmax(Q K^T * sm_scale) V on NVFP4 operands.
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
// A first, untuned kernel: every wave owns 32 query rows and reads its operands straight from global
// memory (the four waves of a workgroup share the K and V tiles through the caches).
//
// The MFMAs are issued so that a lane owns ONE query row: S^T = Khat . Qhat^T and O^T = Vhat . Phat^T
// (v_mfma_f32_32x32x16_f16, exact fp16 decode as in the linear).  Lane (r, h) of a wave then holds, per
// 32-row kv fragment, the 16 values S[r][8g + 4h + j]: exactly one P block, so its maximum, scale and
// nibbles are formed inside the lane, and the row maximum and row sum need one exchange between the two
// halves of the wave.  The k slots of the second product are paired through the stored (swizzled) order
// of V: slot s of step t holds kv position 8 (2t + (s>>1 & 1)) + 4h + 2 (s>>2) + (s & 1).
#include "ac4k_common.h"

namespace ac4k {

struct MhaArgs {
  uint16_t *O;
  int64_t o_b, o_h, o_n, o_d;  // element strides of O [B, H, Nq, 128]
  const uint8_t *q, *k, *v, *q_sf, *k_sf, *v_sf;
  const float *q_gs, *k_gs, *v_gs;
  int64_t H, Nq, Nkv, Nqp, Nkvp, Nkv64;  // padded: rows of the Q / K scale planes (16), stored kv length of V (64)
  float sm_scale;
};

constexpr int MHA_D = 128;
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

// A row-major packed row (Q or K): the lane's 32 elements [32 h, 32 h + 32) of 64-chunk c, and the two block
// scales that go with them, decoded into the four 16-k operands of that chunk.  `valid` false: zeros.
__device__ __forceinline__ void mha_load_row_chunk(const uint8_t *row, const uint8_t *sf_chunk_row, int c, int h,
                                                   bool valid, f16x8 (&out)[4]) {
  uint4 w = make_uint4(0, 0, 0, 0);
  uint32_t sc = 0;
  if (valid) {
    w = *reinterpret_cast<const uint4 *>(row + c * 32 + h * 16);
    sc = *reinterpret_cast<const uint16_t *>(sf_chunk_row + 2 * h);
  }
  const f16x2 s2 = __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(sc, 1.0f, false);
  const f16x2 lo = {s2.x, s2.x}, hi = {s2.y, s2.y};
  out[0] = mha_decode8(w.x, lo);
  out[1] = mha_decode8(w.y, lo);
  out[2] = mha_decode8(w.z, hi);
  out[3] = mha_decode8(w.w, hi);
}

__device__ __forceinline__ float mha_xor32(float x) {  // value of the lane 32 away
  return __shfl_xor(x, 32, 64);
}

__global__ __launch_bounds__(256) void mha_nvfp4_fwd_d128_kernel(MhaArgs a) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, r = lane & 31, h = lane >> 5;
  const int64_t b = blockIdx.z, head = blockIdx.y, bh = b * a.H + head;
  const int64_t m = (int64_t)blockIdx.x * 128 + wave * 32 + r;   // this lane's query row
  const int64_t mq = m < a.Nq ? m : a.Nq - 1;                    // rows past Nq read the last row; never stored

  // Qhat of the lane's row: 8 operands of 16 k (chunk c, sub-step s), kept for the whole kernel
  f16x8 QF[2][4];
#pragma unroll
  for (int c = 0; c < 2; ++c)
    mha_load_row_chunk(a.q + (bh * a.Nq + mq) * (MHA_D / 2), a.q_sf + ((bh * 2 + c) * a.Nqp + mq) * 4, c, h, true, QF[c]);

  const float qk_scale = (*a.q_gs) * (*a.k_gs) * a.sm_scale;
  float m_run = -__builtin_inff(), l_run = 0.0f;
  f32x16 OT[4];  // O^T: d = 32 fd + 8 (e >> 2) + 4 h + (e & 3), for the lane's query row
#pragma unroll
  for (int fd = 0; fd < 4; ++fd)
#pragma unroll
    for (int e = 0; e < 16; ++e) OT[fd][e] = 0.0f;

  const int64_t v_row_bytes = a.Nkv64 / 2, v_chunks = a.Nkv64 / 64;
  for (int64_t n0 = 0; n0 < a.Nkv; n0 += 128) {
    // ---- S^T = Khat . Qhat^T for the 128 kv positions of the tile (four 32-row fragments)
    f32x16 ST[4];
#pragma unroll
    for (int f = 0; f < 4; ++f) {
#pragma unroll
      for (int e = 0; e < 16; ++e) ST[f][e] = 0.0f;
      const int64_t n = n0 + f * 32 + r;
      const bool valid = n < a.Nkv;  // rows past Nkv are zero: S = 0 there
      const int64_t nn = valid ? n : 0;
#pragma unroll
      for (int c = 0; c < 2; ++c) {
        f16x8 KF[4];
        mha_load_row_chunk(a.k + (bh * a.Nkv + nn) * (MHA_D / 2), a.k_sf + ((bh * 2 + c) * a.Nkvp + nn) * 4, c, h, valid, KF);
#pragma unroll
        for (int s = 0; s < 4; ++s) ST[f] = __builtin_amdgcn_mfma_f32_32x32x16_f16(KF[s], QF[c][s], ST[f], 0, 0, 0);
      }
    }
    // ---- online softmax of the lane's row: its 64 values here, the other 64 in the lane 32 away
    float mx = m_run;
#pragma unroll
    for (int f = 0; f < 4; ++f)
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        ST[f][e] *= qk_scale;
        mx = __builtin_fmaxf(mx, ST[f][e]);
      }
    const float m_new = __builtin_fmaxf(mx, mha_xor32(mx));
    const float ml = m_new * MHA_LOG2E;
    float lsum = 0.0f;
#pragma unroll
    for (int f = 0; f < 4; ++f)
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        ST[f][e] = __builtin_amdgcn_exp2f(ST[f][e] * MHA_LOG2E - ml);  // p
        lsum += ST[f][e];
      }
    float l_new = lsum + mha_xor32(lsum);
    if (n0 + 128 > a.Nkv)  // the zero-filled positions of the last tile each added exp(0 - m)
      l_new -= (float)(n0 + 128 - a.Nkv) / __builtin_amdgcn_exp2f(ml);
    const float alpha = __builtin_amdgcn_exp2f(m_run * MHA_LOG2E - ml);
    l_run = alpha * l_run + l_new;
    m_run = m_new;
#pragma unroll
    for (int fd = 0; fd < 4; ++fd)
#pragma unroll
      for (int e = 0; e < 16; ++e) OT[fd][e] *= alpha;

    // ---- P -> NVFP4 (the lane's 16 values of a fragment are one block), then O^T += Vhat . Phat^T
#pragma unroll
    for (int f = 0; f < 4; ++f) {
      float bm = ST[f][0];
#pragma unroll
      for (int e = 1; e < 16; ++e) bm = __builtin_fmaxf(bm, ST[f][e]);
      const uint32_t code = f32_to_ue4m3_satfinite(MHA_P_ALPHA * (bm * 0.16666666666666666f));
      const float s = e4m3_to_f32(code);
      const float o = s != 0.0f ? MHA_P_ALPHA * (1.0f / s) : 0.0f;
      const _Float16 sh = (_Float16)s;  // an e4m3 value: exact in fp16
      const f16x2 psc = {sh, sh};
      // the 32-group of V that holds these kv positions: 16 stored bytes per d row
      const int64_t g32 = (n0 + f * 32) / 32;
      const bool v_valid = (n0 + f * 32) < a.Nkv64;
#pragma unroll
      for (int t = 0; t < 2; ++t) {
        // k slots of this step in the order the stored nibbles of V come in (see the header)
        const float pv[8] = {ST[f][8 * t + 0] * o, ST[f][8 * t + 1] * o, ST[f][8 * t + 4] * o, ST[f][8 * t + 5] * o,
                             ST[f][8 * t + 2] * o, ST[f][8 * t + 3] * o, ST[f][8 * t + 6] * o, ST[f][8 * t + 7] * o};
        const f16x8 PF = mha_decode8(f32x8_to_e2m1x8(pv), psc);
#pragma unroll
        for (int fd = 0; fd < 4; ++fd) {
          const int64_t d = fd * 32 + r;
          uint32_t w = 0, vs = 0;
          if (v_valid) {
            const uint32_t *grp = reinterpret_cast<const uint32_t *>(a.v + (bh * MHA_D + d) * v_row_bytes + g32 * 16);
            const uint32_t lo = (grp[2 * h] >> (16 * t)) & 0xffffu, hi = (grp[2 * h + 1] >> (16 * t)) & 0xffffu;
            w = lo | (hi << 16);
            vs = a.v_sf[((bh * v_chunks + g32 / 2) * MHA_D + d) * 4 + 2 * (g32 & 1) + h];
          }
          const f16x2 v2 = __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(vs, 1.0f, false);
          const f16x2 vsc = {v2.x, v2.x};
          OT[fd] = __builtin_amdgcn_mfma_f32_32x32x16_f16(mha_decode8(w, vsc), PF, OT[fd], 0, 0, 0);
        }
      }
    }
  }

  // ---- O = O * ((1/l) * (1/2688) * v_gs) -> bf16
  if (m >= a.Nq) return;
  const float scale = (1.0f / l_run) * (1.0f / MHA_P_ALPHA) * (*a.v_gs);
  uint16_t *orow = a.O + b * a.o_b + head * a.o_h + m * a.o_n;
#pragma unroll
  for (int fd = 0; fd < 4; ++fd)
#pragma unroll
    for (int e = 0; e < 16; ++e) {
      const int d = fd * 32 + (e >> 2) * 8 + h * 4 + (e & 3);
      orow[d * a.o_d] = __builtin_bit_cast(uint16_t, (__bf16)(OT[fd][e] * scale));
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
  AC4K_REQUIRE(Dqk == MHA_D && Dv == MHA_D, "this build of the attention kernel takes head dim 128 only (Dqk=%lld Dv=%lld)",
               (long long)Dqk, (long long)Dv);
  AC4K_REQUIRE((((uintptr_t)q | (uintptr_t)k | (uintptr_t)v) & 15) == 0 && (((uintptr_t)q_sf | (uintptr_t)k_sf | (uintptr_t)v_sf) & 3) == 0,
               "q, k, v must be 16-byte aligned and the scale tensors 4-byte aligned");
  AC4K_REQUIRE(H <= 65535 && B <= 65535 && ceil_div(Nq, 128) < (1ll << 31), "problem too large");
  AC4K_REQUIRE(o_b_stride >= 0 && o_h_stride >= 0 && o_n_stride >= 1 && o_d_stride >= 1, "strides of O must be positive");
  MhaArgs a{static_cast<uint16_t *>(O), o_b_stride, o_h_stride, o_n_stride, o_d_stride,
            static_cast<const uint8_t *>(q), static_cast<const uint8_t *>(k), static_cast<const uint8_t *>(v),
            static_cast<const uint8_t *>(q_sf), static_cast<const uint8_t *>(k_sf), static_cast<const uint8_t *>(v_sf),
            q_gs, k_gs, v_gs, H, Nq, Nkv, align_up(Nq, 16), align_up(Nkv, 16), align_up(Nkv, 64), sm_scale};
  hipLaunchKernelGGL(mha_nvfp4_fwd_d128_kernel, dim3((unsigned)ceil_div(Nq, 128), (unsigned)H, (unsigned)B), dim3(256), 0,
                     (hipStream_t)stream, a);
  return check_launch("ac4k_mha_nvfp4_fwd");
}
