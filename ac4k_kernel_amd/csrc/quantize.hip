// BF16 -> NVFP4 / FP8E4M3 / INT8 quantizers and the global-scale reduction for gfx950.
//
// Arithmetic follows the reference kernels' operation order in IEEE round-to-nearest fp32:
//   global scale  python/ac4k_kernel/ops/quant.py:33-59
//   nvfp4         lib/cuda/sm120/quantize_nvfp4.cu:49-157
//   fp8 per row   lib/cuda/sm120/quantize_fp8.cu:57-185
//   int8 per row  lib/cuda/sm120/quantize_int8.cu:61-168
// The reference's rcp.approx / fast-math divisions are replaced by correctly rounded
// divisions, and the file is compiled with -ffp-contract=off so that the separate
// multiplies of the spec stay separate.
//
// All kernels are bandwidth-bound: the row-major paths move 16 bytes per lane per load,
// reduce amax inside the wavefront with DPP, and store packed words.
#include <string.h>

#include <atomic>
#include <mutex>
#include <type_traits>

#include "ac4k_common.h"

namespace ac4k {

// ===========================================================================
// global scale:  *gs = fp32(max |x|) / max_scale
// ===========================================================================

__global__ void zero_u32_kernel(uint32_t *p) { *p = 0u; }

constexpr int AMAX_THREADS = 256;
constexpr int AMAX_UNROLL = 4;
constexpr int AMAX_MAX_BLOCKS = 1024;  // four workgroups per CU

// |x| maximum of this block's share of x[0..n) as a bf16 bit pattern (valid in thread 0).
__device__ __forceinline__ uint32_t block_absmax_bf16(const uint16_t *__restrict__ x, int64_t n, int64_t head,
                                                     int64_t nvec) {
  // x[0..head) and the tail after the vectors are handled by scalar loads of block 0; the
  // 16-byte aligned middle is cut into one contiguous span per block (measured on 774 MB: 129 us
  // against 145 us for grid-stride loads), streamed with uint4 loads, four in flight per lane.
  // Plain (cached) loads: the quantize pass that follows reads the same data again.
  const uint4 *xv = reinterpret_cast<const uint4 *>(x + head);
  uint32_t m = 0;
  constexpr int64_t STEP = (int64_t)AMAX_THREADS * AMAX_UNROLL;
  const int64_t span = ceil_div(ceil_div(nvec, (int64_t)gridDim.x), STEP) * STEP;
  const int64_t beg = (int64_t)blockIdx.x * span;
  const int64_t end = beg + span < nvec ? beg + span : nvec;
  int64_t i = beg + threadIdx.x;
  for (; i + (AMAX_UNROLL - 1) * AMAX_THREADS < end; i += STEP) {
    uint4 v[AMAX_UNROLL];
#pragma unroll
    for (int u = 0; u < AMAX_UNROLL; ++u) v[u] = xv[i + u * AMAX_THREADS];
#pragma unroll
    for (int u = 0; u < AMAX_UNROLL; ++u) m = umax32(m, absmax_bf16x8(v[u]));
  }
  for (; i < end; i += AMAX_THREADS) m = umax32(m, absmax_bf16x8(xv[i]));
  if (blockIdx.x == 0) {
    for (int64_t j = threadIdx.x; j < head; j += AMAX_THREADS) m = umax32(m, x[j] & 0x7fffu);
    for (int64_t j = head + nvec * 8 + threadIdx.x; j < n; j += AMAX_THREADS)
      m = umax32(m, x[j] & 0x7fffu);
  }
  m = group_umax<64>(m);
  __shared__ uint32_t part[AMAX_THREADS / 64];
  if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = m;
  __syncthreads();
  if (threadIdx.x == 0) {
#pragma unroll
    for (int w = 1; w < AMAX_THREADS / 64; ++w) m = umax32(m, part[w]);
  }
  return m;
}

// Global scale without any memory of the library's own: *gs is zeroed by a fill kernel, then every
// block folds its quotient in with an atomic max - but only when the quotient beats the value it
// reads first, so that after the first few blocks almost none touches the (cross-XCD, serialising)
// atomic.  Division is monotone, so the max of the per-block quotients is the quotient of the max;
// non-negative floats order like unsigned integers.
__global__ __launch_bounds__(AMAX_THREADS) void amax_scale_bf16_atomic_kernel(
    uint32_t *__restrict__ gs_bits, const uint16_t *__restrict__ x, int64_t n, int64_t head, int64_t nvec,
    float max_scale) {
  const uint32_t m = block_absmax_bf16(x, n, head, nvec);
  if (threadIdx.x == 0) {
    const float q = bf16_bits_to_f32(m) / max_scale;
    const uint32_t qb = __float_as_uint(q);
    if ((q > 0.0f || q != q) && qb > *(volatile uint32_t *)gs_bits) atomicMax(gs_bits, qb);
  }
}

// ===========================================================================
// nvfp4
// ===========================================================================

struct QuantGeom {
  int64_t d1, R, K, Kp, Rp;
  int64_t s0, s1, sR, sK;
  int64_t lead0;  // first leading index of this launch (grids carry at most 65535 of them)
  // cross-major kernels: the leading index, not the position along the reduce dim, is the fast grid
  // index (its stride is the smaller one, so workgroups that run together read neighbouring memory)
  int lead_fast = 0;
};

// grid indices of the cross-major kernels: (position along the reduce dim, leading index)
struct CrossMajorIdx {
  int64_t kblock, lead;
};
__device__ __forceinline__ CrossMajorIdx crossmajor_idx(const QuantGeom &g) {
  return g.lead_fast ? CrossMajorIdx{(int64_t)blockIdx.z, (int64_t)blockIdx.x + g.lead0}
                     : CrossMajorIdx{(int64_t)blockIdx.x, (int64_t)blockIdx.z + g.lead0};
}
static dim3 crossmajor_grid(const QuantGeom &g, int64_t kblocks, int64_t rowblocks, int64_t lead) {
  return g.lead_fast ? dim3((unsigned)lead, (unsigned)rowblocks, (unsigned)kblocks)
                     : dim3((unsigned)kblocks, (unsigned)rowblocks, (unsigned)lead);
}
// the leading index goes first when its stride is below the reduce stride (and the grid's z can hold
// the reduce blocks)
static int crossmajor_lead_fast(int64_t d1, int64_t s1, int64_t sK, int64_t kblocks) {
  return d1 > 1 && s1 < sK && kblocks <= 65535;
}

// The swizzles on a contiguous reduce dim are small in-register transpositions between adjacent
// lanes (a lane holds 8 consecutive elements = 4 dwords of 2).
// nvfp4, 32-groups = 4 lanes: out[t*8 + q*2 + r] = in[q*8 + t*2 + r], i.e. lane t / dword q receives
// lane q / dword t: a 4x4 transpose of dwords inside the quad, done as two butterfly stages.
__device__ __forceinline__ uint4 swizzle_nvfp4_quad(uint4 v, int lane) {
  uint32_t d[4] = {v.x, v.y, v.z, v.w};
  const bool o1 = lane & 1, o2 = lane & 2;
#pragma unroll
  for (int b = 0; b < 2; ++b) {  // 2x2 blocks: (q even, t odd) <-> (q odd, t even)
    const uint32_t got = dpp_u32<DPP_QUAD_XOR1>(o1 ? d[2 * b] : d[2 * b + 1]);
    if (o1) d[2 * b] = got; else d[2 * b + 1] = got;
  }
#pragma unroll
  for (int c = 0; c < 2; ++c) {  // off-diagonal 2x2 blocks: (q < 2, t >= 2) <-> (q >= 2, t < 2)
    const uint32_t got = dpp_u32<DPP_QUAD_XOR2>(o2 ? d[c] : d[c + 2]);
    if (o2) d[c] = got; else d[c + 2] = got;
  }
  return make_uint4(d[0], d[1], d[2], d[3]);
}
// fp8, 16-groups = 2 lanes: out[t*4 + q*2 + r] = in[q*8 + t*2 + r]: lane 0 gets dwords (a0, b0, a1, b1)
// and lane 1 gets (a2, b2, a3, b3) of the pair's inputs a (lane 0) and b (lane 1).
__device__ __forceinline__ uint4 swizzle_fp8_pair(uint4 v, int lane) {
  const bool o = lane & 1;
  // each lane needs two dwords of its partner: lane 0 wants b0, b1; lane 1 wants a2, a3
  const uint32_t g0 = dpp_u32<DPP_QUAD_XOR1>(o ? v.x : v.z);  // lane 0 receives b.x, lane 1 receives a.z
  const uint32_t g1 = dpp_u32<DPP_QUAD_XOR1>(o ? v.y : v.w);  // lane 0 receives b.y, lane 1 receives a.w
  return o ? make_uint4(g0, v.z, g1, v.w) : make_uint4(v.x, g0, v.y, g1);
}

// Row-major fast path: reduce dim contiguous, K % 8 == 0, 16-byte aligned rows.
// A lane owns 8 consecutive elements (half a 16-block); lane pairs share the block amax
// through one DPP quad_perm; the four scale bytes of a 64-chunk are gathered into the
// chunk's first lane with three DPP row shifts and stored as one dword.
//   CPR  = 64-element chunks per wave row (8*CPR lanes per row, 8/CPR rows per wave pass)
//   ITER = wave passes per workgroup (independent loads in flight per lane)
template <int CPR, int ITER, bool SWIZZLE>
__global__ __launch_bounds__(256) void quantize_nvfp4_rowmajor_kernel(
    uint8_t *__restrict__ out, uint8_t *__restrict__ sf, const uint16_t *__restrict__ in, const float *__restrict__ gs_ptr,
    QuantGeom g) {
  __shared__ float lut[128];
  load_rcp_table(lut);
  const float alpha = 1.0f / *gs_ptr;
  constexpr int LPR = 8 * CPR;   // lanes per row
  constexpr int RW = 64 / LPR;   // rows per wave pass
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int64_t lead = blockIdx.y + g.lead0;
  const int64_t ngroups = ceil_div(g.Kp / 64, CPR);  // chunk groups along the reduce dim
  const int64_t k = ((int64_t)(blockIdx.x % ngroups) * LPR + (lane % LPR)) * 8;
  const int64_t row0 = (int64_t)(blockIdx.x / ngroups) * (4 * RW * ITER) + lane / LPR;
  if (k >= g.Kp) return;
  const uint16_t *src = in + (lead / g.d1) * g.s0 + (lead % g.d1) * g.s1 + k;
  const bool kvalid = k < g.K;

  uint4 v[ITER];
#pragma unroll
  for (int it = 0; it < ITER; ++it) {
    const int64_t r = row0 + (int64_t)(it * 4 + wave) * RW;
    v[it] = make_uint4(0, 0, 0, 0);
    if (kvalid && r < g.R)
      v[it] = ld_stream_u4(src + r * g.sR);
    if (SWIZZLE) v[it] = swizzle_nvfp4_quad(v[it], lane);
  }
#pragma unroll
  for (int it = 0; it < ITER; ++it) {
    const int64_t r = row0 + (int64_t)(it * 4 + wave) * RW;
    uint32_t m = absmax_bf16x8(v[it]);
    m = umax32(m, dpp_u32<DPP_QUAD_XOR1>(m));
    uint32_t code;
    float o = nvfp4_block_scale(bf16_bits_to_f32(m), alpha, lut, code);
    if (r >= g.R) code = 0;  // pad rows carry zero scales
    uint32_t packed = nvfp4_pack8(v[it], o);
    uint32_t sfw = code | (dpp_u32<DPP_ROW_SHL(2)>(code) << 8) | (dpp_u32<DPP_ROW_SHL(4)>(code) << 16) |
                   (dpp_u32<DPP_ROW_SHL(6)>(code) << 24);
    if (r < g.R)
      st_stream_u1(out + (lead * g.R + r) * (g.Kp / 2) + k / 2, packed);
    if ((lane & 7) == 0 && r < g.Rp)
      reinterpret_cast<uint32_t *>(sf)[(lead * (g.Kp / 64) + k / 64) * g.Rp + r] = sfw;
  }
}

// Generic path: any strides, optional swizzle.  One lane owns one (row, 64-chunk): it reads
// its 64 elements with scalar loads (coalesced across lanes when the cross dim is the
// contiguous one), and writes 32 packed bytes and one scale dword.
template <bool SWIZZLE>
__global__ __launch_bounds__(256) void quantize_nvfp4_generic_kernel(
    uint8_t *__restrict__ out, uint8_t *__restrict__ sf, const uint16_t *__restrict__ in, const float *__restrict__ gs_ptr,
    QuantGeom g) {
  __shared__ float lut[128];
  load_rcp_table(lut);
  const float alpha = 1.0f / *gs_ptr;
  const int64_t r = (int64_t)blockIdx.x * 256 + threadIdx.x;
  const int64_t chunk = blockIdx.y, lead = blockIdx.z + g.lead0;
  if (r >= g.Rp) return;
  uint32_t *sfp = reinterpret_cast<uint32_t *>(sf) + (lead * (g.Kp / 64) + chunk) * g.Rp + r;
  if (r >= g.R) {
    *sfp = 0u;
    return;
  }
  const uint16_t *src = in + (lead / g.d1) * g.s0 + (lead % g.d1) * g.s1 + r * g.sR;
  uint32_t sfw = 0;
  uint32_t *op = reinterpret_cast<uint32_t *>(out + (lead * g.R + r) * (g.Kp / 2) + chunk * 32);
#pragma unroll
  for (int b = 0; b < 4; ++b) {
    uint32_t h[16];
    uint32_t m = 0;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      int p = b * 16 + i;  // position inside the 64-chunk, output order
      if (SWIZZLE) {
        int q32 = p & 31;
        p = (p & 32) + ((q32 & 7) >> 1) * 8 + (q32 >> 3) * 2 + (q32 & 1);
      }
      const int64_t kk = chunk * 64 + p;
      h[i] = kk < g.K ? (uint32_t)src[kk * g.sK] : 0u;
      m = umax32(m, h[i] & 0x7fffu);
    }
    uint32_t code;
    float o = nvfp4_block_scale(bf16_bits_to_f32(m), alpha, lut, code);
    sfw |= code << (8 * b);
    float f0[8], f1[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      f0[i] = bf16_bits_to_f32(h[i]) * o;
      f1[i] = bf16_bits_to_f32(h[8 + i]) * o;
    }
    op[2 * b] = (o != o) ? 0x77777777u : f32x8_to_e2m1x8(f0);
    op[2 * b + 1] = (o != o) ? 0x77777777u : f32x8_to_e2m1x8(f1);
  }
  *sfp = sfw;
}

// ---------------------------------------------------------------------------
// Single-launch nvfp4 quantize of a contiguous tensor that fits in the register files.
//
// The global scale needs the maximum of the whole tensor before the first nibble can be
// produced, so a two-kernel quantize reads its input twice.  Here every workgroup keeps its share
// of the input in registers (NV 16-byte vectors per lane, 1024 lanes, one workgroup per CU),
// publishes its maximum, waits until every workgroup has published, and quantizes from registers:
// the input crosses the memory bus once, and the call is ONE launch.
//
// Grid synchronisation: arrive[w] = (tag << 16) | bf16 maximum, one word per workgroup, written
// and polled with device-coherent accesses.  The tag is a 16-bit launch number (never the 0 of
// untouched memory) that the host hands out per slot and passes as a kernel argument, so nothing
// is ever cleared.  Every launch on a device uses the same number of workgroups, so each launch
// overwrites every word the next one polls.  The wait is bounded (timeout in 100 MHz ticks): a
// workgroup whose peers have not all published by then - they were not all resident (the GPU is
// shared with other kernels), or another launch is using the same slot - stops waiting and computes
// the maxima of the missing workgroups' shares itself, from memory.  Every workgroup therefore
// finishes on its own whatever else runs on the GPU; words of a foreign tag are never used.  A
// scale that is not a positive finite number takes the full-range arithmetic of the two-kernel
// path in the same launch.
//
// Work split: the tensor is cut into groups of GS = min(NV, 8) segments of 1024 vectors (16 KB);
// group g of workgroup w is group number g * gridDim.x + w, so that at any moment the grid reads
// one contiguous stretch of memory, while a workgroup still owns whole runs of rows for the scale
// layout (scales go through LDS and leave as runs along the row dimension).
constexpr int OP_THREADS = 1024;
constexpr int OP_MAX_WGS = 256;
constexpr int OP_MAX_NV = 16;
constexpr int OP_SLOTS = 32;  // concurrent (device, stream) pairs with synchronisation words of their own
struct OnePassSync {
  uint32_t arrive[OP_SLOTS][OP_MAX_WGS];  // the words of 32 workgroups share a 128-byte line
};
__device__ __align__(256) OnePassSync g_onepass;

// Build with -DAC4K_ONEPASS_TIMELINE to record, per workgroup, the 100 MHz clock at the phase
// boundaries of the single-launch quantizer (a profiling aid; not compiled into the library).
#ifdef AC4K_ONEPASS_TIMELINE
__device__ uint64_t g_onepass_timeline[OP_MAX_WGS][8];
#define AC4K_TL(i)                                                         \
  do {                                                                     \
    if (threadIdx.x == 0) g_onepass_timeline[blockIdx.x][i] = wall_clock64(); \
  } while (0)
#else
#define AC4K_TL(i)
#endif

struct OnePassGeom {
  uint32_t total_chunks;  // 64-element chunks in the tensor
  uint32_t ncc;           // chunks per row (K / 64)
  uint32_t R, Rp, lead;   // rows per leading index, padded rows, number of leading indices
  uint32_t swizzle;       // reduce dim permuted inside every 32-group (a lane quad holds one group)
};

// 16-byte load that bypasses the per-XCD L2 (device-coherent), completed before it returns
__device__ __forceinline__ uint4 ld_coherent_u4(const void *p) {
  u32x4 v;
  asm volatile("global_load_dwordx4 %0, %1, off sc0 sc1\n\ts_waitcnt vmcnt(0)" : "=v"(v) : "v"(p) : "memory");
  return make_uint4(v.x, v.y, v.z, v.w);
}

// |bf16| maximum over this lane's part of the share of workgroup `u` (the slow path of a workgroup
// that stopped waiting for `u`): same split as the main kernel, read from memory, rolled loops.
template <int NV>
__device__ __forceinline__ uint32_t onepass_share_absmax(const uint4 *__restrict__ in, const OnePassGeom &g, uint32_t u,
                                                        uint32_t nwg, uint32_t tid) {
  constexpr int GS = NV < 8 ? NV : 8;
  constexpr int NG = NV / GS;
  constexpr uint32_t GC = GS * 128;
  uint32_t m = 0;
#pragma unroll 1
  for (int q = 0; q < NG; ++q) {
    const uint64_t first = ((uint64_t)q * nwg + u) * GC;
    if (first >= g.total_chunks) break;
    const uint32_t left = g.total_chunks - (uint32_t)first;
    const uint32_t nvalid = left < GC ? left : GC;
#pragma unroll 2
    for (int jj = 0; jj < GS; ++jj) {
      const uint32_t lv = jj * OP_THREADS + tid;
      if ((lv >> 3) < nvalid) m = umax32(m, absmax_bf16x8(in[first * 8 + lv]));
    }
  }
  return m;
}

template <int NV>
__global__ __launch_bounds__(OP_THREADS) void quantize_nvfp4_onepass_kernel(
    uint32_t *__restrict__ out, uint32_t *__restrict__ sf, const uint4 *__restrict__ in, float *__restrict__ gs_out,
    OnePassGeom g, int slot, uint32_t tag, float max_scale, uint64_t timeout_ticks, uint32_t *__restrict__ report,
    uint32_t seq) {
  constexpr int GS = NV < 8 ? NV : 8;  // segments per group
  constexpr int NG = NV / GS;          // groups per workgroup
  constexpr uint32_t GC = GS * 128;    // chunks per group
  __shared__ float lut[128];
  __shared__ uint32_t sfs[128 * NV];
  __shared__ uint32_t red[OP_THREADS / 64];
  __shared__ uint32_t gmax_s, helping_s;
  __shared__ uint32_t miss4[OP_MAX_WGS / 4];  // one byte per workgroup: 1 = its maximum has to be recomputed here
  const uint32_t w = blockIdx.x, nwg = gridDim.x, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;

  AC4K_TL(0);
  // The deadline of the grid wait counts from here: reading the 100 MHz clock takes about as long as a
  // trip to memory, and here that time hides behind the loads.
  const uint64_t t_end = wall_clock64() + timeout_ticks;
  uint32_t cb[NG], nvalid[NG];  // first chunk and number of chunks of each group
#pragma unroll
  for (int q = 0; q < NG; ++q) {
    const uint64_t first = ((uint64_t)q * nwg + w) * GC;
    cb[q] = first < g.total_chunks ? (uint32_t)first : g.total_chunks;
    const uint32_t left = g.total_chunks - cb[q];
    nvalid[q] = left < GC ? left : GC;
  }
  uint4 v[NV];
#pragma unroll
  for (int j = 0; j < NV; ++j) {
    const uint32_t lv = (j % GS) * OP_THREADS + tid;  // vector inside the group
    v[j] = make_uint4(0, 0, 0, 0);
    if ((lv >> 3) < nvalid[j / GS]) v[j] = in[(uint64_t)cb[j / GS] * 8 + lv];
  }
  if (g.swizzle) {  // wave-uniform; four consecutive lanes hold one 32-group, valid or not as a whole
#pragma unroll
    for (int j = 0; j < NV; ++j) v[j] = swizzle_nvfp4_quad(v[j], (int)lane);
  }
  if (tid < 128) lut[tid] = g_rcp_e4m3.v[tid];
  float bm6[NV];  // 16-block maxima times 1/6 (first product of the block scale; it does not need the global scale)
  {
    uint32_t m = 0;
#pragma unroll
    for (int j = 0; j < NV; ++j) {
      uint32_t b = absmax_bf16x8(v[j]);
      b = umax32(b, dpp_u32<DPP_QUAD_XOR1>(b));
      m = umax32(m, b);
      bm6[j] = bf16_bits_to_f32(b) * 0.16666666666666666f;
      asm volatile("" : "+v"(bm6[j]));  // formed here, while the loads are still arriving, not after the wait
    }
    m = group_umax<64>(m);
    if (lane == 0) red[wave] = m;
  }
  __syncthreads();
  AC4K_TL(1);
  // The last wave publishes the workgroup's maximum; wave 0 polls (a wave that did both would wait for
  // the store's acknowledgement, a round trip of its own, before its first poll returns).  The first
  // poll goes out about 1 us after the store (40 x 64 cycles): measured on MI355X, a poll sent right
  // behind the workgroup's own loads and store comes back about 3 us later, one sent 1 us later within
  // 0.5 us, and until the last workgroup arrives there is nothing to see anyway (the workgroups finish
  // their loads within about 2.5 us of each other).  Measured time from the last arrival until every
  // workgroup knows the maximum: 3.1 us without the delay, 1.0 - 1.6 us with it; delays of 20 / 30 /
  // 50 / 80 x 64 cycles gave up to 2.2 / 1.9 / 1.9 / 2.7 us.
  if (wave == OP_THREADS / 64 - 1) {
    const uint32_t own = group_umax<16>(red[lane & 15]);
    if (lane == 0)
      __hip_atomic_store(&g_onepass.arrive[slot][w], (tag << 16) | own, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
  if (wave == 0) {
    const uint32_t own = group_umax<16>(red[lane & 15]);
    const uint32_t i0 = lane * 4;
    // (bounds of up to 1 us - 100 ticks - are there to force the slow path from the host: no delay in front of the
    // first poll, the clock looked at on every poll, so that the first workgroup to arrive finds peers missing)
    const bool forced = timeout_ticks <= 100;
    if (!forced) __builtin_amdgcn_s_sleep(40);
    bool ok, r0, r1, r2, r3, lane_ready = false;
    uint4 a = make_uint4(0, 0, 0, 0);
    for (uint32_t it = 0;; ++it) {  // at least one poll, whatever the timeout
      // only lanes that still miss one of their four words look again: towards the end of the wait a
      // poll touches one or two lines instead of eight, and every workgroup polls the same ones
      if (!lane_ready) a = ld_coherent_u4(&g_onepass.arrive[slot][i0]);
      // (the own word counts as published: its store may not have reached memory yet)
      r0 = (a.x >> 16) == tag || i0 + 0 == w;
      r1 = (a.y >> 16) == tag || i0 + 1 == w;
      r2 = (a.z >> 16) == tag || i0 + 2 == w;
      r3 = (a.w >> 16) == tag || i0 + 3 == w;
      lane_ready = (i0 + 0 >= nwg || r0) && (i0 + 1 >= nwg || r1) && (i0 + 2 >= nwg || r2) && (i0 + 3 >= nwg || r3);
      ok = __all(lane_ready);
      if (ok) break;
      // the clock is looked at on every fourth poll only (and at once when the bound is zero or forced)
      if ((forced || (it & 3) == 3) && wall_clock64() >= t_end) break;
      __builtin_amdgcn_s_sleep(2);
    }
    // maxima that were published under this launch's tag; the others are marked for recomputation
    // (the own word may be stale in `a`: its maximum comes from `own`)
    uint32_t mm = own;
    mm = umax32(mm, (i0 + 0 < nwg && r0 && i0 + 0 != w) ? a.x & 0xffffu : 0u);
    mm = umax32(mm, (i0 + 1 < nwg && r1 && i0 + 1 != w) ? a.y & 0xffffu : 0u);
    mm = umax32(mm, (i0 + 2 < nwg && r2 && i0 + 2 != w) ? a.z & 0xffffu : 0u);
    mm = umax32(mm, (i0 + 3 < nwg && r3 && i0 + 3 != w) ? a.w & 0xffffu : 0u);
    mm = group_umax<64>(mm);
    miss4[lane] = ((i0 + 0 < nwg && !r0) ? 1u : 0u) | ((i0 + 1 < nwg && !r1) ? 0x100u : 0u) |
                  ((i0 + 2 < nwg && !r2) ? 0x10000u : 0u) | ((i0 + 3 < nwg && !r3) ? 0x1000000u : 0u);
    if (lane == 0) {
      gmax_s = mm;
      helping_s = ok ? 0u : 1u;
    }
  }
  __syncthreads();
  uint32_t gm = gmax_s;
  if (helping_s) {  // workgroup-uniform: the wait ran out
    // tell the host (a word of mapped host memory per slot, read without synchronising before a later call):
    // launch number `seq` did not find its peers resident
    if (tid == 0 && report && timeout_ticks) __hip_atomic_store(report + slot, seq, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
    const uint8_t *miss = reinterpret_cast<const uint8_t *>(miss4);
    uint32_t m = 0;
#pragma unroll 1
    for (uint32_t u = 0; u < nwg; ++u)
      if (miss[u]) m = umax32(m, onepass_share_absmax<NV>(in, g, u, nwg, tid));
    m = group_umax<64>(m);
    if (lane == 0) red[wave] = m;  // wave 0 finished reading `red` before the barrier above
    __syncthreads();
    gm = umax32(gm, group_umax<16>(red[lane & 15]));
  }
  AC4K_TL(2);
  const float gs = bf16_bits_to_f32(gm) / max_scale;
  const float alpha = 1.0f / gs;
  if (w == 0 && tid == 0) *gs_out = gs;
  // With a positive finite alpha no product below is NaN and no block scale reaches 464 (it is at
  // most 448 * (1 + 3e-7)), so the clamp and the NaN cases of the full arithmetic are not needed.
  const bool fast = alpha > 0.0f && alpha < __builtin_inff();

  uint8_t *sfb = reinterpret_cast<uint8_t *>(sfs);
  if (fast) {
#pragma unroll
    for (int q = 0; q < NG; ++q) {
      // block scale codes, four to a register (two conversions), and the multipliers
      uint32_t codes[(GS + 3) / 4];
      float oo[GS];
#pragma unroll
      for (int c4 = 0; c4 < (GS + 3) / 4; ++c4) {
        float s32[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) s32[i] = c4 * 4 + i < GS ? alpha * bm6[q * GS + c4 * 4 + i] : 0.0f;
        int wd = __builtin_amdgcn_cvt_pk_fp8_f32(s32[0], s32[1], 0, false);
        codes[c4] = (uint32_t)__builtin_amdgcn_cvt_pk_fp8_f32(s32[2], s32[3], wd, true);
      }
#pragma unroll
      for (int jj = 0; jj < GS; ++jj) oo[jj] = alpha * lut[(codes[jj / 4] >> (8 * (jj % 4))) & 0xffu];
      uint32_t *op = out + (uint64_t)cb[q] * 8 + tid;
      uint8_t *sp = sfb + q * GC * 4 + (tid >> 1);
      // a whole group (every group but the tensor's last ones) needs no predicates at all
      auto store_group = [&](auto whole_group) {
        constexpr bool WHOLE = decltype(whole_group)::value;
#pragma unroll
        for (int jj = 0; jj < GS; ++jj) {
          const int j = q * GS + jj;
          const float m_ = oo[jj];
          const float f[8] = {bf16_lo(v[j].x) * m_, bf16_hi(v[j].x) * m_, bf16_lo(v[j].y) * m_, bf16_hi(v[j].y) * m_,
                              bf16_lo(v[j].z) * m_, bf16_hi(v[j].z) * m_, bf16_lo(v[j].w) * m_, bf16_hi(v[j].w) * m_};
          const uint32_t packed = f32x8_to_e2m1x8(f);
          if (WHOLE || ((jj * OP_THREADS + tid) >> 3) < nvalid[q]) st_stream_u1(op + jj * OP_THREADS, packed);
        }
        // scale byte (lv % 8) / 2 of chunk lv / 8; both lanes of a 16-block hold the same code
        if ((lane & 1) == 0) {
#pragma unroll
          for (int jj = 0; jj < GS; ++jj)
            if (WHOLE || ((jj * OP_THREADS + tid) >> 3) < nvalid[q])
              sp[jj * (OP_THREADS / 2)] = (uint8_t)(codes[jj / 4] >> (8 * (jj % 4)));
        }
      };
      if (nvalid[q] == GC)  // workgroup-uniform
        store_group(std::true_type{});
      else
        store_group(std::false_type{});
    }
  } else {
#pragma unroll
    for (int q = 0; q < NG; ++q) {
#pragma unroll
      for (int jj = 0; jj < GS; ++jj) {
        const int j = q * GS + jj;
        const uint32_t lv = jj * OP_THREADS + tid;
        uint32_t code;
        // (amax / 6 was formed before the wait; nvfp4_block_scale forms the same product)
        const float s32 = alpha * bm6[j];
        code = f32_to_ue4m3_satfinite(s32);
        const uint32_t packed = nvfp4_pack8(v[j], alpha * lut[code]);
        if ((lv >> 3) < nvalid[q]) {
          st_stream_u1(out + (uint64_t)cb[q] * 8 + lv, packed);
          if ((lane & 1) == 0) sfb[q * GC * 4 + (lv >> 1)] = (uint8_t)code;
        }
      }
    }
  }
  __syncthreads();
  AC4K_TL(3);
  // scales: LDS holds one dword per chunk in (row, chunk column) order; memory wants, per chunk
  // column, runs along the rows
#pragma unroll
  for (int q = 0; q < NG; ++q) {
    if (nvalid[q] == 0) continue;
    const uint32_t row_first = cb[q] / g.ncc, row_last = (cb[q] + nvalid[q] - 1) / g.ncc;
    const uint32_t span = row_last - row_first + 1;
    for (uint32_t i = tid; i < span * g.ncc; i += OP_THREADS) {
      const uint32_t cc = i / span, row = row_first + (i - cc * span);
      const uint32_t ch = row * g.ncc + cc;
      if (ch < cb[q] || ch >= cb[q] + nvalid[q]) continue;
      const uint32_t l = g.lead > 1 ? row / g.R : 0u, r = row - l * g.R;
      sf[((uint64_t)l * g.ncc + cc) * g.Rp + r] = sfs[q * GC + (ch - cb[q])];
    }
  }
  // zero scales of the pad rows R..Rp-1, shared out evenly
  if (g.Rp > g.R) {
    const uint32_t pad = g.Rp - g.R, npad = g.lead * g.ncc * pad, per = (npad + nwg - 1) / nwg;
    const uint32_t hi = (w + 1) * per < npad ? (w + 1) * per : npad;
    for (uint32_t i = w * per + tid; i < hi; i += OP_THREADS) sf[(uint64_t)(i / pad) * g.Rp + g.R + i % pad] = 0u;
  }
  AC4K_TL(4);
}

// ---------------------------------------------------------------------------
// Small dense tensors (at most NSEG segments of 1024 16-byte vectors, 16 KB each): one launch, no
// grid wait.  Workgroup b quantizes segment b; for the global scale every workgroup reads the
// whole tensor itself (all loads in flight at once; after the first workgroup they are cache hits),
// so nothing has to be exchanged between workgroups.
template <int NSEG>
__global__ __launch_bounds__(OP_THREADS) void quantize_nvfp4_small_kernel(
    uint32_t *__restrict__ out, uint32_t *__restrict__ sf, const uint4 *__restrict__ in, float *__restrict__ gs_out,
    OnePassGeom g, float max_scale) {
  __shared__ float lut[128];
  __shared__ uint32_t red[OP_THREADS / 64];
  // Only every eighth workgroup works (NSEG > 1): workgroups are dealt round-robin to the 8 XCDs, so the
  // working ones share ONE L2 and their reads of the whole tensor meet there instead of crossing the
  // fabric eight times.
  if (NSEG > 1 && (blockIdx.x & 7)) return;
  const uint32_t seg = NSEG > 1 ? blockIdx.x >> 3 : blockIdx.x;
  const uint32_t tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const uint32_t nvec = g.total_chunks * 8;
  const uint32_t lv = seg * OP_THREADS + tid;  // this lane's vector of the workgroup's own segment
  uint4 own = make_uint4(0, 0, 0, 0);
  if (lv < nvec) own = in[lv];
  uint4 v[NSEG];
#pragma unroll
  for (int j = 0; j < NSEG; ++j) {
    const uint32_t ov = j * OP_THREADS + tid;
    v[j] = make_uint4(0, 0, 0, 0);
    if (ov < nvec) v[j] = in[ov];
  }
  if (tid < 128) lut[tid] = g_rcp_e4m3.v[tid];
  uint32_t m = 0;
#pragma unroll
  for (int j = 0; j < NSEG; ++j) m = umax32(m, absmax_bf16x8(v[j]));
  m = group_umax<64>(m);
  if (lane == 0) red[wave] = m;
  __syncthreads();
  const uint32_t gm = group_umax<16>(red[lane & 15]);
  const float gs = bf16_bits_to_f32(gm) / max_scale;
  if (seg == 0 && tid == 0) *gs_out = gs;
  const float alpha = 1.0f / gs;
  if (g.swizzle) own = swizzle_nvfp4_quad(own, (int)lane);  // the maximum above does not depend on the order
  uint32_t bm = absmax_bf16x8(own);
  bm = umax32(bm, dpp_u32<DPP_QUAD_XOR1>(bm));
  uint32_t code;
  const float o = nvfp4_block_scale(bf16_bits_to_f32(bm), alpha, lut, code);
  const uint32_t packed = nvfp4_pack8(own, o);
  const uint32_t sfw = code | (dpp_u32<DPP_ROW_SHL(2)>(code) << 8) | (dpp_u32<DPP_ROW_SHL(4)>(code) << 16) |
                       (dpp_u32<DPP_ROW_SHL(6)>(code) << 24);
  if (lv < nvec) {
    out[lv] = packed;
    if ((lane & 7) == 0) {
      const uint32_t ch = lv >> 3, row = ch / g.ncc, cc = ch - row * g.ncc;
      const uint32_t l = g.lead > 1 ? row / g.R : 0u, r = row - l * g.R;
      sf[((uint64_t)l * g.ncc + cc) * g.Rp + r] = sfw;
    }
  }
  if (g.Rp > g.R && seg == 0) {  // zero scales of the pad rows R..Rp-1
    const uint32_t pad = g.Rp - g.R, npad = g.lead * g.ncc * pad;
    for (uint32_t i = tid; i < npad; i += OP_THREADS) sf[(uint64_t)(i / pad) * g.Rp + g.R + i % pad] = 0u;
  }
}

// ===========================================================================
// per-row fp8 / int8
// ===========================================================================

enum class RowFmt { FP8, INT8 };

// scale_max is a device scalar: fp32 for fp8 (quantize_fp8.cu:205), int32 for int8
// (quantize_int8.cu:189), converted to float where it is used (:127,135).
template <RowFmt FMT>
__device__ __forceinline__ float load_scale_max(const void *p) {
  return FMT == RowFmt::FP8 ? *static_cast<const float *>(p) : (float)*static_cast<const int32_t *>(p);
}

// satfinite e4m3 of four floats -> four bytes, element 0 in the low byte.
__device__ __forceinline__ uint32_t f32x4_to_e4m3x4(float a, float b, float c, float d) {
  a = __builtin_amdgcn_fmed3f(a, -448.0f, 448.0f);
  b = __builtin_amdgcn_fmed3f(b, -448.0f, 448.0f);
  c = __builtin_amdgcn_fmed3f(c, -448.0f, 448.0f);
  d = __builtin_amdgcn_fmed3f(d, -448.0f, 448.0f);
  int w = __builtin_amdgcn_cvt_pk_fp8_f32(a, b, 0, false);
  w = __builtin_amdgcn_cvt_pk_fp8_f32(c, d, w, true);
  return (uint32_t)w;
}

__device__ __forceinline__ uint32_t f32_to_s8_sat(float x) {
  // cvt.rni.sat.s8.f32: round half to even, clamp, NaN -> 0
  int i = (int)__builtin_rintf(x);  // v_cvt_i32_f32 saturates and maps NaN to 0
  i = i < -128 ? -128 : (i > 127 ? 127 : i);
  return (uint32_t)i & 0xffu;
}

template <RowFmt FMT>
__device__ __forceinline__ uint2 rowfmt_pack8(uint4 v, float recp, bool nan_row) {
  float f[8] = {bf16_lo(v.x) * recp, bf16_hi(v.x) * recp, bf16_lo(v.y) * recp, bf16_hi(v.y) * recp,
                bf16_lo(v.z) * recp, bf16_hi(v.z) * recp, bf16_lo(v.w) * recp, bf16_hi(v.w) * recp};
  uint2 o;
  if (FMT == RowFmt::FP8) {
    o.x = f32x4_to_e4m3x4(f[0], f[1], f[2], f[3]);
    o.y = f32x4_to_e4m3x4(f[4], f[5], f[6], f[7]);
    if (nan_row) o.x = o.y = 0x7f7f7f7fu;  // amax == 0: 0 * inf = NaN in every position
  } else {
    o.x = f32_to_s8_sat(f[0]) | (f32_to_s8_sat(f[1]) << 8) | (f32_to_s8_sat(f[2]) << 16) |
          (f32_to_s8_sat(f[3]) << 24);
    o.y = f32_to_s8_sat(f[4]) | (f32_to_s8_sat(f[5]) << 8) | (f32_to_s8_sat(f[6]) << 16) |
          (f32_to_s8_sat(f[7]) << 24);
  }
  return o;
}

// Row-major fast path: the whole row lives in registers between the amax pass and the
// convert pass, so the input is read from memory once.  LPR lanes share a row (DPP / swizzle
// reduction), each lane holds NV 16-byte vectors at a stride of LPR*8 elements.
template <RowFmt FMT, int LPR, int NV, bool SWIZZLE>
__global__ __launch_bounds__(256) void quantize_rowwise_rowmajor_kernel(
    uint8_t *__restrict__ out, float *__restrict__ sf, const uint16_t *__restrict__ in,
    const void *__restrict__ smax_p, QuantGeom g) {
  const float smax = load_scale_max<FMT>(smax_p);
  constexpr int RPB = 256 / LPR;  // rows per block
  const int sub = threadIdx.x % LPR;
  const int64_t r = (int64_t)blockIdx.x * RPB + threadIdx.x / LPR;
  const int64_t lead = blockIdx.y + g.lead0;
  const uint16_t *src = in + (lead / g.d1) * g.s0 + (lead % g.d1) * g.s1 + r * g.sR;
  uint4 v[NV];
  uint32_t m = 0;
#pragma unroll
  for (int j = 0; j < NV; ++j) {
    const int64_t k = ((int64_t)j * LPR + sub) * 8;
    v[j] = make_uint4(0, 0, 0, 0);
    if (r < g.R && k < g.K) v[j] = ld_stream_u4(src + k);
    m = umax32(m, absmax_bf16x8(v[j]));
    if (SWIZZLE) v[j] = swizzle_fp8_pair(v[j], threadIdx.x);
  }
  m = group_umax<LPR>(m);
  const float amax = bf16_bits_to_f32(m);
  if (sub == 0 && r < g.Rp) sf[lead * g.Rp + r] = amax / smax;
  if (r >= g.R) return;
  const float recp = smax / amax;
  const bool nan_row = (FMT == RowFmt::FP8) && (amax == 0.0f);
  uint8_t *op = out + (lead * g.R + r) * g.Kp;
#pragma unroll
  for (int j = 0; j < NV; ++j) {
    const int64_t k = ((int64_t)j * LPR + sub) * 8;
    if (k < g.Kp)
      st_stream_u2(op + k, rowfmt_pack8<FMT>(v[j], recp, nan_row));
  }
}

// Rows longer than the register budget of the kernel above: one wave per row, two passes over the
// row (the second one is served by the caches), 16-byte loads, 8-byte stores.
template <RowFmt FMT>
__global__ __launch_bounds__(256) void quantize_rowwise_longrow_kernel(
    uint8_t *__restrict__ out, float *__restrict__ sf, const uint16_t *__restrict__ in,
    const void *__restrict__ smax_p, QuantGeom g) {
  const float smax = load_scale_max<FMT>(smax_p);
  const int lane = threadIdx.x & 63;
  const int64_t r = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  const int64_t lead = blockIdx.y + g.lead0;
  if (r >= g.Rp) return;
  if (r >= g.R) {
    if (lane == 0) sf[lead * g.Rp + r] = 0.0f / smax;
    return;
  }
  const uint16_t *src = in + (lead / g.d1) * g.s0 + (lead % g.d1) * g.s1 + r * g.sR;
  uint32_t m = 0;
  for (int64_t k = lane * 8; k < g.K; k += 512) m = umax32(m, absmax_bf16x8(*reinterpret_cast<const uint4 *>(src + k)));
  m = group_umax<64>(m);
  const float amax = bf16_bits_to_f32(m);
  if (lane == 0) sf[lead * g.Rp + r] = amax / smax;
  const float recp = smax / amax;
  const bool nan_row = (FMT == RowFmt::FP8) && (amax == 0.0f);
  uint8_t *op = out + (lead * g.R + r) * g.Kp;
  for (int64_t k = lane * 8; k < g.Kp; k += 512) {
    uint4 v = make_uint4(0, 0, 0, 0);
    if (k < g.K) v = *reinterpret_cast<const uint4 *>(src + k);
    st_stream_u2(op + k, rowfmt_pack8<FMT>(v, recp, nan_row));
  }
}

// Generic path: any strides / swizzle / K.  One lane per row, two passes over the row.
template <RowFmt FMT, bool SWIZZLE>
__global__ __launch_bounds__(256) void quantize_rowwise_generic_kernel(
    uint8_t *__restrict__ out, float *__restrict__ sf, const uint16_t *__restrict__ in,
    const void *__restrict__ smax_p, QuantGeom g) {
  const float smax = load_scale_max<FMT>(smax_p);
  const int64_t r = (int64_t)blockIdx.x * 256 + threadIdx.x;
  const int64_t lead = blockIdx.y + g.lead0;
  if (r >= g.Rp) return;
  if (r >= g.R) {
    sf[lead * g.Rp + r] = 0.0f / smax;
    return;
  }
  const uint16_t *src = in + (lead / g.d1) * g.s0 + (lead % g.d1) * g.s1 + r * g.sR;
  uint32_t m = 0;
  for (int64_t k = 0; k < g.K; ++k) m = umax32(m, src[k * g.sK] & 0x7fffu);
  const float amax = bf16_bits_to_f32(m);
  sf[lead * g.Rp + r] = amax / smax;
  const float recp = smax / amax;
  const bool nan_row = (FMT == RowFmt::FP8) && (amax == 0.0f);
  uint32_t *op = reinterpret_cast<uint32_t *>(out + (lead * g.R + r) * g.Kp);
  for (int64_t k4 = 0; k4 < g.Kp; k4 += 4) {
    float f[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      int64_t kk = k4 + i;
      if (SWIZZLE) {
        int p = (int)(kk & 15);
        kk = (kk & ~(int64_t)15) + ((p & 3) >> 1) * 8 + (p >> 2) * 2 + (p & 1);
      }
      f[i] = (kk < g.K ? bf16_bits_to_f32(src[kk * g.sK]) : 0.0f) * recp;
    }
    uint32_t w;
    if (FMT == RowFmt::FP8) {
      w = nan_row ? 0x7f7f7f7fu : f32x4_to_e4m3x4(f[0], f[1], f[2], f[3]);
    } else {
      w = f32_to_s8_sat(f[0]) | (f32_to_s8_sat(f[1]) << 8) | (f32_to_s8_sat(f[2]) << 16) |
          (f32_to_s8_sat(f[3]) << 24);
    }
    op[k4 / 4] = w;
  }
}

// ===========================================================================
// Cross dim contiguous, reduce dim strided (the layout of V in attention: quantize(v, 3, N_dim)).
//
// A lane (kb = lane % 4, rg = lane / 4) owns eight consecutive rows (one 16-byte load along the
// contiguous cross dim) and the 16 reduce positions of output block kb of a 64-chunk: 16 loads,
// each of which a wave issues as four 256-byte row segments.  Blocks run along the loop index,
// so block maxima, products and nibble/byte packing all stay inside the lane - no transposition -
// and the swizzles are only a different choice of the 16 source positions.  Four adjacent lanes
// hold the four blocks of a chunk: their stores of one row are contiguous.
// ===========================================================================

// bf16 component j (0..7) of a 16-byte vector as float
__device__ __forceinline__ float bf16_comp(const uint4 &v, int j) {
  const uint32_t w = (j >> 1) == 0 ? v.x : (j >> 1) == 1 ? v.y : (j >> 1) == 2 ? v.z : v.w;
  return (j & 1) ? bf16_hi(w) : bf16_lo(w);
}

// element-wise |bf16| maximum of two vectors of eight
__device__ __forceinline__ uint4 absmax_bf16x8_pairwise(uint4 acc, uint4 v) {
  auto mx = [](uint32_t a, uint32_t b) {
    const u16x2 r = __builtin_elementwise_max(__builtin_bit_cast(u16x2, a), __builtin_bit_cast(u16x2, b & 0x7fff7fffu));
    return __builtin_bit_cast(uint32_t, r);
  };
  return make_uint4(mx(acc.x, v.x), mx(acc.y, v.y), mx(acc.z, v.z), mx(acc.w, v.w));
}
__device__ __forceinline__ uint32_t u16_comp(const uint4 &v, int j) {
  const uint32_t w = (j >> 1) == 0 ? v.x : (j >> 1) == 1 ? v.y : (j >> 1) == 2 ? v.z : v.w;
  return (j & 1) ? (w >> 16) : (w & 0xffffu);
}

// source position inside a 32-group (nvfp4) or 16-group (fp8) of output position p
__device__ __forceinline__ int nvfp4_swizzle_src(int p) { return ((p & 7) >> 1) * 8 + (p >> 3) * 2 + (p & 1); }
__device__ __forceinline__ int fp8_swizzle_src(int p) { return ((p & 3) >> 1) * 8 + (p >> 2) * 2 + (p & 1); }

template <bool SWIZZLE>
__global__ __launch_bounds__(256) void quantize_nvfp4_crossmajor_kernel(
    uint8_t *__restrict__ out, uint8_t *__restrict__ sf, const uint16_t *__restrict__ in, const float *__restrict__ gs_ptr,
    QuantGeom g) {
  __shared__ float lut[128];
  load_rcp_table(lut);
  const float alpha = 1.0f / *gs_ptr;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int kb = lane & 3, rg = lane >> 2;
  const CrossMajorIdx gi = crossmajor_idx(g);
  const int64_t cc = gi.kblock * 4 + wave;                      // 64-chunk along the reduce dim
  const int64_t row0 = (int64_t)blockIdx.y * 128 + rg * 8;      // first of the lane's eight rows
  const int64_t lead = gi.lead;
  if (cc * 64 >= g.Kp || row0 >= g.Rp) return;
  const uint16_t *src = in + (lead / g.d1) * g.s0 + (lead % g.d1) * g.s1 + row0;
  const bool rows_valid = row0 < g.R;  // R % 8 == 0: all eight or none

  uint4 v[16];
  uint4 m8 = make_uint4(0, 0, 0, 0);
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    const int p = (kb & 1) * 16 + i;  // output position inside the 32-group
    const int64_t k = cc * 64 + (kb >> 1) * 32 + (SWIZZLE ? nvfp4_swizzle_src(p) : p);
    v[i] = make_uint4(0, 0, 0, 0);
    if (rows_valid && k < g.K) v[i] = *reinterpret_cast<const uint4 *>(src + k * g.sK);
  }
#pragma unroll
  for (int i = 0; i < 16; ++i) m8 = absmax_bf16x8_pairwise(m8, v[i]);

  uint32_t code[8];
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    const float o = nvfp4_block_scale(bf16_bits_to_f32(u16_comp(m8, j)), alpha, lut, code[j]);
    if (!rows_valid) code[j] = 0;  // pad rows carry zero scales
    float f0[8], f1[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      f0[i] = bf16_comp(v[i], j) * o;
      f1[i] = bf16_comp(v[8 + i], j) * o;
    }
    const uint2 packed = (o != o) ? make_uint2(0x77777777u, 0x77777777u) : make_uint2(f32x8_to_e2m1x8(f0), f32x8_to_e2m1x8(f1));
    if (rows_valid)
      *reinterpret_cast<uint2 *>(out + (lead * g.R + row0 + j) * (g.Kp / 2) + cc * 32 + kb * 8) = packed;
  }
  // scale dword of (row, chunk) = the codes of the four lanes of the quad; lane kb stores rows 2kb, 2kb+1
  uint32_t sfw[8];
#pragma unroll
  for (int j = 0; j < 8; ++j)
    sfw[j] = dpp_u32<0x00>(code[j]) | (dpp_u32<0x55>(code[j]) << 8) | (dpp_u32<0xAA>(code[j]) << 16) |
             (dpp_u32<0xFF>(code[j]) << 24);
  const uint2 mine = kb == 0 ? make_uint2(sfw[0], sfw[1])
                   : kb == 1 ? make_uint2(sfw[2], sfw[3])
                   : kb == 2 ? make_uint2(sfw[4], sfw[5]) : make_uint2(sfw[6], sfw[7]);
  *reinterpret_cast<uint2 *>(reinterpret_cast<uint32_t *>(sf) + (lead * (g.Kp / 64) + cc) * g.Rp + row0 + 2 * kb) = mine;
}

// ---- per-row fp8 / int8 with the reduce dim strided: the row maximum is collected with atomic
// maxima of bf16 bit patterns into the (zeroed) scale array, the quantize kernel reads them, and a
// last kernel turns them into amax / scale_max in place.
__global__ void fill_u32_kernel(uint32_t *__restrict__ p, int64_t n, uint32_t v) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i < n) p[i] = v;
}

constexpr int CM_KSPAN = 2048;  // reduce positions per workgroup of the maximum kernel

__global__ __launch_bounds__(256) void rowwise_crossmajor_amax_kernel(uint32_t *__restrict__ amax_bits,
                                                                       const uint16_t *__restrict__ in, QuantGeom g) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int kq = lane & 3, rg = lane >> 2;
  const CrossMajorIdx gi = crossmajor_idx(g);
  const int64_t row0 = (int64_t)blockIdx.y * 128 + rg * 8;
  const int64_t lead = gi.lead;
  const uint16_t *src = in + (lead / g.d1) * g.s0 + (lead % g.d1) * g.s1 + row0;
  uint4 m8 = make_uint4(0, 0, 0, 0);
  if (row0 < g.R) {
    const int64_t kbeg = gi.kblock * CM_KSPAN, kend = kbeg + CM_KSPAN < g.K ? kbeg + CM_KSPAN : g.K;
    for (int64_t k = kbeg + wave * 4 + kq; k < kend; k += 64) {  // four loads in flight per lane
      uint4 a[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        a[u] = make_uint4(0, 0, 0, 0);
        if (k + u * 16 < kend) a[u] = *reinterpret_cast<const uint4 *>(src + (k + u * 16) * g.sK);
      }
#pragma unroll
      for (int u = 0; u < 4; ++u) m8 = absmax_bf16x8_pairwise(m8, a[u]);
    }
  }
  // quad (same rows, different k) -> one value per row; then across the four waves through LDS
  auto quad_max = [](uint32_t w) {
    u16x2 x = __builtin_bit_cast(u16x2, w);
    x = __builtin_elementwise_max(x, __builtin_bit_cast(u16x2, dpp_u32<DPP_QUAD_XOR1>(w)));
    const uint32_t y = __builtin_bit_cast(uint32_t, x);
    x = __builtin_elementwise_max(x, __builtin_bit_cast(u16x2, dpp_u32<DPP_QUAD_XOR2>(y)));
    return __builtin_bit_cast(uint32_t, x);
  };
  m8 = make_uint4(quad_max(m8.x), quad_max(m8.y), quad_max(m8.z), quad_max(m8.w));
  __shared__ uint4 red[4][16];
  if (kq == 0) red[wave][rg] = m8;
  __syncthreads();
  if (wave == 0 && kq == 0 && row0 < g.R) {
    uint4 t = red[0][rg];
#pragma unroll
    for (int w2 = 1; w2 < 4; ++w2) t = absmax_bf16x8_pairwise(t, red[w2][rg]);
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const uint32_t b = u16_comp(t, j);
      if (b) atomicMax(amax_bits + lead * g.Rp + row0 + j, b);
    }
  }
}

template <RowFmt FMT, bool SWIZZLE>
__global__ __launch_bounds__(256) void quantize_rowwise_crossmajor_kernel(
    uint8_t *__restrict__ out, const uint32_t *__restrict__ amax_bits, const uint16_t *__restrict__ in,
    const void *__restrict__ smax_p, QuantGeom g) {
  const float smax = load_scale_max<FMT>(smax_p);
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int kb = lane & 3, rg = lane >> 2;
  const CrossMajorIdx gi = crossmajor_idx(g);
  const int64_t k0 = (gi.kblock * 4 + wave) * 64 + kb * 16;  // the lane's 16 output positions
  const int64_t row0 = (int64_t)blockIdx.y * 128 + rg * 8;
  const int64_t lead = gi.lead;
  if (k0 >= g.Kp || row0 >= g.R) return;
  const uint16_t *src = in + (lead / g.d1) * g.s0 + (lead % g.d1) * g.s1 + row0;
  uint4 v[16];
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    const int64_t k = k0 + (SWIZZLE ? fp8_swizzle_src(i) : i);
    v[i] = make_uint4(0, 0, 0, 0);
    if (k < g.K) v[i] = *reinterpret_cast<const uint4 *>(src + k * g.sK);
  }
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    const float amax = bf16_bits_to_f32(amax_bits[lead * g.Rp + row0 + j]);
    const float recp = smax / amax;
    const bool nan_row = (FMT == RowFmt::FP8) && (amax == 0.0f);
    float f[16];
#pragma unroll
    for (int i = 0; i < 16; ++i) f[i] = bf16_comp(v[i], j) * recp;
    uint4 w;
    if (FMT == RowFmt::FP8) {
      w = make_uint4(f32x4_to_e4m3x4(f[0], f[1], f[2], f[3]), f32x4_to_e4m3x4(f[4], f[5], f[6], f[7]),
                     f32x4_to_e4m3x4(f[8], f[9], f[10], f[11]), f32x4_to_e4m3x4(f[12], f[13], f[14], f[15]));
      if (nan_row) w = make_uint4(0x7f7f7f7fu, 0x7f7f7f7fu, 0x7f7f7f7fu, 0x7f7f7f7fu);
    } else {
      auto p4 = [&](int b) {
        return f32_to_s8_sat(f[b]) | (f32_to_s8_sat(f[b + 1]) << 8) | (f32_to_s8_sat(f[b + 2]) << 16) |
               (f32_to_s8_sat(f[b + 3]) << 24);
      };
      w = make_uint4(p4(0), p4(4), p4(8), p4(12));
    }
    *reinterpret_cast<uint4 *>(out + (lead * g.R + row0 + j) * g.Kp + k0) = w;
  }
}

// amax bit patterns -> amax / scale_max, in place (pad rows hold 0 -> 0 / scale_max)
template <RowFmt FMT>
__global__ void rowwise_crossmajor_finalize_kernel(float *__restrict__ sf, const void *__restrict__ smax_p, int64_t n) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i < n) sf[i] = bf16_bits_to_f32(__float_as_uint(sf[i])) / load_scale_max<FMT>(smax_p);
}

// ---------------------------------------------------------------------------
// host launchers
// ---------------------------------------------------------------------------

static int check_geom(const void *out, const void *sf, const void *in, const void *scalar, int64_t d0,
                      int64_t d1, int64_t R, int64_t K, int64_t s0, int64_t s1, int64_t sR, int64_t sK) {
  AC4K_REQUIRE(out && sf && in && scalar, "null pointer argument");
  AC4K_REQUIRE(d0 >= 1 && d1 >= 1 && R >= 1 && K >= 1, "sizes must be positive (d0=%lld d1=%lld R=%lld K=%lld)",
               (long long)d0, (long long)d1, (long long)R, (long long)K);
  AC4K_REQUIRE(s0 >= 0 && s1 >= 0 && sR >= 1 && sK >= 1 && (d0 == 1 || s0 >= 1) && (d1 == 1 || s1 >= 1),
               "strides must be positive");
  return 0;
}

// Do the four dims, in some order, tile d0*d1*R*K contiguous elements exactly?  (Dims of size 1 may
// carry any stride.)
static bool dense_permutation(int64_t d0, int64_t d1, int64_t R, int64_t K, int64_t s0, int64_t s1, int64_t sR,
                              int64_t sK) {
  int64_t size[4] = {d0, d1, R, K}, stride[4] = {s0, s1, sR, sK};
  for (int i = 1; i < 4; ++i)  // insertion sort by stride
    for (int j = i; j > 0 && stride[j] < stride[j - 1]; --j) {
      const int64_t ts = stride[j], tz = size[j];
      stride[j] = stride[j - 1]; size[j] = size[j - 1];
      stride[j - 1] = ts; size[j - 1] = tz;
    }
  int64_t expect = 1;
  for (int i = 0; i < 4; ++i) {
    if (size[i] == 1) continue;
    if (stride[i] != expect) return false;
    expect *= size[i];
  }
  return true;
}

static bool rowmajor_ok(const void *in, int64_t K, int64_t s0, int64_t s1, int64_t sR, int64_t sK) {
  return sK == 1 && K % 8 == 0 && (reinterpret_cast<uintptr_t>(in) & 15) == 0 && sR % 8 == 0 &&
         s0 % 8 == 0 && s1 % 8 == 0;
}

// cross dim contiguous, every row group of eight 16-byte aligned
static bool crossmajor_ok(const void *in, int64_t R, int64_t s0, int64_t s1, int64_t sR, int64_t sK) {
  return sR == 1 && R % 8 == 0 && (reinterpret_cast<uintptr_t>(in) & 15) == 0 && sK % 8 == 0 && s0 % 8 == 0 &&
         s1 % 8 == 0;
}

template <int CPR>
static void launch_nvfp4_rowmajor(uint8_t *out, uint8_t *sf, const uint16_t *in, const float *gs,
                                  const QuantGeom &g, int64_t lead, hipStream_t st, bool swizzle) {
  constexpr int ITER = 4;
  constexpr int ROWS = 4 * (8 / CPR) * ITER;
  dim3 grid((unsigned)(ceil_div(g.Kp / 64, CPR) * ceil_div(g.Rp, ROWS)), (unsigned)lead);
  if (swizzle)
    hipLaunchKernelGGL((quantize_nvfp4_rowmajor_kernel<CPR, ITER, true>), grid, dim3(256), 0, st, out, sf, in, gs, g);
  else
    hipLaunchKernelGGL((quantize_nvfp4_rowmajor_kernel<CPR, ITER, false>), grid, dim3(256), 0, st, out, sf, in, gs, g);
}

}  // namespace ac4k

using namespace ac4k;

namespace ac4k {

// (device, stream) -> slot of synchronisation words for the single-launch quantizer, plus the launch
// tag.  A stream keeps its slot while it is among the OP_SLOTS most recently used streams of its
// device; a newcomer takes a free slot or evicts the least recently used one.  Tags count on per
// slot, so two launches that meet on one slot (an evicted stream whose kernel is still running)
// carry different tags: each of them then misses words of its own tag, stops waiting after the
// timeout and finishes through the kernel's slow path - slower, never wrong.
constexpr int OP_MAX_DEVICES = 16;
struct OnePassSlot {
  hipStream_t st;
  uint64_t last_use;  // 0 = never used
  uint32_t tag;
  uint32_t seq;       // launches of the single-launch kernel on this slot
  uint32_t seen;      // highest launch number whose timeout report has been acted on
  uint32_t backoff;   // calls that still take the three-launch path
};
static std::mutex g_slot_mutex;
static OnePassSlot g_slots[OP_MAX_DEVICES][OP_SLOTS];
static uint64_t g_slot_clock = 0;

// Timeout reports: one word per slot in mapped host memory, written by a workgroup of the single-launch
// kernel whose grid wait ran out (its peers were not all resident: the GPU is shared with other kernels),
// read here before a later call on that slot - no synchronisation, no copy.  A stream that has just seen a
// timeout takes the three-launch path for the next ONEPASS_BACKOFF_CALLS calls, whose cost does not depend
// on what else runs, and then tries the single launch again.  The page is allocated once per GPU on the
// first call that needs it (not while any stream of the thread captures); without it nothing is reported
// and every call keeps the single launch, which stays correct.
constexpr uint32_t ONEPASS_BACKOFF_CALLS = 64;
struct TimeoutReports {
  uint32_t *host = nullptr, *dev = nullptr;
  bool tried = false;
};
static TimeoutReports g_reports[OP_MAX_DEVICES];
static std::atomic<uint64_t> g_timeouts_seen{0};

static uint32_t *timeout_reports(int dev) {  // called with g_slot_mutex held
  TimeoutReports &r = g_reports[dev];
  if (!r.tried) {
    r.tried = true;
    void *h = nullptr, *d = nullptr;
    if (hipHostMalloc(&h, OP_SLOTS * sizeof(uint32_t), hipHostMallocMapped) == hipSuccess && h &&
        hipHostGetDevicePointer(&d, h, 0) == hipSuccess && d) {
      memset(h, 0, OP_SLOTS * sizeof(uint32_t));
      r.host = static_cast<uint32_t *>(h);
      r.dev = static_cast<uint32_t *>(d);
    } else {
      (void)hipGetLastError();
      if (h) (void)hipHostFree(h);
    }
  }
  return r.dev;
}

// -> false: take the three-launch path (no slot for this device, or the stream is backing off after a timeout)
static bool onepass_slot(hipStream_t st, int *slot, uint32_t *tag, uint32_t **report, uint32_t *seq) {
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= OP_MAX_DEVICES) return false;
  std::lock_guard<std::mutex> lock(g_slot_mutex);
  OnePassSlot *t = g_slots[dev];
  int pick = -1, oldest = 0;
  for (int i = 0; i < OP_SLOTS; ++i) {
    if (t[i].last_use && t[i].st == st) {
      pick = i;
      break;
    }
    if (t[i].last_use < t[oldest].last_use) oldest = i;  // never-used slots (0) come first
  }
  if (pick < 0) {
    pick = oldest;
    t[pick].st = st;
    t[pick].backoff = 0;
  }
  t[pick].last_use = ++g_slot_clock;
  *report = timeout_reports(dev);
  if (g_reports[dev].host) {
    const uint32_t reported = *reinterpret_cast<volatile uint32_t *>(g_reports[dev].host + pick);
    if ((int32_t)(reported - t[pick].seen) > 0) {  // a launch since the last look ran out of time
      t[pick].seen = reported;
      t[pick].backoff = ONEPASS_BACKOFF_CALLS;
      g_timeouts_seen.fetch_add(1, std::memory_order_relaxed);
    }
  }
  if (t[pick].backoff > 0) {
    --t[pick].backoff;
    return false;
  }
  t[pick].tag = t[pick].tag % 0xffffu + 1;  // 1 .. 65535
  t[pick].seq += 1;
  *slot = pick;
  *tag = t[pick].tag;
  *seq = t[pick].seq;
  return true;
}

// True while `st` records into a graph (or when that cannot be told).  A captured launch would replay
// with the tag and the slot of the capture, possibly next to other replays or eager launches on the
// same slot, so captured calls take the path whose whole state lives in the caller's buffers.
static bool stream_is_capturing(hipStream_t st) {
  hipStreamCaptureStatus status = hipStreamCaptureStatusNone;
  if (hipStreamIsCapturing(st, &status) != hipSuccess) {
    (void)hipGetLastError();
    return true;
  }
  return status != hipStreamCaptureStatusNone;
}

// *gs = max|x| / max_scale with no scratch of the library's own: *gs zeroed by a fill kernel, then
// block maxima folded in with (mostly skipped) atomics.
static void launch_global_scale(float *gs, const void *x, int64_t n, float max_scale, hipStream_t st) {
  hipLaunchKernelGGL(zero_u32_kernel, dim3(1), dim3(1), 0, st, reinterpret_cast<uint32_t *>(gs));
  if (n == 0) return;
  const uintptr_t addr = reinterpret_cast<uintptr_t>(x);
  int64_t head = ((16 - (addr & 15)) & 15) / 2;
  if (head > n) head = n;
  const int64_t nvec = (n - head) / 8;
  int64_t blocks = ceil_div(nvec, (int64_t)AMAX_THREADS * AMAX_UNROLL);
  if (blocks < 1) blocks = 1;
  if (blocks > AMAX_MAX_BLOCKS) blocks = AMAX_MAX_BLOCKS;
  hipLaunchKernelGGL(amax_scale_bf16_atomic_kernel, dim3((unsigned)blocks), dim3(AMAX_THREADS), 0, st,
                     reinterpret_cast<uint32_t *>(gs), static_cast<const uint16_t *>(x), n, head, nvec, max_scale);
}

// Bound of the single-launch quantizer's grid wait in 100 MHz ticks (200 us); 0 = one look at the
// other workgroups' words, then the slow path; a negative value switches the single-launch path off.
static std::atomic<int64_t> g_sync_timeout_ticks{20000};

// which path the last ac4k_quantize_nvfp4_bf16 call of this host thread took (introspection for tests)
enum QuantPath { QPATH_NONE = 0, QPATH_SMALL = 1, QPATH_ONEPASS = 2, QPATH_TWO_KERNEL = 3 };
static thread_local int g_last_quantize_path = QPATH_NONE;

static int device_cu_count() {
  static std::atomic<int> cached[64];
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 0;
  int n = cached[dev].load();
  if (n == 0) {
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess) return 0;
    cached[dev].store(n);
  }
  return n;
}

struct OnePassLaunch {
  int slot;
  uint32_t tag, seq;
  uint32_t *report;
};
template <int NV>
static void launch_onepass(uint32_t *out, uint32_t *sf, const uint4 *in, float *gs, const OnePassGeom &g, int nwg,
                           const OnePassLaunch &l, float max_scale, uint64_t ticks, hipStream_t st) {
  hipLaunchKernelGGL((quantize_nvfp4_onepass_kernel<NV>), dim3(nwg), dim3(OP_THREADS), 0, st, out, sf, in, gs, g, l.slot,
                     l.tag, max_scale, ticks, l.report, l.seq);
}

// Up to 16 segments (256 KB) every workgroup can afford to read the whole tensor for its maximum:
// one launch of a few microseconds, no grid wait.
constexpr int SMALL_MAX_SEGS = 16;

static void launch_small(uint32_t *out, uint32_t *sf, const uint4 *in, float *gs, const OnePassGeom &g,
                         float max_scale, hipStream_t st) {
  const unsigned nseg = (unsigned)ceil_div((int64_t)g.total_chunks, 128);
  const dim3 grid(nseg <= 1 ? 1 : nseg * 8), block(OP_THREADS);  // NSEG > 1: one working workgroup in eight, all on one XCD
  if (nseg <= 1) hipLaunchKernelGGL(quantize_nvfp4_small_kernel<1>, grid, block, 0, st, out, sf, in, gs, g, max_scale);
  else if (nseg <= 2) hipLaunchKernelGGL(quantize_nvfp4_small_kernel<2>, grid, block, 0, st, out, sf, in, gs, g, max_scale);
  else if (nseg <= 4) hipLaunchKernelGGL(quantize_nvfp4_small_kernel<4>, grid, block, 0, st, out, sf, in, gs, g, max_scale);
  else if (nseg <= 8) hipLaunchKernelGGL(quantize_nvfp4_small_kernel<8>, grid, block, 0, st, out, sf, in, gs, g, max_scale);
  else hipLaunchKernelGGL(quantize_nvfp4_small_kernel<16>, grid, block, 0, st, out, sf, in, gs, g, max_scale);
}

// Global scale + nvfp4 quantize of a dense [lead, R, K] tensor in one launch, when the shape allows
// it.  Returns QPATH_NONE (nothing launched) when the caller has to take the two-kernel path.
static int try_quantize_nvfp4_onepass(void *out, void *sf, float *gs, const void *in, int64_t d0, int64_t d1,
                                      int64_t R, int64_t K, int64_t s0, int64_t s1, int64_t sR, int64_t sK,
                                      int swizzle, float max_scale, hipStream_t st) {
  const int64_t ticks = g_sync_timeout_ticks.load();
  if (ticks < 0 || sK != 1 || K % 64 != 0 || sR != K) return QPATH_NONE;
  if ((d1 > 1 && s1 != R * K) || (d0 > 1 && s0 != d1 * R * K)) return QPATH_NONE;
  if (reinterpret_cast<uintptr_t>(in) & 15) return QPATH_NONE;
  const int64_t lead = d0 * d1, chunks = lead * R * (K / 64);
  int nwg = device_cu_count();
  if (nwg > OP_MAX_WGS) nwg = OP_MAX_WGS;
  if (nwg < 8 || chunks > (int64_t)nwg * 128 * OP_MAX_NV) return QPATH_NONE;
  const OnePassGeom g{(uint32_t)chunks, (uint32_t)(K / 64), (uint32_t)R, (uint32_t)align_up(R, 16), (uint32_t)lead,
                      swizzle ? 1u : 0u};
  // small: one launch, no grid wait, no state.  Above eight segments the kernel with the grid wait is
  // faster (256 KB: 5.0 against 6.1 us in front of a dependent kernel), but it is not available under
  // capture, where the stateless kernel keeps the call at one launch.
  if (chunks <= 128 * 8 || (chunks <= 128 * SMALL_MAX_SEGS && stream_is_capturing(st))) {
    launch_small(static_cast<uint32_t *>(out), static_cast<uint32_t *>(sf), static_cast<const uint4 *>(in), gs, g,
                 max_scale, st);
    return QPATH_SMALL;
  }
  if (stream_is_capturing(st)) return QPATH_NONE;
  OnePassLaunch l{-1, 0, 0, nullptr};
  if (!onepass_slot(st, &l.slot, &l.tag, &l.report, &l.seq)) return QPATH_NONE;
  const int64_t per_wg = ceil_div(chunks, (int64_t)nwg * 128);  // 16 KB segments per workgroup
  uint32_t *o = static_cast<uint32_t *>(out), *s = static_cast<uint32_t *>(sf);
  const uint4 *x = static_cast<const uint4 *>(in);
  if (per_wg <= 1)
    launch_onepass<1>(o, s, x, gs, g, nwg, l, max_scale, (uint64_t)ticks, st);
  else if (per_wg <= 2)
    launch_onepass<2>(o, s, x, gs, g, nwg, l, max_scale, (uint64_t)ticks, st);
  else if (per_wg <= 4)
    launch_onepass<4>(o, s, x, gs, g, nwg, l, max_scale, (uint64_t)ticks, st);
  else if (per_wg <= 8)
    launch_onepass<8>(o, s, x, gs, g, nwg, l, max_scale, (uint64_t)ticks, st);
  else
    launch_onepass<16>(o, s, x, gs, g, nwg, l, max_scale, (uint64_t)ticks, st);
  return QPATH_ONEPASS;
}

static int launch_quantize_nvfp4(void *out, void *sf, const void *in, const float *gsrc, int64_t d0,
                                 int64_t d1, int64_t R, int64_t K, int64_t s0, int64_t s1, int64_t sR, int64_t sK,
                                 int swizzle, hipStream_t st) {
  QuantGeom g{d1, R, K, align_up(K, 64), align_up(R, 16), s0, s1, sR, sK, 0};
  uint8_t *o = static_cast<uint8_t *>(out), *s = static_cast<uint8_t *>(sf);
  const uint16_t *x = static_cast<const uint16_t *>(in);
  const int64_t lead_all = d0 * d1;
  for (g.lead0 = 0; g.lead0 < lead_all; g.lead0 += 65535) {
    const int64_t lead = lead_all - g.lead0 < 65535 ? lead_all - g.lead0 : 65535;
    if (rowmajor_ok(in, K, s0, s1, sR, sK) && ceil_div(g.Kp, 64) * ceil_div(g.Rp, 16) < (1ll << 31)) {
      const int64_t chunks = g.Kp / 64;
      const bool sw = swizzle != 0;
      // four chunks per wave row: a workgroup then covers 32 rows x 256 elements, and each scale
      // column gets a 128-byte run; eight chunks per row measured 4-12 % slower on every shape
      if (chunks >= 3)
        launch_nvfp4_rowmajor<4>(o, s, x, gsrc, g, lead, st, sw);
      else if (chunks == 2)
        launch_nvfp4_rowmajor<2>(o, s, x, gsrc, g, lead, st, sw);
      else
        launch_nvfp4_rowmajor<1>(o, s, x, gsrc, g, lead, st, sw);
    } else if (crossmajor_ok(in, R, s0, s1, sR, sK) && ceil_div(g.Rp, 128) <= 65535) {
      // (position along the reduce dim as the fast grid index: the packed rows are written in runs along it)
      const dim3 grid = crossmajor_grid(g, ceil_div(g.Kp / 64, 4), ceil_div(g.Rp, 128), lead);
      if (swizzle)
        hipLaunchKernelGGL(quantize_nvfp4_crossmajor_kernel<true>, grid, dim3(256), 0, st, o, s, x, gsrc, g);
      else
        hipLaunchKernelGGL(quantize_nvfp4_crossmajor_kernel<false>, grid, dim3(256), 0, st, o, s, x, gsrc, g);
    } else {
      AC4K_REQUIRE(g.Kp / 64 <= 65535, "reduce dim too large for the strided path (%lld)", (long long)K);
      dim3 grid((unsigned)ceil_div(g.Rp, 256), (unsigned)(g.Kp / 64), (unsigned)lead);
      if (swizzle)
        hipLaunchKernelGGL(quantize_nvfp4_generic_kernel<true>, grid, dim3(256), 0, st, o, s, x, gsrc, g);
      else
        hipLaunchKernelGGL(quantize_nvfp4_generic_kernel<false>, grid, dim3(256), 0, st, o, s, x, gsrc, g);
    }
  }
  return 0;
}

}  // namespace ac4k

extern "C" __attribute__((visibility("default"))) int ac4k_global_scale_bf16(float *gs, const void *x, int64_t n, float max_scale,
                                      ac4k_stream_t stream) {
  AC4K_REQUIRE(gs && (x || n == 0), "null pointer argument");
  AC4K_REQUIRE(n >= 0, "n must be non-negative");
  AC4K_REQUIRE((reinterpret_cast<uintptr_t>(x) & 1) == 0, "x must be 2-byte aligned");
  launch_global_scale(gs, x, n, max_scale, (hipStream_t)stream);
  return check_launch("ac4k_global_scale_bf16");
}

extern "C" __attribute__((visibility("default"))) int ac4k_quantize_nvfp4(void *out, void *sf, const void *in, const float *global_scale, int64_t d0,
                                   int64_t d1, int64_t R, int64_t K, int64_t s0, int64_t s1, int64_t sR,
                                   int64_t sK, int swizzle, ac4k_stream_t stream) {
  if (int rc = check_geom(out, sf, in, global_scale, d0, d1, R, K, s0, s1, sR, sK)) return rc;
  if (int rc = launch_quantize_nvfp4(out, sf, in, global_scale, d0, d1, R, K, s0, s1, sR, sK, swizzle, (hipStream_t)stream))
    return rc;
  return check_launch("ac4k_quantize_nvfp4");
}

extern "C" __attribute__((visibility("default"))) int ac4k_quantize_nvfp4_bf16(void *out, void *sf, float *global_scale, const void *in, int64_t d0,
                                        int64_t d1, int64_t R, int64_t K, int64_t s0, int64_t s1, int64_t sR,
                                        int64_t sK, int swizzle, float max_scale, ac4k_stream_t stream) {
  if (int rc = check_geom(out, sf, in, global_scale, d0, d1, R, K, s0, s1, sR, sK)) return rc;
  // the global scale is the maximum over the d0*d1*R*K elements that start at `in`: the four dims
  // must tile that range exactly (any order), as the contiguous tensor of the reference op does
  AC4K_REQUIRE(dense_permutation(d0, d1, R, K, s0, s1, sR, sK),
               "in must be a dense (permuted) tensor: its strides do not tile d0*d1*R*K contiguous elements");
  hipStream_t st = (hipStream_t)stream;
  g_last_quantize_path = try_quantize_nvfp4_onepass(out, sf, global_scale, in, d0, d1, R, K, s0, s1, sR, sK, swizzle,
                                                    max_scale, st);
  if (g_last_quantize_path != QPATH_NONE) return check_launch("ac4k_quantize_nvfp4_bf16");
  // two passes over the input, all state in the caller's buffers: fill, maxima into *global_scale,
  // then the quantize kernel that reads it
  g_last_quantize_path = QPATH_TWO_KERNEL;
  launch_global_scale(global_scale, in, d0 * d1 * R * K, max_scale, st);
  if (int rc = launch_quantize_nvfp4(out, sf, in, global_scale, d0, d1, R, K, s0, s1, sR, sK, swizzle, st)) return rc;
  return check_launch("ac4k_quantize_nvfp4_bf16");
}

extern "C" __attribute__((visibility("default"))) int ac4k_debug_last_quantize_path(void) { return ac4k::g_last_quantize_path; }

extern "C" __attribute__((visibility("default"))) int64_t ac4k_debug_quantize_timeouts_seen(void) {
  return (int64_t)ac4k::g_timeouts_seen.load(std::memory_order_relaxed);
}

namespace ac4k {

template <RowFmt FMT, int LPR, int NV>
static void launch_rowwise_rowmajor(uint8_t *out, float *sf, const uint16_t *in, const void *smax,
                                    const QuantGeom &g, int64_t lead, hipStream_t st, bool swizzle) {
  dim3 grid((unsigned)ceil_div(g.Rp, 256 / LPR), (unsigned)lead);
  if (swizzle && FMT == RowFmt::FP8)
    hipLaunchKernelGGL((quantize_rowwise_rowmajor_kernel<FMT, LPR, NV, FMT == RowFmt::FP8>), grid, dim3(256), 0, st, out,
                       sf, in, smax, g);
  else
    hipLaunchKernelGGL((quantize_rowwise_rowmajor_kernel<FMT, LPR, NV, false>), grid, dim3(256), 0, st, out, sf, in,
                       smax, g);
}

template <RowFmt FMT>
static int quantize_rowwise(void *out, float *sf, const void *in, const void *smax, int64_t d0, int64_t d1,
                            int64_t R, int64_t K, int64_t s0, int64_t s1, int64_t sR, int64_t sK, int swizzle,
                            hipStream_t st, const char *what) {
  if (int rc = check_geom(out, sf, in, smax, d0, d1, R, K, s0, s1, sR, sK)) return rc;
  QuantGeom g{d1, R, K, align_up(K, 16), align_up(R, 16), s0, s1, sR, sK, 0};
  uint8_t *o = static_cast<uint8_t *>(out);
  const uint16_t *x = static_cast<const uint16_t *>(in);
  const int64_t lead_all = d0 * d1;
  for (g.lead0 = 0; g.lead0 < lead_all; g.lead0 += 65535) {
    const int64_t lead = lead_all - g.lead0 < 65535 ? lead_all - g.lead0 : 65535;
    if (rowmajor_ok(in, K, s0, s1, sR, sK) && K <= 16384) {
      const bool sw = swizzle != 0;
      if (K <= 64)
        launch_rowwise_rowmajor<FMT, 8, 1>(o, sf, x, smax, g, lead, st, sw);
      else if (K <= 128)
        launch_rowwise_rowmajor<FMT, 16, 1>(o, sf, x, smax, g, lead, st, sw);
      else if (K <= 256)
        launch_rowwise_rowmajor<FMT, 32, 1>(o, sf, x, smax, g, lead, st, sw);
      else if (K <= 512)
        launch_rowwise_rowmajor<FMT, 64, 1>(o, sf, x, smax, g, lead, st, sw);
      else if (K <= 1024)
        launch_rowwise_rowmajor<FMT, 64, 2>(o, sf, x, smax, g, lead, st, sw);
      else if (K <= 2048)
        launch_rowwise_rowmajor<FMT, 64, 4>(o, sf, x, smax, g, lead, st, sw);
      else if (K <= 4096)
        launch_rowwise_rowmajor<FMT, 64, 8>(o, sf, x, smax, g, lead, st, sw);
      else if (K <= 8192)
        launch_rowwise_rowmajor<FMT, 64, 16>(o, sf, x, smax, g, lead, st, sw);
      else
        launch_rowwise_rowmajor<FMT, 64, 32>(o, sf, x, smax, g, lead, st, sw);
    } else if (!swizzle && rowmajor_ok(in, K, s0, s1, sR, sK)) {  // rows too long for the register file
      dim3 grid((unsigned)ceil_div(g.Rp, 4), (unsigned)lead);
      hipLaunchKernelGGL((quantize_rowwise_longrow_kernel<FMT>), grid, dim3(256), 0, st, o, sf, x, smax, g);
    } else if (crossmajor_ok(in, R, s0, s1, sR, sK) && ceil_div(g.Rp, 128) <= 65535 && ceil_div(K, CM_KSPAN) <= 65535) {
      // row maxima as bf16 bit patterns in the scale array, quantize from them, then scale them in place
      uint32_t *bits = reinterpret_cast<uint32_t *>(sf) + g.lead0 * g.Rp;  // the kernels index by absolute lead
      const int64_t nsf = lead * g.Rp;
      hipLaunchKernelGGL(fill_u32_kernel, dim3((unsigned)ceil_div(nsf, 256)), dim3(256), 0, st, bits, nsf, 0u);
      // Both kernels walk the grid along the dim of smaller input stride first (measured on
      // (1,75600,40,128), cross 3, reduce 1: 412 us against 440 us; the nvfp4 kernel, whose packed
      // rows are a quarter as long, loses 6% by the same change and keeps the reduce dim first).
      const int64_t kblocks = ceil_div(g.Kp / 16, 16);  // of the quantize kernel; the maxima kernel has fewer
      g.lead_fast = crossmajor_lead_fast(d1, s1, sK, kblocks);
      hipLaunchKernelGGL(rowwise_crossmajor_amax_kernel, crossmajor_grid(g, ceil_div(K, CM_KSPAN), ceil_div(g.Rp, 128), lead),
                         dim3(256), 0, st, reinterpret_cast<uint32_t *>(sf), x, g);
      const dim3 grid = crossmajor_grid(g, kblocks, ceil_div(g.Rp, 128), lead);
      if (swizzle)
        hipLaunchKernelGGL((quantize_rowwise_crossmajor_kernel<FMT, true>), grid, dim3(256), 0, st, o,
                           reinterpret_cast<const uint32_t *>(sf), x, smax, g);
      else
        hipLaunchKernelGGL((quantize_rowwise_crossmajor_kernel<FMT, false>), grid, dim3(256), 0, st, o,
                           reinterpret_cast<const uint32_t *>(sf), x, smax, g);
      hipLaunchKernelGGL(rowwise_crossmajor_finalize_kernel<FMT>, dim3((unsigned)ceil_div(nsf, 256)), dim3(256), 0, st,
                         sf + g.lead0 * g.Rp, smax, nsf);
    } else {
      dim3 grid((unsigned)ceil_div(g.Rp, 256), (unsigned)lead);
      if (swizzle)
        hipLaunchKernelGGL((quantize_rowwise_generic_kernel<FMT, true>), grid, dim3(256), 0, st, o, sf, x, smax, g);
      else
        hipLaunchKernelGGL((quantize_rowwise_generic_kernel<FMT, false>), grid, dim3(256), 0, st, o, sf, x, smax, g);
    }
  }
  return check_launch(what);
}

}  // namespace ac4k

extern "C" __attribute__((visibility("default"))) int ac4k_quantize_fp8(void *out, float *sf, const void *in, const float *scale_max, int64_t d0,
                                 int64_t d1, int64_t R, int64_t K, int64_t s0, int64_t s1, int64_t sR,
                                 int64_t sK, int swizzle, ac4k_stream_t stream) {
  return quantize_rowwise<RowFmt::FP8>(out, sf, in, scale_max, d0, d1, R, K, s0, s1, sR, sK, swizzle,
                                       (hipStream_t)stream, "ac4k_quantize_fp8");
}

extern "C" __attribute__((visibility("default"))) int ac4k_quantize_int8(void *out, float *sf, const void *in, const int32_t *scale_max, int64_t d0,
                                  int64_t d1, int64_t R, int64_t K, int64_t s0, int64_t s1, int64_t sR,
                                  int64_t sK, ac4k_stream_t stream) {
  return quantize_rowwise<RowFmt::INT8>(out, sf, in, scale_max, d0, d1, R, K, s0, s1, sR, sK, 0,
                                        (hipStream_t)stream, "ac4k_quantize_int8");
}

extern "C" __attribute__((visibility("default"))) void ac4k_set_quantize_sync_timeout_us(int64_t us) {
  ac4k::g_sync_timeout_ticks.store(us < 0 ? -1 : us * 100);
  // a new bound starts with a clean slate: no stream keeps backing off because of waits under the old one,
  // reported and acted on or reported and not yet looked at
  std::lock_guard<std::mutex> lock(ac4k::g_slot_mutex);
  for (int d = 0; d < ac4k::OP_MAX_DEVICES; ++d)
    for (int i = 0; i < ac4k::OP_SLOTS; ++i) {
      ac4k::g_slots[d][i].backoff = 0;
      if (ac4k::g_reports[d].host) ac4k::g_slots[d][i].seen = *reinterpret_cast<volatile uint32_t *>(ac4k::g_reports[d].host + i);
    }
}

#ifdef AC4K_ONEPASS_TIMELINE
// Timeline build only: copies the per-workgroup clock stamps of the last single-launch quantize to
// host memory ([256][8] 100 MHz ticks: 0 kernel entry, 1 loads in registers and own maximum known,
// 2 global maximum known, 3 nibbles stored, 4 scales stored).  Synchronises the device.
extern "C" __attribute__((visibility("default"))) int ac4k_debug_onepass_timeline(uint64_t *host_out) {
  hipError_t e = hipDeviceSynchronize();
  if (e == hipSuccess)
    e = hipMemcpyFromSymbol(host_out, HIP_SYMBOL(ac4k::g_onepass_timeline), sizeof(uint64_t) * ac4k::OP_MAX_WGS * 8);
  return e == hipSuccess ? 0 : ac4k::set_error("ac4k_debug_onepass_timeline: %s", hipGetErrorString(e));
}
#endif
