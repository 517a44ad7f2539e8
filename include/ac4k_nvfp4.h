/*
 * ac4k_nvfp4.h — C ABI of the MI355X (gfx950) NVFP4 path.
 *
 * One shared library, plain pointers and sizes, no torch / pybind types.  It
 * takes the place of the reference's pybind11 module `ac4k_kernel._cuda_ops`
 * (lib/cuda_bindings.cc:37-97, declarations in include/ac4k_kernel/ops.h:27-48)
 * for the quantize and linear entry points, and of the Triton global-scale
 * helper (python/ac4k_kernel/ops/quant.py:33-59).
 *
 * Conventions (identical to the reference binding):
 *   - every pointer is DEVICE memory owned by the caller; the library never
 *     allocates, frees or synchronises; work is enqueued on `stream`
 *     (a hipStream_t; NULL = the default stream) and returns immediately;
 *   - scalars that the reference passes as 0-dim device tensors
 *     (global_scale, scale_max) are device pointers here too;
 *   - return value 0 = launched; non-zero = rejected, nothing was launched and
 *     ac4k_last_error() (thread-local) says why.  The conditions are the
 *     reference's TORCH_CHECKs that can be stated on raw pointers and sizes.
 *
 * Quantizer geometry.  The reference host code left-pads the input to 4-D and
 * passes the sizes/strides of the two dims that are neither cross nor reduce
 * (quantize_nvfp4.cu:226-241,257-260); the same is passed here:
 *   d0,d1 : sizes of the two leading (batch-like) dims, 1 when absent
 *   R, K  : cross (row) and reduce sizes
 *   s0,s1,sR,sK : element strides of those four dims in `in`
 * Outputs are dense: out [d0,d1,R,*], sf as documented per function.
 */
#ifndef AC4K_NVFP4_H_
#define AC4K_NVFP4_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef void *ac4k_stream_t; /* hipStream_t */

/* dtype tags for D and bias of ac4k_linear_nvfp4 */
enum { AC4K_DTYPE_BF16 = 0, AC4K_DTYPE_FP16 = 1, AC4K_DTYPE_FP32 = 2 };

/* Module attributes of lib/cuda_bindings.cc:41-44 (__arch__, __backend__, __version__,
 * __arch_description__). */
const char *ac4k_arch(void);             /* "gfx950" */
const char *ac4k_arch_description(void); /* "AMD Instinct MI355X (CDNA4)" */
const char *ac4k_backend(void);          /* "rocm" */
const char *ac4k_version(void);          /* "0.1.0" */
const char *ac4k_last_error(void);

/* Replaces _global_scale / _triton_global_scale_kernel
 * (python/ac4k_kernel/ops/quant.py:33-59):  *gs = fp32(max|x|) / max_scale over n
 * contiguous bf16 values.  *gs needs no initialisation by the caller. */
int ac4k_global_scale_bf16(float *gs, const void *x, int64_t n, float max_scale,
                           ac4k_stream_t stream);

/* Replaces ac4k::quantize_nvfp4 (lib/cuda/sm120/quantize_nvfp4.cu:164-271).
 * out: uint8 [d0,d1,R,align_up(K,64)/2], low nibble = even element.
 * sf : e4m3   [d0,d1,align_up(K,64)/64,align_up(R,16),4].
 * Every byte of both is written (pad nibbles and pad-row scales are 0).
 * swizzle != 0: reduce dim permuted as reshape(-1,4,4,2).permute(0,2,1,3). */
int ac4k_quantize_nvfp4(void *out, void *sf, const void *in, const float *global_scale, int64_t d0,
                        int64_t d1, int64_t R, int64_t K, int64_t s0, int64_t s1, int64_t sR,
                        int64_t sK, int swizzle, ac4k_stream_t stream);

/* The nvfp4 branch of Ac4kQuantizeOp.forward in one call
 * (python/ac4k_kernel/ops/quant.py:187-242): *global_scale = max|in| / max_scale over the whole
 * input, then ac4k_quantize_nvfp4 with it.  `in` must be dense: the four dims, in any order, tile
 * d0*d1*R*K contiguous elements (the reference op makes its input contiguous, :201); other strides
 * are rejected.  Nothing to initialise, no host synchronisation.
 *   - dense row-major tensors (sK == 1, K % 64 == 0, 16-byte aligned) of up to 128 KB (256 KB while
 *     `stream` is capturing): one launch;
 *   - the same up to 64 MiB: one launch of a kernel whose workgroups exchange their maxima through
 *     synchronisation words inside the library (32 sets per GPU, handed to the most recently used
 *     streams), see ac4k_set_quantize_sync_timeout_us;
 *   - everything else, and every call made while `stream` is capturing into a graph: three launches
 *     (fill, maxima, quantize) whose whole state is *global_scale - safe to replay on any stream,
 *     next to anything. */
int ac4k_quantize_nvfp4_bf16(void *out, void *sf, float *global_scale, const void *in, int64_t d0,
                             int64_t d1, int64_t R, int64_t K, int64_t s0, int64_t s1, int64_t sR,
                             int64_t sK, int swizzle, float max_scale, ac4k_stream_t stream);

/* Tuning knob of ac4k_quantize_nvfp4_bf16 (no counterpart in the reference): the workgroups of the
 * single-launch kernel wait for each other's maxima for at most this many microseconds (default
 * 200).  A workgroup whose wait runs out - its peers were not all resident because other kernels
 * hold the GPU - recomputes the missing maxima from memory itself and finishes: slower, same bits.
 * 0 = look once, then recompute (used by the tests; not reported as a timeout); 1 = the same, but
 * reported (a wait that runs out for certain, forced from the host by the tests); a negative value
 * switches the single-launch kernel off (three launches, as under graph capture).  A wait that runs
 * out costs the bound plus a second read of the missing workgroups' shares, so a stream on which it
 * happened takes the three-launch path for its next 64 calls (see ac4k_debug_quantize_timeouts_seen);
 * setting the bound also ends every such back-off. */
void ac4k_set_quantize_sync_timeout_us(int64_t us);

/* Introspection for tests (no counterpart in the reference): which path the last
 * ac4k_quantize_nvfp4_bf16 call of the calling host thread took: 0 none yet, 1 small one-launch
 * kernel, 2 single-launch kernel with the grid wait, 3 fill + maxima + quantize. */
int ac4k_debug_last_quantize_path(void);

/* Introspection (no counterpart in the reference): how many times this process has noticed that a launch of
 * the single-launch kernel ran out of waiting time.  The kernel reports it through a word of mapped host
 * memory; the next ac4k_quantize_nvfp4_bf16 call on that stream reads the word (no synchronisation) and
 * sends that stream's next 64 calls down the three-launch path, whose cost does not depend on what else
 * runs on the GPU; then the single launch is tried again. */
int64_t ac4k_debug_quantize_timeouts_seen(void);

/* Replaces ac4k::quantize_fp8 (lib/cuda/sm120/quantize_fp8.cu:192-290).
 * out: e4m3 [d0,d1,R,align_up(K,16)];  sf: fp32 [d0,d1,align_up(R,16)] = amax/scale_max.
 * swizzle != 0: reduce dim permuted as reshape(-1,2,4,2).permute(0,2,1,3). */
int ac4k_quantize_fp8(void *out, float *sf, const void *in, const float *scale_max, int64_t d0,
                      int64_t d1, int64_t R, int64_t K, int64_t s0, int64_t s1, int64_t sR,
                      int64_t sK, int swizzle, ac4k_stream_t stream);

/* Replaces ac4k::quantize_int8 (lib/cuda/sm120/quantize_int8.cu:175-262).
 * scale_max is an int32 device scalar, as in the reference (:189). */
int ac4k_quantize_int8(void *out, float *sf, const void *in, const int32_t *scale_max, int64_t d0,
                       int64_t d1, int64_t R, int64_t K, int64_t s0, int64_t s1, int64_t sR,
                       int64_t sK, ac4k_stream_t stream);

/* Replaces ac4k::linear_nvfp4 (lib/cuda/sm120/linear_nvfp4.cu:753-901).
 * D [M,N] (d_dtype) = (A . B^T) * (*A_gs * *B_gs) + bias.
 * A [M,K/2], B [N,K/2] packed e2m1 (uint8); A_sf [ceil(K/64),align_up(M,16),4],
 * B_sf [ceil(K/64),align_up(N,16),4] e4m3; bias [1,N] of bias_dtype or NULL.
 * K = 2 * (bytes per packed row), K % 16 == 0. */
int ac4k_linear_nvfp4(void *D, int d_dtype, const void *A, const void *A_sf, const float *A_gs,
                      const void *B, const void *B_sf, const float *B_gs, const void *bias,
                      int bias_dtype, int64_t M, int64_t N, int64_t K, ac4k_stream_t stream);

/* Linear for shapes that need device scratch to run at their best: same contract as ac4k_linear_nvfp4
 * (lib/cuda/sm120/linear_nvfp4.cu:753-901; the reference runs every shape through its one
 * 128x128 tile kernel).  Two families:
 *   - decode-sized, 1 <= M <= 32 and K % 256 == 0: kernels that stream the weights once (into
 *     registers for small M, through an LDS ring with 128- or 64-row tiles for larger M and for
 *     weights of 12225 to 24448 rows); the workspace receives the fp32 partial sums
 *     of their K ranges when they split K; A and B 16-byte aligned;
 *   - 32 < M with too few output tiles to fill the GPU and K % 128 == 0: split-K (the K-split-waves
 *     kernel up to M = 128 when K % 256 == 0, the tile kernel otherwise; tile shape and number of K
 *     ranges chosen by a cost model); the workspace receives the fp32 partial sums; A and B 16-byte
 *     aligned.
 * `workspace` = ac4k_linear_nvfp4_skinny_workspace_bytes(M,N,K) bytes of device memory, 256-byte
 * aligned, contents irrelevant.  The size function returns 0 for shapes that need no scratch: those
 * go to ac4k_linear_nvfp4, which runs the same kernels with one K range (a decode-sized shape with
 * 0 bytes may also come here, with a NULL workspace).  ac4k_linear_nvfp4 takes every shape; where this
 * entry point would split K it runs one K range per tile instead: fewer workgroups, same contract. */
int64_t ac4k_linear_nvfp4_skinny_workspace_bytes(int64_t M, int64_t N, int64_t K);
int ac4k_linear_nvfp4_skinny(void *D, int d_dtype, const void *A, const void *A_sf, const float *A_gs,
                             const void *B, const void *B_sf, const float *B_gs, const void *bias,
                             int bias_dtype, int64_t M, int64_t N, int64_t K, void *workspace,
                             int64_t workspace_bytes, ac4k_stream_t stream);

/* ac4k_linear_nvfp4_skinny without the workspace argument, for callers that cannot allocate
 * device memory (code under HIP graph capture, tight serving loops, harnesses that forbid
 * hipMalloc).  It has no counterpart in the reference.  The partial sums go to an array of
 * AC4K_STATIC_SCRATCH_BYTES that is part of the library's device image: every GPU the library runs
 * on holds one copy from the first call on that GPU until the process ends, and the call itself
 * allocates and frees nothing.  Same shapes, checks and results as ac4k_linear_nvfp4_skinny; a
 * shape whose ac4k_linear_nvfp4_skinny_workspace_bytes exceeds AC4K_STATIC_SCRATCH_BYTES is
 * rejected.  All calls on one GPU share that GPU's array: calls that overlap on one GPU (two
 * streams, two host threads on different streams) race on it; calls on one stream do not.  Make the
 * first call on a GPU outside graph capture (it looks up the array's address). */
#define AC4K_STATIC_SCRATCH_BYTES (32ll << 20)
int ac4k_linear_nvfp4_skinny_static(void *D, int d_dtype, const void *A, const void *A_sf,
                                    const float *A_gs, const void *B, const void *B_sf,
                                    const float *B_gs, const void *bias, int bias_dtype, int64_t M,
                                    int64_t N, int64_t K, ac4k_stream_t stream);

/* Tuning aid of the linear entry points (no counterpart in the reference; results stay within the
 * same tolerance): forces the tile of the packed-operand kernel to (64 mi) x (64 nj) with `splits` K
 * ranges (mi in {2,4}, nj in {1,2,4}, not (4,1); splits > 1 only takes effect in the workspace entry
 * points), the length of a K range of the decode-sized kernels (a multiple of 256; the register
 * kernel takes 256, 512 or 1024) and which decode-sized kernel runs (1 = weights streamed into
 * registers, 2 = weights streamed through an LDS ring in 128-row tiles, 3 = in 64-row tiles).  Zeros give each choice back to the library.
 * Process-wide; returns non-zero on values outside these sets. */
int ac4k_set_linear_tuning(int mi, int nj, int splits, int skinny_ks, int decode_kernel);

/* Pre-packed weight image.  No counterpart in the reference, which fetches the weights in their
 * tensor layout on every call (lib/cuda/sm120/linear_nvfp4.cu:586-633); it would sit beside
 * ac4k::linear_nvfp4 (lib/cuda/sm120/linear_nvfp4.cu:753-901).  Static weights are re-laid ONCE into
 * the order the kernels fetch them, and the linear then reads the image instead of B and B_sf.
 * The arithmetic is untouched: same nibbles, same scale bytes, same order of accumulation, so the
 * output is bit-identical to the entry point of the plain layout that runs the same kernel
 * (ac4k_linear_nvfp4, or ac4k_linear_nvfp4_skinny for the shapes it splits along K or streams
 * through the LDS ring).
 * Image: one block of 9216 bytes per (128 rows, 128 k), blocks of a 128-row band consecutive along
 * k, bands consecutive along n, N padded with zero rows to a whole band.  A block holds 128 rows x
 * 64 packed bytes, the 16-byte piece p of row r at position p ^ ((r >> 1) & 3) of its row, then the
 * scale dwords of the block's two 64-chunks, [2][128 rows].
 * ac4k_prepack_weight_nvfp4_bytes: size of the image, 0 when there is none (K % 128 != 0, or an
 * image of 4 GiB and more).  ac4k_prepack_weight_nvfp4: B [N,K/2], B_sf [K/64,align_up(N,16),4] ->
 * image (16-byte aligned).
 * ac4k_linear_nvfp4_prepacked: contract of ac4k_linear_nvfp4 with W_image in place of B and B_sf;
 * `workspace` as for ac4k_linear_nvfp4_skinny, of ac4k_linear_nvfp4_prepacked_workspace_bytes(M,N,K)
 * bytes (may be NULL when that is 0).  M <= 32 with K % 256 == 0 streams the image through the LDS
 * ring; everything else runs the tile kernel, split along K when there are too few tiles. */
int64_t ac4k_prepack_weight_nvfp4_bytes(int64_t N, int64_t K);
int ac4k_prepack_weight_nvfp4(void *image, const void *B, const void *B_sf, int64_t N, int64_t K,
                              ac4k_stream_t stream);
int64_t ac4k_linear_nvfp4_prepacked_workspace_bytes(int64_t M, int64_t N, int64_t K);
int ac4k_linear_nvfp4_prepacked(void *D, int d_dtype, const void *A, const void *A_sf,
                                const float *A_gs, const void *W_image, const float *B_gs,
                                const void *bias, int bias_dtype, int64_t M, int64_t N, int64_t K,
                                void *workspace, int64_t workspace_bytes, ac4k_stream_t stream);

/* Fused decode-sized linear: quantize(X,0,1) followed by linear(...) in one call.  No single
 * reference function: it equals the composition the reference's tests make
 * (test/test_linear_bench.py:128-137) — the activation bytes, scales and global scale it
 * produces are those of ac4k_quantize_nvfp4_bf16 (it is that call), and they are returned:
 * X bf16 [M,K] contiguous -> X_q [M,K/2], X_sf [K/64,align_up(M,16),4], X_gs (1 float).
 * workspace as for ac4k_linear_nvfp4_skinny. */
int ac4k_linear_nvfp4_fused_bf16(void *D, int d_dtype, const void *X, void *X_q, void *X_sf,
                                 float *X_gs, const void *B, const void *B_sf, const float *B_gs,
                                 const void *bias, int bias_dtype, int64_t M, int64_t N, int64_t K,
                                 void *workspace, int64_t workspace_bytes, ac4k_stream_t stream);

/* Replaces ac4k::mha_nvfp4_fwd (include/ac4k_kernel/ops.h:12-16, lib/cuda/sm120/mha_nvfp4.cu:911-1077):
 * O = softmax(Q K^T * sm_scale) V on NVFP4 operands, the consumer of the quantizer's swizzled layout.
 * q [B,H,Nq,Dqk/2], k [B,H,Nkv,Dqk/2] packed e2m1 with scales [B,H,Dqk/64,align_up(rows,16),4];
 * v [B,H,Dv,align_up(Nkv,64)/2] quantized along the kv dim with swizzle (quantize(v, 3, N_dim, swizzle=True)),
 * v_sf [B,H,align_up(Nkv,64)/64,align_up(Dv,16),4]; the three global scales are device scalars;
 * O bf16 [B,H,Nq,Dv] addressed through its four element strides (the reference passes a permuted view).
 * The attention probabilities are re-quantized to NVFP4 per 16-block with the global scale 1/2688, as in
 * mha_nvfp4.cu:248-319.  Dqk = 2 * (packed row bytes) must be 64 or 128 (the quantizer pads packed rows to whole 64-chunks), Dv any
 * number up to 128. */
int ac4k_mha_nvfp4_fwd(void *O, int64_t o_b_stride, int64_t o_h_stride, int64_t o_n_stride,
                       int64_t o_d_stride, const void *q, const void *q_sf, const float *q_gs,
                       const void *k, const void *k_sf, const float *k_gs, const void *v,
                       const void *v_sf, const float *v_gs, int64_t B, int64_t H, int64_t Nq,
                       int64_t Nkv, int64_t Dqk, int64_t Dv, float sm_scale, ac4k_stream_t stream);

/* Replaces ac4k::mha_int8_x_fp8_fwd (include/ac4k_kernel/ops.h:18-21, lib/cuda/sm120/mha_int8_x_fp8.cu:979-1137):
 * O = softmax(Q K^T * sm_scale) V with Q K^T on int8 and P V on e4m3.
 * q int8 [B,H,Nq,Dqk], q_sf fp32 [B,H,ceil(Nq/q_quantize_block_size)] (block 32 or 64);
 * k int8 [B,H,Nkv,Dqk], k_sf fp32 [B,H,ceil(Nkv/128)] (k_quantize_block_size must be 128);
 * v e4m3 [B,H,Dv,align_up(Nkv,16)] quantized per (head, d) row along kv with the 16-group swizzle
 * (quantize(v, 3, N_dim, swizzle=True, max_scale=2.25, precision="fp8e4m3")), v_sf fp32 [B,H,align_up(Dv,16)];
 * O bf16 [B,H,Nq,Dv] addressed through its four element strides.  The probabilities are held up to 2^7.5 and
 * converted to e4m3 per element (mha_int8_x_fp8.cu:718-736,323-345); P V accumulates in fp32 (the reference's MMA
 * accumulates each kv tile in fp16).  Dqk: a multiple of 16 up to 128 (the quantizer pads the head dim to 16), Dv any
 * number up to 128. */
int ac4k_mha_int8_x_fp8_fwd(void *O, int64_t o_b_stride, int64_t o_h_stride, int64_t o_n_stride,
                            int64_t o_d_stride, const void *q, const float *q_sf,
                            int q_quantize_block_size, const void *k, const float *k_sf,
                            int k_quantize_block_size, const void *v, const float *v_sf, int64_t B,
                            int64_t H, int64_t Nq, int64_t Nkv, int64_t Dqk, int64_t Dv, float sm_scale,
                            ac4k_stream_t stream);

/* Replaces _int8_quantize / _triton_block_token_quantize (python/ac4k_kernel/ops/attention.py:18-99), the
 * quantizer of Q and K in front of ac4k_mha_int8_x_fp8_fwd: x bf16 [B,H,N,D] with element strides
 * (s_b, s_h, s_n, 1) -> y int8 [B,H,N,align_up(D,16)] (pad columns 0), scale fp32 [B,H,ceil(N/block)];
 * one scale = max|x| / 127 per block of `block` tokens of a head, y = int8(trunc(x / scale)), 0 where the
 * scale is 0.  block: a power of two, at least 16. */
int ac4k_quantize_int8_token_block_bf16(void *y, float *scale, const void *x, int64_t B, int64_t H,
                                        int64_t N, int64_t D, int64_t s_b, int64_t s_h, int64_t s_n,
                                        int block, ac4k_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* AC4K_NVFP4_H_ */
