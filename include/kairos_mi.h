/*
 * kairos_mi.h -- C ABI of the MI355X (gfx950) switched mixed-precision linear path.
 *
 * Every entry point takes raw DEVICE pointers, sizes and a HIP stream (passed as void*, i.e. a
 * hipStream_t; NULL = the null stream).  The caller owns and allocates every buffer, outputs and
 * scratch included; nothing here allocates, frees or synchronises, and no call leaves state behind
 * that a later call's result depends on.  Functions may be called from any host thread; the only
 * per-thread state is the last error message and the test hooks kmi_gemm_force_tile /
 * kmi_gemm_force_splits (marked below).  A LUT handle must not be used from two threads at once.
 * Return value: KMI_OK (0) or a negative KMI_E_* code; kmi_get_last_error_string() gives the
 * calling thread's last message.  Nothing throws across this boundary.
 *
 * Conventions.  N = out_features, K = in_features, M = tokens, G = group size (128 only).
 *   qweight       int16  [N/4, K]   packed uint4, four-row interleave, 64-wide K blocks
 *                                   (thirdparty/AWQ/awq_method.py:5-38)
 *   scales,       fp16   [Gp, N]    Gp = 8*ceil((K/G)/8) rows, row g = group g, padded rows unused
 *   scaled_zeros                    (thirdparty/AWQ/awq_method.py:40-75); row stride is N
 *   x / out       fp16   [M, K] / [M, N] row-major
 *   w8 / w16      int8 / fp16 [N, K] row-major (K contiguous)
 *   bias          fp16   [N] or NULL; added in fp16 after the product is rounded to fp16, as
 *                 `out += bias` does (kairos/dynamic_linear.py:165-166)
 * File:line citations name the reference interface each entry point replaces.
 */
#ifndef KAIROS_MI_H
#define KAIROS_MI_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define KMI_OK 0
#define KMI_E_NULL (-1)        /* a required pointer is NULL */
#define KMI_E_SHAPE (-2)       /* a size is non-positive or violates a divisibility rule */
#define KMI_E_GROUP (-3)       /* group size other than 128 */
#define KMI_E_M_RANGE (-4)     /* M outside the range the kernel family supports */
#define KMI_E_ALIGN (-5)       /* a pointer is not 16-byte aligned */
#define KMI_E_LAUNCH (-6)      /* the HIP runtime rejected the launch */
#define KMI_E_HANDLE (-7)      /* invalid LUT handle */

#define KMI_GEMV_MAX_M 64      /* largest M kmi_gemv_w4a16 accepts */

int kmi_version(void);
const char* kmi_get_last_error_string(void);

/* ---- on-demand weight conversion ------------------------------------------------------------ */

/* out_f16[n,k] = fma_f16(q[n,k], scales[k/G,n], scaled_zeros[k/G,n]), single rounding.
 * Replaces dequant_interleaved_int4_to_fp16 (kernels/csrc/pybind.cpp:22,
 * kernels/csrc/kairos_kernel/dequant_awq_format/dequant_i4_to_f16.cu:155-185).
 * Needs N%4==0, K%128==0. */
int kmi_cvt_i4_to_f16(void* out_f16, const void* qweight, const void* scales, const void* scaled_zeros,
                      int N, int K, int G, void* stream);

/* out_i8[n,k] = (int8) fma_f16(q, scales_to8, scaled_zeros_to8): truncation toward zero, clipped
 * to [-128,127].  Replaces dequant_interleaved_int4_to_int8 (kernels/csrc/pybind.cpp:23,
 * kernels/csrc/kairos_kernel/dequant_awq_format/dequant_i4_to_i8.cu:152-180). */
int kmi_cvt_i4_to_i8(void* out_i8, const void* qweight, const void* scales_to8, const void* scaled_zeros_to8,
                     int N, int K, int G, void* stream);

/* The same two conversions, written in the tiled layout the MFMA GEMMs copy straight into LDS:
 * [N/KMI_TILE_N][K/kb][KMI_TILE_N rows][64 bytes], kb = 32 (fp16) or 64 (int8); inside a tile row r
 * sits at r*64 and its four 16-byte chunks are XOR-swizzled: chunk c is stored at c ^ ((r>>2)&3).
 * No reference counterpart exists (the reference's permute_weight.cu is an uncompiled stub).
 * Needs N%KMI_TILE_N==0. */
#define KMI_TILE_N 128
int kmi_cvt_i4_to_f16_tiled(void* out_f16, const void* qweight, const void* scales, const void* scaled_zeros,
                            int N, int K, int G, void* stream);
int kmi_cvt_i4_to_i8_tiled(void* out_i8, const void* qweight, const void* scales_to8, const void* scaled_zeros_to8,
                           int N, int K, int G, void* stream);
/* Inverse of the tiled layout (row-major out), for round-trip checks: elem_size 1 or 2. */
int kmi_untile(void* out_rowmajor, const void* tiled, int N, int K, int elem_size, void* stream);

/* ---- per-token activation quantiser ---------------------------------------------------------- */

/* out_i8[m,k] = sat_s8(rint_half_even(float(x[m,k]) * (127.0f/amax_m))), scale[m] = fp16(amax_m/127.0f);
 * an all-zero token gives zeros and scale 0.  Replaces quant_fp16_to_int8 (kernels/csrc/pybind.cpp:18,
 * kernels/csrc/kairos_kernel/quant/quant_f16_to_i8.cu:86-104).  Needs K%8==0, K<=32768. */
int kmi_quant_act_i8(void* out_i8, void* scale_f16, const void* x_f16, int M, int K, void* stream);

/* Both preparation steps of the W8A8 lane in ONE launch: kmi_cvt_i4_to_i8 (tiled != 0: kmi_cvt_i4_to_i8_tiled)
 * into w8_out and kmi_quant_act_i8 of x into a8_out / ascale_f16.  The results are bit-identical to the two
 * separate calls; the shared launch saves a kernel boundary on every call that has to convert.  No reference
 * counterpart (the reference issues the two kernels one after the other, kairos/dynamic_linear.py:150-162).
 * Argument rules as for the two separate entry points. */
int kmi_prep_w8a8(void* w8_out, int tiled, const void* qweight, const void* scales_to8, const void* scaled_zeros_to8,
                  int N, int K, int G, void* a8_out, void* ascale_f16, const void* x_f16, int M, void* stream);

/* RMSNorm in front of a switched linear, emitting the activation format the consumer's lane needs from one read
 * of the hidden state ("activation matching", README.md:23-27; the reference vendors a fused norm + per-token
 * quantiser, thirdparty/AWQ/kernels/csrc/w8a8/layernorm.cu:51-231 `rms_norm_general`, which kairos/ never calls:
 * its modules run the eager norm and then quant_fp16_to_int8).  With h = x, or h = fp16(x + residual) when
 * residual_f16 is given (then also written to h_f16_out if that is not NULL):
 *   r = 1.0f / sqrtf(sum_k float(h[m,k])^2 / K + eps);  y[m,k] = fp16(float(gamma[k]) * float(fp16(float(h[m,k]) * r)))
 * which is the fp16 RMSNorm of the Llama / Qwen decoder modules with every intermediate rounded as there.
 * y_f16_out (may be NULL) receives y; a8_out / ascale_f16 (may both be NULL) receive kmi_quant_act_i8 of y, bit for
 * bit.  At least one output is required.  Needs K%8==0, K<=32768, eps>=0, 16-byte aligned tensors. */
int kmi_rmsnorm_quant_act(void* a8_out, void* ascale_f16, void* y_f16_out, void* h_f16_out, const void* x_f16,
                          const void* residual_f16, const void* gamma_f16, float eps, int M, int K, void* stream);

/* The operator in front of the down projection, in the format of its lane (same idea as kmi_rmsnorm_quant_act; the
 * reference runs the checkpoint's eager act_fn(gate) * up and quantises inside _forward, kairos/dynamic_linear.py:150-152).
 * gate_up_f16 [M, 2*I]: gate in columns 0..I-1, up in columns I..2I-1.  s = fp16(g / (1 + exp(-g))) evaluated in fp32
 * with the hardware exponential and reciprocal; y = fp16(float(s) * float(u)).  y_f16_out [M, I] (may be NULL) receives
 * y; a8_out [M, I] / ascale_f16 [M] (may both be NULL) receive kmi_quant_act_i8 of y, bit for bit.  s is within one
 * fp16 step of the correctly rounded SiLU (y within two).  Needs I%8==0, I<=32768, 16-byte aligned tensors. */
int kmi_silu_mul_quant_act(void* a8_out, void* ascale_f16, void* y_f16_out, const void* gate_up_f16, int M, int I,
                           void* stream);

/* ---- offline weight preparation ----------------------------------------------------------------- */

/* fp16 weight [N, K] (row-major) -> the resident format of one linear, in one launch:
 *   qweight [N/4, K] int16 (four-row interleave, 4 nibbles per word), scales / scaled_zeros [Gp, N] fp16 (W4A16
 *   lanes), scales_to8 / scaled_zeros_to8 [Gp, N] fp16 (int4 -> int8 conversion), scales_1 [N] fp16 (per channel),
 *   Gp = kmi_padded_groups(K, G); padded table rows are written as zeros.
 * Replaces the torch chain of DynamicLinear.from_module (kairos/dynamic_linear.py:86-115): quantize_tensor_int8
 * (kairos/quantization.py:112-141), kairos_quantize_tensor_int4 (kairos/dynamic_linear_v2.py:15-41), pack_int_awq
 * and trans_qfactor_layout_awq (thirdparty/AWQ/awq_method.py:5-75), with the same fp32 / fp16 operations in the
 * same order, so every output equals the host chain bit for bit.  Needs N%4==0, K%128==0, G==128; weights must be
 * finite. */
int kmi_prepare_weight(const void* w_f16, int N, int K, int G, void* qweight, void* scales, void* scaled_zeros,
                       void* scales_to8, void* scaled_zeros_to8, void* scales_1, void* stream);

/* Rows of the scale tables for in_features K: 8 * ceil((K/G) / 8) (calculate_zeros_width,
 * thirdparty/AWQ/awq_method.py:40-54).  Host only; negative error code for unsupported arguments. */
int kmi_padded_groups(int K, int G);

/* ---- re-pack for the version-2 W4A8 candidate --------------------------------------------------- */

/* Resident packed int4 [N/4, K] -> int8 [N, K/2] in the W4A8 operand layout (32x32 blocks of 512 bytes; byte
 * (n%8)*64 + ((k%16)/4)*16 + ((k%32)/16)*8 + ((n%16)/8)*4 + k%4 of block (n/32, k/32) holds row n in the low and
 * row n+16 in the high nibble).  Replaces trans_layout_c16_to_c8_awq (kernels/csrc/pybind.cpp:24,
 * kernels/csrc/kairos_kernel/trans_layout/trans_layout_marlin_c16_to_c8.cu:183-205); bit-exact contract
 * test/test_trans_layout.py:46-52.  Needs N%32==0, K%64==0. */
int kmi_trans_layout_w4a8(void* out_i8, const void* qweight, int N, int K, void* stream);

/* ---- W4A16, small M ---------------------------------------------------------------------------- */

/* out = x . dequant(qweight)^T (+bias), weights streamed once, fp32 accumulation on MFMA.
 * Replaces gemv_forward_cuda_new (thirdparty/AWQ/kernels/csrc/pybind.cpp:23,
 * thirdparty/AWQ/kernels/csrc/quantization_new/gemv/gemv_cuda.cu:245-463).
 * Needs 1<=M<=KMI_GEMV_MAX_M, G==128, N%16==0, K%128==0.
 * workspace (optional, NULL = none): caller-owned device scratch that lets long, narrow weights split K over
 * several workgroups per column strip.  Layout: the first KMI_GEMV_WS_HEADER bytes hold arrival counters, which must be
 * ZERO before the first call that uses the buffer and are zero again when every call's kernel has finished; fp32 partial
 * sums follow.  Calls that share a workspace must be ordered on one stream.  Results do not depend on which
 * workgroup finishes last (partial sums are added in split order); the split count depends on the arguments only. */
#define KMI_GEMV_WS_HEADER 65536
int kmi_gemv_w4a16(void* out_f16, const void* x_f16, const void* qweight, const void* scales,
                   const void* scaled_zeros, const void* bias, int M, int N, int K, int G,
                   void* workspace, size_t workspace_bytes, void* stream);

/* Tuning variant of the register form (a wave keeps the K groups of a trip in registers): nt = 16-column tiles per wave
 * (1..8), nw = waves per workgroup (4,8,16), ks = workgroups that share the K range of one column strip (1 = no split;
 * more needs a workspace of KMI_GEMV_WS_HEADER + ks*M*N*4 bytes); nt<=0 or nw<=0 selects the built-in choice of form
 * and split (what kmi_gemv_w4a16 runs).  No reference counterpart. */
int kmi_gemv_w4a16_cfg(void* out_f16, const void* x_f16, const void* qweight, const void* scales,
                       const void* scaled_zeros, const void* bias, int M, int N, int K, int G,
                       int nt, int nw, int ks, void* workspace, size_t workspace_bytes, void* stream);

/* Tuning variant of the ring form: every operand of a K group travels global -> LDS by direct-to-LDS buffer loads into
 * a per-wave ring of `depth` slots, so loads for later groups stay in flight while a group is multiplied.  nt as above,
 * nw = 1, 2, 4 or 8, ks as above, depth = slots per wave (<= 0: as deep as the wave's share of K, the wait counter and
 * LDS allow; larger values are reduced to that).  Same arithmetic and summation order as the register form with the
 * same (nt, nw, ks).  Needs 4-byte aligned tables and operands below 4 GiB.  No reference counterpart. */
int kmi_gemv_w4a16_ring_cfg(void* out_f16, const void* x_f16, const void* qweight, const void* scales,
                            const void* scaled_zeros, const void* bias, int M, int N, int K, int G,
                            int nt, int nw, int ks, int depth, void* workspace, size_t workspace_bytes, void* stream);

/* Host only: what kmi_gemv_w4a16 does for this shape with a workspace of that many bytes (0 = none).  *form: 0 register
 * form, 1 ring form; *nt, *nw, *ks as above; *depth: ring slots asked for (0 for the register form).  Any output pointer
 * may be NULL. */
int kmi_gemv_w4a16_plan(int M, int N, int K, size_t workspace_bytes, int* form, int* nt, int* nw, int* ks, int* depth);

/* Writes zeros over the arrival counters of a small-M workspace (its first KMI_GEMV_WS_HEADER bytes) with a small
 * kernel on `stream`.  Needed once before a buffer's first use unless it was allocated zeroed, and after any call on it
 * that did not run to completion (a launch error, an aborted stream): counters left non-zero would make later split
 * calls on that buffer add their partial sums at the wrong arrival.  A kernel, not a memset, so the call can be
 * captured into a graph.  No reference counterpart. */
int kmi_gemv_ws_reset(void* workspace, size_t workspace_bytes, void* stream);

/* ---- MFMA GEMMs, any M -------------------------------------------------------------------------
 *
 * Every GEMM entry point ends with (workspace, workspace_bytes, stream).  workspace is optional caller-owned device
 * scratch (16-byte aligned; NULL = none) for split-K: when the output tiles alone cannot fill the GPU (mid-sized M)
 * the call writes fp32 / int32 partial sums there and reduces them with a second kernel on the same stream, in a
 * fixed order (deterministic).  The library keeps no reference to it after the call's launches; calls that share
 * one buffer must be ordered on one stream.  The number of splits depends on the arguments only (shape, buffer
 * size; kmi_gemm_splits_for reports it), never on earlier calls or on the calling thread; the int8 lane's results
 * do not depend on it at all, the fp16 lanes' fp32 summation order does.  64 MiB covers every split the library
 * would choose for outputs up to 2 Mi elements. */

/* W4A16: replaces gemm_forward_cuda_new (thirdparty/AWQ/kernels/csrc/pybind.cpp:22,
 * thirdparty/AWQ/kernels/csrc/quantization_new/gemm/gemm_cuda.cu:1126-1235); the caller supplies out. */
int kmi_gemm_w4a16(void* out_f16, const void* x_f16, const void* qweight, const void* scales,
                   const void* scaled_zeros, const void* bias, int M, int N, int K, int G,
                   void* workspace, size_t workspace_bytes, void* stream);

/* W8A16: out = fp16((x . w8^T) * wscales[n]) (+bias).  The reference only declares the ids
 * (kairos/dynamic_linear.py:8-9). */
int kmi_gemm_w8a16(void* out_f16, const void* x_f16, const void* w8, const void* wscales_f16,
                   const void* bias, int M, int N, int K, void* workspace, size_t workspace_bytes, void* stream);

/* W8A8: acc = a8 . w8^T in int32; out = fp16(float(acc) * (float(wscales[n]) * float(ascales[m]))) (+bias).
 * Replaces w8a8_gemm_forward_cuda (thirdparty/AWQ/kernels/csrc/pybind.cpp:21,
 * thirdparty/AWQ/kernels/csrc/w8a8/w8a8_gemm_cuda.cu:909-954). */
int kmi_gemm_w8a8(void* out_f16, const void* a8, const void* w8, const void* wscales_f16,
                  const void* ascales_f16, const void* bias, int M, int N, int K,
                  void* workspace, size_t workspace_bytes, void* stream);

/* The same product with the raw int32 accumulators written out [M, N] (bit-exact tier). */
int kmi_gemm_w8a8_acc_i32(void* acc_i32, const void* a8, const void* w8, int M, int N, int K,
                          void* workspace, size_t workspace_bytes, void* stream);

/* W4A8: the W8A8 product computed from the resident packed int4 weight, with no converted copy:
 *   acc = a8 . W8^T,  W8[n,k] = (int8) fma_f16(q[n,k], scales_to8[k/G,n], scaled_zeros_to8[k/G,n])  (what kmi_cvt_i4_to_i8 writes),
 *   out = fp16(float(acc) * (float(wscales[n]) * float(ascales[m]))) (+bias),
 * so accumulators and outputs equal kmi_cvt_i4_to_i8 + kmi_gemm_w8a8 bit for bit.  It takes the place of the
 * version-2 candidate `w4a8_qserve` (kairos/dynamic_linear_v2.py:161-179: trans_layout_c16_to_c8_awq + a third-party
 * int4 x int8 GEMM with its own second-level quantiser): same operand precisions, weights decoded inside the GEMM.
 * kmi_gemm_w4a8_acc_i32 writes the raw int32 accumulators [M, N] (bit-exact tier).  kmi_gemm_w4a8_pick_tile: host-only,
 * the tile selector the call would use (128 = 128 x 128, 130 = 128 x 128 with two wave quartets per workgroup that
 * each take half of its K range (needs K % 256 == 0), 192 = 256 rows x 128 columns, 512 = 512 rows x 128 columns,
 * 256 = 256 x 256, 448 / 640 = 256 x 256 / 512 x 128 tiles in whole rounds over the CUs and the remaining columns as
 * 256 x 128 tiles in a second launch on the same stream);
 * kmi_gemm_force_tile accepts the same selectors for this lane. */
int kmi_gemm_w4a8(void* out_f16, const void* a8, const void* qweight, const void* scales_to8, const void* scaled_zeros_to8,
                  const void* wscales_f16, const void* ascales_f16, const void* bias, int M, int N, int K, int G,
                  void* workspace, size_t workspace_bytes, void* stream);
int kmi_gemm_w4a8_acc_i32(void* acc_i32, const void* a8, const void* qweight, const void* scales_to8,
                          const void* scaled_zeros_to8, int M, int N, int K, int G,
                          void* workspace, size_t workspace_bytes, void* stream);
int kmi_gemm_w4a8_pick_tile(int M, int N, int K);

/* W4A8 with INTEGER per-group factors, the arithmetic of the version-2 candidate itself (kairos/dynamic_linear_v2.py:161-179
 * -> qgemm_w4a8_per_group.gemm_forward_cuda, thirdparty/Qserve/qserve_kernels/csrc/qgemm/w4a8_per_group/gemm_cuda.cu:299-329,
 * 620-627), read from the resident packed int4 weight (no trans_layout_c16_to_c8_awq call in front):
 *   W8[n,k] = (int8)((q[n,k] * s2_scales[k/G,n] + s2_zeros[k/G,n]) mod 256),  acc = a8 . W8^T,
 *   out = fp16(float(acc) * (float(wscales[n]) * float(ascales[m]))) (+bias).
 * s2_scales / s2_zeros: int8 [K/G, N] in plain column order (the reference stores them shuffled inside blocks of 32 columns
 * for its tensor-core fragments, thirdparty/Qserve/w4a8_linear.py:215-262); s2_scales is read as an unsigned byte, s2_zeros
 * is the negated zero point times the scale as a two's-complement byte.  Every weight byte wraps on its own; the CUDA kernel
 * multiplies four packed bytes at once and agrees as long as 15 * scale < 256, which its quantiser guarantees.
 * Same tiles, workspace and selectors as kmi_gemm_w4a8. */
int kmi_gemm_w4a8_int(void* out_f16, const void* a8, const void* qweight, const void* s2_scales_i8, const void* s2_zeros_i8,
                      const void* wscales_f16, const void* ascales_f16, const void* bias, int M, int N, int K, int G,
                      void* workspace, size_t workspace_bytes, void* stream);
int kmi_gemm_w4a8_int_acc_i32(void* acc_i32, const void* a8, const void* qweight, const void* s2_scales_i8,
                              const void* s2_zeros_i8, int M, int N, int K, int G,
                              void* workspace, size_t workspace_bytes, void* stream);

/* FP16: out = x . w16^T (+bias), fp32 accumulation.  Replaces `input @ tmp_weight.T`
 * (kairos/dynamic_linear.py:163). */
int kmi_gemm_f16(void* out_f16, const void* x_f16, const void* w16, const void* bias,
                 int M, int N, int K, void* workspace, size_t workspace_bytes, void* stream);

/* Variants reading the weight operand in the tiled layout written by kmi_cvt_*_tiled. */
int kmi_gemm_w8a8_tiled(void* out_f16, const void* a8, const void* w8_tiled, const void* wscales_f16,
                        const void* ascales_f16, const void* bias, int M, int N, int K,
                        void* workspace, size_t workspace_bytes, void* stream);
int kmi_gemm_f16_tiled(void* out_f16, const void* x_f16, const void* w16_tiled, const void* bias,
                       int M, int N, int K, void* workspace, size_t workspace_bytes, void* stream);

/* kmi_gemm_w4a16 for callers that cannot allocate device memory (code under HIP graph capture, tight serving loops,
 * harnesses that forbid hipMalloc): no counterpart in the reference.  Same kernels, same results, but the split-K
 * partial sums go to a 16 MiB array that is part of the library's code object (one copy per GPU, held until the
 * process ends) instead of a caller-owned workspace; the call allocates and frees nothing.  Limits: M*N <=
 * KMI_NOALLOC_MAX_OUTPUTS (KMI_E_M_RANGE beyond); the stream must belong to the current device; the first call on a
 * device looks the array's address up and must not run inside a graph capture.  Every call on a GPU shares that GPU's
 * array: calls that overlap on one GPU (different streams, or replays of graphs that contain one) race on it.
 * Nothing needs clearing between calls (every partial sum that is read was written by the same call). */
#define KMI_NOALLOC_MAX_OUTPUTS (512 * 1024)
#define KMI_NOALLOC_MAX_DEVICES 64
int kmi_gemm_w4a16_noalloc(void* out_f16, const void* x_f16, const void* qweight, const void* scales,
                           const void* scaled_zeros, const void* bias, int M, int N, int K, int G, void* stream);

/* Host-only queries of the automatic choices (no GPU work).
 * kmi_gemm_pick_tile: the workgroup tile (64, 128 or 256 rows; 192 = 256 rows x 128 columns; 320 = 256 rows x 192
 *   columns, used with tiled weights only -- row-major operands run 256 x 256 instead) of the W8A8 lane for an
 *   M x N x K product.  With the 256 tile the library may run the columns of a thin last round of tiles with the 128
 *   tile in a second launch on the same stream (same results).
 * kmi_gemm_w4a16_wp_rows: rows per tile (32, 64, 128) of the small-M variant kmi_gemm_w4a16 uses (weights decoded in
 *   registers by the wave that owns their columns), or 0 when the LDS-staged variant runs.
 * kmi_gemm_splits_for: K splits a call would use with a workspace of that many bytes (1 = none); lane 0 = W4A16,
 *   1 = W8A16, 2 = W8A8, 3 = fp16. */
int kmi_gemm_pick_tile(int M, int N, int K);
int kmi_gemm_w4a16_wp_rows(int M, int N, int K);
int kmi_gemm_splits_for(int lane, int M, int N, int K, size_t workspace_bytes);

/* TEST AND TUNING HOOKS (state of the calling host thread, 0 = automatic; production callers never set them).
 * kmi_gemm_force_tile: 64, 128, 256, or 192 (W8A8 and fp16 operand-copy lanes only: 256 rows x 128 columns, two
 *   workgroups per CU); for kmi_gemm_w4a16 also 1032 / 1064 / 1128 (small-M variant, two wave quartets per
 *   workgroup) and 2032 / 2064 / 2128 (one).
 * kmi_gemm_force_splits: the number of K splits (needs a workspace in the call).
 * kmi_gemm_force_group_m: tile rows per group of the workgroup -> tile order of the GEMM kernels (every XCD takes a
 *   contiguous run of a sequence that walks the tiles column-major in groups of that many tile rows; default 8); it
 *   changes which tiles share an XCD's L2, never a result. */
void kmi_gemm_force_tile(int tile);
void kmi_gemm_force_splits(int splits);
void kmi_gemm_force_group_m(int group_m);

/* ---- interval lookup table (host only) --------------------------------------------------------- */

/* Replaces LUT_module.LUT (kernels/csrc/kairos_kernel/lut/lut.h:8-45, lut_bindings.cpp:5-13).
 * record(r, c): append a segment with inclusive right edge r; get(m): c of the first segment with
 * m <= r, the last segment's c beyond the last edge.  A one-entry memo makes repeated queries O(1);
 * like the reference's, a table is not safe for concurrent use from several threads. */
void* kmi_lut_new(void);
void kmi_lut_free(void* lut);
int kmi_lut_record(void* lut, int right_edge, int comp_type);
int kmi_lut_get(void* lut, int m);   /* comp_type, or KMI_E_HANDLE for a NULL/empty table */
int kmi_lut_shrink_to_fit(void* lut);
int kmi_lut_size(void* lut);

/* ---- measurement probes ------------------------------------------------------------------------- */

/* Kernels that only read, for the floors the streaming kernels are measured against; no product path calls them and
 * nothing in the reference corresponds to them.  kmi_probe_empty: one empty launch of 256 workgroups.
 * kmi_probe_stream_read: a plain reader of `bytes` bytes, 16 contiguous KiB per workgroup.  kmi_probe_gemv_read: exactly
 * the weight loads of kmi_gemv_w4a16's register form with nt column tiles per wave and nw waves per workgroup
 * (kmi_gemv_w4a16_plan reports what a call uses), no activations, tables, arithmetic or stores. */
int kmi_probe_empty(void* stream);
int kmi_probe_stream_read(const void* buf, size_t bytes, void* stream);
int kmi_probe_gemv_read(const void* qweight, int N, int K, int nt, int nw, void* stream);

/* Register-only probes of the matrix and vector pipes (no counterpart in the reference either).
 * kmi_probe_mfma_stream: `workgroups` x 4 waves each issue iters x 16 independent MFMAs (kind 0: v_mfma_i32_32x32x32_i8,
 * 1: v_mfma_f32_32x32x16_f16) on the 32 KiB of operands at `operands` (device; their bit pattern decides the power drawn);
 * clocks_u64x2 (device) receives the shader cycles and the ticks of the constant 100 MHz counter around the loop of
 * workgroup 0, so cycles / ticks * 100 is the shader clock in MHz under that load.
 * kmi_probe_pipe_overlap: one workgroup of eight waves (two per SIMD), 2048 int8 MFMAs and / or 16384 vector instructions
 * per wave; cycles_u64x8 (device) receives each wave's cycles.  mode 1: waves 0-3 MFMAs only; 2: waves 4-7 vector
 * instructions only; 3: both; 4..8: waves 0-3 with 0, 4, 8, 12, 16 vector instructions behind every MFMA; 9: all waves
 * vector only; 10: waves 0-3 MFMA + 16, waves 4-7 MFMAs only; 11: all waves MFMA + 8; 12: all waves MFMAs only. */
int kmi_probe_mfma_stream(int kind, const void* operands, size_t operand_bytes, int workgroups, int iters,
                          void* clocks_u64x2, void* stream);
int kmi_probe_pipe_overlap(int mode, void* cycles_u64x8, void* stream);

/* ---- bounded conversion buffer (host only) ------------------------------------------------------ */

/* The lanes that convert on demand (W8A8, fp16, W8A16) write the converted weight into a temporary buffer; the
 * reference allocates `torch.empty(self.shape)` per call and leaves the bound to the caching allocator
 * (kairos/dynamic_linear.py:145,159).  A binder without such an allocator keeps ONE device buffer, sized for the largest
 * converted weight of its model, and lets this handle do the bookkeeping: nothing here allocates or touches device
 * memory.  kmi_cache_create wraps the caller's buffer (NULL on error).  kmi_cache_acquire(owner, format, nbytes): owner =
 * any id unique to the layer, format = caller-defined (e.g. 1 int8 row-major, 2 int8 tiled, 3 fp16 row-major, 4 fp16
 * tiled); returns 1 if the buffer already holds exactly that copy (skip the conversion), 0 if not (convert into
 * *out_ptr now; the handle records the new content), KMI_E_SHAPE if nbytes exceeds the buffer -- the bound holds.
 * kmi_cache_invalidate forgets the content (the buffer was used for something else, or the weights changed).  Use one
 * handle per stream of execution; a hit is valid only for work ordered after the conversion that filled the buffer. */
void* kmi_cache_create(void* device_buffer, size_t capacity_bytes);
void kmi_cache_destroy(void* cache);
int kmi_cache_acquire(void* cache, uint64_t owner, int format, size_t nbytes, void** out_ptr);
int kmi_cache_invalidate(void* cache);
int kmi_cache_stats(void* cache, size_t* capacity, size_t* high_water, uint64_t* hits, uint64_t* misses);

#ifdef __cplusplus
}
#endif
#endif /* KAIROS_MI_H */
