/*
 * fpq.h — C ABI of libfpq_hip.so, the MI355X (gfx950) engine behind FP-Quant's inference path.
 *
 * Every entry point takes raw device pointers, sizes and a HIP stream (passed as void*, 0 = the
 * null stream), launches asynchronously on that stream and returns an int status:
 *   0  success;  <0  invalid argument (FPQ_E_*);  >0  a hipError_t reported by the runtime.
 * No entry point allocates device memory, and all of them may be called from any host thread.
 * Scalars the reference passes as one-element tensors (alpha, global scale) stay device pointers
 * so no host sync is introduced.  Two pieces of per-device state exist, both set up by
 * fpq_prepare_device (or by the first call that needs them):
 *   - a 128 KB lookup table of bf16 silu values used by fpq_silu_mul_quantize_*: the first such
 *     call on a device fills it on the caller's stream and WAITS for that stream once; if that
 *     first call is being captured into a graph, the fill is recorded into the capture and
 *     repeated by every later first call until one runs outside a capture;
 *   - the device address of the scratch array of fpq_gemm_mxf4_packed_noalloc.
 * Apart from that no entry point synchronises a stream or keeps mutable global state.
 *
 * Each declaration cites the reference interface it stands in for (paths relative to the
 * reference checkout, inference_lib/src/fp_quant/module/).
 */
#ifndef FPQ_H_
#define FPQ_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define FPQ_VERSION 1

/* status codes */
#define FPQ_OK 0
#define FPQ_E_NULL -1        /* a required pointer is null                       */
#define FPQ_E_SHAPE -2       /* sizes violate the divisibility rules below       */
#define FPQ_E_ROTATION -3    /* unknown rotation kind / unsupported block size   */
#define FPQ_E_ALIGN -4       /* a pointer is not aligned as documented           */
#define FPQ_E_POLICY -5      /* unknown zero-nibble policy or scale layout       */
#define FPQ_E_UNSUPPORTED -6 /* valid request this build has no kernel for       */
#define FPQ_E_LIMIT -7       /* a size is beyond the entry point's stated maximum */

/* rotation kinds: how the [g, g] matrix of the reference (linear.py:24-41) is applied */
#define FPQ_ROT_HADAMARD 0 /* +-norm Sylvester matrix: fp32 radix-2 butterflies, strides 1..g/2 */
#define FPQ_ROT_IDENTITY 1 /* no rotation                                                      */
#define FPQ_ROT_GSR 2      /* Hadamard with sequency-ordered columns (outputs permuted)         */
#define FPQ_ROT_GENERAL 3  /* arbitrary bf16 matrix, sequential fp32 fma accumulation           */

/* zero-nibble policies: which code a value that rounds to zero gets */
#define FPQ_ZERO_REFERENCE 0 /* always 0x8, what src/quantization/quant_ops.py:31-40 packs */
#define FPQ_ZERO_SIGNED 1    /* sign bit of the scaled value (+0 -> 0x0, -0 -> 0x8)         */

int fpq_version(void);

/* Static, NUL-terminated description of a status returned by this library. */
const char* fpq_status_string(int status);

/* 1 if `device` is a gfx950 GPU this library has code for, 0 if not, <0 / >0 on error. */
int fpq_device_supported(int device);

/* Compute units of the current device (256 on an MI355X; 256 also where no device answers).  The GEMM
 * entry points choose their kernels by problem size relative to this number. */
int fpq_compute_units(void);

/*
 * Sets up the per-device state described at the top for the current device, on `stream`, and waits
 * for it: call it once per device before capturing graphs or entering a loop that must not block.
 * Returns FPQ_E_UNSUPPORTED if `stream` is being captured.  Idempotent and cheap after the first call.
 */
int fpq_prepare_device(void* stream);

/*
 * *id = 0 if `stream` is not being captured into a graph, else a value unique to the capture in
 * progress.  Host code that keeps results of one call for the next (activations quantized once for
 * several layers) uses it to reuse them only within the same capture, or only outside any: work
 * recorded during a capture has not run when the capture ends.
 */
int fpq_stream_capture_id(void* stream, unsigned long long* id);

/*
 * Fused rotate + MXFP4 abs-max quantize.
 * Stands in for qutlass.fusedQuantizeMx behind fused_quantize_mx_op (qutlass_ops.py:36-71,
 * called from forward_quantize, linear_fns.py:34-41) with method "abs_max".
 *
 *   x            bf16 [rows, cols] row-major, 16-byte aligned; cols % max(g, 32) == 0
 *   rot_kind/g   rotation kind and block size (g in 16/32/64/128; identity ignores g)
 *   norm         value every Hadamard entry has in magnitude (float(H[0][0]))
 *   h            bf16 [g, g] matrix, only read for FPQ_ROT_GENERAL (may be null otherwise)
 *   codes        uint8 [rows, cols/2], 4-byte aligned: element 2j in the low nibble of byte j
 *   scales       uint8 E8M0 [scale_rows, scale_stride]; entry [r, c/32]; rows >= `rows` and
 *                columns >= cols/32 are zero-filled (the reference pads to 128 rows / 4 columns)
 *   zero_policy  FPQ_ZERO_*
 */
int fpq_quantize_mx(const void* x, int64_t rows, int64_t cols, int rot_kind, int g, float norm,
                    const void* h, void* codes, void* scales, int64_t scale_rows,
                    int64_t scale_stride, int zero_policy, void* stream);

/*
 * fpq_quantize_mx with the reference's "quest" scale rule instead of abs-max
 * (method="quest" of qutlass.fusedQuantizeMx, qutlass_ops.py:36-71; arithmetic as stated by
 * module/triton/mxfp4.py:51-59 with the constant of pseudoquant_linear_fns.py:20-22):
 *   s = 2^floor(log2(fl32(2.92247856/6) * std + 1e-8)),  std = population standard deviation of the
 *   32 rotated values (fp32; sums per octet left to right, octets combined (o0+o1)+(o2+o3),
 *   variance clamped at 0);  codes = E2M1 RNE of x/s saturated at +-6;  stored byte = e8m0(s).
 *   mask  uint8 [rows, cols/8] or null: bit (c % 8) of byte [r, c/8] is 1 where |x/s| < 6
 *         (mxfp4.py:105-110; bit order of linear_fns.py:67-76).
 * Global scale for this method is 1.0 (linear.py:190-192).
 */
int fpq_quantize_mx_quest(const void* x, int64_t rows, int64_t cols, int rot_kind, int g, float norm,
                          const void* h, void* codes, void* scales, int64_t scale_rows,
                          int64_t scale_stride, void* mask, int zero_policy, void* stream);
/*
 * fpq_quantize_mx_quest (without a mask) writing the packed operand layout directly, as
 * fpq_quantize_mx_packed does for the abs-max rule: same codes and scale bytes, re-tiled; same
 * conditions (cols % 256 == 0; Hadamard 16..128, identity, sequency-ordered Hadamard up to 64 wide;
 * other rotations return FPQ_E_UNSUPPORTED).
 */
int fpq_quantize_mx_quest_packed(const void* x, int64_t rows, int64_t cols, int rot_kind, int g, float norm,
                                 void* packed_codes, void* packed_scales, int zero_policy, void* stream);

/*
 * Fused rotate + NVFP4 quantize (group 16, E4M3 scales, fp32 per-tensor multiplier).
 * Stands in for qutlass.fusedQuantizeNv behind fused_quantize_nv_op (qutlass_ops.py:74-105).
 *   global_scale  device pointer to one fp32 (the reference passes a 1-element tensor)
 *   scales        uint8 E4M3 [scale_rows, scale_stride]; entry [r, c/16]; cols % max(g,16) == 0
 */
int fpq_quantize_nv(const void* x, int64_t rows, int64_t cols, int rot_kind, int g, float norm,
                    const void* h, const float* global_scale, void* codes, void* scales,
                    int64_t scale_rows, int64_t scale_stride, int zero_policy, void* stream);

/*
 * y[m, n] = bf16(alpha * sum_k dq(xq)[m, k] * dq(wq)[n, k]) (+ bias[n]), MXFP4 operands.
 * Stands in for qutlass.matmul_mxf4_bf16_tn behind matmul_mxf4_bf16_tn_op and the disabled
 * small-M matmul_ada_mxf4_bf16_tn_op (qutlass_ops.py:111-146), plus the bias add of
 * FPQuant4x16NoMasterFn.forward (linear_fns.py:512-514).  Scales are taken row-major (the
 * reference re-tiles them with to_blocked on every call; this engine needs no re-tiling).
 *   xq uint8 [M, K/2], wq uint8 [N, K/2] (16-byte aligned rows: K % 32 == 0)
 *   xs uint8 E8M0 [>=M, xs_stride], ws uint8 E8M0 [>=N, ws_stride], entry [row, k/32]
 *   alpha device pointer to one fp32; bias bf16 [N] or null; y bf16 [M, N], 16-byte aligned
 */
int fpq_gemm_mxf4(const void* xq, const void* xs, int64_t xs_stride, const void* wq,
                  const void* ws, int64_t ws_stride, const float* alpha, const void* bias,
                  void* y, int64_t M, int64_t N, int64_t K, void* stream);

/*
 * Same contract with NVFP4 operands: E4M3 scales per 16 elements, entry [row, k/16].
 * Stands in for qutlass.matmul_nvf4_bf16_tn behind matmul_nvf4_bf16_tn_op (qutlass_ops.py:149-168).
 */
int fpq_gemm_nvf4(const void* xq, const void* xs, int64_t xs_stride, const void* wq,
                  const void* ws, int64_t ws_stride, const float* alpha, const void* bias,
                  void* y, int64_t M, int64_t N, int64_t K, void* stream);

/*
 * Packed MXFP4 operands: the codes and scales of a [rows, K] operand re-tiled into the order the
 * 32x32x64 block-scaled matrix instruction consumes them, so that one operand of one instruction
 * is one contiguous kilobyte (K % 256 == 0; rows padded to a multiple of 32 with zero codes):
 *   codes   block (rt, ks) = rows [32 rt, +32) x K [64 ks, +64) at byte (rt * K/64 + ks) * 1024;
 *           16 bytes at (32 kh + r) * 16 inside it = row 32 rt + r, K [64 ks + 32 kh, +32)
 *   scales  block (rt, kb) = the same rows x K [256 kb, +256) at byte (rt * K/256 + kb) * 256;
 *           byte q of the dword at (32 kh + r) * 4 = E8M0 scale of row 32 rt + r, group 8 kb + 2 q + kh
 * This is the counterpart of the scale re-tiling the reference performs with to_blocked() before
 * every CUTLASS GEMM (qutlass_ops.py:111-146), extended to the codes; it is done once per weight.
 * fpq_packed_*_bytes return the buffer sizes; fpq_pack_mxf4 converts from the row-major layout of
 * fpq_quantize_mx (codes 16-byte aligned; packed buffers 16-byte aligned).
 */
int64_t fpq_packed_codes_bytes(int64_t rows, int64_t K);
int64_t fpq_packed_scales_bytes(int64_t rows, int64_t K);
int fpq_pack_mxf4(const void* codes, const void* scales, int64_t scale_stride, int64_t rows,
                  int64_t K, void* packed_codes, void* packed_scales, void* stream);
/*
 * The inverse of fpq_pack_mxf4 for the first `rows` rows: row-major codes [rows, K/2] (16-byte aligned)
 * and E8M0 scales (entry [row, k/32], row stride scale_stride >= K/32; only those entries are written)
 * from a packed operand.  A layer that holds its weights in the packed layout only uses it to hand
 * the reference's `qweight` / `scales` tensors (linear.py:87-88) to state_dict().
 */
int fpq_unpack_mxf4(const void* packed_codes, const void* packed_scales, int64_t rows, int64_t K,
                    void* codes, void* scales, int64_t scale_stride, void* stream);

/*
 * fpq_quantize_mx writing the packed layout directly (same codes and scale bytes; rows past
 * `rows` in the last 32-row tile get zero codes and zero scale bytes).  cols % 256 == 0;
 * Hadamard 16..128, identity and sequency-ordered Hadamard up to 64 wide; other rotations return
 * FPQ_E_UNSUPPORTED (quantize row-major and call fpq_pack_mxf4).  Same reference counterpart as
 * fpq_quantize_mx (qutlass_ops.py:36-71).
 */
int fpq_quantize_mx_packed(const void* x, int64_t rows, int64_t cols, int rot_kind, int g, float norm,
                           void* packed_codes, void* packed_scales, int zero_policy, void* stream);

/*
 * fpq_gemm_mxf4 on packed operands (same arithmetic, bit-identical y): the kernel for large M.
 * Stands in for qutlass.matmul_mxf4_bf16_tn (qutlass_ops.py:111-128) like fpq_gemm_mxf4.
 */
int fpq_gemm_mxf4_packed(const void* xq_packed, const void* xs_packed, const void* wq_packed,
                         const void* ws_packed, const float* alpha, const void* bias, void* y,
                         int64_t M, int64_t N, int64_t K, void* stream);

/*
 * Quantizers fused with the elementwise producer of their input, so that the bf16 tensor between
 * the two never travels through memory.  The reference's Llama blocks quantize exactly these
 * tensors: act_fn(gate) * up before down_proj (src/utils/llama_utils.py:60-71) and the RMSNorm
 * output before q/k/v and gate/up; each stands in for that elementwise sequence followed by
 * qutlass.fusedQuantizeMx / fusedQuantizeNv (qutlass_ops.py:36-105).  Every PyTorch operator of
 * the unfused sequence rounds to bf16 once, and so do these, in IEEE fp32 with a fixed operation
 * order (no fused multiply-add, exp as a fixed polynomial), so codes and scales are bit-identical
 * to quantizing the bf16 tensor the stated formula gives:
 *   rmsnorm   v[r, c] = bf16(weight[c] * bf16(x[r, c] * inv_rms[r]))
 *   silu_mul  v[r, c] = bf16(bf16(g / (1 + exp(-g))) * up[r, c]),  g = gate[r, c]
 * x / gate / up are bf16 with row strides ld* (elements, multiples of 8, >= cols); `normed` /
 * `product` is null or a bf16 [rows, cols] buffer that receives v; codes, scales, rot_kind, g,
 * norm, zero_policy and global_scale as for fpq_quantize_mx / fpq_quantize_nv.  Hadamard
 * (16..128) and identity rotations; others return FPQ_E_UNSUPPORTED.
 *
 * fpq_row_inv_rms: inv_rms[r] = 1 / sqrt(sum_c x[r, c]^2 / cols + eps), fp32, with the summation
 * order: squares of 8 consecutive elements left to right, octet k into accumulator k % 64 in
 * increasing k, accumulators combined by the butterfly a[i] += a[i ^ m], m = 1, 2, ..., 32.
 */
int fpq_row_inv_rms(const void* x, int64_t ld, int64_t rows, int64_t cols, float eps, float* inv_rms,
                    void* stream);
int fpq_rmsnorm_quantize_mx(const void* x, int64_t ld, const float* inv_rms, const void* weight,
                            int64_t rows, int64_t cols, int rot_kind, int g, float norm, void* normed,
                            void* codes, void* scales, int64_t scale_rows, int64_t scale_stride,
                            int zero_policy, void* stream);
int fpq_rmsnorm_quantize_nv(const void* x, int64_t ld, const float* inv_rms, const void* weight,
                            int64_t rows, int64_t cols, int rot_kind, int g, float norm,
                            const float* global_scale, void* normed, void* codes, void* scales,
                            int64_t scale_rows, int64_t scale_stride, int zero_policy, void* stream);
int fpq_silu_mul_quantize_mx(const void* gate, int64_t ld_gate, const void* up, int64_t ld_up,
                             int64_t rows, int64_t cols, int rot_kind, int g, float norm, void* product,
                             void* codes, void* scales, int64_t scale_rows, int64_t scale_stride,
                             int zero_policy, void* stream);
int fpq_silu_mul_quantize_nv(const void* gate, int64_t ld_gate, const void* up, int64_t ld_up,
                             int64_t rows, int64_t cols, int rot_kind, int g, float norm,
                             const float* global_scale, void* product, void* codes, void* scales,
                             int64_t scale_rows, int64_t scale_stride, int zero_policy, void* stream);
/* The MXFP4 ones writing the packed operand layout (as fpq_quantize_mx_packed; cols % 256 == 0). */
int fpq_rmsnorm_quantize_mx_packed(const void* x, int64_t ld, const float* inv_rms, const void* weight,
                                   int64_t rows, int64_t cols, int rot_kind, int g, float norm,
                                   void* normed, void* packed_codes, void* packed_scales, int zero_policy,
                                   void* stream);
/*
 * fpq_row_inv_rms followed by fpq_rmsnorm_quantize_mx_packed in ONE launch, for the few rows of a decode
 * step: same bits (the row statistic keeps its summation order), one kernel instead of two.
 *   rows      at most fpq_rmsnorm_rows_max_rows() (64); cols % 256 == 0, cols <= 16384; FPQ_E_LIMIT beyond
 *   inv_rms   null, or fp32 [rows] that receives the row statistic
 *   normed    null, or bf16 [rows, cols] that receives weight * (x / rms)
 * Hadamard 16..128 and identity rotations; others return FPQ_E_UNSUPPORTED.  No counterpart in the reference,
 * which normalises with PyTorch's RMSNorm module and then quantizes (llama_utils.py:132-160).
 */
int64_t fpq_rmsnorm_rows_max_rows(void);
int fpq_rmsnorm_rows_quantize_mx_packed(const void* x, int64_t ld, const void* weight, int64_t rows,
                                        int64_t cols, float eps, int rot_kind, int g, float norm,
                                        float* inv_rms, void* normed, void* packed_codes,
                                        void* packed_scales, int zero_policy, void* stream);
int fpq_rmsnorm_rows_quantize_nv_packed(const void* x, int64_t ld, const void* weight, int64_t rows,
                                        int64_t cols, float eps, int rot_kind, int g, float norm,
                                        const float* global_scale, float* inv_rms, void* normed,
                                        void* packed_codes, void* packed_scales, int zero_policy, void* stream);
/*
 * The NVFP4 fused producers writing the packed operand layout of fpq_gemm_nvf4_packed (cols % 256 == 0, as for
 * fpq_quantize_nv_packed).  Arguments as fpq_rmsnorm_quantize_nv / fpq_silu_mul_quantize_nv.
 */
int fpq_rmsnorm_quantize_nv_packed(const void* x, int64_t ld, const float* inv_rms, const void* weight,
                                   int64_t rows, int64_t cols, int rot_kind, int g, float norm,
                                   const float* global_scale, void* normed, void* packed_codes,
                                   void* packed_scales, int zero_policy, void* stream);
int fpq_silu_mul_quantize_nv_packed(const void* gate, int64_t ld_gate, const void* up, int64_t ld_up,
                                    int64_t rows, int64_t cols, int rot_kind, int g, float norm,
                                    const float* global_scale, void* product, void* packed_codes,
                                    void* packed_scales, int zero_policy, void* stream);
int fpq_silu_mul_quantize_mx_packed(const void* gate, int64_t ld_gate, const void* up, int64_t ld_up,
                                    int64_t rows, int64_t cols, int rot_kind, int g, float norm,
                                    void* product, void* packed_codes, void* packed_scales, int zero_policy,
                                    void* stream);

/*
 * *amax = max(*amax, max |rotate(x)|) as fp32, with the rotation of the quantize entry points
 * (rot_kind, g, norm, h as there; cols % g == 0).  The NVFP4 per-tensor multiplier the reference's
 * exporter tracks is 448 * 6 / this maximum, minimised over calls
 * (src/quantization/quantizer.py:145-150); the caller zeroes *amax before the first call and may
 * keep folding further tensors (calibration batches, fused q/k/v weights) into it.
 */
int fpq_rotated_absmax(const void* x, int64_t rows, int64_t cols, int rot_kind, int g, float norm,
                       const void* h, float* amax, void* stream);

/*
 * fpq_gemm_mxf4_packed followed by the addition of a bf16 [M, N] tensor in the same kernel:
 *   y = bf16(bf16(alpha * acc (+ bias)) + residual)   -- the rounding of a separate bf16 add.
 * For the output projections of a decoder block, whose result the reference's models add to the
 * residual stream right away (src/utils/llama_utils.py:60-71 computes the projection, the block
 * adds).  `residual` may be `y` itself (every element is read before it is written).
 */
int fpq_gemm_mxf4_packed_residual(const void* xq_packed, const void* xs_packed, const void* wq_packed,
                                  const void* ws_packed, const float* alpha, const void* bias,
                                  const void* residual, void* y, int64_t M, int64_t N, int64_t K,
                                  void* stream);

/*
 * fpq_gemm_mxf4_packed (with `residual` non-null: fpq_gemm_mxf4_packed_residual) that may split K
 * across workgroups.  With at most 128 activation rows the time is one pass over the weights, and a
 * shape with few weight rows or a long K fills the chip only if several workgroups share one output
 * tile: each stores its fp32 partial tile into `workspace`, and the last one to arrive (a counter
 * per tile) adds the partials of all parts in part order, so the result is deterministic.  It is
 * the counterpart of the small-M entry the reference keeps disabled (matmul_ada_mxf4_bf16_tn_op,
 * qutlass_ops.py:133-146; linear_fns.py:55).
 *   workspace        null (K stays whole) or a 256-byte aligned device buffer whose first 16384 bytes
 *                    are zero before the first call; every call leaves them zero again.  Calls that
 *                    share a workspace must not overlap (same stream, or ordered by events).
 *   workspace_bytes  its size; fpq_gemm_mxf4_packed_workspace_bytes(M, N, K) is what the shape can
 *                    use (0: it never splits).  A smaller buffer means fewer parts, not an error.
 * Larger M runs the tile kernels of fpq_gemm_mxf4_packed and ignores the workspace.
 */
int64_t fpq_gemm_mxf4_packed_workspace_bytes(int64_t M, int64_t N, int64_t K);
int fpq_gemm_mxf4_packed_splitk(const void* xq_packed, const void* xs_packed, const void* wq_packed,
                                const void* ws_packed, const float* alpha, const void* bias,
                                const void* residual, void* y, int64_t M, int64_t N, int64_t K,
                                void* workspace, int64_t workspace_bytes, void* stream);
/* The same for packed NVFP4 operands (fpq_gemm_nvf4_packed, with `residual` non-null fpq_gemm_nvf4_packed_residual);
 * workspace as above, sized by fpq_gemm_nvf4_packed_workspace_bytes(M, N, K).  Up to 128 rows the split is
 * that of the MXFP4 entry; 129-256 rows on few weight rows (129-192 where the tile kernels can halve K inside
 * their workgroups, below) run as two passes over at most 128 rows each, and each pass may use the workspace.  Beyond, where the tile kernels have at most one workgroup tile per CU, a
 * K with an even number of 256-blocks is halved INSIDE the workgroups (eight waves, the halves meet in LDS:
 * no workspace, the size function returns 0); with an odd number and a long K the tile kernels split K across
 * workgroups the way the weight-streaming kernel does (fp32 parts of their workgroup tiles, a counter per tile,
 * parts added in part order) -- the NVFP4 loop is bound by its in-register dequantization, so more waves pay
 * there (MXFP4 measured slower with either and never does). */
int64_t fpq_gemm_nvf4_packed_workspace_bytes(int64_t M, int64_t N, int64_t K);
int fpq_gemm_nvf4_packed_splitk(const void* xq_packed, const void* xs_packed, const void* wq_packed,
                                const void* ws_packed, const float* alpha, const void* bias,
                                const void* residual, void* y, int64_t M, int64_t N, int64_t K,
                                void* workspace, int64_t workspace_bytes, void* stream);

/*
 * One GEMM for several layers that read the same activations (the q, k and v projections of an
 * attention block, the gate and up projections of a gated MLP): the layers' packed weights lie end
 * to end in wq_packed / ws_packed (a packed operand is a sequence of 32-row tiles, so the packed
 * form of the row-wise concatenation of weights whose row counts are multiples of 32 is the
 * concatenation of their packed forms), and layer i's result goes to its own dense matrix
 * ys[i] of shape [M, ns[i]].  The reference launches one GEMM per layer (FPQuantLinear.forward,
 * linear.py:250-368, once per nn.Linear it replaced); the values are the same, column by column.
 *   count   1 .. 4 layers
 *   ns[i]   layer i's output features, a positive multiple of 256
 *   ys[i]   16-byte aligned device pointers to bf16 [M, ns[i]]
 *   bias    null or bf16 [sum ns], the layers' biases end to end
 * Status codes as fpq_gemm_mxf4_packed; FPQ_E_SHAPE also for a count or an ns[i] outside the above.
 */
int fpq_gemm_mxf4_packed_multi(const void* xq_packed, const void* xs_packed, const void* wq_packed,
                               const void* ws_packed, const float* alpha, const void* bias,
                               void* const* ys, const int64_t* ns, int64_t count, int64_t M, int64_t K,
                               void* stream);
/* The same for packed NVFP4 operands (fpq_gemm_nvf4_packed). */
int fpq_gemm_nvf4_packed_multi(const void* xq_packed, const void* xs_packed, const void* wq_packed,
                               const void* ws_packed, const float* alpha, const void* bias,
                               void* const* ys, const int64_t* ns, int64_t count, int64_t M, int64_t K,
                               void* stream);

/*
 * fpq_gemm_mxf4_packed_splitk for callers that cannot allocate or hold a workspace (code recorded
 * into a HIP graph, tight serving loops, harnesses that forbid hipMalloc): the counters and partial
 * tiles of a split K live in a file-scope device array of the library (4 210 688 bytes per GPU, held
 * until the process ends) instead of a caller-provided buffer.  It has no counterpart in the
 * reference.  Same arguments, results and status codes as fpq_gemm_mxf4_packed_splitk called with a
 * workspace of that size, with these limits:
 *   M <= fpq_gemm_mxf4_packed_noalloc_max_rows() (128), the weight-streaming regime; more rows
 *   return FPQ_E_LIMIT (the tile kernels of fpq_gemm_mxf4_packed use no scratch memory at all);
 *   K is split into at most as many parts as the array holds partial tiles for (on a device of 256
 *   compute units that is every split fpq_gemm_mxf4_packed_splitk would make).
 * The call makes no hipMalloc/hipFree and launches the same kernels.  All calls on one GPU share
 * that GPU's array: calls that may overlap on one GPU (different streams without an ordering
 * event) race on it and must use fpq_gemm_mxf4_packed_splitk with their own workspaces.  The
 * counters start at zero (static storage) and every call leaves them at zero.
 */
int64_t fpq_gemm_mxf4_packed_noalloc_max_rows(void);
int fpq_gemm_mxf4_packed_noalloc(const void* xq_packed, const void* xs_packed, const void* wq_packed,
                                 const void* ws_packed, const float* alpha, const void* bias,
                                 const void* residual, void* y, int64_t M, int64_t N, int64_t K,
                                 void* stream);

/*
 * Test hook: copies the first `bytes` (at most 16384) of the current device's scratch array -- the split-K
 * counters of fpq_gemm_mxf4_packed_noalloc -- to `out` (device memory) in stream order.  They read zero
 * between calls.
 */
int fpq_test_noalloc_counters(void* out, int64_t bytes, void* stream);

/*
 * Test hook: E2M1 codes of n fp32 values exactly as the quantize kernels round them
 * (out[i] in 0..15, one byte per value).  Used to check the device rounding exhaustively.
 */
int fpq_test_e2m1(const float* in, uint8_t* out, int64_t n, int zero_policy, void* stream);

/*
 * NVFP4 on the packed layout: codes exactly as for MXFP4; scales in blocks (rt, kb) of 512 bytes at
 * byte (rt * K/256 + kb) * 512, the 8 bytes at (32 kh + r) * 8 being, for K step q = 0..3 of the
 * block, the two E4M3 bytes of row 32 rt + r, groups 16 kb + 4 q + 2 kh and + 1 (bytes 2q, 2q + 1).
 * fpq_pack_nvf4 converts from the row-major layout of fpq_quantize_nv; fpq_gemm_nvf4_packed is
 * fpq_gemm_nvf4 on packed operands (same arithmetic: exact fp16 dequantization, fp32 accumulation in
 * another K order).  Stands in for qutlass.matmul_nvf4_bf16_tn (qutlass_ops.py:149-168).
 */
int64_t fpq_packed_scales_bytes_nv(int64_t rows, int64_t K);
int fpq_pack_nvf4(const void* codes, const void* scales, int64_t scale_stride, int64_t rows,
                  int64_t K, void* packed_codes, void* packed_scales, void* stream);
/* The inverse of fpq_pack_nvf4 for the first `rows` rows (E4M3 scales, entry [row, k/16], scale_stride >= K/16). */
int fpq_unpack_nvf4(const void* packed_codes, const void* packed_scales, int64_t rows, int64_t K,
                    void* codes, void* scales, int64_t scale_stride, void* stream);
int fpq_gemm_nvf4_packed(const void* xq_packed, const void* xs_packed, const void* wq_packed,
                         const void* ws_packed, const float* alpha, const void* bias, void* y,
                         int64_t M, int64_t N, int64_t K, void* stream);
/* fpq_gemm_nvf4_packed with the residual addition of fpq_gemm_mxf4_packed_residual (same rounding, `residual` may be `y`). */
int fpq_gemm_nvf4_packed_residual(const void* xq_packed, const void* xs_packed, const void* wq_packed,
                                  const void* ws_packed, const float* alpha, const void* bias,
                                  const void* residual, void* y, int64_t M, int64_t N, int64_t K,
                                  void* stream);
/*
 * fpq_quantize_nv writing the packed layout directly (same codes and scale bytes; rows past `rows`
 * in the last 32-row tile get zero codes and zero scale bytes).  cols % 256 == 0; rotations as for
 * fpq_quantize_mx_packed, others return FPQ_E_UNSUPPORTED (quantize row-major, then fpq_pack_nvf4).
 * Same reference counterpart as fpq_quantize_nv (qutlass_ops.py:74-105).
 */
int fpq_quantize_nv_packed(const void* x, int64_t rows, int64_t cols, int rot_kind, int g, float norm,
                           const float* global_scale, void* packed_codes, void* packed_scales,
                           int zero_policy, void* stream);

/*
 * Measurement hook: `blocks` workgroups of four waves run `iters` x 16 FP4 32x32x64 block-scaled
 * matrix instructions per wave on register-resident operands (words: blocks*256*32 ints of operand
 * bits; sink: blocks*256 floats; clocks: per workgroup the elapsed shader-clock cycles and 100 MHz
 * ticks).  It gives the matrix throughput and clock this chip sustains for given operand bits with
 * no memory system involved: the practical ceiling a GEMM is compared with next to the nominal
 * peak.  No counterpart in the reference.
 */
int fpq_test_mfma_rate(const int* words, int blocks, int iters, float* sink, unsigned long long* clocks,
                       void* stream);

#ifdef __cplusplus
}
#endif
#endif /* FPQ_H_ */
