/*
 * snnf.h - C ABI of libsnnf: fused temporal spiking-network operators for AMD MI355X (gfx950).
 *
 * One entry point per kernel family of pengjh0111/triton-snn-fusion's Triton layer. Each entry point replaces the
 * Python launcher (and the Triton kernel behind it) that the reference's runtime/triton_*_backend.py modules call;
 * the citation above every declaration names that launcher (paths are relative to the reference checkout).
 *
 * Conventions shared by every entry point
 *   - All pointers are DEVICE pointers of the current HIP device unless the parameter is documented as a host array.
 *   - `xs` / `residuals` are HOST arrays of T device pointers, one per timestep. A packed [T, ...] tensor is passed as
 *     base + t * step_stride. Timesteps may alias (the same analog frame repeated T times is detected and computed once).
 *   - Layouts are the reference's: activations contiguous NCHW per timestep, conv weight OIHW, linear weight [Fout, Fin].
 *   - dtype codes: SNNF_F32 / SNNF_BF16 / SNNF_F16. Spikes are written as 0/1 in the activation dtype `x_dtype`.
 *     The membrane potential is held in fp32 on chip for the whole time loop of a launch; `v_dtype` is only its dtype
 *     in memory (v_init / v_out). A call with more timesteps than one launch takes (16 for the scan, depthwise, linear,
 *     pointwise and time-outer kernels; 1 to 4 for the matrix kernels, reported as `window` / `launches` by
 *     snnf_conv_last_plan) hands the membrane from launch to launch through `v_out`, so a 16-bit `v_dtype` is rounded at
 *     each hand-over: callers that want one rounding after the last step, as the reference's kernels do, pass an fp32
 *     membrane for such calls and round it themselves (the operator layer above this ABI does).
 *   - `v_init == NULL` means a zero initial membrane (the reference's 0-dim v_init). `v_out` may alias `v_init`.
 *   - LIF update per step (runtime/snn_custom_ops.py:384-409):
 *         h = v + x            if tau <= 1        else   h = v + (x - v) / tau
 *         s = (h >= v_threshold)
 *         v = h - s * v_threshold   if v_reset < 0   else   v = s ? v_reset : h
 *   - `stream` is a hipStream_t (NULL = the default stream). Calls only enqueue work: they never synchronise and never
 *     free memory; none allocates device memory (scratch, where needed, is a caller-provided workspace).
 *   - Return value: SNNF_OK (0) or a negative snnf_status; snnf_status_string() names it and snnf_last_error()
 *     returns a thread-local detail message for the most recent failure.
 */
#ifndef SNNF_H_
#define SNNF_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define SNNF_MAX_T_PER_LAUNCH 16

typedef enum snnf_dtype {
    SNNF_F32 = 0,
    SNNF_BF16 = 1,
    SNNF_F16 = 2
} snnf_dtype;

/* Activation layouts. NCHW is the layout of the reference's operators and of every entry point that takes no layout
 * argument. C8 and BITS are internal layouts for tensors that travel between consecutive fused operators of one
 * network without being seen by anyone else (the `*_blocked` entry points); no operator of the reference has them.
 *   C8   : [N, ceil(C / 8), H, W, 8] elements of the activation dtype (16 bytes per pixel and group of 8 channels);
 *          channels beyond C hold zeros.
 *   BITS : [N, ceil(C / 8), H, W] bytes; bit j of a byte is the spike of channel 8 * c8 + j; bits beyond C are zero. */
typedef enum snnf_layout {
    SNNF_LAYOUT_NCHW = 0,
    SNNF_LAYOUT_C8 = 1,
    SNNF_LAYOUT_BITS = 2
} snnf_layout;

typedef enum snnf_status {
    SNNF_OK = 0,
    SNNF_ERR_INVALID_ARGUMENT = -1, /* null pointer, non-positive extent, unknown dtype code */
    SNNF_ERR_UNSUPPORTED = -2,      /* well-formed request outside what the kernels implement */
    SNNF_ERR_LAUNCH = -3,           /* hipLaunchKernel / runtime error; see snnf_last_error() */
    SNNF_ERR_WORKSPACE = -4         /* workspace pointer missing or too small */
} snnf_status;

/* Library identification; no counterpart in the reference. */
int snnf_abi_version(void);
const char* snnf_status_string(int status);
const char* snnf_last_error(void);

/*
 * Temporal LIF scan over T steps of `numel` elements.
 * Replaces run_fused_temporal_lif_state_kernel (kernels/generated_temporal_lif_kernel.py:98-164) as called by
 * run_triton_fused_temporal_lif_state (runtime/triton_temporal_lif_backend.py:57-117).
 *   spikes : [T, numel] in x_dtype, timestep stride `spike_step_stride` elements.
 *   v_out  : [numel] in v_dtype.
 */
int snnf_lif_scan(const void* const* xs, int T, int64_t numel, int x_dtype,
                  const void* v_init, int v_dtype,
                  void* spikes, int64_t spike_step_stride, void* v_out,
                  float v_threshold, float v_reset, float tau, void* stream);

/*
 * Depthwise 3x3 convolution (padding 1, stride 1 or 2) + bias (+ residual) + LIF over T steps.
 * Replaces run_fused_temporal_general[_residual][_autotuned] with kernel keys depthwise_k3_s1_p1 / depthwise_k3_s2_p1
 * (kernels/benchmark_conv_lif_temporal_general.py:971-1323, emitter :713-817) as called from
 * runtime/triton_convlif_backend.py:513-598 and :689-817.
 *   xs[t]        : [N, C, H, W] x_dtype          weight : [C, 1, 3, 3] w_dtype        bias : [C] w_dtype
 *   residuals[t] : [N, C, Ho, Wo] x_dtype or residuals == NULL
 *   spikes       : [T, N, C, Ho, Wo] x_dtype (timestep stride `spike_step_stride` elements), v_out : [N, C, Ho, Wo] v_dtype
 */
int snnf_dwconv3x3_lif(const void* const* xs, const void* const* residuals, int T,
                       int N, int C, int H, int W, int stride, int x_dtype,
                       const void* weight, const void* bias, int w_dtype,
                       const void* v_init, int v_dtype,
                       void* spikes, int64_t spike_step_stride, void* v_out,
                       float v_threshold, float v_reset, float tau, void* stream);

/*
 * The same operator (stride 1, bf16 / fp16 activations, W % 8 == 0, fp32 membrane) with a bit-packed spike output: one
 * byte holds the spikes of 8 consecutive pixels of a row (bit j = pixel 8 x + j), 16 times fewer bytes than the dense
 * 0 / 1 elements the reference's kernel stores (kernels/benchmark_conv_lif_temporal_general.py:707-708, depthwise
 * emitter :713-817). Activations, residuals and membranes must be 16-byte aligned.
 *   xs[t]      : x_packed == 0: [N, C, H, W] x_dtype; x_packed != 0: [N, C, H, W / 8] bytes packed the same way (the
 *                output of this entry point or of snnf_pwconv_lif_rowbits; x_dtype then names the weight / operand dtype)
 *   spike_bits : [T, N, C, H, W / 8] bytes, `bits_step_stride` BYTES between timesteps
 *   v_init     : [N, C, H, W] fp32 or NULL (zeros);  v_out : the same or NULL (final membrane not stored; needs
 *                T <= SNNF_MAX_T_PER_LAUNCH)
 * snnf_rowbits_unpack turns `bytes` such bytes into 8 * bytes dense 0 / 1 elements of x_dtype (16-byte aligned);
 * snnf_rowbits_pack is its inverse (bit j = element j != 0), for a network's first packed operator.
 */
int snnf_dwconv3x3_lif_rowbits(const void* const* xs, const void* const* residuals, int T,
                               int N, int C, int H, int W, int x_dtype, int x_packed,
                               const void* weight, const void* bias, const void* v_init,
                               void* spike_bits, int64_t bits_step_stride, void* v_out,
                               float v_threshold, float v_reset, float tau, void* stream);
int snnf_rowbits_unpack(const void* bits, void* dense, int64_t bytes, int x_dtype, void* stream);
int snnf_rowbits_pack(const void* dense, void* bits, int64_t bytes, int x_dtype, void* stream);

/*
 * Pointwise (1x1, stride 1) convolution + bias + LIF over T steps whose input spikes are row-packed as above: the
 * consumer of snnf_dwconv3x3_lif_rowbits in a depthwise-separable block (the reference hands the depthwise layer's
 * dense 0 / 1 tensor to run_fused_temporal_general with kernel key k1_s1_p0,
 * kernels/benchmark_conv_lif_temporal_general.py:971-1323 as called from runtime/triton_convlif_backend.py:513-598).
 * Same packed weight, arithmetic and outputs as snnf_conv_lif on the unpacked tensor.
 *   xs_bits[t] : [N, Cin, H, W / 8] bytes;  v_init (or NULL), v_out : [N, Cout, H, W] fp32
 *   spikes     : spikes_packed == 0: [T, N, Cout, H, W] x_dtype (bf16 / fp16), `spike_step_stride` elements between timesteps;
 *                spikes_packed != 0: [T, N, Cout, H, W / 8] bytes, `spike_step_stride` BYTES between timesteps, and v_out may be
 *                NULL (final membrane not stored; needs T <= SNNF_MAX_T_PER_LAUNCH)
 * Takes what the pointwise kernel's fast variant takes: the common neuron (tau a power of two above 1, hard reset), Cin % 8 == 0,
 * Cout % 32 == 0, H * W % 64 == 0, 16-byte aligned outputs and membranes; SNNF_ERR_UNSUPPORTED otherwise.
 */
int snnf_pwconv_lif_rowbits(const void* const* xs_bits, int T, int N, int Cin, int H, int W, int x_dtype,
                            const void* packed_weight, int Cout, const void* v_init,
                            void* spikes, int spikes_packed, int64_t spike_step_stride, void* v_out,
                            float v_threshold, float v_reset, float tau, void* stream);

/*
 * LIF -> global average pool -> Linear, summed over T.
 *   out_sum[n, k] = sum_t ( fc_weight[k, :] . mean_hw(s_t[n, :, :, :]) + fc_bias[k] )
 * Replaces run_fused_temporal_lif_avgpool_linear_kernel (kernels/generated_temporal_lif_avgpool_linear_kernel.py:120-209)
 * as called by run_triton_fused_temporal_lif_avgpool_linear (runtime/triton_temporal_lif_avgpool_linear_backend.py:58-108).
 *   xs[t] : [N, C, H, W] x_dtype     fc_weight : [K, C] w_dtype     fc_bias : [K] w_dtype or NULL
 *   out_sum : [N, K] x_dtype         v_out : [N, C, H, W] v_dtype
 *   workspace : at least snnf_lif_pool_linear_workspace_bytes(N, C) bytes of device memory, 16-byte aligned;
 *               it holds per-(n, c) spike counts between the two launches and needs no initialisation.
 * Tails as small as those at the end of a network (T * C * H * W of one sample at most 32 Ki, C % 8 == 0 and at most 2048,
 * C * H * W % 8 == 0, 16-byte aligned operands) run as ONE launch: a workgroup owns a sample and a range of classes, counts the
 * sample's spikes per channel in LDS and multiplies its weight rows with them; the workspace is then not touched.
 * snnf_lif_pool_linear_launches() says which of the two forms a shape takes (1 or 2; 0 for invalid extents), assuming
 * aligned operands.
 */
size_t snnf_lif_pool_linear_workspace_bytes(int N, int C);
int snnf_lif_pool_linear_launches(int T, int N, int C, int H, int W, int K);
int snnf_lif_pool_linear(const void* const* xs, int T, int N, int C, int H, int W, int x_dtype,
                         const void* v_init, int v_dtype,
                         const void* fc_weight, const void* fc_bias, int K, int w_dtype,
                         void* out_sum, void* v_out,
                         void* workspace, size_t workspace_bytes,
                         float v_threshold, float v_reset, float tau, void* stream);

/*
 * snnf_lif_pool_linear without a workspace argument and without any allocation, for callers that cannot allocate device
 * memory (code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc). It has no counterpart in
 * the reference. The per-(n, c) spike counts between the two launches live in a static device array of the library
 * (SNNF_LIF_POOL_LINEAR_STATIC_MAX_PLANES ints = 1 MiB per GPU the library runs on, held until the process ends);
 * N * C beyond that returns SNNF_ERR_WORKSPACE. Arguments, kernels and results are those of snnf_lif_pool_linear.
 * All calls on one GPU share the array: calls that overlap on one GPU (different streams) race; calls on one stream
 * are ordered and safe. The array's address is looked up on the first call on a device (not a stream operation; make
 * that first call outside a graph capture).
 */
#define SNNF_LIF_POOL_LINEAR_STATIC_MAX_PLANES (256 * 1024)
int snnf_lif_pool_linear_static(const void* const* xs, int T, int N, int C, int H, int W, int x_dtype,
                                const void* v_init, int v_dtype,
                                const void* fc_weight, const void* fc_bias, int K, int w_dtype,
                                void* out_sum, void* v_out,
                                float v_threshold, float v_reset, float tau, void* stream);

/*
 * Temporal Linear + LIF: for each t, s_t, v = LIF(x_t . W^T + b, v).
 * Replaces run_fused_temporal_linear_lif_state_kernel (kernels/generated_temporal_linear_lif_kernel.py:205-363) as
 * called by runtime/triton_temporal_linear_lif_backend.py:185-274.
 *   xs[t] : [M, Fin] x_dtype (row stride `x_row_stride` elements)   weight : [Fout, Fin] w_dtype   bias : [Fout] w_dtype or NULL
 *   spikes : [T, M, Fout] x_dtype (timestep stride `spike_step_stride` elements)   v_out : [M, Fout] v_dtype
 * fp32 operands enter the matrix cores as two bf16 terms each (three of the four products, fp32 accumulate: about 16 mantissa
 * bits; the reference multiplies fp32 tensors in TF32, kernels/generated_temporal_linear_lif_kernel.py:142,155-158); fp16
 * operands use the fp16 matrix path.
 */
int snnf_linear_lif(const void* const* xs, int T, int M, int Fin, int64_t x_row_stride, int x_dtype,
                    const void* weight, const void* bias, int Fout, int w_dtype,
                    const void* v_init, int v_dtype,
                    void* spikes, int64_t spike_step_stride, void* v_out,
                    float v_threshold, float v_reset, float tau, void* stream);

/*
 * The same operator with a caller-owned workspace, which lets the library split the K dimension of a tile over
 * several workgroups (partial sums in the workspace, added in the order of their K ranges by the workgroup that
 * finishes last: results do not depend on scheduling and equal those of snnf_linear_lif up to the order of the fp32
 * additions). Layers with few output tiles or a long Fin are bound by memory latency without it. The reference has no
 * counterpart (its Triton kernel, kernels/generated_temporal_linear_lif_kernel.py:138-182, walks K inside one program).
 *   snnf_linear_lif_workspace_bytes : bytes that let this shape split as far as it pays (0: the shape does not split).
 *   workspace : NULL (then this is snnf_linear_lif), or `workspace_bytes` of device memory, 256-byte aligned, whose first
 *               64 KiB were zero before the first call that used it; every call leaves them zero again. A smaller
 *               workspace than asked for splits less. Calls that share a workspace must not overlap in time.
 */
size_t snnf_linear_lif_workspace_bytes(int T, int M, int Fin, int Fout);
int snnf_linear_lif_ws(const void* const* xs, int T, int M, int Fin, int64_t x_row_stride, int x_dtype,
                       const void* weight, const void* bias, int Fout, int w_dtype,
                       const void* v_init, int v_dtype,
                       void* spikes, int64_t spike_step_stride, void* v_out,
                       float v_threshold, float v_reset, float tau,
                       void* workspace, size_t workspace_bytes, void* stream);

/*
 * Dense (groups == 1) convolution + bias (+ residual) + LIF over T steps as an implicit GEMM on the matrix cores.
 * Replaces run_fused_temporal_general[_residual][_autotuned] with kernel keys k1_s1_p0, k3_s1_p1, k3_s2_p1, k5_s1_p2,
 * k7_s2_p3, k11_s4_p2 (kernels/benchmark_conv_lif_temporal_general.py:971-1323, emitter :561-710) as called from
 * runtime/triton_convlif_backend.py:331-817. Any square-or-not kernel size, stride and padding is accepted as long as
 * dilation is 1.
 *
 * Two steps: (1) snnf_conv_pack_weight rewrites the OIHW weight (+ bias) into the matrix-core operand order once per
 * weight tensor and activation dtype; (2) snnf_conv_lif consumes the packed weight on every call. The packed buffer is
 * opaque; its size is snnf_conv_packed_weight_bytes(). fp32 activations / weights enter the matrix cores as two bf16 terms each
 * (the value rounded to bf16 and the rounded remainder; three of the four products are accumulated in fp32, the fourth is
 * below 2^-16 of the result): the reference multiplies fp32 tensors in TF32 (kernels/benchmark_conv_lif_temporal_general.py:
 * 673-674), this keeps about 16 mantissa bits. The depthwise kernel multiplies fp32 tensors in fp32. fp16 activations use the
 * fp16 matrix path, bf16 ones the bf16 path.
 *   xs[t]        : [N, Cin, H, W] x_dtype
 *   residuals[t] : [N, Cout, Ho, Wo] x_dtype or residuals == NULL
 *   spikes       : [T, N, Cout, Ho, Wo] x_dtype (timestep stride `spike_step_stride` elements); v_out : [N, Cout, Ho, Wo] v_dtype
 */
size_t snnf_conv_packed_weight_bytes(int Cout, int Cin, int KH, int KW, int x_dtype);
int snnf_conv_pack_weight(const void* weight, const void* bias /* nullable */, int w_dtype,
                          int Cout, int Cin, int KH, int KW, int x_dtype,
                          void* packed, size_t packed_bytes, void* stream);
int snnf_conv_lif(const void* const* xs, const void* const* residuals, int T,
                  int N, int Cin, int H, int W, int x_dtype,
                  const void* packed_weight, int Cout, int KH, int KW,
                  int stride_h, int stride_w, int pad_h, int pad_w,
                  const void* v_init, int v_dtype,
                  void* spikes, int64_t spike_step_stride, void* v_out,
                  float v_threshold, float v_reset, float tau, void* stream);

/* Convolution + bias (+ residual) WITHOUT a neuron: out[t] = conv2d(xs[t]) + b (+ residuals[t]) in the activation dtype,
 * for T independent frames, with the same packed weight and matrix kernel as snnf_conv_lif. No fused operator of the
 * reference corresponds to it: its rewrite leaves LIF-free Conv+BN nodes (the 1x1 downsample shortcuts of a ResNet,
 * whose output is the `residuals` operand of fused_temporal_conv_add_lif_state, runtime/snn_custom_ops.py:491-518) to
 * the framework's convolution; this entry point keeps such a layer on the NCHW tensors the fused operators exchange.
 * Supported: Cin % 8 == 0 or Cin < 8 (a plain 1x1 stride-1 layer runs with each image as one row of pixels);
 * SNNF_ERR_UNSUPPORTED otherwise.
 *   out : [T, N, Cout, Ho, Wo] x_dtype (frame stride `out_step_stride` elements) */
int snnf_conv_bias(const void* const* xs, const void* const* residuals /* nullable */, int T,
                   int N, int Cin, int H, int W, int x_dtype,
                   const void* packed_weight, int Cout, int KH, int KW,
                   int stride_h, int stride_w, int pad_h, int pad_w,
                   void* out, int64_t out_step_stride, void* stream);

/* 2-D pooling of `planes` independent H x W planes (NCHW with planes = N * C, or T * N * C for a spike sequence):
 * max 3x3 stride 2, max 2x2 stride 2 (padding <= kernel / 2, padded positions never win) and average 2x2 stride 2
 * (no padding), floor output size. No fused operator of the reference corresponds to it: pooling layers stay ordinary
 * framework calls between its fused operators (e.g. the stem's max pool and the 2x2 pools of the VGG / ResNet models in
 * benchmarks/validate_chronos_baselines.py:748-790); this is the same layer for hosts that drive libsnnf directly.
 *   x : [planes, H, W] x_dtype;  y : [planes, Ho, Wo] x_dtype */
int snnf_pool2d(const void* x, void* y, int64_t planes, int H, int W, int kernel, int stride, int pad, int is_max,
                int x_dtype, void* stream);

/*
 * Internal activation layouts between consecutive fused operators (see snnf_layout). The reference stores every spike as
 * a dense 0/1 element of the activation dtype (kernels/benchmark_conv_lif_temporal_general.py:707-708) and copies the T
 * inputs of a layer into one stack (runtime/triton_convlif_backend.py:579); its executor's fast path hands pooled
 * caller-owned buffers to the `_packed_out` operator (runtime/fx_standalone_executor.py:900-952). The entry points below
 * are this library's counterpart of that producer-consumer plumbing: a network executor keeps spikes at one bit each
 * (16 times fewer bytes than bf16) and analog activations channel-blocked, in matrix-operand order.
 *
 * snnf_layout_bytes: bytes of `frames` frames of [C, H, W] in a layout (0 for invalid arguments).
 * snnf_layout_convert: frames of [C, H, W] from one layout to another (any pair). Values written to BITS are
 *   (element != 0); elements read from BITS are 0 / 1 in the activation dtype.
 * snnf_pool2d_blocked: 2-D pooling of frames in C8 or BITS: max k x k / stride s / padding p (k in {2, 3}, s = 2) and
 *   average 2 x 2 / 2. BITS -> BITS for max (a bitwise OR), BITS -> C8 for average (quarters are exact in 16 bits),
 *   C8 -> C8 for both; SNNF_ERR_UNSUPPORTED otherwise. Same window rules as snnf_pool2d.
 */
size_t snnf_layout_bytes(int layout, int64_t frames, int C, int H, int W, int x_dtype);
int snnf_layout_convert(const void* src, int src_layout, void* dst, int dst_layout, int64_t frames, int C, int H, int W,
                        int x_dtype, void* stream);
int snnf_pool2d_blocked(const void* x, int x_layout, void* y, int y_layout, int64_t frames, int C, int H, int W,
                        int kernel, int stride, int pad, int is_max, int x_dtype, void* stream);

/*
 * snnf_conv_lif / snnf_conv_bias on the internal layouts: dense convolution + bias (+ residual) (+ LIF) over T steps
 * with inputs in C8 or BITS, the residual in any layout, the output in any layout (BITS only with a neuron). Same
 * operator semantics, packed weight (snnf_conv_pack_weight for the same activation dtype) and LIF rule as
 * snnf_conv_lif, which replaces run_fused_temporal_general[_residual][_autotuned]
 * (kernels/benchmark_conv_lif_temporal_general.py:971-1323) as called from runtime/triton_convlif_backend.py:513-817.
 *   xs[t]        : N frames [Cin, H, W] in `x_layout` (C8, 16-byte aligned, or BITS); all T pointers equal = one frame
 *                  shared by every timestep (convolved once)
 *   residuals[t] : N frames [Cout, Ho, Wo] in `res_layout`, or residuals == NULL
 *   x_dtype      : SNNF_BF16 or SNNF_F16 (dtype of C8 / NCHW elements and of the matrix operands)
 *   out          : T x N frames [Cout, Ho, Wo] in `out_layout`, `out_step_stride` BYTES between timesteps
 *   v_init       : [N, Cout, Ho, Wo] fp32 NCHW or NULL (zeros);  v_out : the same or NULL (final membrane not stored;
 *                  only allowed when all T timesteps fit one window: T <= 4, or a shared frame)
 *   neuron       : 1 = LIF and spikes; 0 = write conv + bias (+ residual) itself (out_layout C8 or NCHW), v_* ignored
 * T <= SNNF_MAX_T_PER_LAUNCH, Cin and Cout arbitrary (groups of 8 are padded with zeros), dilation 1.
 */
int snnf_conv_lif_blocked(const void* const* xs, int x_layout, const void* const* residuals, int res_layout, int T,
                          int N, int Cin, int H, int W, int x_dtype,
                          const void* packed_weight, int Cout, int KH, int KW,
                          int stride_h, int stride_w, int pad_h, int pad_w,
                          const void* v_init, void* out, int out_layout, int64_t out_step_stride, void* v_out,
                          int neuron, float v_threshold, float v_reset, float tau, void* stream);

/*
 * The second convolution of a residual block together with the block's projection shortcut: out = LIF(conv(xs) + bias +
 * conv1x1(shortcut_xs) + shortcut bias), the shortcut's products accumulated as further K steps of the same output
 * tile. The reference runs the shortcut as a convolution of its own and adds its output through the residual operand of
 * run_fused_temporal_general_residual (kernels/benchmark_conv_lif_temporal_general.py:1097-1323, as called from
 * runtime/triton_convlif_backend.py:689-817); here the shortcut's output never exists in memory (and is not rounded to the
 * activation dtype on the way), and one launch replaces two.
 *   xs[t]          : N frames [Cin, H, W] in BITS; the main convolution is KH x KW, stride 1, padding (KH-1)/2 x (KW-1)/2
 *   shortcut_xs[t] : N frames [shortcut_Cin, shortcut_H, shortcut_W] in BITS, convolved 1 x 1 with the given strides and
 *                    no padding; its output plane must be the main one: (shortcut_H - 1) / shortcut_stride_h + 1 == H
 *   packed_weight, shortcut_packed_weight : snnf_conv_pack_weight of [Cout, Cin, KH, KW] and [Cout, shortcut_Cin, 1, 1]
 *                    (each with its own bias) for `x_dtype`
 *   out, v_init, v_out, neuron, out_layout, out_step_stride : as in snnf_conv_lif_blocked
 * Cin and shortcut_Cin multiples of 16, 3 <= T <= SNNF_MAX_T_PER_LAUNCH, distinct inputs per timestep;
 * SNNF_ERR_UNSUPPORTED ("unsupported_shortcut: ...") otherwise: the caller then runs the two convolutions apart.
 */
int snnf_conv_lif_blocked_shortcut(const void* const* xs, const void* const* shortcut_xs, int T, int N, int Cin, int H, int W,
                                   int x_dtype, const void* packed_weight, int Cout, int KH, int KW, int pad_h, int pad_w,
                                   int shortcut_Cin, int shortcut_H, int shortcut_W, int shortcut_stride_h,
                                   int shortcut_stride_w, const void* shortcut_packed_weight,
                                   const void* v_init, void* out, int out_layout, int64_t out_step_stride, void* v_out,
                                   int neuron, float v_threshold, float v_reset, float tau, void* stream);

/*
 * Convolution + bias + LIF followed by a 2 x 2 / stride 2 average pool of the spikes, in one launch: the four lanes that
 * hold a pooling window add their spikes in registers and the kernel writes the quarters (0, 1/4, ..., 1: exact in 16 bits)
 * channel-blocked at half the plane; the spikes themselves are never stored. The reference runs the pool as a layer of its
 * own between two fused operators (its rewrites replace Conv-BN-LIF chains only, compiler/fx_lif_temporal_rewrite.py:
 * 2037-2113, and leave pooling modules in the graph); results are those of snnf_conv_lif_blocked followed by
 * snnf_pool2d_blocked: bit for bit where both launches share K among waves in the same way, to the summation order
 * otherwise (this form plans patches of even extents, which can change that partition).
 *   xs, x_layout, packed_weight, geometry, LIF parameters : as in snnf_conv_lif_blocked (no residual, zero initial membrane)
 *   out   : T x N frames [Cout, Ho / 2, Wo / 2] in C8, `out_step_stride` BYTES between timesteps
 *   v_out : [N, Cout, Ho, Wo] fp32 NCHW (the membrane of the unpooled neurons) or NULL
 * T == 4 (distinct inputs, or one shared frame), Ho and Wo even, Cout a multiple of 8, tau == 2 with v_reset == 0;
 * SNNF_ERR_UNSUPPORTED ("unsupported_pool: ...") otherwise: the caller then runs the pool as a launch of its own.
 */
int snnf_conv_lif_blocked_avgpool(const void* const* xs, int x_layout, int T, int N, int Cin, int H, int W, int x_dtype,
                                  const void* packed_weight, int Cout, int KH, int KW,
                                  int stride_h, int stride_w, int pad_h, int pad_w,
                                  void* out, int64_t out_step_stride, void* v_out,
                                  float v_threshold, float v_reset, float tau, void* stream);

/*
 * Global average pool and classifier on bit-packed spikes, summed over T and scaled:
 *   out[n, k] = out_scale * sum_t ( fc_weight[k, :] . mean_hw(s_t[n, :, :, :]) + fc_bias[k] )
 * The network's last neuron then fires inside the convolution in front of it (snnf_conv_lif_blocked with a bit-packed
 * output) instead of inside snnf_lif_pool_linear, and this entry point is what remains of the tail: the pooling and the
 * classifier that the reference keeps as nn.AdaptiveAvgPool2d / nn.Linear modules behind its last fused convolution
 * when the convolution patterns have claimed that neuron (the tail pattern only sees the neurons they left over:
 * `excluded_lif_nodes`, compiler/fx_lif_temporal_rewrite.py:791-799), and the mean over the timesteps of its loop
 * wrapper (out_scale = 1 / T). One launch: a workgroup per sample and class range.
 *   spikes[t] : N frames [C, H, W] in BITS     fc_weight : [K, C], fc_bias : [K] or NULL, out : [N, K], all w_dtype
 * C a multiple of 8 and at most 2048, w_dtype SNNF_BF16 or SNNF_F16, T <= SNNF_MAX_T_PER_LAUNCH.
 */
int snnf_spike_pool_linear(const void* const* spikes, int T, int N, int C, int H, int W, const void* fc_weight,
                           const void* fc_bias, int K, int w_dtype, void* out, float out_scale, void* stream);

/*
 * Temporal Linear + LIF on the internal layouts: the operator of snnf_linear_lif_ws with its spikes leaving as bits and its
 * activation rows arriving as 16-bit elements or as bits, for a network executor that owns both tensors. Its use: a
 * convolution + LIF on a plane of a few pixels (the last stage of a VGG on 32 x 32 inputs works on 2 x 2 planes) is a
 * matrix product of a sample's whole frame, [Cin x H x W] -> [Cout x H x W], with a weight matrix that holds every tap at
 * the pair of pixels it connects and no padding; with the frame's features in the order (channel / 8, pixel, channel % 8)
 * a C8 frame is such a row of elements, a BITS frame such a row of bits, and the spike bits written here are a BITS frame.
 * Same launcher as snnf_linear_lif (kernels/generated_temporal_linear_lif_kernel.py:205-363); the reference runs such a
 * layer through its convolution kernel (kernels/benchmark_conv_lif_temporal_general.py:629-676) and has no counterpart.
 *   xs[t]     : [M, Fin] elements of `dtype`, row stride `x_row_stride` elements (x_bits == 0), or [M, Fin / 8] bytes, bit j
 *               of byte b = feature 8 b + j, row stride `x_row_stride` bytes (x_bits != 0)
 *   weight    : [Fout, Fin] `dtype`, bias : [Fout] `dtype` or NULL     v_init : [M, Fout] fp32 or NULL (zero)
 *   spike_bits: [T, M, Fout / 8] bytes, `spike_step_stride` bytes between timesteps     v_out : [M, Fout] fp32 or NULL
 *   workspace : as in snnf_linear_lif_ws, or NULL
 * 3 <= T <= 8, Fin a multiple of 8, Fout of 32, dtype SNNF_BF16 or SNNF_F16; SNNF_ERR_UNSUPPORTED otherwise.
 */
int snnf_linear_lif_bits(const void* const* xs, int x_bits, int T, int M, int Fin, int64_t x_row_stride, int dtype,
                         const void* weight, const void* bias, int Fout, const void* v_init, void* spike_bits,
                         int64_t spike_step_stride, void* v_out, float v_threshold, float v_reset, float tau,
                         void* workspace, size_t workspace_bytes, void* stream);

/*
 * Registers a measured launch choice for snnf_conv_lif_blocked on one layer shape (the counterpart of the per-kernel-key
 * "best config" the reference's autotuner keeps, kernels/benchmark_conv_lif_temporal_general.py:524-558,1332-1369):
 * columns of a wave's output patch (rows follow: 32 / columns), channel groups of 8 per LDS stage (a power of two) and
 * waves of a workgroup that share a tile's K (1, 2, 4 or 8). 0 leaves a choice to the built-in planner; all three 0
 * removes the entry. `shared_frame`: the layer receives one analog frame for all timesteps. A choice that the kernel
 * cannot run on the shape (a stage that does not fit a wave's LDS region, more waves than stages) is ignored at launch.
 * The table is process wide and thread safe; results do not depend on it beyond the order of fp32 additions.
 */
int snnf_conv_blocked_tune(int T, int N, int Cin, int H, int W, int Cout, int KH, int KW, int stride_h, int stride_w,
                           int pad_h, int pad_w, int shared_frame, int patch_cols, int stage_groups, int k_waves);

/* Describes what the most recent snnf_conv_lif / snnf_conv_bias call on this thread selected: kernel family, timesteps per launch, tile
 * and wave decomposition, LDS bytes, grid ("key=value" pairs, empty before the first call). Plays the role of the
 * reference's get_autotune_best_config (kernels/benchmark_conv_lif_temporal_general.py:1332-1369), whose result the
 * operator layer publishes as kernel_temporal_config (runtime/snn_custom_ops.py:341-353): selection here is a
 * deterministic planner, and this is how a host reads its decision. The pointer stays valid for the thread's lifetime. */
const char* snnf_conv_last_plan(void);

#ifdef __cplusplus
}
#endif

#endif /* SNNF_H_ */
