/*
 * tnn_hip.h -- C ABI of the MI355X (gfx950) implementation of tiny-dpcpp-nn's hot path:
 * the fully fused MLP (inference / training forward / fused backward with weight gradients),
 * the L2 loss, an Adam step, and the multi-resolution hash-grid encoding (forward / backward).
 *
 * Conventions
 *  - Every pointer named d_* is DEVICE memory owned by the caller. The library keeps no state between
 *    calls, allocates nothing and is thread-safe; every call is asynchronous on `stream`
 *    (a hipStream_t passed as void*, NULL = the default stream). Two exceptions, both stated where they
 *    are declared: the process-wide limit set by tnn_debug_set_meeting_spin_limit (a testing aid), and the
 *    fixed scratch array behind tnn_mlp_train_step_l2_static, which calls on one GPU share.
 *  - Return value: 0 on success, a negative tnn_status otherwise. No exception crosses this
 *    boundary; tnn_last_error() returns a thread-local message for the last failure.
 *  - "T" is the 2-byte storage type selected by tnn_mlp_desc::dtype (bf16 or fp16); all
 *    contractions accumulate in fp32 (reference: include/network/kernel_esimd.h:92-105).
 *  - Activation codes are the ordinals of the reference's `enum class Activation`
 *    (include/common/common.h:28-38); only None, ReLU and Sigmoid are accepted, as in
 *    include/network/SwiftNetMLP.h:252-291.
 *
 * Each entry point cites the reference interface it stands in for (paths relative to the
 * reference checkout).
 */
#ifndef TNN_HIP_H
#define TNN_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define TNN_HIP_ABI_VERSION 1

typedef void *tnn_stream_t; /* hipStream_t */

typedef enum tnn_status {
    TNN_OK = 0,
    TNN_ERR_INVALID_ARGUMENT = -1, /* reference: std::invalid_argument / std::runtime_error in the checks cited below */
    TNN_ERR_UNSUPPORTED = -2,      /* a variant the reference does not instantiate either */
    TNN_ERR_HIP = -3,              /* a HIP runtime call failed (launch error, no device, wrong architecture) */
    TNN_ERR_WORKSPACE = -4         /* workspace missing or too small */
} tnn_status;

typedef enum tnn_dtype { TNN_BF16 = 0, TNN_FP16 = 1, TNN_FP32 = 2 } tnn_dtype;

/* include/common/common.h:28-38 */
typedef enum tnn_activation {
    TNN_ACT_RELU = 0,
    TNN_ACT_LEAKY_RELU = 1,
    TNN_ACT_EXPONENTIAL = 2,
    TNN_ACT_SINE = 3,
    TNN_ACT_SIGMOID = 4,
    TNN_ACT_SQUAREPLUS = 5,
    TNN_ACT_SOFTPLUS = 6,
    TNN_ACT_TANH = 7,
    TNN_ACT_NONE = 8
} tnn_activation;

/* Shape of one fused MLP. Stands in for the template/ctor arguments of
 * SwiftNetMLP<T, WIDTH>(q, in, out, n_hidden_layers, activation, output_activation)
 * (include/network/SwiftNetMLP.h:50-67) after padding input and output to `width`
 * (include/network/Network.h:64-82). The network has n_hidden_layers + 1 weight matrices,
 * each width x width. width in {16, 32, 64, 128} (include/network/Network.h:160-161). */
typedef struct tnn_mlp_desc {
    int32_t dtype;             /* TNN_BF16 or TNN_FP16 */
    int32_t width;             /* 16, 32, 64, 128 */
    int32_t n_hidden_layers;   /* >= 1 */
    int32_t activation;        /* hidden layers */
    int32_t output_activation; /* last layer */
} tnn_mlp_desc;

const char *tnn_last_error(void);
int tnn_abi_version(void);
/* Number of HIP devices whose architecture is gfx950, or a negative status. */
int tnn_device_check(void);

/* DeviceMatrix::fill / DeviceMatrices::fill (include/common/DeviceMatrix.h:167,381): n elements of dtype := value. */
int tnn_fill(int dtype, void *d_ptr, size_t n, float value, tnn_stream_t stream);
/* DeviceMatrix::fill_random (include/common/DeviceMatrix.h:169-178, the default table of a grid encoding: uniform in
 * +-1e-4) and Network::initialize_xavier_normal (include/network/Network.h:271-295), both host generators plus a copy in
 * the reference: element i := lo + (hi - lo) * u, u in [0, 1) with 24 random bits, a pure function of (seed,
 * first_index + i) (the splitmix64 output function on seed + (first_index + i + 1) * 0x9E3779B97F4A7C15). The reference's
 * sequences (oneMKL philox, std::random_device) are not reproducible; only the distribution is the same. */
int tnn_fill_uniform(int dtype, void *d_ptr, size_t n, float lo, float hi, uint64_t seed, uint64_t first_index, tnn_stream_t stream);
/* DeviceMatrix::copy_from_device / DeviceMem::copy_from_device (include/common/DeviceMatrix.h:198-201,
 * include/common/DeviceMem.h:91-95): element-wise type-converting copy (round to nearest even). */
int tnn_cast(int dst_dtype, void *d_dst, int src_dtype, const void *d_src, size_t n, tnn_stream_t stream);

/* ------------------------------------------------------------------------------------------
 * Weight layouts.
 *   unpacked : per matrix element (k=in, n=out) at k*W + n (test/mlp.h:391-402)
 *   packed   : per matrix element (k, n) at (k & ~1)*W + 2n + (k & 1); the layout of the reference's
 *              parameters, get_params() and gradients (source/common/common.cpp:33-66)
 *   prepared : the MFMA operand order the kernels read; opaque, produced only by
 *              tnn_mlp_prepare_weights. It plays the role of the reference's second device copy,
 *              m_weightsT_matrices (include/network/Network.h:76-77,235-238).
 * ------------------------------------------------------------------------------------------ */

/* get_packed_weights (include/common/common.h:184-212), on device, n_mats W x W matrices of T. */
int tnn_pack_weights(int dtype, int width, int n_mats, const void *d_unpacked, void *d_packed, tnn_stream_t stream);
/* inverse of the above (fromPackedLayoutCoord, source/common/common.cpp:58-66). */
int tnn_unpack_weights(int dtype, int width, int n_mats, const void *d_packed, void *d_unpacked, tnn_stream_t stream);
/* DeviceMatrices::PackedTranspose (include/common/DeviceMatrix.h:429-444): packed W -> packed W^T. */
int tnn_packed_transpose(int dtype, int width, int n_mats, const void *d_packed, void *d_packed_T, tnn_stream_t stream);
/* DeviceMatrices::PackAndTranspose (include/common/DeviceMatrix.h:469-488): raw gradients
 * [out][in] -> parameter layout. In-place (d_raw == d_packed) is NOT allowed. */
int tnn_pack_and_transpose(int dtype, int width, int n_mats, const void *d_raw, void *d_packed, tnn_stream_t stream);
/* Network::ZeroWeightsPadding (include/network/Network.h:171-233) on packed weights: zero the rows of
 * matrix 0 at and beyond the one-padded input width, and the columns of the last matrix at and
 * beyond the unpadded output width. */
int tnn_zero_weights_padding(const tnn_mlp_desc *desc, void *d_packed, int unpadded_input_width,
                             int unpadded_output_width, int use_bias, tnn_stream_t stream);

/* Network::set_weights_matrices for parameters that are already packed and on the device (include/network/Network.h:90-112
 * with ZeroWeightsPadding :171-233 and TransposeWeights :235-238), in one launch: d_src_packed (src_dtype: T or fp32
 * masters, rounded to T) -> the packed copy in T with the padding weights zeroed, its packed transpose, and both prepared
 * operand sets. Bit for bit what tnn_cast + tnn_zero_weights_padding + tnn_packed_transpose + tnn_mlp_prepare_weights give;
 * it is what a module runs in front of every forward pass (dpcpp_bindings/tiny_dpcpp_nn/modules.py:253). */
int tnn_mlp_set_packed_weights(const tnn_mlp_desc *desc, const void *d_src_packed, int src_dtype, int unpadded_input_width,
                               int unpadded_output_width, int use_bias, void *d_packed_T, void *d_packed_transposed_T,
                               void *d_prepared_fwd, void *d_prepared_bwd, tnn_stream_t stream);

/* Bytes of ONE prepared buffer (forward and backward operand sets have the same size). */
size_t tnn_mlp_prepared_bytes(const tnn_mlp_desc *desc);
/* Packed parameters (type T, or fp32 master weights when src_is_fp32 != 0; they are rounded to T) ->
 * prepared forward and backward operand sets. Either output may be NULL. Replaces the device-side
 * work of Network::set_weights_matrices + TransposeWeights (include/network/Network.h:90-112). */
int tnn_mlp_prepare_weights(const tnn_mlp_desc *desc, const void *d_packed, int src_is_fp32, void *d_prepared_fwd,
                            void *d_prepared_bwd, tnn_stream_t stream);

/* ------------------------------------------------------------------------------------------
 * Fused MLP. Batch size M must be a multiple of 8 (include/network/SwiftNetMLP.h:293-300).
 * ------------------------------------------------------------------------------------------ */

/* EsimdKernels::inference_impl (include/network/kernel_esimd.h:242-247,565-640) reached through
 * SwiftNetMLP::inference (include/network/SwiftNetMLP.h:135-179).
 *   d_x: M x W row-major T. d_y: M x W row-major T (matrix 0 of the reference's output view). */
int tnn_mlp_inference(const tnn_mlp_desc *desc, const void *d_prepared_fwd, const void *d_x, void *d_y, size_t M,
                      tnn_stream_t stream);

/* EsimdKernels::forward_impl (include/network/kernel_esimd.h:153-158,565-640) reached through
 * SwiftNetMLP::forward_pass (include/network/SwiftNetMLP.h:69-119).
 *   d_interm_fwd: (n_hidden_layers + 2) matrices M x W: [0] = copy of x, [l] = activated output of
 *   matrix l-1, last = network output (include/common/DeviceMatrix.h:76-94). */
int tnn_mlp_forward(const tnn_mlp_desc *desc, const void *d_prepared_fwd, const void *d_x, void *d_interm_fwd, size_t M,
                    tnn_stream_t stream);

/* Workspace bytes tnn_mlp_backward needs (fp32 partial weight gradients, and staging for the deltas
 * when d_interm_bwd is NULL). */
size_t tnn_mlp_backward_workspace_bytes(const tnn_mlp_desc *desc, size_t M);

/* EsimdKernels::backward_impl (include/network/kernel_esimd.h:160-240: fused delta propagation
 * followed by oneMKL gemm_batch for dW) reached through SwiftNetMLP::backward_pass
 * (include/network/SwiftNetMLP.h:199-248).
 *   d_dLdy: M x W T. d_interm_fwd: as written by tnn_mlp_forward.
 *   d_interm_bwd: (n_hidden_layers + 1) matrices M x W, [l] = delta_l; may be NULL (then the deltas
 *                 are staged in the workspace).
 *   d_dW: (n_hidden_layers + 1) matrices [n=out][k=in] row-major T, unpacked (the gemm_batch output).
 *         If dW_is_fp32 != 0 the same layout is written as fp32 without the final rounding.
 *   d_dLdx: M x W T or NULL (kernel_esimd.h:217-226). */
int tnn_mlp_backward(const tnn_mlp_desc *desc, const void *d_prepared_bwd, const void *d_dLdy,
                     const void *d_interm_fwd, void *d_interm_bwd, void *d_dW, int dW_is_fp32, void *d_dLdx, size_t M,
                     void *d_workspace, size_t workspace_bytes, tnn_stream_t stream);

/* L2Loss (include/losses/l2.h:19-40, include/losses/loss.h:19-25): value_i = (p_i - t_i)^2 / N,
 * grad_i = T(loss_scale * 2 (p_i - t_i) / N), N = n_elements. d_values (fp32) may be NULL. */
int tnn_l2_loss(int dtype, const void *d_predictions, const float *d_targets, size_t n_elements, float loss_scale,
                float *d_values, void *d_grads, tnn_stream_t stream);

/* Workspace bytes for tnn_mlp_train_step_l2. */
size_t tnn_mlp_train_step_workspace_bytes(const tnn_mlp_desc *desc, size_t M);

/* One training step of the MLP in a single call: forward, L2 loss against fp32 targets, backward
 * with weight gradients. Equivalent to Trainer::training_step (include/trainer.h:23-46) with
 * L2Loss::evaluate (include/losses/loss.h:19-25) between its forward and backward pass; the
 * intermediate activations and deltas live in the workspace instead of caller-visible matrices.
 *   d_y: M x W network output (T) or NULL. d_loss_sum: one fp32 that receives sum_i value_i
 *   (the mean squared error), or NULL. d_dW / dW_is_fp32 / d_dLdx as in tnn_mlp_backward.
 *   N of the loss = M * W (all padded columns count, as in the reference). */
int tnn_mlp_train_step_l2(const tnn_mlp_desc *desc, const void *d_prepared_fwd, const void *d_prepared_bwd,
                          const void *d_x, const float *d_targets, float loss_scale, void *d_y, float *d_loss_sum,
                          void *d_dW, int dW_is_fp32, void *d_dLdx, size_t M, void *d_workspace,
                          size_t workspace_bytes, tnn_stream_t stream);

/* Adam on fp32 master parameters with the semantics of torch.optim.Adam (the optimizer the reference's
 * training loops use: dpcpp_bindings/tiny_dpcpp_nn/modules.py:171-175,
 * test/python/test_compare_torch_dpcpp.py:37). grad_dtype selects how d_grad is read (T or fp32);
 * grad is multiplied by grad_scale first (1/loss_scale). step counts from 1. If d_param_T is not NULL
 * it receives the updated parameters rounded to param_T_dtype. */
int tnn_adam_step(float *d_param, float *d_m, float *d_v, const void *d_grad, int grad_dtype, float grad_scale,
                  size_t n, int step, float lr, float beta1, float beta2, float eps, void *d_param_T,
                  int param_T_dtype, tnn_stream_t stream);

/* The optimizer step of a training loop on the fused MLP in one launch: what the reference's loop does
 * with PackAndTranspose of the raw gradients (include/tnn_api.h:599-603), torch.optim.Adam on the packed fp32
 * parameter (dpcpp_bindings/tiny_dpcpp_nn/modules.py:171-175) and set_params (modules.py:184-207, which
 * re-derives the device copies on every forward). Identical, bit for bit, to tnn_pack_and_transpose +
 * tnn_adam_step + tnn_mlp_prepare_weights.
 *   d_master_packed, d_m, d_v: fp32, packed parameter layout. d_dW_raw: fp32 [out][in] as written by
 *   tnn_mlp_backward / tnn_mlp_train_step_l2 with dW_is_fp32 != 0; multiplied by grad_scale (1/loss_scale).
 *   d_packed_T (may be NULL): updated parameters rounded to T, packed layout. d_prepared_fwd / d_prepared_bwd
 *   (may be NULL): the operand-order copies, updated in place. */
int tnn_mlp_adam_update(const tnn_mlp_desc *desc, float *d_master_packed, float *d_m, float *d_v, const float *d_dW_raw,
                        float grad_scale, int step, float lr, float beta1, float beta2, float eps, void *d_packed_T,
                        void *d_prepared_fwd, void *d_prepared_bwd, tnn_stream_t stream);

/* One whole optimisation step in two launches: tnn_mlp_train_step_l2 whose gradient reduction applies Adam
 * (tnn_mlp_adam_update's arithmetic, gradients multiplied by 1 / loss_scale) to the reduced sums directly, i.e. the
 * reference's loss.backward() + optimizer.step() + the weight re-staging of the next forward
 * (dpcpp_bindings/tiny_dpcpp_nn/modules.py:96-136,184-207 around torch.optim.Adam) without the gradients ever
 * reaching HBM as a tensor.
 *   d_prepared_fwd / d_prepared_bwd: read by this step, rewritten with the updated weights for the next one.
 *   d_master_packed, d_m, d_v: fp32, packed parameter layout, updated in place. step counts from 1.
 *   d_y, d_loss_sum, d_packed_T, d_dLdx: optional outputs as in the two functions above.
 *   main_kernel_done_event: NULL, or a hipEvent_t that is recorded on the stream after the step's main kernel
 *   (forward + loss + backward + partial weight gradients) and before the reduction, so that a caller can time the
 *   main kernel without a profiler.
 * Workspace: tnn_mlp_train_step_workspace_bytes. */
int tnn_mlp_train_step_l2_adam(const tnn_mlp_desc *desc, void *d_prepared_fwd, void *d_prepared_bwd, const void *d_x,
                               const float *d_targets, float loss_scale, void *d_y, float *d_loss_sum, float *d_master_packed,
                               float *d_m, float *d_v, int step, float lr, float beta1, float beta2, float eps, void *d_packed_T,
                               void *d_dLdx, size_t M, void *d_workspace, size_t workspace_bytes, void *main_kernel_done_event,
                               tnn_stream_t stream);

/* Network::backward_pass (include/network/SwiftNetMLP.h:199-257 over kernel_esimd.h:160-240) for a caller that kept no
 * activations: the weight gradients (and dL/dx) for a given dL/dy, with the forward pass formed again on chip from d_x in the
 * same kernel. It pairs with tnn_mlp_inference as the forward pass of a training step whose loss is computed by the caller
 * (PyTorch autograd): no M x W matrix except x, y and dL/dy is written or read, where forward_pass + backward_pass move
 * 2 * (n_hidden_layers + 2) of them. Same values as tnn_mlp_forward + tnn_mlp_backward on the same inputs (the activations
 * are the same bits; the weight gradients are fp32 sums over the batch taken in this kernel's fixed order).
 *   d_dLdy: M x W of T, the derivative of the loss with respect to the ACTIVATED output (the output activation's derivative
 *   is applied here, as in backward_pass). d_dW: raw layout [out][in], fp32 or T. d_dLdx: NULL or M x W of T.
 * Shapes: those of the one-kernel training step (width 16 / 32 / 64, up to 5 matrices at width 64 and 6 below);
 * tnn_mlp_backward_recompute_supported returns TNN_OK for them and TNN_ERR_UNSUPPORTED otherwise, and such a network
 * keeps its activations (tnn_mlp_forward + tnn_mlp_backward). Workspace: tnn_mlp_train_step_workspace_bytes. */
int tnn_mlp_backward_recompute_supported(const tnn_mlp_desc *desc);
int tnn_mlp_backward_recompute(const tnn_mlp_desc *desc, const void *d_prepared_fwd, const void *d_prepared_bwd, const void *d_x,
                               const void *d_dLdy, void *d_dW, int dW_is_fp32, void *d_dLdx, size_t M, void *d_workspace,
                               size_t workspace_bytes, tnn_stream_t stream);

/* Testing aid, no counterpart in the reference. In the width-64 training and backward kernels the four waves that share
 * staged tiles meet at a counter in LDS; a wave waits there for at most `iterations` polls (default 2^22, far beyond any
 * real wait) so that a kernel always ends. A wave whose wait runs out marks its workgroup, and the call then delivers NaN
 * in the loss and in EVERY weight gradient (and, through Adam, in the weights) instead of a plausible wrong number.
 * Setting the limit to 0 forces that path from the host while every kernel still runs to its end.
 * Returns a status (a negative limit is TNN_ERR_INVALID_ARGUMENT); *previous, when not NULL, receives the limit that was in
 * force. The limit is process-wide and read at every launch: it is for single-threaded test programs only -- while it is
 * lowered, every width-64 training or backward call of any thread of the process is affected. */
int tnn_debug_set_meeting_spin_limit(int iterations, int *previous);

/* tnn_mlp_train_step_l2 for callers that cannot allocate device memory: code recorded into a HIP graph, tight serving
 * loops, harnesses that forbid hipMalloc. It has no counterpart in the reference. It takes no workspace: the partial
 * weight gradients and partial losses of the step go to a fixed array of TNN_MLP_TRAIN_STEP_STATIC_SCRATCH_BYTES of
 * device memory inside the library, which every GPU that runs the library holds until the process ends. The call
 * allocates and frees nothing. Shapes and batch sizes whose tnn_mlp_train_step_workspace_bytes exceeds that size
 * (the separate-kernel route of wide or deep networks at large batches) are rejected with TNN_ERR_WORKSPACE; every
 * shape that has the fused kernel fits at any batch size. Same arguments and results, bit for bit, as
 * tnn_mlp_train_step_l2. All calls on one GPU share the one array: calls that overlap on a GPU (two streams, two
 * threads) race; serialise them. Nothing in the array has to be cleared between calls. The first call on a device
 * looks up the array's address there (make that call outside a graph capture). */
#define TNN_MLP_TRAIN_STEP_STATIC_SCRATCH_BYTES (21u << 20)
size_t tnn_mlp_train_step_l2_static_max_bytes(void);
int tnn_mlp_train_step_l2_static(const tnn_mlp_desc *desc, const void *d_prepared_fwd, const void *d_prepared_bwd,
                                 const void *d_x, const float *d_targets, float loss_scale, void *d_y, float *d_loss_sum,
                                 void *d_dW, int dW_is_fp32, void *d_dLdx, size_t M, tnn_stream_t stream);

/* ------------------------------------------------------------------------------------------
 * Multi-resolution hash grid (include/encodings/grid.h, include/common/common_device.h:700-775).
 * ------------------------------------------------------------------------------------------ */
#define TNN_GRID_MAX_LEVELS 128 /* include/encodings/grid_interface.h:23 */

typedef enum tnn_grid_type { TNN_GRID_HASH = 0, TNN_GRID_DENSE = 1, TNN_GRID_TILED = 2 } tnn_grid_type;
typedef enum tnn_hash_type {
    TNN_HASH_PRIME = 0,
    TNN_HASH_COHERENT_PRIME = 1,
    TNN_HASH_REVERSED_PRIME = 2,
    TNN_HASH_RNG = 3
} tnn_hash_type;
typedef enum tnn_interpolation { TNN_INTERP_NEAREST = 0, TNN_INTERP_LINEAR = 1, TNN_INTERP_SMOOTHSTEP = 2 } tnn_interpolation;

/* Everything kernel_grid / kernel_grid_backward receive by value (include/encodings/grid.h:37-47,
 * GridOffsetTable include/encodings/grid_interface.h:24-28). Filled by tnn_grid_desc_init, which does
 * the work of the GridEncodingTemplated constructor (include/encodings/grid.h:588-659) on the host:
 * the per-level scale and resolution are evaluated once with the host's float math. */
typedef struct tnn_grid_desc {
    uint32_t n_dims;               /* 2 or 3 */
    uint32_t n_levels;             /* <= TNN_GRID_MAX_LEVELS */
    uint32_t n_features_per_level; /* 1, 2, 4 or 8 */
    uint32_t log2_hashmap_size;
    uint32_t base_resolution;
    float per_level_scale;
    uint32_t grid_type;
    uint32_t hash_type;
    uint32_t interpolation;
    uint32_t param_dtype; /* dtype of the table: TNN_FP32 (reference) or TNN_FP16 */
    uint32_t offsets[TNN_GRID_MAX_LEVELS + 1]; /* in entries; entry e of level l holds its features at (offsets[l]+e)*F */
    float scales[TNN_GRID_MAX_LEVELS];
    uint32_t resolutions[TNN_GRID_MAX_LEVELS];
} tnn_grid_desc;

int tnn_grid_desc_init(tnn_grid_desc *desc, uint32_t n_dims, uint32_t n_levels, uint32_t n_features_per_level,
                       uint32_t log2_hashmap_size, uint32_t base_resolution, float per_level_scale,
                       uint32_t grid_type, uint32_t hash_type, uint32_t interpolation, uint32_t param_dtype);
/* offsets[n_levels] * n_features_per_level */
size_t tnn_grid_n_params(const tnn_grid_desc *desc);

/* kernel_grid + the zero padding kernel (include/encodings/grid.h:37-135,661-734).
 *   d_x: M x n_dims fp32 row-major. d_table: n_params of param_dtype.
 *   d_out: M x padded_width of out_dtype (TNN_FP32 as in the reference, or TNN_BF16/TNN_FP16 so the
 *   MLP can consume it without a cast); column l*F + f, columns >= n_levels*F zero. */
int tnn_grid_forward(const tnn_grid_desc *desc, const float *d_x, const void *d_table, void *d_out, int out_dtype,
                     uint32_t padded_width, size_t M, tnn_stream_t stream);

/* Cell order of a batch, for large batches of scattered points. No counterpart in the reference, whose kernel_grid takes the
 * points as they come (include/encodings/grid.h:37-135, launch :696-731). tnn_grid_order_points writes, into a caller-owned
 * buffer of tnn_grid_order_bytes(desc, M) bytes (256-byte aligned), one 16-byte record per point, coordinates and row number,
 * sorted by the cell of a coarse grid (counting sort on the leading 6 bits of every coordinate in 3-D, 9 in 2-D; coordinates
 * outside [0, 1) and NaN land in an end bin). tnn_grid_forward_ordered is tnn_grid_forward reading those records: thread i
 * evaluates the i-th record and writes that point's row, so d_out equals tnn_grid_forward's bit for bit, while neighbouring
 * lanes gather from the same 128-byte lines of the table (config 5, 2^21 uniform points: 1.8 ms -> 1.0 ms + the ordering).
 * The records depend on d_x only: one ordering serves any number of forward calls on the same points. M < 2^32. */
size_t tnn_grid_order_bytes(const tnn_grid_desc *desc, size_t M);
int tnn_grid_order_points(const tnn_grid_desc *desc, const float *d_x, size_t M, void *d_order, size_t order_bytes,
                          tnn_stream_t stream);
int tnn_grid_forward_ordered(const tnn_grid_desc *desc, const void *d_order, const void *d_table, void *d_out, int out_dtype,
                             uint32_t padded_width, size_t M, tnn_stream_t stream);

/* kernel_grid_backward with GradientMode::Overwrite or Accumulate (include/encodings/grid.h:137-245,
 * 736-797). d_dLdy: M x padded_width of dy_dtype. d_grad_table: n_params fp32 (grad_t = float,
 * grid.h:586). overwrite != 0 zeroes the table first (grid.h:758-762). */
int tnn_grid_backward(const tnn_grid_desc *desc, const float *d_x, const void *d_dLdy, int dy_dtype,
                      uint32_t padded_width, float *d_grad_table, int overwrite, size_t M, tnn_stream_t stream);

/* tnn_grid_backward over the records of tnn_grid_order_points instead of d_x (no counterpart in the reference). Thread
 * groups take the points in cell order and read row `row number` of d_dLdy; neighbouring groups then often add to the same
 * entry, so runs of equal entries inside a wave are summed in registers and added with one atomic per run. The table
 * receives the same contributions as from tnn_grid_backward in another order of addition (the reference defines none,
 * grid.h:215-243). */
int tnn_grid_backward_ordered(const tnn_grid_desc *desc, const void *d_order, const void *d_dLdy, int dy_dtype,
                              uint32_t padded_width, float *d_grad_table, int overwrite, size_t M, tnn_stream_t stream);

/* The same scatter into an fp16 gradient table, two features of an entry per packed atomic (global_atomic_pk_add_f16): half
 * as many atomic operations as the fp32 route and half the gradient table; the same number of 32-byte requests at the memory
 * side, which is what bounds the pass, so about the same time. No counterpart in the reference, whose
 * gradients are float (grad_t, include/encodings/grid.h:586, "we don't have atomics for half precision",
 * dpcpp_bindings/tiny_dpcpp_nn/modules.py:320-324); it is what tiny-cuda-nn does for half-precision grids. Sums are
 * rounded to fp16 at every addition: scale dL/dy (loss scale) so that contributions stay clear of fp16's denormal range.
 * n_features_per_level must be even. d_grad_table_f16: n_params fp16. Coarse levels are still accumulated in fp32 (LDS)
 * and rounded once when they are flushed. */
int tnn_grid_backward_packed(const tnn_grid_desc *desc, const float *d_x, const void *d_dLdy, int dy_dtype,
                             uint32_t padded_width, void *d_grad_table_f16, int overwrite, size_t M, tnn_stream_t stream);

/* Debug/verification aid: entry index (inside its level) of every (point, level, corner), the
 * integer part of kernel_grid (grid.h:95-129 with grid_index, common_device.h:745-765).
 * d_indices: M x n_levels x 2^n_dims uint32. */
int tnn_grid_indices(const tnn_grid_desc *desc, const float *d_x, uint32_t *d_indices, size_t M, tnn_stream_t stream);

/* Grid encoding and network inference in one kernel: y = MLP(pad(grid(x))), the encoded rows stay in registers.
 * Replaces the pair of calls behind NetworkWithInputEncoding in inference
 * (dpcpp_bindings/tiny_dpcpp_nn/modules.py:357-421: Encoding.forward, then Network.forward on its padded output;
 * include/encodings/grid.h:37-135 + include/network/kernel_esimd.h:565-640) and returns the values of
 * tnn_grid_forward(out_dtype = mlp->dtype, padded_width = mlp->width) followed by tnn_mlp_inference, bit for bit.
 * Needs n_levels * n_features_per_level <= mlp->width and weights that fit LDS beside 2.5 KiB of level constants (width 64: up to
 * 19 matrices, width 128: up to 4); TNN_ERR_UNSUPPORTED otherwise, and the two calls do the work.
 * d_x: M x n_dims fp32. d_table: n_params of grid->param_dtype. d_prepared_fwd: tnn_mlp_prepare_weights' forward
 * buffer. d_y: M x width of mlp->dtype. M: positive multiple of 8. */
int tnn_grid_mlp_inference(const tnn_grid_desc *grid, const tnn_mlp_desc *mlp, const float *d_x, const void *d_table,
                           const void *d_prepared_fwd, void *d_y, size_t M, tnn_stream_t stream);
/* tnn_grid_mlp_inference over points in cell order (d_order: the records tnn_grid_order_points wrote): the same rows of d_y,
 * bit for bit. */
int tnn_grid_mlp_inference_ordered(const tnn_grid_desc *grid, const tnn_mlp_desc *mlp, const void *d_order, const void *d_table,
                                   const void *d_prepared_fwd, void *d_y, size_t M, tnn_stream_t stream);

/* One optimisation step of a network behind a hash-grid encoding without the encoded matrix (the training half of the
 * fused path above): what the reference's training loop does with Encoding.forward, Network.forward, the L2 loss,
 * loss.backward() through both modules and optimizer.step() on the network's parameters
 * (dpcpp_bindings/tiny_dpcpp_nn/modules.py:357-421 over include/encodings/grid.h:661-797 and include/trainer.h:23-46).
 * The encoding is evaluated inside the training kernel where tnn_mlp_train_step_l2_adam loads its input rows, so the
 * M x width encoded matrix is neither written nor read; dL/d(encoding) goes through the workspace into the scatter of
 * tnn_grid_backward (tnn_grid_backward_ordered when d_order is given). Same values as tnn_grid_forward (out_dtype = network
 * type, padded_width = width) + tnn_mlp_train_step_l2_adam (with d_dLdx) + tnn_grid_backward. With d_x (the caller's order):
 * outputs, loss, Adam state and re-staged weights bit for bit, the table's gradient up to the order of its fp32 additions
 * (atomic sums, as in the reference). With d_order: every per-row result (d_y, dL/d(encoding)) is still bit-exact, but the
 * place of a point among the points of its cell is taken with atomics when the order is built, so the tiles hold other rows
 * from run to run and every sum over the batch (loss, weight gradients and what Adam makes of them, table gradient) is
 * reproducible to fp32 rounding only, not bit for bit.
 *   d_x: M x n_dims fp32, or NULL when d_order holds the records of tnn_grid_order_points for the batch (rows of d_targets
 *   and d_y keep the caller's order either way). d_table: the encoding's parameters (param_dtype).
 *   d_grad_table: n_params fp32, overwritten or accumulated into as in tnn_grid_backward; it holds loss_scale x the gradient.
 *   Network arguments as in tnn_mlp_train_step_l2_adam. Built for width 64, ReLU, at most 4 hidden layers and 2 features per
 *   level (tnn_grid_mlp_train_supported returns TNN_OK); other shapes get TNN_ERR_UNSUPPORTED and run the three calls.
 * Workspace: tnn_grid_mlp_train_step_workspace_bytes. */
int tnn_grid_mlp_train_supported(const tnn_grid_desc *grid, const tnn_mlp_desc *mlp);
size_t tnn_grid_mlp_train_step_workspace_bytes(const tnn_grid_desc *grid, const tnn_mlp_desc *mlp, size_t M);
int tnn_grid_mlp_train_step_l2_adam(const tnn_grid_desc *grid, const tnn_mlp_desc *mlp, const float *d_x, const void *d_order,
                                    const void *d_table, void *d_prepared_fwd, void *d_prepared_bwd, const float *d_targets,
                                    float loss_scale, void *d_y, float *d_loss_sum, float *d_master_packed, float *d_m, float *d_v,
                                    int step, float lr, float beta1, float beta2, float eps, void *d_packed_T, float *d_grad_table,
                                    int overwrite, size_t M, void *d_workspace, size_t workspace_bytes, tnn_stream_t stream);
/* The backward pass of a network behind a hash-grid encoding for a given dL/dy, without the encoded matrix: what
 * loss.backward() does through NetworkWithInputEncoding in the reference (dpcpp_bindings/tiny_dpcpp_nn/modules.py:84-136 over
 * Network::backward_pass and GridEncoding::backward_impl, include/encodings/grid.h:752-797). The encoding and the
 * network's forward pass are formed again on chip from the positions (tnn_grid_mlp_inference is the forward pass that goes
 * with it), the weight gradients leave as in tnn_mlp_backward_recompute, and dL/d(encoding) goes through the workspace into
 * the scatter of tnn_grid_backward (tnn_grid_backward_ordered when d_order is given). d_grad_table: n_params fp32, or NULL
 * when only the network's gradients are wanted. Shapes and workspace as tnn_grid_mlp_train_step_l2_adam. */
int tnn_grid_mlp_backward(const tnn_grid_desc *grid, const tnn_mlp_desc *mlp, const float *d_x, const void *d_order, const void *d_table,
                          const void *d_prepared_fwd, const void *d_prepared_bwd, const void *d_dLdy, void *d_dW, int dW_is_fp32,
                          float *d_grad_table, int overwrite, size_t M, void *d_workspace, size_t workspace_bytes, tnn_stream_t stream);
/* TNN_OK when tnn_grid_mlp_inference runs this pair of shapes, otherwise the status (and tnn_last_error the reason) it
 * would return: lets a caller choose between the fused call and the two calls once, when the modules are built. */
int tnn_grid_mlp_supported(const tnn_grid_desc *grid, const tnn_mlp_desc *mlp);

/* ------------------------------------------------------------------------------------------
 * Encodings without parameters. Rows are M x padded_width of out_dtype; the columns beyond the encoding's own
 * width are filled with ONES (the grid pads with zeros). Inputs are M x n_dims fp32, row-major.
 * ------------------------------------------------------------------------------------------ */

/* IdentityEncoding::forward_impl (include/encodings/identity.h:33-79): out = x * scale + offset. */
int tnn_identity_forward(const float *d_x, uint32_t n_dims, float scale, float offset, void *d_out, int out_dtype,
                         uint32_t padded_width, size_t M, tnn_stream_t stream);

/* FrequencyEncoding::forward_impl (include/encodings/frequency.h:30-90): column j of a row is
 * sin(x[j / (2 n_f)] * 2^((j / 2) % n_f) * pi + (j % 2) * pi / 2). d_dy_dx: NULL, or M x (n_dims * n_f * 2) fp32
 * that receives the derivative of every output column (the reference's ForwardContext::dy_dx, :41-47,82-84). */
int tnn_frequency_forward(const float *d_x, uint32_t n_dims, uint32_t n_frequencies, void *d_out, int out_dtype,
                          uint32_t padded_width, float *d_dy_dx, size_t M, tnn_stream_t stream);
/* FrequencyEncoding::backward_impl (include/encodings/frequency.h:92-131): dL/dx = sum over a feature's columns of
 * dL/dy * dy/dx. d_dLdx: M x n_dims fp32. */
int tnn_frequency_backward(const void *d_dLdy, int dy_dtype, uint32_t padded_width, const float *d_dy_dx, uint32_t n_dims,
                           uint32_t n_frequencies, float *d_dLdx, size_t M, tnn_stream_t stream);

/* SphericalHarmonicsEncoding::forward_impl with sh_enc (include/encodings/spherical_harmonics.h:38-72,
 * include/common/common_device.h:33-206): the degree^2 real spherical harmonics of bands 0 .. degree-1 at the
 * direction 2x - 1 (x: M x 3). degree 1 .. 8. */
int tnn_sh_forward(const float *d_x, uint32_t degree, void *d_out, int out_dtype, uint32_t padded_width, size_t M,
                   tnn_stream_t stream);

/* Measurement aid, no counterpart in the reference: the rate at which the memory system serves the access pattern that
 * bounds the hash-grid gather (include/encodings/grid.h:95-129 over a table beyond the caches), with nothing else in the
 * kernel. n_threads threads (one per "point", workgroups of 256 as the encoding kernel's) each read 4 bytes from
 * lines_per_thread (a multiple of 32) random 128-byte lines of d_buffer, 32 of them in flight at a time, and write one 4-byte
 * sum to d_sink (n_threads x 4 bytes). The lines per second it reaches over a buffer of the table's size are the ceiling
 * against which the encoding kernel's own line rate is read (bench.py --workload line_probe). */
int tnn_probe_line_gather(const void *d_buffer, size_t buffer_bytes, size_t n_threads, int lines_per_thread, uint32_t seed, void *d_sink,
                          tnn_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* TNN_HIP_H */
