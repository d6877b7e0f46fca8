/*
 * mi355x_int8 -- C ABI of the MI355X (gfx950) implementation of MindSpore Lite's full-quant int8 inference hot path.
 *
 * The library is the drop-in for the arithmetic that Lite's CPU kernels delegate to nnacl.  A Lite provider kernel
 * (mindspore::kernel::Kernel subclass registered with registry::RegisterKernel) maps onto it as
 *     Prepare()/ReSize()  ->  mi_*_create      (quant-parameter derivation, weight packing, bias fold, upload)
 *     Execute()           ->  mi_*_run_host    (host tensors, as a "CPU"-arch provider kernel receives them)
 *                             mi_*_run         (device pointers + HIP stream, for chained device-resident tensors)
 *     ~Kernel()           ->  mi_*_destroy
 *
 * Conventions
 *   - every entry point returns an int status with the numeric values of Lite's RET_* codes
 *     (mindspore/lite/include/errorcode.h:28-39); nothing throws across the boundary;
 *   - plain pointers and sizes only; "host" pointers are ordinary process memory, "dev" pointers are HIP device
 *     memory on the device chosen by mi_init; `stream` is a hipStream_t passed as void* (NULL = default stream);
 *   - handles are thread-compatible: distinct handles may be used from different threads, one handle from one
 *     thread at a time;
 *   - all tensors are dense row-major; images are NHWC; activation types use schema ActivationType values
 *     (mindspore/lite/schema/ops_types.fbs:62-66): 0 none, 1 ReLU, 3 ReLU6.
 *
 * Reference paths below are relative to the reference tree:
 *   NN/ = mindspore/ccsrc/plugin/device/cpu/kernel/nnacl/      LK/ = mindspore/lite/src/litert/kernel/cpu/
 */
#ifndef MI355X_INT8_H_
#define MI355X_INT8_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define MI_OK 0
#define MI_ERROR (-1)         /* RET_ERROR: HIP failure or internal error */
#define MI_NULL_PTR (-2)      /* RET_NULL_PTR */
#define MI_PARAM_INVALID (-3) /* RET_PARAM_INVALID: shape/quant-parameter mismatch, nothing was launched */
#define MI_MEMORY_FAILED (-6) /* RET_MEMORY_FAILED */
#define MI_NOT_SUPPORT (-7)   /* RET_NOT_SUPPORT: the creator should decline and let the builtin CPU kernel run */
#define MI_INFER_ERR (-500)     /* RET_INFER_ERR: the operand shapes do not fit the operator */
#define MI_INFER_INVALID (-501) /* RET_INFER_INVALID: an input dimension is still unknown (negative); infer again later */

#define MI_ACT_NONE 0
#define MI_ACT_RELU 1
#define MI_ACT_RELU6 3

/* ---- library ---------------------------------------------------------------------------------------------- */

/* Selects the HIP device and verifies it is gfx950.  Must be called once before any create/run call.
 * Returns MI_NOT_SUPPORT when no such GPU is present (the provider then registers nothing). */
int mi_init(int device);
/* Message of the last failure on the calling thread ("" if none). */
const char *mi_last_error(void);
/* Test aid: while `bytes` is non-zero, every device allocation the library makes for a handle (packed weights,
 * parameters, workspaces) whose size, rounded up to 4 KiB, equals `bytes` rounded up to 4 KiB fails as if the device
 * were out of memory; 0 switches it off.  Lets a test show what a handle does when one of its allocations fails. */
int mi_debug_fail_alloc(size_t bytes);
/* Test aid: how many times the library has made the host wait for a stream so far (mi_copy_to_device, mi_copy_to_host,
 * mi_stream_synchronize, mi_dynquant_get_params; the *_run_host entry points are not counted). */
int64_t mi_debug_sync_count(void);
const char *mi_version(void);

/* ---- quant-parameter derivation (host arithmetic, no GPU needed) -------------------------------------------- */

/* real multiplier -> (31-bit mantissa, left shift >= 0, right shift <= 0).
 * Replaces QuantizeRoundParameterWithDoublePrecision, NN/int8/quantize.c:39-51 (QuantizeMultiplier :113-161). */
int mi_quantize_multiplier(double real_multiplier, int32_t *multiplier, int32_t *left_shift, int32_t *right_shift);
/* The alternative rounding the convolution wrappers select when a tensor's QuantParam.multiplier is 0
 * (LK/base/convolution_base.cc:421-423,446-456).  Replaces QuantizeRoundParameterWithSinglePrecision,
 * NN/int8/quantize.c:53-72, including its conversion of the double's value (not its bits) to uint32.  A provider
 * kernel cannot see that field, so the create calls always use the double-precision method (the schema default);
 * this entry point exists for callers that read the model themselves.  Domain 0 <= m < 2^32, else MI_PARAM_INVALID. */
int mi_quantize_multiplier_single(double real_multiplier, int32_t *multiplier, int32_t *left_shift,
                                  int32_t *right_shift);
/* Clamp bounds of the fused activation in the quantised domain.
 * Replaces CalculateActivationRangeQuantized, NN/int8/quantize.c:78-94. */
int mi_activation_range(int32_t act_type, int32_t out_zp, double out_scale, int32_t *act_min, int32_t *act_max);
/* (mult, ls, rs)[i] for real multiplier (float)in_scale*(float)filter_scale[i] / (float)out_scale, the derivation of
 * MatmulBaseInt8CPUKernel::InitQuantParam (LK/int8/matmul_base_int8.cc:258-266) and
 * ConvolutionBaseCPUKernel::SetQuantMultiplier (LK/base/convolution_base.cc:416-427). */
int mi_requant_params(double in_scale, const double *filter_scales, int32_t n, double out_scale, int32_t *multiplier,
                      int32_t *left_shift, int32_t *right_shift);
/* One requantisation step on the host: MultiplyByQuantizedMultiplier, NN/int8/fixed_point.c:66-68. */
int32_t mi_multiply_by_quantized_multiplier(int32_t value, int32_t multiplier, int32_t left_shift,
                                            int32_t right_shift);

/* ---- full-quant MatMul / FullConnection ------------------------------------------------------------------- */
/* Replaces MatmulBaseInt8CPUKernel (LK/int8/matmul_base_int8.cc: InitQuantParam :235-273, TransferB :360-384,
 * Run :530-571, RunImpl :129-150), FullconnectionInt8CPUKernel (LK/int8/fullconnection_int8.cc:26-67) and the nnacl
 * functions they call: RowMajor2Row16x4MajorInt8 / RowMajor2Col16x4MajorInt8 (NN/int8/matmul_int8.c:158-236,722-736),
 * CalcInputSums (:786-799), CalcWeightBiasSums (:802-819), MatmulInt8Opt (:296-331). */
typedef struct mi_matmul mi_matmul;

typedef struct mi_matmul_desc {
  int32_t deep;        /* K */
  int32_t col;         /* N: output channels */
  int32_t b_transpose; /* 1: weight is [N,K] (FullConnection, MatMul transpose_b); 0: weight is [K,N] */
  int32_t act_type;
  double in_scale;
  int32_t in_zp;
  double out_scale;
  int32_t out_zp;
  int32_t filter_quant_num;    /* 1 (per tensor) or col (per output channel) */
  const double *filter_scales; /* [filter_quant_num] */
  const int32_t *filter_zps;   /* [filter_quant_num] */
  int32_t flags;               /* 0 or MI_MATMUL_NO_DECODE_PACK */
  int32_t b_batch;             /* 0 or 1: one weight matrix; > 1: weight_host holds this many [deep x col] matrices
                                  one after the other (a constant weight of rank > 2) */
} mi_matmul_desc;

/* All weight packing happens in mi_matmul_create (the role of TransferB, LK/int8/matmul_base_int8.cc:360-384: pack
 * once at Prepare).  Two packed forms are kept: K-contiguous rows (GEMM tiles; one activation row) and 1 KiB
 * blocks of 16 channels x 64 K-bytes in matrix-core operand order (2..64 activation rows, 2..128 against at most
 * 4096 channels with deep >= 1024: the batched decode kernel).  MI_MATMUL_NO_DECODE_PACK skips the second form (deep x col bytes of device memory less) for callers
 * that know they never run with 2..64 rows; such a handle still accepts those row counts and runs two rows on the
 * one-row kernel's two-row form and the others on the GEMM tiles.  mi_matmul_run never packs, allocates for packing or waits. */
#define MI_MATMUL_NO_DECODE_PACK 1

/* weight_host: int8 const weight; bias_host: int32 [col] or NULL.  Both are consumed during the call. */
int mi_matmul_create(const mi_matmul_desc *desc, const int8_t *weight_host, const int32_t *bias_host,
                     mi_matmul **out);
/* Sizes the handle's workspaces for runs of up to `max_rows` rows, so that later runs allocate nothing: the role of
 * the buffers MatmulBaseInt8CPUKernel::ReSize allocates (LK/int8/matmul_base_int8.cc:296-325).  Workspaces exist only
 * for operand shapes the kernels cannot take in place (deep % 16 != 0 or a misaligned activation base: a padded copy
 * of the activations; col % 4 != 0 or a misaligned output base: a padded output).  Without this call the first run
 * that needs a larger workspace allocates it with hipMalloc, at least twice the previous size; the outgrown buffer
 * may still be in use by kernels in flight, so it is kept until the handle is destroyed (a handle therefore holds at
 * most about twice its largest workspace; the same holds for the im2col and output workspaces of mi_conv). */
int mi_matmul_reserve(mi_matmul *h, int32_t max_rows);
/* a_dev: int8 [rows, deep]; c_dev: int8 [rows, col].  Asynchronous on `stream`. */
int mi_matmul_run(mi_matmul *h, const int8_t *a_dev, int32_t rows, int8_t *c_dev, void *stream);
/* Batched MatMul (MatmulBaseInt8CPUKernel::Run, LK/int8/matmul_base_int8.cc:549-568): output matrix i =
 * activation matrix a_offsets[i] x weight matrix b_offsets[i], for i = 0 .. batch-1.  a_dev holds [rows, deep]
 * matrices one after the other, c_dev receives `batch` [rows, col] matrices, the weight matrices are those given to
 * mi_matmul_create (desc.b_batch).  The offsets are what MatmulFp32BaseCPUKernel::InitBroadcastParams
 * (LK/fp32/matmul_fp32_base.cc:576-646) derives from the two shapes; mi_matmul_broadcast_offsets computes them. */
int mi_matmul_run_batched(mi_matmul *h, const int8_t *a_dev, int32_t rows, int32_t batch, const int32_t *a_offsets,
                          const int32_t *b_offsets, int8_t *c_dev, void *stream);
/* The batch broadcast rule of MatMul (InitBroadcastParams, LK/fp32/matmul_fp32_base.cc:576-646; host arithmetic, no
 * GPU needed): for operand shapes a_shape / b_shape (the last two extents are the matrix) the number of output
 * matrices and, per output matrix, the index of the activation and of the weight matrix it is made of.  a_offsets /
 * b_offsets have room for `capacity` entries; MI_PARAM_INVALID when the batch extents cannot be broadcast or the
 * result does not fit. */
int mi_matmul_broadcast_offsets(const int32_t *a_shape, int32_t a_dims, const int32_t *b_shape, int32_t b_dims,
                                int32_t capacity, int32_t *batch, int32_t *a_offsets, int32_t *b_offsets);
/* mi_matmul_run for callers that cannot allocate device memory: code under HIP graph capture, tight serving loops,
 * harnesses that forbid hipMalloc.  No counterpart in the reference.  Same arguments, same results; instead of the
 * handle's growable workspaces it uses one scratch area of MI_NOALLOC_SCRATCH_BYTES of static device memory (held by
 * every GPU the library is initialised on until the process ends) and calls neither hipMalloc nor hipFree nor any
 * allocating routine.  Scratch is needed only for operands the kernels cannot take in place: rows x round_up(deep,
 * 16) bytes when deep % 16 != 0 or a_dev is not 16-byte aligned, plus rows x round_up(col, 4) bytes when col % 4 != 0
 * or c_dev is not 4-byte aligned; a call that needs more than the maximum returns MI_PARAM_INVALID and launches
 * nothing.  All handles on a GPU share the scratch area: calls of this entry point that overlap in time on one
 * GPU (different streams or threads) race on it; calls ordered on one stream do not. */
#define MI_NOALLOC_SCRATCH_BYTES (8u << 20)
int mi_matmul_run_noalloc(mi_matmul *h, const int8_t *a_dev, int32_t rows, int8_t *c_dev, void *stream);
/* Same with host tensors: copies in, runs, copies out, synchronises. */
int mi_matmul_run_host(mi_matmul *h, const int8_t *a_host, int32_t rows, int8_t *c_host);
/* Several MatMul / FullConnection kernels that read the same input tensor (same `deep`), e.g. the gate and up
 * projections of a decoder layer or separate Q, K, V projections: equal to mi_matmul_run(handles[i], a_dev, rows,
 * c_dev[i], stream) for i = 0 .. count-1.  With at most 32 rows and two to four members the weight-streaming kernels
 * run them as ONE launch (one grid, the members' channel ranges side by side), which saves the start-up and drain of
 * the memory stream once per merged member; other cases run member by member.  The reference executes such sibling
 * kernels one after the other (mindspore/lite/src/executor/sub_graph_kernel.cc:456-466; each is a
 * MatmulBaseInt8CPUKernel::Run, LK/int8/matmul_base_int8.cc:530-570). */
int mi_matmul_run_group(mi_matmul *const *handles, int32_t count, const int8_t *a_dev, int32_t rows,
                        int8_t *const *c_dev, void *stream);
/* Derived per-channel parameters (arrays of `col` entries, any may be NULL): multiplier / shifts, the folded bias
 * K*zx*zw - zx*sum(w) + bias, and the clamp bounds. */
int mi_matmul_get_params(const mi_matmul *h, int32_t *multiplier, int32_t *left_shift, int32_t *right_shift,
                         int32_t *folded_bias, int32_t *act_min, int32_t *act_max);
void mi_matmul_destroy(mi_matmul *h);

/* ---- Conv2DFusion int8 (group 1: 1x1 and im2col; group == channels: depthwise) ----------------------------- */
/* Replaces Convolution1x1Int8CPUKernel (LK/int8/convolution_1x1_int8.cc: InitBiasByzp :158-217, InitParam :359-413,
 * Pre1x1Trans :435-444, Run :572-621), ConvolutionInt8CPUKernel (LK/int8/convolution_int8.cc: InitWeightBias :53-157,
 * Run :248-263), ConvolutionDepthwiseInt8CPUKernel (LK/int8/convolution_depthwise_int8.cc:33-197), the quant setup
 * of ConvolutionBaseCPUKernel (LK/base/convolution_base.cc:246-499) and the nnacl functions they call: Conv1x1Int8
 * (NN/int8/conv1x1_int8.c:31-40), Conv1x1InputPack (NN/base/conv1x1_base.c:19-40), ConvInt8 /
 * Im2ColPackUnitInt8Opt (NN/int8/conv_int8.c:758-913), MatMulInt8_8x8_r (NN/int8/matmul_int8.c:333-364),
 * ConvDwInt8 / ConvDwInt8Post (NN/int8/conv_depthwise_int8.c:24-140).
 * mi_conv_create returns MI_NOT_SUPPORT for what the provider must leave to the builtin kernels: grouped
 * convolutions other than depthwise, and 3x3 stride-1 dilation-1 dense convolutions unless MI_CONV_3X3_EXACT is set.
 * For those the reference's choice of kernel depends on the CPU (LK/int8/convolution_int8_creator.cc:81-94): ARM64
 * cores with the dot-product extension run ConvolutionInt8CPUKernel, the exact convolution this library computes,
 * every other build (x86 included) runs Convolution3x3Int8CPUKernel, an integer Winograd whose results differ from
 * the exact convolution.  With the flag the library reproduces the former; without it it declines. */
#define MI_CONV_3X3_EXACT 1
typedef struct mi_conv mi_conv;

typedef struct mi_conv_desc {
  int32_t in_channel, out_channel;
  int32_t kernel_h, kernel_w, stride_h, stride_w, dilation_h, dilation_w;
  int32_t pad_u, pad_d, pad_l, pad_r;
  int32_t group; /* 1, or in_channel == out_channel == group for depthwise */
  int32_t act_type;
  double in_scale;
  int32_t in_zp;
  double out_scale;
  int32_t out_zp;
  int32_t filter_quant_num;    /* 1 or out_channel */
  const double *filter_scales;
  const int32_t *filter_zps;
  int32_t flags; /* 0 or MI_CONV_3X3_EXACT */
} mi_conv_desc;

/* weight_host: [OC][KH][KW][IC] for group 1, [C][KH][KW] for depthwise; bias_host int32 [OC] or NULL. */
int mi_conv_create(const mi_conv_desc *desc, const int8_t *weight_host, const int32_t *bias_host, mi_conv **out);
/* Output spatial size for an input of in_h x in_w with the descriptor's explicit padding. */
int mi_conv_out_shape(const mi_conv *h, int32_t in_h, int32_t in_w, int32_t *out_h, int32_t *out_w);
/* SAME-mode padding as Lite's shape inference computes it (NN/infer/conv2d_infer.c:34-50). */
int mi_conv_same_pad(int32_t in, int32_t kernel, int32_t stride, int32_t dilation, int32_t *pad_before,
                     int32_t *pad_after, int32_t *out);
/* in_dev: int8 NHWC [batch,in_h,in_w,IC]; out_dev: int8 NHWC [batch,out_h,out_w,OC]. */
int mi_conv_run(mi_conv *h, const int8_t *in_dev, int32_t batch, int32_t in_h, int32_t in_w, int8_t *out_dev,
                void *stream);
int mi_conv_run_host(mi_conv *h, const int8_t *in_host, int32_t batch, int32_t in_h, int32_t in_w, int8_t *out_host);
/* Sizes the handle's workspaces (im2col buffer, padded rows / output, where the shape needs them) for this input
 * geometry, so that later runs of it allocate nothing: the role of ConvolutionInt8CPUKernel::InitTmpBuffer
 * (LK/int8/convolution_int8.cc:159-197). */
int mi_conv_reserve(mi_conv *h, int32_t batch, int32_t in_h, int32_t in_w);
void mi_conv_destroy(mi_conv *h);

/* ---- DynamicQuant (fp32 -> int8, per tensor) --------------------------------------------------------------- */
/* Replaces DynamicQuantCPUKernel for axis_num_ == 0 (LK/int8/dynamic_quant.cc: CalculateMinMax :118-143,
 * CalculatePerlayerScaleZp :156-186, QuantData :220-234, Run :288-366) and CalculateMinMaxFp32
 * (NN/int8/dynamic_quant_int8.c:19-27), DoQuantizeFp32ToInt8 (NN/int8/quant_dtype_cast_int8.c:180-203). */
typedef struct mi_dynquant mi_dynquant;

/* The {scale, zero point} a run produced, as it lives in device memory for chaining into mi_dynmm_run_chained. */
typedef struct mi_dq_params {
  double scale;  /* what DynamicQuant publishes on the output tensor (LiteQuantParam.scale) */
  float scale_f; /* the same narrowed to float, as both consumers use it */
  int32_t zero_point;
  float real_min, real_max;
} mi_dq_params;

int mi_dynquant_create(int32_t symmetric, mi_dynquant **out);
/* x_dev: fp32 [n]; q_dev: int8 [n].  Asynchronous; the parameters stay on the device. */
int mi_dynquant_run(mi_dynquant *h, const float *x_dev, int64_t n, int8_t *q_dev, void *stream);
/* Waits for the last run on `stream` and returns its parameters (what the provider writes with SetQuantParams). */
int mi_dynquant_get_params(mi_dynquant *h, void *stream, mi_dq_params *params_host);
/* Device address of the mi_dq_params block of the last run. */
const mi_dq_params *mi_dynquant_device_params(const mi_dynquant *h);
int mi_dynquant_run_host(mi_dynquant *h, const float *x_host, int64_t n, int8_t *q_host, mi_dq_params *params_host);
/* DynamicQuant with preferred axes (per-channel activation scales; replaces the axis_num_ != 0 branch of
 * DynamicQuantCPUKernel: ReSize LK/int8/dynamic_quant.cc:59-94, CalculateMinMax :118-143,
 * CalculatePerChannelScaleZp :188-218, QuantData :236-246).  The tensor is given in the layout the reference works
 * on after moving the preferred axes to the front: `segments` contiguous runs of `unit` elements, one
 * {scale, zero point} each; for a MatMul activation [.., rows, K] that is the tensor as it stands (segments = rows,
 * unit = K, insert_quant_node_manager.cc:138-160).  Layouts that need the transposition stay with the builtin kernel.
 * params_dev / params_host: `segments` entries. */
int mi_dynquant_run_segments(mi_dynquant *h, const float *x_dev, int64_t segments, int64_t unit, int8_t *q_dev,
                             mi_dq_params *params_dev, void *stream);
int mi_dynquant_run_segments_host(mi_dynquant *h, const float *x_host, int64_t segments, int64_t unit,
                                  int8_t *q_host, mi_dq_params *params_host);
void mi_dynquant_destroy(mi_dynquant *h);

/* ---- dynamic-quant MatMul (int8 x int8 -> fp32) -------------------------------------------------------------- */
/* Replaces MatmulDynamicInt8CPUKernel (LK/int8/matmul_dynamic_int8.cc: RunImpl :40-65, Run :86-147), its base
 * (LK/int8/matmul_dynamic_base_int8.cc: InitFilterQuantParam :66-110, InitInputQuantParam :146-176, TransferB
 * :178-202) and DynamicMatmul4x16x4AIWI / CalcWeightSums (NN/int8/dynamic_matmul_int8.c:99-143,380-399). */
typedef struct mi_dynmm mi_dynmm;

typedef struct mi_dynmm_desc {
  int32_t deep, col;
  int32_t b_transpose;
  int32_t act_type;
  int32_t filter_quant_num; /* 1 or col; the zero point used is always filter_zps[0] (matmul_dynamic_int8.cc:52) */
  const double *filter_scales;
  const int32_t *filter_zps;
  int32_t flags;               /* 0 or MI_DYNMM_WEIGHT_PACKED_SDOT | MI_DYNMM_NO_DECODE_PACK */
  const int32_t *weight_sums;  /* with MI_DYNMM_WEIGHT_PACKED_SDOT: the model's weight-sums tensor
                                  [round_up(col, 16)], or NULL to have the sums computed from the weight */
} mi_dynmm_desc;

/* The weight arrives as a model converted with `cpu_option = ARM64_SIMD_DOT` stores it: packed offline for
 * MatMulDynamicSdotInt8Kernel by RowMajor2Row4x16MajorInt8 (transpose_b) or RowMajor2Col4x16MajorInt8 (NN/int8/
 * matmul_int8.c:143-156,770-784; LK/int8/matmul_dynamic_sdot_int8.cc:197-201) -- both produce the same bytes,
 * [round_up(col, 16) / 16][round_up(deep, 4) / 4][16 channels][4 K-bytes], zero padded -- together with a tensor of
 * per-channel weight sums (mindspore/lite/tools/converter/converter_packed_node.cc:47-70,129-141).  The reference
 * takes both as they are (weight_is_packed_, LK/int8/matmul_dynamic_base_int8.cc:178-184,439-443); this library
 * unpacks the weight once in mi_dynmm_create, on the host (the inverse that MatmulDynamicSdotInt8Unpack computes,
 * mindspore/lite/src/litert/runtime_packed_node_pass.cc:158-192), repacks it into its own layout and uses the given
 * sums.  b_transpose is ignored with this flag. */
#define MI_DYNMM_WEIGHT_PACKED_SDOT 1
/* Like mi_matmul, a dynamic MatMul handle holds a second, blocked form of its weights (deep x col bytes more) that
 * serves 1..64 activation rows (decode) with the matrix-core weight-streaming kernel; MI_DYNMM_NO_DECODE_PACK skips it
 * for handles that will only see larger row counts (few rows then run on the GEMM tiles, same results). */
#define MI_DYNMM_NO_DECODE_PACK 2
/* The unpacking by itself (host arithmetic, no GPU needed): packed -> weight_nk [col][deep] row-major. */
int mi_unpack_weight_4x16(const int8_t *packed, int32_t col, int32_t deep, int8_t *weight_nk);

/* bias_host: fp32 [col] or NULL */
int mi_dynmm_create(const mi_dynmm_desc *desc, const int8_t *weight_host, const float *bias_host, mi_dynmm **out);
/* Input scale / zero point given by value (read from the input tensor's quant params at every Run). */
int mi_dynmm_run(mi_dynmm *h, const int8_t *a_dev, int32_t rows, double in_scale, int32_t in_zp, float *c_dev,
                 void *stream);
/* Input scale / zero point read on the device from the block a preceding mi_dynquant_run wrote. */
int mi_dynmm_run_chained(mi_dynmm *h, const int8_t *a_dev, int32_t rows, const mi_dq_params *params_dev,
                         float *c_dev, void *stream);
int mi_dynmm_run_host(mi_dynmm *h, const int8_t *a_host, int32_t rows, double in_scale, int32_t in_zp,
                      float *c_host);
/* One input scale per row (input_per_channel_, LK/int8/matmul_dynamic_base_int8.cc:152-171; NN/int8/
 * dynamic_matmul_int8.c:126-128): row r uses row_params_dev[r].scale_f; the zero point is that of the first row
 * (LK/int8/matmul_dynamic_int8.cc:61), as in the reference, whose converter only produces symmetric per-row
 * quantisation.  row_params_dev is what mi_dynquant_run_segments wrote. */
int mi_dynmm_run_rows(mi_dynmm *h, const int8_t *a_dev, int32_t rows, const mi_dq_params *row_params_dev,
                      float *c_dev, void *stream);
/* Dynamic MatMuls that read the same activation rows (q / k / v, gate / up of a dynamic-quant transformer), as
 * mi_matmul_run_group does for the full-quant MatMul: up to four handles with the same deep at up to 32 rows run as
 * one launch, anything else member by member.  The input's scale and zero point come by value (params_dev NULL), from
 * the block a DynamicQuant run left on the device (params_dev, per_row 0) or as one scale per row (per_row 1);
 * member i writes c_dev[i], fp32 [rows, col_i].  No counterpart in the reference, which runs one node at a time. */
int mi_dynmm_run_group(mi_dynmm *const *handles, int32_t count, const int8_t *a_dev, int32_t rows, double in_scale,
                       int32_t in_zp, const mi_dq_params *params_dev, int32_t per_row, float *const *c_dev,
                       void *stream);
int mi_dynmm_run_rows_host(mi_dynmm *h, const int8_t *a_host, int32_t rows, const double *in_scales, int32_t in_zp,
                           float *c_host);
/* As mi_matmul_reserve (the buffers of MatmulDynamicBaseInt8CPUKernel::ReSize, LK/int8/matmul_dynamic_base_int8.cc:
 * 204-232). */
int mi_dynmm_reserve(mi_dynmm *h, int32_t max_rows);
void mi_dynmm_destroy(mi_dynmm *h);

/* ---- shape inference (host arithmetic, no GPU needed) --------------------------------------------------------------
 * What a provider's kernel::KernelInterface::Infer (mindspore/lite/include/kernel_interface.h:42-59) computes for the
 * operators of this path; Lite calls it in place of its builtin inference when one is registered
 * (mindspore/lite/src/litert/infer_manager.cc:90-145).  Shapes are int32 arrays of at most MI_MAX_DIMS entries;
 * out_shape must have room for MI_MAX_DIMS.  MI_INFER_INVALID when any input dimension is negative (the reference's
 * InferFlag, NN/infer/common_infer.c:274-295), MI_INFER_ERR when the shapes do not fit, as Lite maps every other nnacl
 * error (infer_manager.cc:147-160).  DynamicQuant needs no entry point: its output has the input's shape
 * (NN/infer/dynamic_quant_infer.c:21-40). */
#define MI_MAX_DIMS 8

/* MatMulFusion.  Replaces MatmulInferShape / SetShape / CheckMatmulInputShape, NN/infer/matmul_infer.c:23-124: the
 * shorter shape is left-padded with 1s, a pair of 1-D operands is treated as [1,K]x[K,1] and collapses to a scalar
 * (out_dims 0), leading dimensions broadcast when one divides the other.  bias_dims 0 = no bias tensor. */
int mi_infer_matmul(const int32_t *a_shape, int32_t a_dims, const int32_t *b_shape, int32_t b_dims,
                    const int32_t *bias_shape, int32_t bias_dims, int32_t transpose_a, int32_t transpose_b,
                    int32_t *out_shape, int32_t *out_dims);
/* FullConnection.  Replaces FullConnectionInferShape, NN/infer/full_connection_infer.c:20-89.  w_shape is [N, K];
 * bias_dims 0 = no bias tensor, which must agree with has_bias; with use_axis the input's dimensions from `axis` on
 * are folded into K and the output keeps the leading ones, otherwise the output is [elements / K, N]. */
int mi_infer_fullconnection(const int32_t *a_shape, int32_t a_dims, const int32_t *w_shape, int32_t w_dims,
                            const int32_t *bias_shape, int32_t bias_dims, int32_t has_bias, int32_t use_axis,
                            int32_t axis, int32_t *out_shape, int32_t *out_dims);

#define MI_PAD_EXPLICIT 0 /* schema PadMode PAD */
#define MI_PAD_SAME 1
#define MI_PAD_VALID 2
typedef struct mi_conv_infer {
  int32_t kernel_h, kernel_w; /* -1: taken from the weight shape */
  int32_t stride_h, stride_w, dilation_h, dilation_w;
  int32_t pad_mode;
  int32_t pad_u, pad_d, pad_l, pad_r; /* in: explicit padding; out: what SAME mode derived */
  int32_t group;                      /* 0: taken from the weight shape (depthwise) */
} mi_conv_infer;
/* Conv2DFusion on an NHWC input [N,H,W,C] and a weight [OC,KH,KW,IC].  Replaces Conv2dInferShape / ConvInferShape /
 * CheckConvAttr, NN/infer/conv2d_infer.c:20-166, including the float ceil of VALID mode and the clamp of a negative
 * output extent to 1.  Updates p (kernel size, group, SAME-mode pads) as the reference updates its ConvParameter. */
int mi_infer_conv2d(const int32_t *in_shape, int32_t in_dims, const int32_t *w_shape, int32_t w_dims,
                    mi_conv_infer *p, int32_t *out_shape, int32_t *out_dims);

/* ---- device memory for tensors that stay on the GPU between provider kernels ------------------------------------------
 * What a provider needs to keep an activation in HBM from one of its kernels to the next and publish the address on
 * the tensor with MSTensor::SetDeviceData (include/api/types.h:295-305; the consumer reads it with GetDeviceData):
 * the role a device Allocator's Malloc / Free (include/api/allocator.h:33,48) and the OpenCL kernels' host<->device
 * copies play in the reference.  Copies are ordered on `stream` like the *_run entry points and return when they
 * are complete (the host buffer may be reused at once).  All of them act on the device given to mi_init. */
int mi_device_malloc(size_t bytes, void **out_dev);
/* Page-locked host memory, which the GPU copies from and to directly: what a host-side Allocator for the device info
 * (Allocator::Malloc / Free, include/api/allocator.h:33,48; DeviceInfoContext::SetAllocator, include/api/context.h:217)
 * hands to tensors so that graph inputs and outputs cross PCIe without a bounce buffer.
 * mindspore_amd/provider/mi355x_allocator.h builds such an allocator on these two. */
int mi_host_malloc(size_t bytes, void **out_host);
int mi_host_free(void *host); /* NULL is allowed */
int mi_device_free(void *dev); /* NULL is allowed */
int mi_copy_to_device(void *dst_dev, const void *src_host, size_t bytes, void *stream);
int mi_copy_to_host(void *dst_host, const void *src_dev, size_t bytes, void *stream);
/* The same copy without the wait: it is ordered on `stream` and complete once something has waited for the stream
 * (mi_stream_synchronize, a later mi_copy_to_host).  dst_host should be page-locked memory from mi_host_malloc;
 * into ordinary memory the runtime may make the call wait after all. */
int mi_copy_to_host_async(void *dst_host, const void *src_dev, size_t bytes, void *stream);
int mi_stream_synchronize(void *stream);
/* A HIP stream of the library's device (default priority, not ordered against the null stream) and its release.  A
 * provider gives every session (every mindspore::Context it is handed) a stream of its own and passes it to all run
 * and copy calls of that session, so that sessions running on different threads do not wait for one another: the
 * part of the reference this stands for is the per-kernel thread-pool context each kernel executes under
 * (mindspore/lite/src/executor/sub_graph_kernel.cc:456-466, InnerContext::thread_pool_). */
int mi_stream_create(void **out_stream);
int mi_stream_destroy(void *stream); /* NULL is allowed */

#ifdef __cplusplus
}
#endif
#endif /* MI355X_INT8_H_ */
