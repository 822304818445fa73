/*
 * itexhip.h - C ABI of the MI355X (gfx950) kernels behind ITEX's INT8 quantized-inference ops.
 *
 * Every entry point takes plain device pointers, sizes, POD parameter structs and a HIP stream
 * (passed as void*, i.e. a hipStream_t; NULL = the default stream), enqueues its work on that
 * stream and returns without synchronising.  Return value: 0 on success, otherwise one of the
 * ITEXHIP_* codes below (the values are TF_Code values so that the op kernels can forward them);
 * itexhip_last_error() returns a thread-local message for the last failure.
 *
 * These functions sit where the reference calls oneDNN primitives; each declaration cites the
 * reference call site it replaces (paths relative to the reference tree).  The host-side parameter
 * math (ranges -> scale / zero point / shift) stays in the op kernels, as in the reference.
 */
#ifndef ITEXHIP_H_
#define ITEXHIP_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* status codes (subset of TF_Code) */
enum {
  ITEXHIP_OK = 0,
  ITEXHIP_INVALID_ARGUMENT = 3,
  ITEXHIP_UNIMPLEMENTED = 12,
  ITEXHIP_INTERNAL = 13
};

/* element types, numbered like TF_DataType */
enum {
  ITEXHIP_FLOAT = 1,
  ITEXHIP_INT32 = 3,
  ITEXHIP_QINT8 = 11,
  ITEXHIP_QUINT8 = 12,
  ITEXHIP_QINT32 = 13,
  ITEXHIP_BFLOAT16 = 14,
  ITEXHIP_HALF = 19
};

/* QuantizeMode, numbered like itex/core/utils/quantization_util.h:29-33 */
enum { ITEXHIP_MIN_COMBINED = 0, ITEXHIP_MIN_FIRST = 1, ITEXHIP_SCALED = 2,
       /* itexhip_quantize_dynamic{,_rows} only: MIN_FIRST with classic_asymmetric_algorithm (scale and rounded zero point) */
       ITEXHIP_MIN_FIRST_CLASSIC = 3 };

const char* itexhip_last_error(void);
/* "gfx950" and the library version; no GPU call. */
const char* itexhip_build_info(void);
/* Test hook (no counterpart in the reference): forces the tile shape of the MatMul tile kernel (0..4 = 256x256,
 * 256x192, 256x128, 128x128, 64x64) and of the implicit-GEMM Conv2D (0..2 = 256x128, 128x128, 64x64) for every later
 * call of the process; -1 gives the choice back to the library.  Results do not depend on the shape. */
void itexhip_test_force_tile_shape(int matmul_shape, int conv_shape);

/* ------------------------------------------------------------------------------------------
 * Stream-ordered host-to-device copy of small parameter vectors (per-channel ranges, per-axis
 * scales), and a stream wait for the synchronous-execution debug mode.  They stand where the
 * reference uses the device stream's memcpy().wait() (itex/core/kernels/common/host_data_cache.h:
 * 84-88) and ITEX_SYNC_EXEC (itex/core/utils/op_kernel.h:869-905).  The host buffer must stay valid
 * until the copy has executed; pageable memory is staged by the runtime before the call returns.
 * ---------------------------------------------------------------------------------------- */
int itexhip_memcpy_h2d_async(void* dst_device, const void* src_host, size_t bytes, void* stream);
/* device-to-host copy ordered after the work already on `stream`; returns when the data has arrived */
int itexhip_memcpy_d2h(void* dst_host, const void* src_device, size_t bytes, void* stream);
int itexhip_stream_synchronize(void* stream);
/* device-to-device copy as a kernel on `stream` (16 B per lane, any alignment and size); it stands
 * where the reference's stream copies device buffers (itex/core/devices/gpu/gpu_device_plugin.cc:
 * 251-281, gpu_memcpy_dtod) and is the kernel of known traffic that calibrates the HBM counters */
int itexhip_memcpy_d2d_async(void* dst_device, const void* src_device, size_t bytes, void* stream);

/* ------------------------------------------------------------------------------------------
 * Device runtime: what a StreamExecutor device plugin needs from HIP.  They stand where the reference
 * calls its SYCL runtime wrappers ITEX_GPU* (itex/core/devices/gpu/gpu_device_plugin.cc:27-376:
 * device count / handles :27-42, raw allocation under its BFC allocator :57-83, pinned host memory
 * :85-97, streams :121-150, events :159-207, copies :233-297, synchronisation :299-316, fills :318-342,
 * host callbacks :344-360).  Streams are created at the default priority.  Fills are kernels, so they
 * can be captured into HIP graphs.
 * ---------------------------------------------------------------------------------------- */
int itexhip_device_count(int* count);
int itexhip_device_info(int device, char* name, size_t name_len, char* pci_bus_id, size_t pci_len,
                        int64_t* total_memory, int* compute_units);
int itexhip_mem_info(int device, int64_t* free_bytes, int64_t* total_bytes);
int itexhip_malloc(int device, size_t bytes, void** ptr);
int itexhip_free(int device, void* ptr);
int itexhip_host_malloc(size_t bytes, void** ptr); /* pinned */
int itexhip_host_free(void* ptr);
int itexhip_stream_create(int device, void** stream);
int itexhip_stream_destroy(void* stream);
int itexhip_stream_query(void* stream, int* done);
int itexhip_event_create(int device, void** event);
int itexhip_event_destroy(void* event);
int itexhip_event_record(void* event, void* stream);
int itexhip_event_query(void* event, int* done);
int itexhip_event_synchronize(void* event);
int itexhip_stream_wait_event(void* stream, void* event);
int itexhip_device_synchronize(int device);
int itexhip_memcpy_d2h_async(void* dst_host, const void* src_device, size_t bytes, void* stream);
int itexhip_memset8_async(void* dst, uint8_t pattern, size_t bytes, void* stream);
int itexhip_memset32_async(void* dst, uint32_t pattern, size_t bytes, void* stream);
int itexhip_launch_host_func(void* stream, void (*fn)(void*), void* arg);

/* ------------------------------------------------------------------------------------------
 * QuantizeV2.  q[i] = sat_T(rne(fl(x[i] * scale) + addend))
 *   SCALED            : addend = 0            (oneDNN reorder, src scale;
 *                                              itex/core/kernels/common/quantize_op.h:256-275,394)
 *   classic MIN_FIRST : addend = (float)zp    (reorder, src scale + dst zero point; :276-291)
 *   legacy MIN_FIRST  : addend = fl(shift * scale), shift = -min'  (binary_add with both sources
 *                                              scaled; :292-314, 383-391)
 * dst_type is ITEXHIP_QINT8 or ITEXHIP_QUINT8.  The per-axis form views the tensor as
 * [outer, slices, inner] and reads scale[s] / addend[s] from device vectors (addend may be NULL).
 * ---------------------------------------------------------------------------------------- */
int itexhip_quantize(const float* x, void* q, int64_t n, int dst_type, float scale, float addend,
                     void* stream);
int itexhip_quantize_axis(const float* x, void* q, int64_t outer, int64_t slices, int64_t inner,
                          int dst_type, const float* scales, const float* addends, void* stream);

/* ------------------------------------------------------------------------------------------
 * Dequantize.  y[i] = ((float)q[i] - zero_point) * scale
 * (oneDNN reorder with src scale and src zero point;
 *  itex/core/kernels/common/dequantize_op.h:129-145,169).  src_type QINT8 or QUINT8.
 * ---------------------------------------------------------------------------------------- */
int itexhip_dequantize(const void* q, float* y, int64_t n, int src_type, float scale,
                       int32_t zero_point, void* stream);
int itexhip_dequantize_axis(const void* q, float* y, int64_t outer, int64_t slices, int64_t inner,
                            int src_type, const float* scales, const int32_t* zero_points,
                            void* stream);

/* 16-bit floating point ends of the two ops: QuantizeV2 from a bfloat16 tensor (_ITEXQuantizeV2 with
 * dtype = bfloat16, itex/core/kernels/gpu/quantize_op.cc:38-51) and Dequantize to bfloat16 or half
 * (itex/core/kernels/gpu/dequantize_op.cc:24-48).  Same arithmetic in fp32: the bfloat16 source is
 * widened exactly, the 16-bit result is the fp32 value rounded to nearest even. */
int itexhip_quantize_bf16(const void* x, void* q, int64_t n, int dst_type, float scale, float addend,
                          void* stream);
int itexhip_quantize_axis_bf16(const void* x, void* q, int64_t outer, int64_t slices, int64_t inner,
                               int dst_type, const float* scales, const float* addends, void* stream);
int itexhip_dequantize16(const void* q, void* y, int64_t n, int src_type, int y_type, float scale,
                         int32_t zero_point, void* stream);
int itexhip_dequantize_axis16(const void* q, void* y, int64_t outer, int64_t slices, int64_t inner,
                              int src_type, int y_type, const float* scales, const int32_t* zero_points,
                              void* stream);

/* ------------------------------------------------------------------------------------------
 * RequantizePerChannel.  q[r, c] = sat_T(rne((float)x[r, c] * scale[c])), channel = last dim
 * (oneDNN reorder s32 -> s8/u8 with per-channel src scale;
 *  itex/core/kernels/onednn/block/requantize_per_channel_op.cc:97-140).
 * `scales` is a device vector of `depth` floats; depth == 1 is the per-tensor case.
 * ---------------------------------------------------------------------------------------- */
int itexhip_requantize_per_channel(const int32_t* x, void* q, int64_t rows, int64_t depth,
                                   int dst_type, const float* scales, void* stream);
/* per-tensor form with the scale passed by value */
int itexhip_requantize(const int32_t* x, void* q, int64_t n, int dst_type, float scale,
                       void* stream);

/* ------------------------------------------------------------------------------------------
 * RequantizationRangePerChannel reduction: per channel c (last dim) the minimum and maximum of
 * x[:, c] (Eigen reductions at
 * itex/core/kernels/onednn/block/requantization_range_per_channel_op.cc:110-127).
 * min_out / max_out are device vectors of `depth` int32.  The float range itself is scalar host
 * math on these 2*depth integers and stays in the op kernel.
 * itexhip_minmax_f32 is the fp32 counterpart (2 floats: min, max) for computing QuantizeV2 ranges
 * on the device; NaNs are ignored.
 * ---------------------------------------------------------------------------------------- */
int itexhip_minmax_i32_per_channel(const int32_t* x, int64_t rows, int64_t depth, int32_t* min_out,
                                   int32_t* max_out, void* stream);
int itexhip_minmax_f32(const float* x, int64_t n, float* minmax_out, void* stream);

/* QuantizeV2 of a float tensor with the tensor's own range, nothing crossing to the host: the range reduction, the
 * op's parameter math (range adjustment quantize_op.h:130-152; SCALED scale quantization_util.h:54-84; legacy
 * MIN_FIRST scale quantize_op.h:204-214 — per tensor, the same fp32 / fp64 operations as the host code) in a one-thread
 * kernel, and the quantization reading scale and addend from device memory.  mode: ITEXHIP_SCALED (qint8 / quint8) or
 * ITEXHIP_MIN_FIRST (quint8, the non-classic algorithm) or ITEXHIP_MIN_FIRST_CLASSIC (the zero-point form,
 * quantization_util.h:54-84).  `state` is a device array of ITEXHIP_DYNAMIC_STATE_FLOATS floats (the first 8 carry
 * results, the rest is room for the partial ranges of the reduction's workgroups):
 * [0..1] the tensor's min and max, [2..3] the op's output_min / output_max (what a consuming MatMul takes as
 * min_a / max_a: pass state + 2 to itexhip_qmatmul_device_range), [4..5] scale and addend.  n > 0.  The reference
 * (Up to 128 K elements, 16-byte aligned, n a multiple of 4: all three steps in one launch; larger aligned tensors:
 * two launches.)  The reference
 * has no such op (its QuantizeV2 takes the range from the host); this is the producer half of the
 * Min/Max -> QuantizeV2 -> MatMul fusion of this plugin's graph pass. */
#define ITEXHIP_DYNAMIC_STATE_FLOATS 1032
int itexhip_quantize_dynamic(const float* x, void* q, int64_t n, int dst_type, int mode, float ensure_minimum_range,
                             float* state, void* stream);
/* The per-row (per-token) form: row m of x [rows, cols] is quantized against its own range (QuantizeV2 with axis = 0 and
 * the rows' min / max as ranges, quantize_op.h:166-190, same parameter math per row), one workgroup per row, one launch;
 * row_min_out / row_max_out (device arrays of `rows` floats) receive the rows' output_min / output_max, which is what
 * itexhip_qmatmul_per_row takes.  cols > 0. */
int itexhip_quantize_dynamic_rows(const float* x, void* q, int64_t rows, int64_t cols, int dst_type, int mode,
                                  float ensure_minimum_range, float* row_min_out, float* row_max_out, void* stream);

/* itexhip_quantize_dynamic without a workspace argument and without any allocation.  It has no counterpart in the
 * reference; it is for callers that cannot allocate device memory around the call: code under HIP graph capture,
 * tight serving loops, harnesses that forbid allocation.  The partial ranges of the reduction (one {min, max} pair per
 * workgroup of the range pass, at most 512 pairs = 4 KiB whatever n) live in a fixed array of the library's own device
 * memory, one copy per GPU, kept until the process ends; the call itself allocates and frees nothing.  Always two
 * launches (partial ranges, then parameters + quantization).  range_out: 6 floats of device memory, filled like
 * state[0..5] of itexhip_quantize_dynamic ([0..1] the tensor's min and max, [2..3] the op's output_min / output_max,
 * [4..5] scale and addend).  4 <= n <= 2^36; x 16-byte, q 4-byte, range_out 8-byte aligned; anything else is rejected.
 * Same bytes in q and the same six floats as itexhip_quantize_dynamic.  Calls that overlap in time on one GPU (two
 * streams, two threads) share the array and race: serialise them.
 * The first call on each device looks the array's address up (hipGetDevice + hipGetSymbolAddress, which may load the
 * code object); every later call on that device only launches the two kernels.  A caller that captures the call into a
 * HIP graph therefore makes one ordinary call on that device before the capture starts.  `stream` must belong to the
 * current device, as for any kernel launch. */
int itexhip_quantize_dynamic_static(const float* x, void* q, int64_t n, int dst_type, int mode, float ensure_minimum_range,
                                    float* range_out, void* stream);

/* ------------------------------------------------------------------------------------------
 * Quantized MatMul (oneDNN inner_product_forward u8/s8 x s8 -> s32 with fused epilogue;
 * itex/core/kernels/common/quantized_matmul_common.h:223-226 (primitive), :92 (execute)).
 * ---------------------------------------------------------------------------------------- */

/* Which kernel class prepares the epilogue (quantized_matmul_common.h). */
enum {
  ITEXHIP_API_V2 = 0,     /* QuantizedFusedMatMulV2Op (:1711-1909) */
  ITEXHIP_API_V1 = 1,     /* QuantizedFusedMatMulOp   (:1539-1708) */
  ITEXHIP_API_LEGACY = 2  /* QuantizedMatMulOp / QuantizedMatMulReluOp (:1412-1531) */
};
enum { ITEXHIP_ACT_NONE = 0, ITEXHIP_ACT_RELU = 1, ITEXHIP_ACT_RELU6 = 2, ITEXHIP_ACT_LEAKYRELU = 3,
       ITEXHIP_ACT_GELU_APPROX = 4, ITEXHIP_ACT_GELU_EXACT = 5,
       /* "Elu", "Sigmoid", "Tanh", "_ITEXSwish", "_ITEXMish" of the post-op table (onednn_post_op_util.cc:34-68) */
       ITEXHIP_ACT_ELU = 6, ITEXHIP_ACT_SIGMOID = 7, ITEXHIP_ACT_TANH = 8, ITEXHIP_ACT_SWISH = 9, ITEXHIP_ACT_MISH = 10 };
/* post-ops of the epilogue chain (itex/core/utils/onednn/onednn_post_op_util.cc:34-68); SUM is the
 * "Add" fusion: y += alpha * addend[m, n] */
enum { ITEXHIP_ELT_RELU = 1, ITEXHIP_ELT_CLIP = 2, ITEXHIP_ELT_LINEAR = 3, ITEXHIP_ELT_GELU_TANH = 4,
       ITEXHIP_ELT_GELU_ERF = 5, ITEXHIP_ELT_SUM = 6,
       /* oneDNN eltwise_elu (x > 0 ? x : alpha (e^x - 1)), eltwise_logistic (1 / (1 + e^-x)), eltwise_tanh,
        * eltwise_swish (x / (1 + e^(-alpha x))), eltwise_mish (x tanh(ln(1 + e^x))) */
       ITEXHIP_ELT_ELU = 7, ITEXHIP_ELT_LOGISTIC = 8, ITEXHIP_ELT_TANH = 9, ITEXHIP_ELT_SWISH = 10, ITEXHIP_ELT_MISH = 11 };

typedef struct {
  int alg;      /* ITEXHIP_ELT_* */
  float alpha;
  float beta;
} itexhip_eltwise;

/* What the fused epilogue applies after the integer accumulation:
 *   y = fl(fl((float)acc * scale[n]) + bias[n]); eltwise chain; convert to the output type. */
typedef struct {
  int n_scales;   /* 0: no scale, 1: scales[0] for all channels, N: per output channel */
  int n_eltwise;  /* 0..3, in fused_ops order */
  itexhip_eltwise elt[3];
} itexhip_epilogue;

/* Attributes and host-memory scalars of one quantized MatMul node. */
typedef struct {
  int api;             /* ITEXHIP_API_* */
  int t_in;            /* T1: QUINT8 | QINT8 */
  int t_out;           /* QINT32 | QINT8 | QUINT8 | FLOAT | BFLOAT16 | HALF (the fp32 result rounded to nearest even) */
  int input_mode;      /* input_quant_mode: MIN_FIRST | SCALED */
  int out_min_first;   /* V2: output_quant_mode == "MIN_FIRST" */
  int activation;      /* ITEXHIP_ACT_* */
  int has_requantize;  /* V2: "Requantize" in fused_ops */
  int has_dequantize;  /* V2: "Dequantize" in fused_ops */
  int n_fused_ops;     /* V1: fused_ops.size() */
  float leakyrelu_alpha;
  float min_a, max_a;      /* host scalars */
  float min_out, max_out;  /* min/max_freezed_output (requantize) */
  int add_position;        /* "Add" in fused_ops: 0 absent, 1 before the activation, 2 after it (fp32 output only) */
  int t_bias;              /* Tbias: 0 or ITEXHIP_FLOAT = fp32, ITEXHIP_QINT32 = qint32 (:1153-1334),
                            * ITEXHIP_BFLOAT16 / ITEXHIP_HALF = 16-bit patterns; the adjusted bias is rounded to
                            * that type again, as GetScaledBias stores it in Tbias (:578-599, 609-617) */
} itexhip_matmul_params;

/* Host-only: the epilogue descriptor (scale count, eltwise chain with the reference's alpha/beta
 * overrides) for a node; follows ExtendInt8PostOps (quantized_matmul_common.h:1472-1508,
 * 1610-1702, 1809-1908) and PostOpUtil::SetPostOp
 * (itex/core/utils/onednn/onednn_post_op_util.cc:237-273).  nb = number of weight ranges. */
int itexhip_qmatmul_epilogue_desc(const itexhip_matmul_params* p, int64_t nb, itexhip_epilogue* ep);

/* Device: per-channel output scales and the scaled / zero-point-compensated bias
 * (ExtendInt8PostOps as above; GetScaledBias, quantized_matmul_common.h:466-660), computed by one
 * small kernel from device copies of min_b / max_b (nb floats each), the bias (N floats; N int32 when p->t_bias is QINT32, N uint16 when BFLOAT16 / HALF) and
 * the weight column sums (N int32, from itexhip_qgemm_prepack_b).  Writes `scales_out`
 * (max(ep.n_scales,1) floats) and `bias_out` (N floats).  No host synchronisation. */
int itexhip_qmatmul_prepare(const itexhip_matmul_params* p, const float* min_b, const float* max_b,
                            int64_t nb, const void* bias, const int32_t* colsum, int64_t N,
                            float* scales_out, float* bias_out, void* stream);

/* Weight prepack: the s8 weight (TF layout [K,N] row-major, or [N,K] when transpose_b) is
 * rearranged into MFMA operand chunks (32 output channels x 32 k per 1 KiB chunk, ordered
 * [N/32][K/32], K zero-padded to a multiple of 64) and
 * its column sums over k are written to colsum[N].  This replaces the reference's cached weight
 * reorder (quantized_matmul_common.h:238-275) and its host-side column-sum loop (:569-573).
 * `packed` must hold itexhip_qgemm_packed_bytes(K, N) bytes. */
int64_t itexhip_qgemm_packed_bytes(int64_t K, int64_t N);
int itexhip_qgemm_prepack_b(const int8_t* w, int transpose_b, int64_t K, int64_t N, int8_t* packed,
                            int32_t* colsum, void* stream);

/* out[M,N] = epilogue( a[M,K] (u8 or s8, row-major) x packed weight ), exact int32 accumulation.
 * a_type QUINT8 | QINT8; out_type QINT32 | QINT8 | QUINT8 | FLOAT | BFLOAT16 | HALF.  `colsum` is needed for QUINT8
 * activations (they are fed to the signed MFMA as a-128 and corrected by 128*colsum[n]).
 * `scales` has ep->n_scales floats (may be NULL when 0), `bias` N floats (NULL = no bias add).
 * Dispatches to the bandwidth-bound small-M kernel (M <= 32; up to 128 rows when the weight is small or the tile
 * kernel would leave most CUs idle) and to the MFMA tile kernel otherwise; both give the same bytes.  The two
 * explicit entry points below force one path (itexhip_qgemv: M <= 128). */
int itexhip_qgemm(const void* a, int a_type, const int8_t* packed_b, const int32_t* colsum,
                  int64_t M, int64_t K, int64_t N, const float* scales, const float* bias,
                  const itexhip_epilogue* ep, int out_type, void* out, void* stream);
int itexhip_qgemm_tile(const void* a, int a_type, const int8_t* packed_b, const int32_t* colsum,
                       int64_t M, int64_t K, int64_t N, const float* scales, const float* bias,
                       const itexhip_epilogue* ep, int out_type, void* out, void* stream);
int itexhip_qgemv(const void* a, int a_type, const int8_t* packed_b, const int32_t* colsum,
                  int64_t M, int64_t K, int64_t N, const float* scales, const float* bias,
                  const itexhip_epilogue* ep, int out_type, void* out, void* stream);

/* itexhip_qgemm with one ITEXHIP_ELT_SUM in ep->elt: y = y + elt.alpha * addend[m, n] at that place of the chain.
 * `addend` is an [M, N] tensor of addend_type ITEXHIP_FLOAT, ITEXHIP_QINT8 or ITEXHIP_QUINT8 (the 8-bit values are
 * converted to fp32 exactly): the sum post-op of oneDNN that the reference uses for the "Add" fusion of the MatMul
 * (quantized_matmul_common.h:352-389) and the "Sum" fusions of the convolution (quantized_conv_ops.h:398-433,
 * 604-640, where the summand buffer doubles as the output).  `out` may be the addend buffer itself when both have
 * the same element size (every element is read before it is written); any other overlap is not allowed. */
int itexhip_qgemm_sum(const void* a, int a_type, const int8_t* packed_b, const int32_t* colsum,
                      int64_t M, int64_t K, int64_t N, const float* scales, const float* bias,
                      const itexhip_epilogue* ep, const void* addend, int addend_type, int out_type, void* out,
                      void* stream);

/* The whole op in one launch: as itexhip_qmatmul_prepare followed by itexhip_qgemm, but the MatMul
 * kernel derives each channel's output scale and bias itself from the op's ranges (the same fp32
 * operation sequence), so no parameter vectors and no second kernel are needed.  This is what the
 * op kernel calls per Compute (quantized_matmul_common.h:62-460: Init + primitive execute);
 * a changed min_a / max_a costs nothing extra.  `bias` is the op's raw bias (fp32; int32 when
 * p->t_bias is QINT32, 16-bit patterns when BFLOAT16 / HALF; may be null).  `addend` is the [M, N] tensor of the "Add" fusion
 * (p->add_position != 0; the reference adds it in place into the output buffer, :341-389, so it has the output's type:
 * fp32, or 16-bit patterns for a bfloat16 / half result, widened exactly before the addition), else null. */
int itexhip_qmatmul(const itexhip_matmul_params* p, const void* a, const int8_t* packed_b,
                    const int32_t* colsum, int64_t M, int64_t K, int64_t N, const float* min_b,
                    const float* max_b, int64_t nb, const void* bias, const void* addend, void* out,
                    void* stream);

/* Decode batches quantized per token: row m of `a` was quantized with its own range
 * (row_min_a[m], row_max_a[m]; device arrays of M floats, e.g. from QuantizeV2 with axis = 0,
 * quantize_op.h:166-190) and row m of the result is what itexhip_qmatmul gives for the 1 x K problem
 * with p->min_a / max_a replaced by that row's range.  The reference's MatMul ops only take a
 * per-tensor activation range (they read element 0 of min_a / max_a, quantized_matmul_common.h:95-96),
 * so this entry point is an extension; M <= 16. */
int itexhip_qmatmul_per_row(const itexhip_matmul_params* p, const void* a, const int8_t* packed_b,
                            const int32_t* colsum, int64_t M, int64_t K, int64_t N, const float* row_min_a,
                            const float* row_max_a, const float* min_b, const float* max_b, int64_t nb,
                            const void* bias, const void* addend, void* out, void* stream);

/* itexhip_qmatmul with the per-tensor activation range in device memory (range_a[0] = min_a, range_a[1] = max_a, e.g.
 * state + 2 of itexhip_quantize_dynamic enqueued earlier on the same stream) in place of p->min_a / p->max_a, which are
 * ignored: the kernels derive scales and bias from it exactly as from the host values.  Not for a qint32 result (its
 * output range, quantized_ops.h:40-54, is host math on the activation range).  An extension, as itexhip_qmatmul_per_row. */
int itexhip_qmatmul_device_range(const itexhip_matmul_params* p, const void* a, const int8_t* packed_b,
                                 const int32_t* colsum, int64_t M, int64_t K, int64_t N, const float* range_a,
                                 const float* min_b, const float* max_b, int64_t nb, const void* bias,
                                 const void* addend, void* out, void* stream);

/* itexhip_qmatmul on the unpacked TF-layout weight ([K, N], or [N, K] with transpose_b), any K, no
 * prepack and no column-sum buffer: one thread per output element.  For the shapes the MFMA kernels
 * do not take (K not a multiple of 16). */
int itexhip_qmatmul_unpacked(const itexhip_matmul_params* p, const void* a, const int8_t* w, int transpose_b,
                             int64_t M, int64_t K, int64_t N, const float* min_b, const float* max_b,
                             int64_t nb, const void* bias, const void* addend, void* out, void* stream);

/* Same contract on the unpacked TF-layout weight, any shape (no alignment requirements): one
 * thread per output element.  Used for shapes the tile kernels do not cover (K not a multiple of
 * 16) and as an on-device cross-check. */
int itexhip_qgemm_naive(const void* a, int a_type, const int8_t* w, int transpose_b, int64_t M,
                        int64_t K, int64_t N, const float* scales, const float* bias,
                        const itexhip_epilogue* ep, int out_type, void* out, void* stream);

/* ---- quantized BatchMatMul (qint8 x qint8 -> float / bfloat16 / half) --------------------------
 * The INT8 batch MatMul either side of the linears in attention blocks:
 *   _QuantizedBatchMatMul, _QuantizedBatchMatMulV2AndDequantize, _QuantizedFusedBatchMatMulV2AndDequantize
 *   (itex/core/kernels/common/batch_matmul_op.h:36-522, registered for a device in
 *   itex/core/kernels/gpu/matmul_op.cc:612-655).
 * out[b, m, n] = convert( binary_1( binary_0( float(sum_k x[b, m, k] * y[b, k, n]) * scale ) ) ):
 * exact int32 accumulation, one fp32 multiply by the output scale
 * (range_x * range_y) / (127 * 127)  (:497-515), then each fused "Mul" / "Add" as a separately rounded
 * fp32 operation with its operand broadcast to the output (oneDNN binary post-ops, :377-413), then the
 * conversion to the output type (round to nearest even). */
enum { ITEXHIP_BIN_MUL = 1, ITEXHIP_BIN_ADD = 2 };
enum { ITEXHIP_BMM_MAX_BATCH_DIMS = 4, ITEXHIP_BMM_MAX_BINARY = 2 };

typedef struct {
  int alg;                 /* ITEXHIP_BIN_MUL | ITEXHIP_BIN_ADD, applied in array order */
  const void* data;        /* device memory; elements of the OUTPUT type (:393-394 builds the operand's
                            * memory descriptor with OneDnnType<Toutput>) */
  int64_t batch_stride[ITEXHIP_BMM_MAX_BATCH_DIMS]; /* element strides per batch dim; 0 = broadcast */
  int64_t stride_m, stride_n;                       /* element strides in the matrix; 0 = broadcast */
} itexhip_bmm_binary;

typedef struct {
  int n_batch_dims;                                  /* 0..4; the output is [batch_dims..., M, N], row-major */
  int64_t batch_dims[ITEXHIP_BMM_MAX_BATCH_DIMS];
  int64_t x_batch_stride[ITEXHIP_BMM_MAX_BATCH_DIMS]; /* element strides of x per batch dim; 0 = broadcast (MatMulBCast, :105-109) */
  int64_t y_batch_stride[ITEXHIP_BMM_MAX_BATCH_DIMS];
  int64_t M, K, N;
  int adj_x, adj_y;        /* x matrices are [M, K] row-major, or [K, M] with adj_x; y [K, N], or [N, K] with adj_y */
  int out_type;            /* ITEXHIP_FLOAT | ITEXHIP_BFLOAT16 | ITEXHIP_HALF */
  float scale;             /* the output scale, computed by the caller in fp32 as written above */
  int n_binary;            /* 0..2 */
  itexhip_bmm_binary binary[ITEXHIP_BMM_MAX_BINARY];
} itexhip_bmm_params;

/* x, y, out: device memory.  Any M, K, N >= 0 and any alignment; 16-byte-aligned operands with K (and, for
 * the transposed layouts, the row length) a multiple of 16 take the vector-load path.  MFMA 32x32x32 i8,
 * tiles of 64 x 64 outputs per workgroup, 128 x 128 / 128 x 64 for calls with at least 1024 such tiles, aligned
 * operands and fused operands that do not depend on the row. */
int itexhip_qbatch_matmul(const itexhip_bmm_params* p, const int8_t* x, const int8_t* y, void* out, void* stream);

/* ---- quantized Transpose ------------------------------------------------------------------------
 * y = transpose(x, perm) for a tensor of 1-byte (qint8 / quint8) or 4-byte (qint32) elements: dimension i
 * of y is dimension perm[i] of x (_QuantizedTranspose, itex/core/kernels/common/transpose_op.h:197-236,
 * registered for a device in itex/core/kernels/gpu/transpose_op.cc:48-55; its min / max pass through on
 * the host).  rank <= 8; adjacent dimensions that stay adjacent are merged first; a permutation that keeps
 * the innermost run of at least 16 bytes moves 16-byte vectors (the [B, S, H, D] <-> [B, H, S, D] moves
 * of an attention block), any other one moves single elements. */
int itexhip_transpose(const void* x, void* y, int elem_size, int rank, const int64_t* dims, const int32_t* perm,
                      void* stream);

/* ---- quantized Conv2D --------------------------------------------------------------------------
 * The quantized convolutions (QuantizedConv2D*, _QuantizedConv2D; itex/core/kernels/common/
 * quantized_conv_ops.h:63-597 over the oneDNN convolution primitive, conv_ops.h:615-1150) run here as
 * patch matrix x prepacked filter.  The receptive field of an output position is one row of the patch matrix,
 * k = (kh * KW + kw) * C + c, which is the row order of the HWIO filter read as a [KH*KW*C, O] matrix, so
 * itexhip_qgemm_prepack_b packs the filter as it is.  itexhip_qconv2d (below) never builds the patch matrix: the
 * MatMul kernel gathers its rows from the input; itexhip_im2col8 writes it out for the shapes that kernel does
 * not take, and itexhip_qgemm does the rest.  Quantization is SCALED (zero points are 0): padding positions hold
 * the integer 0. */
typedef struct {
  int64_t batch, in_h, in_w, in_c;   /* NHWC input */
  int64_t k_h, k_w;                  /* filter window */
  int64_t out_h, out_w;              /* output extent (the caller applies the padding rule) */
  int stride_h, stride_w, dil_h, dil_w;
  int64_t pad_top, pad_left;         /* leading padding */
} itexhip_conv_geometry;
/* cols: [batch * out_h * out_w, row_bytes] bytes; row_bytes >= k_h * k_w * in_c, a multiple of 16; the tail of
 * every row is zero-filled.  1-byte elements (qint8 / quint8). */
int itexhip_im2col8(const void* x, const itexhip_conv_geometry* g, int64_t row_bytes, void* cols, void* stream);
/* Zero-padded copy of a 4-d tensor of 1-byte elements: out[n][oh][ow][oc] = x[n][oh - lead_h][ow - lead_w][oc] where
 * that element exists, else 0; out is [n, out_h, out_w, out_c] with out_h >= lead_h + h, out_w >= lead_w + w,
 * out_c >= c a multiple of 4.  What a convolution with fewer than 16 input channels (the first layer of a vision
 * network: in_c = 3) needs to run as an implicit GEMM: the NHWC input padded to 4 (or 8) channels together with the
 * window's spatial padding, and the HWIO filter (as the 4-d tensor [k_h, k_w, in_c, out_c]: n = k_h, h = k_w, w = in_c)
 * padded to the same channel count and to a window row of a multiple of 16 bytes; the padding bytes are zero on both
 * sides, so the integer sums are those of the reference's convolution (conv_ops.h:615-1150 over the oneDNN primitive,
 * which pads implicitly). */
int itexhip_pad_nhwc8(const void* x, int64_t n, int64_t h, int64_t w, int64_t c, int64_t lead_h, int64_t lead_w,
                      int64_t out_h, int64_t out_w, int64_t out_c, void* out, void* stream);
/* out[j] = float(bias[j]) * factors[n_factors == 1 ? 0 : j], j < n: the reorder with source scales that the
 * reference applies to the bias (quantized_conv_ops.h:560-590).  bias_type ITEXHIP_FLOAT or ITEXHIP_QINT32. */
int itexhip_scale_vector(const void* bias, int bias_type, const float* factors, int64_t n_factors, int64_t n,
                         float* out, void* stream);

/* Depthwise Conv2D (QuantizedDepthwiseConv2D*, _QuantizedDepthwiseConv2D; the reference runs them as a grouped oneDNN
 * convolution with one group per input channel, conv_ops.h:238-246, 395-397): `filter` is TensorFlow's
 * [k_h, k_w, in_c, multiplier] qint8 tensor as it is, output channel c * multiplier + m reads input channel c; scales
 * (0, 1 or in_c * multiplier of them), bias (fp32, may be null) and post-ops as in itexhip_qgemm, without a sum.
 * Zero points are 0 (SCALED quantization): padding contributes nothing. */
int itexhip_qdepthwise_conv2d(const void* x, int x_type, const itexhip_conv_geometry* g, int64_t multiplier,
                              const int8_t* filter, const float* scales, const float* bias,
                              const itexhip_epilogue* ep, int out_type, void* out, void* stream);

/* The convolution without the patch matrix: the MatMul tile kernel gathers its activation tiles straight from the
 * NHWC input (an implicit GEMM; it stands where the reference executes its oneDNN
 * convolution primitive, conv_ops.h:1021, 1119), same arguments otherwise as itexhip_qgemm with M = batch * out_h * out_w and
 * K = k_h * k_w * in_c; `packed_filter` / `colsum` from itexhip_qgemm_prepack_b(filter, 0, K, out_channels, ...).
 * Takes the calls for which itexhip_qconv2d_implicit_ok returns 1 (in_c a multiple of 16, or in_c 4 / 8 with no window
 * in the padding, no dilation along the row and k_w * in_c a multiple of 16; k_h * k_w * in_c <= 16384,
 * 16-byte aligned input of less than 2 GiB; output qint32 / qint8 / quint8 / float / bfloat16 with 16-byte aligned
 * rows) and rejects the others, which go through itexhip_im2col8 + itexhip_qgemm.  `bias` must not be null. */
int itexhip_qconv2d_implicit_ok(const itexhip_conv_geometry* g, const void* x, int64_t out_channels, int out_type,
                                const void* out);
int itexhip_qconv2d(const void* x, int x_type, const itexhip_conv_geometry* g, const int8_t* packed_filter,
                    const int32_t* colsum, int64_t out_channels, const float* scales, const float* bias,
                    const itexhip_epilogue* ep, int out_type, void* out, void* stream);
/* itexhip_qconv2d with one ITEXHIP_ELT_SUM in ep->elt, as itexhip_qgemm_sum: `addend` is the summand in the output's
 * layout [batch, out_h, out_w, out_channels], 4-byte (8-bit types) or 16-byte (float) aligned, out_channels a
 * multiple of 4. */
int itexhip_qconv2d_sum(const void* x, int x_type, const itexhip_conv_geometry* g, const int8_t* packed_filter,
                        const int32_t* colsum, int64_t out_channels, const float* scales, const float* bias,
                        const itexhip_epilogue* ep, const void* addend, int addend_type, int out_type, void* out,
                        void* stream);

/* Diagnostic, no counterpart in the reference: `workgroups` x 4 wavefronts each issue iters (even) x 8
 * independent 32x32x32 i8 MFMAs (2 * 32768 ops each) on the 8 KiB of operand fragments at `operands`
 * (device memory, 16-byte aligned: 4 KiB for the first MFMA operand, which the MatMul kernels use for the
 * weights and keep for 4 consecutive MFMAs, then 4 KiB for the second, the activations, changed with
 * every MFMA) and nothing else.  Timed by the caller, it gives the rate the matrix
 * cores sustain for that operand data on this device, the practical ceiling next to the published
 * peak.  `sink` takes 256 ints that are practically never written. */
int itexhip_mfma_probe(int workgroups, int iters, const void* operands, int32_t* sink, void* stream);

/* Diagnostic, no counterpart in the reference: one launch that reads `bytes` (a multiple of 16 KiB is read in full;
 * 16-byte aligned) from `src` and keeps nothing (`sink`: 256 ints, practically never written).  Timed by the caller,
 * it gives what a single launch that only streams that many bytes from HBM costs on this device: the floor next to
 * which the bandwidth-bound kernels (the decode MatMul above all) are to be read. */
int itexhip_read_probe(const void* src, size_t bytes, int32_t* sink, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* ITEXHIP_H_ */
