/*
 * CPU oracle for the INT8 quantized-inference path of intel-extension-for-tensorflow (ITEX).
 *
 * TEST INFRASTRUCTURE ONLY.  This library is a plain-C restatement of what the reference
 * computes on its CPU (oneDNN) path.  It is the checker for the HIP kernels and the timed
 * "cpu_baseline" of the benchmark; nothing in the shipped library links, loads or calls it.
 *
 * Every function cites the reference file:line it follows (paths relative to the reference
 * tree).  The arithmetic that the reference delegates to oneDNN (reorder, binary,
 * inner_product_forward; oneDNN is not vendored in the reference tree, pinned at commit
 * 242d4d9 by itex/workspace.bzl:64-75) is restated from oneDNN's documented int8 semantics:
 *   exact int32 accumulation;  y = fl(fl((float)acc * scale[oc]) + bias[oc]);
 *   eltwise post-ops in order;  saturate to the destination type;  round to nearest even.
 *
 * Parity pins (see tests/test_oracle_*.py):
 *   - QuantizeV2 / Dequantize: the reference's own golden vectors
 *     (test/tensorflow/python/kernel_tests/block_layout/quantized_ops_test.py:49-268,
 *      dequantize_op_test.py:102-170).
 *   - integer GEMM: brute force against numpy int64.
 *   - parameter math: closed forms evaluated independently in numpy float32/float64.
 *   - epilogue order (multiply, then add, separately rounded; saturate; RNE), the sum / binary-add
 *     post-op, and the bfloat16 / half destination conversion are cross-checked bit for bit against
 *     the oneDNN build bundled with PyTorch where that is importable; the GELU post-ops agree
 *     with it to 1e-6 absolute (more than 90 % of elements bit for bit).
 *   - quantized BatchMatMul: numpy int64 matmul on broadcast operands; the three cases of the
 *     reference's quantized_batch_matmul_test.py.
 * Parity unpinned (no reference-held vector and no way to execute oneDNN@242d4d9 here):
 *   NaN / Inf inputs to the quantizers; the result of the size-mismatched bias reorder in
 *   orc_qmatmul_prepare (SCALED input, per-channel weights; see the comment there);
 *   abs(INT32_MIN) in orc_requantization_range_per_channel (undefined behaviour upstream);
 *   the last bits of the GELU post-ops (oneDNN evaluates tanh / erf with its own polynomial
 *   kernels; here libm's tanhf / erff): pinned only against a float64 evaluation and at the
 *   reference tests' own tolerance.  The device evaluates the exact GELU's erf with a five-term
 *   rational-exponential form good to 1.5e-7 absolute, so it is compared with this oracle to 1e-6
 *   absolute (2e-6 relative), which near zero is many last-place units;
 *   the bfloat16 / half bias (Tbias): the adjusted bias is rounded to Tbias as the code is
 *   written (quantized_matmul_common.h:578-599, 609-617); the reference's tests only use float and
 *   qint32 biases;
 *   classic MIN_FIRST QuantizeV2 (classic_asymmetric_algorithm): orc_quantize_v2 adds the zero point in fp32 BEFORE
 *   rounding, sat(rne(fl(x * scale) + zp)), which is how a oneDNN reorder applies a destination zero point; the
 *   other reading, rne(x * scale) + zp, differs when x * scale lies just under a half and the sum rounds up to one
 *   (1.4999999 + 64 -> 65.5 -> 66 against 65).  The reference's vector [0,144,176,223,239,255] holds no such
 *   element, so it does not separate the two;
 *   legacy MIN_FIRST QuantizeV2 with an axis (per-slice ranges): the reference describes the shift operand of its
 *   binary_add as a one-element tensor (quantize_op.h:302-303, dims all 1) while handing it a shift per slice and
 *   per-axis scale masks that the oneDNN binary primitive does not take; its tests run per-axis quantization in
 *   SCALED mode only.  orc_quantize_v2 gives every slice its own shift -min'[s] and scale (the evident intent;
 *   pinned as such by tests/test_oracle_quantize.py::test_min_first_per_axis_uses_each_slices_shift);
 *   the quantized convolution's host arithmetic at the last bit and its Sum fusions (orc_qconv2d_sum): the
 *   reference's conv tests hold no vectors, see the comments at those functions.
 *   The bfloat16 / half OUTPUT is pinned: it must equal the nearest-even 16-bit
 *   value of the float output of the same node, which the tests check against PyTorch's conversion.
 */
#ifndef ITEX_ORACLE_H_
#define ITEX_ORACLE_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* TF_DataType values used at the op boundary (tensorflow/c/tf_datatype.h). */
enum { ORC_FLOAT = 1, ORC_INT32 = 3, ORC_QINT8 = 11, ORC_QUINT8 = 12, ORC_QINT32 = 13, ORC_BFLOAT16 = 14, ORC_HALF = 19 };
/* QuantizeMode, same order as itex/core/utils/quantization_util.h:29-33. */
enum { ORC_MIN_COMBINED = 0, ORC_MIN_FIRST = 1, ORC_SCALED = 2 };
/* status */
enum { ORC_OK = 0, ORC_INVALID_ARGUMENT = 3, ORC_UNIMPLEMENTED = 12 };

/* Which kernel class of quantized_matmul_common.h prepares the epilogue. */
enum {
  ORC_API_V2 = 0,     /* QuantizedFusedMatMulV2Op: _QuantizedMatMul, _ITEXQuantizedMatMul */
  ORC_API_V1 = 1,     /* QuantizedFusedMatMulOp: _QuantizedFusedMatMul{,AndRequantize,AndDequantize} */
  ORC_API_LEGACY = 2  /* QuantizedMatMulOp / QuantizedMatMulReluOp: QuantizedMatMulWithBias* */
};

/* eltwise post-op algorithms (subset of onednn_post_op_util.cc:34-68) */
enum { ORC_ELT_RELU = 1, ORC_ELT_CLIP = 2, ORC_ELT_LINEAR = 3, ORC_ELT_GELU_TANH = 4, ORC_ELT_GELU_ERF = 5,
       ORC_ELT_SUM = 6, /* the "Add" post-op: y += alpha * addend[m,n] (append_sum, :256) */
       ORC_ELT_ELU = 7, ORC_ELT_LOGISTIC = 8, ORC_ELT_TANH = 9, ORC_ELT_SWISH = 10, ORC_ELT_MISH = 11 };
/* activation names accepted in fused_ops */
enum { ORC_ACT_NONE = 0, ORC_ACT_RELU = 1, ORC_ACT_RELU6 = 2, ORC_ACT_LEAKYRELU = 3, ORC_ACT_GELU_APPROX = 4,
       ORC_ACT_GELU_EXACT = 5, ORC_ACT_ELU = 6, ORC_ACT_SIGMOID = 7, ORC_ACT_TANH = 8, ORC_ACT_SWISH = 9, ORC_ACT_MISH = 10 };

typedef struct {
  int alg;
  float alpha;
  float beta;
} orc_eltwise;

typedef struct {
  int api;               /* ORC_API_* */
  int t_in;              /* ORC_QUINT8 | ORC_QINT8 (T1) */
  int t_out;             /* ORC_QINT32 | ORC_QINT8 | ORC_QUINT8 | ORC_FLOAT | ORC_BFLOAT16 | ORC_HALF (fp32 result rounded to nearest even) */
  int input_mode;        /* ORC_MIN_FIRST | ORC_SCALED */
  int out_min_first;     /* V2 only: output_quant_mode == "MIN_FIRST" */
  int activation;        /* ORC_ACT_* fused after BiasAdd */
  int has_requantize;    /* V2: "Requantize" in fused_ops */
  int has_dequantize;    /* V2: "Dequantize" in fused_ops */
  int n_fused_ops;       /* V1: fused_ops.size() (1 = BiasAdd only, 2 = BiasAdd + activation) */
  float leakyrelu_alpha;
  int add_position;      /* "Add" in fused_ops: 0 absent, 1 before the activation, 2 after it */
  int t_bias;            /* 0 or ORC_FLOAT: fp32 bias;  ORC_QINT32: Tbias = qint32 (:1153-1334);  ORC_BFLOAT16 / ORC_HALF: uint16 bit patterns */
} orc_matmul_attrs;

typedef struct {
  int n_scales;          /* 0 (no output scale), 1 (per tensor) or N (per output channel) */
  int n_eltwise;         /* 0..3, post-ops in fused_ops order */
  orc_eltwise elt[3];
} orc_epilogue_desc;

int orc_adjust_input_range(float in_min, float in_max, float ensure_minimum_range,
                           float* adj_min, float* adj_max);
int orc_scale_zeropoint_align(int T, int mode, int dequantize, float* min_data, float* max_data,
                              int length, float* scales, int32_t* zero_points);
float orc_legacy_min_first_scale(int T, float adj_min, float adj_max);

int orc_quantize_v2(const float* x, int64_t outer, int64_t slices, int64_t inner, int T, int mode,
                    int classic_asymmetric, float ensure_minimum_range, const float* in_min,
                    const float* in_max, void* q, float* out_min, float* out_max);
int orc_dequantize(const void* q, int64_t outer, int64_t slices, int64_t inner, int T, int mode,
                   const float* in_min, const float* in_max, float* y);

int orc_requantize_per_channel(const int32_t* x, int64_t rows, int64_t depth, const float* in_min,
                               const float* in_max, float req_min, float req_max, int out_type,
                               void* q, float* out_min, float* out_max);
int orc_requantization_range_per_channel(const int32_t* x, int64_t rows, int64_t depth,
                                         const float* in_min, const float* in_max,
                                         float clip_value_max, float* out_min, float* out_max);

void orc_int_gemm(const void* a, int a_type, const int8_t* w, int transpose_b, int64_t M, int64_t K,
                  int64_t N, int32_t* acc);
void orc_weight_colsum(const int8_t* w, int64_t K, int64_t N, int32_t* colsum);

int orc_qmatmul_prepare(const orc_matmul_attrs* at, int64_t N, const int32_t* colsum, float min_a,
                        float max_a, const float* min_b, const float* max_b, int64_t nb,
                        float min_out, float max_out, const void* bias, float* scales,
                        float* bias_out, orc_epilogue_desc* ep);
void orc_qmatmul_epilogue(const int32_t* acc, int64_t M, int64_t N, const orc_epilogue_desc* ep,
                          const float* scales, const float* bias, const float* addend, int t_out,
                          void* out);
int orc_qmatmul_output_minmax(const orc_matmul_attrs* at, float min_a, float max_a,
                              const float* min_b, const float* max_b, int64_t nb, int b_rank,
                              float min_out, float max_out, float* out_min, float* out_max,
                              int64_t* n_out);
int orc_qmatmul(const orc_matmul_attrs* at, const void* a, const int8_t* w, int transpose_b,
                int64_t M, int64_t K, int64_t N, const void* bias, const float* addend, float min_a,
                float max_a, const float* min_b, const float* max_b, int64_t nb, float min_out,
                float max_out, void* out);

/*
 * Quantized BatchMatMul, qint8 x qint8 -> float / bfloat16 / half
 * (itex/core/kernels/common/batch_matmul_op.h: Init :88-273, GetPrimitiveDesc :361-419,
 *  QuantizedBatchMatMulV2Op::AccumulateMulAndInt8Scale :497-515).
 * x: [..., M, K] (or [..., K, M] with adj_x), y: [..., K, N] (or [..., N, K] with adj_y); the leading
 * dimensions broadcast against each other (MatMulBCast).  Each binary operand is a tensor of the
 * OUTPUT element type with one element, or with the rank of the output and every dimension equal to
 * the output's or 1 (oneDNN binary post-op broadcast).
 * Pinned by: brute force in numpy int64 / float32; the three cases of the reference's
 * quantized_batch_matmul_test.py at its own tolerance; linearity / broadcast identities.
 */
enum { ORC_BIN_MUL = 1, ORC_BIN_ADD = 2 };
typedef struct {
  int alg;            /* ORC_BIN_MUL | ORC_BIN_ADD */
  const void* data;   /* elements of the output type */
  int rank;           /* 0 (one element) or the output's rank */
  int64_t dims[8];
} orc_bmm_binary;
int orc_qbatch_matmul(const int8_t* x, int x_rank, const int64_t* x_dims, const int8_t* y, int y_rank,
                      const int64_t* y_dims, int adj_x, int adj_y, float min_x, float max_x,
                      float min_y, float max_y, int n_binary, const orc_bmm_binary* bin, int t_out,
                      void* out, int out_rank, const int64_t* out_dims);

/*
 * Quantized Conv2D (NHWC input, HWIO qint8 filter, SCALED quantization: zero points are 0, so the
 * padding value is the integer 0): itex/core/kernels/common/quantized_conv_ops.h
 * (constructor :63-318, ExtendInt8PostOps :329-446, GetBiasHandle :448-597) over the geometry of
 * itex/core/kernels/common/conv_ops.h:615-716 / TensorFlow's GetWindowedOutputSizeVerbose.
 * Fusions restated: BiasAdd, Relu, LeakyRelu, Elu, Sigmoid, Requantize, Dequantize (Sum and the depthwise form: the
 * functions further down).  Swish, HardSwish and the 3-D variants are not.
 * Pinned by: brute force against float64 direct convolution of the integer operands; the fp32
 * convolution at the reference's own tolerance (native_quantized_conv_test.py: rtol = atol = 0.3) and
 * at the bound the quantization steps allow; closed forms of the scales; padding identities.
 * Parity unpinned: none of the reference's conv tests holds fixed vectors (their inputs are unseeded
 * random numbers), so nothing beyond those properties pins the restatement.
 */
enum { ORC_PAD_VALID = 0, ORC_PAD_SAME = 1, ORC_PAD_EXPLICIT = 2 };
typedef struct {
  int64_t batch, in_h, in_w, in_c, k_h, k_w, out_c;
  int stride_h, stride_w, dil_h, dil_w;
  int padding;                                   /* ORC_PAD_* */
  int pad_top, pad_bottom, pad_left, pad_right;  /* ORC_PAD_EXPLICIT only */
} orc_conv_geom;
typedef struct {
  int t_in;              /* ORC_QUINT8 | ORC_QINT8 */
  int t_out;             /* ORC_QINT32 | ORC_QINT8 | ORC_QUINT8 | ORC_FLOAT | ORC_BFLOAT16 */
  int t_bias;            /* 0: no BiasAdd;  ORC_FLOAT | ORC_QINT32 */
  int activation;        /* ORC_ACT_NONE | ORC_ACT_RELU | ORC_ACT_LEAKYRELU | ORC_ACT_ELU | ORC_ACT_SIGMOID */
  float alpha;           /* LeakyRelu */
} orc_conv_attrs;
/* output extent and leading padding of one spatial dimension; returns ORC_INVALID_ARGUMENT for a negative extent */
int orc_conv_out_dim(int64_t in, int64_t k, int stride, int dil, int padding, int pad_before, int pad_after,
                     int64_t* out, int64_t* pad_lead);
void orc_int_conv2d(const void* x, int x_type, const int8_t* w, const orc_conv_geom* g, int64_t out_h,
                    int64_t out_w, int64_t pad_top, int64_t pad_left, int32_t* acc);
int orc_qconv_prepare(const orc_conv_attrs* at, int64_t N, float min_in, float max_in, const float* min_f,
                      const float* max_f, int64_t depth, float min_out, float max_out, const void* bias,
                      float* scales, float* bias_out, orc_epilogue_desc* ep);
int orc_qconv2d(const orc_conv_attrs* at, const orc_conv_geom* g, const void* x, const int8_t* w,
                const void* bias, float min_in, float max_in, const float* min_f, const float* max_f,
                int64_t depth, float min_out, float max_out, void* out, int64_t* out_h, int64_t* out_w);
/* Depthwise form (QuantizedDepthwiseConv2D*, _QuantizedDepthwiseConv2D): w is [k_h, k_w, in_c, mult], the output has
 * in_c * mult channels (g->out_c is ignored), scales / bias / ranges as for orc_qconv2d with that many channels. */
void orc_int_depthwise_conv2d(const void* x, int x_type, const int8_t* w, const orc_conv_geom* g, int64_t mult,
                              int64_t out_h, int64_t out_w, int64_t pad_top, int64_t pad_left, int32_t* acc);
int orc_qdepthwise_conv2d(const orc_conv_attrs* at, const orc_conv_geom* g, int64_t mult, const void* x, const int8_t* w,
                          const void* bias, float min_in, float max_in, const float* min_f, const float* max_f,
                          int64_t depth, float min_out, float max_out, void* out, int64_t* out_h, int64_t* out_w);
/* The "Sum" fusions (QuantizedConv2DWithBias[Signed]SumAndReluAndRequantize, "Sum" in fused_ops of _QuantizedConv2D)
 * with an 8-bit output, quantized_conv_ops.h:202-218 (type rule), :398-433 (scale of the sum post-op from the frozen
 * output range and the summand's range), :604-640 (the summand buffer becomes the destination; a qint8 summand under
 * a quint8 output is bit-cast to quint8, i.e. its bytes are read as unsigned, as written there).
 * position: 1 = before the activation ([BiasAdd, Sum, Relu]), 2 = after it ([BiasAdd, Relu, Sum]).
 * `summand` has the output's shape.  parity unpinned: no vectors of the reference cover these ops. */
typedef struct {
  int position;
  int t_summand;                  /* ORC_QINT8 | ORC_QUINT8 */
  float min_summand, max_summand;
} orc_conv_sum;
int orc_qconv2d_sum(const orc_conv_attrs* at, const orc_conv_geom* g, const void* x, const int8_t* w,
                    const void* bias, float min_in, float max_in, const float* min_f, const float* max_f,
                    int64_t depth, float min_out, float max_out, const orc_conv_sum* sum, const void* summand,
                    void* out, int64_t* out_h, int64_t* out_w);

#ifdef __cplusplus
}
#endif
#endif /* ITEX_ORACLE_H_ */
