/*
 * CPU oracle for the sparse_conv2d path.  TEST INFRASTRUCTURE ONLY.
 *
 * This library restates, in plain C, the algorithms of Paddle-Lite's
 * sparse 1x1 convolution: the weight packers of sparse_conv_detect_pass,
 * the pointer-walking SpMM of the ARM math functions (semantics only), the
 * naive dense reference of the unit tests and the parameter merging of the
 * ARM kernel class.  It exists so that tests, the smoke check and the
 * benchmark's cpu_baseline leg can check / time something that is NOT the
 * shipped HIP path.  Nothing in the product may link or load it.
 *
 * Pinning status of each group is stated next to its declaration.
 */
#ifndef PL_SPARSE_CONV_ORACLE_H_
#define PL_SPARSE_CONV_ORACLE_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* lite_api::ActivationType values used by the path
 * (reference: lite/api/paddle_place.h:122-149). */
enum {
  PLO_ACT_NONE = 0,
  PLO_ACT_RELU = 1,
  PLO_ACT_RELU6 = 2,
  PLO_ACT_LEAKY_RELU = 4,
  PLO_ACT_HARD_SWISH = 10
};

/* Activation constants exactly as the math functions consume them
 * (reference: lite/backends/arm/math/sparse_conv_impl.cc:1193-1215). */
typedef struct plo_act {
  int32_t type;          /* PLO_ACT_* ; anything else behaves as none        */
  float relu6_coef;      /* Relu_clipped_coef                                */
  float leaky_alpha;     /* Leaky_relu_alpha                                 */
  float hs_scale;        /* hard_swish_scale; kernel uses (float)(1.0/scale) */
  float hs_offset;       /* hard_swish_offset                                */
  float hs_threshold;    /* hard_swish_threshold                             */
} plo_act;

/* ---------------------------------------------------------------------------
 * Packers.  Pinned by the reference-generated known-answer vectors in
 * tests/golden/packer_kat.json and by decode round trips.
 * dtype: 0 = fp32 weights, 1 = int8 weights.
 * ------------------------------------------------------------------------ */

/* reference: lite/core/optimizer/mir/sparse_conv_detect_pass.cc:493-517
 * (test copy lite/tests/math/conv_ut.h:183-207). Returns the zero count. */
int plo_count_zeros_pad4(int dtype, const void* w, int rows, int cols,
                         int* num_build_nonzeroes);

/* reference: sparse_conv_detect_pass.cc:303-368 (conv_ut.h:209-274).
 * need_rows_gt1 selects the test copy's extra "rows > 1" condition
 * (conv_ut.h:262); the pass itself has none. Returns rows*cols - stored. */
int plo_count_semi(int dtype, const void* w, int rows, int cols,
                   int need_rows_gt1, int* count_nonzeroes,
                   int* count_channels, int* count_blocks, int* flag_semi);

/* reference: sparse_conv_detect_pass.cc:35-91 (conv_ut.h:483-538).
 * int8 unstructured layout. Returns first_ic. */
int plo_pack_unpadded(int dtype, const void* w, int M, int K, int N,
                      void* nonzero_weights, uint32_t* oc_nonzeros,
                      int32_t* diffs);

/* reference: sparse_conv_detect_pass.cc:93-194 (conv_ut.h:276-375).
 * fp32 unstructured layout, rows padded to a multiple of four entries.
 * Arrays hold num_build_nonzeroes entries. Returns first_ic. */
int plo_pack_padded(int dtype, const void* w, int M, int K, int N,
                    void* nonzero_weights, uint32_t* oc_nonzeros,
                    int32_t* diffs);

/* reference: sparse_conv_detect_pass.cc:196-301 (conv_ut.h:377-481).
 * Two output channels share one index entry; an odd last row is appended
 * entry by entry. Returns first_ic. */
int plo_pack_semi(int dtype, const void* w, int M, int K, int N,
                  void* nonzero_weights, uint32_t* oc_nonzeros,
                  int32_t* diffs);

/* Inverse of the three packers: rebuild the dense [M x K] matrix from a
 * layout (layout: 0 unpadded, 1 padded, 2 semi). Own code, no reference
 * counterpart; follows the per-row start rules of
 * lite/backends/arm/math/sparse_conv_impl.cc:1226-1243 and
 * sparse_semi_conv_impl.cc:1788-1823. Returns 0, or -1 when an index
 * leaves [0,K). */
int plo_decode(int dtype, int layout, const void* nonzero_weights,
               const uint32_t* oc_nonzeros, const int32_t* diffs,
               int first_ic, int M, int K, int N, void* dense_out);

/* ---------------------------------------------------------------------------
 * SpMM over the compressed layout, walking activation pointers by the byte
 * offsets in Diffs exactly like the ARM functions do, one image after the
 * other (batch > 1 is the per-image repetition; the ARM kernel itself only
 * ever computes image 0, lite/kernels/arm/sparse_conv_compute.cc:114-153).
 *   x    : [batch, K, N]   (N = H*W),  out : [batch, M, N]
 *   scale/bias are the merged per-channel arrays (bias may be NULL).
 * Epilogue: fp32  a = bias; a = fmaf(x, w, a) in index order
 *           int8  v = fmaf((float)acc_i32, scale[oc], bias[oc])
 *           act ; int8 out: max(v,-127), round half away, saturate.
 * Pinned by: exact integer matmul and the reference's dense naive path
 * (plo_basic_gemm and oracle/_ref) on the same inputs; the int8 variants of
 * relu6 / leaky_relu / hard_swish are parity unpinned (the reference never
 * tests them) beyond agreeing with the dense formula.
 * ------------------------------------------------------------------------ */
void plo_sparse_conv_fp32(const float* nonzero_weights, const float* x,
                          const int32_t* diffs, const uint32_t* oc_nonzeros,
                          const float* bias, float* out, int batch, int M,
                          int K, int N, int first_ic, int flag_semi,
                          const plo_act* act);

void plo_sparse_conv_int8_fp32(const int8_t* nonzero_weights, const int8_t* x,
                               const int32_t* diffs,
                               const uint32_t* oc_nonzeros, const float* bias,
                               const float* scale, float* out, int batch,
                               int M, int K, int N, int first_ic,
                               int flag_semi, const plo_act* act);

void plo_sparse_conv_int8_int8(const int8_t* nonzero_weights, const int8_t* x,
                               const int32_t* diffs,
                               const uint32_t* oc_nonzeros, const float* bias,
                               const float* scale, int8_t* out, int batch,
                               int M, int K, int N, int first_ic,
                               int flag_semi, const plo_act* act);

/* fp16 path: values are IEEE binary16 bit patterns.  Weights and bias are the
 * fp32 layout of the pass converted element by element (round to nearest
 * even), `diffs` are the byte offsets as the pass wrote them for fp32 (the
 * function halves them like the kernel class does); accumulation, bias and
 * activation all happen in half precision, one rounding per instruction.
 * reference: lite/kernels/arm/sparse_conv_compute.cc:270-356,
 * lite/backends/arm/math/fp16/sparse_conv_fp16.cc (fmla chains, activation
 * macros :668-1173, constants :1301-1325), sparse_semi_conv_fp16.cc.
 * Parity unpinned: the reference has no vectors for it and its test only
 * compares with an fp32 computation under a tolerance. */
uint16_t plo_f32_to_f16(float f);
float plo_f16_to_f32(uint16_t h);
void plo_fp32_to_fp16(const float* in, uint16_t* out, int64_t n);
void plo_fp16_to_fp32(const uint16_t* in, float* out, int64_t n);
void plo_sparse_conv_fp16(const uint16_t* nonzero_weights, const uint16_t* x,
                          const int32_t* diffs, const uint32_t* oc_nonzeros,
                          const uint16_t* bias, uint16_t* out, int batch,
                          int M, int K, int N, int first_ic, int flag_semi,
                          const plo_act* act);

/* Raw int32 accumulators of the int8 path (no epilogue), for the bit-exact
 * accumulator check. */
void plo_sparse_conv_int8_acc(const int8_t* nonzero_weights, const int8_t* x,
                              const int32_t* diffs,
                              const uint32_t* oc_nonzeros, int32_t* acc_out,
                              int batch, int M, int K, int N, int first_ic,
                              int flag_semi);

/* ---------------------------------------------------------------------------
 * Naive dense reference of the unit tests.
 * reference: lite/tests/utils/naive_math_impl.h:246-331 (basic_gemm, no
 * transposes, alpha = 1, beta = 0 as the sparse tests call it).
 * Pinned against oracle/_ref (the real header compiled as is) when built.
 * ------------------------------------------------------------------------ */
void plo_basic_gemm_f32(int m, int n, int k, const float* a, const float* b,
                        float* c, const float* bias, int flag_bias,
                        int flag_act, float six, float leaky_alpha,
                        float hs_scale, float hs_offset, float hs_threshold);

/* reference: lite/backends/arm/math/type_trans.cc:35-110 (fp32_to_int8,
 * axis_size = outer_size = 1) and :268-... (int8_to_fp32). */
void plo_fp32_to_int8(const float* in, int8_t* out, float scale, int64_t n);
void plo_int8_to_fp32(const int8_t* in, float* out, float scale, int64_t n);

/* ---------------------------------------------------------------------------
 * Parameter merging of the ARM kernel class.
 * reference: lite/kernels/arm/sparse_conv_compute.cc:34-101.
 * out_kind: 0 fp32 (no merging), 1 int8->fp32, 2 int8->int8.
 * weight_scale has n_scale (1 or M) entries; returns -1 otherwise.
 * act is updated in place like the reference mutates its param copy.
 * Parity unpinned: no reference test runs the kernel class.
 * ------------------------------------------------------------------------ */
int plo_merge_params(int out_kind, int M, const float* weight_scale,
                     int n_scale, float input_scale, float output_scale,
                     const float* bias, float* merged_scale,
                     float* merged_bias, plo_act* act);

/* ---------------------------------------------------------------------------
 * Dense CPU comparator: per-image GEMM M=OC, N=H*W, K=IC over the batch,
 * as Paddle-Lite's x86 conv2d does for 1x1 kernels
 * (reference: lite/kernels/x86/conv_compute.cc:132-213, :292-341, :423-470).
 * Own blocked loops with exact int32 accumulation; threads over images and
 * row blocks with OpenMP. Returns the thread count used.
 * out_kind as above; for out_kind 0 w and x are float, else int8.
 * ------------------------------------------------------------------------ */
int plo_dense_conv1x1(int out_kind, const void* w_dense, const void* x,
                      const float* bias, const float* scale, void* out,
                      int batch, int M, int K, int N, const plo_act* act,
                      int threads);

/* ---------------------------------------------------------------------------
 * int8 depthwise 3x3 convolution, stride 1 or 2, zero padding 0 or 1
 * (reference: lite/tests/utils/naive_math_impl.h:395-519 for the sums,
 * lite/backends/arm/math/conv_block_utils.h:3696-3753 for the epilogue; note
 * that hard_swish multiplies by act->hs_scale here).
 * x [batch, channels, h, w], w [channels, 3, 3]; out_kind 1 fp32, 2 int8,
 * 3 raw int32 accumulators.  Returns 0, or -1 for a bad argument.
 * ------------------------------------------------------------------------ */
int plo_dwconv3x3_int8(const int8_t* x, const int8_t* w, const float* scale,
                       const float* bias, const plo_act* act, int out_kind,
                       int batch, int channels, int h, int wd, int stride,
                       int pad, void* out);

#ifdef __cplusplus
}
#endif
#endif /* PL_SPARSE_CONV_ORACLE_H_ */
