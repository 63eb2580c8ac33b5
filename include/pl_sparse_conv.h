/*
 * C ABI of the MI355X (gfx950) sparse 1x1 convolution.
 *
 * This is the boundary a Paddle-Lite HIP-target kernel binds to: plain
 * pointers, sizes and POD structs only, every function returns a status and
 * never throws or aborts.  The math entry points take exactly what the ARM
 * math functions of the reference take (compressed weights, merged
 * per-channel scale and bias, activation constants) so that a kernel class
 * written like lite/kernels/arm/sparse_conv_compute.cc can call them from
 * PrepareForRun() / Run().
 *
 * Thread compatibility: functions may be called from any thread; a handle
 * must not be used by two threads at once.
 */
#ifndef PL_SPARSE_CONV_H_
#define PL_SPARSE_CONV_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define PL_SPARSE_CONV_ABI_VERSION 1

/* status codes (negative = failure; HIP errors are reported as
 * PL_ERR_HIP with the text available from pl_last_error()) */
enum {
  PL_OK = 0,
  PL_ERR_BAD_ARG = -1,
  PL_ERR_BAD_LAYOUT = -2,   /* OcNonZeros / Diffs do not describe a matrix */
  PL_ERR_UNSUPPORTED = -3,
  PL_ERR_HIP = -4,
  PL_ERR_NO_DEVICE = -5
};

/* Kernel variants = the registrations of the reference
 * (lite/kernels/arm/sparse_conv_compute.cc:369-430): fp32 "def",
 * "int8_fp32_out" and "int8_int8_out".  PL_KIND_INT8_ACC32 additionally
 * exposes the raw int32 accumulators of the int8 path for verification.
 * PL_KIND_FP16 is the half-precision kernel (sparse_conv_compute.cc:270-356,
 * lite/backends/arm/math/fp16/sparse_conv_fp16.cc, sparse_semi_conv_fp16.cc):
 * the descriptor carries the fp32 sparse tensors and the fp32 bias of the
 * pass, which prepare converts to binary16 like that kernel's PrepareForRun;
 * x_dev / out_dev are binary16, and accumulation and activation run in
 * half precision. */
enum {
  PL_KIND_FP32 = 0,
  PL_KIND_INT8_FP32 = 1,
  PL_KIND_INT8_INT8 = 2,
  PL_KIND_INT8_ACC32 = 3,
  PL_KIND_FP16 = 4
};

/* lite_api::ActivationType values the sparse kernels implement
 * (lite/api/paddle_place.h:122-149; selection as in
 * lite/backends/arm/math/sparse_conv_impl.cc:1197-1215: any other value
 * means "no activation"). */
enum {
  PL_ACT_NONE = 0,
  PL_ACT_RELU = 1,
  PL_ACT_RELU6 = 2,
  PL_ACT_LEAKY_RELU = 4,
  PL_ACT_HARD_SWISH = 10
};

/* How the SpMM is executed.
 *   PL_ALGO_AUTO      library picks (see pl_sparse_conv_info.algo)
 *   PL_ALGO_ROW_WALK  one wavefront per output channel (pair) walks its
 *                     nonzero list over an activation tile held in LDS
 *   PL_ALGO_BLOCK_MFMA int8 only: 32x32 blocks of the weight matrix that
 *                     hold at least one nonzero are multiplied on the matrix
 *                     cores, empty blocks are skipped
 *   PL_ALGO_IMAGE_MFMA int8 only, oc a multiple of 128, ic = 128 / 256 / 512,
 *                     H*W a multiple of 4 in [16, 256]: one workgroup per
 *                     (image, 128 output rows) keeps the whole image in LDS
 *                     and multiplies it with dense 16x64 weight tiles; also
 *                     7 x 7 maps with ic = 256 / 512 / 1024 (two images per
 *                     workgroup), and larger maps of a multiple of 196
 *                     positions (28 x 28, 56 x 56, 112 x 112) in slabs of 196
 *                     positions
 * With PL_ALGO_AUTO an int8 handle holds every form its shape allows and
 * chooses per call by batch and H*W (the image kernels where the whole map
 * fits, or in slabs while batch * slabs * oc / 128 is at most half the CU
 * count; else the row walk for at most 256 positions in all;
 * else the block kernel): see pl_sparse_conv_algo_for(). */
enum { PL_ALGO_AUTO = 0, PL_ALGO_ROW_WALK = 1, PL_ALGO_BLOCK_MFMA = 2, PL_ALGO_IMAGE_MFMA = 3 };

/* Activation constants, used as given (replaces the fields of
 * ActivationParam the math functions read,
 * lite/operators/op_params.h:331-362). */
typedef struct pl_activation {
  int32_t type;        /* PL_ACT_*                                          */
  float relu6_coef;    /* Relu_clipped_coef                                 */
  float leaky_alpha;   /* Leaky_relu_alpha                                  */
  float hs_scale;      /* hard_swish_scale; the kernel multiplies by
                          (float)(1.0 / hs_scale)                           */
  float hs_offset;     /* hard_swish_offset                                 */
  float hs_threshold;  /* hard_swish_threshold                              */
} pl_activation;

/* Tuning overrides of one handle; every field 0 = the library's own rule.
 * The reference configures its kernels through setters and a config struct,
 * never through process state (lite/api/paddle_api.h:542-547); this struct is
 * the counterpart for the choices this library makes per handle.  Fields
 * marked (switch) take PL_TUNE_RULE / PL_TUNE_NEVER / PL_TUNE_ALWAYS, where
 * ALWAYS means "whenever the shape allows it". */
enum { PL_TUNE_RULE = 0, PL_TUNE_NEVER = 1, PL_TUNE_ALWAYS = 2 };
typedef struct pl_sparse_conv_tuning {
  int32_t image_kernel;      /* PL_ALGO_IMAGE_MFMA: 3 (and the rule wherever it
                                applies) = one row tile per wavefront, image
                                through registers; 1 = a pair of wavefronts per
                                two row tiles, image regrouped in LDS (the rule
                                for 7 x 7 maps); 2 = the kernel with transposing
                                LDS reads (H*W = 4 mod 8 only); a kernel asked
                                for outside its shapes is PL_ERR_UNSUPPORTED   */
  int32_t image_min_items;   /* fewest (image, 128 rows) work items for which
                                PL_ALGO_AUTO takes the image kernel (rule: 1)  */
  int32_t mfma_stream;       /* (switch) streaming form of the block kernel    */
  int32_t mfma_sub_tiles;    /* (switch) several tiles per workgroup, ic <= 64 */
  int32_t mfma_tile_quads;   /* block kernel: position quads per tile, 8 .. 32 */
  int32_t mfma_narrow_i8_stores; /* 1 = 4-byte int8 stores in the block kernel */
  int32_t wg_slots;          /* workgroups taken as resident at once           */
  int32_t walk_tiled;        /* (switch) fp32 / fp16 walk with tile and lists in LDS */
  int32_t walk_split;        /* that walk: 1 = row groups not divided between
                                CUs, 1 + k = k sixteenths to the spare CUs     */
  int32_t walk_chunked;      /* (switch) fp32 / fp16 walk over channel chunks  */
  int32_t chunk_walk_groups; /* that walk: row groups per wavefront, 4 or 8    */
  int32_t walk_tile;         /* plain walk: positions per tile (power of two)  */
  int32_t walk_threads;      /* plain walk: threads per workgroup              */
  int32_t walk_slices;       /* plain walk: row slices                         */
  int32_t image_tr_regroup;  /* (switch) regrouping image kernel: the regrouping
                                done by transposing LDS reads where that exists
                                (ic = 512, 14 x 14 maps); NEVER = by the vector
                                ALU everywhere                                 */
  int32_t walk_pairs;        /* (switch) the fp32 walk with tile and lists in LDS
                                takes several row groups per wavefront
                                instruction (two: lanes 0 - 31 walk one, lanes
                                32 - 63 the other, four positions per lane; with
                                more than 271 channels 4 / 8 / 16 on smaller
                                tiles).  NEVER = one row group per instruction:
                                that form exists up to 271 channels and for maps
                                of a multiple of 4 positions only             */
} pl_sparse_conv_tuning;

/* Everything PrepareForRun() knows.  All pointers are HOST pointers and are
 * only read during pl_sparse_conv_prepare(). Replaces the argument list of
 * sparse_conv_*_pipelined (lite/backends/arm/math/sparse_conv_impl.h:38-73,
 * sparse_semi_conv_impl.h:30-68) minus the activation/output pointers. */
typedef struct pl_sparse_conv_desc {
  uint32_t struct_size;          /* sizeof(pl_sparse_conv_desc)             */
  int32_t kind;                  /* PL_KIND_*                               */
  int32_t flag_semi;             /* SparseConvParam::flag_semi              */
  int32_t first_ic;              /* SparseConvParam::first_ic               */
  int32_t oc;                    /* M: output channels                      */
  int32_t ic;                    /* K: input channels                       */
  int32_t im_size;               /* H*W the Diffs tensor was baked for      */
  int32_t algo;                  /* PL_ALGO_*                               */
  const void* nonzero_weights;   /* float or int8_t, n_weights elements     */
  int64_t n_weights;
  const uint32_t* oc_nonzeros;   /* oc entries (semi: oc/2 + oc%2 are read) */
  const int32_t* diffs;          /* n_diffs entries, byte offsets           */
  int64_t n_diffs;
  const float* scale;            /* oc merged scales; int8 kinds only       */
  const float* bias;             /* oc merged biases or NULL                */
  pl_activation act;
  pl_sparse_conv_tuning tuning;  /* struct_size may also be the offset of this
                                    field: then every rule applies            */
} pl_sparse_conv_desc;

typedef struct pl_sparse_conv_info {
  int32_t algo;          /* the algorithm run() will use                    */
  int32_t oc, ic;
  int64_t nnz;           /* nonzero weights actually present in the layout  */
  int64_t stored_weights;/* weights stored in the layout (semi keeps zeros) */
  int64_t index_entries; /* Diffs entries describing real weights           */
  int64_t device_bytes;  /* device memory held by the handle                */
  int64_t mfma_blocks;   /* 32x32 weight blocks with a nonzero (int8)       */
  int64_t mfma_blocks_total;
} pl_sparse_conv_info;

typedef struct pl_sparse_conv_handle pl_sparse_conv_handle;

/* Library / device ------------------------------------------------------- */
int pl_sparse_conv_abi_version(void);
/* Text of the last failure on the calling thread ("" if none). */
const char* pl_last_error(void);
/* Number of usable gfx950 devices (0 on a machine without one). */
int pl_device_count(void);

/* The op's hot path ------------------------------------------------------ */

/* Replaces SparseConvCompute::PrepareForRun's device-side part: validates the
 * layout, converts the byte offsets to channel indices and uploads the
 * GPU-side form to the current HIP device. */
int pl_sparse_conv_prepare(const pl_sparse_conv_desc* desc,
                           pl_sparse_conv_handle** out_handle);

/* Replaces sparse_conv_{fp32,int8_fp32,int8_int8}_pipelined and their
 * sparse_semi_ twins, called from SparseConvCompute::Run
 * (lite/kernels/arm/sparse_conv_compute.cc:104-267).
 *   x_dev   : device pointer, NCHW [batch, ic, im_size] float or int8_t
 *   out_dev : device pointer, NCHW [batch, oc, im_size] float / int8_t /
 *             int32_t per kind
 *   im_size : H*W of this call (may differ from the baked one)
 *   stream  : hipStream_t (NULL = default stream); the call only enqueues. */
int pl_sparse_conv_run(pl_sparse_conv_handle* handle, const void* x_dev,
                       void* out_dev, int32_t batch, int32_t im_size,
                       void* stream);

/* The repeat loop of the reference's unit-test benchmark
 * (lite/tests/math/sparse_conv_int8_compute_test.cc:285-360: warm-up, then
 * `repeats` timed calls) as one call: enqueues `steps` runs back to back on
 * `stream`, run i reading x_dev[i % n_sets] and writing out_dev[i % n_sets]
 * (rotating buffers keep the working set out of the last-level cache).
 * With elapsed_ms != NULL the runs are bracketed by two HIP events on
 * `stream`, the call waits for the second one and stores the time between
 * them in milliseconds. */
int pl_sparse_conv_run_sequence(pl_sparse_conv_handle* handle,
                                const void* const* x_dev, void* const* out_dev,
                                int32_t n_sets, int32_t batch, int32_t im_size,
                                int32_t steps, void* stream,
                                float* elapsed_ms);

int pl_sparse_conv_get_info(const pl_sparse_conv_handle* handle,
                            pl_sparse_conv_info* info);

/* The algorithm (PL_ALGO_*, never PL_ALGO_AUTO) a pl_sparse_conv_run() call
 * with this batch and H*W would use on 16-byte aligned tensors, or a negative
 * status.  No counterpart in the reference, whose kernel choice is fixed by
 * the registration (lite/kernels/arm/sparse_conv_compute.cc:369-430). */
int pl_sparse_conv_algo_for(const pl_sparse_conv_handle* handle, int32_t batch,
                            int32_t im_size);

/* Replace scale / bias / activation without re-uploading weights (what a
 * second PrepareForRun with new quantisation parameters would do). Either
 * pointer may be NULL to keep the current values. */
int pl_sparse_conv_set_epilogue(pl_sparse_conv_handle* handle,
                                const float* scale, const float* bias,
                                const pl_activation* act);

void pl_sparse_conv_destroy(pl_sparse_conv_handle* handle);

/* Opt-time packers (host only) -------------------------------------------
 * dtype: 0 = fp32 weights, 1 = int8 weights.  Dense weights are [oc x ic]
 * row major. */

/* Replaces SparseConvDetectPass::ComputeSemiSparseZeros
 * (lite/core/optimizer/mir/sparse_conv_detect_pass.cc:303-368). Returns the
 * zero count the pass compares with sparse_threshold. */
int pl_sparse_count_semi(int32_t dtype, const void* dense, int32_t oc,
                         int32_t ic, int32_t* count_nonzeroes,
                         int32_t* count_channels, int32_t* count_blocks,
                         int32_t* flag_semi);

/* Replaces SparseConvDetectPass::ComputeSparseZeros
 * (sparse_conv_detect_pass.cc:480-517). */
int pl_sparse_count_zeros(int32_t dtype, const void* dense, int32_t oc,
                          int32_t ic, int32_t* num_build_nonzeroes);

/* Replaces ComputeSparseWeight (both overloads) and ComputeSemiSparseWeight
 * (sparse_conv_detect_pass.cc:35-301) with the pass's own choice between
 * them (:732-780): semi layout when flag_semi, else rows padded to four for
 * fp32 and unpadded for int8.  Output arrays must hold n_weights / oc /
 * n_diffs elements as computed by the two counting functions. Returns
 * first_ic (>= 0) or a negative status. */
int pl_sparse_pack(int32_t dtype, int32_t flag_semi, const void* dense,
                   int32_t oc, int32_t ic, int32_t im_size,
                   void* nonzero_weights, int64_t n_weights,
                   uint32_t* oc_nonzeros, int32_t* diffs, int64_t n_diffs);

/* Host: float -> IEEE binary16 bit patterns, round to nearest even.  Replaces
 * lite::arm::math::fp16::fp32_to_fp16 as the half-precision kernel class
 * uses it on weights and bias (lite/kernels/arm/sparse_conv_compute.cc:
 * 275-297); prepare applies the same conversion for PL_KIND_FP16. */
int pl_fp32_to_fp16(const float* in, uint16_t* out, int64_t n);

/* Precision changes either side of an int8 sparse convolution (device
 * pointers, n elements, per-tensor scale; enqueued on `stream`) -----------
 * Replaces lite::arm::math::fp32_to_int8 as CalibComputeFp32ToInt8::Run calls
 * it (lite/kernels/arm/calib_compute.cc:31-38, lite/backends/arm/math/
 * type_trans.cc:35-160): out = saturate(round-half-away(x * (1 / scale))),
 * never below -127. */
int pl_calib_fp32_to_int8(const float* x_dev, int8_t* out_dev, int64_t n,
                          float scale, void* stream);

/* Replaces lite::arm::math::int8_to_fp32 as CalibComputeInt8ToFp32::Run calls
 * it (calib_compute.cc:60-68, type_trans.cc:int8_to_fp32): out = x * scale. */
int pl_calib_int8_to_fp32(const int8_t* x_dev, float* out_dev, int64_t n,
                          float scale, void* stream);

/* ---- int8 depthwise 3x3 convolution (the layer between the pointwise
 * convolutions of a MobileNet) -------------------------------------------
 * Replaces lite::arm::math::conv_depthwise_3x3_int8_fp32 / _int8_int8 as
 * DepthwiseConv<kInt8, *>::Run calls them (lite/kernels/arm/conv_depthwise.cc:
 * 359-412, lite/backends/arm/math/conv_impl.cc:1858-2090): one 3x3 filter per
 * channel, stride 1 or 2, zero padding 0 or 1 on all four sides, dilation 1;
 * int32 accumulation, then fmaf(float(acc), scale[c], bias[c]), activation,
 * and for int8 output max(v, -127), round half away from zero, saturate
 * (conv_block_utils.h:3888-3950, :4328-4420).  hard_swish follows
 * cvt_kernel there: (v * hs_scale) * min(max(v + hs_offset, 0), hs_threshold),
 * i.e. hs_scale multiplies.  scale / bias are the merged per-channel values
 * of PrepareForRun (conv_depthwise.cc:158-322).  All desc pointers are host
 * pointers read only during prepare. */
typedef struct pl_dwconv_desc {
  uint32_t struct_size;     /* sizeof(pl_dwconv_desc)                        */
  int32_t kind;             /* PL_KIND_INT8_FP32 or PL_KIND_INT8_INT8        */
  int32_t channels;
  int32_t stride;           /* 1 or 2 (both directions)                      */
  int32_t pad;              /* 0 or 1 (all four sides)                       */
  const int8_t* weights;    /* [channels][3][3]                              */
  const float* scale;       /* [channels]                                    */
  const float* bias;        /* [channels] or NULL                            */
  pl_activation act;
  /* tuning, 0 = the library's rule (struct_size may also be the offset of
   * item_rows: then every rule applies) */
  int32_t item_rows;        /* output rows per thread: 1, 2 or 4             */
  int32_t item_cols;        /* groups of four output columns per thread      */
  int32_t share_lanes;      /* PL_TUNE_*: neighbouring lanes exchange dwords  */
  int32_t row_items;        /* PL_TUNE_*: one output row per thread through
                               LDS (narrow planes)                           */
} pl_dwconv_desc;

typedef struct pl_dwconv_handle pl_dwconv_handle;

int pl_dwconv3x3_prepare(const pl_dwconv_desc* desc, pl_dwconv_handle** out_handle);

/* x_dev: int8 NCHW [batch, channels, h, w]; out_dev: fp32 or int8 NCHW
 * [batch, channels, oh, ow] with oh = (h + 2 * pad - 3) / stride + 1.
 * Enqueues on `stream` and returns. */
int pl_dwconv3x3_run(pl_dwconv_handle* handle, const int8_t* x_dev, void* out_dev,
                     int32_t batch, int32_t h, int32_t w, void* stream);

void pl_dwconv3x3_destroy(pl_dwconv_handle* handle);

/* ---- sparse_conv2d followed by the depthwise 3x3 convolution, one launch ----
 * No counterpart in the reference, where the two layers are two kernels
 * (Instruction::Run per op, lite/core/program.cc:789-816) with the tensor
 * between them in memory.  Here the pointwise kernel keeps the 16 output
 * channels of a wavefront in LDS as int8 planes and runs the depthwise layer
 * on them: the intermediate tensor is never written, one launch instead of
 * two.  Results are those of pl_sparse_conv_run followed by pl_dwconv3x3_run,
 * bit for bit.  Both handles int8 -> int8, 14 x 14 maps, depthwise padding 1
 * and stride 1 or 2, depthwise channels = pointwise output channels, a
 * pointwise handle that the image algorithm with one row tile per wavefront
 * serves (oc % 128 == 0, ic = 128, 256 or 512, algo AUTO or IMAGE_MFMA).
 * _fits returns 1 when a pair can run this way, else 0; _run returns
 * PL_ERR_UNSUPPORTED with the reason for a pair that cannot (it does not
 * consult _pays).
 * x_dev: int8 NCHW [batch, ic, h, w]; out_dev: int8 NCHW [batch, oc, oh, ow]
 * of the depthwise layer; both 4-byte aligned. */
int pl_sparse_conv_dwconv3x3_fits(const pl_sparse_conv_handle* conv, const pl_dwconv_handle* dw,
                                  int32_t h, int32_t w);
/* 1 when the pair fits and the one launch is expected to be faster than the
 * two at this batch: always for stride 2; for stride 1 when the launch has
 * at least half as many workgroups (batch * oc / 128) as the device has CUs -
 * the one launch keeps the depthwise work of a workgroup's 128 planes on its
 * CU, which loses to the depthwise kernel's spread at small batches. */
int pl_sparse_conv_dwconv3x3_pays(const pl_sparse_conv_handle* conv, const pl_dwconv_handle* dw,
                                  int32_t batch, int32_t h, int32_t w);
int pl_sparse_conv_dwconv3x3_run(pl_sparse_conv_handle* conv, pl_dwconv_handle* dw,
                                 const void* x_dev, void* out_dev, int32_t batch,
                                 int32_t h, int32_t w, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* PL_SPARSE_CONV_H_ */
