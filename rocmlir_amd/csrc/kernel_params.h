// By-value parameter blocks passed to the gfx950 kernels after their pointer
// arguments.  Shared between the host library (which fills them from the
// parsed problem) and the device code.  Plain C layout, no padding surprises:
// every field is 4 or 8 bytes and 8-byte fields come first.
//
// The reference bakes shapes into each generated kernel and passes only bare
// pointers (mlir/lib/Dialect/Rock/Pipelines/Pipelines.cpp:246-248); the
// hand-written kernels take the same bare pointers followed by one of these
// blocks, which the C-ABI hands to the caller together with the code object.
#pragma once
#include <stdint.h>

// element types; values are part of the C-ABI (rocmlir_amd.h)
enum RockDType : int32_t {
  ROCK_F32 = 0,
  ROCK_F16 = 1,
  ROCK_BF16 = 2,
  ROCK_I8 = 3,
  ROCK_FP8 = 4, // OCP e4m3fn
  ROCK_BF8 = 5, // OCP e5m2
  ROCK_I32 = 6,
  ROCK_DTYPE_COUNT = 7
};

// Epilogue applied to the accumulator tile before the store
// (MIGraphXToTosa.cpp:874-982 formulas; GemmToGridwise.cpp:241-263 cast; the
// element-wise operations MIGraphX fuses behind a contraction,
// MIGraphXToTosa.cpp:1009-1016 relu, :1089-1100 clip, :1283-1295 add, mul,
// erf, exp, sigmoid, tanh).  Steps, in this order:
//   1. float accumulators:  v = acc * scale
//      int32 accumulators:  v = (float(acc) - float(zero_point)) * scale
//   2. v += bias[n]                       one value per output channel
//   3. v = v + r  or  v * r               r = residual tensor, same type and
//                                         layout as the output
//   4. v = activation(v)
//   5. out i8:  q = clamp(roundeven(v * inv_quant_scale) + out_zero_point)
//      else:    round to the output type
// int32 accumulators leaving as int32 skip 1, 4 and 5 and take 2 and 3 in
// integer arithmetic.
enum RockActivation : int32_t {
  ROCK_ACT_NONE = 0,
  ROCK_ACT_RELU = 1,    // max(v, 0)
  ROCK_ACT_CLIP = 2,    // min(max(v, act_lo), act_hi)
  ROCK_ACT_SIGMOID = 3, // 1 / (1 + exp(-v))
  ROCK_ACT_TANH = 4,
  ROCK_ACT_ERF = 5,
  ROCK_ACT_GELU = 6,    // 0.5 v (1 + erf(v / sqrt 2)), the mul/erf/add chain of a traced GELU
  ROCK_ACT_EXP = 7,
};
enum RockResidualOp : int32_t { ROCK_RES_NONE = 0, ROCK_RES_ADD = 1, ROCK_RES_MUL = 2 };

struct RockEpilogue {
  float scale;          // 1.0f = identity
  float inv_quant_scale; // 1/scale of the requantisation step (out i8 only)
  int32_t zero_point;   // subtracted from an int32 accumulator
  int32_t out_zero_point;
  int32_t has_bias;     // aux pointer holds one f32 (or i32 for i32 out) per output channel
  int32_t out_dtype;    // RockDType
  int32_t activation;   // RockActivation
  int32_t residual_op;  // RockResidualOp; the residual pointer follows the bias pointer
  float act_lo, act_hi; // clamp applied for relu [0, +inf) and clip [lo, hi]; (-inf, +inf) otherwise
  // Per-channel (broadcast-vector) quantisation, the form the reference lowers for scale and zero-point tensors
  // shaped like one value per output channel (MIGraphXToTosa.cpp:874-982; mixr-resnet-fusion-case-1-
  // quantization.mlir:8-9 dequantises and re-quantises with a <1x128x1x1xf32> scale): a set bit replaces
  // the scalar above by element n of the vector.  Only the kernels with the rolled epilogue ("_e") and the
  // element-wise kernels read them.
  int32_t chan_flags;            // RockChannelVector bits
  int32_t pad_;
  const float *scale_vec;        // step 1: scale[n]
  const void *zero_point_vec;    // step 1: zero_point[n], int32 or int8 (ROCK_CHAN_ZP_I8)
  const float *quant_scale_vec;  // step 5: the quantisation scale[n] (the kernel multiplies by its reciprocal)
  const void *out_zero_point_vec; // step 5: out_zero_point[n], int32 or int8 (ROCK_CHAN_OUT_ZP_I8)
};
enum RockChannelVector : int32_t {
  ROCK_CHAN_SCALE = 1,
  ROCK_CHAN_ZP = 2,
  ROCK_CHAN_QUANT_SCALE = 4,
  ROCK_CHAN_OUT_ZP = 8,
  ROCK_CHAN_ZP_I8 = 16,     // the zero-point vector holds int8 elements
  ROCK_CHAN_OUT_ZP_I8 = 32, // the output zero-point vector holds int8 elements
};

struct RockGemmParams {
  // element strides of the logical views A[g,m,k], B[g,n,k], C[g,m,n]
  int64_t a_gs, a_ms, a_ks;
  int64_t b_gs, b_ns, b_ks;
  int64_t c_gs, c_ms, c_ns;
  int32_t G, M, N, K;
  int32_t tiles_m, tiles_n; // block tiles per batch entry
  int32_t group_m;          // tile rows per L2 group
  int32_t xcd_remap;        // 1: undo the round-robin block->XCD dispatch
  RockEpilogue epi;
};

// Forward convolution as an implicit GEMM:
//   M = N*Ho*Wo (output pixels), N = K_out per group, K = Y*X*C per group.
// Strides are in elements of the respective tensor.
// Division of a block or chunk index (below 2^31) by a divisor fixed at plan
// time: n / d == (n * mul) >> shift in 64-bit arithmetic, with
// mul = ceil(2^shift / d) and shift = 31 + ceil(log2 d).
struct RockFastDiv {
  uint32_t mul, shift;
};
struct RockConvParams {
  int64_t in_ns, in_gs, in_cs, in_hs, in_ws;
  int64_t fil_gs, fil_ks, fil_cs, fil_ys, fil_xs;
  int64_t out_ns, out_gs, out_ks, out_hs, out_ws;
  int32_t n, g, c, k; // c, k per group
  int32_t hi, wi, y, x, ho, wo;
  int32_t stride_h, stride_w, pad_h, pad_w, dil_h, dil_w;
  int32_t M, N, K;    // implicit GEMM sizes
  int32_t tiles_m, tiles_n;
  int32_t group_m, xcd_remap;
  int32_t k_order_yxc; // 1: reduction index runs (y,x,c) with c fastest; 0: (c,y,x)
  int32_t rows_per_tile; // window-resident kernel: output rows (n, ho) per block; else 0
  RockEpilogue epi;
  // Kernels named "_runs": a channel run of c elements is a row of filter taps over neighbouring narrow pixels
  // padded to whole 16-byte chunks; its first run_valid elements are data, what the load brings along behind
  // them (the next pixel) is cleared in LDS before it is multiplied.  0 elsewhere.
  int32_t run_valid;
  // Reduction split over the groups of a one-group problem (few output tiles, long reduction): group s
  // reduces the elements [s * k_group_stride, s * k_group_stride + K) of every row of taps-and-channels,
  // a whole number of K-steps, into an f32 partial result of its own (in_gs = 0, fil_gs = K).  0 elsewhere.
  int32_t k_group_stride;
  // plan-time constants for the divisions of the fast loader's set-up (row -> image, output row, output
  // pixel; reduction index -> tap, channel; tap -> filter row, filter column): by ho * wo, wo, c, x
  RockFastDiv div_image, div_row, div_c, div_x;
};

// Filter gradient of a convolution as one K-major GEMM over the tensors as they
// lie (channels-last input and output gradient, one group):
//   dW[k, (y, x, c)] = sum over pixels m = (n, ho, wo) of dY[m, k] * X[n, ho*s + y*d - p, wo*s + x*d - p, c]
// The GEMM part describes A = dY as [k][pixel] (K-major: a_ms = 1, a_ks = pixel
// stride), C = the gradient (or its f32 partial sums) as [k][(y, x, c)], and
// the batch index G = the split of the pixel range (batch entry g reduces the
// pixels [g*K, (g+1)*K)); the second operand is the forward im2col matrix,
// gathered by the loader from what follows (b_* are unused).
struct RockConvBwdWeightParams : RockGemmParams {
  int64_t in_pix_stride; // elements between neighbouring input pixels along w; rows and images follow densely
  int32_t c;             // input channels (the columns run (y, x, c) with c fastest)
  int32_t hi, wi, ho, wo;
  int32_t x;             // filter width (a column's tap is (col / c) / x, (col / c) % x)
  int32_t stride_h, stride_w, pad_h, pad_w, dil_h, dil_w;
  int32_t pad_;
};

// Layout conversion of a 5-D tensor (the utility "converting copy" of the
// reference's multi-kernel flows, ConvGenerator.cpp:279-344): element (i0..i4)
// moves from src[sum i_d * src_stride[d]] to dst[sum i_d * dst_stride[d]].
// The destination may be longer than the source along a dimension (channel
// padding): positions at or beyond src_size read as zero.
enum RockRelayoutMode {
  RELAYOUT_TRANSPOSE = 0, // contiguous dimensions differ: tile_d x (1024/tile_d) tiles through LDS
  RELAYOUT_COPY = 1,      // one 16-byte destination chunk (along dimension 4) per thread
  RELAYOUT_TRANSPOSE_VEC = 2, // as TRANSPOSE with 16-byte accesses: tiles of tile_d x (AREA / tile_d), relayout_body.h
};
struct RockRelayoutParams {
  int64_t src_stride[5], dst_stride[5]; // in elements
  int32_t size[5];                      // of the destination
  int32_t src_size[5];
  int32_t src_fast, dst_fast; // dimension indices
  int32_t mode;               // RockRelayoutMode
  int32_t tile_d;             // tile extent along dst_fast (TRANSPOSE: 8, 16 or 32; TRANSPOSE_VEC: a power of two);
                              // COPY: positions of dimension 3 whose runs share one chunk (1: runs of whole chunks)
  // the divisors of the kernel's index decoding, in the order it divides by them.
  // TRANSPOSE, TRANSPOSE_VEC: tiles along src_fast, tiles along dst_fast, then the sizes of the other three
  // dimensions from the last to the first.  COPY: blocks per (i0, i1) pair, size[1], chunks per run,
  // chunk positions along dimension 3 (size[3] / tile_d).
  RockFastDiv div[5];
  // TRANSPOSE, TRANSPOSE_VEC: the same description resolved for the kernel, which then indexes nothing by
  // src_fast / dst_fast: the tiled dimensions (s = src_fast, d = dst_fast) and the other three from the last
  // to the first
  int64_t ss_s, ss_d, ds_s, ds_d;       // strides of the tiled dimensions in source / destination
  int64_t outer_ss[3], outer_ds[3];
  int32_t size_s, size_d, src_s, src_d; // destination extents and source extents of the tiled dimensions
  int32_t outer_size[3], outer_src[3];
  int32_t tiles_s, tiles_d;             // tiles along each
  int32_t ts_shift, td_shift;           // log2 of the tile extents
};

// rock_relayout_pair_b{1,2,4}(src0, dst0, src1, dst1, p): two conversions in one
// launch; blocks [0, first_blocks) run `first`, the others `second`.
struct RockRelayoutPairParams {
  RockRelayoutParams first, second;
  int32_t first_blocks;
  int32_t pad_;
};

// Utility kernels of the backward convolutions (the reference's zero-init and
// converting-copy utility kernels, ConvGenerator.cpp:279-344, 434-480).
// rock_fill_zero(dst, p): clears `bytes` bytes.
struct RockFillParams {
  int64_t bytes;
};
// rock_reduce_splits(partials, dst, p): partial sums of a K-split contraction,
// `splits` dense f32 arrays of size[0]*size[1]*size[2]*size[3] elements each
// `split_stride` elements apart, are added in split order and written in the
// destination's type to dst[sum i_d * dst_stride[d]].
struct RockReduceParams {
  int64_t split_stride;
  int64_t dst_stride[4];
  int32_t size[4];
  int32_t splits;
  int32_t out_dtype; // RockDType: f32, f16 or bf16
  int32_t valid[4];  // elements at or beyond valid[d] along dimension d are padding and are not written (0: none)
  int32_t int_partials; // 1: the partial sums and the result are int32 (out_dtype ROCK_I32)
  int32_t pad_;
};

// rock_fold_depth(T, dst, p): last step of the input gradient of a convolution
// over three spatial dimensions.  T[n, do, h, w, g, z, c] (c padded to cp,
// t_pix = g * z * cp elements per pixel) holds the gradient with the depth
// taps still unfolded; every input element (n, g, c, h, w, d) is the sum, in
// ascending z, of T at the (do, z) with do * stride_d + z * dil_d - pad_d == d,
// added in f32 and written once in the tensor's type at
// dst[n*s0 + g*s1 + c*s2 + h*s3 + w*s4 + d*s5].
struct RockFoldDepthParams {
  int64_t dst_stride[6];
  int64_t t_pix;
  int32_t n, g, c, cp, hi, wi, di, d_out, z;
  int32_t stride_d, dil_d, pad_d;
  int32_t dtype; // RockDType: f32, f16 or bf16
  int32_t pad_;
};

#define ROCK_ATTN_PROGRAM_MAX 24
#define ROCK_ATTN_PROGRAM_INPUTS 8
enum RockAttnOp : int32_t {
  ROCK_AOP_SCORE = 1,  // push the score
  ROCK_AOP_TENSOR = 2, // push element [g, i, j] of input tensor `argument`
  ROCK_AOP_CONST = 3,  // push consts[argument]
  ROCK_AOP_ADD = 10, ROCK_AOP_SUB, ROCK_AOP_MUL, ROCK_AOP_DIV, ROCK_AOP_MAX, ROCK_AOP_MIN, // a b -> a op b
  ROCK_AOP_EXP = 20, ROCK_AOP_NEG, ROCK_AOP_TANH, ROCK_AOP_SIGMOID, ROCK_AOP_RELU, ROCK_AOP_ABS, ROCK_AOP_ERF,
  ROCK_AOP_WHERE = 30, // c a b -> c != 0 ? a : b
};

// rock_softmax_rows(S, scale_tensor, bias, p): the middle kernel of attention
// run as three kernels (head dimensions beyond the fused kernel's, f32).  S
// holds G*seq_q rows of seq_k f32 scores, `row_pitch` floats apart; row by row
//   x_j = S_j * scale_tensor_j * scale + bias_j ; P_j = exp(x_j - max) / sum
// and P is written IN PLACE in the element type `dtype` from the start of the
// row (so rows of P are row_pitch * 4 bytes apart).
struct RockSoftmaxParams {
  int64_t row_pitch;
  int64_t t_gs, t_is, t_js; // element strides of the [g, i, j] scale tensor and bias
  int32_t G, seq_q, seq_k;
  float scale;
  int32_t has_bias, has_scale_tensor;
  int32_t dtype; // RockDType of P, the scale tensor and the bias: f32, f16 or bf16
  int32_t has_mask; // where(mask, score, other): an int8 mask and a tensor of `dtype`, both [g, i, j] like the bias
  // A pre-softmax element-wise program (the body of rock.attention's preSoftmaxBody region, RockOps.td:208-254,
  // which may hold any element-wise tree over the scores and further [g, i, j] tensors): postfix code for a
  // four-deep stack machine, run per score in f32.  prog_len = 0: the fixed chain above.
  int32_t prog_len;
  // P[i, seq_k .. seq_k_padded) is written as zeros (0: nothing): the second GEMM then reads rows of whole 16-byte chunks
  int32_t seq_k_padded;
  int32_t prog[ROCK_ATTN_PROGRAM_MAX]; // RockAttnOp | argument << 8
  float consts[ROCK_ATTN_PROGRAM_INPUTS];
  int32_t tensor_dtype[ROCK_ATTN_PROGRAM_INPUTS];      // RockDType of each input tensor (f32, f16, bf16, i8)
  const void *tensors[ROCK_ATTN_PROGRAM_INPUTS];       // written at launch from the caller's pointer list
  int64_t t_base;                                      // elements from the tensors' starts to this launch's first row
};

struct RockAttentionParams {
  // element strides of the logical views Q[g,i,d], K[g,j,d], V[g,j,e], O[g,i,e]
  int64_t q_gs, q_is, q_ds;
  int64_t k_gs, k_js, k_ds;
  int64_t v_gs, v_js, v_es;
  int64_t o_gs, o_is, o_es;
  int64_t bias_gs, bias_is, bias_js; // optional pre-softmax tensors [g,i,j]: additive bias, multiplicative scale
  int32_t G, seq_q, seq_k, d_qk, d_v;
  int32_t q_blocks;    // blocks of query rows per g
  float scale;         // multiplies Q*K^T before the softmax
  int32_t has_bias;
  int32_t xcd_remap;
  int32_t has_scale_tensor; // scores are multiplied element-wise by the scale tensor before `scale`
  int32_t zero_point;       // int8 Q and K: the scores are (int32 sum - zero_point) * scale
  // migraphx.where(mask, scores, other) in front of the softmax (mixr-attn-where.mlir:11): where the int8 mask
  // [g,i,j] is zero, the score (after scale tensor, scale and bias) is REPLACED by other[g,i,j]
  int32_t has_mask;
};
