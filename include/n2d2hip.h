/*
 * n2d2hip.h - C ABI of the MI355X (gfx950) implementation of N2D2's quantized
 * inference hot path ("Frame_HIP" model).
 *
 * Plain C: opaque handles, plain pointers and sizes, int status codes
 * (0 = success).  No exceptions cross this boundary; the C++ cell glue turns a
 * non-zero status into std::runtime_error(n2d2hip_last_error()), which is how
 * the reference reports errors.  All tensors are caller-owned DEVICE buffers
 * unless a parameter is documented as HOST.  Every call takes an explicit HIP
 * stream (hipStream_t passed as void*) and is asynchronous on it.
 *
 * Citations "ref: file:line" name the N2D2 (v1.3.0) interface an entry point
 * replaces; paths are relative to the N2D2 source tree.
 */
#ifndef N2D2HIP_H
#define N2D2HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef void* n2d2hip_stream_t; /* hipStream_t */

/* ---------------------------------------------------------------- status */
enum {
    N2D2HIP_OK = 0,
    N2D2HIP_ERR_INVALID = 1,       /* null pointer, shape mismatch, bad enum */
    N2D2HIP_ERR_UNSUPPORTED = 2,   /* valid in N2D2 but outside this path */
    N2D2HIP_ERR_HIP = 3,           /* a HIP runtime call failed */
    N2D2HIP_ERR_NOT_QUANTIZED = 4, /* integer rescale on nb_bits == 0 (the reference throws) */
    N2D2HIP_ERR_WORKSPACE = 5      /* workspace too small */
};
const char* n2d2hip_strerror(int status);
/* Message of the last failing call on the calling thread ("" if none). */
const char* n2d2hip_last_error(void);
/* Library version string and the gfx target the kernels were built for. */
const char* n2d2hip_version(void);

/* Diagnostic, no counterpart in the reference: the engine clock in MHz the GPU holds while every CU runs int8 matrix
 * instructions for about `busy_microseconds` (shader clocks per tick of the constant 100 MHz counter, read inside a
 * kernel).  Published matrix-core peaks assume the maximum clock; a measured fraction of the peak is read against this.
 * Allocates a small device buffer and waits for the stream. */
int n2d2hip_measure_clock(double busy_microseconds, double* mhz, n2d2hip_stream_t stream);

/* Diagnostic, no counterpart in the reference: the launch log of the calling thread.  Between _begin and _end every kernel
 * the library launches from this thread is recorded (the launches still happen); afterwards _entry gives launch `index`:
 * the kernel's name with its template arguments ("conv_pipe_kernel<4, 128, ...>", truncated to `capacity`), its grid
 * and block sizes in threads-groups / threads, and the index of its first record in a probe buffer (-1 outside probe builds,
 * see n2d2hip_probe.h).  It is how a caller learns which kernel a cell runs on without restating the library's choice. */
int n2d2hip_launch_log_begin(void);
int n2d2hip_launch_log_end(int* count);
int n2d2hip_launch_log_entry(int index, char* name, size_t capacity, int* grid, int* block, long long* probe_slot);

/* --------------------------------------------------------------- tensors */
/* Element types.  N2D2 holds integer values in float storage
 * (ref: src/Cell/ConvCell_Frame.cpp:28-44); here they are stored narrow. */
enum {
    N2D2HIP_U8 = 0,  /* unsigned 8-bit value */
    N2D2HIP_I8 = 1,  /* signed 8-bit value */
    N2D2HIP_I32 = 2, /* signed 32-bit value (accumulators, logits) */
    N2D2HIP_F32 = 3, /* float holding an integer value (graph edges) */
    N2D2HIP_U8B = 4  /* unsigned 8-bit value v stored as the signed byte v-128:
                        the form the signed int8 matrix cores consume */
};
/* Layouts.  NCHW is N2D2's Tensor order {X,Y,Z,B}, X fastest
 * (ref: include/containers/Tensor.hpp:162-193).  NHWC is the private
 * channel-inner order used between Frame_HIP cells; its channel stride `cs`
 * is a multiple of 16 (4 is accepted for network inputs with <= 4 channels). */
enum {
    N2D2HIP_NCHW = 0,
    N2D2HIP_NHWC = 1,
    /* Space-to-depth form of a network input with at most 4 channels, read by first-layer convolutions of stride 2
     * (n2d2hip_conv_s2d_halo): pixel (Y, X) of the stored image is 16 bytes, the 2 x 2 block of input pixels
     * (2Y + dy, 2X + dx) with 4 channel slots each, byte (dy * 2 + dx) * 4 + channel; an image is stored as
     * (ceil(H/2) + 2*halo) x (ceil(W/2) + 2*halo) such pixels.  Whatever lies outside the H x W input (the border, an odd
     * last row / column, the channel slots past C) holds the storage form of 0.  B, C, H, W stay the logical shape, cs is
     * 16.  Only n2d2hip_convert writes it (border included, so no n2d2hip_tensor_clear is needed) and only
     * n2d2hip_conv_forward / n2d2hip_conv_forward_maxpool read it.  No counterpart in the reference, whose first layer
     * reads the float NCHW stimuli directly. */
    N2D2HIP_S2D = 2
};

typedef struct n2d2hip_tensor {
    void* data;
    int dtype;  /* N2D2HIP_U8 ... */
    int layout; /* N2D2HIP_NCHW / N2D2HIP_NHWC */
    int B, C, H, W;
    int cs;     /* NHWC: bytes-per-pixel channel stride in elements (>= C); NCHW: ignored */
    /* NHWC byte tensors between two convolutions may carry their padding physically: every image is stored as
     * (H + 2*halo) x (W + 2*halo) pixels, `data` points at the first border pixel, and the border holds the storage form
     * of the value 0 (n2d2hip_tensor_clear writes it; nothing writes there afterwards).  A convolution whose padding is
     * not larger than the halo then reads every tap of every window from memory, which is what the reference's tap-skipping
     * loop computes (ref: src/Cell/ConvCell_Frame_Kernels.cpp:72-83: a skipped tap adds nothing, as a tap on a zero does).
     * 0 everywhere else; only the entry points that say so accept a halo. */
    int halo;
} n2d2hip_tensor;

/* Channel stride the library uses for an NHWC tensor with C channels. */
int n2d2hip_nhwc_cs(int C);
/* Bytes needed for a tensor (uses cs for NHWC, and the halo). */
size_t n2d2hip_tensor_bytes(const n2d2hip_tensor* t);
/* Fills the whole buffer of a byte tensor, halo included, with the storage form of the value 0 (a kernel launch, no memset:
 * it can be captured).  To be called once on a tensor with a halo before its producer first runs. */
int n2d2hip_tensor_clear(const n2d2hip_tensor* t, n2d2hip_stream_t stream);

/* Graph-edge conversion between any two dtype/layout combinations of the same
 * logical shape (e.g. F32 NCHW <-> U8B NHWC).  Values that do not fit the
 * destination type are saturated.  Channels C..cs-1 of an NHWC destination
 * are written as logical zero. */
int n2d2hip_convert(const n2d2hip_tensor* in, const n2d2hip_tensor* out, n2d2hip_stream_t stream);

/* ------------------------------------------------- scaling + activation */
/* ref: include/ScalingMode.hpp:27-62 (same order as N2D2::ScalingMode) */
enum {
    N2D2HIP_SCALING_NONE = 0,
    N2D2HIP_SCALING_FLOAT_MULT = 1,
    N2D2HIP_SCALING_FIXED_MULT16 = 2,
    N2D2HIP_SCALING_FIXED_MULT32 = 3,
    N2D2HIP_SCALING_SINGLE_SHIFT = 4,
    N2D2HIP_SCALING_DOUBLE_SHIFT = 5
};
enum { N2D2HIP_ACT_LINEAR = 0, N2D2HIP_ACT_RECTIFIER = 1 };

/* What an N2D2 Activation carries on the quantized path
 * (ref: include/Activation/Activation.hpp:36-110, include/Scaling.hpp:336-432).
 * All pointers are HOST pointers to per-output-channel vectors. */
typedef struct n2d2hip_activation {
    int kind;               /* N2D2HIP_ACT_LINEAR / N2D2HIP_ACT_RECTIFIER */
    float leak_slope;       /* Rectifier LeakSlope; must be 0 on the integer path */
    int scaling_mode;       /* N2D2HIP_SCALING_* */
    const void* scaling;    /* FLOAT_MULT: float[C]; FIXED_*: int32_t[C];
                               SINGLE_SHIFT: uint8_t[C]; DOUBLE_SHIFT: uint8_t[C][2] = {first, second} */
    int frac_bits;          /* FIXED_*: nbFractionalBits (one value per cell) */
    int is_clipped;         /* FLOAT_MULT / FIXED_*: apply Clip before the rescale */
    const float* clipping;  /* float[C] when is_clipped */
    int nb_bits;            /* quantizedNbBits handed to Scaling::propagate: the activation's
                               bits if set, else the cell's (ref: RectifierActivation_Frame.hpp:65-66) */
    int unsigned_out;       /* DeepNetExport::isCellOutputUnsigned(cell) (ref: src/Export/DeepNetExport.cpp:370-388) */
} n2d2hip_activation;

typedef struct n2d2hip_act_s* n2d2hip_act_t;

/* Builds the per-channel device tables for `Scaling::propagate` followed by
 * the Rectifier / Linear pass (ref: include/Scaling.hpp:434-459,
 * src/Scaling_Kernels.cpp:29-199, include/Activation/RectifierActivation_Frame.hpp:55-87,
 * include/Activation/LinearActivation_Frame.hpp:56-81). */
int n2d2hip_act_create(const n2d2hip_activation* desc, int nb_channels, n2d2hip_act_t* act);
int n2d2hip_act_destroy(n2d2hip_act_t act);

/* Stand-alone Scaling (+ activation) over a tensor: ScalingCell_Frame::propagate
 * (ref: src/Cell/ScalingCell_Frame.cpp:67-75) and the tail of Cell_Frame::propagate
 * (ref: src/Cell/Cell_Frame.cpp:473-478).  `in` is U8/I8/U8B/I32/F32 of either layout,
 * `out` has the same layout and shape. */
int n2d2hip_scaling_forward(n2d2hip_act_t act, const n2d2hip_tensor* in, const n2d2hip_tensor* out,
                            n2d2hip_stream_t stream);

/* ------------------------------------------------------------------ conv */
/* ref: include/Cell/ConvCell_Frame_Kernels.hpp:40-54 (Descriptor), include/Cell/ConvCell.hpp:45-55 */
typedef struct n2d2hip_conv_desc {
    int C, O;               /* input channels, output channels */
    int kW, kH;
    int strideX, strideY;
    int padL, padT, padR, padB;
    int dilX, dilY;
    int groups;             /* Cell::getNbGroups of the mapping (ref: src/Cell/Cell.cpp:251-300): G equal groups, weights
                               [O][C/G][kH][kW] (ConvCell_Frame_Kernels.cpp:89-96).  G == C == O (depthwise) has its own
                               kernels; 1 < G otherwise runs as a full connection with zeros outside the groups */
    int weight_bits;        /* 8: int8_t weights; 4: two weights per byte, element 2i in the low nibble */
    int kernel_choice;      /* 0: the library chooses among its kernels.  Otherwise N2D2HIP_KERNEL_* bits, which only steer
                               that choice among kernels that compute the same result (tests use them to cover every
                               kernel); read from the descriptor when the cell is created (integer cells) or on each call
                               (float passes: give the same value to n2d2hip_conv2d_f32_workspace_bytes and to the pass).
                               No counterpart in the reference. */
    int subX, subY;         /* Descriptor::subSample (ref: src/Cell/ConvCell_Frame_Kernels.cpp:46-52,135-140): the sums of
                               subX x subY neighbouring positions are added up into one output (the last window of a row
                               or column may hold fewer), the bias is added once and the activation applied to that;
                               0 or 1: none.  Integer cells only; such a cell runs as the convolution proper plus one
                               launch that adds the windows up, and takes part in no graph-level fusion */
} n2d2hip_conv_desc;
enum {
    N2D2HIP_KERNEL_NO_PIPE = 1,     /* integer cells: general register-staged kernel instead of the pipelined one */
    N2D2HIP_KERNEL_NO_STEM = 2,     /* no first-layer kernel */
    N2D2HIP_KERNEL_NO_HI16 = 4,     /* 32-bit rescale epilogue instead of the scaled-up 16-bit one */
    N2D2HIP_KERNEL_NO_SUM16 = 8,    /* folded residual sum on 32 bits (read by n2d2hip_conv_fuse_sum) */
    N2D2HIP_KERNEL_TILE_M64 = 16,   /* force 64-pixel tiles */
    N2D2HIP_KERNEL_TILE_M128 = 32,  /* force 128-pixel tiles */
    N2D2HIP_KERNEL_F32_DIRECT = 64, /* float passes: direct kernels that add in the reference's order */
    N2D2HIP_KERNEL_F32_GEMM = 128,  /* float passes: matrix-core implicit GEMM */
    N2D2HIP_KERNEL_NO_PATCH = 256,  /* integer cells: 3x3 convolutions on the pipelined kernel instead of the patch kernel */
    N2D2HIP_KERNEL_PATCH = 512,     /* the patch kernel wherever it can run, also where the library finds the pipelined one faster */
    N2D2HIP_KERNEL_NO_DIRECT = 1024,/* integer cells with at most 4 input channels and 32 outputs: matrix-core kernel instead of the direct one */
    N2D2HIP_KERNEL_DIRECT = 2048,   /* the direct kernel wherever it can run (up to 16 input channels), also where the library finds the matrix cores faster */
    N2D2HIP_KERNEL_TILE_M256 = 4096 /* patch kernel: tiles of 256 positions (N2D2HIP_KERNEL_TILE_M128: of 128; _M64: four waves of 64 positions) instead of its own choice */
};

typedef struct n2d2hip_conv_s* n2d2hip_conv_t;

/* Prepares a quantized ConvCell: weights HOST int8 OCHW ({kW,kH,C/groups,O}, kW fastest;
 * nibble-packed in the same order when weight_bits == 4), bias HOST int32[O] or NULL
 * (NoBias).  `act` is borrowed and must outlive the conv.  `in_dtype` is the element
 * type the cell will be fed (U8B, I8 or U8), fixed at creation.
 * Replaces ConvCell_Frame<T>::initialize + propagate
 * (ref: src/Cell/ConvCell_Frame.cpp:418-473, src/Cell/ConvCell_Frame_Kernels.cpp:26-174). */
int n2d2hip_conv_create(const n2d2hip_conv_desc* desc, const void* weights, const int32_t* bias,
                        n2d2hip_act_t act, int in_dtype, n2d2hip_conv_t* conv);
int n2d2hip_conv_destroy(n2d2hip_conv_t conv);
/* Output spatial size (ref: src/Cell/ConvCell.cpp:1169-1195), sub-sampling included. */
int n2d2hip_conv_out_dims(const n2d2hip_conv_desc* desc, int H, int W, int* outH, int* outW);
/* in / out: NHWC with the channel stride of n2d2hip_nhwc_cs (4 for at most 4 channels, a multiple of 16 otherwise).  out dtype U8B/U8/I8 (rescaled) or I32 (scaling NONE).  `in` and a byte `out`
 * may have a halo if n2d2hip_conv_accepts_halo says so. */
int n2d2hip_conv_forward(n2d2hip_conv_t conv, const n2d2hip_tensor* in, const n2d2hip_tensor* out,
                         n2d2hip_stream_t stream);
/* Border (halo) a space-to-depth input of logical size H x W must carry for this convolution to read it
 * (n2d2hip_conv_forward then takes `in` with layout N2D2HIP_S2D; with `pool` non-null the question is about
 * n2d2hip_conv_forward_maxpool with that pooling behind the convolution), or -1 when it is not served that way.
 * Served: at most 4 input channels, 8-bit weights, a square kernel of 3, 5 or 7, stride 2, no dilation, at most 64
 * outputs, integer rescale to bytes, bordered rows of at most 128 pixels; with a pooling, what
 * n2d2hip_conv_accepts_maxpool asks and at most 62 pooled columns.  No counterpart in the reference: the stride-2
 * K x K window becomes a stride-1 window of ceil(K / 2)^2 16-byte pixels whose padding is the border of stored zeros
 * (ref: src/Cell/ConvCell_Frame_Kernels.cpp:72-83 skips those taps). */
struct n2d2hip_pool_desc;
int n2d2hip_conv_s2d_halo(n2d2hip_conv_t conv, const struct n2d2hip_pool_desc* pool, int H, int W);
/* 1 if this convolution runs on the kernel that reads and writes tensors with a halo (8-bit weights, ungrouped, input
 * channels a multiple of 64), else 0.  No counterpart in the reference, whose padding is implicit in its tap loop. */
int n2d2hip_conv_accepts_halo(n2d2hip_conv_t conv);
/* The part of that rule a planner can ask before the cell exists, from the descriptor alone: 1 if a convolution of this
 * shape can be one that n2d2hip_conv_accepts_halo accepts (ungrouped, 4- or 8-bit weights, input channels a multiple of 64,
 * at most 31 taps, no dilation, no sub-sampling, more than 4 outputs), else 0.  n2d2hip_conv_accepts_halo has the last word (it also knows
 * the cell's rescale).  No counterpart in the reference. */
int n2d2hip_conv_desc_reads_halo(const n2d2hip_conv_desc* desc);


/* -------------------------------------------------------------------- fc */
typedef struct n2d2hip_conv_s* n2d2hip_fc_t;
/* Quantized FcCell over a C x H x W input: weights HOST int8 [O][C*H*W] in N2D2's CHW
 * flattening, bias HOST int32[O] or NULL.  Executed as a convolution whose kernel spans
 * the input (ref: src/Cell/FcCell_Frame.cpp:234-340). */
int n2d2hip_fc_create(int C, int H, int W, int O, int weight_bits, const void* weights, const int32_t* bias,
                      n2d2hip_act_t act, int in_dtype, n2d2hip_fc_t* fc);
int n2d2hip_fc_destroy(n2d2hip_fc_t fc);
int n2d2hip_fc_forward(n2d2hip_fc_t fc, const n2d2hip_tensor* in, const n2d2hip_tensor* out,
                       n2d2hip_stream_t stream);

/* Graph-level fusion of a classifier head: two or three FcCells, each after the first reading the 1 x 1 output of the one
 * before and nothing else reading it, in one launch; that is FcCell_Frame::propagate two or three times
 * (ref: src/Cell/FcCell_Frame.cpp:234-340) with the vectors between the cells kept on the chip; results are those of the
 * cells run in turn, bit for bit (same int32 sums, same rescale).  The handles are borrowed, must outlive the chain and
 * stay usable on their own.  Returns N2D2HIP_ERR_UNSUPPORTED (the caller keeps the separate launches) unless every cell
 * has 8-bit weights, at most 1024 inputs and at most 128 outputs.  `in`: the first cell's input (NHWC bytes, as
 * n2d2hip_fc_forward takes it); `out`: the last cell's output. */
typedef struct n2d2hip_fc_chain_s* n2d2hip_fc_chain_t;
int n2d2hip_fc_chain_create(int nb_cells, const n2d2hip_fc_t* cells, n2d2hip_fc_chain_t* chain);
int n2d2hip_fc_chain_destroy(n2d2hip_fc_chain_t chain);
int n2d2hip_fc_chain_forward(n2d2hip_fc_chain_t chain, const n2d2hip_tensor* in, const n2d2hip_tensor* out,
                             n2d2hip_stream_t stream);

/* ------------------------------------------------------------------ pool */
enum { N2D2HIP_POOL_MAX = 0, N2D2HIP_POOL_AVERAGE = 1 };
/* ref: include/Cell/PoolCell_Frame_Kernels.hpp (Descriptor), include/Cell/PoolCell.hpp:47-55 */
typedef struct n2d2hip_pool_desc {
    int pooling;            /* N2D2HIP_POOL_MAX / N2D2HIP_POOL_AVERAGE */
    int poolW, poolH;
    int strideX, strideY;
    int padX, padY;
} n2d2hip_pool_desc;
int n2d2hip_pool_out_dims(const n2d2hip_pool_desc* desc, int H, int W, int* outH, int* outW);
/* Per-channel (unit map) quantized pooling on NHWC U8/I8/U8B; average is the truncated
 * quotient sum / (poolW*poolH) (ref: src/Cell/PoolCell_Frame_Kernels.cpp:26-197,
 * src/Cell/PoolCell_Frame.cpp:123-174).  out has the dtype of in; a 2x2 or 3x3 max pooling whose channel stride is a
 * multiple of 16 may write an `out` with a halo (its readers' padding), the other poolings refuse one. */
int n2d2hip_pool_forward(const n2d2hip_pool_desc* desc, const n2d2hip_tensor* in, const n2d2hip_tensor* out,
                         n2d2hip_stream_t stream);
/* 1 if n2d2hip_pool_forward with this descriptor on an NHWC byte tensor of H x W pixels and channel stride `cs` writes an
 * output with a halo (the rule above, and every window holding at least one input element), else 0: what a planner asks
 * before it gives a pooling's output a border.  No counterpart in the reference. */
int n2d2hip_pool_writes_halo(const n2d2hip_pool_desc* desc, int H, int W, int cs);

/* Pooling with a connection map (ref: src/Cell/PoolCell_Frame_Kernels.cpp:60-75,150-185, the `maps` argument of forwardMax /
 * forwardAverage): output o pools its window over every input channel c with maps[o * map_channels + c] != 0 (`maps`:
 * map_outputs x map_channels bytes in device memory, which must be the tensors' out->C x in->C: the call refuses any other
 * size instead of reading past the map), the average dividing by window size x connected channels.  An output without a
 * connected channel is 0.  `out` has out->C outputs in the dtype of `in`, no halo. */
int n2d2hip_pool_forward_mapped(const n2d2hip_pool_desc* desc, const unsigned char* maps, int map_outputs, int map_channels,
                                const n2d2hip_tensor* in, const n2d2hip_tensor* out, n2d2hip_stream_t stream);

/* Graph-level fusion of a first-layer convolution with the max pooling behind it: ConvCell_Frame::propagate followed by
 * PoolCell_Frame_Kernels::forwardMax (ref: src/Cell/ConvCell_Frame.cpp:418-473, src/Cell/PoolCell_Frame_Kernels.cpp:102-197)
 * in one launch; the convolution's own output is never stored.  n2d2hip_conv_accepts_maxpool says whether the library takes
 * the pair for an H x W input: a convolution on the first-layer kernel (at most 4 input channels, horizontal stride 2, at
 * most 64 output channels, rows of at most 128 outputs, integer rescale to bytes) and a 3x3 stride-2 max pooling with
 * padding 0 or 1.  `out` is the pooled tensor (channel stride 64), with or without a halo. */
int n2d2hip_conv_accepts_maxpool(n2d2hip_conv_t conv, const n2d2hip_pool_desc* pool, int H, int W);
int n2d2hip_conv_forward_maxpool(n2d2hip_conv_t conv, const n2d2hip_pool_desc* pool, const n2d2hip_tensor* in,
                                 const n2d2hip_tensor* out, n2d2hip_stream_t stream);

/* -------------------------------------------------------------- elemwise */
enum { N2D2HIP_COEFF_PER_LAYER = 0, N2D2HIP_COEFF_PER_INPUT = 1, N2D2HIP_COEFF_PER_CHANNEL = 2 };
typedef struct n2d2hip_elemwise_s* n2d2hip_elemwise_t;
/* ElemWiseCell Sum: out = act( w[c0]*in0 + s[c0] + sum_k (w[c1]*in_k + s[c1]) ), float
 * coefficient arithmetic exactly as the reference (ref: src/Cell/ElemWiseCell_Frame.cpp:116-136).
 * weights / shifts: HOST float vectors already sized as ElemWiseCell_Frame::initialize leaves
 * them (nb_inputs entries, or C entries for PER_CHANNEL); NULL means all 1 / all 0. */
int n2d2hip_elemwise_create(int nb_inputs, int nb_channels, int coeff_mode, const float* weights,
                            const float* shifts, n2d2hip_act_t act, n2d2hip_elemwise_t* ew);
/* Graph-level fusion: folds the ScalingCell that feeds input `input_index` into this cell.  That input is then
 * the ScalingCell's own input and the Scaling is applied on the fly, i.e. ScalingCell_Frame::propagate
 * (ref: src/Cell/ScalingCell_Frame.cpp:67-75) followed by ElemWiseCell_Frame::propagate in one pass, without
 * materialising the rescaled tensor.  `scaling` (built with n2d2hip_act_create, kind LINEAR) is borrowed; NULL undoes
 * the fold.  Returns N2D2HIP_ERR_UNSUPPORTED (and folds nothing) unless the sum has unit coefficients and the Scaling is
 * an integer mode whose products fit 32 bits: the caller then keeps the ScalingCell as a separate launch. */
int n2d2hip_elemwise_fold_input_scaling(n2d2hip_elemwise_t ew, int input_index, n2d2hip_act_t scaling);
int n2d2hip_elemwise_destroy(n2d2hip_elemwise_t ew);

/* Graph-level fusion: the two-input ElemWise sum that consumes this convolution's output is computed in the
 * convolution's epilogue, i.e. ConvCell_Frame::propagate followed by ElemWiseCell_Frame::propagate (Sum)
 * (ref: src/Cell/ConvCell_Frame.cpp:418-473, src/Cell/ElemWiseCell_Frame.cpp:104-136) in one launch; the convolution's
 * own output tensor is never written.  `conv_input_index` (0 or 1) is the sum's input the convolution feeds; the other
 * input is passed to n2d2hip_conv_forward_sum and has storage type `other_dtype`.  A ScalingCell folded into the sum
 * with n2d2hip_elemwise_fold_input_scaling must sit on that other input and is applied too.  `sum` is borrowed and must
 * outlive the convolution; NULL undoes the fusion.  Returns N2D2HIP_ERR_UNSUPPORTED (and changes nothing) unless the
 * convolution is 1x1, unpadded and 8-bit, or undilated with 4-bit weights, with input and output channel counts that are
 * multiples of 64, and both cells rescale with an integer Scaling mode: the caller then keeps the two launches. */
int n2d2hip_conv_fuse_sum(n2d2hip_conv_t conv, n2d2hip_elemwise_t sum, int conv_input_index, int other_dtype);
/* out = sum(conv(in), other) for a convolution prepared with n2d2hip_conv_fuse_sum; `out` has the sum cell's range.
 * `in`, `other` and `out` may each carry a border of zeros of their own (halo). */
int n2d2hip_conv_forward_sum(n2d2hip_conv_t conv, const n2d2hip_tensor* in, const n2d2hip_tensor* other,
                             const n2d2hip_tensor* out, n2d2hip_stream_t stream);
int n2d2hip_elemwise_forward(n2d2hip_elemwise_t ew, const n2d2hip_tensor* const* inputs, const n2d2hip_tensor* out,
                             n2d2hip_stream_t stream);

/* The channels of 1 to 8 NHWC byte tensors of one dtype and size, one input behind the other, into `out` (whose C is the
 * sum of theirs).  ref: src/Cell/ConvCell_Frame.cpp:438-459: a cell with several inputs adds up one weighted sum per input,
 * each with its own slice of the weights (Cell::getNbChannels counts all inputs' channels), which is the convolution of
 * the concatenated channels; this is the one extra launch such a cell costs here.  Inputs and output may carry a halo;
 * only the interior of `out` is written. */
int n2d2hip_concat_channels(int nb_inputs, const n2d2hip_tensor* const* inputs, const n2d2hip_tensor* out,
                            n2d2hip_stream_t stream);

/* Graph-level fusion of a residual bottleneck with 64 middle channels into one launch: `reduce` (1x1, 64 or 256 -> 64),
 * `conv3x3` (3x3, stride 1, padding 1, 64 -> 64) and, unless `expand` is NULL, `expand` (1x1, 64 -> 256) with the two-input
 * ElemWise sum that n2d2hip_conv_fuse_sum has folded into it; the sum's other input is the block's input itself (256
 * channels, through the ScalingCell folded into the sum if there is one) or, if `projection` is not NULL, that 1x1
 * convolution (64 -> 256) of the block's input.  That is ConvCell_Frame::propagate three or four times and
 * ElemWiseCell_Frame::propagate (ref: src/Cell/ConvCell_Frame.cpp:418-473, src/Cell/ElemWiseCell_Frame.cpp:104-136) without
 * the tensors in between ever reaching memory; results are those of the separate cells, bit for bit.  The handles are
 * borrowed, must outlive the bottleneck and stay usable on their own.  Returns N2D2HIP_ERR_UNSUPPORTED (the caller keeps
 * the separate launches) unless every cell is 8-bit with an integer rescale that fits the scaled-up tables, and the sum
 * runs on 16-bit pairs. */
typedef struct n2d2hip_bottleneck_s* n2d2hip_bottleneck_t;
int n2d2hip_bottleneck_create(n2d2hip_conv_t reduce, n2d2hip_conv_t conv3x3, n2d2hip_conv_t expand, n2d2hip_conv_t projection,
                              n2d2hip_bottleneck_t* bottleneck);
int n2d2hip_bottleneck_destroy(n2d2hip_bottleneck_t bottleneck);
/* 1 where the one launch is expected to be faster than the plan the cells would otherwise run in, for `batch` images of
 * in_h x in_w pixels: today a block with a projection shortcut (one launch for four); a block without one is as fast as
 * its reduce convolution followed by n2d2hip_conv_chain_forward.  Planners ask this instead of restating the rule. */
int n2d2hip_bottleneck_pays(n2d2hip_bottleneck_t bottleneck, int batch, int in_h, int in_w);
/* `in`: the block's input, NHWC bytes with a border of one pixel (halo 1; rows of at most 61 pixels); `out`: the sum's
 * output (the 3x3 convolution's when `expand` is NULL), NHWC bytes of the same height and width, with or without a border. */
int n2d2hip_bottleneck_forward(n2d2hip_bottleneck_t bottleneck, const n2d2hip_tensor* in, const n2d2hip_tensor* out,
                               n2d2hip_stream_t stream);

/* Graph-level fusion of the second half of a residual bottleneck into one launch: `conv3x3` (3x3, stride 1 or 2, padding 1,
 * C -> C channels, C = 64, 128 or 256), the only reader of whose output is `expand` (1x1, C -> 4C) with the two-input
 * ElemWise sum that n2d2hip_conv_fuse_sum has folded into it.  That is ConvCell_Frame::propagate twice and
 * ElemWiseCell_Frame::propagate (ref: src/Cell/ConvCell_Frame.cpp:418-473, src/Cell/ElemWiseCell_Frame.cpp:104-136) without
 * the 3x3 convolution's output ever reaching memory; results are those of the separate cells, bit for bit.  Nothing is
 * created: the two handles stay usable on their own.  n2d2hip_conv_chain_supported returns 1 when the pair can run so (both
 * cells 8-bit with integer rescales that fit the scaled-up tables, the sum on 16-bit pairs), else 0: the caller then keeps
 * the separate launches.  `in`: the 3x3 convolution's input, NHWC bytes that carry the padding as a border (halo >= 1);
 * `other`: the sum's other input; `out`: the sum's output; the last two with or without a border. */
int n2d2hip_conv_chain_supported(n2d2hip_conv_t conv3x3, n2d2hip_conv_t expand);
int n2d2hip_conv_chain_forward(n2d2hip_conv_t conv3x3, n2d2hip_conv_t expand, const n2d2hip_tensor* in, const n2d2hip_tensor* other,
                               const n2d2hip_tensor* out, n2d2hip_stream_t stream);

/* Graph-level fusion of the MobileNet building block: `depthwise` (3x3, groups == channels, stride 1 or 2, undilated) and
 * `pointwise` (1x1, stride 1, unpadded), the only reader of its output.  That is ConvCell_Frame::propagate twice
 * (ref: src/Cell/ConvCell_Frame.cpp:418-473, kernels src/Cell/ConvCell_Frame_Kernels.cpp:26-179) in one launch: the
 * depthwise output goes from the vector ALU through LDS straight into the matrix cores and is never written to memory;
 * results are those of the separate cells, bit for bit.  The handles are borrowed, must outlive this one and stay usable
 * on their own.  Returns N2D2HIP_ERR_UNSUPPORTED (the caller keeps the separate launches) unless both cells are 8-bit
 * with integer rescales (32-bit multiply-add) and byte outputs, over 32 or a multiple of 64 channels, to 64, 128 or a
 * multiple of 256 channels. */
typedef struct n2d2hip_dw_pw_s* n2d2hip_dw_pw_t;
int n2d2hip_dw_pw_create(n2d2hip_conv_t depthwise, n2d2hip_conv_t pointwise, n2d2hip_dw_pw_t* fused);
int n2d2hip_dw_pw_destroy(n2d2hip_dw_pw_t fused);
/* 1 when the one launch is expected to be faster than the two cells' own on `batch` inputs of in_h x in_w (measured rule:
 * at most 256 outputs and at least 32768 output pixels), else 0.  No counterpart in the reference: a planner's question
 * (DeepNet::planFusion asks it). */
int n2d2hip_dw_pw_pays(n2d2hip_dw_pw_t fused, int batch, int in_h, int in_w);
/* `in`: input of `depthwise`; `out`: output of `pointwise`.  NHWC bytes without a border, channel stride equal to the
 * channel count. */
int n2d2hip_dw_pw_forward(n2d2hip_dw_pw_t fused, const n2d2hip_tensor* in, const n2d2hip_tensor* out, n2d2hip_stream_t stream);

/* --------------------------------------------------- SAT / LSQ fake-quant */
/* Weight quantizer modes, numbered as SATQuantizerCell_Frame::propagate selects them
 * (ref: src/Quantizer/QAT/Cell/SAT/SATQuantizerCell_Frame.cpp:188-200). */
enum {
    N2D2HIP_SAT_NONE = 0, N2D2HIP_SAT_DEFAULT = 1, N2D2HIP_SAT_FULLRANGE = 2,
    N2D2HIP_SAT_SYMRANGE = 3, N2D2HIP_SAT_ASYMRANGE = 4, N2D2HIP_SAT_NONE_ASYM = 5
};
/* Bytes of device scratch the SAT/LSQ entry points need for their reductions. */
size_t n2d2hip_quantizer_workspace_bytes(size_t n);
/* tanh-normalised DoReFa weight fake-quant, optional SAT scaling
 * (ref: src/Quantizer/QAT/Kernel/SATQuantizer_Frame_Kernels.cpp:66-262).
 * stats (device float[2]) receives {tanh_max, sat_scaling}. */
int n2d2hip_sat_weight_forward(const float* w, float* wq, size_t n, float range, int mode,
                               int apply_scaling, unsigned outputs_size, float* stats,
                               void* workspace, size_t workspace_bytes, n2d2hip_stream_t stream);
/* The same quantizer for callers that cannot allocate device memory or pass a workspace (code under HIP graph capture,
 * tight serving loops, harnesses that forbid hipMalloc): no counterpart in the reference.  The reductions' scratch (8448
 * bytes) is a static array in device memory that every GPU the library runs on holds until the process ends; the call
 * allocates nothing, on the host or on the device (the array's address is looked up once per device, on the first call
 * there).  Same arguments and results as n2d2hip_sat_weight_forward without the workspace; tensors of more than
 * N2D2HIP_SAT_STATIC_MAX_WEIGHTS elements are rejected with N2D2HIP_ERR_UNSUPPORTED.  All calls on one GPU share the one
 * array: calls that overlap on a GPU (two streams, two threads) race; calls on one stream are ordered and safe. */
#define N2D2HIP_SAT_STATIC_MAX_WEIGHTS (1u << 28)
int n2d2hip_sat_weight_forward_static(const float* w, float* wq, size_t n, float range, int mode, int apply_scaling,
                                      unsigned outputs_size, float* stats, n2d2hip_stream_t stream);
/* ref: SATQuantizer_Frame_Kernels.cpp:349-404; factor = tanh_max * scaling read from stats */
int n2d2hip_sat_weight_backward(const float* diff_wq, const float* w, float* diff_w, size_t n, float range,
                                int mode, int apply_scaling, const float* stats, n2d2hip_stream_t stream);
/* ref: SATQuantizer_Frame_Kernels.cpp:268-322; alpha: device float[1]; fp_copy NULL when inference */
int n2d2hip_sat_act_forward(float* x, float* fp_copy, size_t n, float range, const float* alpha,
                            n2d2hip_stream_t stream);
/* ref: SATQuantizer_Frame_Kernels.cpp:410-448 + SATQuantizerActivation_Frame.cpp:133-135:
 * diff_alpha[0] = sum_i dalpha_i + beta * diff_alpha[0]; diff_in and diff_out may be the same buffer (the cells apply
 * an activation's backward in place) */
int n2d2hip_sat_act_backward(const float* diff_in, const float* fp_x, float* diff_out, size_t n, float range,
                             const float* alpha, float beta, float* diff_alpha,
                             void* workspace, size_t workspace_bytes, n2d2hip_stream_t stream);
/* LSQ forward for weights (lo,hi) = (-(R+1)/2,(R-1)/2) and activations (0,R); step: device float[1]
 * (ref: src/Quantizer/QAT/Cell/LSQ/LSQQuantizerCell_Frame.cpp:194-208,
 *       src/Quantizer/QAT/Activation/LSQ/LSQQuantizerActivation_Frame.cpp:131-141). */
int n2d2hip_lsq_forward(const float* x, float* xq, size_t n, const float* step, int lo, int hi,
                        n2d2hip_stream_t stream);
/* STE mask + step-size gradient.  diff_step[0] = (sum_i term_i + beta * diff_step[0]) * grad_scale:
 * the update of LSQQuantizerCell_Frame::back_propagate (ref: ...LSQQuantizerCell_Frame.cpp:234-303)
 * and LSQQuantizerActivation_Frame::back_propagate (ref: ...LSQQuantizerActivation_Frame.cpp:193-271);
 * beta = 0 on a new solver iteration, 1 otherwise; grad_scale = 1/sqrt(N*hi). */
int n2d2hip_lsq_backward(const float* diff_q, const float* fp_x, float* diff_fp, size_t n, const float* step,
                         int lo, int hi, float grad_scale, float beta, float* diff_step,
                         void* workspace, size_t workspace_bytes, n2d2hip_stream_t stream);

/* ------------------------------------------- float cells of a training step */
/* The float32 cells a quantization-aware training graph runs between the fake-quant kernels above.  Tensors are
 * N2D2's own: activations NCHW ({X,Y,Z,B}, X fastest), weights OCHW ({kW,kH,C/groups,O}); `desc->weight_bits` is not
 * read; groups is 1 or C == O (depthwise).  "diff" tensors carry the descent direction, as in the reference
 * (target - output at the loss), so the solver adds rate * diff.  Ungrouped convolutions without dilation of at
 * least 2e7 flops run as an implicit GEMM on the fp32 matrix cores, the others on direct kernels that add their terms
 * in the reference's order.
 *
 * y = conv(x, w) (+ bias[o] if bias != NULL) + beta * y; the window is clipped at the borders (ref: src/Cell/ConvCell_Frame_Kernels.cpp:26-174, called from
 * ConvCell_Frame<T>::propagate, src/Cell/ConvCell_Frame.cpp:418-473). */
int n2d2hip_conv2d_f32_forward(const n2d2hip_conv_desc* desc, int B, int H, int W, const float* x, const float* w,
                               const float* bias, float beta, float* y, void* workspace, size_t workspace_bytes,
                               n2d2hip_stream_t stream);
/* diff_x = backwardData(w, diff_y) + beta * diff_x (ref: src/Cell/ConvCell_Frame_Kernels.cpp:176-333).  Dilation
 * must be 1: the reference's backward kernels do not read it. */
int n2d2hip_conv2d_f32_backward_data(const n2d2hip_conv_desc* desc, int B, int H, int W, const float* w,
                                     const float* diff_y, float beta, float* diff_x, void* workspace,
                                     size_t workspace_bytes, n2d2hip_stream_t stream);
/* diff_w = backwardFilter(x, diff_y) + beta * diff_w (ref: src/Cell/ConvCell_Frame_Kernels.cpp:335-427).
 *
 * `workspace` (device memory) of the three passes: n2d2hip_conv2d_f32_workspace_bytes bytes (may be 0) serve all of
 * them.  Backward-filter splits its sum over batch and pixels into ranges whose partial results go through the
 * workspace and are added in a fixed order; it fails with N2D2HIP_ERR_WORKSPACE when the workspace is too small.
 * Forward and backward-data do the same to fill the chip when their output is small, and run as one range when the
 * workspace is NULL or too small. */
size_t n2d2hip_conv2d_f32_workspace_bytes(const n2d2hip_conv_desc* desc, int B, int H, int W);
int n2d2hip_conv2d_f32_backward_filter(const n2d2hip_conv_desc* desc, int B, int H, int W, const float* x,
                                       const float* diff_y, float beta, float* diff_w, void* workspace,
                                       size_t workspace_bytes, n2d2hip_stream_t stream);
/* diff_bias[o] = sum over batch and pixels of diff_y + beta * diff_bias (ref: ...ConvCell_Frame_Kernels.cpp:429-452). */
int n2d2hip_conv2d_f32_backward_bias(int B, int O, int oH, int oW, const float* diff_y, float beta, float* diff_bias,
                                     n2d2hip_stream_t stream);
/* Rectifier of an unquantized cell, in place: x > 0 ? (clipping > 0 ? min(x, clipping) : x) : leak_slope * x, and its
 * backward diff_out = diff_in * (output == clipping ? 0 : output > 0 ? 1 : leak_slope), where `output` is what the cell
 * holds after its activation and the activation's quantizer (ref: include/Activation/RectifierActivation_Frame.hpp:55-139;
 * diff_in and diff_out may be the same buffer). */
int n2d2hip_rectifier_f32_forward(float* x, size_t n, float leak_slope, float clipping, n2d2hip_stream_t stream);
int n2d2hip_rectifier_f32_backward(const float* output, const float* diff_in, float* diff_out, size_t n, float leak_slope,
                                   float clipping, n2d2hip_stream_t stream);
/* Batch normalisation of float NCHW, one input: y = scale[c] * (x - m[c]) / sqrt(v[c] + epsilon) + bias[c].
 * use_running != 0 (inference) or moving_average_momentum == 0: m, v are the running `mean`, `variance`, which are not
 * changed.  Otherwise m, v are the batch's mean and biased variance over batch and pixels, written to saved_mean /
 * saved_variance, and the running ones move towards them: mean = m * momentum + mean * (1 - momentum), variance likewise
 * with v * n / (n - 1) (ref: BatchNormCell_Frame<T>::propagate, src/Cell/BatchNormCell_Frame.cpp:287-393).  x and y may
 * be the same buffer.  With a workspace of n2d2hip_batchnorm_f32_workspace_bytes() the sums of the learning pass and of
 * the backward are spread over several blocks per channel (partial sums added in a fixed order); without one (NULL) one
 * block per channel adds them.  Forward and backward may share the workspace. */
size_t n2d2hip_batchnorm_f32_workspace_bytes(int B, int C, int H, int W);
int n2d2hip_batchnorm_f32_forward(int B, int C, int H, int W, const float* x, const float* scale, const float* bias,
                                  float* mean, float* variance, float* saved_mean, float* saved_variance, double epsilon,
                                  double moving_average_momentum, int use_running, float* y, void* workspace,
                                  size_t workspace_bytes, n2d2hip_stream_t stream);
/* Its backward, from the x and the saved statistics of the learning pass: diff_scale[c] = sum(diff_y * x_hat) +
 * beta_scale * diff_scale[c], diff_bias[c] = sum(diff_y) + beta_bias * diff_bias[c], the gradients of the saved mean and
 * variance ({C} each, always written), and, when diff_x != NULL, diff_x = diff_y * scale / sigma + dVar * 2 (x - m) / n
 * + dMean / n (ref: BatchNormCell_Frame<T>::backPropagate, src/Cell/BatchNormCell_Frame.cpp:396-506).  diff_y and diff_x
 * may be the same buffer. */
int n2d2hip_batchnorm_f32_backward(int B, int C, int H, int W, const float* x, const float* scale, const float* saved_mean,
                                   const float* saved_variance, double epsilon, const float* diff_y, float beta_scale,
                                   float* diff_scale, float beta_bias, float* diff_bias, float* diff_saved_mean,
                                   float* diff_saved_variance, float* diff_x, void* workspace, size_t workspace_bytes,
                                   n2d2hip_stream_t stream);
/* Max pooling of float NCHW, one output per channel; output size as PoolCell computes it, (in + 2 pad - pool + stride) /
 * stride.  argmax {B,C,oH,oW} receives row * W + column of the first largest element of each window in row-major order,
 * -1 for a window that lies in the padding (output 0) (ref: PoolCell_Frame_Kernels::forwardMax with its ArgMax tensor,
 * src/Cell/PoolCell_Frame_Kernels.cpp:102-197). */
int n2d2hip_pool_max_f32_forward(int B, int C, int H, int W, int pool_w, int pool_h, int stride_x, int stride_y, int pad_x,
                                 int pad_y, const float* x, float* y, int* argmax, n2d2hip_stream_t stream);
/* diff_x[i] = sum of diff_y over the outputs whose maximum input i was + beta * diff_x[i]
 * (ref: PoolCell_Frame_Kernels::backwardMax, src/Cell/PoolCell_Frame_Kernels.cpp:295-379). */
int n2d2hip_pool_max_f32_backward(int B, int C, int H, int W, int pool_w, int pool_h, int stride_x, int stride_y, int pad_x,
                                  int pad_y, const float* diff_y, const int* argmax, float beta, float* diff_x,
                                  n2d2hip_stream_t stream);
/* Average pooling of float NCHW, one output per channel: the window's values inside the input, added in row-major
 * order, divided by pool_w * pool_h (count_include_padding != 0) or by their number (ref:
 * PoolCell_Frame_Kernels::forwardAverage with alpha 1, beta 0, not quantized, src/Cell/PoolCell_Frame_Kernels.cpp:26-100). */
int n2d2hip_pool_average_f32_forward(int B, int C, int H, int W, int pool_w, int pool_h, int stride_x, int stride_y,
                                     int pad_x, int pad_y, int count_include_padding, const float* x, float* y,
                                     n2d2hip_stream_t stream);
/* diff_x[i] = (sum of diff_y over the windows that hold input i) / (pool_w * pool_h) + beta * diff_x[i];
 * N2D2HIP_ERR_UNSUPPORTED without count_include_padding, where the reference throws (ref:
 * PoolCell_Frame_Kernels::backwardAverage, src/Cell/PoolCell_Frame_Kernels.cpp:199-293). */
int n2d2hip_pool_average_f32_backward(int B, int C, int H, int W, int pool_w, int pool_h, int stride_x, int stride_y,
                                      int pad_x, int pad_y, int count_include_padding, const float* diff_y, float beta,
                                      float* diff_x, n2d2hip_stream_t stream);
/* y = (weights[0] * x0 + shifts[0]) + (weights[1] * x1 + shifts[1]) + ... over n values, every product and sum rounded
 * to float in that order; `inputs`, `weights` and `shifts` are host arrays of nb_inputs entries (device pointers in
 * `inputs`), which is the PerLayer / PerInput coefficient mode (ref: ElemWiseCell_Frame::propagate, Sum,
 * src/Cell/ElemWiseCell_Frame.cpp:115-134). */
#define N2D2HIP_ELEMWISE_F32_MAX_INPUTS 8
int n2d2hip_elemwise_sum_f32_forward(int nb_inputs, const float* const* inputs, size_t n, const float* weights,
                                     const float* shifts, float* y, n2d2hip_stream_t stream);
/* The gradient towards one input of that sum: diff_x = weight * diff_y + beta * diff_x (ref:
 * ElemWiseCell_Frame::backPropagate, Sum, src/Cell/ElemWiseCell_Frame.cpp:194-233). */
int n2d2hip_elemwise_sum_f32_backward(size_t n, float weight, const float* diff_y, float beta, float* diff_x,
                                      n2d2hip_stream_t stream);
/* Softmax over the channels of each pixel, one group (ref: src/Cell/SoftmaxCell_Frame.cpp:93-137). */
int n2d2hip_softmax_f32_forward(const float* x, float* y, int B, int C, int H, int W, n2d2hip_stream_t stream);
/* diff = target - output, formed in double; loss[0] (device double) = sum of squares / batch
 * (ref: Cell_Frame_Top::applyLoss, src/Cell/Cell_Frame_Top.cpp:27-40); target and diff may be the same buffer, as they
 * are in the reference. */
size_t n2d2hip_loss_workspace_bytes(size_t n);
int n2d2hip_loss_f32(const float* target, const float* output, float* diff, size_t n, int batch, double* loss,
                     void* workspace, size_t workspace_bytes, n2d2hip_stream_t stream);
/* One SGDSolver_Frame<float>::update on a device tensor (ref: include/Solver/SGDSolver_Frame.hpp:77-146):
 * momentum_data == NULL: data += rate_diff * diff; otherwise m = m * momentum + rate_diff * diff
 * - decay_times_rate * data, data += m.  rate_diff = rate / (batchSize * IterationSize), computed by the caller from
 * SGDSolver::getLearningRate.  clamp != 0 clamps the result to [clamp_min, clamp_max]. */
int n2d2hip_sgd_update_f32(float* data, const float* diff, size_t n, float rate_diff, float momentum,
                           float decay_times_rate, float* momentum_data, int clamp, float clamp_min, float clamp_max,
                           n2d2hip_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* N2D2HIP_H */
