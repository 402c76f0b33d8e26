/*
 * neus2_amd.h - C ABI of the MI355X (gfx950) implementation of NeuS2's SDF-field hot path.
 *
 * The reference reaches this path through C++ virtual classes of its tcnn
 * submodule (tcnn::Encoding<T>, tcnn::Network<float,T>); the entry points
 * below are the flat C equivalents a binding for that interface would call.
 * Each declaration cites the reference call site it replaces
 * (paths relative to the reference checkout).
 *
 * Conventions
 *  - Every pointer named d_* is DEVICE memory owned by the caller.  The library
 *    allocates no device memory in any of these calls.
 *  - "SoA rows x N": element (r, i) at r*N + i  (tcnn RM / SoA layout,
 *    nerf_network.h:121-122).  fp16 buffers are IEEE binary16 (uint16_t here).
 *  - stream is a hipStream_t passed as void* (NULL = the default stream).
 *    Calls only enqueue work; they never synchronise.
 *  - Every function returning int returns N2_OK (0) or an n2_status error;
 *    n2_last_error() gives the message for the calling thread.
 *  - Not re-entrant per object: one host thread, one stream per object, like
 *    the reference (src/testbed.cu:2620-2621).
 */
#ifndef NEUS2_AMD_H
#define NEUS2_AMD_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum n2_status {
	N2_OK = 0,
	N2_ERR_INVALID_ARGUMENT = 1, /* shape / alignment / null-pointer checks failed; nothing was launched */
	N2_ERR_HIP = 2,              /* a HIP runtime call failed */
	N2_ERR_UNSUPPORTED = 3       /* configuration outside what the kernels implement */
} n2_status;

/* tcnn::EGradientMode as used at nerf_network.h:229,340,402,429,543,570 */
typedef enum n2_grad_mode {
	N2_GRAD_IGNORE = 0,    /* do not touch parameter gradients */
	N2_GRAD_OVERWRITE = 1, /* zero the gradient buffer, then accumulate this call */
	N2_GRAD_ACCUMULATE = 2 /* add to what the gradient buffer holds */
} n2_grad_mode;

typedef void* n2_stream_t;
typedef uint16_t n2_half;

const char* n2_last_error(void);
/* Library version string, e.g. "neus2_amd 0.1 gfx950". */
const char* n2_version(void);

/* ------------------------------------------------------------------------
 * Multi-resolution hash grid encoding: tcnn::GridEncoding<__half, 3, 2>
 * created by tcnn::create_encoding at nerf_network.h:46 from
 * configs/nerf/base.json:29-39.
 * ---------------------------------------------------------------------- */
typedef struct n2_grid n2_grid_t;

/* create_encoding<T>(3, {otype HashGrid, n_levels, n_features_per_level = 2,
 * log2_hashmap_size, base_resolution, per_level_scale}); nerf_network.h:46.
 * The per-level table (scale, resolution, entries, offset) is computed once
 * on the host in fp32 and handed to every kernel. */
int n2_grid_create(uint32_t n_levels, uint32_t n_features_per_level, uint32_t log2_hashmap_size,
                   uint32_t base_resolution, float per_level_scale, n2_grid_t** out);
void n2_grid_destroy(n2_grid_t* grid);

/* Encoding::n_params / output_width (takikawa_encoding.cuh:424-447 shows the in-tree form). */
uint32_t n2_grid_n_params(const n2_grid_t* grid);
uint32_t n2_grid_output_width(const n2_grid_t* grid);
uint32_t n2_grid_n_levels(const n2_grid_t* grid);

/* Host copy of the level table; arrays of n_levels (offset: n_levels + 1) entries.
 * Counterpart of GridEncoding::level_params_offset / level_n_params used at
 * src/testbed.cu:3070-3091. */
int n2_grid_level_table(const n2_grid_t* grid, float* scale, uint32_t* resolution, uint32_t* entries,
                        uint32_t* offset);

/* Tuning knob without a counterpart in the reference: the relative cost of one tile of points on each level
 * (n_levels values > 0).  The gather kernels split the levels over the GPU's 8 XCDs in proportion to it so
 * that each XCD's L2 holds only the tables of its own levels.  Defaults: 1 for hashed levels, 0.6 for dense ones.
 * Results do not depend on it. */
int n2_grid_set_level_costs(n2_grid_t* grid, const float* costs);

/* Hint for n2_grid_forward calls without dy_dx: non-zero says that the points of the following calls come in lattice
 * order (neighbouring points in neighbouring cells, as in Testbed::get_density_on_grid, src/testbed_nerf.cu:4082-4133).
 * Such calls are served by a kernel with one lane per point, which is faster when the gathers hit cached lines; values
 * agree with the default kernel's up to fp32 summation order.  Off by default. */
int n2_grid_set_point_order(n2_grid_t* grid, int lattice_order);

/* Level mask of the grid encoding.
 *  - n2_grid_set_max_level: GridEncoding::set_max_level as driven by Testbed::set_max_level (src/testbed.cu:1861-1866,
 *    2618): max_level is the fraction of the levels in use, 1 = all.  Level l is switched off when
 *    l >= (max_level * n_levels * n_features) / n_features + 1e-3 (fp32, tcnn's arithmetic): its output features and
 *    dy_dx are zero, it receives no parameter gradient and its dL_ddLdy rows are zero.
 *  - n2_grid_set_max_level_gpu: set_max_level_gpu (src/testbed_nerf.cu:3837, 3843, 3985): one fraction per point
 *    (device pointer, n_points floats, read by every later call until reset with NULL) replaces the global one;
 *    the reference fills it with random_val * 2 per ray when max_level_rand_training is on (:1305, 1440-1444).
 *  - n2_grid_set_progressive + n2_grid_set_training_step: the encoding keys valid_level_scale, base_valid_level_scale,
 *    base_training_step (configs/nerf/base.json:36-38) and Encoding::set_training_step (src/testbed.cu:2643-2646).
 *    The arithmetic lives in the tcnn fork, which the reference tree does not hold: PARITY UNPINNED.  Implemented as
 *    levels_in_use = clamp(floor(n_levels * (base_valid_level_scale + valid_level_scale * (step / base_training_step))
 *    + 1e-3), 1, n_levels), with an integer division; base_training_step 0 (the default) switches the mask off.
 *  - n2_grid_active_levels: levels in use under the global settings (per-point fractions not counted). */
int n2_grid_set_max_level(n2_grid_t* grid, float max_level);
int n2_grid_set_max_level_gpu(n2_grid_t* grid, const float* d_max_level);
int n2_grid_set_progressive(n2_grid_t* grid, float base_valid_level_scale, float valid_level_scale, uint32_t base_training_step);
int n2_grid_set_training_step(n2_grid_t* grid, uint32_t training_step);
uint32_t n2_grid_active_levels(const n2_grid_t* grid);

/* Encoding::set_params(params, inference_params, backward_params, gradients),
 * nerf_network.h:746-753.  One fp16 parameter buffer (n_params) and one fp16
 * gradient buffer (n_params, may be NULL until a backward needs it). */
int n2_grid_set_params(n2_grid_t* grid, const n2_half* d_params, n2_half* d_gradients);

/* Optional scratch for the parameter-gradient scatter (the reference takes temporaries from tcnn's arena).
 * With it, batches of up to max_points points scatter through an LDS counting sort (no global atomics, exact integer
 * accumulation, partial sums of split buckets added in a fixed order): the gradients do not depend on the order in which the
 * GPU runs the work, two calls on the same inputs give the same bits.  Without it, or for tables with more than 2^19
 * entries per level, packed fp16 global atomics are used (as in the reference; sums then depend on arrival order in the
 * last bit).  Results agree within the stated tolerance either way.
 * n2_grid_workspace_bytes returns 0 when the table shape does not support the sorted path. */
uint64_t n2_grid_workspace_bytes(const n2_grid_t* grid, uint32_t max_points);
int n2_grid_set_workspace(n2_grid_t* grid, void* d_workspace, uint64_t n_bytes, uint32_t max_points);

/* Encoding::forward(stream, input, &output, use_inference_params, prepare_input_gradients),
 * nerf_network.h:184-190 and inference at :671-676.
 *  d_xyz      positions in [0,1]^3; coordinate d of point i at d_xyz[i*point_stride + d*dim_stride]
 *             (the 7 x N column-major NerfCoordinate batch is point_stride = 7, dim_stride = 1;
 *              a 3 x N SoA matrix is point_stride = 1, dim_stride = N)
 *  d_out      fp16, SoA output_width x N
 *  d_dy_dx    NULL, or fp32 [output_width][N][3]: the saved forward context the
 *             input-gradient passes read (prepare_input_gradients = true) */
int n2_grid_forward(n2_grid_t* grid, n2_stream_t stream, const float* d_xyz, uint32_t point_stride,
                    uint32_t dim_stride, uint32_t n_points, n2_half* d_out, float* d_dy_dx);

/* Encoding::backward(stream, ctx, input, output, dL_doutput, &dL_dinput, use_inference_params, mode),
 * nerf_network.h:234 (normals, Ignore) and :419-429 (training, Overwrite).
 *  d_dL_dy    fp16 SoA output_width x N
 *  d_dy_dx    context saved by the forward (needed only when d_dL_dx != NULL)
 *  d_dL_dx    NULL or fp32 SoA 3 x N
 *  mode       what to do with the parameter gradients set by n2_grid_set_params */
int n2_grid_backward(n2_grid_t* grid, n2_stream_t stream, const float* d_xyz, uint32_t point_stride,
                     uint32_t dim_stride, uint32_t n_points, const n2_half* d_dL_dy, const float* d_dy_dx,
                     float* d_dL_dx, n2_grad_mode mode);

/* Encoding::backward_backward_input(stream, ctx, input, dL_ddLdinput, dL_doutput,
 * &dL_ddLdoutput, &dL_dinput, use_inference_params, mode), nerf_network.h:534-544.
 *  d_dL_ddLdx       fp32 SoA 3 x N: gradient w.r.t. the first backward's dL_dx
 *  d_dL_dy          fp16 SoA output_width x N: the dL_doutput the first backward was run with
 *  d_dL_ddLdy       NULL or fp16 SoA output_width x N
 *  d_dL_dx          NULL or fp32 SoA 3 x N (cross second derivatives; the reference
 *                   computes and then drops it, nerf_network.h:529-541) */
int n2_grid_backward_backward_input(n2_grid_t* grid, n2_stream_t stream, const float* d_xyz,
                                    uint32_t point_stride, uint32_t dim_stride, uint32_t n_points,
                                    const float* d_dL_ddLdx, const n2_half* d_dL_dy, n2_half* d_dL_ddLdy,
                                    float* d_dL_dx, n2_grad_mode mode);

/* First- and second-order parameter gradients in ONE scatter pass: the fusion of the two calls above as
 * NerfNetwork::backward_impl issues them back to back (nerf_network.h:419-429 then :534-544).  Each table
 * entry receives dL_dy*weight + dL_dy_second*(second-order coefficient) as a single packed fp16 atomic,
 * which halves the atomic traffic of the backward pass.  No dL_dx outputs.
 *  d_dL_dy          fp16 SoA output_width x N: first-order output gradient
 *  d_dL_ddLdx       fp32 SoA 3 x N;  d_dL_dy_second fp16 SoA output_width x N (see backward_backward_input)
 *  d_dL_ddLdy       NULL or fp16 SoA output_width x N
 *  mode             OVERWRITE or ACCUMULATE */
int n2_grid_backward_fused(n2_grid_t* grid, n2_stream_t stream, const float* d_xyz, uint32_t point_stride,
                           uint32_t dim_stride, uint32_t n_points, const n2_half* d_dL_dy, const float* d_dL_ddLdx,
                           const n2_half* d_dL_dy_second, n2_half* d_dL_ddLdy, n2_grad_mode mode);

/* Test hook for the bit-exact contract: entry index (without the level offset)
 * of the 8 trilinear corners, uint32 [n_levels][8][N], corner c uses +1 on
 * dimension d iff bit d of c is set (takikawa_encoding.cuh:82-92). */
int n2_grid_corner_indices(n2_grid_t* grid, n2_stream_t stream, const float* d_xyz, uint32_t point_stride,
                           uint32_t dim_stride, uint32_t n_points, uint32_t* d_indices);

/* ------------------------------------------------------------------------
 * Fully fused 64-wide MLP: tcnn::FullyFusedMLP<__half, 64>, ReLU hidden
 * activations, linear output, no bias; created by tcnn::create_network at
 * nerf_network.h:57 (SDF net, configs/nerf/base.json:40-47) and :65 (colour
 * net, base.json:63-69).
 * Weights: fp16, layers concatenated, each row-major [out][in]:
 *   W_0 [64][in_width], W_1 .. W_{H-1} [64][64], W_H [16][64]
 * (the order utils/mlp_weights.txt is stored in, nerf_network.h:774-803).
 * Batch sizes must be multiples of 8 (the reference demands multiples of
 * 128, src/testbed_nerf.cu:3429,3768).
 * ---------------------------------------------------------------------- */
typedef struct n2_mlp n2_mlp_t;

/* Matrix layout of the 16-row network output / its gradient.  Inputs and
 * input gradients are always SoA (the layout both encodings prefer). */
typedef enum n2_layout {
	N2_LAYOUT_SOA = 0, /* rows x N, element (r,i) at r*N + i                                   */
	N2_LAYOUT_AOS = 1  /* N x 16, element (r,i) at i*16 + r: the testbed's column-major 16 x N
	                      network output, src/testbed_nerf.cu:3771-3777                        */
} n2_layout;

/* create_network<T>({otype FullyFusedMLP, activation ReLU, output_activation None,
 * n_neurons 64, n_hidden_layers, n_input_dims, n_output_dims 16}); nerf_network.h:53-57,63-65.
 * in_width must be a multiple of 16 in [16, 64]; n_hidden_layers 1 or 2. */
int n2_mlp_create(uint32_t in_width, uint32_t n_hidden_layers, n2_mlp_t** out);
void n2_mlp_destroy(n2_mlp_t* mlp);
uint32_t n2_mlp_n_params(const n2_mlp_t* mlp);
uint32_t n2_mlp_input_width(const n2_mlp_t* mlp);
uint32_t n2_mlp_output_width(const n2_mlp_t* mlp); /* padded_output_width() = 16 */

/* Network::set_params(params, inference_params, backward_params, gradients), nerf_network.h:730-743. */
int n2_mlp_set_params(n2_mlp_t* mlp, const n2_half* d_params, n2_half* d_gradients);

/* Scratch for the batch reduction of weight gradients: fp32 partial sums, one
 * slab per workgroup.  Needed by n2_mlp_backward with mode != IGNORE and by
 * n2_mlp_backward_backward_input.  The reference takes this from tcnn's
 * stream-ordered arena (src/testbed_nerf.cu:3723-3749); here the caller owns it. */
uint64_t n2_mlp_workspace_bytes(const n2_mlp_t* mlp);
int n2_mlp_set_workspace(n2_mlp_t* mlp, void* d_workspace, uint64_t n_bytes);

/* Network::forward / inference_mixed_precision, nerf_network.h:212, 271, 686.
 *  d_input   fp16 SoA in_width x N
 *  d_output  fp16 16 x N in out_layout
 *  d_hidden  NULL, or fp16 SoA (64*n_hidden_layers) x N: post-activation values of
 *            every hidden layer (the forward context; Network::forward_activations).
 *            The backward passes recompute them from d_input and never need it. */
int n2_mlp_forward(n2_mlp_t* mlp, n2_stream_t stream, const n2_half* d_input, uint32_t n, n2_half* d_output,
                   n2_layout out_layout, n2_half* d_hidden);

/* Network::backward(stream, ctx, input, output, dL_doutput, &dL_dinput, use_inference_params, mode),
 * nerf_network.h:229 (normals, Ignore), :340, :402 (training), :509.
 *  d_dL_doutput  fp16 16 x N in dL_layout
 *  d_dL_dinput   NULL or fp16 SoA in_width x N */
int n2_mlp_backward(n2_mlp_t* mlp, n2_stream_t stream, const n2_half* d_input, uint32_t n,
                    const n2_half* d_dL_doutput, n2_layout dL_layout, n2_half* d_dL_dinput, n2_grad_mode mode);

/* n2_mlp_backward that uses only the first n_rows rows of dL_doutput and takes the others as zero.  The reference
 * extracts the three colour rows of dL_doutput into a zero-padded matrix before the colour net's backward
 * (nerf_network.h:338-340); this call reads them in place. */
int n2_mlp_backward_rows(n2_mlp_t* mlp, n2_stream_t stream, const n2_half* d_input, uint32_t n, const n2_half* d_dL_doutput,
                         n2_layout dL_layout, uint32_t n_rows, n2_half* d_dL_dinput, n2_grad_mode mode);

/* DifferentiableObject::input_gradient(stream, dim, input, d_dinput): gradient of output
 * row `dim` w.r.t. the input, i.e. backward with dL_doutput = e_dim and no parameter
 * gradients.  The reference builds e_0 by hand and calls backward with Ignore to get the
 * SDF normal (nerf_network.h:215-229, 497-512); this entry point reads no dL_doutput.
 *  d_dinput  fp16 SoA in_width x N */
int n2_mlp_input_gradient(n2_mlp_t* mlp, n2_stream_t stream, uint32_t dim, const n2_half* d_input, uint32_t n,
                          n2_half* d_dinput);

/* forward and input_gradient(dim) of the same batch in one pass over the input (the reference calls them back to back
 * on the SDF net, nerf_network.h:212 and :229); results equal those of the two separate calls. */
int n2_mlp_forward_and_input_gradient(n2_mlp_t* mlp, n2_stream_t stream, uint32_t dim, const n2_half* d_input, uint32_t n,
                                      n2_half* d_output, n2_layout out_layout, n2_half* d_dinput);

/* Weight gradients are summed per workgroup and a small second launch folds those partial sums into the gradient buffer.
 * With deferred reduction switched on, n2_mlp_backward / n2_mlp_backward_backward_input leave their partial sums pending
 * (the gradient buffer is NOT up to date until n2_mlp_reduce_deferred has run; after a pending pass only ACCUMULATE may
 * follow) and n2_mlp_reduce_deferred folds everything pending for up to two networks in one launch.  Off by default;
 * no counterpart in the reference, which uses GEMMs for the weight gradients. */
int n2_mlp_set_deferred_reduction(n2_mlp_t* mlp, int enable);

/* Numerical head-room of n2_mlp_backward / n2_mlp_backward_rows with weight gradients.  The fully fused network rounds the
 * gradients of its hidden layers to fp16 for the matrix cores (as tcnn's FullyFusedMLP does); with the reference's loss scale
 * (LOSS_SCALE = 128, testbed.h:237, divided by the ray count, src/testbed_nerf.cu:1756) the colour rows of dL/doutput lie in
 * fp16's SUBNORMAL range and that rounding costs 1-2 % per value.  With exponent k the kernel multiplies dL/doutput by 2^k as
 * it loads it (exact), runs the chain on the larger values and multiplies dL/dinput and the weight gradients by 2^-k in
 * fp32 before it stores them: the same results as k = 0 wherever k = 0 loses nothing, and no subnormal intermediate.
 * k in [-14, 14], default 0; the caller must keep |dL/doutput| * 2^k well inside fp16's range.  Ignored by the passes with
 * a second-order part.  No counterpart in the reference. */
int n2_mlp_set_output_gradient_exponent(n2_mlp_t* mlp, int exponent);
/* The exponent the trainer uses for the colour net: the largest k with loss_scale / n_rays * 2^k <= 16 (clamped to
 * [0, 14]).  The colour rows of the compositor's dL/doutput are bounded by 0.05 * loss_scale / n_rays (weight <= 1, Huber
 * slope / 5 <= 0.2, sigmoid' <= 0.25; src/testbed_nerf.cu:1700-1760), i.e. by 0.8 after the scaling. */
int n2_colour_gradient_exponent(float loss_scale, uint32_t n_rays);
int n2_mlp_reduce_deferred(n2_mlp_t* a, n2_mlp_t* b /* may be NULL */, n2_stream_t stream);

/* Network::backward_backward_input(stream, ctx, input, dL_ddLdinput, dL_doutput,
 * dL_ddLdoutput, dL_dinput, use_inference_params, mode): the second-order pass the
 * reference fork adds for the eikonal loss, nerf_network.h:560-571.  One hidden
 * layer only (the SDF net); dL_dinput is identically zero for ReLU and is not produced.
 *  d_dL_ddLdinput  fp16 SoA in_width x N
 *  d_dL_doutput    fp16 SoA 16 x N, or NULL for the constant e_0 (unit gradient on output
 *                  row 0), the only value the reference passes (nerf_network.h:499-504, 565)
 *  d_dL_ddLdoutput NULL or fp16 SoA 16 x N */
int n2_mlp_backward_backward_input(n2_mlp_t* mlp, n2_stream_t stream, const n2_half* d_input, uint32_t n,
                                   const n2_half* d_dL_ddLdinput, const n2_half* d_dL_doutput,
                                   n2_half* d_dL_ddLdoutput, n2_grad_mode mode);

/* Network::backward(..., mode) followed by Network::backward_backward_input(..., nullptr, nullptr, Accumulate) on the
 * same input, as NerfNetwork::backward_impl calls them on the SDF net (nerf_network.h:402 and :560-571), in one pass:
 * both sets of weight gradients have the same shape and are summed in the same accumulators.  The parameter
 * gradients equal those of the two calls up to fp32 summation order.  One hidden layer only.
 *  d_dL_doutput         fp16 16 x N in dL_layout (first-order output gradient)
 *  d_dL_dinput          fp16 SoA in_width x N (first-order input gradient, written)
 *  d_dL_ddLdinput       fp16 SoA in_width x N
 *  d_second_dL_doutput  the dL_doutput of the second-order call: fp16 SoA 16 x N, or NULL for the constant e_0
 *  mode                 OVERWRITE or ACCUMULATE */
int n2_mlp_backward_and_second_order(n2_mlp_t* mlp, n2_stream_t stream, const n2_half* d_input, uint32_t n,
                                     const n2_half* d_dL_doutput, n2_layout dL_layout, n2_half* d_dL_dinput,
                                     const n2_half* d_dL_ddLdinput, const n2_half* d_second_dL_doutput, n2_grad_mode mode);

/* ------------------------------------------------------------------------
 * The NeuS field: NerfNetwork<__half> (include/neural-graphics-primitives/nerf_network.h),
 * static scene (delta network off, src/testbed.cu:2695-2697).  Composes the hash grid, the
 * SDF MLP (3 centred coordinates + encoding, padded to a multiple of 16 -> 64 -> 16), the
 * degree-4 spherical-harmonics direction encoding, the colour MLP (16 SDF features + 16 SH +
 * xyz + normal, padded to 48 -> 64 -> 64 -> 16) and the learnable variance scalar.
 *
 * One parameter vector in the trainer's order (nerf_network.h:728-772):
 *   [SDF MLP | colour MLP | grid | variance (4 slots, slot 0 used)]
 * ---------------------------------------------------------------------- */
typedef struct n2_field n2_field_t;

typedef struct n2_field_config {
	uint32_t n_levels;             /* configs/nerf/base.json:31 */
	uint32_t n_features_per_level; /* 2 */
	uint32_t log2_hashmap_size;    /* 19 */
	uint32_t base_resolution;      /* 16 */
	float per_level_scale;         /* derived from top_resolution at src/testbed.cu:2165-2177 */
	uint32_t sdf_hidden_layers;    /* 1, base.json:45 */
	uint32_t rgb_hidden_layers;    /* 2, base.json:68 */
	float sdf_bias;                /* -0.1, base.json:46, nerf_network.h:74 */
} n2_field_config;

/* NerfNetwork<T>::NerfNetwork(...), nerf_network.h:40-83 */
int n2_field_create(const n2_field_config* config, n2_field_t** out);
void n2_field_destroy(n2_field_t* field);

/* The field's grid encoding (NerfNetwork::encoding(), used at src/testbed.cu:2643-2646 and src/testbed_nerf.cu:3837):
 * owned by the field; for the level-mask setters above. */
n2_grid_t* n2_field_encoding(n2_field_t* field);
uint32_t n2_field_n_params(const n2_field_t* field);
/* Offsets of the five segments [sdf mlp, colour mlp, grid, variance, end] in the parameter
 * vector; everything before offsets[2] is a matrix parameter for the optimiser
 * (NerfNetwork::layer_sizes, nerf_network.h:902-990). */
int n2_field_param_offsets(const n2_field_t* field, uint32_t offsets[5]);

/* Tuning switch without a counterpart in the reference.  On (the default): n2_field_forward, n2_field_sdf and
 * n2_field_density run as ONE kernel each (grid gather, both networks and the row bookkeeping fused) whenever the
 * configuration allows it: at most 16 levels with power-of-two hash tables, one hidden layer in the SDF net, two in the
 * colour net, no per-point level mask.  Off, or for other configurations: the same results from separate grid, network
 * and element-wise kernels (values agree within fp32 summation order). */
int n2_field_set_fused(n2_field_t* field, int enable);
/* n2_mlp_set_output_gradient_exponent for the field's colour net (rows 0..2 of n2_field_backward's dL/doutput); the
 * trainer sets n2_colour_gradient_exponent(loss_scale, n_rays) before every step.  Default 0. */
int n2_field_set_colour_gradient_exponent(n2_field_t* field, int exponent);

/* NerfNetwork::set_params, nerf_network.h:728-772 (fp16 params and gradients, n_params each). */
int n2_field_set_params(n2_field_t* field, const n2_half* d_params, n2_half* d_gradients);

/* Scratch the reference takes from tcnn's arena inside forward_impl/backward_impl
 * (every GPUMatrixDynamic temporary, nerf_network.h:137-267, 332-557): network inputs,
 * the grid's dy_dx context, input gradients and the MLP weight-gradient slabs.
 * max_batch bounds forward / sdf / density calls, max_batch_backward (<= max_batch) the batches
 * that are also run backward: the training step runs the forward over every marched sample
 * (up to 16 x 2^18) but the backward only over the compacted 2^18 (src/testbed_nerf.cu:3840, 3931-3932).
 * The workspace belongs to the field until another one is set: between calls it keeps the activations a backward or a
 * selection reads and the zero padding rows of the networks' inputs, which are cleared once per batch size and not
 * in every call; do not write to it. */
uint64_t n2_field_workspace_bytes(const n2_field_t* field, uint32_t max_batch, uint32_t max_batch_backward);
int n2_field_set_workspace(n2_field_t* field, void* d_workspace, uint64_t n_bytes, uint32_t max_batch,
                           uint32_t max_batch_backward);

/* NerfNetwork::forward_impl / inference_mixed_precision_impl (which the reference routes
 * to forward_impl), nerf_network.h:87-90, 132-315.
 *  d_coords  fp32, N rows of 7: x y z dt dx dy dz (NerfCoordinate, nerf.h:76-102), positions
 *            in [0,1]^3, directions warped to [0,1]^3
 *  d_output  fp16 N x 16 (N2_LAYOUT_AOS): [r g b raw | sdf + bias | normal xyz | variance |
 *            direction xyz | 5 unused colour-net rows]
 * The forward context stays in the workspace until the next forward. */
int n2_field_forward(n2_field_t* field, n2_stream_t stream, const float* d_coords, uint32_t n, n2_half* d_output);

/* Makes the samples d_source_index[0 .. n) of the last n2_field_forward (over n_source samples) the batch that the next
 * n2_field_backward differentiates: their saved activations are gathered instead of being computed again.  The
 * result is bit-identical to n2_field_forward on those samples' coordinates followed by n2_field_backward, because
 * every sample is evaluated independently of its batch.  n <= the workspace's backward capacity; indices may repeat.
 * No counterpart in the reference, which runs the network a second time on the compacted batch
 * (src/testbed_nerf.cu:3919-3936). */
int n2_field_select(n2_field_t* field, n2_stream_t stream, const uint32_t* d_source_index, uint32_t n_source, uint32_t n);

/* NerfNetwork::backward_impl, nerf_network.h:317-588, for the batch of the last forward.
 *  d_dL_doutput   fp16 N x 16 (AoS): rows 0..2 colour, 3 sdf, 4..6 eikonal (divided here by
 *                 ek_batch_size), 7 variance, 8..10 gradient w.r.t. the normal through cos
 *  ek_batch_size  NerfNetwork::indeed_batch_size (src/testbed_nerf.cu:3927)
 *  mode           OVERWRITE as the reference calls it; ACCUMULATE adds to existing gradients
 * Includes the second-order passes through grid and SDF MLP. */
int n2_field_backward(n2_field_t* field, n2_stream_t stream, const float* d_coords, uint32_t n,
                      const n2_half* d_dL_doutput, uint32_t ek_batch_size, n2_grad_mode mode);

/* NerfNetwork::sdf, nerf_network.h:643-709: encoding + SDF MLP, bias added on row 0.
 *  d_xyz     positions with the strides of n2_grid_forward
 *  d_output  fp16 SoA 16 x N */
int n2_field_sdf(n2_field_t* field, n2_stream_t stream, const float* d_xyz, uint32_t point_stride,
                 uint32_t dim_stride, uint32_t n, n2_half* d_output);

/* NerfNetwork::density, nerf_network.h:711-726: sdf, then row 0 becomes the logistic density
 * s*sigmoid(s*sdf)*(1 - sigmoid(s*sdf)) with s = exp(10*variance) (common_operation.cuh:310-328). */
int n2_field_density(n2_field_t* field, n2_stream_t stream, const float* d_xyz, uint32_t point_stride,
                     uint32_t dim_stride, uint32_t n, n2_half* d_output);

/* ------------------------------------------------------------------------
 * The SDF network trained on its own with the eikonal term (no colour branch): the element-wise steps that
 * NerfNetwork performs between the encoding's and the network's calls, for a caller that composes
 * n2_grid_* and n2_mlp_* itself (this repository's neus2_amd/sdf_net.py, BASELINE configuration 3):
 *   n2_sdf_pack_input     rows 0..2 of the network input = (T)x - (T)0.5 and zero padding rows behind the encoding
 *                         (fill_positions_view_with_fixed_offset, nerf_network.h:193-195, common_operation.cuh:186-199)
 *   n2_sdf_eikonal_loss   d_normal_encoding holds the encoding's backward of rows 3.. of d sdf / d input (n2_grid_backward
 *                         with d_dL_dx, nerf_network.h:230-234); the call writes d_normal = that + rows 0..2 of
 *                         d sdf / d input (add_positions_view, :236-238; the two may be the same buffer), forms  loss = mean |sdf| + ek_weight mean (|normal| - 1)^2  and writes what the backward
 *                         passes take: d_dL_doutput (fp16 SoA 16 x n: row 0 = sign(sdf) loss_scale / n), d_dL_dnormal
 *                         (fp32 SoA 3 x n, times loss_scale) and rows 0..2 and the padding rows of the network's
 *                         second-order input (fp16 SoA input_width x n, nerf_network.h:546-557; rows 3.. are the encoding's
 *                         dL_ddLdoutput: written by n2_grid_backward_fused when d_dy_dx is null; with d_dy_dx, the Jacobian
 *                         n2_grid_forward saved for the same points, this call writes them as dy_dx . d_dL_dnormal and
 *                         n2_grid_backward_fused can be called with d_dL_ddLdy = null, which spares its pass over the
 *                         table).  d_loss: one float.
 * ---------------------------------------------------------------------- */
int n2_sdf_pack_input(n2_stream_t stream, const float* d_xyz, uint32_t point_stride, uint32_t dim_stride, uint32_t n,
                      uint32_t encoding_width, uint32_t input_width, n2_half* d_input);
uint64_t n2_sdf_eikonal_workspace_bytes(uint32_t n);
int n2_sdf_eikonal_loss(n2_stream_t stream, uint32_t n, uint32_t encoding_width, uint32_t input_width, const n2_half* d_sdf_output,
                        const n2_half* d_dsdf_dinput, const float* d_normal_encoding, float* d_normal, float ek_weight, float loss_scale, n2_half* d_dL_doutput,
                        float* d_dL_dnormal, n2_half* d_second_order_input, float* d_loss, void* d_workspace, uint64_t workspace_bytes,
                        const float* d_dy_dx);

/* ------------------------------------------------------------------------
 * Adam on fp32 master weights with an fp16 working copy: tcnn's Adam as the
 * trainer runs it, Trainer::optimizer_step(stream, LOSS_SCALE) at
 * src/testbed_nerf.cu:3498, hyper-parameters from configs/nerf/base.json:13-26
 * (the Ema wrapper is n2_ema_step, the ExponentialDecay wrapper is host logic over n2_trainer_set_learning_rate).
 * Per parameter i:  g = grad/loss_scale;  i >= n_matrix_params and g == 0: skipped entirely;
 * i < n_matrix_params: g += l2_reg*w;  moments with beta1/beta2;  per-parameter step counter t;
 * w -= lr*sqrt(1-beta2^t)/(1-beta1^t) * m/(sqrt(v)+epsilon);  fp16 copy refreshed.
 * The bias-correction factors come from a per-device table per (beta1, beta2); the first call with a new pair on a
 * device builds it and waits for it on the host (the one exception to "calls never synchronise").
 * ---------------------------------------------------------------------- */
typedef struct n2_adam_config {
	float learning_rate; /* 1e-3 */
	float beta1;         /* 0.9 */
	float beta2;         /* 0.99 */
	float epsilon;       /* 1e-15 */
	float l2_reg;        /* 1e-6 */
} n2_adam_config;

/* tcnn's EmaOptimizer step after nested step `step` (1-based), over all parameters:
 *   tmp = (tmp*decay*(1 - decay^(step-1)) + w*(1 - decay)) / (1 - decay^step);  ema = half(tmp)
 *  d_weights fp16 working weights (read), d_tmp fp32 moving average (read/written), d_ema fp16 copy (written). */
int n2_ema_step(n2_stream_t stream, uint32_t n_params, float decay, uint32_t step, const n2_half* d_weights, float* d_tmp,
                n2_half* d_ema);

/* All buffers hold n_params elements and are caller-owned device memory:
 *  d_master fp32 weights, d_params fp16 copy (written), d_gradients fp16 (read),
 *  d_m1 / d_m2 fp32 moments, d_steps uint32 per-parameter step counters.
 * The first call on a device with a new pair of betas fills a table of bias corrections and waits for it (a stream
 * synchronisation, a device synchronisation when all four table slots are taken): make that call outside graph capture. */
int n2_adam_step(n2_stream_t stream, const n2_adam_config* config, uint32_t n_params, uint32_t n_matrix_params,
                 float loss_scale, float* d_master, n2_half* d_params, const n2_half* d_gradients, float* d_m1,
                 float* d_m2, uint32_t* d_steps);

/* ------------------------------------------------------------------------
 * NeuS logistic-density alpha compositing, Huber(0.1)/5 colour loss and the hand-derived
 * backward to the 16 network outputs, with compaction of the samples that survive early
 * termination: compute_loss_kernel_train_nerf_with_global_movement,
 * src/testbed_nerf.cu:1465-1996 (static scene: no global movement, envmap, exposure,
 * depth or mask supervision; Logistic colour activation; BENT_DIR 1).
 *
 * The reference runs one thread per ray with two serial loops; here one wavefront owns a ray
 * and transmittance / colour prefixes are wave-level scans over 64 samples at a time.
 * The reference hands out compacted ranges with atomicAdd (ray order is a race); here they are
 * an exclusive scan in ray order, i.e. deterministic.
 * ---------------------------------------------------------------------- */
typedef struct n2_composite_config {
	float loss_scale;       /* LOSS_SCALE = 128, testbed.h:237 */
	float ek_loss_weight;   /* hyperparams.ek_loss_weight, configs/nerf/base.json:80 */
	float cos_anneal_ratio; /* NerfNetwork::cos_anneal_ratio, nerf_network.h:1109-1118 (1 when anneal_end = 0) */
	float background[3];    /* m_background_color, added as T*background to rays that are not cut short */
	uint32_t n_rays_norm;   /* n_rays_per_batch: loss and gradients are divided by it (:1717, :1756) */
} n2_composite_config;

uint64_t n2_composite_workspace_bytes(uint32_t max_rays);

/*  n_rays                upper bound of rays; d_ray_counter (may be NULL) holds the live count (rays_counter)
 *  d_numsteps            uint32 [n_rays][2] in: (samples, first sample) per ray; out: (kept samples, compacted first)
 *  d_network_output      fp16 [S][16] (AoS) field output of every marched sample
 *  d_coords              fp32 [S][7] NerfCoordinate of every marched sample
 *  d_rgb_target          fp32 [n_rays][3] target colour of each ray's pixel (the dataset side of :1619-1662)
 *  max_samples_compacted target batch size (2^18)
 *  d_compacted_counter   uint32 out: total samples the rays wanted to keep (numsteps_counter; may exceed the maximum)
 *  d_coords_compacted    fp32 [max][7] out
 *  d_dloss_doutput       fp16 [max][16] out (rows 11..15, which the reference leaves unset, are zero)
 *  d_loss                NULL or fp32 [n_rays] out: per-ray mean loss / n_rays_norm */
int n2_composite_loss(n2_stream_t stream, const n2_composite_config* config, uint32_t n_rays,
                      const uint32_t* d_ray_counter, uint32_t* d_numsteps, const n2_half* d_network_output,
                      const float* d_coords, const float* d_rgb_target, uint32_t max_samples_compacted,
                      uint32_t* d_compacted_counter, float* d_coords_compacted, n2_half* d_dloss_doutput,
                      float* d_loss, void* d_workspace, uint64_t workspace_bytes);
/* n2_composite_loss that also writes, for every compacted sample, the index of the marched sample it is
 * (d_source_index: uint32 [max_samples_compacted], may be NULL).  No counterpart in the reference, whose step evaluates
 * the network a second time on the compacted coordinates; with the index the saved activations of the first evaluation
 * can be selected instead (n2_field_select). */
int n2_composite_loss_indexed(n2_stream_t stream, const n2_composite_config* config, uint32_t n_rays,
                              const uint32_t* d_ray_counter, uint32_t* d_numsteps, const n2_half* d_network_output,
                              const float* d_coords, const float* d_rgb_target, uint32_t max_samples_compacted,
                              uint32_t* d_compacted_counter, float* d_coords_compacted, n2_half* d_dloss_doutput,
                              float* d_loss, uint32_t* d_source_index, void* d_workspace, uint64_t workspace_bytes);

/* n2_composite_loss_indexed without a workspace argument, for callers that cannot allocate device memory (code under
 * HIP graph capture, tight serving loops, harnesses that forbid hipMalloc).  No counterpart in the reference.  The
 * per-ray scratch (composited colour, kept-sample count and the count's prefix sum of every ray, 24 bytes per ray) lives in an array inside
 * the library's device image, 1.5 MiB that each GPU the library runs on holds until the process ends; the call
 * allocates and frees nothing.  n_rays above N2_COMPOSITE_STATIC_MAX_RAYS is rejected with N2_ERR_INVALID_ARGUMENT.
 * All calls on one GPU share that GPU's array: calls that overlap in time on one GPU (different streams or host threads
 * without ordering between them) race; calls ordered on one stream are safe.  Nothing in the array has to start at
 * zero: the forward kernel writes every ray's slot below n_rays (and, from 8192 rays on, the scan kernel every prefix sum)
 * before the backward kernel reads it.  Results are
 * bit-identical to n2_composite_loss_indexed's.
 * The first call on a device takes a lock and looks the array's address up (hipGetSymbolAddress, which may load the
 * library's code object): make one call per device outside graph capture before capturing any. */
#define N2_COMPOSITE_STATIC_MAX_RAYS 65536u
int n2_composite_loss_static(n2_stream_t stream, const n2_composite_config* config, uint32_t n_rays,
                             const uint32_t* d_ray_counter, uint32_t* d_numsteps, const n2_half* d_network_output,
                             const float* d_coords, const float* d_rgb_target, uint32_t max_samples_compacted,
                             uint32_t* d_compacted_counter, float* d_coords_compacted, n2_half* d_dloss_doutput,
                             float* d_loss, uint32_t* d_source_index);

/* tcnn fill_rollover / fill_rollover_and_rescale, src/testbed_nerf.cu:3908-3916: pad a compacted
 * batch of *d_n_in rows to n_total rows by wrapping around; the fp16 variant scales the wrapped
 * copies by n_in/n_total.  No-op when *d_n_in is 0 or >= n_total. */
int n2_fill_rollover_f32(n2_stream_t stream, uint32_t n_total, uint32_t stride, const uint32_t* d_n_in, float* d_inout);
int n2_fill_rollover_and_rescale_f16(n2_stream_t stream, uint32_t n_total, uint32_t stride, const uint32_t* d_n_in,
                                     n2_half* d_inout);

/* ------------------------------------------------------------------------
 * Training-sample generator: one pixel per ray, ray/unit-cube intersection, march through the
 * 128^3 morton-ordered occupancy bitfield with the fixed step sqrt(3)/1024, one NerfCoordinate per
 * occupied step: generate_training_samples_nerf_with_global_movement,
 * src/testbed_nerf.cu:1253-1446 (static path, cone_angle_constant = 0, unit aabb).
 * Random draws come from a counter-based hash (tcnn's pcg32 is not part of the reference
 * checkout); sample ranges and ray slots are handed out in ray order, not by atomicAdd.
 * ---------------------------------------------------------------------- */
typedef struct n2_camera {
	float xform[12];          /* row-major 3x4 camera-to-world [R | origin] (TrainingXForm::start) */
	float focal_length[2];    /* pixels (TrainingImageMetadata::focal_length) */
	float principal_point[2]; /* fraction of the image (0.5 = centre) */
	uint32_t resolution[2];
	uint32_t pixel_offset_lo; /* index of the image's first pixel in the RGBA array, low / high word */
	uint32_t pixel_offset_hi;
} n2_camera;

uint64_t n2_sampler_workspace_bytes(uint32_t max_rays);

/*  n_rays            rays to try (n_rays_per_batch);  n_rays_total: rays drawn in earlier steps (image rotation)
 *  d_cameras         n_images cameras;  d_rgba fp32 [pixels][4] premultiplied-alpha training images
 *  background        colour behind transparent pixels (host array of 3)
 *  d_bitfield        occupancy bits of mip 0: 128^3/8 bytes, bit (idx%8) of byte idx/8, idx = morton3D(x,y,z)
 *                    (grid_to_bitfield, src/testbed_nerf.cu:738-759)
 *  max_samples       capacity of d_coords; rays from the first one that does not fit are dropped
 *  d_ray_counter     out: live rays;  d_sample_counter out: samples all rays with >= 1 step asked for
 *  d_ray_indices     out uint32 [n_rays]: original ray id per live slot
 *  d_numsteps        out uint32 [n_rays][2]: (samples, first sample) per live slot
 *  d_rgb_target      out fp32 [n_rays][3]: pixel colour composited over the background
 *  d_coords          out fp32 [max_samples][7] */
int n2_generate_training_samples(n2_stream_t stream, uint32_t n_rays, uint32_t n_rays_total, uint32_t seed,
                                 const n2_camera* d_cameras, uint32_t n_images, const float* d_rgba,
                                 const float background[3], const uint8_t* d_bitfield, uint32_t max_samples,
                                 uint32_t* d_ray_counter, uint32_t* d_sample_counter, uint32_t* d_ray_indices,
                                 uint32_t* d_numsteps, float* d_rgb_target, float* d_coords, void* d_workspace,
                                 uint64_t workspace_bytes);

/* Training images as the loader decodes them (8-bit sRGB RGBA, stb_image order) -> what the ray generator reads (fp32
 * RGBA, linear, premultiplied by alpha): convert_rgba32 (src/nerf_loader.cu:59-81) with its white/black-is-transparent
 * and mask-colour rules, then the Byte branch of read_rgba (common_device.cuh:635-655): srgb_to_linear(c/255)*alpha,
 * alpha = a/255; a pixel equal to 0x00FF00FF afterwards (the mask marker) becomes (-1, -1, -1, -1). */
int n2_convert_rgba8(n2_stream_t stream, uint64_t n_pixels, const uint8_t* d_rgba8, float* d_rgba, int white_transparent,
                     int black_transparent, uint32_t mask_color);

/* ------------------------------------------------------------------------
 * One training step: counterpart of Testbed::train_nerf_step followed by
 * Trainer::optimizer_step (src/testbed_nerf.cu:3717-3987, 3498):
 *   generate samples -> field forward over every marched sample -> compositing / loss /
 *   compaction -> roll the compacted batch over to exactly target_batch_size -> field forward
 *   and backward on it -> Adam.
 * Nothing in a step synchronises with the host; counters are read on request.
 * ---------------------------------------------------------------------- */
typedef struct n2_trainer n2_trainer_t;

typedef struct n2_trainer_config {
	n2_field_config field;
	n2_adam_config adam;
	n2_composite_config composite;  /* n_rays_norm is overwritten per step with the step's n_rays */
	uint32_t target_batch_size;     /* 2^18, src/testbed.cu:2110 */
	uint32_t max_rays_per_batch;    /* upper bound of n_rays in a step */
	uint32_t max_samples;           /* capacity for marched samples; the reference uses 16 x target (src/testbed_nerf.cu:3719) */
	float loss_scale;               /* 128, testbed.h:237 */
	uint32_t prefetch_samples;      /* non-zero: each step also starts the NEXT step's sample generation (same n_rays and
	                                   n_inference, seed + 1) on a stream the trainer owns, so that it overlaps this step's
	                                   field kernels; a following step called with other arguments regenerates in line.
	                                   Results are bit-identical either way (every sum of a step is formed in a fixed
	                                   order).  The trainer must then be driven from one stream
	                                   (or from streams the caller orders against each other). */
	float ema_decay;                /* 0: plain Adam.  In (0, 1): the Ema wrapper of configs/nerf/base.json:5-7 (0.95) keeps a
	                                   bias-corrected moving average of the fp16 weights as the inference parameters */
	uint32_t recompute_training_forward; /* non-zero: the field is evaluated a second time on the compacted batch, as the
	                                   reference does (src/testbed_nerf.cu:3919-3936).  0: the activations that the first
	                                   evaluation saved are selected for the compacted samples (n2_field_select); the
	                                   gradients are bit-identical either way */
} n2_trainer_config;

/* All device memory a trainer uses (parameters, optimiser state, every temporary) lives in one
 * caller-owned workspace, counterpart of the Trainer's parameter buffer plus the arena allocation
 * of src/testbed_nerf.cu:3723-3749. */
uint64_t n2_trainer_workspace_bytes(const n2_trainer_config* config);
int n2_trainer_create(const n2_trainer_config* config, void* d_workspace, uint64_t workspace_bytes, n2_trainer_t** out);
void n2_trainer_destroy(n2_trainer_t* trainer);

/* Parameter buffers inside the workspace ([fp32 master | fp16 params | fp16 gradients], the Trainer's
 * layout mirrored at nerf_network.h:1010-1016).  The caller initialises d_master (NerfNetwork::
 * initialize_params, nerf_network.h:805-876) and calls n2_trainer_sync_params to refresh the fp16 copy. */
int n2_trainer_buffers(n2_trainer_t* trainer, float** d_master, n2_half** d_params, n2_half** d_gradients, uint32_t* n_params);
int n2_trainer_sync_params(n2_trainer_t* trainer, n2_stream_t stream);
n2_field_t* n2_trainer_field(n2_trainer_t* trainer);

/* Training images, cameras and the occupancy bitfield (see n2_generate_training_samples). */
int n2_trainer_set_scene(n2_trainer_t* trainer, const n2_camera* d_cameras, uint32_t n_images, const float* d_rgba,
                         const uint8_t* d_bitfield);

/* The ExponentialDecay wrapper (configs/nerf/base.json:8-12) is host logic: after nested step t, if t >= decay_start and
 * (t - decay_start) % decay_interval == 0, the learning rate is multiplied by decay_base.  The caller applies it here. */
int n2_trainer_set_learning_rate(n2_trainer_t* trainer, float learning_rate);

/* Optimizer state inside the workspace (what Trainer::serialize(include_optimizer_state) stores, src/testbed.cu:3134-3137):
 * Adam moments and per-parameter step counters, the fp32 moving average of the Ema wrapper (NULL without it) and the
 * parameters to use for inference (the Ema copy when it exists, else the working copy).
 * The step counters are param_steps_bits wide: uint32_t, or uint16_t that stop at 65535 when the Adam betas are such that
 * 1 - beta^t is exactly 1 in fp32 from step 4096 on (the defaults are): the bias correction no longer depends on the
 * count then, and the narrow counters save 4 bytes of traffic per parameter and step.  n2_snapshot_save and
 * n2_snapshot_read take either width and keep the file's 32-bit form. */
typedef struct n2_trainer_optimizer_buffers {
	float* first_moments;
	float* second_moments;
	void* param_steps;
	float* ema_weights;
	n2_half* inference_params;
	uint32_t optimizer_steps;
	float learning_rate;
	uint32_t param_steps_bits;
} n2_trainer_optimizer_buffers;
int n2_trainer_optimizer_state(n2_trainer_t* trainer, n2_trainer_optimizer_buffers* out);
int n2_trainer_set_optimizer_steps(n2_trainer_t* trainer, uint32_t steps);
/* The Ema wrapper's own step count (its bias correction 1 - decay^steps).  With ema_steps = 0 the moving average starts
 * again from the current working parameters: the fp32 average and the fp16 inference copy are overwritten with them.
 * Call it with 0 after parameters were loaded without Ema state (a snapshot without optimizer state, or
 * n2_trainer_sync_params after writing the master weights), with the saved optimizer step count when the Ema weights
 * were loaded too.  Without the wrapper (ema_decay 0) it only records the count. */
int n2_trainer_restart_ema(n2_trainer_t* trainer, n2_stream_t stream, uint32_t ema_steps);
/* Testbed::m_training_step: the number of training steps taken so far.  It is the clock of the encoding's progressive
 * level mask (the reference sets it on the encoding at the top of Testbed::train, before the occupancy-grid update and the
 * step, src/testbed.cu:2641-2647): this call also tells the encoding, so that an occupancy update that follows sees the
 * mask of the step about to run.  n2_trainer_step uses it and adds one.  Set it after loading a snapshot (its
 * training_step), whether or not the file holds optimizer state. */
int n2_trainer_set_training_step(n2_trainer_t* trainer, uint32_t step);

/* Call before the bitfield passed to n2_trainer_set_scene is rewritten in place (an occupancy-grid update): waits for a
 * sample generation that is running ahead on the trainer's own stream and discards it, so that the next step marches
 * through the new bitfield like the reference does (training_prep_nerf runs before train_nerf_step,
 * src/testbed.cu:2658-2674).  No counterpart in the reference, which generates its samples inside the step. */
int n2_trainer_invalidate_prefetch(n2_trainer_t* trainer);

/* Forward pass in depth chunks.  The compositor consumes a ray's samples only while the transmittance in front of them is
 * >= 1e-4 (src/testbed_nerf.cu:1562-1566); on a trained field most rays reach that point long before their last marched
 * sample, and nothing behind it enters the loss, the compaction or a gradient.  With n_rounds >= 2 the step evaluates the
 * field in rounds: every round takes the next chunk_size samples of the rays that are still in front of their cut (the
 * last round: all that is left of them).  Parameters, gradients and counters are bit-identical to the plain step's, which
 * evaluates every marched sample as the reference does (src/testbed_nerf.cu:3771-3777); each round costs three short
 * launches, so the setting pays when a step marches well over one and a half times the samples it keeps.
 * n_rounds 0 or 1: off (the default).  n_rounds <= 8.  Needs the fused field kernels. */
int n2_trainer_set_depth_chunks(n2_trainer_t* trainer, uint32_t chunk_size, uint32_t n_rounds);
/* How many samples each round evaluated in a recent step (n2_trainer_step_view.evaluated_counts, read by the caller when it
 * reads the step's counters): the following steps size their launches by these figures instead of by the most a round can
 * hold.  Estimates only decide how the work is dealt to workgroups, never what is computed.  n2_trainer_set_depth_chunks
 * forgets them. */
int n2_trainer_set_depth_chunk_estimates(n2_trainer_t* trainer, const uint32_t* samples_per_round, uint32_t n_rounds);

/*  n_rays       rays to draw this step (<= max_rays_per_batch)
 *  n_inference  how many marched samples the first forward covers (a multiple of 8, <= max_samples); the
 *               reference uses the sample count measured in earlier steps, rounded up to 128
 *               (src/testbed_nerf.cu:3751-3756)
 *  seed         seed of this step's random draws
 * A step whose rays kept no sample leaves parameters and optimiser state alone (the reference stops training there,
 * src/testbed_nerf.cu:3536-3542), but the host-side counts (optimizer_steps, the training step, the Ema's step count)
 * advance with every call: they count calls, the device decides about the update. */
int n2_trainer_step(n2_trainer_t* trainer, n2_stream_t stream, uint32_t n_rays, uint32_t n_inference, uint32_t seed);

/* Device buffers of the last step, for inspection and tests (the reference keeps the same data in its arena allocation,
 * src/testbed_nerf.cu:3723-3749): valid until the next step overwrites them.  After this call the next n2_trainer_step
 * orders its sample generation (which overwrites the sample set) behind everything enqueued on the step's stream so far, so
 * work that reads the view may simply be enqueued on that stream before the next step. */
typedef struct n2_trainer_step_view {
	const float* coords;              /* [marched samples][7] of the step's sample set */
	const uint32_t* numsteps;         /* [rays][2] after compositing: (kept samples, first compacted sample) per live ray */
	const float* rgb_target;          /* [rays][3] */
	const uint32_t* ray_indices;      /* [rays] */
	const n2_half* network_output;    /* [n_inference][16] field output over the marched samples */
	const float* coords_compacted;    /* [target_batch_size][7] after the roll-over */
	const n2_half* dloss_doutput;     /* [target_batch_size][16] after the roll-over */
	const uint32_t* source_index;     /* [target_batch_size] marched sample behind every compacted sample; after a step in depth
	                                     chunks: its place in evaluated_samples */
	const uint32_t* evaluated_samples;/* NULL, or (a step in depth chunks) the marched samples the field was evaluated on, in the
	                                     order in which it stored them */
	const uint32_t* evaluated_counts; /* NULL, or [8]: how many of them each round evaluated (their sum is the list's length) */
} n2_trainer_step_view;
int n2_trainer_last_step_view(n2_trainer_t* trainer, n2_trainer_step_view* out);

/* Waits for the stream, then returns the last step's counters: live rays, marched samples, samples the
 * rays wanted to keep (before the clamp to target_batch_size), and the summed loss
 * (counters.update_after_training, src/testbed_nerf.cu:3406-3429). */
int n2_trainer_read_counters(n2_trainer_t* trainer, n2_stream_t stream, uint32_t* rays, uint32_t* samples,
                             uint32_t* compacted, float* loss);

/* ------------------------------------------------------------------------
 * Occupancy grid: the running density estimate on 128^3 cells per cascade, and the morton-ordered
 * 1-bit-per-cell bitfield with 8 mip levels (level m at byte m * 128^3 / 8) that the sample generator
 * marches through.  Testbed::update_density_grid_nerf and update_density_grid_mean_and_bitfield,
 * src/testbed_nerf.cu:3286-3391; kernels generate_grid_samples_nerf_nonuniform (:630-660),
 * splat_grid_samples_nerf_max_nearest_neighbor (:662-680), ema_grid_samples_nerf (:698-727),
 * grid_to_bitfield (:738-764), bitfield_max_pool (:766-786).  Unit aabb; threshold
 * min(NERF_MIN_OPTICAL_THICKNESS = 0.1, mean density of the first cascade).
 * Random numbers: PCG32 seeded as pcg32(seed) (the reference's density_grid_rng, src/testbed.cu:2090),
 * passed to each sample launch by value and advanced by 2^32 afterwards.
 * ---------------------------------------------------------------------- */
typedef struct n2_occupancy n2_occupancy_t;

typedef struct n2_occupancy_buffers {
	float* density_grid;      /* [n_cascades][128^3] running estimate */
	float* density_grid_tmp;  /* [n_cascades][128^3] maxima splatted by the last update */
	uint8_t* bitfield;        /* [8][128^3 / 8] */
	float* mean;              /* [1] mean of max(density, 0) over the first cascade */
	float* positions;         /* [n_samples][3] sample positions of the last update: first the n_uniform samples of the */
	uint32_t* indices;        /* [n_samples] their cells            uniform group, then the others.  Within a group of n */
	                          /* samples, slot t holds the reference's sample t (56924617^-1 mod 2^32) mod n when n is a   */
	                          /* power of two (consecutive slots then fall into consecutive cells), else sample t          */
	uint32_t n_samples, n_cascades, ema_step, n_uniform;
	uint64_t rng_state, rng_inc;
} n2_occupancy_buffers;

/*  n_cascades  max_cascade + 1 (1 for aabb_scale 1, src/testbed_nerf.cu:3077-3080) */
int n2_occupancy_create(uint32_t n_cascades, uint64_t seed, n2_occupancy_t** out);
void n2_occupancy_destroy(n2_occupancy_t* occupancy);
/*  max_samples  largest n_uniform + n_nonuniform of an update
 *  max_chunk    largest batch the field accepts (its workspace's max_batch); densities are evaluated in chunks */
uint64_t n2_occupancy_workspace_bytes(const n2_occupancy_t* occupancy, uint32_t max_samples, uint32_t max_chunk);
int n2_occupancy_set_workspace(n2_occupancy_t* occupancy, void* d_workspace, uint64_t n_bytes, uint32_t max_samples,
                               uint32_t max_chunk);
/* The training_step == 0 branch of update_density_grid_nerf (:3310-3329): zero grid, ema step 0. */
int n2_occupancy_reset(n2_occupancy_t* occupancy, n2_stream_t stream);
/* update_density_grid_nerf(decay, n_uniform, n_nonuniform, stream): sample cells, evaluate NerfNetwork::density,
 * max-splat, decayed maximum, mean, bitfield and mips.  training_prep_nerf (:3989-4002) calls it with
 * (128^3 * n_cascades, 0) for the first 256 steps and a quarter of that for each kind afterwards, decay 0.95. */
int n2_occupancy_update(n2_occupancy_t* occupancy, n2_field_t* field, n2_stream_t stream, float decay, uint32_t n_uniform,
                        uint32_t n_nonuniform);
/* update_density_grid_mean_and_bitfield alone (after the density grid was written from outside, e.g. a snapshot). */
int n2_occupancy_update_bitfield(n2_occupancy_t* occupancy, n2_stream_t stream);
int n2_occupancy_view(n2_occupancy_t* occupancy, n2_occupancy_buffers* out);
/* Restores the host-side state that n2_occupancy_view reports (resuming from a saved state). */
int n2_occupancy_set_state(n2_occupancy_t* occupancy, uint32_t ema_step, uint64_t rng_state, uint64_t rng_inc);

/* ------------------------------------------------------------------------
 * Mesh extraction: marching cubes with shared vertices over a density lattice, marching_cubes_gpu
 * (src/marching_cubes.cu:794-822; gen_vertices :276-329, gen_faces :377-718), the lattice itself
 * (Testbed::get_density_on_grid, src/testbed_nerf.cu:4082-4133) and the area-weighted vertex normals of
 * accumulate_1ring (src/marching_cubes.cu:331-366).
 * density[x + y*rx + z*rx*ry]; inside = density > thresh; vertex at dt = (thresh - f0)/(f1 - f0) along a cut edge,
 * times (aabb_max - aabb_min)/res plus aabb_min.  Vertices are numbered by lattice point (x fastest) and edge
 * direction, triangles by cube (the reference's order is an atomicAdd race).  The case table is derived on the host;
 * it has the contour of the reference's table on every cube face in all 256 cases (same surface and orientation),
 * with the polygons of some cases cut into triangles along other diagonals.
 * ---------------------------------------------------------------------- */
/* The derived case table: 256 rows of up to 5 edge triples, -1 terminated (the layout of the reference's
 * triangle_table, src/marching_cubes.cu:400-657). */
int n2_marching_cubes_table(int8_t* out_256x16);
uint64_t n2_marching_cubes_workspace_bytes(const uint32_t res[3]);
/* First pass: counts (the reference's "count only" launches, :807-811).  Synchronises with the stream. */
int n2_marching_cubes_count(n2_stream_t stream, const uint32_t res[3], const float aabb_min[3], const float aabb_max[3],
                            float thresh, const float* d_density, void* d_workspace, uint64_t workspace_bytes,
                            uint32_t* n_vertices, uint32_t* n_triangles);
/* Second pass with the workspace of the first (it holds the per-tile prefix sums; this pass adds the vertex slots of
 * the lattice points that own a vertex): d_vertices fp32 [n_vertices][3], d_indices uint32 [n_triangles][3],
 * d_normals fp32 [n_vertices][3] or NULL (not normalised, like the reference's). */
int n2_marching_cubes_emit(n2_stream_t stream, const uint32_t res[3], const float aabb_min[3], const float aabb_max[3],
                           float thresh, const float* d_density, void* d_workspace, float* d_vertices,
                           uint32_t* d_indices, float* d_normals, uint32_t n_vertices, uint32_t n_triangles);
/* get_density_on_grid: the field's SDF (row 0 of NerfNetwork::sdf, fp16 widened to fp32) at the lattice points
 * (x, y, z)/res * (aabb_max - aabb_min) + aabb_min, evaluated `chunk` points at a time (a multiple of 8, at most the
 * field's max_batch; the reference uses 2^20).  d_density fp32 [rx*ry*rz]. */
uint64_t n2_density_on_grid_scratch_bytes(uint32_t chunk);
int n2_density_on_grid(n2_field_t* field, n2_stream_t stream, const uint32_t res[3], const float aabb_min[3],
                       const float aabb_max[3], float* d_density, void* d_scratch, uint64_t scratch_bytes, uint32_t chunk);

/* ------------------------------------------------------------------------
 * Snapshot files: MessagePack of the network configuration plus a "snapshot" object, the format of
 * Testbed::save_snapshot / load_snapshot (src/testbed.cu:3134-3244): n_params, params_type, params_binary,
 * [optimizer], density_grid_size, density_grid_binary (fp16), nerf { aabb_scale, rgb { rays_per_batch,
 * measured_batch_size, measured_batch_size_before_compaction } }, training_step, loss.
 * Device pointers in, device pointers out; the file image lives in host memory in between.
 * ---------------------------------------------------------------------- */
typedef struct n2_snapshot n2_snapshot_t;

typedef struct n2_snapshot_desc {
	const uint8_t* config_msgpack;   /* host: an encoded MessagePack map (the network configuration, m_network_config); its entries
	                                    become the file's top-level entries.  May be NULL */
	uint64_t config_bytes;
	uint32_t n_params;
	const n2_half* d_params;         /* fp16 working parameters (written as params_type "__half") */
	uint32_t include_optimizer_state;
	const float* d_first_moments;    /* Adam state, n_params each (only with include_optimizer_state) */
	const float* d_second_moments;
	const void* d_param_steps;       /* uint32_t, or uint16_t when param_steps_bits (below) is 16 */
	const float* d_ema_weights;      /* fp32 moving average of the Ema wrapper, or NULL */
	uint32_t optimizer_steps;
	float learning_rate;
	const float* d_density_grid;     /* fp32, density_grid_cells = n_cascades * 128^3 (0: never populated) */
	uint64_t density_grid_cells;
	void* d_scratch;                 /* device scratch for the fp16 copy of the density grid: 2 bytes per cell */
	uint64_t scratch_bytes;
	uint32_t aabb_scale;
	uint32_t rays_per_batch, measured_batch_size, measured_batch_size_before_compaction;
	uint32_t training_step;
	float loss;
	uint32_t param_steps_bits;       /* width of d_param_steps: 16, or 32 (0 reads as 32); the file always holds 32-bit counters */
} n2_snapshot_desc;

/* Testbed::save_snapshot(path, include_optimizer_state).  Synchronises with the stream. */
int n2_snapshot_save(const char* path, const n2_snapshot_desc* desc, n2_stream_t stream);

typedef struct n2_snapshot_info {
	uint32_t n_params;
	uint32_t params_are_fp32;        /* params_type "float" (newer tiny-cuda-nn) instead of "__half" */
	uint32_t density_grid_size;
	uint64_t density_grid_cells;
	uint32_t aabb_scale;
	uint32_t rays_per_batch, measured_batch_size, measured_batch_size_before_compaction;
	uint32_t training_step;
	float loss;
	uint32_t has_optimizer_state, has_ema_weights;
	uint32_t optimizer_steps;
	float learning_rate;
} n2_snapshot_info;

typedef struct n2_snapshot_targets {
	uint32_t n_params;               /* of the model that receives the parameters: must match the file */
	float* d_master;                 /* fp32 master weights (any of the pointers may be NULL: that part is not loaded) */
	n2_half* d_params;               /* fp16 working copy */
	float* d_density_grid;           /* fp32, density_grid_cells cells; follow with n2_occupancy_update_bitfield */
	uint64_t density_grid_cells;
	float* d_first_moments;
	float* d_second_moments;
	void* d_param_steps;             /* uint32_t, or uint16_t when param_steps_bits is 16 (counts above 65535 stop there) */
	float* d_ema_weights;
	void* d_scratch;                 /* device staging: max(params_binary bytes, 2 bytes per density cell) */
	uint64_t scratch_bytes;
	uint32_t param_steps_bits;       /* 16, or 32 (0 reads as 32) */
} n2_snapshot_targets;

/* Testbed::load_snapshot: reads and checks the file ("does not contain a snapshot", parameter count, grid size). */
int n2_snapshot_open(const char* path, n2_snapshot_t** out, n2_snapshot_info* info);
/* Copies the requested parts to the device, converting fp16 <-> fp32 as needed.  Synchronises with the stream. */
int n2_snapshot_read(n2_snapshot_t* snapshot, n2_stream_t stream, const n2_snapshot_targets* targets);
void n2_snapshot_close(n2_snapshot_t* snapshot);

/* ------------------------------------------------------------------------
 * Optional event timing of the dominant kernels (off by default; the reference has only
 * wall-clock timers, src/testbed.cu:2707-2710).  When enabled, every launch of a listed kernel is
 * bracketed by a pair of events on its own stream.
 * ---------------------------------------------------------------------- */
typedef enum n2_prof_id {
	N2_PROF_GRID_FORWARD = 0,
	N2_PROF_GRID_BACKWARD_PARAMS = 1,
	N2_PROF_GRID_SECOND_ORDER = 2,
	N2_PROF_MLP_FORWARD = 3,
	N2_PROF_MLP_BACKWARD = 4,
	N2_PROF_MLP_SECOND_ORDER = 5,
	N2_PROF_COMPOSITE = 6,
	N2_PROF_SAMPLER = 7,
	N2_PROF_ADAM = 8,
	N2_PROF_FIELD_FORWARD = 9, /* the fused forward kernels of the field (grid + networks in one launch) */
	N2_PROF_FIELD_GATHER = 10, /* the level-major gather launch inside N2_PROF_FIELD_FORWARD */
	N2_PROF_COUNT = 11
} n2_prof_id;

int n2_profile_enable(int enable);
/* Restricts the timing to the ids whose bit (1 << id) is set (default: all).  An event pair costs a few microseconds of
 * stream time, so a benchmark that times whole steps selects only the kernel it reports on. */
int n2_profile_select(uint32_t id_mask);
/* Time only every `every`-th launch of each selected id (1: all).  An event pair costs a few microseconds of stream time,
 * so a benchmark that times a kernel inside its own timed region samples it. */
int n2_profile_set_period(uint32_t every);
/* Waits for all recorded events; total milliseconds and launch count per id since the last reset. */
int n2_profile_read(n2_prof_id id, float* total_ms, uint32_t* launches);
int n2_profile_reset(void);

#ifdef __cplusplus
}
#endif
#endif /* NEUS2_AMD_H */
