// Internal helpers shared by the HIP sources of libneus2_amd (not installed).
#pragma once
#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>
#include <cstdarg>
#include <cstdint>
#include <cstdio>

#include "neus2_amd.h"

#define N2_API extern "C" __attribute__((visibility("default")))

void n2_set_error(const char* fmt, ...) __attribute__((format(printf, 1, 2)));

#define N2_REQUIRE(cond, ...)                      \
	do {                                           \
		if (!(cond)) {                             \
			n2_set_error(__VA_ARGS__);             \
			return N2_ERR_INVALID_ARGUMENT;        \
		}                                          \
	} while (0)

#define N2_HIP(call)                                                                         \
	do {                                                                                     \
		hipError_t e_ = (call);                                                              \
		if (e_ != hipSuccess) {                                                              \
			n2_set_error("%s failed: %s (%s:%d)", #call, hipGetErrorString(e_), __FILE__, __LINE__); \
			return N2_ERR_HIP;                                                               \
		}                                                                                    \
	} while (0)

// After a kernel launch: launch-configuration errors surface here.
#define N2_LAUNCH_CHECK() N2_HIP(hipGetLastError())

constexpr uint32_t N2_MAX_LEVELS = 32;

struct N2SlabReduce;
struct N2StepEpilogue;  // slab_reduce.h

// How a level turns integer grid coordinates into an entry index.
enum : uint32_t {
	N2_LEVEL_DENSE = 0,  // x + y*res + z*res^2, one conditional subtract stands in for the modulo
	N2_LEVEL_HASH = 1,   // spatial hash, entries is a power of two -> mask
	N2_LEVEL_DENSE_MOD = 2,  // dense index with a true modulo (tables too small for the subtract trick)
	N2_LEVEL_HASH_MOD = 3    // spatial hash with a true modulo
};

// Host-computed per-level constants, passed to kernels by value so that host
// and device can never disagree on exp2f/ceilf rounding.
struct N2LevelTable {
	float scale[N2_MAX_LEVELS];
	uint32_t resolution[N2_MAX_LEVELS];
	uint32_t entries[N2_MAX_LEVELS];
	uint32_t offset[N2_MAX_LEVELS + 1];
	uint32_t mode[N2_MAX_LEVELS];
	uint32_t n_levels;
	// level mask: level l is switched off (zero output, zero derivatives, no gradient) for point i when
	//   l >= max_level * n_levels + 1e-3   (max_level = max_level_gpu[i] when that pointer is set)   or   l >= valid_levels
	float max_level;               // fraction of the levels in use, 1 = all
	const float* max_level_gpu;    // per point, or null
	uint32_t valid_levels;         // progressive training: number of levels switched on so far
	uint32_t active_levels;        // levels in use under max_level and valid_levels (kept up to date by the setters)
	uint32_t n_features;
	// bit l set: level l's bucketed scatter writes one record per PAIR of x-neighbour corners (see grid_bin_kernel)
	uint32_t pair_levels;
	// log2 of the entries per bucket of level l's bucketed scatter (set per launch: small levels take small buckets, so
	// that every bucket has about a workgroup's worth of records and none has to be split)
	uint8_t bucket_shift[N2_MAX_LEVELS];
};

// What the fused field kernels need of a field's parts: the grid's level table and parameters, the weights of the two
// networks, the variance parameter.  Filled by the field from its sub-objects.
struct N2FusedNets {
	const N2LevelTable* tab;
	const __half2* table;
	const n2_half* sdf_w;
	const n2_half* rgb_w;
	const n2_half* variance;
	uint32_t sdf_in_w;
	float sdf_bias;
	// N2_FUSED_FRAG_BYTES of scratch, or null: the gather launch of a full forward leaves the weight fragments of its network
	// kernel there (the first N2_FUSED_FRAG_FORWARD bytes) and, behind them, those of the backward's two weight-gradient
	// kernels (colour net, then SDF net when it has 48 inputs): built once per step instead of once per workgroup
	n2_half* frag_image;
};
constexpr uint64_t N2_FUSED_FRAG_FORWARD = 40 * 1024, N2_FUSED_FRAG_RGB = 36 * 1024, N2_FUSED_FRAG_SDF = 20 * 1024;
constexpr uint64_t N2_FUSED_FRAG_BYTES = N2_FUSED_FRAG_FORWARD + N2_FUSED_FRAG_RGB + N2_FUSED_FRAG_SDF;
// the weight-gradient launches of `mlp` read their fragments from `image` (as mlp_frag_value lays them out; null: every
// workgroup builds them from the weights).  Borrowed: the caller keeps it valid and matching the weights.
void n2_mlp_borrow_fragment_image(n2_mlp_t* mlp, const n2_half* image);
uint32_t n2_mlp_fragment_image_bytes(uint32_t in_w, uint32_t n_hidden);
const N2LevelTable* n2_grid_table(const n2_grid_t* grid);
const __half2* n2_grid_params(const n2_grid_t* grid);
bool n2_grid_lattice_order(const n2_grid_t* grid);
const n2_half* n2_mlp_params(const n2_mlp_t* mlp);
uint32_t n2_mlp_hidden_layers(const n2_mlp_t* mlp);

// The fused forward serves grids of at most 16 levels with two features whose levels are dense or hashed with a
// power-of-two table, one hidden layer in the SDF net and two in the colour net, without per-point level masks.
bool n2_fused_supported(const N2LevelTable& tab, uint32_t sdf_hidden_layers, uint32_t rgb_hidden_layers);
// NerfNetwork::forward_impl as a level-major gather kernel plus one kernel for everything behind it: writes the network
// inputs and d sdf / d input (SoA, n columns), the slopes of the encoding (16 bytes per level and sample, [n_levels][n]:
// d feature / d position without the level's scale factor, n2_slopes_pack) and the [n][16] output.
// d_live (or null): a device counter; only samples below min(*d_live, n) are evaluated, n stays the matrices' column count.
int n2_fused_field_forward(const N2FusedNets& nets, hipStream_t s, const float* d_coords, uint32_t n, n2_half* sdf_in, float* xyz_rows,
                           void* slopes, n2_half* dsdf_din, n2_half* rgb_in, n2_half* d_output, const uint32_t* d_live = nullptr,
                           const uint32_t* d_list = nullptr, const uint32_t* d_counts = nullptr, uint32_t round = 0, uint32_t est_samples = 0,
                           const float* d_xyz_soa = nullptr);
// d_xyz_soa (or null): the samples' positions once more as three rows of n floats ([3][n]), which the gather then reads
// instead of the coordinate rows
// One round of a forward pass in depth chunks (n2_composite_chunk_next): the samples begin .. begin + d_counts[round] of
// d_coords_listed, begin = d_counts[0] + ... + d_counts[round - 1].  The output of sample c goes to row d_list[c] of d_output;
// what the backward reads is stored at column c (n2_field_select then takes list positions).  est_samples: the caller's
// estimate of d_counts[round], which sizes the launches (any value gives the same results).
int n2_field_forward_listed(n2_field_t* field, n2_stream_t stream, const float* d_coords_listed, uint32_t n, const uint32_t* d_list, const uint32_t* d_counts,
                            uint32_t round, uint32_t est_samples, n2_half* d_output);
// n2_field_forward over the samples below min(*d_live, n): the trainer's marched samples fill only part of the window it
// evaluates (the window is the count measured some steps earlier, rounded up); what lies behind them is not computed.
int n2_field_forward_live(n2_field_t* field, n2_stream_t stream, const float* d_coords, uint32_t n, const uint32_t* d_live, n2_half* d_output,
                          const float* d_xyz_soa = nullptr);
// n2_generate_training_samples that also writes the positions as three rows of max_samples floats (d_xyz_rows, or null)
int n2_generate_training_samples_rows(n2_stream_t stream, uint32_t n_rays, uint32_t n_rays_total, uint32_t seed, const n2_camera* d_cameras, uint32_t n_images,
                                      const float* d_rgba, const float background[3], const uint8_t* d_bitfield, uint32_t max_samples,
                                      uint32_t* d_ray_counter, uint32_t* d_sample_counter, uint32_t* d_ray_indices, uint32_t* d_numsteps, float* d_rgb_target,
                                      float* d_coords, void* d_workspace, uint64_t workspace_bytes, float* d_xyz_rows);
// NerfNetwork::sdf / density: d_out_soa (16 x n, may be null) and / or d_row0 (fp32 copy of row 0, may be null).
// sdf_in null: one kernel that gathers sample by sample (points in lattice order, whose table lines stay cached);
// else a level-major gather into the feature rows 3.. of sdf_in (SoA, n columns) followed by the network kernel.
// lattice (with d_xyz and sdf_in null): sample i is lattice point first + i, x fastest, at (c / res) * extent + corner.
struct N2Lattice {
	uint32_t res[3], first, total;  // total = res[0] res[1] res[2]
	float inv_res[3], extent[3], corner[3];
};
int n2_fused_field_sdf(const N2FusedNets& nets, hipStream_t s, const float* d_xyz, uint32_t ps, uint32_t ds, uint32_t n, n2_half* d_out_soa,
                       float* d_row0, bool density, n2_half* sdf_in, uint32_t row0_n = 0xFFFFFFFFu, const N2Lattice* lattice = nullptr);

// n2_composite_loss_indexed that also fills the compacted batch up to max_samples_compacted samples (fill = true): slot j
// behind the n_in = min(*d_compacted_counter, max_samples_compacted) kept samples holds a copy of slot j % n_in (coordinates,
// source index, output gradient scaled by n_in / max_samples_compacted), what n2_fill_rollover_f32 and
// n2_fill_rollover_and_rescale_f16 would write in launches of their own.
int n2_composite_loss_filled(n2_stream_t stream, const n2_composite_config* cfg, uint32_t n_rays, const uint32_t* d_ray_counter, uint32_t* d_numsteps,
                             const n2_half* d_network_output, const float* d_coords, const float* d_rgb_target, uint32_t max_samples_compacted,
                             uint32_t* d_compacted_counter, float* d_coords_compacted, n2_half* d_dloss_doutput, float* d_loss, uint32_t* d_source_index,
                             void* d_workspace, uint64_t workspace_bytes, bool fill, const uint32_t* d_column_of = nullptr);
// Forward pass in depth chunks (composite.hip): round `round` retires the rays whose transmittance behind the samples
// listed last is below the compositor's cut and lists the next `chunk` samples of the others.  d_counts[r]: samples of
// round r (d_counts_other: the counters of the following step, cleared by round 0); d_list: marched sample of every listed
// sample, rounds side by side; d_column_of: the inverse map; d_coords_listed: the coordinate rows of the listed samples in
// list order.  d_column_of goes to n2_composite_loss_filled, whose source_index then names list positions.
constexpr uint32_t N2_CHUNK_MAX_ROUNDS = 8;
uint64_t n2_composite_chunk_state_bytes(uint32_t max_rays);
int n2_composite_chunk_next(n2_stream_t stream, const n2_composite_config* cfg, uint32_t n_rays, const uint32_t* d_ray_counter, const uint32_t* d_numsteps,
                            const n2_half* d_network_output, const float* d_coords, uint32_t round, uint32_t chunk, void* d_state, uint32_t* d_counts,
                            uint32_t* d_counts_other, uint32_t* d_list, uint32_t* d_column_of, float* d_coords_listed);

// What the field hangs on its colour net's backward launch (n2_mlp_backward_rows_indexed): for the same samples,
//   * row 0 of d_dL_dinput also takes row 3 of d_dL_doutput (the direct gradient of the SDF output);
//   * v[d] = row 35 + d of d_dL_dinput + row 4 + d of d_dL_doutput / ek_batch + row 8 + d of d_dL_doutput (dL/dnormal), written
//     as fp32 rows (v, [3][n]) and as rows 0..2 of the SDF net's second-order input (d_density_in, fp16 rows of n columns);
//   * rows 3.. of that input: the encoding's dL_ddLdoutput = J v from the slopes the fused forward saved ([levels][n_src] 16-byte
//     blocks, read at the sample's column of the index; scale[l] = the level's scale factor);
//   * var_part[workgroup] = the workgroup's sum of row 7 of d_dL_doutput (n2_mlp_wgrad_blocks(n) workgroups).
// With it the launch takes d_input sample-major ([n_cols][N2_RGB_IN_PITCH], the rows behind are zero) and writes only rows 0..15 of d_dL_dinput, sample-major too
// ([n][16]: the AoS output gradient of the SDF net's backward).
constexpr uint32_t N2_RGB_IN_PITCH = 40;  // values per sample of the colour net's saved input (38 in use)
struct N2FieldPrepTail {
	float ek_batch;
	const void* slopes;
	uint32_t n_src, enc_w;
	float scale[16];
	float* v;
	void* d_density_in;
	float* var_part;
};
uint32_t n2_mlp_wgrad_blocks(uint32_t n);

// n2_mlp_backward_rows / n2_mlp_backward_and_second_order whose input is read through an index: sample i of the batch is
// column d_index[i] of d_input, a matrix with n_cols columns (d_index null: column i of n columns).  Every other operand is
// indexed by i.  The field's backward uses them to read the activations its forward saved for ALL marched samples.
// dx_out_and_normal_only (48-input network with two hidden layers, the field's colour net): of d_dL_dinput only rows 0..15
// and 35..37 are written (the gradients of the SDF net's output and of the normal; nothing reads the others).
// dx_encoding_only (48-input network, the field's SDF net): only rows 3..34, the encoding's, are written.
int n2_mlp_backward_rows_indexed(n2_mlp_t* mlp, n2_stream_t stream, const n2_half* d_input, uint32_t n_cols, const uint32_t* d_index, uint32_t n,
                                 const n2_half* d_dL_doutput, n2_layout dL_layout, uint32_t n_rows, n2_half* d_dL_dinput, n2_grad_mode mode,
                                 bool dx_out_and_normal_only, const N2FieldPrepTail* tail = nullptr);
int n2_mlp_backward_and_second_order_indexed(n2_mlp_t* mlp, n2_stream_t stream, const n2_half* d_input, uint32_t n_cols, const uint32_t* d_index,
                                             uint32_t n, const n2_half* d_dL_doutput, n2_layout dL_layout, n2_half* d_dL_dinput,
                                             const n2_half* d_dL_ddLdinput, const n2_half* d_second_dL_doutput, n2_grad_mode mode,
                                             bool dx_encoding_only);
// n2_adam_step that does nothing when *d_gate is zero on the device (d_gate null: always steps)
// sums (or null): a slab summation whose gradients lie inside d_gradients; the kernel's first workgroups run it, store the
// fp16 gradients and step those parameters themselves (the other workgroups leave them alone)
// d_steps: uint32_t (steps_bits 32) or uint16_t counters (16)
// epilogue (or null): one more workgroup of the launch does the caller's bookkeeping (slab_reduce.h), gated or not
// done_event (or null): recorded by the completion of the launch itself (hipExtLaunchKernel's stop event)
int n2_adam_step_gated(n2_stream_t stream, const n2_adam_config* config, uint32_t n_params, uint32_t n_matrix_params,
                       float loss_scale, float* d_master, n2_half* d_params, const n2_half* d_gradients, float* d_m1,
                       float* d_m2, void* d_steps, uint32_t steps_bits, const uint32_t* d_gate, const N2SlabReduce* sums = nullptr,
                       const N2StepEpilogue* epilogue = nullptr, hipEvent_t done_event = nullptr);
// true when 1 - beta^t is exactly 1 in fp32 for both betas from the end of the kernel's bias-correction table on: the step
// counters may then be 16 bits wide (steps_bits 16, saturating at 65535) instead of 32
bool n2_adam_counters_may_saturate(float beta1, float beta2);
// n2_mlp_reduce_deferred that also adds up n_parts floats, in a fixed order, into one fp16 value ([+=] when accumulate)
int n2_mlp_reduce_deferred_sum(n2_mlp_t* a, n2_mlp_t* b, n2_stream_t stream, const float* d_parts, uint32_t n_parts, n2_half* d_sum, int accumulate);
// The same work as a plan instead of a launch: what is pending is handed to *out (and no longer pending), for
// n2_slab_reduce_launch or for a kernel that carries the summation (n2_adam_step_gated).
// forgets the gradient passes that are pending (their partial sums are dropped): for the error path of a caller that will
// not run the reduction
void n2_mlp_drop_pending(n2_mlp_t* mlp);
int n2_mlp_reduce_deferred_plan(n2_mlp_t* a, n2_mlp_t* b, const float* d_parts, uint32_t n_parts, n2_half* d_sum, int accumulate, N2SlabReduce* out);
int n2_slab_reduce_launch(n2_stream_t stream, const N2SlabReduce& plan);
// n2_field_backward that leaves the summation of the networks' weight-gradient slabs and of the variance gradient's partial
// sums to the caller: *sums is the plan (their fp16 gradients are not written until it has run)
int n2_field_backward_deferred(n2_field_t* field, n2_stream_t stream, const float* d_coords, uint32_t n, const n2_half* d_dL_doutput, uint32_t n_rays_ek,
                               n2_grad_mode mode, N2SlabReduce* sums);
// n2_field_select without the copy of the index: d_source_index must stay valid and unchanged until the backward has run
int n2_field_select_borrow(n2_field_t* field, const uint32_t* d_source_index, uint32_t n_source, uint32_t n);
// n2_grid_backward_fused whose positions (SoA 3 x n_cols) and d_dL_dy_second rows (n_cols columns) are read through d_index.
int n2_grid_backward_fused_indexed(n2_grid_t* grid, n2_stream_t stream, const float* d_xyz_rows, uint32_t n_cols, const uint32_t* d_index,
                                   uint32_t n_points, const n2_half* d_dL_dy, const float* d_dL_ddLdx, const n2_half* d_dL_dy_second,
                                   n2_grad_mode mode);

// row 0 of n2_field_sdf (density: of n2_field_density) for the first n_keep <= n samples as fp32 (d_scratch16: [16][n] fp16, used when the fused kernels do not serve the field)
int n2_field_sdf_row0(n2_field_t* field, n2_stream_t stream, const float* d_xyz, uint32_t point_stride, uint32_t dim_stride, uint32_t n, uint32_t n_keep,
                      float* d_row0, n2_half* d_scratch16, bool density = false);
// the same on n points of a lattice, generated inside the kernel; false when the field's fused kernels do not serve it (the
// caller then writes the positions out and uses n2_field_sdf_row0)
bool n2_field_sdf_row0_lattice(n2_field_t* field, n2_stream_t stream, const N2Lattice& lattice, uint32_t n, uint32_t n_keep, float* d_row0, int* rc);

static inline hipStream_t n2_stream(n2_stream_t s) { return reinterpret_cast<hipStream_t>(s); }

// Zero-fill with a kernel (safe to record into HIP graphs, unlike memset nodes).
int n2_fill_zero_u32(hipStream_t stream, void* d_ptr, size_t n_bytes);
// Store one 32-bit value with a one-thread kernel.
int n2_set_u32(hipStream_t stream, uint32_t* d_ptr, uint32_t value);

// Event timing of a kernel launch; a no-op unless n2_profile_enable(1) was called.
void n2_prof_begin(int id, hipStream_t stream);
void n2_prof_end(int id, hipStream_t stream);
struct N2ProfScope {
	int id;
	hipStream_t s;
	N2ProfScope(int id_, hipStream_t s_) : id(id_), s(s_) { n2_prof_begin(id, s); }
	~N2ProfScope() { n2_prof_end(id, s); }
};
