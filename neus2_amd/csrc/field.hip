// The NeuS field: host-side composition of grid, SDF MLP, direction encoding,
// colour MLP and variance (counterpart of NerfNetwork<T>::forward_impl /
// backward_impl / sdf / density) plus the few element-wise kernels it needs.
//
// Where the reference moves rows between temporaries with ~25 tiny launches,
// the buffers here are laid out so that producers write straight into their
// consumer's rows (the grid writes rows 3..34 of the SDF net's input, the SDF
// net writes rows 0..15 of the colour net's input, the second-order grid pass
// writes rows 3..34 of the MLP's second-order input), which leaves three glue
// kernels in the forward and three in the backward.
#include "n2_common.h"
#include "slab_reduce.h"
#include "grid_device.h"

#include <new>

typedef _Float16 hf;

struct n2_field {
	n2_grid_t* grid;
	n2_mlp_t* sdf;
	n2_mlp_t* rgb;
	uint32_t enc_w, sdf_in_w, rgb_in_w;
	float sdf_bias;
	uint32_t off_sdf, off_rgb, off_grid, off_var, n_params;
	const hf* params;
	hf* grads;
	unsigned char* ws;
	uint64_t ws_bytes;
	uint32_t max_batch, max_batch_bwd;
	// Batch size for which the padding rows of each input-side matrix of the two networks hold zeros (0: not known).
	// The matrices are rows x N with N the batch size of the call, so the padding rows move when N changes.
	struct { uint32_t sdf_in, rgb_in, d_density_in; } pad_n;
	// carved from the workspace
	hf* sdf_in;        // [sdf_in_w][N]
	float* xyz;        // [3][N]  positions of the last forward, row per coordinate (the grid kernels read each row 16 times)
	hf* rgb_in;        // [48][N]; after a fused forward [N][N2_RGB_IN_PITCH] (sample-major: the networks' kernels hold 8 consecutive rows per lane)
	float* dy_dx;      // [enc_w][N][3] fp32, or (slopes_saved) 16-byte slope blocks [levels][N] without the levels' scale factors
	hf* dsdf_din;      // [sdf_in_w][N]  d sdf / d (SDF net input)
	hf* d_rgb_in;      // [48][N]; behind a fused forward [N][16], rows 0..15 only
	hf* d_sdf_in;      // [sdf_in_w][N]
	float* v;          // [3][N]  dL / d normal
	hf* d_density_in;  // [sdf_in_w][N]  second-order input of the SDF net
	float* var_part;    // one partial sum of the variance gradient per workgroup of the backward's preparation kernel
	// a selection of the last forward's samples (n2_field_select): the backward reads the rows above through this index
	uint32_t* sel_index;  // [n]
	const uint32_t* sel_use;  // the index in use: sel_index, or the caller's own buffer (n2_field_select_borrow)
	uint32_t last_n;      // samples of the last forward
	uint32_t sel_n;       // samples selected (0: the backward's batch is the forward's)
	void* ws_sdf;
	void* ws_rgb;
	void* ws_grid;
	hf* frag_image;  // the fused forward's weight fragments
	bool fused;  // forward passes go through the fused kernels where the configuration allows (n2_field_set_fused)
	bool frags_ready;   // the last forward's gather launch left the weight-gradient kernels' fragments in frag_image (same weights since)
	bool slopes_saved;  // the last forward left the encoding's Jacobian as fp16 slopes (fused forward), not as fp32 dy_dx
};

constexpr uint32_t FB = 256;
constexpr uint32_t RGB_IN_ROWS = 38;  // colour net input: 16 SDF-net outputs, 16 SH, xyz, normal (padded to 48)

// ----------------------------------------------------------------------------
// glue kernels
// ----------------------------------------------------------------------------
// rows 0..2 = half(x) - half(0.5) (computed in half precision like the reference's (T)pos - (T)0.5f).  The padding rows
// [3 + enc_w, sdf_in_w) are zero as in the reference, but not written here: they are cleared once per batch size
// (zero_padding below) and nothing writes them afterwards.
__global__ void __launch_bounds__(FB) field_pack_sdf_input_kernel(const float* __restrict__ xyz, uint32_t ps, uint32_t ds, uint32_t N,
                                                                  hf* __restrict__ sdf_in, float* __restrict__ xyz_rows) {
	const uint32_t i = blockIdx.x * FB + threadIdx.x;
	if (i >= N) return;
	const float* q = xyz + (size_t)i * ps;
#pragma unroll
	for (int d = 0; d < 3; ++d) {
		const float x = q[(size_t)d * ds];
		sdf_in[(size_t)d * N + i] = (hf)x - (hf)0.5f;
		xyz_rows[(size_t)d * N + i] = x;
	}
}

__device__ __forceinline__ void sh4_eval(float x, float y, float z, float* o) {
	const float xy = x * y, xz = x * z, yz = y * z, x2 = x * x, y2 = y * y, z2 = z * z;
	o[0] = 0.28209479177387814f;
	o[1] = -0.48860251190291987f * y;
	o[2] = 0.48860251190291987f * z;
	o[3] = -0.48860251190291987f * x;
	o[4] = 1.0925484305920792f * xy;
	o[5] = -1.0925484305920792f * yz;
	o[6] = 0.94617469575755997f * z2 - 0.31539156525251999f;
	o[7] = -1.0925484305920792f * xz;
	o[8] = 0.54627421529603959f * x2 - 0.54627421529603959f * y2;
	o[9] = 0.59004358992664352f * y * (-3.0f * x2 + y2);
	o[10] = 2.8906114426405538f * xy * z;
	o[11] = 0.45704579946446572f * y * (1.0f - 5.0f * z2);
	o[12] = 0.3731763325901154f * z * (5.0f * z2 - 3.0f);
	o[13] = 0.45704579946446572f * x * (1.0f - 5.0f * z2);
	o[14] = 1.4453057213202769f * z * (x2 - y2);
	o[15] = 0.59004358992664352f * x * (-x2 + 3.0f * y2);
}

// normal = dy_dx^T dsdf_din[3..3+enc_w) + dsdf_din[0..3); then the colour net's input rows
// 16..31 (SH of the direction), 32..34 (xyz), 35..37 (normal); the padding rows 38..47 stay zero (zero_padding).
__global__ void __launch_bounds__(FB) field_normals_rgb_input_kernel(const float* __restrict__ coords, uint32_t N, uint32_t enc_w,
                                                                     const hf* __restrict__ dsdf_din, const float* __restrict__ dy_dx,
                                                                     hf* __restrict__ rgb_in) {
	const uint32_t i = blockIdx.x * FB + threadIdx.x;
	if (i >= N) return;
	float n0 = 0.f, n1 = 0.f, n2 = 0.f;
	// eight rows' loads are issued before the first is used: the kernel is a stream of 14 bytes per lane and row, and one
	// row in flight per lane leaves it waiting on memory latency
	constexpr uint32_t U = 8;
	uint32_t k = 0;
	for (; k + U <= enc_w; k += U) {
		float g[U], j[U][3];
#pragma unroll
		for (uint32_t u = 0; u < U; ++u) {
			g[u] = (float)dsdf_din[(size_t)(3 + k + u) * N + i];
			const float* q = dy_dx + ((size_t)(k + u) * N + i) * 3;
			j[u][0] = q[0]; j[u][1] = q[1]; j[u][2] = q[2];
		}
#pragma unroll
		for (uint32_t u = 0; u < U; ++u) {
			n0 = fmaf(g[u], j[u][0], n0);
			n1 = fmaf(g[u], j[u][1], n1);
			n2 = fmaf(g[u], j[u][2], n2);
		}
	}
	for (; k < enc_w; ++k) {
		const float g = (float)dsdf_din[(size_t)(3 + k) * N + i];
		const float* j = dy_dx + ((size_t)k * N + i) * 3;
		n0 = fmaf(g, j[0], n0);
		n1 = fmaf(g, j[1], n1);
		n2 = fmaf(g, j[2], n2);
	}
	n0 += (float)dsdf_din[i];
	n1 += (float)dsdf_din[(size_t)N + i];
	n2 += (float)dsdf_din[(size_t)2 * N + i];
	const float* c = coords + (size_t)i * 7;
	float sh[16];
	sh4_eval(c[4] * 2.f - 1.f, c[5] * 2.f - 1.f, c[6] * 2.f - 1.f, sh);
#pragma unroll
	for (int k = 0; k < 16; ++k) rgb_in[(size_t)(16 + k) * N + i] = (hf)sh[k];
	rgb_in[(size_t)32 * N + i] = (hf)c[0];
	rgb_in[(size_t)33 * N + i] = (hf)c[1];
	rgb_in[(size_t)34 * N + i] = (hf)c[2];
	rgb_in[(size_t)35 * N + i] = (hf)n0;
	rgb_in[(size_t)36 * N + i] = (hf)n1;
	rgb_in[(size_t)37 * N + i] = (hf)n2;
}

// output rows 3 (sdf + bias), 4..6 (normal), 7 (variance), 8..10 (direction); rows 0..2 and
// 11..15 keep what the colour net wrote.  The SDF and the normal are taken from the colour net's input (rows 0 and
// 35..37), where they already stand in half precision.
__global__ void __launch_bounds__(FB) field_finish_output_kernel(const float* __restrict__ coords, uint32_t N, const hf* __restrict__ rgb_in,
                                                                 hf bias, const hf* __restrict__ variance, hf* __restrict__ output) {
	const uint32_t i = blockIdx.x * FB + threadIdx.x;
	if (i >= N) return;
	hf* o = output + (size_t)i * 16;
	const float* c = coords + (size_t)i * 7;
	o[3] = rgb_in[i] + bias;
	o[4] = rgb_in[(size_t)35 * N + i];
	o[5] = rgb_in[(size_t)36 * N + i];
	o[6] = rgb_in[(size_t)37 * N + i];
	o[7] = variance[0];
	o[8] = (hf)c[4];
	o[9] = (hf)c[5];
	o[10] = (hf)c[6];
}

// After the colour net's backward, one pass over the samples prepares everything the SDF net's and the grid's
// backward read:
//  * the SDF output also receives dL_doutput row 3 directly (the density path): added to row 0 of the colour net's
//    input gradient, which is the SDF net's output gradient;
//  * v = dL/dnormal = colour-net input gradient rows 35..37 + eikonal rows 4..6 / batch + cos rows 8..10;
//  * second-order MLP input rows 0..2 = half(v), rows 3 .. 3+enc_w = dy_dx v (the encoding's
//    backward_backward_input output dL_ddLdoutput, taken from the Jacobian the forward stored instead of
//    gathering the table again); the padding rows above stay zero (zero_padding);
//  * the variance gradient is the sum of row 7: every workgroup leaves its partial sum in var_part[blockIdx.x] and
//    the launch that reduces the networks' weight gradients adds them up in a fixed order.
struct LevelScales { float s[16]; };
// The unfused path's form of this work (the Jacobian as the grid encoding's fp32 dy_dx [enc_w][n_src][3]); after a fused
// forward the same work rides in the colour net's backward launch (N2FieldPrepTail), which reads the slopes instead.
__global__ void __launch_bounds__(FB) field_backward_prep_kernel(uint32_t N, uint32_t enc_w, hf* __restrict__ d_rgb_in,
                                                                 const hf* __restrict__ dL_dout, float ek_batch, const float* __restrict__ dy_dx,
                                                                 float* __restrict__ v, hf* __restrict__ d_density_in,
                                                                 float* __restrict__ var_part, const uint32_t* __restrict__ src_index,
                                                                 uint32_t n_src) {
	typedef _Float16 half8 __attribute__((ext_vector_type(8)));
	__shared__ float part[FB / 64];
	const uint32_t i = blockIdx.x * FB + threadIdx.x;
	float s = 0.f;
	if (i < N) {
		// the Jacobian rows are those of the forward: of sample src_index[i] among n_src when a selection is active
		const size_t js = src_index ? min(src_index[i], n_src - 1u) : i, jn = src_index ? n_src : N;
		const half8 lo = *reinterpret_cast<const half8*>(dL_dout + (size_t)i * 16), hi = *reinterpret_cast<const half8*>(dL_dout + (size_t)i * 16 + 8);
		d_rgb_in[i] = d_rgb_in[i] + lo[3];
		s = (float)lo[7];
		float vv[3];
#pragma unroll
		for (int d = 0; d < 3; ++d) {
			float x = (float)d_rgb_in[(size_t)(35 + d) * N + i];
			x += (float)lo[4 + d] / ek_batch;
			x += (float)hi[d];
			vv[d] = x;
			v[(size_t)d * N + i] = x;
			d_density_in[(size_t)d * N + i] = (hf)x;
		}
		// eight rows' loads in flight per lane
		constexpr uint32_t U = 8;
		uint32_t r = 0;
		for (; r + U <= enc_w; r += U) {
			float j[U][3];
#pragma unroll
			for (uint32_t u = 0; u < U; ++u) {
				const float* q = dy_dx + ((size_t)(r + u) * jn + js) * 3;
				j[u][0] = q[0]; j[u][1] = q[1]; j[u][2] = q[2];
			}
#pragma unroll
			for (uint32_t u = 0; u < U; ++u) d_density_in[(size_t)(3 + r + u) * N + i] = (hf)(j[u][0] * vv[0] + j[u][1] * vv[1] + j[u][2] * vv[2]);
		}
		for (; r < enc_w; ++r) {
			const float* j = dy_dx + ((size_t)r * jn + js) * 3;
			d_density_in[(size_t)(3 + r) * N + i] = (hf)(j[0] * vv[0] + j[1] * vv[1] + j[2] * vv[2]);
		}
	}
#pragma unroll
	for (int o = 32; o > 0; o >>= 1) s += __shfl_xor(s, o);
	if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = s;
	__syncthreads();
	if (threadIdx.x == 0) {
		float t = 0.f;
		for (uint32_t w = 0; w < FB / 64; ++w) t += part[w];
		var_part[blockIdx.x] = t;
	}
}

// The selection of a backward batch among the forward's samples: the index is copied (clamped into the forward's batch)
// so that the caller's buffer is free again; the backward kernels read the saved rows through it.
__global__ void __launch_bounds__(FB) field_select_kernel(uint32_t n, uint32_t n_src, const uint32_t* __restrict__ index, uint32_t* __restrict__ o_index) {
	const uint32_t j = blockIdx.x * FB + threadIdx.x;
	if (j < n) o_index[j] = min(index[j], n_src - 1u);
}

__global__ void __launch_bounds__(FB) field_add_bias_kernel(uint32_t N, hf bias, hf* __restrict__ row0) {
	const uint32_t i = blockIdx.x * FB + threadIdx.x;
	if (i >= N) return;
	row0[i] = row0[i] + bias;
}

// sdf -> logistic density, computed in half precision like the reference kernel
__global__ void __launch_bounds__(FB) field_sdf_to_density_kernel(uint32_t N, const hf* __restrict__ variance, hf* __restrict__ row0) {
	const uint32_t i = blockIdx.x * FB + threadIdx.x;
	if (i >= N) return;
	const hf s = (hf)__expf((float)(variance[0] * (hf)10.0f));
	const hf x = row0[i] * s;
	const hf sig = (hf)(1.0f / (1.0f + __expf(-(float)x)));
	row0[i] = s * sig * ((hf)1.0f - sig);
}

// ----------------------------------------------------------------------------
// host side
// ----------------------------------------------------------------------------
static inline uint64_t align256(uint64_t x) { return (x + 255) / 256 * 256; }

N2_API int n2_field_create(const n2_field_config* cfg, n2_field_t** out) {
	N2_REQUIRE(out != nullptr && cfg != nullptr, "n2_field_create: null argument");
	*out = nullptr;
	n2_field* f = new (std::nothrow) n2_field();
	N2_REQUIRE(f != nullptr, "n2_field_create: out of host memory");
	*f = n2_field{};
	int rc = n2_grid_create(cfg->n_levels, cfg->n_features_per_level, cfg->log2_hashmap_size, cfg->base_resolution,
	                        cfg->per_level_scale, &f->grid);
	if (rc == N2_OK) {
		f->enc_w = n2_grid_output_width(f->grid);
		f->sdf_in_w = (3 + f->enc_w + 15) / 16 * 16;  // next_multiple(3 + encoding, 16)
		f->rgb_in_w = 48;                             // next_multiple(3 + 3 + 16 + 16, 16)
		rc = n2_mlp_create(f->sdf_in_w, cfg->sdf_hidden_layers, &f->sdf);
	}
	if (rc == N2_OK) rc = n2_mlp_create(f->rgb_in_w, cfg->rgb_hidden_layers, &f->rgb);
	if (rc == N2_OK) rc = n2_mlp_set_deferred_reduction(f->sdf, 1);
	if (rc == N2_OK) rc = n2_mlp_set_deferred_reduction(f->rgb, 1);
	if (rc != N2_OK) {
		n2_field_destroy(f);
		return rc;
	}
	f->sdf_bias = cfg->sdf_bias;
	f->fused = true;
	f->off_sdf = 0;
	f->off_rgb = n2_mlp_n_params(f->sdf);
	f->off_grid = f->off_rgb + n2_mlp_n_params(f->rgb);
	f->off_var = f->off_grid + n2_grid_n_params(f->grid);
	f->n_params = f->off_var + 4;
	*out = f;
	return N2_OK;
}

N2_API void n2_field_destroy(n2_field_t* f) {
	if (!f) return;
	n2_grid_destroy(f->grid);
	n2_mlp_destroy(f->sdf);
	n2_mlp_destroy(f->rgb);
	delete f;
}

N2_API n2_grid_t* n2_field_encoding(n2_field_t* field) { return field ? field->grid : nullptr; }

N2_API int n2_field_set_fused(n2_field_t* field, int enable) {
	N2_REQUIRE(field != nullptr, "n2_field_set_fused: field is null");
	field->fused = enable != 0;
	return N2_OK;
}
N2_API int n2_field_set_colour_gradient_exponent(n2_field_t* field, int exponent) {
	N2_REQUIRE(field != nullptr, "n2_field_set_colour_gradient_exponent: field is null");
	return n2_mlp_set_output_gradient_exponent(field->rgb, exponent);
}
N2_API uint32_t n2_field_n_params(const n2_field_t* f) { return f ? f->n_params : 0; }

N2_API int n2_field_param_offsets(const n2_field_t* f, uint32_t offsets[5]) {
	N2_REQUIRE(f != nullptr && offsets != nullptr, "n2_field_param_offsets: null argument");
	offsets[0] = f->off_sdf; offsets[1] = f->off_rgb; offsets[2] = f->off_grid; offsets[3] = f->off_var; offsets[4] = f->n_params;
	return N2_OK;
}

N2_API int n2_field_set_params(n2_field_t* f, const n2_half* d_params, n2_half* d_gradients) {
	N2_REQUIRE(f != nullptr && d_params != nullptr, "n2_field_set_params: null argument");
	N2_REQUIRE(reinterpret_cast<uintptr_t>(d_params) % 16 == 0 && reinterpret_cast<uintptr_t>(d_gradients) % 16 == 0,
	           "n2_field_set_params: buffers must be 16-byte aligned");
	f->params = reinterpret_cast<const hf*>(d_params);
	f->frags_ready = false;
	f->grads = reinterpret_cast<hf*>(d_gradients);
	auto g = [&](uint32_t off) { return d_gradients ? d_gradients + off : nullptr; };
	if (int rc = n2_mlp_set_params(f->sdf, d_params + f->off_sdf, g(f->off_sdf))) return rc;
	if (int rc = n2_mlp_set_params(f->rgb, d_params + f->off_rgb, g(f->off_rgb))) return rc;
	return n2_grid_set_params(f->grid, d_params + f->off_grid, g(f->off_grid));
}

struct FieldCarve {
	uint64_t sdf_in, xyz, rgb_in, dy_dx, dsdf_din, d_rgb_in, d_sdf_in, v, d_density_in, var_part, sel_index, frag_image, ws_sdf, ws_rgb, ws_grid, total;
};

// nf: largest forward batch, nbw: largest batch that is also run backward
static FieldCarve carve(const n2_field_t* f, uint32_t nf, uint32_t nbw) {
	FieldCarve c{};
	uint64_t o = 0;
	uint64_t n = nf;
	auto take = [&](uint64_t bytes) { const uint64_t at = o; o = align256(o + bytes); return at; };
	c.sdf_in = take(2ull * f->sdf_in_w * n);
	c.xyz = take(12ull * n);
	c.rgb_in = take(2ull * f->rgb_in_w * n);
	c.dy_dx = take(12ull * f->enc_w * n);
	c.dsdf_din = take(2ull * f->sdf_in_w * n);
	n = nbw;
	c.d_rgb_in = take(2ull * f->rgb_in_w * n);
	c.d_sdf_in = take(2ull * f->sdf_in_w * n);
	c.v = take(12ull * n);
	c.d_density_in = take(2ull * f->sdf_in_w * n);
	c.var_part = take(4ull * ((n + 127) / 128 + 1));  // one float per workgroup of whichever kernel forms the partial sums
	c.sel_index = take(4ull * n);
	c.frag_image = take(N2_FUSED_FRAG_BYTES);
	c.ws_sdf = take(n2_mlp_workspace_bytes(f->sdf));
	c.ws_rgb = take(n2_mlp_workspace_bytes(f->rgb));
	c.ws_grid = take(n2_grid_workspace_bytes(f->grid, (uint32_t)nbw));
	c.total = o;
	return c;
}

N2_API uint64_t n2_field_workspace_bytes(const n2_field_t* f, uint32_t max_batch, uint32_t max_batch_backward) {
	return f ? carve(f, max_batch, max_batch_backward < max_batch ? max_batch_backward : max_batch).total : 0;
}

N2_API int n2_field_set_workspace(n2_field_t* f, void* d_workspace, uint64_t n_bytes, uint32_t max_batch, uint32_t max_batch_backward) {
	N2_REQUIRE(f != nullptr, "n2_field_set_workspace: field is null");
	N2_REQUIRE(d_workspace != nullptr, "n2_field_set_workspace: workspace is null");
	N2_REQUIRE(reinterpret_cast<uintptr_t>(d_workspace) % 256 == 0, "n2_field_set_workspace: workspace must be 256-byte aligned");
	N2_REQUIRE(max_batch % 8 == 0, "n2_field_set_workspace: max_batch %u must be a multiple of 8", max_batch);
	if (max_batch_backward > max_batch) max_batch_backward = max_batch;
	const FieldCarve c = carve(f, max_batch, max_batch_backward);
	N2_REQUIRE(n_bytes >= c.total, "n2_field_set_workspace: %llu bytes given, %llu needed for batch %u", (unsigned long long)n_bytes,
	           (unsigned long long)c.total, max_batch);
	unsigned char* b = reinterpret_cast<unsigned char*>(d_workspace);
	f->ws = b; f->ws_bytes = n_bytes; f->max_batch = max_batch; f->max_batch_bwd = max_batch_backward;
	f->sdf_in = reinterpret_cast<hf*>(b + c.sdf_in);
	f->xyz = reinterpret_cast<float*>(b + c.xyz);
	f->rgb_in = reinterpret_cast<hf*>(b + c.rgb_in);
	f->dy_dx = reinterpret_cast<float*>(b + c.dy_dx);
	f->dsdf_din = reinterpret_cast<hf*>(b + c.dsdf_din);
	f->d_rgb_in = reinterpret_cast<hf*>(b + c.d_rgb_in);
	f->d_sdf_in = reinterpret_cast<hf*>(b + c.d_sdf_in);
	f->v = reinterpret_cast<float*>(b + c.v);
	f->d_density_in = reinterpret_cast<hf*>(b + c.d_density_in);
	f->var_part = reinterpret_cast<float*>(b + c.var_part);
	f->sel_index = reinterpret_cast<uint32_t*>(b + c.sel_index);
	f->frag_image = reinterpret_cast<hf*>(b + c.frag_image);
	f->frags_ready = false;
	f->last_n = 0;
	f->sel_n = 0;
	f->pad_n = {0, 0, 0};
	f->ws_sdf = b + c.ws_sdf;
	f->ws_rgb = b + c.ws_rgb;
	f->ws_grid = b + c.ws_grid;
	if (int rc = n2_mlp_set_workspace(f->sdf, f->ws_sdf, n2_mlp_workspace_bytes(f->sdf))) return rc;
	if (int rc = n2_mlp_set_workspace(f->rgb, f->ws_rgb, n2_mlp_workspace_bytes(f->rgb))) return rc;
	const uint64_t gb = n2_grid_workspace_bytes(f->grid, max_batch_backward);
	return n2_grid_set_workspace(f->grid, gb ? f->ws_grid : nullptr, gb, max_batch_backward);
}

static int check_field(const n2_field_t* f, const char* fn, uint32_t n) {
	N2_REQUIRE(f != nullptr, "%s: field is null", fn);
	N2_REQUIRE(f->params != nullptr, "%s: n2_field_set_params has not been called", fn);
	N2_REQUIRE(f->ws != nullptr, "%s: n2_field_set_workspace has not been called", fn);
	N2_REQUIRE(n <= f->max_batch, "%s: batch %u exceeds the workspace's max_batch %u", fn, n, f->max_batch);
	N2_REQUIRE(n % 8 == 0, "%s: batch size %u is not a multiple of 8", fn, n);
	return N2_OK;
}

static inline dim3 fgrid(uint32_t n) { return dim3((n + FB - 1) / FB); }

static N2FusedNets fused_nets(const n2_field_t* f) {
	N2FusedNets nets;
	nets.tab = n2_grid_table(f->grid);
	nets.table = n2_grid_params(f->grid);
	nets.sdf_w = reinterpret_cast<const n2_half*>(f->params + f->off_sdf);
	nets.rgb_w = reinterpret_cast<const n2_half*>(f->params + f->off_rgb);
	nets.variance = reinterpret_cast<const n2_half*>(f->params + f->off_var);
	nets.sdf_in_w = f->sdf_in_w;
	nets.sdf_bias = f->sdf_bias;
	nets.frag_image = reinterpret_cast<n2_half*>(f->frag_image);
	return nets;
}
// the level mask can change between calls (n2_grid_set_max_level_gpu), so the check is made per call
static bool fused_ok(const n2_field_t* f) {
	return n2_fused_supported(*n2_grid_table(f->grid), n2_mlp_hidden_layers(f->sdf), n2_mlp_hidden_layers(f->rgb));
}

// Rows [first_row, n_rows) of the rows x n matrix m are padding: the networks read them and they must be zero.  No kernel
// writes them, so they are cleared when the batch size (the row pitch) differs from the one they were last cleared for.
static int zero_padding(hipStream_t s, hf* m, uint32_t first_row, uint32_t n_rows, uint32_t n, uint32_t& cleared_for) {
	if (cleared_for == n || first_row >= n_rows) return N2_OK;
	if (int rc = n2_fill_zero_u32(s, m + (size_t)first_row * n, (size_t)(n_rows - first_row) * n * sizeof(hf))) return rc;
	cleared_for = n;
	return N2_OK;
}

N2_API int n2_field_forward(n2_field_t* f, n2_stream_t stream, const float* d_coords, uint32_t n, n2_half* d_output) {
	return n2_field_forward_live(f, stream, d_coords, n, nullptr, d_output);
}

int n2_field_forward_live(n2_field_t* f, n2_stream_t stream, const float* d_coords, uint32_t n, const uint32_t* d_live, n2_half* d_output,
                          const float* d_xyz_soa) {
	if (int rc = check_field(f, "n2_field_forward", n)) return rc;
	if (n == 0) return N2_OK;
	N2_REQUIRE(d_coords != nullptr && d_output != nullptr, "n2_field_forward: null buffer");
	N2_REQUIRE(reinterpret_cast<uintptr_t>(d_output) % 16 == 0, "n2_field_forward: d_output must be 16-byte aligned");
	hipStream_t s = n2_stream(stream);
	f->last_n = n;
	f->sel_n = 0;
	if (int rc = zero_padding(s, f->sdf_in, 3 + f->enc_w, f->sdf_in_w, n, f->pad_n.sdf_in)) return rc;
	f->slopes_saved = f->fused && fused_ok(f);
	f->frags_ready = f->slopes_saved;
	if (f->slopes_saved) {
		f->pad_n.rgb_in = 0;  // the fused kernel writes sample-major, over what the row layout keeps zero
		N2ProfScope prof(N2_PROF_FIELD_FORWARD, s);
		return n2_fused_field_forward(fused_nets(f), s, d_coords, n, reinterpret_cast<n2_half*>(f->sdf_in), f->xyz, f->dy_dx,
		                              reinterpret_cast<n2_half*>(f->dsdf_din), reinterpret_cast<n2_half*>(f->rgb_in), d_output, d_live, nullptr, nullptr, 0, 0,
		                              d_xyz_soa);
	}
	field_pack_sdf_input_kernel<<<fgrid(n), dim3(FB), 0, s>>>(d_coords, 7, 1, n, f->sdf_in, f->xyz);
	N2_LAUNCH_CHECK();
	if (int rc = n2_grid_forward(f->grid, stream, f->xyz, 1, n, n, reinterpret_cast<n2_half*>(f->sdf_in + (size_t)3 * n), f->dy_dx)) return rc;
	// SDF net forward (into rows 0..15 of the colour net's input) and d sdf / d input in one pass over the input
	if (int rc = zero_padding(s, f->rgb_in, RGB_IN_ROWS, f->rgb_in_w, n, f->pad_n.rgb_in)) return rc;
	if (int rc = n2_mlp_forward_and_input_gradient(f->sdf, stream, 0, reinterpret_cast<const n2_half*>(f->sdf_in), n,
	                                               reinterpret_cast<n2_half*>(f->rgb_in), N2_LAYOUT_SOA, reinterpret_cast<n2_half*>(f->dsdf_din))) return rc;
	field_normals_rgb_input_kernel<<<fgrid(n), dim3(FB), 0, s>>>(d_coords, n, f->enc_w, f->dsdf_din, f->dy_dx, f->rgb_in);
	N2_LAUNCH_CHECK();
	if (int rc = n2_mlp_forward(f->rgb, stream, reinterpret_cast<const n2_half*>(f->rgb_in), n, d_output, N2_LAYOUT_AOS, nullptr)) return rc;
	field_finish_output_kernel<<<fgrid(n), dim3(FB), 0, s>>>(d_coords, n, f->rgb_in, (hf)f->sdf_bias, f->params + f->off_var,
	                                                         reinterpret_cast<hf*>(d_output));
	N2_LAUNCH_CHECK();
	return N2_OK;
}

int n2_field_forward_listed(n2_field_t* f, n2_stream_t stream, const float* d_coords, uint32_t n, const uint32_t* d_list, const uint32_t* d_counts,
                            uint32_t round, uint32_t est_samples, n2_half* d_output) {
	if (int rc = check_field(f, "n2_field_forward", n)) return rc;
	if (n == 0) return N2_OK;
	N2_REQUIRE(d_coords != nullptr && d_output != nullptr && d_list != nullptr && d_counts != nullptr, "n2_field_forward: null buffer");
	N2_REQUIRE(reinterpret_cast<uintptr_t>(d_output) % 16 == 0, "n2_field_forward: d_output must be 16-byte aligned");
	N2_REQUIRE(f->fused && fused_ok(f), "n2_field_forward: a listed pass needs the fused kernels (n2_field_set_fused, no per-point level mask)");
	hipStream_t s = n2_stream(stream);
	f->last_n = n;
	f->sel_n = 0;
	if (int rc = zero_padding(s, f->sdf_in, 3 + f->enc_w, f->sdf_in_w, n, f->pad_n.sdf_in)) return rc;
	f->slopes_saved = true;
	if (round == 0) f->frags_ready = true;
	f->pad_n.rgb_in = 0;
	N2ProfScope prof(N2_PROF_FIELD_FORWARD, s);
	return n2_fused_field_forward(fused_nets(f), s, d_coords, n, reinterpret_cast<n2_half*>(f->sdf_in), f->xyz, f->dy_dx, reinterpret_cast<n2_half*>(f->dsdf_din),
	                              reinterpret_cast<n2_half*>(f->rgb_in), d_output, nullptr, d_list, d_counts, round, est_samples);
}

N2_API int n2_field_backward(n2_field_t* f, n2_stream_t stream, const float* d_coords, uint32_t n,
                             const n2_half* d_dL_doutput, uint32_t ek_batch_size, n2_grad_mode mode) {
	N2SlabReduce sums = {};
	if (int rc = n2_field_backward_deferred(f, stream, d_coords, n, d_dL_doutput, ek_batch_size, mode, &sums)) return rc;
	return n2_slab_reduce_launch(stream, sums);
}

static int field_backward_passes(n2_field_t* f, n2_stream_t stream, const float* d_coords, uint32_t n, const n2_half* d_dL_doutput, uint32_t ek_batch_size,
                                 n2_grad_mode mode, N2SlabReduce* sums);

int n2_field_backward_deferred(n2_field_t* f, n2_stream_t stream, const float* d_coords, uint32_t n, const n2_half* d_dL_doutput, uint32_t ek_batch_size,
                               n2_grad_mode mode, N2SlabReduce* sums) {
	if (f != nullptr && f->frags_ready) {
		// the weight-gradient kernels' fragments as the forward's gather launch built them, once for all workgroups
		const n2_half* image = reinterpret_cast<const n2_half*>(f->frag_image);
		n2_mlp_borrow_fragment_image(f->rgb, image + N2_FUSED_FRAG_FORWARD / 2);
		if (f->sdf_in_w == 48) n2_mlp_borrow_fragment_image(f->sdf, image + (N2_FUSED_FRAG_FORWARD + N2_FUSED_FRAG_RGB) / 2);
	}
	const int rc = field_backward_passes(f, stream, d_coords, n, d_dL_doutput, ek_batch_size, mode, sums);
	if (f != nullptr) {
		n2_mlp_borrow_fragment_image(f->rgb, nullptr);
		n2_mlp_borrow_fragment_image(f->sdf, nullptr);
	}
	if (rc != N2_OK && f != nullptr) {
		// a pass that ran before the failure left partial sums pending in its network: nobody will reduce them
		n2_mlp_drop_pending(f->rgb);
		n2_mlp_drop_pending(f->sdf);
		*sums = N2SlabReduce{};
	}
	return rc;
}

static int field_backward_passes(n2_field_t* f, n2_stream_t stream, const float* d_coords, uint32_t n, const n2_half* d_dL_doutput, uint32_t ek_batch_size,
                                 n2_grad_mode mode, N2SlabReduce* sums) {
	*sums = N2SlabReduce{};
	if (int rc = check_field(f, "n2_field_backward", n)) return rc;
	N2_REQUIRE(n <= f->max_batch_bwd, "n2_field_backward: batch %u exceeds the workspace's backward capacity %u", n, f->max_batch_bwd);
	N2_REQUIRE(mode == N2_GRAD_OVERWRITE || mode == N2_GRAD_ACCUMULATE, "n2_field_backward: mode must be OVERWRITE or ACCUMULATE");
	N2_REQUIRE(f->grads != nullptr, "n2_field_backward: no gradient buffer (n2_field_set_params)");
	N2_REQUIRE(ek_batch_size > 0, "n2_field_backward: ek_batch_size must be positive");
	if (n == 0) return N2_OK;
	N2_REQUIRE(d_coords != nullptr && d_dL_doutput != nullptr, "n2_field_backward: null buffer");
	N2_REQUIRE(reinterpret_cast<uintptr_t>(d_dL_doutput) % 16 == 0, "n2_field_backward: d_dL_doutput must be 16-byte aligned");
	hipStream_t s = n2_stream(stream);
	const hf* dL = reinterpret_cast<const hf*>(d_dL_doutput);
	// the saved activations: those of the last forward, or the samples n2_field_select picked from them
	const bool sel = f->sel_n != 0;
	N2_REQUIRE(n == (sel ? f->sel_n : f->last_n), "n2_field_backward: batch %u, but the last %s was over %u samples", n,
	           sel ? "n2_field_select" : "n2_field_forward", sel ? f->sel_n : f->last_n);
	// with a selection, sample i of the batch is column index[i] of the rows the forward saved over its n_src samples
	const uint32_t* index = sel ? f->sel_use : nullptr;
	const uint32_t n_src = f->last_n;
	if (int rc = zero_padding(s, f->d_density_in, 3 + f->enc_w, f->sdf_in_w, n, f->pad_n.d_density_in)) return rc;
	LevelScales scales{};
	for (uint32_t l = 0; l < 16 && 2 * l < f->enc_w; ++l) scales.s[l] = n2_grid_table(f->grid)->scale[l];
	uint32_t var_parts = fgrid(n).x;
	if (f->slopes_saved) {
		// colour net (only rows 0..2 of dL_doutput belong to it); dL/dnormal, the second-order inputs, the direct gradient of
		// the SDF output and the variance gradient's partial sums ride in the same launch
		N2FieldPrepTail tail{};
		tail.ek_batch = (float)ek_batch_size;
		tail.slopes = f->dy_dx;
		tail.n_src = f->last_n;
		tail.enc_w = f->enc_w;
		for (int l = 0; l < 16; ++l) tail.scale[l] = scales.s[l];
		tail.v = f->v;
		tail.d_density_in = f->d_density_in;
		tail.var_part = f->var_part;
		var_parts = n2_mlp_wgrad_blocks(n);
		if (int rc = n2_mlp_backward_rows_indexed(f->rgb, stream, reinterpret_cast<const n2_half*>(f->rgb_in), n_src, index, n, d_dL_doutput, N2_LAYOUT_AOS, 3,
		                                          reinterpret_cast<n2_half*>(f->d_rgb_in), mode, true, &tail)) return rc;
	} else {
		// colour net: only rows 0..2 of dL_doutput belong to it
		if (int rc = n2_mlp_backward_rows_indexed(f->rgb, stream, reinterpret_cast<const n2_half*>(f->rgb_in), n_src, index, n, d_dL_doutput, N2_LAYOUT_AOS, 3,
		                                          reinterpret_cast<n2_half*>(f->d_rgb_in), mode, true)) return rc;
		// dL/dnormal, the second-order inputs, the direct gradient of the SDF output and the variance gradient
		field_backward_prep_kernel<<<fgrid(n), dim3(FB), 0, s>>>(n, f->enc_w, f->d_rgb_in, dL, (float)ek_batch_size, f->dy_dx, f->v, f->d_density_in,
		                                                         f->var_part, index, f->last_n);
		N2_LAUNCH_CHECK();
	}
	// SDF net: its output gradient is rows 0..15 of the colour net's input gradient; the second-order pass through the
	// net (the reference's backward_backward_input with Accumulate) rides along
	if (int rc = n2_mlp_backward_and_second_order_indexed(f->sdf, stream, reinterpret_cast<const n2_half*>(f->sdf_in), n_src, index, n,
	                                                      reinterpret_cast<const n2_half*>(f->d_rgb_in), f->slopes_saved ? N2_LAYOUT_AOS : N2_LAYOUT_SOA,
	                                                      reinterpret_cast<n2_half*>(f->d_sdf_in),
	                                                      reinterpret_cast<const n2_half*>(f->d_density_in), nullptr, mode, true)) return rc;
	// grid: first-order and second-order gradients in one scatter pass (the reference's backward with
	// Overwrite followed by backward_backward_input with Accumulate)
	if (int rc = n2_grid_backward_fused_indexed(f->grid, stream, f->xyz, n_src, index, n, reinterpret_cast<const n2_half*>(f->d_sdf_in + (size_t)3 * n), f->v,
	                                            reinterpret_cast<const n2_half*>(f->dsdf_din + (size_t)3 * n_src), mode)) return rc;
	// the three weight-gradient passes (colour net, SDF net first and second order) left their per-workgroup partial sums
	// pending: one plan sums them, and with them the partial sums of the variance gradient (the caller runs it: as a launch,
	// or inside the optimiser's kernel)
	return n2_mlp_reduce_deferred_plan(f->rgb, f->sdf, f->var_part, var_parts, reinterpret_cast<n2_half*>(f->grads + f->off_var),
	                                   mode == N2_GRAD_ACCUMULATE ? 1 : 0, sums);
}

N2_API int n2_field_select(n2_field_t* f, n2_stream_t stream, const uint32_t* d_source_index, uint32_t n_source, uint32_t n) {
	if (int rc = check_field(f, "n2_field_select", n)) return rc;
	N2_REQUIRE(n <= f->max_batch_bwd, "n2_field_select: batch %u exceeds the workspace's backward capacity %u", n, f->max_batch_bwd);
	N2_REQUIRE(n_source == f->last_n && n_source > 0, "n2_field_select: n_source %u, but the last n2_field_forward was over %u samples", n_source,
	           f->last_n);
	N2_REQUIRE(n > 0 && d_source_index != nullptr, "n2_field_select: empty selection");
	field_select_kernel<<<fgrid(n), dim3(FB), 0, n2_stream(stream)>>>(n, n_source, d_source_index, f->sel_index);
	N2_LAUNCH_CHECK();
	f->sel_n = n;
	f->sel_use = f->sel_index;
	return N2_OK;
}

int n2_field_select_borrow(n2_field_t* f, const uint32_t* d_source_index, uint32_t n_source, uint32_t n) {
	if (int rc = check_field(f, "n2_field_select", n)) return rc;
	N2_REQUIRE(n <= f->max_batch_bwd, "n2_field_select: batch %u exceeds the workspace's backward capacity %u", n, f->max_batch_bwd);
	N2_REQUIRE(n_source == f->last_n && n_source > 0, "n2_field_select: n_source %u, but the last n2_field_forward was over %u samples", n_source,
	           f->last_n);
	N2_REQUIRE(n > 0 && d_source_index != nullptr, "n2_field_select: empty selection");
	f->sel_n = n;
	f->sel_use = d_source_index;  // every kernel that reads through it clamps the entries into the forward's batch
	return N2_OK;
}

// ----------------------------------------------------------------------------
// The SDF network on its own with the eikonal term (no colour branch): the glue between the encoding's and the
// network's kernels, i.e. what NerfNetwork does with small element-wise kernels at nerf_network.h:193-199 (input),
// :230-238 (normal = encoding backward of d sdf / d encoding, plus the direct coordinate rows) and :546-557 (input of
// the network's second-order pass), with the loss  mean |sdf| + w_ek mean (|normal| - 1)^2  in between.
// ----------------------------------------------------------------------------
__global__ void __launch_bounds__(FB) sdf_pack_input_kernel(const float* __restrict__ xyz, uint32_t ps, uint32_t ds, uint32_t N, uint32_t first_pad,
                                                            uint32_t in_w, hf* __restrict__ input) {
	const uint32_t i = blockIdx.x * FB + threadIdx.x;
	if (i >= N) return;
	const float* q = xyz + (size_t)i * ps;
#pragma unroll
	for (int d = 0; d < 3; ++d) input[(size_t)d * N + i] = (hf)q[(size_t)d * ds] - (hf)0.5f;
	for (uint32_t r = first_pad; r < in_w; ++r) input[(size_t)r * N + i] = (hf)0;
}

__global__ void __launch_bounds__(FB) sdf_eikonal_loss_kernel(uint32_t N, uint32_t first_pad, uint32_t in_w, const hf* __restrict__ sdf_out,
                                                              const hf* __restrict__ g, const float* __restrict__ normal_enc, float* __restrict__ normal, float ek_weight, float scale,
                                                              hf* __restrict__ dL_dy, float* __restrict__ v, hf* __restrict__ v_in,
                                                              float* __restrict__ parts, const float* __restrict__ dy_dx) {
	__shared__ float part[FB / 64];
	const uint32_t i = blockIdx.x * FB + threadIdx.x;
	float term = 0.f;
	if (i < N) {
		const float sdf = (float)sdf_out[i];
		float nrm[3], len2 = 0.f;
#pragma unroll
		for (int d = 0; d < 3; ++d) {
			nrm[d] = normal_enc[(size_t)d * N + i] + (float)g[(size_t)d * N + i];  // add_positions_view: the direct coordinate rows
			normal[(size_t)d * N + i] = nrm[d];
			len2 = fmaf(nrm[d], nrm[d], len2);
		}
		const float len = fmaxf(sqrtf(len2), 1e-12f);
		term = fabsf(sdf) + ek_weight * (len - 1.f) * (len - 1.f);
		dL_dy[i] = (hf)((sdf > 0.f ? 1.f : sdf < 0.f ? -1.f : 0.f) * scale);
		for (uint32_t r = 1; r < 16; ++r) dL_dy[(size_t)r * N + i] = (hf)0;
		const float k = 2.f * ek_weight * (len - 1.f) / len * scale;
		float x[3];
#pragma unroll
		for (int d = 0; d < 3; ++d) {
			x[d] = nrm[d] * k;  // d loss / d normal
			v[(size_t)d * N + i] = x[d];
			v_in[(size_t)d * N + i] = (hf)x[d];
		}
		if (dy_dx) {
			// the encoding's dL_ddLdoutput = J v from the Jacobian the forward saved ([row][N][3]), eight rows' loads in flight
			const uint32_t enc_w = first_pad - 3;
			for (uint32_t r0 = 0; r0 < enc_w; r0 += 8) {
				float j[8][3];
#pragma unroll
				for (uint32_t u = 0; u < 8; ++u) {
					const float* q = dy_dx + ((size_t)min(r0 + u, enc_w - 1) * N + i) * 3;
					j[u][0] = q[0]; j[u][1] = q[1]; j[u][2] = q[2];
				}
#pragma unroll
				for (uint32_t u = 0; u < 8; ++u)
					if (r0 + u < enc_w) v_in[(size_t)(3 + r0 + u) * N + i] = (hf)fmaf(j[u][0], x[0], fmaf(j[u][1], x[1], j[u][2] * x[2]));
			}
		}
		for (uint32_t r = first_pad; r < in_w; ++r) v_in[(size_t)r * N + i] = (hf)0;
	}
#pragma unroll
	for (int o = 32; o > 0; o >>= 1) term += __shfl_xor(term, o);
	if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = term;
	__syncthreads();
	if (threadIdx.x == 0) parts[blockIdx.x] = (part[0] + part[1]) + (part[2] + part[3]);
}

// loss = sum of the workgroups' partial sums / N, in a fixed order
__global__ void __launch_bounds__(256) sdf_loss_sum_kernel(const float* __restrict__ parts, uint32_t n_parts, float inv_n, float* __restrict__ loss) {
	__shared__ float part[4];
	float s = 0.f;
	for (uint32_t i = threadIdx.x; i < n_parts; i += 256) s += parts[i];
#pragma unroll
	for (int o = 32; o > 0; o >>= 1) s += __shfl_xor(s, o);
	if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = s;
	__syncthreads();
	if (threadIdx.x == 0) loss[0] = ((part[0] + part[1]) + (part[2] + part[3])) * inv_n;
}

N2_API int n2_sdf_pack_input(n2_stream_t stream, const float* d_xyz, uint32_t point_stride, uint32_t dim_stride, uint32_t n, uint32_t encoding_width,
                             uint32_t input_width, n2_half* d_input) {
	if (n == 0) return N2_OK;
	N2_REQUIRE(d_xyz != nullptr && d_input != nullptr, "n2_sdf_pack_input: null buffer");
	N2_REQUIRE(point_stride >= 1 && dim_stride >= 1, "n2_sdf_pack_input: strides must be >= 1");
	N2_REQUIRE(input_width >= 3 + encoding_width && input_width <= 64, "n2_sdf_pack_input: input width %u does not hold 3 + %u rows", input_width, encoding_width);
	sdf_pack_input_kernel<<<fgrid(n), dim3(FB), 0, n2_stream(stream)>>>(d_xyz, point_stride, dim_stride, n, 3 + encoding_width, input_width,
	                                                                   reinterpret_cast<hf*>(d_input));
	N2_LAUNCH_CHECK();
	return N2_OK;
}

N2_API uint64_t n2_sdf_eikonal_workspace_bytes(uint32_t n) { return 4ull * ((n + FB - 1) / FB + 1); }

N2_API int n2_sdf_eikonal_loss(n2_stream_t stream, uint32_t n, uint32_t encoding_width, uint32_t input_width, const n2_half* d_sdf_output,
                               const n2_half* d_dsdf_dinput, const float* d_normal_encoding, float* d_normal, float ek_weight, float loss_scale, n2_half* d_dL_doutput,
                               float* d_dL_dnormal, n2_half* d_second_order_input, float* d_loss, void* d_workspace, uint64_t workspace_bytes,
                               const float* d_dy_dx) {
	N2_REQUIRE(n > 0, "n2_sdf_eikonal_loss: empty batch");
	N2_REQUIRE(d_sdf_output && d_dsdf_dinput && d_normal_encoding && d_normal && d_dL_doutput && d_dL_dnormal && d_second_order_input && d_loss && d_workspace,
	           "n2_sdf_eikonal_loss: null buffer");
	N2_REQUIRE(input_width >= 3 + encoding_width && input_width <= 64, "n2_sdf_eikonal_loss: input width %u does not hold 3 + %u rows", input_width, encoding_width);
	N2_REQUIRE(workspace_bytes >= n2_sdf_eikonal_workspace_bytes(n), "n2_sdf_eikonal_loss: workspace of %llu bytes, %llu needed",
	           (unsigned long long)workspace_bytes, (unsigned long long)n2_sdf_eikonal_workspace_bytes(n));
	hipStream_t s = n2_stream(stream);
	float* parts = reinterpret_cast<float*>(d_workspace);
	sdf_eikonal_loss_kernel<<<fgrid(n), dim3(FB), 0, s>>>(n, 3 + encoding_width, input_width, reinterpret_cast<const hf*>(d_sdf_output),
	                                                      reinterpret_cast<const hf*>(d_dsdf_dinput), d_normal_encoding, d_normal, ek_weight, loss_scale / (float)n,
	                                                      reinterpret_cast<hf*>(d_dL_doutput), d_dL_dnormal, reinterpret_cast<hf*>(d_second_order_input), parts,
	                                                      d_dy_dx);
	N2_LAUNCH_CHECK();
	sdf_loss_sum_kernel<<<dim3(1), dim3(256), 0, s>>>(parts, fgrid(n).x, 1.f / (float)n, d_loss);
	N2_LAUNCH_CHECK();
	return N2_OK;
}

// The inference paths for points in no particular order gather the features into the rows of the SDF net's input, at the
// pitch of THEIR batch: whatever the training forward left there is gone, and with another batch size the rows land on what
// the training layout keeps as zero padding (rows 3 + enc_w .. sdf_in_w, which the weight-gradient kernels read against
// non-zero weight columns).  So the padding counts as not cleared, and a backward pass has to follow a new forward.
static void inference_takes_sdf_in(n2_field_t* f) {
	f->pad_n.sdf_in = 0;
	f->last_n = 0;
	f->sel_n = 0;
}

static int field_sdf_impl(n2_field_t* f, const char* fn, n2_stream_t stream, const float* d_xyz, uint32_t ps, uint32_t ds, uint32_t n,
                          n2_half* d_output, bool density) {
	if (int rc = check_field(f, fn, n)) return rc;
	if (n == 0) return N2_OK;
	N2_REQUIRE(d_xyz != nullptr && d_output != nullptr, "%s: null buffer", fn);
	N2_REQUIRE(ps >= 1 && ds >= 1, "%s: strides must be >= 1", fn);
	N2_REQUIRE(reinterpret_cast<uintptr_t>(d_output) % 16 == 0, "%s: d_output must be 16-byte aligned", fn);
	hipStream_t s = n2_stream(stream);
	if (f->fused && fused_ok(f)) {
		N2ProfScope prof(N2_PROF_FIELD_FORWARD, s);
		const bool scratch = !n2_grid_lattice_order(f->grid);
		if (scratch) inference_takes_sdf_in(f);
		return n2_fused_field_sdf(fused_nets(f), s, d_xyz, ps, ds, n, d_output, nullptr, density,
		                          scratch ? reinterpret_cast<n2_half*>(f->sdf_in) : nullptr);
	}
	if (int rc = zero_padding(s, f->sdf_in, 3 + f->enc_w, f->sdf_in_w, n, f->pad_n.sdf_in)) return rc;
	f->last_n = 0;  // the rows below are overwritten: a backward pass needs a new n2_field_forward
	f->sel_n = 0;
	field_pack_sdf_input_kernel<<<fgrid(n), dim3(FB), 0, s>>>(d_xyz, ps, ds, n, f->sdf_in, f->xyz);
	N2_LAUNCH_CHECK();
	if (int rc = n2_grid_forward(f->grid, stream, f->xyz, 1, n, n, reinterpret_cast<n2_half*>(f->sdf_in + (size_t)3 * n), nullptr)) return rc;
	if (int rc = n2_mlp_forward(f->sdf, stream, reinterpret_cast<const n2_half*>(f->sdf_in), n, d_output, N2_LAYOUT_SOA, nullptr)) return rc;
	field_add_bias_kernel<<<fgrid(n), dim3(FB), 0, s>>>(n, (hf)f->sdf_bias, reinterpret_cast<hf*>(d_output));
	N2_LAUNCH_CHECK();
	if (density) {
		field_sdf_to_density_kernel<<<fgrid(n), dim3(FB), 0, s>>>(n, f->params + f->off_var, reinterpret_cast<hf*>(d_output));
		N2_LAUNCH_CHECK();
	}
	return N2_OK;
}

__global__ void __launch_bounds__(FB) field_widen_row_kernel(uint32_t n, const hf* __restrict__ in, float* __restrict__ out) {
	const uint32_t i = blockIdx.x * FB + threadIdx.x;
	if (i < n) out[i] = (float)in[i];
}

// Row 0 of n2_field_sdf (or n2_field_density) as fp32 (the fp16 value widened; what get_density_on_grid keeps,
// src/testbed_nerf.cu:4082-4133, and what the occupancy update splats):
// the fused kernel writes it directly and the other 15 rows not at all; d_scratch16 ([16][n] fp16) serves the unfused path.
int n2_field_sdf_row0(n2_field_t* f, n2_stream_t stream, const float* d_xyz, uint32_t ps, uint32_t ds, uint32_t n, uint32_t n_keep, float* d_row0,
                      n2_half* d_scratch16, bool density) {
	if (int rc = check_field(f, "n2_field_sdf", n)) return rc;
	if (n == 0) return N2_OK;
	N2_REQUIRE(d_xyz != nullptr && d_row0 != nullptr, "n2_field_sdf: null buffer");
	N2_REQUIRE(ps >= 1 && ds >= 1, "n2_field_sdf: strides must be >= 1");
	hipStream_t s = n2_stream(stream);
	if (f->fused && fused_ok(f)) {
		N2ProfScope prof(N2_PROF_FIELD_FORWARD, s);
		const bool scratch = !n2_grid_lattice_order(f->grid);
		if (scratch) inference_takes_sdf_in(f);
		return n2_fused_field_sdf(fused_nets(f), s, d_xyz, ps, ds, n, nullptr, d_row0, density,
		                          scratch ? reinterpret_cast<n2_half*>(f->sdf_in) : nullptr, n_keep);
	}
	if (int rc = field_sdf_impl(f, "n2_field_sdf", stream, d_xyz, ps, ds, n, d_scratch16, density)) return rc;
	const uint32_t keep = n_keep < n ? n_keep : n;
	field_widen_row_kernel<<<fgrid(keep), dim3(FB), 0, s>>>(keep, reinterpret_cast<const hf*>(d_scratch16), d_row0);
	N2_LAUNCH_CHECK();
	return N2_OK;
}

bool n2_field_sdf_row0_lattice(n2_field_t* f, n2_stream_t stream, const N2Lattice& lattice, uint32_t n, uint32_t n_keep, float* d_row0, int* rc) {
	*rc = check_field(f, "n2_field_sdf", n);
	if (*rc != N2_OK) return true;
	if (!(f->fused && fused_ok(f) && n2_grid_lattice_order(f->grid))) return false;
	if (n == 0) return true;
	if (d_row0 == nullptr) { n2_set_error("n2_field_sdf: null buffer"); *rc = N2_ERR_INVALID_ARGUMENT; return true; }
	hipStream_t s = n2_stream(stream);
	N2ProfScope prof(N2_PROF_FIELD_FORWARD, s);
	*rc = n2_fused_field_sdf(fused_nets(f), s, nullptr, 0, 0, n, nullptr, d_row0, false, nullptr, n_keep, &lattice);
	return true;
}

N2_API int n2_field_sdf(n2_field_t* f, n2_stream_t stream, const float* d_xyz, uint32_t point_stride, uint32_t dim_stride, uint32_t n,
                        n2_half* d_output) {
	return field_sdf_impl(f, "n2_field_sdf", stream, d_xyz, point_stride, dim_stride, n, d_output, false);
}

N2_API int n2_field_density(n2_field_t* f, n2_stream_t stream, const float* d_xyz, uint32_t point_stride, uint32_t dim_stride, uint32_t n,
                            n2_half* d_output) {
	return field_sdf_impl(f, "n2_field_density", stream, d_xyz, point_stride, dim_stride, n, d_output, true);
}
