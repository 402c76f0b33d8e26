// Occupancy-grid update: the running 128^3 (x cascades) density estimate, its
// decayed-maximum merge with fresh field densities, the mean threshold, the
// 1-bit-per-cell morton bitfield the ray marcher reads and its 8 mip levels
// (Testbed::update_density_grid_nerf and update_density_grid_mean_and_bitfield,
// src/testbed_nerf.cu:3286-3391, kernels at :630-786).
//
// Sample positions and cell indices are part of the bit-exact contract with
// the CPU oracle, so floating-point contraction is off for this file.
#include "n2_common.h"

#include <new>

#pragma clang fp contract(off)

typedef _Float16 hf;

constexpr uint32_t OCC_GRIDSIZE = 128;
constexpr uint32_t OCC_CELLS = OCC_GRIDSIZE * OCC_GRIDSIZE * OCC_GRIDSIZE;
constexpr uint32_t OCC_LEVELS = 8;                          // NERF_CASCADES()
constexpr uint32_t OCC_LEVEL_BYTES = OCC_CELLS / 8;
constexpr float OCC_MIN_OPTICAL_THICKNESS = 0.1f;           // NERF_MIN_OPTICAL_THICKNESS(), SDF_GRID 0
constexpr uint32_t OCC_BLOCK = 256;
constexpr uint32_t OCC_MEAN_BLOCKS = OCC_CELLS / (OCC_BLOCK * 32);  // 256 partial sums of 8192 cells each

struct n2_occupancy {
	uint32_t n_cascades;
	uint64_t rng_state, rng_inc;
	uint32_t ema_step;
	unsigned char* ws;
	uint32_t max_samples, chunk;
	float* grid;         // [n_cascades][128^3]
	float* tmp;          // same
	float* positions;    // [max_samples + 8][3]
	uint32_t* indices;   // [max_samples + 8]
	hf* mlp_out;         // [16][chunk] fp16 (the field's full output, unfused path only), then [chunk] fp32: the density row
	uint8_t* bitfield;   // [8][128^3 / 8]
	float* partial;      // [OCC_MEAN_BLOCKS]
	float* mean;         // [1]
	uint32_t last_n, last_n_uniform;
};

// ---------------------------------------------------------------------------
// PCG32 (XSH-RR 64/32) as tiny-cuda-nn ships it: the reference hands the generator to the kernel by value,
// every thread skips 4*i draws ahead and takes four floats.
// ---------------------------------------------------------------------------
constexpr uint64_t PCG32_MULT = 0x5851f42d4c957f2dULL;

struct Pcg32 {
	uint64_t state, inc;
	__host__ __device__ uint32_t next_uint() {
		const uint64_t old = state;
		state = old * PCG32_MULT + inc;
		const uint32_t xorshifted = (uint32_t)(((old >> 18u) ^ old) >> 27u);
		const uint32_t rot = (uint32_t)(old >> 59u);
		return (xorshifted >> rot) | (xorshifted << ((~rot + 1u) & 31));
	}
	__device__ float next_float() { return __uint_as_float((next_uint() >> 9) | 0x3f800000u) - 1.0f; }
	__host__ __device__ void advance(uint64_t delta) {
		uint64_t cur_mult = PCG32_MULT, cur_plus = inc, acc_mult = 1u, acc_plus = 0u;
		while (delta > 0) {
			if (delta & 1) {
				acc_mult *= cur_mult;
				acc_plus = acc_plus * cur_mult + cur_plus;
			}
			cur_plus = (cur_mult + 1) * cur_plus;
			cur_mult *= cur_mult;
			delta /= 2;
		}
		state = acc_mult * state + acc_plus;
	}
};

__device__ __forceinline__ uint32_t occ_expand_bits(uint32_t v) {
	v = (v * 0x00010001u) & 0xFF0000FFu;
	v = (v * 0x00000101u) & 0x0F00F00Fu;
	v = (v * 0x00000011u) & 0xC30C30C3u;
	v = (v * 0x00000005u) & 0x49249249u;
	return v;
}
__device__ __forceinline__ uint32_t occ_morton3d(uint32_t x, uint32_t y, uint32_t z) {
	return occ_expand_bits(x) | (occ_expand_bits(y) << 1) | (occ_expand_bits(z) << 2);
}
__device__ __forceinline__ uint32_t occ_morton3d_invert(uint32_t x) {
	x = x & 0x49249249u;
	x = (x | (x >> 2)) & 0xc30c30c3u;
	x = (x | (x >> 4)) & 0x0f00f00fu;
	x = (x | (x >> 8)) & 0xff0000ffu;
	x = (x | (x >> 16)) & 0x0000ffffu;
	return x;
}

// generate_grid_samples_nerf_nonuniform (:630-660), unit aabb.  Slots [n, n_pad) are filled with the cube centre
// so that the field can run on a multiple of 8 points.
//
// Which sample a slot holds.  The first candidate cell of sample i is ((i + step n) P + R) mod 128^3 with P = 56924617: a
// pseudo-random walk over the cells, so that consecutive samples would splat their maxima into unrelated memory lines
// (one atomic request per sample).  The samples are independent of each other, so the order they are generated and
// evaluated in is free: when n is a power of two, slot t holds sample i(t) = t P^-1 mod n (P^-1 mod 2^32, masked), whose
// candidate cell is t + const mod n: consecutive slots splat into consecutive cells of (at most 128^3 / n) runs, and a
// wave's 64 atomics fall into a few lines.  Other n: slot t holds sample t.
constexpr uint32_t OCC_WALK = 56924617u;
constexpr uint32_t occ_inverse_mod_2_32(uint32_t a) {  // a odd; Newton's iteration doubles the number of correct low bits
	uint32_t x = a;                                     // a * a = 1 mod 8
	for (int k = 0; k < 5; ++k) x *= 2u - a * x;
	return x;
}
constexpr uint32_t OCC_WALK_INV = occ_inverse_mod_2_32(OCC_WALK);
static_assert(OCC_WALK * OCC_WALK_INV == 1u, "inverse of the walk's multiplier");
static inline uint32_t occ_order_mul(uint32_t n) { return (n >= 2 && (n & (n - 1)) == 0) ? OCC_WALK_INV : 0u; }

__global__ void __launch_bounds__(OCC_BLOCK) occ_generate_kernel(uint32_t n, uint32_t n_pad, Pcg32 rng, uint32_t step, const float* __restrict__ grid,
                                                                 uint32_t n_cascades, float thresh, uint32_t order_mul,
                                                                 float* __restrict__ positions, uint32_t* __restrict__ indices) {
	const uint32_t slot = blockIdx.x * OCC_BLOCK + threadIdx.x;
	if (slot >= n_pad) return;
	if (slot >= n) {
		positions[(size_t)slot * 3] = 0.5f; positions[(size_t)slot * 3 + 1] = 0.5f; positions[(size_t)slot * 3 + 2] = 0.5f;
		return;
	}
	const uint32_t i = order_mul ? (slot * order_mul) & (n - 1u) : slot;
	rng.advance((uint64_t)i * 4);
	const uint32_t level = (uint32_t)(rng.next_float() * n_cascades) % n_cascades;
	uint32_t idx = 0;
	for (uint32_t j = 0; j < 10; ++j) {
		idx = ((i + step * n) * OCC_WALK + j * 19349663u + 96925573u) % OCC_CELLS;
		idx += level * OCC_CELLS;
		if (grid[idx] > thresh) break;
	}
	const uint32_t pos_idx = idx % OCC_CELLS;
	const float scale = scalbnf(1.0f, (int)level);
#pragma unroll
	for (int d = 0; d < 3; ++d) {
		const float c = (float)occ_morton3d_invert(pos_idx >> d);
		const float u = rng.next_float();
		positions[(size_t)slot * 3 + d] = ((c + u) / (float)OCC_GRIDSIZE - 0.5f) * scale + 0.5f;
	}
	indices[slot] = idx;
}

// splat_grid_samples_nerf_max_nearest_neighbor (:662-680): positive floats order like their bit patterns
__global__ void __launch_bounds__(OCC_BLOCK) occ_splat_kernel(uint32_t n, const uint32_t* __restrict__ indices, const float* __restrict__ density,
                                                              float* __restrict__ tmp) {
	const uint32_t i = blockIdx.x * OCC_BLOCK + threadIdx.x;
	if (i >= n) return;
	atomicMax(reinterpret_cast<uint32_t*>(tmp) + indices[i], __float_as_uint(density[i]));
}

// ema_grid_samples_nerf (:698-727), fused with the partial sums of max(v, 0) over the first cascade (:3383).
// A block covers 8192 consecutive cells; its partial sum is built in a fixed order, so the mean is reproducible.
// MERGE false: only the partial sums (the grid was written from outside).
template <bool MERGE>
__global__ void __launch_bounds__(OCC_BLOCK) occ_ema_kernel(uint32_t n_elements, float decay, float* __restrict__ grid, const float* __restrict__ tmp,
                                                            float* __restrict__ partial) {
	__shared__ float red[OCC_BLOCK / 64];
	const uint32_t base = blockIdx.x * (OCC_BLOCK * 32);
	float sum = 0.f;
	for (uint32_t k = 0; k < 32; ++k) {
		const uint32_t i = base + k * OCC_BLOCK + threadIdx.x;
		if (i < n_elements) {
			float val = grid[i];
			if (MERGE) {
				val = (val < 0.f) ? val : fmaxf(val * decay, tmp[i]);
				grid[i] = val;
			}
			sum += fmaxf(val, 0.f);
		}
	}
#pragma unroll
	for (int o = 32; o > 0; o >>= 1) sum += __shfl_down(sum, o);
	if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = sum;
	__syncthreads();
	if (threadIdx.x == 0 && blockIdx.x < OCC_MEAN_BLOCKS) partial[blockIdx.x] = (red[0] + red[1]) + (red[2] + red[3]);
}

__global__ void __launch_bounds__(OCC_MEAN_BLOCKS) occ_mean_kernel(const float* __restrict__ partial, float* __restrict__ mean) {
	__shared__ float red[OCC_MEAN_BLOCKS / 64];
	float sum = partial[threadIdx.x];
#pragma unroll
	for (int o = 32; o > 0; o >>= 1) sum += __shfl_down(sum, o);
	if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = sum;
	__syncthreads();
	if (threadIdx.x == 0) mean[0] = ((red[0] + red[1]) + (red[2] + red[3])) / (float)OCC_CELLS;
}

// grid_to_bitfield (:738-764): one byte = 8 consecutive (morton-ordered) cells; levels beyond the scene's cascades are cleared
__global__ void __launch_bounds__(OCC_BLOCK) occ_bitfield_kernel(uint32_t n_bytes, uint32_t n_nonzero_bytes, const float* __restrict__ grid,
                                                                 uint8_t* __restrict__ bitfield, const float* __restrict__ mean) {
	const uint32_t i = blockIdx.x * OCC_BLOCK + threadIdx.x;
	if (i >= n_bytes) return;
	if (i >= n_nonzero_bytes) {
		bitfield[i] = 0;
		return;
	}
	const float thresh = fminf(OCC_MIN_OPTICAL_THICKNESS, mean[0]);
	const float4 a = reinterpret_cast<const float4*>(grid)[(size_t)i * 2], b = reinterpret_cast<const float4*>(grid)[(size_t)i * 2 + 1];
	uint32_t bits = 0;
	bits |= a.x > thresh ? 1u : 0u; bits |= a.y > thresh ? 2u : 0u; bits |= a.z > thresh ? 4u : 0u; bits |= a.w > thresh ? 8u : 0u;
	bits |= b.x > thresh ? 16u : 0u; bits |= b.y > thresh ? 32u : 0u; bits |= b.z > thresh ? 64u : 0u; bits |= b.w > thresh ? 128u : 0u;
	bitfield[i] = (uint8_t)bits;
}

// bitfield_max_pool (:766-786): a byte of the next level collects "any bit set" of 8 bytes (8 blocks of 2^3 cells) of
// the previous one and lands in the central half of the next level's grid.  Distinct i write distinct bytes.
__global__ void __launch_bounds__(OCC_BLOCK) occ_pool_kernel(const uint8_t* __restrict__ prev, uint8_t* __restrict__ next) {
	const uint32_t i = blockIdx.x * OCC_BLOCK + threadIdx.x;
	if (i >= OCC_CELLS / 64) return;
	const uint2 p = reinterpret_cast<const uint2*>(prev)[i];
	uint32_t bits = 0;
#pragma unroll
	for (uint32_t j = 0; j < 4; ++j) {
		bits |= ((p.x >> (8 * j)) & 0xFFu) ? (1u << j) : 0u;
		bits |= ((p.y >> (8 * j)) & 0xFFu) ? (16u << j) : 0u;
	}
	const uint32_t x = occ_morton3d_invert(i >> 0) + OCC_GRIDSIZE / 8;
	const uint32_t y = occ_morton3d_invert(i >> 1) + OCC_GRIDSIZE / 8;
	const uint32_t z = occ_morton3d_invert(i >> 2) + OCC_GRIDSIZE / 8;
	next[occ_morton3d(x, y, z)] |= (uint8_t)bits;
}

// ---------------------------------------------------------------------------
// host side
// ---------------------------------------------------------------------------
static inline uint64_t o256(uint64_t x) { return (x + 255) / 256 * 256; }

struct OccCarve {
	uint64_t grid, tmp, positions, indices, mlp_out, bitfield, partial, mean, total;
};
static OccCarve occ_carve(uint32_t n_cascades, uint32_t max_samples, uint32_t chunk) {
	OccCarve c{};
	uint64_t o = 0;
	auto take = [&](uint64_t bytes) { const uint64_t at = o; o = o256(o + bytes); return at; };
	c.grid = take(4ull * n_cascades * OCC_CELLS);
	c.tmp = take(4ull * n_cascades * OCC_CELLS);
	c.positions = take(12ull * ((uint64_t)max_samples + 8));
	c.indices = take(4ull * ((uint64_t)max_samples + 8));
	c.mlp_out = take(32ull * chunk + 4ull * chunk);
	c.bitfield = take((uint64_t)OCC_LEVELS * OCC_LEVEL_BYTES);
	c.partial = take(4ull * OCC_MEAN_BLOCKS);
	c.mean = take(4);
	c.total = o;
	return c;
}

N2_API int n2_occupancy_create(uint32_t n_cascades, uint64_t seed, n2_occupancy_t** out) {
	N2_REQUIRE(out != nullptr, "n2_occupancy_create: out is null");
	*out = nullptr;
	N2_REQUIRE(n_cascades >= 1 && n_cascades <= OCC_LEVELS, "n2_occupancy_create: n_cascades %u outside [1, %u]", n_cascades, OCC_LEVELS);
	n2_occupancy* o = new (std::nothrow) n2_occupancy();
	N2_REQUIRE(o != nullptr, "n2_occupancy_create: out of host memory");
	o->n_cascades = n_cascades;
	// pcg32(initstate = seed, initseq = 1)
	Pcg32 r{0u, (1ull << 1u) | 1u};
	r.next_uint();
	r.state += seed;
	r.next_uint();
	o->rng_state = r.state; o->rng_inc = r.inc;
	o->ema_step = 0;
	o->ws = nullptr;
	*out = o;
	return N2_OK;
}

N2_API void n2_occupancy_destroy(n2_occupancy_t* occ) { delete occ; }

static uint32_t occ_chunk(uint32_t max_samples, uint32_t max_chunk) {
	uint32_t c = (max_samples + 7) / 8 * 8;
	if (c > max_chunk) c = max_chunk / 8 * 8;
	return c;
}

N2_API uint64_t n2_occupancy_workspace_bytes(const n2_occupancy_t* occ, uint32_t max_samples, uint32_t max_chunk) {
	if (!occ || max_chunk < 8 || max_samples == 0) return 0;
	return occ_carve(occ->n_cascades, max_samples, occ_chunk(max_samples, max_chunk)).total;
}

N2_API int n2_occupancy_set_workspace(n2_occupancy_t* occ, void* d_workspace, uint64_t n_bytes, uint32_t max_samples, uint32_t max_chunk) {
	N2_REQUIRE(occ != nullptr && d_workspace != nullptr, "n2_occupancy_set_workspace: null argument");
	N2_REQUIRE(reinterpret_cast<uintptr_t>(d_workspace) % 256 == 0, "n2_occupancy_set_workspace: workspace must be 256-byte aligned");
	N2_REQUIRE(max_samples >= 1 && max_chunk >= 8, "n2_occupancy_set_workspace: max_samples >= 1 and max_chunk >= 8 required");
	const uint32_t chunk = occ_chunk(max_samples, max_chunk);
	const OccCarve c = occ_carve(occ->n_cascades, max_samples, chunk);
	N2_REQUIRE(n_bytes >= c.total, "n2_occupancy_set_workspace: %llu bytes given, %llu needed", (unsigned long long)n_bytes, (unsigned long long)c.total);
	unsigned char* b = reinterpret_cast<unsigned char*>(d_workspace);
	occ->ws = b; occ->max_samples = max_samples; occ->chunk = chunk;
	occ->grid = reinterpret_cast<float*>(b + c.grid);
	occ->tmp = reinterpret_cast<float*>(b + c.tmp);
	occ->positions = reinterpret_cast<float*>(b + c.positions);
	occ->indices = reinterpret_cast<uint32_t*>(b + c.indices);
	occ->mlp_out = reinterpret_cast<hf*>(b + c.mlp_out);
	occ->bitfield = b + c.bitfield;
	occ->partial = reinterpret_cast<float*>(b + c.partial);
	occ->mean = reinterpret_cast<float*>(b + c.mean);
	occ->last_n = 0;
	occ->last_n_uniform = 0;
	return N2_OK;
}

N2_API int n2_occupancy_reset(n2_occupancy_t* occ, n2_stream_t stream) {
	N2_REQUIRE(occ != nullptr && occ->ws != nullptr, "n2_occupancy_reset: no workspace");
	occ->ema_step = 0;
	if (int rc = n2_fill_zero_u32(n2_stream(stream), occ->grid, 4ull * occ->n_cascades * OCC_CELLS)) return rc;
	if (int rc = n2_fill_zero_u32(n2_stream(stream), occ->bitfield, (uint64_t)OCC_LEVELS * OCC_LEVEL_BYTES)) return rc;
	return n2_fill_zero_u32(n2_stream(stream), occ->mean, 4);
}

static inline dim3 ogrid(uint64_t n) { return dim3((uint32_t)((n + OCC_BLOCK - 1) / OCC_BLOCK)); }

static int occ_bitfield_from_partials(n2_occupancy_t* occ, hipStream_t s);

N2_API int n2_occupancy_update_bitfield(n2_occupancy_t* occ, n2_stream_t stream) {
	N2_REQUIRE(occ != nullptr && occ->ws != nullptr, "n2_occupancy_update_bitfield: no workspace");
	hipStream_t s = n2_stream(stream);
	const uint32_t n_elements = occ->n_cascades * OCC_CELLS;
	occ_ema_kernel<false><<<dim3((n_elements + OCC_BLOCK * 32 - 1) / (OCC_BLOCK * 32)), dim3(OCC_BLOCK), 0, s>>>(n_elements, 1.f, occ->grid, occ->tmp,
	                                                                                                             occ->partial);
	N2_LAUNCH_CHECK();
	return occ_bitfield_from_partials(occ, s);
}

static int occ_bitfield_from_partials(n2_occupancy_t* occ, hipStream_t s) {
	const uint32_t n_bytes = OCC_LEVELS * OCC_LEVEL_BYTES;
	occ_mean_kernel<<<dim3(1), dim3(OCC_MEAN_BLOCKS), 0, s>>>(occ->partial, occ->mean);
	N2_LAUNCH_CHECK();
	occ_bitfield_kernel<<<ogrid(n_bytes), dim3(OCC_BLOCK), 0, s>>>(n_bytes, occ->n_cascades * OCC_LEVEL_BYTES, occ->grid, occ->bitfield, occ->mean);
	N2_LAUNCH_CHECK();
	for (uint32_t level = 1; level < OCC_LEVELS; ++level) {
		occ_pool_kernel<<<ogrid(OCC_CELLS / 64), dim3(OCC_BLOCK), 0, s>>>(occ->bitfield + (size_t)(level - 1) * OCC_LEVEL_BYTES,
		                                                                  occ->bitfield + (size_t)level * OCC_LEVEL_BYTES);
		N2_LAUNCH_CHECK();
	}
	return N2_OK;
}

N2_API int n2_occupancy_update(n2_occupancy_t* occ, n2_field_t* field, n2_stream_t stream, float decay, uint32_t n_uniform,
                               uint32_t n_nonuniform) {
	N2_REQUIRE(occ != nullptr && occ->ws != nullptr, "n2_occupancy_update: n2_occupancy_set_workspace has not been called");
	N2_REQUIRE(field != nullptr, "n2_occupancy_update: field is null");
	const uint64_t n64 = (uint64_t)n_uniform + n_nonuniform;
	N2_REQUIRE(n64 <= occ->max_samples, "n2_occupancy_update: %llu samples exceed the workspace's %u", (unsigned long long)n64, occ->max_samples);
	hipStream_t s = n2_stream(stream);
	const uint32_t n = (uint32_t)n64, n_elements = occ->n_cascades * OCC_CELLS;
	if (int rc = n2_fill_zero_u32(s, occ->tmp, 4ull * n_elements)) return rc;
	Pcg32 rng{occ->rng_state, occ->rng_inc};
	if (n_uniform) {
		// slots of the second group are written by the second launch; only the last launch pads
		const uint32_t pad = n_nonuniform ? n_uniform : (n_uniform + 7) / 8 * 8;
		occ_generate_kernel<<<ogrid(pad), dim3(OCC_BLOCK), 0, s>>>(n_uniform, pad, rng, occ->ema_step, occ->grid, occ->n_cascades, -0.01f,
		                                                          occ_order_mul(n_uniform), occ->positions, occ->indices);
		N2_LAUNCH_CHECK();
	}
	rng.advance(1ull << 32);
	if (n_nonuniform) {
		const uint32_t pad = (n + 7) / 8 * 8 - n_uniform;
		occ_generate_kernel<<<ogrid(pad), dim3(OCC_BLOCK), 0, s>>>(n_nonuniform, pad, rng, occ->ema_step, occ->grid, occ->n_cascades,
		                                                          OCC_MIN_OPTICAL_THICKNESS, occ_order_mul(n_nonuniform),
		                                                          occ->positions + (size_t)n_uniform * 3, occ->indices + n_uniform);
		N2_LAUNCH_CHECK();
	}
	rng.advance(1ull << 32);
	occ->rng_state = rng.state;
	// densities, a chunk at a time (row 0 of the field's 16 x chunk output)
	for (uint32_t a = 0; a < n; a += occ->chunk) {
		const uint32_t m = (n - a < occ->chunk) ? n - a : occ->chunk, m8 = (m + 7) / 8 * 8;
		// only the density row is kept, as fp32 (the fp16 output widened); the row sits behind the fp16 scratch the unfused path needs
		float* row0 = reinterpret_cast<float*>(occ->mlp_out + (size_t)16 * occ->chunk);
		if (int rc = n2_field_sdf_row0(field, stream, occ->positions + (size_t)a * 3, 3, 1, m8, m8, row0, reinterpret_cast<n2_half*>(occ->mlp_out), true)) return rc;
		occ_splat_kernel<<<ogrid(m), dim3(OCC_BLOCK), 0, s>>>(m, occ->indices + a, row0, occ->tmp);
		N2_LAUNCH_CHECK();
	}
	occ_ema_kernel<true><<<dim3((n_elements + OCC_BLOCK * 32 - 1) / (OCC_BLOCK * 32)), dim3(OCC_BLOCK), 0, s>>>(n_elements, decay, occ->grid, occ->tmp,
	                                                                                                            occ->partial);
	N2_LAUNCH_CHECK();
	occ->ema_step += 1;
	occ->last_n = n;
	occ->last_n_uniform = n_uniform;
	return occ_bitfield_from_partials(occ, s);
}

N2_API int n2_occupancy_view(n2_occupancy_t* occ, n2_occupancy_buffers* out) {
	N2_REQUIRE(occ != nullptr && out != nullptr, "n2_occupancy_view: null argument");
	N2_REQUIRE(occ->ws != nullptr, "n2_occupancy_view: n2_occupancy_set_workspace has not been called");
	out->density_grid = occ->grid;
	out->density_grid_tmp = occ->tmp;
	out->bitfield = occ->bitfield;
	out->mean = occ->mean;
	out->positions = occ->positions;
	out->indices = occ->indices;
	out->n_samples = occ->last_n;
	out->n_uniform = occ->last_n_uniform;
	out->n_cascades = occ->n_cascades;
	out->ema_step = occ->ema_step;
	out->rng_state = occ->rng_state;
	out->rng_inc = occ->rng_inc;
	return N2_OK;
}

N2_API int n2_occupancy_set_state(n2_occupancy_t* occ, uint32_t ema_step, uint64_t rng_state, uint64_t rng_inc) {
	N2_REQUIRE(occ != nullptr, "n2_occupancy_set_state: occupancy is null");
	N2_REQUIRE((rng_inc & 1u) == 1u, "n2_occupancy_set_state: a PCG32 increment is odd");
	occ->ema_step = ema_step; occ->rng_state = rng_state; occ->rng_inc = rng_inc;
	return N2_OK;
}
