// Mesh extraction from a density lattice: marching cubes with shared vertices
// (marching_cubes_gpu, src/marching_cubes.cu:794-822, with gen_vertices :276-329
// and gen_faces :377-718) and the area-weighted vertex normals of
// accumulate_1ring (:331-366).
//
// Same geometry as the reference: lattice value at (x, y, z) is
// density[x + y*rx + z*rx*ry], a point is inside when density > thresh, one
// vertex per lattice edge whose ends differ, at dt = (thresh - f0) / (f1 - f0)
// along the edge, scaled by (aabb.max - aabb.min) / res and shifted by
// aabb.min; cube corner bits and edge numbers as in gen_faces.
//
// Two things are done differently.  The reference numbers vertices and
// triangles with atomicAdd, which is a race; here a lattice point's vertices
// (x, y, z edge in that order) and a cube's triangles get their slots from
// exclusive prefix sums in lattice order, so the mesh is reproducible.  And the
// 256-case table is derived on the host instead of being typed in: the cut
// edges on every cube face are joined into directed segments (an ambiguous face
// always separates its two inside corners), the segments chain into closed
// loops, every loop is cut into a fan of triangles from its lowest edge.
// The reference's table has the same segments on every face in all 256 cases,
// i.e. the same surface with the same orientation; only the diagonals inside
// polygons of more than three corners differ in some cases.
//
// Vertex positions are part of the bit-exact contract with the CPU oracle:
// floating-point contraction is off for this file.
#include "n2_common.h"

#include <cstring>

#pragma clang fp contract(off)

constexpr uint32_t MC_BLOCK = 256;
constexpr uint32_t MC_SCAN_ITEMS = 16;                       // elements per thread of the scan kernels
constexpr uint32_t MC_SCAN_TILE = MC_BLOCK * MC_SCAN_ITEMS;  // 4096 elements per workgroup

struct McTable {
	int8_t tri[256][16];
};

// ---------------------------------------------------------------------------
// case table (host)
// ---------------------------------------------------------------------------
namespace {

const int MC_EDGE_CORNERS[12][2] = {{0, 1}, {1, 2}, {2, 3}, {3, 0}, {4, 5}, {5, 6}, {6, 7}, {7, 4}, {0, 4}, {1, 5}, {2, 6}, {3, 7}};
// the six faces as corner cycles, counter-clockwise seen from outside: x = 0, x = 1, y = 0, y = 1, z = 0, z = 1
const int MC_FACES[6][4] = {{4, 7, 3, 0}, {1, 2, 6, 5}, {1, 5, 4, 0}, {3, 7, 6, 2}, {3, 2, 1, 0}, {4, 5, 6, 7}};

int mc_edge_between(int a, int b) {
	for (int e = 0; e < 12; ++e)
		if ((MC_EDGE_CORNERS[e][0] == a && MC_EDGE_CORNERS[e][1] == b) || (MC_EDGE_CORNERS[e][0] == b && MC_EDGE_CORNERS[e][1] == a)) return e;
	return -1;
}

void mc_build_table(McTable& t) {
	memset(t.tri, -1, sizeof(t.tri));
	for (int mask = 0; mask < 256; ++mask) {
		int next[12];
		for (int e = 0; e < 12; ++e) next[e] = -1;
		for (const auto& cyc : MC_FACES) {
			int in[4], n_in = 0;
			for (int k = 0; k < 4; ++k) { in[k] = (mask >> cyc[k]) & 1; n_in += in[k]; }
			if (n_in == 0 || n_in == 4) continue;
			// every maximal run of inside corners is cut off by one segment, directed from the edge after the run to the
			// edge before it (the surface normal then points to the inside)
			for (int k = 0; k < 4; ++k) {
				if (!in[k] || in[(k + 3) % 4]) continue;
				int j = k;
				while (in[(j + 1) % 4]) ++j;
				const int before = mc_edge_between(cyc[(k + 3) % 4], cyc[k]);
				const int after = mc_edge_between(cyc[j % 4], cyc[(j + 1) % 4]);
				next[after] = before;
			}
		}
		bool seen[12] = {};
		int n = 0;
		for (int e = 0; e < 12; ++e) {
			if (next[e] < 0 || seen[e]) continue;
			int loop[12], len = 0;
			for (int c = e; !seen[c]; c = next[c]) { seen[c] = true; loop[len++] = c; }
			for (int k = 1; k + 1 < len; ++k) {
				t.tri[mask][n++] = (int8_t)loop[0];
				t.tri[mask][n++] = (int8_t)loop[k];
				t.tri[mask][n++] = (int8_t)loop[k + 1];
			}
		}
	}
}

const McTable& mc_table() {
	static McTable t = [] { McTable x; mc_build_table(x); return x; }();
	return t;
}

}  // namespace

// ---------------------------------------------------------------------------
// kernels
// ---------------------------------------------------------------------------
struct McGrid {
	uint32_t rx, ry, rz;
	float thresh;
	float scale[3], offset[3];
};

__device__ __forceinline__ uint32_t mc_cube_mask(const McGrid& g, const float* __restrict__ density, uint32_t idx) {
	const uint32_t r1 = g.rx, r2 = g.rx * g.ry;
	uint32_t mask = 0;
	if (density[idx] > g.thresh) mask |= 1;
	if (density[idx + 1] > g.thresh) mask |= 2;
	if (density[idx + 1 + r1] > g.thresh) mask |= 4;
	if (density[idx + r1] > g.thresh) mask |= 8;
	if (density[idx + r2] > g.thresh) mask |= 16;
	if (density[idx + r2 + 1] > g.thresh) mask |= 32;
	if (density[idx + r2 + 1 + r1] > g.thresh) mask |= 64;
	if (density[idx + r2 + r1] > g.thresh) mask |= 128;
	return mask;
}

// Per lattice point: which of its three edges (towards +x, +y, +z) carry a vertex, and how many triangles its cube has.
__global__ void __launch_bounds__(MC_BLOCK) mc_count_kernel(McGrid g, const McTable* __restrict__ table, const float* __restrict__ density,
                                                            uint32_t* __restrict__ vcount, uint32_t* __restrict__ tcount) {
	const uint64_t n = (uint64_t)g.rx * g.ry * g.rz;
	const uint64_t i = (uint64_t)blockIdx.x * MC_BLOCK + threadIdx.x;
	if (i >= n) return;
	const uint32_t idx = (uint32_t)i;
	const uint32_t x = idx % g.rx, y = (idx / g.rx) % g.ry, z = idx / (g.rx * g.ry);
	const bool inside = density[idx] > g.thresh;
	uint32_t flags = 0;
	if (x + 1 < g.rx && inside != (density[idx + 1] > g.thresh)) flags |= 1;
	if (y + 1 < g.ry && inside != (density[idx + g.rx] > g.thresh)) flags |= 2;
	if (z + 1 < g.rz && inside != (density[idx + g.rx * g.ry] > g.thresh)) flags |= 4;
	// the count travels in the low bits, the flags in bits 29..31 (a mesh has fewer than 2^29 vertices)
	vcount[idx] = (uint32_t)__popc(flags) | (flags << 29);
	uint32_t tris = 0;
	if (x + 1 < g.rx && y + 1 < g.ry && z + 1 < g.rz) {
		const uint32_t mask = mc_cube_mask(g, density, idx);
		if (mask != 0 && mask != 255) {  // almost every cube of a lattice lies on one side of the surface
			const int8_t* row = table->tri[mask];
			while (tris < 15 && row[tris] >= 0) tris += 3;
			tris /= 3;
		}
	}
	tcount[idx] = tris;
}

// Exclusive prefix sum in three passes over tiles of 4096 elements.  `keep_mask` bits of every element are carried through
// unchanged (the vertex counts keep their flags); sums must stay below the lowest kept bit.
__global__ void __launch_bounds__(MC_BLOCK) mc_scan_tiles_kernel(uint64_t n, uint32_t* __restrict__ data, uint32_t keep_mask, uint32_t* __restrict__ tile_sums) {
	__shared__ uint32_t wave_sum[MC_BLOCK / 64];
	const uint64_t base = (uint64_t)blockIdx.x * MC_SCAN_TILE + (uint64_t)threadIdx.x * MC_SCAN_ITEMS;
	uint32_t v[MC_SCAN_ITEMS], kept[MC_SCAN_ITEMS], sum = 0;
#pragma unroll
	for (uint32_t k = 0; k < MC_SCAN_ITEMS; ++k) {
		const uint32_t raw = (base + k < n) ? data[base + k] : 0u;
		kept[k] = raw & keep_mask;
		v[k] = raw & ~keep_mask;
		sum += v[k];
	}
	const uint32_t lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
	uint32_t incl = sum;
#pragma unroll
	for (int o = 1; o < 64; o <<= 1) {
		const uint32_t u = __shfl_up(incl, o);
		if ((int)lane >= o) incl += u;
	}
	if (lane == 63) wave_sum[wave] = incl;
	__syncthreads();
	uint32_t run = incl - sum;
	for (uint32_t w = 0; w < wave; ++w) run += wave_sum[w];
#pragma unroll
	for (uint32_t k = 0; k < MC_SCAN_ITEMS; ++k) {
		if (base + k < n) data[base + k] = run | kept[k];
		run += v[k];
	}
	if (threadIdx.x == MC_BLOCK - 1) tile_sums[blockIdx.x] = run;
}
// one workgroup scans the tile sums in place (exclusive) and leaves the grand total behind them
__global__ void __launch_bounds__(1024) mc_scan_sums_kernel(uint32_t n_tiles, uint32_t* __restrict__ tile_sums, uint32_t* __restrict__ total) {
	__shared__ uint32_t wave_sum[16];
	__shared__ uint32_t carry;
	if (threadIdx.x == 0) carry = 0;
	__syncthreads();
	for (uint32_t base = 0; base < n_tiles; base += 1024) {
		const uint32_t i = base + threadIdx.x;
		const uint32_t v = i < n_tiles ? tile_sums[i] : 0u;
		const uint32_t lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
		uint32_t incl = v;
#pragma unroll
		for (int o = 1; o < 64; o <<= 1) {
			const uint32_t u = __shfl_up(incl, o);
			if ((int)lane >= o) incl += u;
		}
		if (lane == 63) wave_sum[wave] = incl;
		__syncthreads();
		uint32_t run = carry + incl - v;
		for (uint32_t w = 0; w < wave; ++w) run += wave_sum[w];
		if (i < n_tiles) tile_sums[i] = run;
		__syncthreads();
		if (threadIdx.x == 1023) carry = run + v;
		__syncthreads();
	}
	if (threadIdx.x == 0) *total = carry;
}
__global__ void __launch_bounds__(MC_BLOCK) mc_scan_add_kernel(uint64_t n, uint32_t* __restrict__ data, const uint32_t* __restrict__ tile_sums) {
	const uint64_t i = (uint64_t)blockIdx.x * MC_BLOCK + threadIdx.x;
	if (i < n) data[i] += tile_sums[i / MC_SCAN_TILE];
}

// slot of the vertex on the edge that leaves lattice point `p` in direction `axis`
__device__ __forceinline__ uint32_t mc_vertex_slot(const uint32_t* __restrict__ voff, uint32_t p, uint32_t axis) {
	const uint32_t w = voff[p];
	return (w & 0x1FFFFFFFu) + (uint32_t)__popc((w >> 29) & ((1u << axis) - 1u));
}

__global__ void __launch_bounds__(MC_BLOCK) mc_vertices_kernel(McGrid g, const float* __restrict__ density, const uint32_t* __restrict__ voff,
                                                               float* __restrict__ verts) {
	const uint64_t n = (uint64_t)g.rx * g.ry * g.rz;
	const uint64_t i = (uint64_t)blockIdx.x * MC_BLOCK + threadIdx.x;
	if (i >= n) return;
	const uint32_t idx = (uint32_t)i;
	const uint32_t w = voff[idx], flags = w >> 29;
	if (!flags) return;
	uint32_t slot = w & 0x1FFFFFFFu;
	const float p[3] = {(float)(idx % g.rx), (float)((idx / g.rx) % g.ry), (float)(idx / (g.rx * g.ry))};
	const uint32_t step[3] = {1u, g.rx, g.rx * g.ry};
	const float f0 = density[idx];
#pragma unroll
	for (uint32_t a = 0; a < 3; ++a) {
		if (!((flags >> a) & 1u)) continue;
		const float f1 = density[idx + step[a]];
		const float dt = (g.thresh - f0) / (f1 - f0);
		float* v = verts + (size_t)slot * 3;
#pragma unroll
		for (uint32_t d = 0; d < 3; ++d) v[d] = (d == a ? p[d] + dt : p[d]) * g.scale[d] + g.offset[d];
		++slot;
	}
}

__global__ void __launch_bounds__(MC_BLOCK) mc_faces_kernel(McGrid g, const McTable* __restrict__ table, const float* __restrict__ density,
                                                            const uint32_t* __restrict__ voff, const uint32_t* __restrict__ toff,
                                                            uint32_t* __restrict__ indices) {
	const uint64_t n = (uint64_t)g.rx * g.ry * g.rz;
	const uint64_t i = (uint64_t)blockIdx.x * MC_BLOCK + threadIdx.x;
	if (i >= n) return;
	const uint32_t idx = (uint32_t)i;
	const uint32_t x = idx % g.rx, y = (idx / g.rx) % g.ry, z = idx / (g.rx * g.ry);
	if (x + 1 >= g.rx || y + 1 >= g.ry || z + 1 >= g.rz) return;
	const uint32_t mask = mc_cube_mask(g, density, idx);
	if (mask == 0 || mask == 255) return;
	const uint32_t r1 = g.rx, r2 = g.rx * g.ry;
	// lattice point and direction that own each cube edge (src/marching_cubes.cu:690-706)
	const uint32_t own_p[12] = {idx, idx + 1, idx + r1, idx, idx + r2, idx + r2 + 1, idx + r2 + r1, idx + r2, idx, idx + 1, idx + 1 + r1, idx + r1};
	const uint32_t own_a[12] = {0, 1, 0, 1, 0, 1, 0, 1, 2, 2, 2, 2};
	const int8_t* row = table->tri[mask];
	uint32_t* out = indices + (size_t)toff[idx] * 3;
	for (uint32_t k = 0; k < 15 && row[k] >= 0; ++k) out[k] = mc_vertex_slot(voff, own_p[row[k]], own_a[row[k]]);
}

// accumulate_1ring's normals: per triangle (pb - pa) x (pa - pc), added to its three vertices
__global__ void __launch_bounds__(MC_BLOCK) mc_normals_kernel(uint32_t n_tris, const uint32_t* __restrict__ indices, const float* __restrict__ verts,
                                                              float* __restrict__ normals) {
	const uint32_t i = blockIdx.x * MC_BLOCK + threadIdx.x;
	if (i >= n_tris) return;
	const uint32_t ia = indices[i * 3], ib = indices[i * 3 + 1], ic = indices[i * 3 + 2];
	const float* pa = verts + (size_t)ia * 3;
	const float* pb = verts + (size_t)ib * 3;
	const float* pc = verts + (size_t)ic * 3;
	const float u[3] = {pb[0] - pa[0], pb[1] - pa[1], pb[2] - pa[2]}, w[3] = {pa[0] - pc[0], pa[1] - pc[1], pa[2] - pc[2]};
	const float nrm[3] = {u[1] * w[2] - u[2] * w[1], u[2] * w[0] - u[0] * w[2], u[0] * w[1] - u[1] * w[0]};
	const uint32_t who[3] = {ia, ib, ic};
#pragma unroll
	for (int k = 0; k < 3; ++k)
#pragma unroll
		for (int d = 0; d < 3; ++d) atomicAdd(normals + (size_t)who[k] * 3 + d, nrm[d]);
}

// ---------------------------------------------------------------------------
// C ABI
// ---------------------------------------------------------------------------
static inline dim3 mgrid(uint64_t n) { return dim3((uint32_t)((n + MC_BLOCK - 1) / MC_BLOCK)); }
static inline uint64_t m256(uint64_t x) { return (x + 255) / 256 * 256; }

N2_API int n2_marching_cubes_table(int8_t* out_256x16) {
	N2_REQUIRE(out_256x16 != nullptr, "n2_marching_cubes_table: out is null");
	memcpy(out_256x16, mc_table().tri, sizeof(McTable));
	return N2_OK;
}

static int mc_check(const char* fn, const uint32_t res[3], uint64_t& n) {
	N2_REQUIRE(res != nullptr, "%s: res is null", fn);
	N2_REQUIRE(res[0] >= 2 && res[1] >= 2 && res[2] >= 2, "%s: every resolution must be at least 2 (got %u x %u x %u)", fn, res[0], res[1], res[2]);
	n = (uint64_t)res[0] * res[1] * res[2];
	N2_REQUIRE(n <= (1ull << 31), "%s: %llu lattice points exceed 2^31", fn, (unsigned long long)n);
	return N2_OK;
}

N2_API uint64_t n2_marching_cubes_workspace_bytes(const uint32_t res[3]) {
	uint64_t n;
	if (mc_check("n2_marching_cubes_workspace_bytes", res, n) != N2_OK) return 0;
	const uint64_t tiles = (n + MC_SCAN_TILE - 1) / MC_SCAN_TILE;
	return 2 * m256(4 * n) + 2 * m256(4 * tiles) + 256 + m256(sizeof(McTable));
}

N2_API int n2_marching_cubes_count(n2_stream_t stream, const uint32_t res[3], const float aabb_min[3], const float aabb_max[3], float thresh,
                                   const float* d_density, void* d_workspace, uint64_t workspace_bytes, uint32_t* n_vertices,
                                   uint32_t* n_triangles) {
	uint64_t n;
	if (int rc = mc_check("n2_marching_cubes_count", res, n)) return rc;
	N2_REQUIRE(d_density && d_workspace && n_vertices && n_triangles && aabb_min && aabb_max, "n2_marching_cubes_count: null argument");
	N2_REQUIRE(reinterpret_cast<uintptr_t>(d_workspace) % 256 == 0, "n2_marching_cubes_count: workspace must be 256-byte aligned");
	N2_REQUIRE(workspace_bytes >= n2_marching_cubes_workspace_bytes(res), "n2_marching_cubes_count: %llu bytes of workspace given, %llu needed",
	           (unsigned long long)workspace_bytes, (unsigned long long)n2_marching_cubes_workspace_bytes(res));
	hipStream_t s = n2_stream(stream);
	const uint32_t tiles = (uint32_t)((n + MC_SCAN_TILE - 1) / MC_SCAN_TILE);
	unsigned char* b = reinterpret_cast<unsigned char*>(d_workspace);
	uint32_t* voff = reinterpret_cast<uint32_t*>(b);
	uint32_t* toff = reinterpret_cast<uint32_t*>(b + m256(4 * n));
	uint32_t* vsums = reinterpret_cast<uint32_t*>(b + 2 * m256(4 * n));
	uint32_t* tsums = reinterpret_cast<uint32_t*>(b + 2 * m256(4 * n) + m256(4ull * tiles));
	uint32_t* totals = reinterpret_cast<uint32_t*>(b + 2 * m256(4 * n) + 2 * m256(4ull * tiles));
	McTable* table = reinterpret_cast<McTable*>(b + 2 * m256(4 * n) + 2 * m256(4ull * tiles) + 256);
	N2_HIP(hipMemcpyAsync(table, &mc_table(), sizeof(McTable), hipMemcpyHostToDevice, s));
	McGrid g;
	g.rx = res[0]; g.ry = res[1]; g.rz = res[2]; g.thresh = thresh;
	for (int d = 0; d < 3; ++d) { g.scale[d] = (aabb_max[d] - aabb_min[d]) / (float)res[d]; g.offset[d] = aabb_min[d]; }
	mc_count_kernel<<<mgrid(n), dim3(MC_BLOCK), 0, s>>>(g, table, d_density, voff, toff);
	N2_LAUNCH_CHECK();
	mc_scan_tiles_kernel<<<dim3(tiles), dim3(MC_BLOCK), 0, s>>>(n, voff, 0xE0000000u, vsums);
	N2_LAUNCH_CHECK();
	mc_scan_sums_kernel<<<dim3(1), dim3(1024), 0, s>>>(tiles, vsums, totals);
	N2_LAUNCH_CHECK();
	mc_scan_add_kernel<<<mgrid(n), dim3(MC_BLOCK), 0, s>>>(n, voff, vsums);
	N2_LAUNCH_CHECK();
	mc_scan_tiles_kernel<<<dim3(tiles), dim3(MC_BLOCK), 0, s>>>(n, toff, 0u, tsums);
	N2_LAUNCH_CHECK();
	mc_scan_sums_kernel<<<dim3(1), dim3(1024), 0, s>>>(tiles, tsums, totals + 1);
	N2_LAUNCH_CHECK();
	mc_scan_add_kernel<<<mgrid(n), dim3(MC_BLOCK), 0, s>>>(n, toff, tsums);
	N2_LAUNCH_CHECK();
	uint32_t host[2] = {0, 0};
	N2_HIP(hipMemcpyAsync(host, totals, sizeof(host), hipMemcpyDeviceToHost, s));
	N2_HIP(hipStreamSynchronize(s));
	N2_REQUIRE(host[0] < (1u << 29), "n2_marching_cubes_count: %u vertices exceed the 2^29 limit", host[0]);
	*n_vertices = host[0];
	*n_triangles = host[1];
	return N2_OK;
}

N2_API int n2_marching_cubes_emit(n2_stream_t stream, const uint32_t res[3], const float aabb_min[3], const float aabb_max[3], float thresh,
                                  const float* d_density, const void* d_workspace, float* d_vertices, uint32_t* d_indices, float* d_normals,
                                  uint32_t n_vertices, uint32_t n_triangles) {
	uint64_t n;
	if (int rc = mc_check("n2_marching_cubes_emit", res, n)) return rc;
	N2_REQUIRE(d_density && d_workspace && aabb_min && aabb_max, "n2_marching_cubes_emit: null argument");
	N2_REQUIRE((d_vertices || n_vertices == 0) && (d_indices || n_triangles == 0), "n2_marching_cubes_emit: null output");
	hipStream_t s = n2_stream(stream);
	const unsigned char* b = reinterpret_cast<const unsigned char*>(d_workspace);
	const uint32_t* voff = reinterpret_cast<const uint32_t*>(b);
	const uint32_t* toff = reinterpret_cast<const uint32_t*>(b + m256(4 * n));
	const uint64_t tiles = (n + MC_SCAN_TILE - 1) / MC_SCAN_TILE;
	const McTable* table = reinterpret_cast<const McTable*>(b + 2 * m256(4 * n) + 2 * m256(4 * tiles) + 256);
	N2_REQUIRE(d_normals == nullptr || reinterpret_cast<uintptr_t>(d_normals) % 16 == 0, "n2_marching_cubes_emit: d_normals must be 16-byte aligned");
	McGrid g;
	g.rx = res[0]; g.ry = res[1]; g.rz = res[2]; g.thresh = thresh;
	for (int d = 0; d < 3; ++d) { g.scale[d] = (aabb_max[d] - aabb_min[d]) / (float)res[d]; g.offset[d] = aabb_min[d]; }
	if (n_vertices) {
		mc_vertices_kernel<<<mgrid(n), dim3(MC_BLOCK), 0, s>>>(g, d_density, voff, d_vertices);
		N2_LAUNCH_CHECK();
	}
	if (n_triangles) {
		mc_faces_kernel<<<mgrid(n), dim3(MC_BLOCK), 0, s>>>(g, table, d_density, voff, toff, d_indices);
		N2_LAUNCH_CHECK();
	}
	if (d_normals && n_vertices) {
		if (int rc = n2_fill_zero_u32(s, d_normals, 12ull * n_vertices)) return rc;
		if (n_triangles) {
			mc_normals_kernel<<<mgrid(n_triangles), dim3(MC_BLOCK), 0, s>>>(n_triangles, d_indices, d_vertices, d_normals);
			N2_LAUNCH_CHECK();
		}
	}
	return N2_OK;
}

// ---------------------------------------------------------------------------
// The lattice the mesh is extracted from: Testbed::get_density_on_grid (src/testbed_nerf.cu:4082-4133) with
// generate_grid_samples_nerf_uniform (:586-598) and grid_samples_half_to_float (:682-696): positions
// (x, y, z) / res * (aabb.max - aabb.min) + aabb.min, the field's SDF (row 0 of NerfNetwork::sdf) widened to fp32.
// ---------------------------------------------------------------------------
typedef _Float16 hf;

__global__ void __launch_bounds__(MC_BLOCK) mc_lattice_positions_kernel(McGrid g, uint64_t first, uint32_t count, uint32_t padded,
                                                                        float* __restrict__ positions) {
	const uint32_t i = blockIdx.x * MC_BLOCK + threadIdx.x;
	if (i >= padded) return;
	float* p = positions + (size_t)i * 3;
	if (i >= count) { p[0] = p[1] = p[2] = 0.5f; return; }
	const uint64_t idx = first + i;
	const uint32_t c[3] = {(uint32_t)(idx % g.rx), (uint32_t)((idx / g.rx) % g.ry), (uint32_t)(idx / ((uint64_t)g.rx * g.ry))};
	const uint32_t r[3] = {g.rx, g.ry, g.rz};
#pragma unroll
	for (int d = 0; d < 3; ++d) p[d] = ((float)c[d] * (1.f / (float)r[d])) * g.scale[d] + g.offset[d];
}
__global__ void __launch_bounds__(MC_BLOCK) mc_widen_kernel(uint32_t n, const hf* __restrict__ in, float* __restrict__ out) {
	const uint32_t i = blockIdx.x * MC_BLOCK + threadIdx.x;
	if (i < n) out[i] = (float)in[i];
}

N2_API uint64_t n2_density_on_grid_scratch_bytes(uint32_t chunk) { return m256(12ull * chunk) + m256(32ull * chunk); }

N2_API int n2_density_on_grid(n2_field_t* field, n2_stream_t stream, const uint32_t res[3], const float aabb_min[3], const float aabb_max[3],
                              float* d_density, void* d_scratch, uint64_t scratch_bytes, uint32_t chunk) {
	uint64_t n;
	if (int rc = mc_check("n2_density_on_grid", res, n)) return rc;
	N2_REQUIRE(field && d_density && d_scratch && aabb_min && aabb_max, "n2_density_on_grid: null argument");
	N2_REQUIRE(chunk >= 8 && chunk % 8 == 0, "n2_density_on_grid: chunk %u must be a positive multiple of 8", chunk);
	N2_REQUIRE(reinterpret_cast<uintptr_t>(d_scratch) % 256 == 0 && scratch_bytes >= n2_density_on_grid_scratch_bytes(chunk),
	           "n2_density_on_grid: scratch must be 256-byte aligned and hold %llu bytes", (unsigned long long)n2_density_on_grid_scratch_bytes(chunk));
	hipStream_t s = n2_stream(stream);
	float* positions = reinterpret_cast<float*>(d_scratch);
	hf* mlp_out = reinterpret_cast<hf*>(reinterpret_cast<unsigned char*>(d_scratch) + m256(12ull * chunk));
	McGrid g;
	g.rx = res[0]; g.ry = res[1]; g.rz = res[2]; g.thresh = 0.f;
	// here scale is the aabb's extent (the division by the resolution is part of the position formula)
	for (int d = 0; d < 3; ++d) { g.scale[d] = aabb_max[d] - aabb_min[d]; g.offset[d] = aabb_min[d]; }
	// lattice points arrive x fastest: neighbouring lanes in neighbouring cells
	n2_grid_set_point_order(n2_field_encoding(field), 1);
	int rc = N2_OK;
	for (uint64_t first = 0; first < n && rc == N2_OK; first += chunk) {
		const uint32_t m = (uint32_t)((n - first < chunk) ? n - first : chunk), m8 = (m + 7) / 8 * 8;
		mc_lattice_positions_kernel<<<mgrid(m8), dim3(MC_BLOCK), 0, s>>>(g, first, m, m8, positions);
		rc = n2_field_sdf(field, stream, positions, 3, 1, m8, reinterpret_cast<n2_half*>(mlp_out));
		if (rc == N2_OK) mc_widen_kernel<<<mgrid(m), dim3(MC_BLOCK), 0, s>>>(m, mlp_out, d_density + first);
	}
	n2_grid_set_point_order(n2_field_encoding(field), 0);
	if (rc != N2_OK) return rc;
	N2_LAUNCH_CHECK();
	return N2_OK;
}
