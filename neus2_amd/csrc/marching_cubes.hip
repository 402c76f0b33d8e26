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

struct McTable {
	int8_t tri[256][16];
	uint8_t ntri[256];  // triangles of each case
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
		t.ntri[mask] = (uint8_t)(n / 3);
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

// A wave looks at 64 consecutive lattice points (a chunk) at a time.  Whether a point is inside is one bit of a ballot, so
// a chunk costs four coalesced loads (the rows at y, y + 1, z + 1 and both) plus the four values right behind them, however
// many of the eight cube corners and three edges a point shares with its neighbours; a chunk whose four rows lie entirely
// on one side of the surface (almost all of them) is decided from the ballots alone.
constexpr uint32_t MC_CHUNKS = 4;                  // chunks per tile
constexpr uint32_t MC_WAVE_TILE = 64 * MC_CHUNKS;  // lattice points per tile: the unit the prefix sums are kept for (small, so that
                                                   // the few tiles the surface crosses spread over many waves when they are emitted)
constexpr uint32_t MC_COUNT_TILES = 4;             // consecutive tiles per wave of the count kernel

struct McPoint {
	uint32_t flags;  // bit a: the edge towards +axis a carries a vertex
	uint32_t mask;   // corner bits of the point's cube, 0 when it has none
};

// The ballots of MC_GROUP consecutive chunks are formed together, so that a wave has 4 x MC_GROUP loads in flight instead
// of one round trip per chunk; only the last chunk of a group needs the values right behind its rows, the others take them
// from the next chunk's ballots.
constexpr uint32_t MC_GROUP = 4;
static_assert(MC_CHUNKS % MC_GROUP == 0, "a wave's chunks come in whole groups");

struct McBallots {
	unsigned long long m[MC_GROUP][4];  // [chunk][row]: inside bits of 64 consecutive points of the rows at +0, +rx, +rx ry, +rx ry + rx
	bool next[4];                       // the point right behind the last chunk's rows
};

__device__ __forceinline__ void mc_load_group(const McGrid& g, const float* __restrict__ density, uint64_t n, uint32_t first, uint32_t lane, McBallots& B) {
	const uint32_t r1 = g.rx, r2 = g.rx * g.ry;
	const uint32_t off[4] = {0u, r1, r2, r2 + r1};
	float v[MC_GROUP][4], e[4];
#pragma unroll
	for (uint32_t c = 0; c < MC_GROUP; ++c)
#pragma unroll
		for (int j = 0; j < 4; ++j) {
			const uint64_t q = (uint64_t)first + c * 64u + off[j] + lane;
			v[c][j] = q < n ? density[q] : -INFINITY;
		}
#pragma unroll
	for (int j = 0; j < 4; ++j) {
		const uint64_t q = (uint64_t)first + MC_GROUP * 64u + off[j];  // the same address in every lane
		e[j] = q < n ? density[q] : -INFINITY;
	}
#pragma unroll
	for (uint32_t c = 0; c < MC_GROUP; ++c)
#pragma unroll
		for (int j = 0; j < 4; ++j) B.m[c][j] = __ballot(v[c][j] > g.thresh);
#pragma unroll
	for (int j = 0; j < 4; ++j) B.next[j] = e[j] > g.thresh;
}

// (x, y, z) of lattice point first + lane
__device__ __forceinline__ void mc_point_xyz(const McGrid& g, uint32_t first, uint32_t lane, uint32_t* c) {
	if (g.rx >= 64u) {  // at most one row ends inside the chunk
		uint32_t x = first % g.rx + lane;
		const uint32_t row = first / g.rx + (x >= g.rx ? 1u : 0u);
		x -= x >= g.rx ? g.rx : 0u;
		c[0] = x; c[1] = row % g.ry; c[2] = row / g.ry;
	} else {
		const uint32_t idx = first + lane;
		c[0] = idx % g.rx; c[1] = (idx / g.rx) % g.ry; c[2] = idx / (g.rx * g.ry);
	}
}

// Chunk c of a group.  False: no point of the chunk has an edge vertex or a triangle (p is then not filled in).
__device__ __forceinline__ bool mc_chunk(const McGrid& g, uint64_t n, const McBallots& B, uint32_t c, uint32_t first, uint32_t lane, McPoint& p) {
	unsigned long long m[4];
	bool next[4];
	bool all0 = true, all1 = true;
#pragma unroll
	for (int j = 0; j < 4; ++j) {
		m[j] = B.m[c][j];
		next[j] = c + 1 < MC_GROUP ? (B.m[c + 1 < MC_GROUP ? c + 1 : c][j] & 1ull) != 0ull : B.next[j];
		all0 = all0 && m[j] == 0ull && !next[j];
		all1 = all1 && m[j] == ~0ull && next[j];
	}
	if (all0 || all1) return false;
	uint32_t xyz[3];
	mc_point_xyz(g, first, lane, xyz);
	const bool here = (uint64_t)first + lane < n;
	const bool xok = xyz[0] + 1 < g.rx, yok = xyz[1] + 1 < g.ry, zok = xyz[2] + 1 < g.rz;
	bool in[4], in1[4];
#pragma unroll
	for (int j = 0; j < 4; ++j) {
		in[j] = (m[j] >> lane) & 1ull;
		in1[j] = lane < 63u ? ((m[j] >> (lane + 1u)) & 1ull) != 0ull : next[j];
	}
	p.flags = 0;
	p.mask = 0;
	if (here) {
		if (xok && in[0] != in1[0]) p.flags |= 1u;
		if (yok && in[0] != in[1]) p.flags |= 2u;
		if (zok && in[0] != in[2]) p.flags |= 4u;
		if (xok && yok && zok)  // corner bits as in gen_faces: round the bottom face from the point itself, then the top face
			p.mask = (in[0] ? 1u : 0u) | (in1[0] ? 2u : 0u) | (in1[1] ? 4u : 0u) | (in[1] ? 8u : 0u) | (in[2] ? 16u : 0u) | (in1[2] ? 32u : 0u) |
			         (in1[3] ? 64u : 0u) | (in[3] ? 128u : 0u);
	}
	return true;
}

// number of set bits of `b` below this lane
__device__ __forceinline__ uint32_t mc_below(unsigned long long b, uint32_t lane) { return (uint32_t)__popcll(b & ((1ull << lane) - 1ull)); }

// Per tile (256 consecutive lattice points): how many edge vertices and triangles its points own.
__global__ void __launch_bounds__(MC_BLOCK) mc_count_kernel(McGrid g, const McTable* __restrict__ table, const float* __restrict__ density,
                                                            uint32_t n_tiles, uint32_t* __restrict__ vsum, uint32_t* __restrict__ tsum,
                                                            uint8_t* __restrict__ busy) {
	const uint64_t n = (uint64_t)g.rx * g.ry * g.rz;
	const uint32_t lane = threadIdx.x & 63u;
	for (uint32_t tile = (blockIdx.x * (MC_BLOCK / 64) + (threadIdx.x >> 6)) * MC_COUNT_TILES, last = tile + MC_COUNT_TILES; tile < last && tile < n_tiles; ++tile) {
	uint32_t nv = 0, nt = 0, groups = 0;  // bit k of groups: group k of the tile has a chunk that is not all on one side
	for (uint32_t c0 = 0; c0 < MC_CHUNKS; c0 += MC_GROUP) {
		const uint32_t first0 = tile * MC_WAVE_TILE + c0 * 64u;
		if ((uint64_t)first0 >= n) break;
		McBallots B;
		mc_load_group(g, density, n, first0, lane, B);
#pragma unroll
		for (uint32_t c = 0; c < MC_GROUP; ++c) {
			McPoint p;
			if (!mc_chunk(g, n, B, c, first0 + c * 64u, lane, p)) continue;
			groups |= 1u << (c0 / MC_GROUP);
			nv += (uint32_t)__popc(p.flags);
			nt += table->ntri[p.mask];
		}
	}
#pragma unroll
	for (int o = 32; o > 0; o >>= 1) { nv += __shfl_xor(nv, o); nt += __shfl_xor(nt, o); }
	if (lane == 0) { vsum[tile] = nv; tsum[tile] = nt; busy[tile] = (uint8_t)groups; }
	}
}

// Exclusive prefix sums of the two per-tile arrays in place, by blocks of 1024 tiles (blockIdx.y 0: vertices, 1: triangles):
// first the blocks' totals, then every block adds up the totals before it and scans its own elements; element n_tiles
// receives the grand total.
__global__ void __launch_bounds__(1024) mc_block_totals_kernel(uint32_t n_tiles, const uint32_t* __restrict__ vsum, const uint32_t* __restrict__ tsum,
                                                               uint32_t* __restrict__ vblock, uint32_t* __restrict__ tblock) {
	__shared__ uint32_t wave_sum[16];
	const uint32_t* data = blockIdx.y == 0 ? vsum : tsum;
	const uint32_t i = blockIdx.x * 1024u + threadIdx.x;
	uint32_t v = i < n_tiles ? data[i] : 0u;
#pragma unroll
	for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o);
	if ((threadIdx.x & 63u) == 0) wave_sum[threadIdx.x >> 6] = v;
	__syncthreads();
	if (threadIdx.x == 0) {
		uint32_t all = 0;
#pragma unroll
		for (int w = 0; w < 16; ++w) all += wave_sum[w];
		(blockIdx.y == 0 ? vblock : tblock)[blockIdx.x] = all;
	}
}
__global__ void __launch_bounds__(1024) mc_scan_kernel(uint32_t n_tiles, uint32_t* __restrict__ vsum, uint32_t* __restrict__ tsum,
                                                       const uint32_t* __restrict__ vblock, const uint32_t* __restrict__ tblock) {
	__shared__ uint32_t wave_before[16], wave_sum[16];
	uint32_t* data = blockIdx.y == 0 ? vsum : tsum;
	const uint32_t* block = blockIdx.y == 0 ? vblock : tblock;
	const uint32_t lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
	const uint32_t i = blockIdx.x * 1024u + threadIdx.x;
	const uint32_t v = i < n_tiles ? data[i] : 0u;
	uint32_t before = 0;
	for (uint32_t q = threadIdx.x; q < blockIdx.x; q += 1024u) before += block[q];
#pragma unroll
	for (int o = 32; o > 0; o >>= 1) before += __shfl_xor(before, o);
	uint32_t incl = v;
#pragma unroll
	for (int o = 1; o < 64; o <<= 1) {
		const uint32_t u = __shfl_up(incl, o);
		if ((int)lane >= o) incl += u;
	}
	if (lane == 63) { wave_before[wave] = before; wave_sum[wave] = incl; }
	__syncthreads();
	uint32_t run = incl - v, all = 0;
#pragma unroll
	for (uint32_t w = 0; w < 16; ++w) { run += wave_before[w] + (w < wave ? wave_sum[w] : 0u); all += wave_before[w] + wave_sum[w]; }
	if (i < n_tiles) data[i] = run;
	if (blockIdx.x + 1 == gridDim.x && threadIdx.x == 0) data[n_tiles] = all;
}

// The emitting kernels run a fixed number of waves that stride over the tiles.  Most tiles own nothing: a wave looks at 64
// of its tiles at once (one per lane) and then visits those that own something.
constexpr uint32_t MC_EMIT_BLOCKS = 2048;

// Calls visit(tile, first slot, busy groups) for every tile of this wave whose prefix sum moves.
template <class Visit>
__device__ __forceinline__ void mc_for_owning_tiles(uint32_t n_tiles, const uint32_t* __restrict__ sums, const uint8_t* __restrict__ busy, Visit visit) {
	const uint32_t lane = threadIdx.x & 63u;
	const uint32_t wave = blockIdx.x * (MC_BLOCK / 64) + (threadIdx.x >> 6), n_waves = gridDim.x * (MC_BLOCK / 64);
	// Slot k of the walk deals the tiles k n_waves .. (k + 1) n_waves - 1 to the waves, rotated by 37 k: with a plain stride the
	// tiles of a wave would sit at one place of the planes they fall into (n_waves is a multiple of a plane's tiles for the
	// usual resolutions), and the waves that look at the middle of the object would own all the work.
	for (uint32_t k0 = 0; (uint64_t)k0 * n_waves < n_tiles; k0 += 64u) {
		const uint32_t k = k0 + lane;
		const uint64_t mine64 = (uint64_t)k * n_waves + (wave + k * 37u) % n_waves;
		const uint32_t mine = mine64 < n_tiles ? (uint32_t)mine64 : n_tiles;
		uint32_t begin = 0, end = 0, groups = 0;
		if (mine < n_tiles) { begin = sums[mine]; end = sums[mine + 1]; groups = busy[mine]; }
		unsigned long long owning = __ballot(end != begin);
		while (owning) {
			const int l = __ffsll((long long)owning) - 1;
			owning &= owning - 1ull;
			visit((uint32_t)__shfl((int)mine, l), (uint32_t)__shfl((int)begin, l), (uint32_t)__shfl((int)groups, l));
		}
	}
}

// Vertices of the tiles that have any, numbered in lattice order (x, y, z edge of a point in that order); voff[point] =
// first slot | edge flags << 29 is written for the points that own a vertex: the only ones the faces look up.
__global__ void __launch_bounds__(MC_BLOCK) mc_vertices_kernel(McGrid g, const float* __restrict__ density, uint32_t n_tiles,
                                                               const uint32_t* __restrict__ vsum, const uint8_t* __restrict__ busy,
                                                               uint32_t* __restrict__ voff, float* __restrict__ verts) {
	const uint64_t n = (uint64_t)g.rx * g.ry * g.rz;
	const uint32_t lane = threadIdx.x & 63u;
	const uint32_t step[3] = {1u, g.rx, g.rx * g.ry};
	mc_for_owning_tiles(n_tiles, vsum, busy, [&](uint32_t tile, uint32_t run, uint32_t groups) {
		for (uint32_t c0 = 0; c0 < MC_CHUNKS; c0 += MC_GROUP) {
			const uint32_t first0 = tile * MC_WAVE_TILE + c0 * 64u;
			if (!((groups >> (c0 / MC_GROUP)) & 1u)) continue;
			McBallots B;
			mc_load_group(g, density, n, first0, lane, B);
#pragma unroll
			for (uint32_t c = 0; c < MC_GROUP; ++c) {
				const uint32_t first = first0 + c * 64u;
				McPoint p;
				if (!mc_chunk(g, n, B, c, first, lane, p)) continue;
				const unsigned long long b0 = __ballot(p.flags & 1u), b1 = __ballot(p.flags & 2u), b2 = __ballot(p.flags & 4u);
				uint32_t slot = run + mc_below(b0, lane) + mc_below(b1, lane) + mc_below(b2, lane);
				run += (uint32_t)(__popcll(b0) + __popcll(b1) + __popcll(b2));
				if (!p.flags) continue;
				const uint32_t idx = first + lane;
				voff[idx] = slot | (p.flags << 29);
				uint32_t xyz[3];
				mc_point_xyz(g, first, lane, xyz);
				const float pos[3] = {(float)xyz[0], (float)xyz[1], (float)xyz[2]};
				const float f0 = density[idx];
#pragma unroll
				for (uint32_t a = 0; a < 3; ++a) {
					if (!((p.flags >> a) & 1u)) continue;
					const float f1 = density[idx + step[a]];
					const float dt = (g.thresh - f0) / (f1 - f0);
					float* v = verts + (size_t)slot * 3;
#pragma unroll
					for (uint32_t d = 0; d < 3; ++d) v[d] = (d == a ? pos[d] + dt : pos[d]) * g.scale[d] + g.offset[d];
					++slot;
				}
			}
		}
	});
}

// Triangles of the tiles that have any, numbered in lattice order of their cubes.
__global__ void __launch_bounds__(MC_BLOCK) mc_faces_kernel(McGrid g, const McTable* __restrict__ table, const float* __restrict__ density,
                                                            uint32_t n_tiles, const uint32_t* __restrict__ tsum, const uint8_t* __restrict__ busy,
                                                            const uint32_t* __restrict__ voff, uint32_t* __restrict__ indices) {
	const uint64_t n = (uint64_t)g.rx * g.ry * g.rz;
	const uint32_t lane = threadIdx.x & 63u;
	const uint32_t r1 = g.rx, r2 = g.rx * g.ry;
	mc_for_owning_tiles(n_tiles, tsum, busy, [&](uint32_t tile, uint32_t run, uint32_t groups) {
		for (uint32_t c0 = 0; c0 < MC_CHUNKS; c0 += MC_GROUP) {
			const uint32_t first0 = tile * MC_WAVE_TILE + c0 * 64u;
			if (!((groups >> (c0 / MC_GROUP)) & 1u)) continue;
			McBallots B;
			mc_load_group(g, density, n, first0, lane, B);
#pragma unroll
			for (uint32_t c = 0; c < MC_GROUP; ++c) {
				const uint32_t first = first0 + c * 64u;
				McPoint p;
				if (!mc_chunk(g, n, B, c, first, lane, p)) continue;
				const uint32_t tris = table->ntri[p.mask];  // 0 .. 5: three bit planes
				const unsigned long long b0 = __ballot(tris & 1u), b1 = __ballot(tris & 2u), b2 = __ballot(tris & 4u);
				const uint32_t mine = run + mc_below(b0, lane) + 2u * mc_below(b1, lane) + 4u * mc_below(b2, lane);
				run += (uint32_t)(__popcll(b0) + 2 * __popcll(b1) + 4 * __popcll(b2));
				if (!tris) continue;
				const uint32_t idx = first + lane;
				// Lattice point and direction that own each cube edge (src/marching_cubes.cu:690-706), five bits per edge:
				// the owner's offset from this point in x, y, z and the edge's axis.  The case's row is one 16-byte load and
				// all look-ups of a cube are in flight together.
				constexpr uint64_t OWNER = 0ull | 9ull << 5 | 2ull << 10 | 8ull << 15 | 4ull << 20 | 13ull << 25 | 6ull << 30 | 12ull << 35 |
				                           16ull << 40 | 17ull << 45 | 19ull << 50 | 18ull << 55;
				const uint4 row4 = *reinterpret_cast<const uint4*>(table->tri[p.mask]);
				const uint32_t row[4] = {row4.x, row4.y, row4.z, row4.w};
				uint32_t w[15], axis[15];
#pragma unroll
				for (uint32_t k = 0; k < 15; ++k) {
					const uint32_t e = (row[k >> 2] >> (8u * (k & 3u))) & 0xFu;  // rows end with -1: the low four bits of an unused entry name no edge that is read
					const uint32_t code = (uint32_t)(OWNER >> (5u * (e < 12u ? e : 0u))) & 31u;
					axis[k] = code >> 3;
					w[k] = k < 3u * tris ? voff[idx + (code & 1u) + ((code >> 1) & 1u) * r1 + ((code >> 2) & 1u) * r2] : 0u;
				}
				uint32_t* out = indices + (size_t)mine * 3;
#pragma unroll
				for (uint32_t k = 0; k < 15; ++k)
					if (k < 3u * tris)  // the owner's first slot plus the number of its edges before this one
						out[k] = (w[k] & 0x1FFFFFFFu) + (uint32_t)__popc((w[k] >> 29) & ((1u << axis[k]) - 1u));
			}
		}
	});
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
	memcpy(out_256x16, mc_table().tri, sizeof(mc_table().tri));
	return N2_OK;
}

static int mc_check(const char* fn, const uint32_t res[3], uint64_t& n) {
	N2_REQUIRE(res != nullptr, "%s: res is null", fn);
	N2_REQUIRE(res[0] >= 2 && res[1] >= 2 && res[2] >= 2, "%s: every resolution must be at least 2 (got %u x %u x %u)", fn, res[0], res[1], res[2]);
	n = (uint64_t)res[0] * res[1] * res[2];
	N2_REQUIRE(n <= (1ull << 31), "%s: %llu lattice points exceed 2^31", fn, (unsigned long long)n);
	return N2_OK;
}

// Workspace: voff (one word per lattice point, written only where a point owns a vertex), the two per-tile prefix-sum
// arrays (one entry more than tiles: the total), the case table.
struct McCarve {
	uint32_t n_tiles;
	uint32_t n_blocks;  // blocks of 1024 tiles
	uint64_t voff, vsum, tsum, busy, vblock, tblock, table, total;
};
static McCarve mc_carve(uint64_t n) {
	McCarve c;
	c.n_tiles = (uint32_t)((n + MC_WAVE_TILE - 1) / MC_WAVE_TILE);
	uint64_t o = 0;
	auto take = [&](uint64_t bytes) { const uint64_t at = o; o += m256(bytes); return at; };
	c.voff = take(4 * n);
	c.vsum = take(4ull * (c.n_tiles + 4));
	c.tsum = take(4ull * (c.n_tiles + 4));
	c.busy = take(c.n_tiles);
	c.n_blocks = (c.n_tiles + 1023u) / 1024u;
	c.vblock = take(4ull * c.n_blocks);
	c.tblock = take(4ull * c.n_blocks);
	c.table = take(sizeof(McTable));
	c.total = o;
	return c;
}

N2_API uint64_t n2_marching_cubes_workspace_bytes(const uint32_t res[3]) {
	uint64_t n;
	if (mc_check("n2_marching_cubes_workspace_bytes", res, n) != N2_OK) return 0;
	return mc_carve(n).total;
}

static McGrid mc_grid(const uint32_t res[3], const float aabb_min[3], const float aabb_max[3], float thresh) {
	McGrid g;
	g.rx = res[0]; g.ry = res[1]; g.rz = res[2]; g.thresh = thresh;
	for (int d = 0; d < 3; ++d) { g.scale[d] = (aabb_max[d] - aabb_min[d]) / (float)res[d]; g.offset[d] = aabb_min[d]; }
	return g;
}
static inline dim3 mc_tile_grid(uint32_t n_tiles) { const uint32_t per = MC_BLOCK / 64 * MC_COUNT_TILES; return dim3((n_tiles + per - 1) / per); }
static inline dim3 mc_emit_grid(uint32_t n_tiles) { const uint32_t b = (n_tiles + MC_BLOCK / 64 - 1) / (MC_BLOCK / 64); return dim3(b < MC_EMIT_BLOCKS ? b : MC_EMIT_BLOCKS); }

N2_API int n2_marching_cubes_count(n2_stream_t stream, const uint32_t res[3], const float aabb_min[3], const float aabb_max[3], float thresh,
                                   const float* d_density, void* d_workspace, uint64_t workspace_bytes, uint32_t* n_vertices,
                                   uint32_t* n_triangles) {
	uint64_t n;
	if (int rc = mc_check("n2_marching_cubes_count", res, n)) return rc;
	N2_REQUIRE(d_density && d_workspace && n_vertices && n_triangles && aabb_min && aabb_max, "n2_marching_cubes_count: null argument");
	N2_REQUIRE(reinterpret_cast<uintptr_t>(d_workspace) % 256 == 0, "n2_marching_cubes_count: workspace must be 256-byte aligned");
	const McCarve c = mc_carve(n);
	N2_REQUIRE(workspace_bytes >= c.total, "n2_marching_cubes_count: %llu bytes of workspace given, %llu needed",
	           (unsigned long long)workspace_bytes, (unsigned long long)c.total);
	hipStream_t s = n2_stream(stream);
	unsigned char* b = reinterpret_cast<unsigned char*>(d_workspace);
	uint32_t* vsum = reinterpret_cast<uint32_t*>(b + c.vsum);
	uint32_t* tsum = reinterpret_cast<uint32_t*>(b + c.tsum);
	McTable* table = reinterpret_cast<McTable*>(b + c.table);
	N2_HIP(hipMemcpyAsync(table, &mc_table(), sizeof(McTable), hipMemcpyHostToDevice, s));
	const McGrid g = mc_grid(res, aabb_min, aabb_max, thresh);
	mc_count_kernel<<<mc_tile_grid(c.n_tiles), dim3(MC_BLOCK), 0, s>>>(g, table, d_density, c.n_tiles, vsum, tsum, b + c.busy);
	N2_LAUNCH_CHECK();
	uint32_t* vblock = reinterpret_cast<uint32_t*>(b + c.vblock);
	uint32_t* tblock = reinterpret_cast<uint32_t*>(b + c.tblock);
	mc_block_totals_kernel<<<dim3(c.n_blocks, 2), dim3(1024), 0, s>>>(c.n_tiles, vsum, tsum, vblock, tblock);
	N2_LAUNCH_CHECK();
	mc_scan_kernel<<<dim3(c.n_blocks, 2), dim3(1024), 0, s>>>(c.n_tiles, vsum, tsum, vblock, tblock);
	N2_LAUNCH_CHECK();
	uint32_t host[2] = {0, 0};
	N2_HIP(hipMemcpyAsync(&host[0], vsum + c.n_tiles, sizeof(uint32_t), hipMemcpyDeviceToHost, s));
	N2_HIP(hipMemcpyAsync(&host[1], tsum + c.n_tiles, sizeof(uint32_t), hipMemcpyDeviceToHost, s));
	N2_HIP(hipStreamSynchronize(s));
	N2_REQUIRE(host[0] < (1u << 29), "n2_marching_cubes_count: %u vertices exceed the 2^29 limit", host[0]);
	*n_vertices = host[0];
	*n_triangles = host[1];
	return N2_OK;
}

N2_API int n2_marching_cubes_emit(n2_stream_t stream, const uint32_t res[3], const float aabb_min[3], const float aabb_max[3], float thresh,
                                  const float* d_density, void* d_workspace, float* d_vertices, uint32_t* d_indices, float* d_normals,
                                  uint32_t n_vertices, uint32_t n_triangles) {
	uint64_t n;
	if (int rc = mc_check("n2_marching_cubes_emit", res, n)) return rc;
	N2_REQUIRE(d_density && d_workspace && aabb_min && aabb_max, "n2_marching_cubes_emit: null argument");
	N2_REQUIRE((d_vertices || n_vertices == 0) && (d_indices || n_triangles == 0), "n2_marching_cubes_emit: null output");
	hipStream_t s = n2_stream(stream);
	const McCarve c = mc_carve(n);
	unsigned char* b = reinterpret_cast<unsigned char*>(d_workspace);
	uint32_t* voff = reinterpret_cast<uint32_t*>(b + c.voff);
	const uint32_t* vsum = reinterpret_cast<const uint32_t*>(b + c.vsum);
	const uint32_t* tsum = reinterpret_cast<const uint32_t*>(b + c.tsum);
	const McTable* table = reinterpret_cast<const McTable*>(b + c.table);
	N2_REQUIRE(d_normals == nullptr || reinterpret_cast<uintptr_t>(d_normals) % 16 == 0, "n2_marching_cubes_emit: d_normals must be 16-byte aligned");
	const McGrid g = mc_grid(res, aabb_min, aabb_max, thresh);
	if (n_vertices) {
		mc_vertices_kernel<<<mc_emit_grid(c.n_tiles), dim3(MC_BLOCK), 0, s>>>(g, d_density, c.n_tiles, vsum, b + c.busy, voff, d_vertices);
		N2_LAUNCH_CHECK();
	}
	if (n_triangles) {
		mc_faces_kernel<<<mc_emit_grid(c.n_tiles), dim3(MC_BLOCK), 0, s>>>(g, table, d_density, c.n_tiles, tsum, b + c.busy, voff, d_indices);
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
		// the fused kernel forms the lattice points itself; other fields get them written out
		N2Lattice lat;
		for (int d = 0; d < 3; ++d) { lat.res[d] = res[d]; lat.inv_res[d] = 1.f / (float)res[d]; lat.extent[d] = g.scale[d]; lat.corner[d] = g.offset[d]; }
		lat.first = (uint32_t)first; lat.total = (uint32_t)n;
		if (n < (1ull << 32) && n2_field_sdf_row0_lattice(field, stream, lat, m8, m, d_density + first, &rc)) continue;
		mc_lattice_positions_kernel<<<mgrid(m8), dim3(MC_BLOCK), 0, s>>>(g, first, m, m8, positions);
		// the padded tail of the last chunk (m8 - m points at most 7) is evaluated but not kept
		rc = n2_field_sdf_row0(field, stream, positions, 3, 1, m8, m, d_density + first, reinterpret_cast<n2_half*>(mlp_out));
	}
	n2_grid_set_point_order(n2_field_encoding(field), 0);
	if (rc != N2_OK) return rc;
	N2_LAUNCH_CHECK();
	return N2_OK;
}
