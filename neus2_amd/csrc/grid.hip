// Multi-resolution hash grid encoding for gfx950: forward, backward
// (parameter scatter + input gradient) and the second-order
// backward_backward_input, behind the n2_grid_* C ABI.
//
// Work decomposition: one workgroup handles a tile of points for ONE level.
// The gather kernels number their (level, tile) work items level-major and cut
// that list into 8 contiguous pieces of equal estimated cost, one per XCD: the
// hardware deals consecutive workgroup ids round-robin over the 8 XCDs, so
// workgroup id b runs on XCD b % 8 and takes item number b / 8 of that XCD's
// piece.  Each XCD then streams all points through about two levels, and its
// private 4 MiB L2 fetches only those levels' tables (<= 2 MiB each at
// T = 2^19) instead of all 24 MiB.  (With plain level-major ids every XCD
// walks every level and the table crosses the fabric 8 times per launch.)
#include "n2_common.h"
#include "grid_device.h"
#include "slab_reduce.h"

#include <cmath>
#include <new>

struct n2_grid {
	N2LevelTable tab;
	uint32_t n_features;
	uint32_t n_params;
	const __half2* params;
	__half2* grads;
	// relative cost of one tile of each level (balances the levels over the XCDs)
	float level_cost[N2_MAX_LEVELS];
	// progressive training (base_training_step 0: off)
	float base_valid_level_scale, valid_level_scale;
	uint32_t base_training_step;
	uint32_t training_step;  // as last told by n2_grid_set_training_step
	// optional scratch of the bucketed scatter
	unsigned char* ws;
	uint64_t ws_bytes;
	uint32_t ws_max_points;
	bool lattice_order;  // points of the next forwards come in lattice order (n2_grid_set_point_order)
};

struct N2Point {
	float w[3];
	uint32_t c[3];
};

__device__ __forceinline__ N2Point n2_load_point(const float* __restrict__ xyz, uint32_t point_stride, uint32_t dim_stride,
                                                 uint32_t i, float scale) {
	N2Point p;
	const float* q = xyz + (size_t)i * point_stride;
#pragma unroll
	for (int d = 0; d < 3; ++d) n2_locate(q[(size_t)d * dim_stride], scale, p.w[d], p.c[d]);
	return p;
}

template <uint32_t MODE>
__device__ __forceinline__ void n2_corner_entries(const N2Point& p, uint32_t entries, uint32_t res, uint32_t e[8]) {
#pragma unroll
	for (uint32_t k = 0; k < 8; ++k) {
		e[k] = n2_entry<MODE>(entries, res, p.c[0] + (k & 1u), p.c[1] + ((k >> 1) & 1u), p.c[2] + ((k >> 2) & 1u));
	}
}

__device__ __forceinline__ float n2_corner_weight(const N2Point& p, uint32_t k) {
	float wt = (k & 1u) ? p.w[0] : 1.f - p.w[0];
	wt *= (k & 2u) ? p.w[1] : 1.f - p.w[1];
	wt *= (k & 4u) ? p.w[2] : 1.f - p.w[2];
	return wt;
}

#define N2_DISPATCH_MODE(mode, CALL)                        \
	switch (mode) {                                         \
		case N2_LEVEL_DENSE: { CALL(N2_LEVEL_DENSE); } break;       \
		case N2_LEVEL_HASH: { CALL(N2_LEVEL_HASH); } break;         \
		case N2_LEVEL_DENSE_MOD: { CALL(N2_LEVEL_DENSE_MOD); } break; \
		default: { CALL(N2_LEVEL_HASH_MOD); } break;                \
	}

constexpr uint32_t GRID_BLOCK = 256;
constexpr uint32_t N_XCD = 8;  // gfx950: 8 XCDs, workgroup ids are dealt round-robin

// Piece x of the level-major item list [begin[x], begin[x + 1]) belongs to XCD x.
struct N2XcdPlan {
	uint32_t begin[N_XCD + 1];
};

// The (level, tile) item of this workgroup, or false if its XCD's piece is shorter than the longest one.
__device__ __forceinline__ bool n2_xcd_item(const N2XcdPlan& plan, uint32_t tiles, uint32_t& level, uint32_t& tile) {
	const uint32_t xcd = blockIdx.x % N_XCD, item = plan.begin[xcd] + blockIdx.x / N_XCD;
	if (item >= plan.begin[xcd + 1]) return false;
	level = item / tiles;
	tile = item - level * tiles;
	return true;
}

// ----------------------------------------------------------------------------
// forward
// ----------------------------------------------------------------------------
// A point is handled by a PAIR of adjacent lanes: lane bit 0 selects the x corner, each lane gathers the four
// (y, z) corners of its x.  The two x corners are neighbours in the table (dense levels: index + 1; hashed
// levels: x enters the hash with prime 1), so the two lanes of a pair read the same cache line almost always and
// the memory pipeline, which looks up one line per clock, sees half as many lines per point.  The pair then
// exchanges its partial sums and lane b finishes feature b.
constexpr uint32_t FWD_POINTS = GRID_BLOCK / 2;  // points per workgroup and level

// value held by the other lane of the pair (lane ^ 1): a quad permute [1, 0, 3, 2] inside the VALU, no LDS crossbar
__device__ __forceinline__ float n2_pair_swap(float x) {
	return __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, x), 0xB1, 0xF, 0xF, true));
}

template <uint32_t MODE, bool WANT_DYDX>
__device__ __forceinline__ void grid_forward_pair(const N2LevelTable& tab, uint32_t level, uint32_t i, uint32_t b, uint32_t N,
                                                  const float* __restrict__ xyz, uint32_t point_stride, uint32_t dim_stride,
                                                  const __half2* __restrict__ params, __half* __restrict__ out,
                                                  float* __restrict__ dy_dx) {
	const float scale = tab.scale[level];
	const uint32_t entries = tab.entries[level], res = tab.resolution[level];
	const __half2* P = params + tab.offset[level];
	const size_t row = (size_t)level * 2 + b;
	if (n2_level_masked(tab, level, i)) {  // both lanes of a pair share i
		out[row * N + i] = __float2half_rn(0.f);
		if (WANT_DYDX) {
			float* j = dy_dx + (row * N + i) * 3;
			j[0] = 0.f; j[1] = 0.f; j[2] = 0.f;
		}
		return;
	}
	const N2Point p = n2_load_point(xyz, point_stride, dim_stride, i, scale);
	const uint32_t gx = p.c[0] + b;
	float2 v[4];
#pragma unroll
	for (uint32_t k = 0; k < 4; ++k) v[k] = __half22float2(P[n2_entry<MODE>(entries, res, gx, p.c[1] + (k & 1u), p.c[2] + (k >> 1))]);
	const float wy = p.w[1], wz = p.w[2], uy = 1.f - wy, uz = 1.f - wz;
	// this lane's x plane: bilinear value s, and its y and z differences ty, tz (k = y + 2 z)
	float2 s, ty, tz;
	s.x = fmaf(uy * uz, v[0].x, fmaf(wy * uz, v[1].x, fmaf(uy * wz, v[2].x, wy * wz * v[3].x)));
	s.y = fmaf(uy * uz, v[0].y, fmaf(wy * uz, v[1].y, fmaf(uy * wz, v[2].y, wy * wz * v[3].y)));
	if (WANT_DYDX) {
		ty.x = fmaf(uz, v[1].x - v[0].x, wz * (v[3].x - v[2].x));
		ty.y = fmaf(uz, v[1].y - v[0].y, wz * (v[3].y - v[2].y));
		tz.x = fmaf(uy, v[2].x - v[0].x, wy * (v[3].x - v[1].x));
		tz.y = fmaf(uy, v[2].y - v[0].y, wy * (v[3].y - v[1].y));
	}
	// lane b keeps feature b of its own plane and receives feature b of the partner's plane
	const float s_mine = b ? s.y : s.x, s_other = n2_pair_swap(b ? s.x : s.y);
	const float s_lo = b ? s_other : s_mine, s_hi = b ? s_mine : s_other;  // x corner 0 / 1
	const float wx = p.w[0], ux = 1.f - wx;
	out[row * N + i] = __float2half_rn(fmaf(ux, s_lo, wx * s_hi));
	if (WANT_DYDX) {
		const float ty_mine = b ? ty.y : ty.x, ty_other = n2_pair_swap(b ? ty.x : ty.y);
		const float tz_mine = b ? tz.y : tz.x, tz_other = n2_pair_swap(b ? tz.x : tz.y);
		const float w_mine = b ? wx : ux, w_other = b ? ux : wx;
		float* j = dy_dx + (row * N + i) * 3;
		j[0] = (s_hi - s_lo) * scale;
		j[1] = fmaf(w_mine, ty_mine, w_other * ty_other) * scale;
		j[2] = fmaf(w_mine, tz_mine, w_other * tz_other) * scale;
	}
}

template <bool WANT_DYDX>
__global__ void __launch_bounds__(GRID_BLOCK) grid_forward_kernel(N2LevelTable tab, N2XcdPlan plan, uint32_t N, uint32_t tiles,
                                                                  const float* __restrict__ xyz, uint32_t point_stride,
                                                                  uint32_t dim_stride, const __half2* __restrict__ params,
                                                                  __half* __restrict__ out, float* __restrict__ dy_dx) {
	uint32_t level, tile;
	if (!n2_xcd_item(plan, tiles, level, tile)) return;
	const uint32_t i = tile * FWD_POINTS + (threadIdx.x >> 1), b = threadIdx.x & 1u;
	if (i >= N) return;  // both lanes of a pair share i, so pairs leave together
#define CALL(M) grid_forward_pair<M, WANT_DYDX>(tab, level, i, b, N, xyz, point_stride, dim_stride, params, out, dy_dx)
	N2_DISPATCH_MODE(tab.mode[level], CALL)
#undef CALL
}

// One lane per (point, level): eight gathers and one fused multiply-add chain per feature.  For points that arrive
// in lattice order (neighbouring lanes in neighbouring cells) the gathers hit lines the wave has just fetched and
// the kernel is bound by instruction issue, where the lane pairs of the kernel above cost twice the lanes.
template <uint32_t MODE>
__device__ __forceinline__ void grid_forward_point(const N2LevelTable& tab, uint32_t level, uint32_t i, uint32_t N,
                                                   const float* __restrict__ xyz, uint32_t point_stride, uint32_t dim_stride,
                                                   const __half2* __restrict__ params, __half* __restrict__ out) {
	const size_t row = (size_t)level * 2;
	if (n2_level_masked(tab, level, i)) {
		out[row * N + i] = __float2half_rn(0.f);
		out[(row + 1) * N + i] = __float2half_rn(0.f);
		return;
	}
	const __half2* P = params + tab.offset[level];
	const N2Point p = n2_load_point(xyz, point_stride, dim_stride, i, tab.scale[level]);
	uint32_t e[8];
	n2_corner_entries<MODE>(p, tab.entries[level], tab.resolution[level], e);
	float2 v[8];
#pragma unroll
	for (uint32_t k = 0; k < 8; ++k) v[k] = __half22float2(P[e[k]]);
	float a0 = 0.f, a1 = 0.f;
#pragma unroll
	for (uint32_t k = 0; k < 8; ++k) {
		const float wt = n2_corner_weight(p, k);
		a0 = fmaf(wt, v[k].x, a0);
		a1 = fmaf(wt, v[k].y, a1);
	}
	out[row * N + i] = __float2half_rn(a0);
	out[(row + 1) * N + i] = __float2half_rn(a1);
}

__global__ void __launch_bounds__(GRID_BLOCK) grid_forward_point_kernel(N2LevelTable tab, uint32_t N, uint32_t tiles,
                                                                        const float* __restrict__ xyz, uint32_t point_stride,
                                                                        uint32_t dim_stride, const __half2* __restrict__ params,
                                                                        __half* __restrict__ out) {
	// level-major workgroup ids, dealt round-robin over the XCDs: every XCD sees an eighth of the tiles of every level.
	// (Giving whole levels to an XCD, as the scattered-point kernel does, makes every XCD stream all positions and
	// nearly doubles the time of a lattice chunk: with coherent points the tables' hot lines fit every L2 anyway.)
	const uint32_t level = blockIdx.x / tiles, tile = blockIdx.x - level * tiles;
	const uint32_t i = tile * GRID_BLOCK + threadIdx.x;
	if (i >= N) return;
#define CALL(M) grid_forward_point<M>(tab, level, i, N, xyz, point_stride, dim_stride, params, out)
	N2_DISPATCH_MODE(tab.mode[level], CALL)
#undef CALL
}

// ----------------------------------------------------------------------------
// corner indices (test hook of the bit-exact contract)
// ----------------------------------------------------------------------------
__global__ void __launch_bounds__(GRID_BLOCK) grid_indices_kernel(N2LevelTable tab, uint32_t N, uint32_t tiles,
                                                                  const float* __restrict__ xyz, uint32_t point_stride,
                                                                  uint32_t dim_stride, uint32_t* __restrict__ idx) {
	const uint32_t level = blockIdx.x / tiles;
	const uint32_t i = (blockIdx.x - level * tiles) * GRID_BLOCK + threadIdx.x;
	if (i >= N) return;
	const N2Point p = n2_load_point(xyz, point_stride, dim_stride, i, tab.scale[level]);
	uint32_t e[8];
#define CALL(M) n2_corner_entries<M>(p, tab.entries[level], tab.resolution[level], e)
	N2_DISPATCH_MODE(tab.mode[level], CALL)
#undef CALL
#pragma unroll
	for (uint32_t k = 0; k < 8; ++k) idx[((size_t)level * 8 + k) * N + i] = e[k];
}

// ----------------------------------------------------------------------------
// backward: parameter scatter (packed fp16 atomics), first and second order in
// one pass.
//
// Atomics retire at a fixed rate per REQUEST, and lanes of one instruction that
// hit the same 8 bytes travel as one request.  Corners that differ only in x
// are neighbours in the table (dense levels: index + 1; hashed levels: the x
// term enters the hash with prime 1, so even x and x+1 differ in bit 0 only).
// A point is therefore handled by a PAIR of adjacent lanes: lane bit 0 selects
// the x corner, each lane issues the four (y, z) corners.  That halves the
// number of atomic requests against one lane per point.
//
// Per corner c of level l the two contributions are
//   first order   dL_dy[l,f] * weight_c
//   second order  g[l,f] * scale_l * sum_d v_d * s_{c,d} * prod_{d' != d} w_{c,d'}
// and they leave as ONE packed fp16 atomic (one rounding instead of two).
// ----------------------------------------------------------------------------
constexpr uint32_t PAIR_POINTS = GRID_BLOCK / 2;  // points per workgroup and level

template <uint32_t MODE, bool FIRST, bool SECOND, bool WANT_OUT>
__device__ __forceinline__ void grid_scatter_pair(const N2LevelTable& tab, uint32_t level, uint32_t i, uint32_t b, uint32_t N,
                                                  const float* __restrict__ xyz, uint32_t point_stride, uint32_t dim_stride,
                                                  const __half* __restrict__ dL_dy, const float* __restrict__ v,
                                                  const __half* __restrict__ g2, const __half2* __restrict__ params,
                                                  __half2* __restrict__ grads, __half* __restrict__ dL_ddLdy, uint32_t xi, uint32_t Ng) {
	// xi: where this point's position and g2 column stand (i itself unless the call reads them through an index); Ng: columns of g2
	const float scale = tab.scale[level];
	const uint32_t entries = tab.entries[level], res = tab.resolution[level];
	const size_t row = (size_t)level * 2;
	if (n2_level_masked(tab, level, i)) {  // both lanes of a pair share i
		if (SECOND && WANT_OUT) dL_ddLdy[(row + b) * N + i] = __float2half_rn(0.f);
		return;
	}
	const N2Point p = n2_load_point(xyz, point_stride, dim_stride, xi, scale);
	float a0 = 0.f, a1 = 0.f, c0 = 0.f, c1 = 0.f, v0 = 0.f, v1 = 0.f, v2 = 0.f;
	if (FIRST) {
		a0 = __half2float(dL_dy[row * N + i]);
		a1 = __half2float(dL_dy[(row + 1) * N + i]);
	}
	if (SECOND) {
		c0 = __half2float(g2[row * Ng + xi]);
		c1 = __half2float(g2[(row + 1) * Ng + xi]);
		v0 = v[i] * scale; v1 = v[(size_t)N + i] * scale; v2 = v[(size_t)2 * N + i] * scale;
	}
	const bool skip = !SECOND && a0 == 0.f && a1 == 0.f;  // nothing to add (both lanes of a pair agree)
	const float wx = b ? p.w[0] : 1.f - p.w[0];
	const float sx = b ? 1.f : -1.f;
	const uint32_t gx = p.c[0] + b;
	const __half2* P = params + tab.offset[level];
	__half2* G = grads ? grads + tab.offset[level] : nullptr;
	float o0 = 0.f, o1 = 0.f;
#pragma unroll
	for (uint32_t k = 0; k < 4; ++k) {
		const uint32_t y = k & 1u, z = k >> 1;
		const uint32_t e = n2_entry<MODE>(entries, res, gx, p.c[1] + y, p.c[2] + z);
		const float wy = y ? p.w[1] : 1.f - p.w[1], wz = z ? p.w[2] : 1.f - p.w[2];
		float r0 = 0.f, r1 = 0.f;
		if (FIRST) {
			const float wt = wx * wy * wz;
			r0 = a0 * wt;
			r1 = a1 * wt;
		}
		if (SECOND) {
			const float sy = y ? 1.f : -1.f, sz = z ? 1.f : -1.f;
			const float coef = v0 * sx * wy * wz + v1 * sy * wx * wz + v2 * sz * wx * wy;
			r0 = fmaf(c0, coef, r0);
			r1 = fmaf(c1, coef, r1);
			if (WANT_OUT) {
				const float2 val = __half22float2(P[e]);
				o0 = fmaf(coef, val.x, o0);
				o1 = fmaf(coef, val.y, o1);
			}
		}
		if (G && !skip) unsafeAtomicAdd(&G[e], __floats2half2_rn(r0, r1));
	}
	if (SECOND && WANT_OUT) {
		// lane b finishes feature b: it needs the partner's partial sum of that feature
		const float mine = b ? o1 : o0, theirs = n2_pair_swap(b ? o0 : o1);
		dL_ddLdy[(row + b) * N + i] = __float2half_rn(mine + theirs);
	}
}

template <bool FIRST, bool SECOND, bool WANT_OUT>
__global__ void __launch_bounds__(GRID_BLOCK) grid_scatter_kernel(N2LevelTable tab, uint32_t N, uint32_t tiles,
                                                                  const float* __restrict__ xyz, uint32_t point_stride,
                                                                  uint32_t dim_stride, const __half* __restrict__ dL_dy,
                                                                  const float* __restrict__ v, const __half* __restrict__ g2,
                                                                  const __half2* __restrict__ params, __half2* __restrict__ grads,
                                                                  __half* __restrict__ dL_ddLdy, const uint32_t* __restrict__ index, uint32_t n_cols) {
	const uint32_t level = blockIdx.x / tiles;
	const uint32_t i = (blockIdx.x - level * tiles) * PAIR_POINTS + (threadIdx.x >> 1);
	const uint32_t b = threadIdx.x & 1u;
	if (i >= N) return;  // both lanes of a pair share i, so pairs leave together
	const uint32_t xi = index ? min(index[i], n_cols - 1u) : i, Ng = index ? n_cols : N;
#define CALL(M) grid_scatter_pair<M, FIRST, SECOND, WANT_OUT>(tab, level, i, b, N, xyz, point_stride, dim_stride, dL_dy, v, g2, params, grads, dL_ddLdy, xi, Ng)
	N2_DISPATCH_MODE(tab.mode[level], CALL)
#undef CALL
}

// ... and input gradient dL_dx[d][i] = sum_k dL_dy[k][i] * dy_dx[k][i][d]
__global__ void __launch_bounds__(GRID_BLOCK) grid_backward_input_kernel(uint32_t N, uint32_t n_out,
                                                                         const __half* __restrict__ dL_dy,
                                                                         const float* __restrict__ dy_dx,
                                                                         float* __restrict__ dL_dx) {
	const uint32_t i = blockIdx.x * GRID_BLOCK + threadIdx.x;
	if (i >= N) return;
	float r0 = 0.f, r1 = 0.f, r2 = 0.f;
	for (uint32_t k = 0; k < n_out; ++k) {
		const float g = __half2float(dL_dy[(size_t)k * N + i]);
		const float* j = dy_dx + ((size_t)k * N + i) * 3;
		r0 = fmaf(g, j[0], r0);
		r1 = fmaf(g, j[1], r1);
		r2 = fmaf(g, j[2], r2);
	}
	dL_dx[i] = r0;
	dL_dx[(size_t)N + i] = r1;
	dL_dx[(size_t)2 * N + i] = r2;
}

// ----------------------------------------------------------------------------
// second order: gradient of <v, dL_dx> w.r.t. the table, dL_dy and x
// ----------------------------------------------------------------------------
template <uint32_t MODE>
__device__ __forceinline__ void grid_bbi_point(const N2LevelTable& tab, uint32_t level, uint32_t i, uint32_t N,
                                               const float* __restrict__ xyz, uint32_t point_stride, uint32_t dim_stride,
                                               const float* __restrict__ v, const __half* __restrict__ dL_dy,
                                               const __half2* __restrict__ params, __half2* __restrict__ grads,
                                               __half* __restrict__ dL_ddLdy, float* __restrict__ dL_dx) {
	const float scale = tab.scale[level];
	const size_t row = (size_t)level * 2;
	if (n2_level_masked(tab, level, i)) {
		if (dL_ddLdy) {
			dL_ddLdy[row * N + i] = __float2half_rn(0.f);
			dL_ddLdy[(row + 1) * N + i] = __float2half_rn(0.f);
		}
		return;
	}
	const N2Point p = n2_load_point(xyz, point_stride, dim_stride, i, scale);
	uint32_t e[8];
	n2_corner_entries<MODE>(p, tab.entries[level], tab.resolution[level], e);
	const float v0 = v[i] * scale, v1 = v[(size_t)N + i] * scale, v2 = v[(size_t)2 * N + i] * scale;
	const float g0 = __half2float(dL_dy[row * N + i]);
	const float g1 = __half2float(dL_dy[(row + 1) * N + i]);
	const bool need_vals = dL_ddLdy != nullptr || dL_dx != nullptr;
	const __half2* P = params + tab.offset[level];
	__half2* G = grads ? grads + tab.offset[level] : nullptr;
	float o0 = 0.f, o1 = 0.f, dx0 = 0.f, dx1 = 0.f, dx2 = 0.f;
#pragma unroll
	for (uint32_t k = 0; k < 8; ++k) {
		const float w0 = (k & 1u) ? p.w[0] : 1.f - p.w[0];
		const float w1 = (k & 2u) ? p.w[1] : 1.f - p.w[1];
		const float w2 = (k & 4u) ? p.w[2] : 1.f - p.w[2];
		const float s0 = (k & 1u) ? 1.f : -1.f, s1 = (k & 2u) ? 1.f : -1.f, s2 = (k & 4u) ? 1.f : -1.f;
		// sum_d v_d * d(weight_k)/dx_d   (v already carries one factor of scale)
		const float coef = v0 * s0 * w1 * w2 + v1 * s1 * w0 * w2 + v2 * s2 * w0 * w1;
		if (G) unsafeAtomicAdd(&G[e[k]], __floats2half2_rn(g0 * coef, g1 * coef));
		if (need_vals) {
			const float2 val = __half22float2(P[e[k]]);
			o0 = fmaf(coef, val.x, o0);
			o1 = fmaf(coef, val.y, o1);
			if (dL_dx) {
				const float gp = (g0 * val.x + g1 * val.y) * scale;  // second factor of scale
				const float h01 = s0 * s1 * w2, h02 = s0 * s2 * w1, h12 = s1 * s2 * w0;
				dx0 = fmaf(gp, v1 * h01 + v2 * h02, dx0);
				dx1 = fmaf(gp, v0 * h01 + v2 * h12, dx1);
				dx2 = fmaf(gp, v0 * h02 + v1 * h12, dx2);
			}
		}
	}
	if (dL_ddLdy) {
		dL_ddLdy[row * N + i] = __float2half_rn(o0);
		dL_ddLdy[(row + 1) * N + i] = __float2half_rn(o1);
	}
	if (dL_dx) {
		unsafeAtomicAdd(&dL_dx[i], dx0);
		unsafeAtomicAdd(&dL_dx[(size_t)N + i], dx1);
		unsafeAtomicAdd(&dL_dx[(size_t)2 * N + i], dx2);
	}
}

__global__ void __launch_bounds__(GRID_BLOCK) grid_bbi_kernel(N2LevelTable tab, uint32_t N, uint32_t tiles,
                                                              const float* __restrict__ xyz, uint32_t point_stride,
                                                              uint32_t dim_stride, const float* __restrict__ v,
                                                              const __half* __restrict__ dL_dy, const __half2* __restrict__ params,
                                                              __half2* __restrict__ grads, __half* __restrict__ dL_ddLdy,
                                                              float* __restrict__ dL_dx) {
	const uint32_t level = blockIdx.x / tiles;
	const uint32_t i = (blockIdx.x - level * tiles) * GRID_BLOCK + threadIdx.x;
	if (i >= N) return;
#define CALL(M) grid_bbi_point<M>(tab, level, i, N, xyz, point_stride, dim_stride, v, dL_dy, params, grads, dL_ddLdy, dL_dx)
	N2_DISPATCH_MODE(tab.mode[level], CALL)
#undef CALL
}

// ----------------------------------------------------------------------------
// bucketed scatter: parameter gradients WITHOUT global atomics
//
// Global atomics retire at ~2e10 requests/s on this part however they are
// issued, which caps the scatter above at ~55 us per level.  Loads, stores and
// LDS atomics are two orders of magnitude faster, so the scatter is turned
// into a two-kernel counting sort on entry ranges:
//
//  bin     one workgroup per (level, tile of 1024 points): computes the 8192
//          (entry, value) records of the tile, sorts them in LDS by bucket
//          (bucket = entry / 8192, at most 64 per level) and writes the sorted
//          tile (64 KiB, fully coalesced) plus its 65 bucket offsets.
//  reduce  one workgroup per (level, bucket[, tile group]): walks the bucket's
//          run in every tile (contiguous, ~1 KiB each), accumulates in an LDS
//          table of 8192 fp32 pairs with LDS atomics, and writes the bucket's
//          entries with plain stores.  Coarse levels have few buckets, so their
//          work is split over tile groups and folded with (few, contention-free)
//          global atomics.
// Accumulation is fp32 until the single rounding to fp16 at the store, which
// also removes the rounding drift of chained fp16 atomics.
// ----------------------------------------------------------------------------
#ifndef N2_BKT_SHIFT
#define N2_BKT_SHIFT 12
#endif
constexpr uint32_t BKT_SHIFT = N2_BKT_SHIFT;           // 4096 entries per bucket: a 64 KiB accumulator image, two reduce workgroups per CU
constexpr uint32_t BKT_ENTRIES = 1u << BKT_SHIFT;
constexpr uint32_t BKT_MAX = (1u << 19) >> BKT_SHIFT;  // buckets per level (entries <= 2^19)
constexpr uint32_t BKT_MIN_SHIFT = 5;                  // smallest bucket of a level that chooses its own size (N2LevelTable::bucket_shift)
constexpr uint32_t PAIR_MAX_CELL = BKT_ENTRIES - 2u;  // pair records (grid_bin_kernel): x + 1 <= BKT_ENTRIES - 1
static_assert(BKT_SHIFT <= 12, "a pair record's 16-bit key holds the entry within the bucket and four bits of carry length");
constexpr uint32_t BIN_POINTS = 1024;    // points per bin workgroup
constexpr uint32_t BIN_RECORDS = BIN_POINTS * 8;
constexpr uint32_t BIN_BLOCK = 512;       // 8 waves: three workgroups (3 x 49 KiB of LDS) keep 6 waves on every SIMD, at 80 registers (with 96 or 128: pair +10 us)
constexpr uint32_t BIN_PER_THREAD = BIN_POINTS / BIN_BLOCK;  // 2

struct N2BucketPlan {
	uint32_t wg_begin[N2_MAX_LEVELS + 1];  // first reduce workgroup of each level
	uint32_t n_buckets[N2_MAX_LEVELS];
	uint32_t groups[N2_MAX_LEVELS];        // tile groups per bucket
	// levels whose buckets are split over several workgroups (groups > 1): where the level's partial images start (images:
	// bucket-major, then group) and the number of split buckets in the levels below
	uint32_t part_begin[N2_MAX_LEVELS];
	uint32_t split_begin[N2_MAX_LEVELS + 1];
};

template <uint32_t MODE, bool FIRST, bool SECOND, bool WANT_OUT, bool CLAMP_X>
__device__ __forceinline__ void grid_bin_point(const N2LevelTable& tab, uint32_t level, uint32_t i, uint32_t N,
                                               const float* __restrict__ xyz, uint32_t point_stride, uint32_t dim_stride,
                                               const __half* __restrict__ dL_dy, const float* __restrict__ v,
                                               const __half* __restrict__ g2, const __half2* __restrict__ params,
                                               __half* __restrict__ dL_ddLdy, uint32_t* e_out, float* r0_out, float* r1_out,
                                               uint32_t* cell, uint32_t xi, uint32_t Ng) {
	const float scale = tab.scale[level];
	N2Point p = n2_load_point(xyz, point_stride, dim_stride, xi, scale);
	if (CLAMP_X) p.c[0] = min(p.c[0], PAIR_MAX_CELL);  // pair records: x + 1 stays inside the bucket's index bits
	cell[0] = p.c[0]; cell[1] = p.c[1]; cell[2] = p.c[2];
	uint32_t e[8];
	n2_corner_entries<MODE>(p, tab.entries[level], tab.resolution[level], e);
	const size_t row = (size_t)level * 2;
	float a0 = 0.f, a1 = 0.f, c0 = 0.f, c1 = 0.f, v0 = 0.f, v1 = 0.f, v2 = 0.f;
	if (FIRST) {
		a0 = __half2float(dL_dy[row * N + i]);
		a1 = __half2float(dL_dy[(row + 1) * N + i]);
	}
	if (SECOND) {
		c0 = __half2float(g2[row * Ng + xi]);
		c1 = __half2float(g2[(row + 1) * Ng + xi]);
		v0 = v[i] * scale; v1 = v[(size_t)N + i] * scale; v2 = v[(size_t)2 * N + i] * scale;
	}
	const __half2* P = params + tab.offset[level];
	float o0 = 0.f, o1 = 0.f;
	// Corner k = i + 2 j + 4 l has weight X_i Y_j Z_l and signs (sx_i, sy_j, sz_l).  Its record is
	//   a X Y Z + c (v0 sx Y Z + v1 sy X Z + v2 sz X Y)  =  (Y Z) (a X + c v0 sx) + (c X) (v1 sy Z + v2 sz Y),
	// so the eight corners share two x terms per feature and four (y, z) terms.
	const float X[2] = {1.f - p.w[0], p.w[0]}, Y[2] = {1.f - p.w[1], p.w[1]}, Z[2] = {1.f - p.w[2], p.w[2]};
	float Pyz[4], Qyz[4], A0[2], A1[2], B0[2] = {0.f, 0.f}, B1[2] = {0.f, 0.f};
#pragma unroll
	for (uint32_t jl = 0; jl < 4; ++jl) {
		const uint32_t j = jl & 1u, l = jl >> 1;
		Pyz[jl] = Y[j] * Z[l];
		Qyz[jl] = SECOND ? (j ? v1 : -v1) * Z[l] + (l ? v2 : -v2) * Y[j] : 0.f;
	}
#pragma unroll
	for (uint32_t ix = 0; ix < 2; ++ix) {
		const float sv = ix ? v0 : -v0;
		A0[ix] = FIRST ? fmaf(a0, X[ix], c0 * sv) : c0 * sv;
		A1[ix] = FIRST ? fmaf(a1, X[ix], c1 * sv) : c1 * sv;
		if (SECOND) { B0[ix] = c0 * X[ix]; B1[ix] = c1 * X[ix]; }
	}
#pragma unroll
	for (uint32_t k = 0; k < 8; ++k) {
		const uint32_t ix = k & 1u, jl = k >> 1;
		float r0 = Pyz[jl] * A0[ix], r1 = Pyz[jl] * A1[ix];
		if (SECOND) {
			r0 = fmaf(B0[ix], Qyz[jl], r0);
			r1 = fmaf(B1[ix], Qyz[jl], r1);
			if (WANT_OUT) {
				const float coef = fmaf(ix ? v0 : -v0, Pyz[jl], X[ix] * Qyz[jl]);
				const float2 val = __half22float2(P[e[k]]);
				o0 = fmaf(coef, val.x, o0);
				o1 = fmaf(coef, val.y, o1);
			}
		}
		e_out[k] = e[k];
		r0_out[k] = r0;
		r1_out[k] = r1;
	}
	if (SECOND && WANT_OUT) {
		dL_ddLdy[row * N + i] = __float2half_rn(o0);
		dL_ddLdy[(row + 1) * N + i] = __float2half_rn(o1);
	}
}

// Samples arrive in ray order, so on the coarser levels consecutive samples (= consecutive lanes)
// fall into the same cell and would hit the same eight entries.  When runs of equal cells are long
// enough (at most MERGE_MAX_HEADS runs in a wave), they are summed across lanes in fp32 and only the
// last lane of a run emits records: fewer records, and no pile-up on a few hot entries in the sort's
// counters or the reduce's accumulators.  The sums are segmented scans inside rows of 16 lanes, which
// the data-parallel-primitive lane shifts do at full ALU rate without touching LDS; a run that
// crosses a row boundary simply emits one record per row.
constexpr uint32_t MERGE_MAX_HEADS = 52;  // measured on the training step: 16: +16 us for the scatter pair, 24: +6, 32: +1, 40: +2 against 48 .. 58
constexpr unsigned long long ROW_HEADS = 0x0001000100010001ull;  // first lane of each 16-lane row

// value of the lane D places below in the same 16-lane row (0 if that leaves the row)
template <int D>
__device__ __forceinline__ float n2_row_shr(float x) {
	return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(x), 0x110 + D, 0xf, 0xf, true));  // lanes without a source read 0
}
constexpr uint32_t REC_SKIP = 0xFFFFFFFFu;

// Pair records.  On a hashed level the entry of corner (x, y, z) is (x ^ y P1 ^ z P2) & (T - 1); while x + 1 stays below
// the bucket size, x only reaches the bits below BKT_SHIFT: the two x-neighbours of a (y, z) corner pair always share a
// bucket, and their places in it differ by x ^ (x + 1) = 2^(t+1) - 1, t = number of trailing one bits of x.  Such levels
// (pair_levels in the level table) sort and store ONE record per pair: both packed values (8 bytes) and a 16-bit key,
// entry of the x corner within the bucket | t << BKT_SHIFT.  Half the counter updates, prefix look-ups and staging
// stores here, half the key traffic and decoding in the reduce kernel.  Points outside the unit cube could carry an x
// beyond that range: their cell is clamped for the records (the dense levels clamp such points too).

template <bool FIRST, bool SECOND, bool WANT_OUT, bool PAIR>
__device__ __forceinline__ void grid_bin_tile(const N2LevelTable& tab, const uint32_t level, const uint32_t tile, uint32_t N, uint32_t tiles,
                                              const float* __restrict__ xyz, uint32_t point_stride, uint32_t dim_stride,
                                              const __half* __restrict__ dL_dy, const float* __restrict__ v, const __half* __restrict__ g2,
                                              const __half2* __restrict__ params, __half* __restrict__ dL_ddLdy,
                                              uint32_t* __restrict__ rec_vals, uint16_t* __restrict__ rec_keys, uint16_t* __restrict__ offsets,
                                              uint32_t* hist, uint32_t* prefix, uint32_t* stage_val, uint16_t* stage_key,
                                              const uint32_t* __restrict__ index, uint32_t n_cols) {
	constexpr uint32_t R = PAIR ? 4 : 8;  // sorted records per point
	const uint32_t lane = threadIdx.x & 63u;
	const uint32_t shift = PAIR ? BKT_SHIFT : (uint32_t)tab.bucket_shift[level], in_bucket = (1u << shift) - 1u;
	// records of this thread: entry | rank << 19 after the counting step (REC_SKIP: merged into a later lane)
	uint32_t re[BIN_PER_THREAD * R], rv[BIN_PER_THREAD * 8], tcode[BIN_PER_THREAD];
#pragma unroll
	for (uint32_t j = 0; j < BIN_PER_THREAD; ++j) {
		const uint32_t i = tile * BIN_POINTS + j * BIN_BLOCK + threadIdx.x;
		bool valid = i < N;
		if (valid && n2_level_masked(tab, level, i)) {  // a switched-off level: no records, zero second-order output
			valid = false;
			if (SECOND && WANT_OUT) {
				dL_ddLdy[(size_t)level * 2 * N + i] = __float2half_rn(0.f);
				dL_ddLdy[((size_t)level * 2 + 1) * N + i] = __float2half_rn(0.f);
			}
		}
		uint32_t e[8], cell[3] = {0, 0, 0};
		float r0[8], r1[8];
#pragma unroll
		for (uint32_t k = 0; k < 8; ++k) { e[k] = 0; r0[k] = 0.f; r1[k] = 0.f; }
		if (valid) {
			// positions and g2 columns may be read through an index (see n2_grid_backward_fused_indexed)
			const uint32_t xi = index ? min(index[i], n_cols - 1u) : i, Ng = index ? n_cols : N;
			if (PAIR) {
				grid_bin_point<N2_LEVEL_HASH, FIRST, SECOND, WANT_OUT, true>(tab, level, i, N, xyz, point_stride, dim_stride, dL_dy, v, g2, params, dL_ddLdy, e, r0, r1, cell, xi, Ng);
			} else {
#define CALL(M) grid_bin_point<M, FIRST, SECOND, WANT_OUT, false>(tab, level, i, N, xyz, point_stride, dim_stride, dL_dy, v, g2, params, dL_ddLdy, e, r0, r1, cell, xi, Ng)
				N2_DISPATCH_MODE(tab.mode[level], CALL)
#undef CALL
			}
		}
		// runs of equal cells among the wave's 64 consecutive points
		const uint32_t up_x = __shfl_up(cell[0], 1), up_y = __shfl_up(cell[1], 1), up_z = __shfl_up(cell[2], 1);
		const int up_valid = __shfl_up((int)valid, 1);
		const bool head = lane == 0 || !valid || !up_valid || cell[0] != up_x || cell[1] != up_y || cell[2] != up_z;
		const unsigned long long heads = __ballot(head) | ROW_HEADS;
		bool emit = valid;
		if (__popcll(heads) <= MERGE_MAX_HEADS) {
			// first lane of this lane's run (same row), and whether the next lane starts a new one
			const uint32_t start = 63u - (uint32_t)__clzll(heads & (~0ull >> (63u - lane)));
			emit = valid && (lane == 63u || ((heads >> (lane + 1u)) & 1ull));
			const uint32_t depth = lane - start;  // lanes of the run below this one
#define N2_SCAN_STEP(D)                                               \
			{                                                         \
				const float take = depth >= D ? 1.f : 0.f;            \
				_Pragma("unroll") for (uint32_t k = 0; k < 8; ++k) {  \
					r0[k] = fmaf(n2_row_shr<D>(r0[k]), take, r0[k]);  \
					r1[k] = fmaf(n2_row_shr<D>(r1[k]), take, r1[k]);  \
				}                                                     \
			}
			N2_SCAN_STEP(1) N2_SCAN_STEP(2) N2_SCAN_STEP(4) N2_SCAN_STEP(8)
#undef N2_SCAN_STEP
		}
		if (PAIR) tcode[j] = ((uint32_t)__popc((e[0] ^ e[1]) & (BKT_ENTRIES - 1u)) - 1u) << BKT_SHIFT;
#pragma unroll
		for (uint32_t k = 0; k < 8; ++k) {
			if (!PAIR || (k & 1u) == 0) {
				uint32_t rec = REC_SKIP;
				if (emit) {
					const uint32_t rank = atomicAdd(&hist[e[k] >> shift], 1u);
					rec = e[k] | (rank << 19);
				}
				re[R * j + (PAIR ? k >> 1 : k)] = rec;
			}
			const __half2 h = __floats2half2_rn(r0[k], r1[k]);
			rv[8 * j + k] = *reinterpret_cast<const uint32_t*>(&h);
		}
	}
	__syncthreads();
	if (threadIdx.x < 64) {  // one wave scans the counters, BKT_MAX / 64 consecutive ones per lane
		constexpr uint32_t PER = BKT_MAX / 64;
		uint32_t c[PER], s = 0;
#pragma unroll
		for (uint32_t q = 0; q < PER; ++q) { c[q] = hist[threadIdx.x * PER + q]; s += c[q]; }
		const uint32_t own = s;
#pragma unroll
		for (int o = 1; o < 64; o <<= 1) {
			const uint32_t u = __shfl_up(s, o);
			if ((int)threadIdx.x >= o) s += u;
		}
		uint32_t run = s - own;
#pragma unroll
		for (uint32_t q = 0; q < PER; ++q) { prefix[threadIdx.x * PER + q] = run; run += c[q]; }
		if (threadIdx.x == 63) prefix[BKT_MAX] = s;
	}
	__syncthreads();
#pragma unroll
	for (uint32_t j = 0; j < BIN_PER_THREAD; ++j) {
#pragma unroll
		for (uint32_t k = 0; k < R; ++k) {
			if (re[R * j + k] != REC_SKIP) {
				const uint32_t e = re[R * j + k] & 0x7FFFFu, rank = re[R * j + k] >> 19;
				const uint32_t pos = prefix[e >> shift] + rank;
				if (PAIR) {
					reinterpret_cast<uint2*>(stage_val)[pos] = make_uint2(rv[8 * j + 2 * k], rv[8 * j + 2 * k + 1]);
					stage_key[pos] = (uint16_t)((e & (BKT_ENTRIES - 1u)) | tcode[j]);
				} else {
					stage_val[pos] = rv[8 * j + k];
					stage_key[pos] = (uint16_t)(e & in_bucket);
				}
			}
		}
	}
	__syncthreads();
	const uint32_t total = prefix[BKT_MAX];
	// 16 bytes per lane; the last store of each array may run past `total` inside the tile's own slot, which nobody reads
	const size_t slot = ((size_t)level * tiles + tile) * BIN_RECORDS;
	uint4* out_val = reinterpret_cast<uint4*>(rec_vals + slot);
	uint4* out_key = reinterpret_cast<uint4*>(rec_keys + slot);
	const uint4* sv = reinterpret_cast<const uint4*>(stage_val);
	const uint4* sk = reinterpret_cast<const uint4*>(stage_key);
	for (uint32_t t = threadIdx.x; (PAIR ? 2 : 4) * t < total; t += BIN_BLOCK) out_val[t] = sv[t];
	for (uint32_t t = threadIdx.x; 8 * t < total; t += BIN_BLOCK) out_key[t] = sk[t];
	if (threadIdx.x <= BKT_MAX) offsets[((size_t)level * tiles + tile) * (BKT_MAX + 1) + threadIdx.x] = (uint16_t)prefix[threadIdx.x];
}

template <bool FIRST, bool SECOND, bool WANT_OUT>
__global__ void __launch_bounds__(BIN_BLOCK, 6) grid_bin_kernel(N2LevelTable tab, uint32_t first_level, uint32_t N, uint32_t tiles,
                                                              const float* __restrict__ xyz, uint32_t point_stride,
                                                              uint32_t dim_stride, const __half* __restrict__ dL_dy,
                                                              const float* __restrict__ v, const __half* __restrict__ g2,
                                                              const __half2* __restrict__ params, __half* __restrict__ dL_ddLdy,
                                                              uint32_t* __restrict__ rec_vals, uint16_t* __restrict__ rec_keys,
                                                              uint16_t* __restrict__ offsets,
                                                              const uint32_t* __restrict__ index, uint32_t n_cols) {
	__shared__ uint32_t hist[BKT_MAX];
	__shared__ uint32_t prefix[BKT_MAX + 1];
	__shared__ __align__(16) uint32_t stage_val[BIN_RECORDS];  // sorted records: packed half2 value (a pair of them on pair levels) ...
	__shared__ __align__(16) uint16_t stage_key[BIN_RECORDS];  // ... and entry within its bucket
	const uint32_t level = first_level + blockIdx.x / tiles, tile = blockIdx.x % tiles;
	if (threadIdx.x < BKT_MAX) hist[threadIdx.x] = 0;
	__syncthreads();
	if ((tab.pair_levels >> level) & 1u)
		grid_bin_tile<FIRST, SECOND, WANT_OUT, true>(tab, level, tile, N, tiles, xyz, point_stride, dim_stride, dL_dy, v, g2, params, dL_ddLdy, rec_vals,
		                                             rec_keys, offsets, hist, prefix, stage_val, stage_key, index, n_cols);
	else
		grid_bin_tile<FIRST, SECOND, WANT_OUT, false>(tab, level, tile, N, tiles, xyz, point_stride, dim_stride, dL_dy, v, g2, params, dL_ddLdy, rec_vals,
		                                              rec_keys, offsets, hist, prefix, stage_val, stage_key, index, n_cols);
}

// LDS float atomics retire about one lane every three clocks on this part, integer ones at ~9 (32-bit) and
// ~5.5 (64-bit) lanes per clock.  The reduce therefore accumulates in 64-bit fixed point: a record holds
// fp16 values, i.e. multiples of 2^-24 below 2^16, so value * 2^32 is an exact integer below 2^48 and the
// sum of a whole bucket stays far inside 64 bits.  The accumulation is exact and independent of order.
constexpr uint32_t RED_BLOCK = 1024;              // 16 waves; two workgroups share a CU
constexpr uint32_t RED_ITEMS = 2;                 // items a wave has in flight per fetch
constexpr uint32_t ITEM_SHIFT = 7;                // a run is cut into items of 128 records
constexpr uint32_t ITEM_RECORDS = 1u << ITEM_SHIFT;
constexpr uint32_t ITEM_LOADS = ITEM_RECORDS / 64;  // loads per lane and item
constexpr uint32_t ITEM_CAP = 2048;               // items listed in LDS at a time
constexpr float FIX_SCALE = 4294967296.0f;        // 2^32

// x * 2^32 as a two's complement 64-bit integer, for |x| < 2^31 with at most 24 significant bits (any fp16 value):
// the high word is floor(x), the low word fract(x) * 2^32, both exact.  Five ALU operations instead of the generic
// float -> int64 sequence.
__device__ __forceinline__ unsigned long long to_fixed(float x) {
	const float fl = floorf(x);
	const uint32_t hi = (uint32_t)(int32_t)fl, lo = (uint32_t)((x - fl) * FIX_SCALE);
	return ((unsigned long long)hi << 32) | lo;
}
__device__ __forceinline__ float from_fixed(unsigned long long q) { return (float)((double)(long long)q * (1.0 / 4294967296.0)); }

// Pair levels: an item is 16 pair records and a wave's load covers four items, one per 16 lanes (a bucket's run in a tile
// is about 32 pair records: whole-wave items would leave half the lanes idle).
constexpr uint32_t PITEM_SHIFT = 4;
constexpr uint32_t PITEM_RECORDS = 1u << PITEM_SHIFT;
constexpr uint32_t PITEM_PER_LOAD = 64 / PITEM_RECORDS;
constexpr uint32_t P_LOADS = 4;  // loads per lane in flight per register set

// Every thread owns the bucket's run of one tile.  The runs are cut into items, the items of all runs are numbered
// consecutively (block scan of the item counts) and listed in LDS (first record, record count), ITEM_CAP at a time:
// a wave then finds an item's records with one LDS read instead of searching the runs' prefix sums, whose chain of
// dependent LDS reads was most of this kernel's time.
template <bool PAIR>
__device__ __forceinline__ void grid_reduce_runs(const uint32_t tiles, const uint32_t level, const uint32_t bucket, const uint32_t group,
                                                 const uint32_t G, const uint32_t* __restrict__ rec_vals, const uint16_t* __restrict__ rec_keys,
                                                 const uint16_t* __restrict__ offsets, unsigned long long* acc, uint32_t* item_src,
                                                 uint8_t* item_n, uint32_t* wave_tot, const uint32_t bucket_entries) {
	constexpr uint32_t SHIFT = PAIR ? PITEM_SHIFT : ITEM_SHIFT, RECS = 1u << SHIFT;
	constexpr uint32_t TILE_RECS = PAIR ? BIN_RECORDS / 2 : BIN_RECORDS;  // records in a tile's slot of the value array
	const uint32_t lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
	const uint32_t my_tiles = (tiles > group) ? (tiles - group + G - 1) / G : 0;  // tiles group, group + G, ...
	const size_t level_tile0 = (size_t)level * tiles;
	const uint32_t* base_val = rec_vals + level_tile0 * BIN_RECORDS;
	const uint16_t* base_key = rec_keys + level_tile0 * BIN_RECORDS;
	for (uint32_t c0 = 0; c0 < my_tiles || c0 == 0; c0 += RED_BLOCK) {
		// this thread's run (the load is in flight while the accumulators are cleared)
		uint32_t src = 0, len = 0;
		const uint32_t t = c0 + threadIdx.x;
		if (t < my_tiles) {
			const size_t tile = level_tile0 + group + (size_t)t * G;
			const uint16_t* off = offsets + tile * (BKT_MAX + 1) + bucket;
			const uint32_t begin = off[0], end = off[1];
			src = (uint32_t)((tile - level_tile0) * TILE_RECS) + begin;
			len = end - begin;
		}
		if (c0 == 0) {
			for (uint32_t e = threadIdx.x; e < bucket_entries; e += RED_BLOCK) { acc[e] = 0ull; acc[BKT_ENTRIES + e] = 0ull; }
		}
		const uint32_t cnt = (len + RECS - 1u) >> SHIFT;
		uint32_t incl = cnt;
#pragma unroll
		for (int o = 1; o < 64; o <<= 1) {
			const uint32_t u = __shfl_up(incl, o);
			if ((int)lane >= o) incl += u;
		}
		__syncthreads();  // the previous chunk's items are done with wave_tot and the item list
		if (lane == 63) wave_tot[wave] = incl;
		__syncthreads();
		uint32_t first = incl - cnt, n_items = 0;  // number of this thread's first item; items of the chunk
		for (uint32_t w = 0; w < RED_BLOCK / 64; ++w) {
			const uint32_t tot = wave_tot[w];
			if (w < wave) first += tot;
			n_items += tot;
		}
		for (uint32_t w0 = 0; w0 < n_items; w0 += ITEM_CAP) {
			if (w0 > 0) __syncthreads();  // the previous window has been read
			// list this thread's items that fall into the window [w0, w0 + ITEM_CAP)
			for (uint32_t i = (first < w0) ? w0 - first : 0u; i < cnt && first + i < w0 + ITEM_CAP; ++i) {
				const uint32_t rest = len - (i << SHIFT);
				item_src[first + i - w0] = src + (i << SHIFT);
				item_n[first + i - w0] = (uint8_t)((rest < RECS ? rest : RECS) - 1u);
			}
			__syncthreads();
			const uint32_t n_win = (n_items - w0 < ITEM_CAP) ? n_items - w0 : ITEM_CAP;
			if constexpr (PAIR) {
				const uint2* base_val2 = reinterpret_cast<const uint2*>(base_val);
				const uint32_t r = lane & (PITEM_RECORDS - 1u), sub = lane >> PITEM_SHIFT;
				// Lanes past the end of an item read the level's first record instead (and ignore it): with every load issued
				// unconditionally the compiler can count them, and waits for the CURRENT set only while the next is in flight.
				auto fetch = [&](uint32_t i0, uint2 (&val)[P_LOADS], uint32_t (&key)[P_LOADS], uint32_t& okmask) {
					okmask = 0;
#pragma unroll
					for (uint32_t h = 0; h < P_LOADS; ++h) {
						const uint32_t it = i0 + PITEM_PER_LOAD * h + sub;
						uint32_t s0 = 0, n = 0;
						if (it < n_win) { s0 = item_src[it]; n = (uint32_t)item_n[it] + 1u; }
						const bool ok = r < n;
						okmask |= (ok ? 1u : 0u) << h;
						const uint32_t at = ok ? s0 + r : 0u;
						val[h] = base_val2[at];
						key[h] = base_key[at + (at & ~(TILE_RECS - 1u))];  // a tile's key slot is twice as long as its pair records
					}
				};
				auto accumulate = [&](const uint2 (&val)[P_LOADS], const uint32_t (&key)[P_LOADS], uint32_t okmask) {
#pragma unroll
					for (uint32_t q = 0; q < P_LOADS; ++q) {
						if (okmask & (1u << q)) {
							const uint32_t a1 = key[q] & (BKT_ENTRIES - 1u);
							const uint32_t a2 = a1 ^ ((2u << (key[q] >> BKT_SHIFT)) - 1u);  // the x + 1 corner: x ^ (x + 1) = 2^(t+1) - 1
							const float2 f = __half22float2(*reinterpret_cast<const __half2*>(&val[q].x));
							const float2 g = __half22float2(*reinterpret_cast<const __half2*>(&val[q].y));
							atomicAdd(&acc[a1], to_fixed(f.x));  // LDS integer atomics
							atomicAdd(&acc[BKT_ENTRIES + a1], to_fixed(f.y));
							atomicAdd(&acc[a2], to_fixed(g.x));
							atomicAdd(&acc[BKT_ENTRIES + a2], to_fixed(g.y));
						}
					}
				};
				constexpr uint32_t PER_WAVE = PITEM_PER_LOAD * P_LOADS, STRIDE = (RED_BLOCK / 64) * PER_WAVE;
				uint2 va[P_LOADS], vb[P_LOADS];
				uint32_t ka[P_LOADS], kb[P_LOADS], ok_a = 0, ok_b = 0;
				uint32_t i0 = wave * PER_WAVE;
				if (i0 < n_win) {
					fetch(i0, va, ka, ok_a);
					for (;;) {
						fetch(i0 + STRIDE, vb, kb, ok_b);
						accumulate(va, ka, ok_a);
						i0 += STRIDE;
						if (i0 >= n_win) break;
						fetch(i0 + STRIDE, va, ka, ok_a);
						accumulate(vb, kb, ok_b);
						i0 += STRIDE;
						if (i0 >= n_win) break;
					}
				}
			} else {
				// a wave takes RED_ITEMS items at a time
				auto fetch = [&](uint32_t i0, uint2 (&rec)[ITEM_LOADS * RED_ITEMS], uint32_t& okmask) {
					okmask = 0;
#pragma unroll
					for (uint32_t j = 0; j < RED_ITEMS; ++j) {
						const uint32_t it = i0 + j;
						uint32_t s0 = 0, n = 0;
						if (it < n_win) { s0 = item_src[it]; n = (uint32_t)item_n[it] + 1u; }
#pragma unroll
						for (uint32_t h = 0; h < ITEM_LOADS; ++h) {
							const uint32_t r = h * 64 + lane;
							const bool ok = r < n;
							okmask |= (ok ? 1u : 0u) << (ITEM_LOADS * j + h);
							// lanes past the end of the run read the level's first record instead (and ignore it): with every
							// load issued unconditionally the compiler can count them, and waits for the CURRENT items only
							// while the next ones are in flight
							const size_t at = ok ? (size_t)s0 + r : 0;
							rec[ITEM_LOADS * j + h] = make_uint2(base_key[at], base_val[at]);
						}
					}
				};
				constexpr uint32_t STRIDE = (RED_BLOCK / 64) * RED_ITEMS;
				auto accumulate = [&](const uint2 (&rec)[ITEM_LOADS * RED_ITEMS], uint32_t okmask) {
#pragma unroll
					for (uint32_t q = 0; q < ITEM_LOADS * RED_ITEMS; ++q) {
						if (okmask & (1u << q)) {
							const __half2 hh = *reinterpret_cast<const __half2*>(&rec[q].y);
							const float2 f = __half22float2(hh);
							atomicAdd(&acc[rec[q].x], to_fixed(f.x));  // LDS integer atomics
							atomicAdd(&acc[BKT_ENTRIES + rec[q].x], to_fixed(f.y));
						}
					}
				};
				// Two register sets take turns: while one is accumulated the loads of the other are in flight.  Every fetch
				// issues the same number of loads (items past the end read the first record and are ignored) and no set is
				// ever copied, so each wait covers exactly the set that is about to be used.
				uint2 ra[ITEM_LOADS * RED_ITEMS], rb[ITEM_LOADS * RED_ITEMS];
				uint32_t ok_a = 0, ok_b = 0;
				uint32_t i0 = wave * RED_ITEMS;
				if (i0 < n_win) {
					fetch(i0, ra, ok_a);
					for (;;) {
						fetch(i0 + STRIDE, rb, ok_b);
						accumulate(ra, ok_a);
						i0 += STRIDE;
						if (i0 >= n_win) break;
						fetch(i0 + STRIDE, ra, ok_a);
						accumulate(rb, ok_b);
						i0 += STRIDE;
						if (i0 >= n_win) break;
					}
				}
			}
		}
	}
}

__global__ void __launch_bounds__(RED_BLOCK, 8) grid_reduce_kernel(N2LevelTable tab, N2BucketPlan plan, uint32_t tiles,
                                                                   const uint32_t* __restrict__ rec_vals, const uint16_t* __restrict__ rec_keys,
                                                                   const uint16_t* __restrict__ offsets,
                                                                   __half2* __restrict__ grads, int accumulate,
                                                                   float2* __restrict__ partials) {
	// one plane per feature: lanes of a wave's atomic then spread over all bank pairs (entry-major pairs of features would
	// leave every other pair unused)
	__shared__ unsigned long long acc[2 * BKT_ENTRIES];
	__shared__ uint32_t item_src[ITEM_CAP];  // index of the item's first record in the level's records
	__shared__ uint8_t item_n[ITEM_CAP];     // its record count - 1
	__shared__ uint32_t wave_tot[RED_BLOCK / 64];
	// which (level, bucket, group) is this workgroup?
	uint32_t level = 0;
	while (blockIdx.x >= plan.wg_begin[level + 1]) ++level;
	const uint32_t local = blockIdx.x - plan.wg_begin[level];
	const uint32_t G = plan.groups[level];
	uint32_t bucket = local / G;
	const uint32_t group = local - bucket * G;
	// A tile's runs for neighbouring buckets meet inside a 128-byte line, which both buckets' workgroups fetch.  Workgroup
	// ids are dealt round-robin over the XCDs: XCD x takes the x-th eighth of the level's buckets, in order, so that both
	// fetches of such a line go through the same L2 at about the same time.
	const uint32_t nb = plan.n_buckets[level];
	// entries per bucket: the level's own size (split buckets always have BKT_ENTRIES)
	const uint32_t bucket_entries = ((tab.pair_levels >> level) & 1u) ? BKT_ENTRIES : 1u << tab.bucket_shift[level];
	if (G == 1 && nb % N_XCD == 0) bucket = (blockIdx.x % N_XCD) * (nb / N_XCD) + local / N_XCD;
	if ((tab.pair_levels >> level) & 1u)
		grid_reduce_runs<true>(tiles, level, bucket, group, G, rec_vals, rec_keys, offsets, acc, item_src, item_n, wave_tot, BKT_ENTRIES);
	else
		grid_reduce_runs<false>(tiles, level, bucket, group, G, rec_vals, rec_keys, offsets, acc, item_src, item_n, wave_tot, bucket_entries);
	__syncthreads();
	const uint32_t entries = tab.entries[level];
	__half2* Gd = grads + tab.offset[level];
	if (G > 1) {
		// Several workgroups hold parts of this bucket's sums (coarse levels of large batches).  Each leaves its image as
		// fp32 and grid_combine_kernel adds the G images up in the order of the groups: every entry is the same sum of the
		// same terms in the same order however the workgroups were scheduled (the images themselves are exact integer sums).
		float2* mine = partials + ((size_t)plan.part_begin[level] + (size_t)bucket * G + group) * BKT_ENTRIES;
		for (uint32_t e = threadIdx.x; e < BKT_ENTRIES; e += RED_BLOCK) mine[e] = make_float2(from_fixed(acc[e]), from_fixed(acc[BKT_ENTRIES + e]));
		return;
	}
	for (uint32_t e = threadIdx.x; e < bucket_entries; e += RED_BLOCK) {
		const uint32_t idx = bucket * bucket_entries + e;
		if (idx >= entries) break;
		const float ax = from_fixed(acc[e]), ay = from_fixed(acc[BKT_ENTRIES + e]);
		if (accumulate) {
			const float2 old = __half22float2(Gd[idx]);
			Gd[idx] = __floats2half2_rn(old.x + ax, old.y + ay);
		} else {
			Gd[idx] = __floats2half2_rn(ax, ay);
		}
	}
}

// Split buckets: the sum of a bucket's G partial images in a fixed order (n2_image_combine_unit, slab_reduce.h: with the
// images added one after the other by one thread the launch was a chain of memory round trips, 9 us for 5 MB).  Run as units
// of the optimiser's kernel instead of a launch of its own it shortens the training step by 0.9 us (measured): not built.
// (Doing this in the reduce kernel, by the workgroup of a bucket that finishes last, needs two device-scope fences per
// workgroup, which write back and invalidate the L2s: the scatter took 150 us longer.  Packed fp16 atomics into the
// gradient buffer cost nothing extra but add in arrival order.)
static_assert(BKT_ENTRIES % N2_CMB_ENTRIES == 0, "whole units per bucket");
__global__ void __launch_bounds__(256) grid_combine_kernel(N2ImageCombine plan) {
	__shared__ float2 part[N2_CMB_SLICES][N2_CMB_ENTRIES];
	n2_image_combine_unit(plan, blockIdx.x, part, [](const _Float16*, _Float16) {});
}

// ----------------------------------------------------------------------------
// host side
// ----------------------------------------------------------------------------
static uint32_t level_mode(uint32_t res, uint32_t entries) {
	// Mirror of the reference index rule: add dimensions while the running
	// stride still fits into the level; hashed iff the final stride exceeds it.
	uint64_t stride = 1;
	for (int d = 0; d < 3 && stride <= entries; ++d) stride *= res;
	const bool hashed = entries < stride;
	const bool pow2 = (entries & (entries - 1u)) == 0;
	if (hashed) return pow2 ? N2_LEVEL_HASH : N2_LEVEL_HASH_MOD;
	const uint64_t r = res;
	const uint64_t max_index = r + r * r + r * r * r;  // every coordinate at most res
	return (max_index < 2ull * entries) ? N2_LEVEL_DENSE : N2_LEVEL_DENSE_MOD;
}

N2_API int n2_grid_create(uint32_t n_levels, uint32_t n_features_per_level, uint32_t log2_hashmap_size,
                          uint32_t base_resolution, float per_level_scale, n2_grid_t** out) {
	N2_REQUIRE(out != nullptr, "n2_grid_create: out is null");
	*out = nullptr;
	N2_REQUIRE(n_levels >= 1 && n_levels <= N2_MAX_LEVELS, "n2_grid_create: n_levels %u outside [1, %u]", n_levels, N2_MAX_LEVELS);
	if (n_features_per_level != 2) {
		n2_set_error("n2_grid_create: only n_features_per_level = 2 is implemented (got %u)", n_features_per_level);
		return N2_ERR_UNSUPPORTED;
	}
	N2_REQUIRE(log2_hashmap_size >= 3 && log2_hashmap_size <= 28, "n2_grid_create: log2_hashmap_size %u outside [3, 28]", log2_hashmap_size);
	N2_REQUIRE(base_resolution >= 1 && per_level_scale >= 1.0f, "n2_grid_create: base_resolution >= 1 and per_level_scale >= 1 required");
	n2_grid* g = new (std::nothrow) n2_grid();
	N2_REQUIRE(g != nullptr, "n2_grid_create: out of host memory");
	g->n_features = n_features_per_level;
	g->tab.n_levels = n_levels;
	g->tab.n_features = n_features_per_level;
	g->tab.max_level = 1.0f;
	g->tab.max_level_gpu = nullptr;
	g->tab.valid_levels = n_levels;
	g->tab.active_levels = n_levels;
	g->tab.pair_levels = 0;
	g->base_valid_level_scale = 1.0f;
	g->valid_level_scale = 0.0f;
	g->base_training_step = 0;
	g->training_step = 0;
	uint64_t off = 0;
	const float log2_b = std::log2(per_level_scale);
	for (uint32_t l = 0; l < n_levels; ++l) {
		const float s = exp2f((float)l * log2_b) * (float)base_resolution - 1.0f;
		const uint32_t res = (uint32_t)ceilf(s) + 1u;
		const uint32_t max_params = 0xFFFFFFFFu / 2u;
		const double cube = (double)res * (double)res * (double)res;
		uint32_t n = cube > (double)max_params ? max_params : res * res * res;
		n = (n + 7u) / 8u * 8u;
		const uint32_t cap = 1u << log2_hashmap_size;
		if (n > cap) n = cap;
		g->tab.scale[l] = s;
		g->tab.resolution[l] = res;
		g->tab.entries[l] = n;
		g->tab.offset[l] = (uint32_t)off;
		g->tab.mode[l] = level_mode(res, n);
		// hashed levels gather from all over their table; the dense ones mostly hit lines their neighbours fetched
		g->level_cost[l] = (g->tab.mode[l] == N2_LEVEL_HASH || g->tab.mode[l] == N2_LEVEL_HASH_MOD) ? 1.0f : 0.6f;
		// pair records in the bucketed scatter: x and x + 1 must stay below the bucket size (see grid_bin_kernel)
		if (g->tab.mode[l] == N2_LEVEL_HASH && res <= PAIR_MAX_CELL + 1u && n >= BKT_ENTRIES) g->tab.pair_levels |= 1u << l;
		off += n;
	}
	if (off * n_features_per_level > 0x7FFFFFFFull) {
		delete g;
		n2_set_error("n2_grid_create: %llu parameters exceed the 2^31 limit", (unsigned long long)(off * n_features_per_level));
		return N2_ERR_UNSUPPORTED;
	}
	g->tab.offset[n_levels] = (uint32_t)off;
	g->n_params = (uint32_t)off * n_features_per_level;
	g->params = nullptr;
	g->grads = nullptr;
	g->ws = nullptr;
	g->ws_bytes = 0;
	g->ws_max_points = 0;
	g->lattice_order = false;
	*out = g;
	return N2_OK;
}

N2_API void n2_grid_destroy(n2_grid_t* grid) { delete grid; }
const N2LevelTable* n2_grid_table(const n2_grid_t* grid) { return &grid->tab; }
const __half2* n2_grid_params(const n2_grid_t* grid) { return grid->params; }
bool n2_grid_lattice_order(const n2_grid_t* grid) { return grid->lattice_order; }
N2_API uint32_t n2_grid_n_params(const n2_grid_t* grid) { return grid ? grid->n_params : 0; }
N2_API uint32_t n2_grid_output_width(const n2_grid_t* grid) { return grid ? grid->tab.n_levels * grid->n_features : 0; }
N2_API uint32_t n2_grid_n_levels(const n2_grid_t* grid) { return grid ? grid->tab.n_levels : 0; }

N2_API int n2_grid_level_table(const n2_grid_t* grid, float* scale, uint32_t* resolution, uint32_t* entries, uint32_t* offset) {
	N2_REQUIRE(grid != nullptr, "n2_grid_level_table: grid is null");
	for (uint32_t l = 0; l < grid->tab.n_levels; ++l) {
		if (scale) scale[l] = grid->tab.scale[l];
		if (resolution) resolution[l] = grid->tab.resolution[l];
		if (entries) entries[l] = grid->tab.entries[l];
		if (offset) offset[l] = grid->tab.offset[l];
	}
	if (offset) offset[grid->tab.n_levels] = grid->tab.offset[grid->tab.n_levels];
	return N2_OK;
}

N2_API int n2_grid_set_level_costs(n2_grid_t* grid, const float* costs) {
	N2_REQUIRE(grid != nullptr && costs != nullptr, "n2_grid_set_level_costs: null argument");
	for (uint32_t l = 0; l < grid->tab.n_levels; ++l) {
		N2_REQUIRE(costs[l] > 0.f && costs[l] <= 1e6f, "n2_grid_set_level_costs: cost of level %u must be in (0, 1e6]", l);
	}
	for (uint32_t l = 0; l < grid->tab.n_levels; ++l) grid->level_cost[l] = costs[l];
	return N2_OK;
}

// levels in use under the global settings, with the device predicate's arithmetic
static uint32_t count_active_levels(const N2LevelTable& tab) {
	const float limit = (tab.max_level * (float)(tab.n_levels * tab.n_features)) / (float)tab.n_features;
	uint32_t n = 0;
	while (n < tab.n_levels && n < tab.valid_levels && !((float)n >= limit + 1e-3f)) ++n;  // both rules cut a suffix of the levels
	return n;
}

N2_API int n2_grid_set_max_level(n2_grid_t* grid, float max_level) {
	N2_REQUIRE(grid != nullptr, "n2_grid_set_max_level: grid is null");
	N2_REQUIRE(max_level >= 0.f && max_level <= 1000.f, "n2_grid_set_max_level: max_level %g outside [0, 1000]", (double)max_level);
	grid->tab.max_level = max_level;
	grid->tab.active_levels = count_active_levels(grid->tab);
	return N2_OK;
}

N2_API int n2_grid_set_max_level_gpu(n2_grid_t* grid, const float* d_max_level) {
	N2_REQUIRE(grid != nullptr, "n2_grid_set_max_level_gpu: grid is null");
	grid->tab.max_level_gpu = d_max_level;
	return N2_OK;
}

N2_API int n2_grid_set_progressive(n2_grid_t* grid, float base_valid_level_scale, float valid_level_scale, uint32_t base_training_step) {
	N2_REQUIRE(grid != nullptr, "n2_grid_set_progressive: grid is null");
	N2_REQUIRE(base_valid_level_scale >= 0.f && valid_level_scale >= 0.f, "n2_grid_set_progressive: scales must be >= 0");
	grid->base_valid_level_scale = base_valid_level_scale;
	grid->valid_level_scale = valid_level_scale;
	grid->base_training_step = base_training_step;
	// the levels in use follow from the keys and the training step last set
	return n2_grid_set_training_step(grid, grid->training_step);
}

// levels in use at a training step: the fraction base + scale * (step / base_training_step), whole periods only,
// of all levels, rounded down (after + 1e-3, so that a fraction that reaches 1 up to rounding gives every level),
// at least one level and at most all of them
N2_API int n2_grid_set_training_step(n2_grid_t* grid, uint32_t training_step) {
	N2_REQUIRE(grid != nullptr, "n2_grid_set_training_step: grid is null");
	grid->training_step = training_step;
	if (grid->base_training_step == 0) {
		grid->tab.valid_levels = grid->tab.n_levels;
		grid->tab.active_levels = count_active_levels(grid->tab);
		return N2_OK;
	}
	const float fraction = grid->base_valid_level_scale + grid->valid_level_scale * (float)(training_step / grid->base_training_step);
	const float levels = fraction * (float)grid->tab.n_levels + 1e-3f;
	uint32_t n = levels >= (float)grid->tab.n_levels ? grid->tab.n_levels : (uint32_t)levels;
	if (n < 1) n = 1;
	grid->tab.valid_levels = n;
	grid->tab.active_levels = count_active_levels(grid->tab);
	return N2_OK;
}

N2_API uint32_t n2_grid_active_levels(const n2_grid_t* grid) { return grid ? grid->tab.active_levels : 0; }

N2_API int n2_grid_set_point_order(n2_grid_t* grid, int lattice_order) {
	N2_REQUIRE(grid != nullptr, "n2_grid_set_point_order: grid is null");
	grid->lattice_order = lattice_order != 0;
	return N2_OK;
}

N2_API int n2_grid_set_params(n2_grid_t* grid, const n2_half* d_params, n2_half* d_gradients) {
	N2_REQUIRE(grid != nullptr, "n2_grid_set_params: grid is null");
	N2_REQUIRE(d_params != nullptr, "n2_grid_set_params: d_params is null");
	N2_REQUIRE(reinterpret_cast<uintptr_t>(d_params) % 16 == 0, "n2_grid_set_params: d_params must be 16-byte aligned");
	N2_REQUIRE(reinterpret_cast<uintptr_t>(d_gradients) % 16 == 0, "n2_grid_set_params: d_gradients must be 16-byte aligned");
	grid->params = reinterpret_cast<const __half2*>(d_params);
	grid->grads = reinterpret_cast<__half2*>(d_gradients);
	return N2_OK;
}

// Shared argument checks.  Row offsets are computed in 64 bits on the device;
// the point index itself is 32 bits.
static int check_batch(const n2_grid_t* grid, const char* fn, const float* d_xyz, uint32_t point_stride, uint32_t dim_stride,
                       uint32_t n_points) {
	N2_REQUIRE(grid != nullptr, "%s: grid is null", fn);
	N2_REQUIRE(grid->params != nullptr, "%s: n2_grid_set_params has not been called", fn);
	N2_REQUIRE(d_xyz != nullptr || n_points == 0, "%s: d_xyz is null", fn);
	N2_REQUIRE(point_stride >= 1 && dim_stride >= 1, "%s: strides must be >= 1", fn);
	N2_REQUIRE(n_points <= (1u << 30), "%s: n_points %u exceeds 2^30", fn, n_points);
	return N2_OK;
}

static inline uint32_t n_tiles(uint32_t n_points) { return (n_points + GRID_BLOCK - 1) / GRID_BLOCK; }

// Cuts the level-major list of n_levels x tiles items into N_XCD contiguous pieces of equal estimated cost.
// Returns the length of the longest piece (the launch needs N_XCD times that many workgroups).
static uint32_t make_xcd_plan(const n2_grid_t* grid, uint32_t tiles, N2XcdPlan& plan) {
	const uint32_t L = grid->tab.n_levels;
	double total = 0.0;
	for (uint32_t l = 0; l < L; ++l) total += (double)grid->level_cost[l] * tiles;
	plan.begin[0] = 0;
	uint32_t level = 0, longest = 0;
	double before = 0.0;  // cost of the levels below `level`
	for (uint32_t x = 1; x < N_XCD; ++x) {
		const double target = total * x / N_XCD;
		while (level + 1 < L && before + (double)grid->level_cost[level] * tiles <= target) {
			before += (double)grid->level_cost[level] * tiles;
			++level;
		}
		double in_level = (target - before) / grid->level_cost[level];
		if (in_level < 0.0) in_level = 0.0;
		if (in_level > tiles) in_level = tiles;
		uint32_t b = level * tiles + (uint32_t)(in_level + 0.5);
		if (b < plan.begin[x - 1]) b = plan.begin[x - 1];
		plan.begin[x] = b;
	}
	plan.begin[N_XCD] = L * tiles;
	for (uint32_t x = 0; x < N_XCD; ++x) {
		const uint32_t len = plan.begin[x + 1] - plan.begin[x];
		if (len > longest) longest = len;
	}
	return longest;
}

N2_API int n2_grid_forward(n2_grid_t* grid, n2_stream_t stream, const float* d_xyz, uint32_t point_stride,
                           uint32_t dim_stride, uint32_t n_points, n2_half* d_out, float* d_dy_dx) {
	if (int rc = check_batch(grid, "n2_grid_forward", d_xyz, point_stride, dim_stride, n_points)) return rc;
	if (n_points == 0) return N2_OK;
	N2_REQUIRE(d_out != nullptr, "n2_grid_forward: d_out is null");
	N2XcdPlan plan;
	N2ProfScope prof(N2_PROF_GRID_FORWARD, n2_stream(stream));
	if (grid->lattice_order && !d_dy_dx) {
		const uint32_t tiles = n_tiles(n_points);
		const dim3 grid_dim(tiles * grid->tab.n_levels);
		grid_forward_point_kernel<<<grid_dim, dim3(GRID_BLOCK), 0, n2_stream(stream)>>>(grid->tab, n_points, tiles, d_xyz, point_stride, dim_stride,
			grid->params, reinterpret_cast<__half*>(d_out));
		N2_LAUNCH_CHECK();
		return N2_OK;
	}
	const uint32_t tiles = (n_points + FWD_POINTS - 1) / FWD_POINTS;
	const dim3 grid_dim(make_xcd_plan(grid, tiles, plan) * N_XCD), block(GRID_BLOCK);
	if (d_dy_dx) {
		grid_forward_kernel<true><<<grid_dim, block, 0, n2_stream(stream)>>>(grid->tab, plan, n_points, tiles, d_xyz, point_stride,
			dim_stride, grid->params, reinterpret_cast<__half*>(d_out), d_dy_dx);
	} else {
		grid_forward_kernel<false><<<grid_dim, block, 0, n2_stream(stream)>>>(grid->tab, plan, n_points, tiles, d_xyz, point_stride,
			dim_stride, grid->params, reinterpret_cast<__half*>(d_out), nullptr);
	}
	N2_LAUNCH_CHECK();
	return N2_OK;
}

N2_API int n2_grid_corner_indices(n2_grid_t* grid, n2_stream_t stream, const float* d_xyz, uint32_t point_stride,
                                  uint32_t dim_stride, uint32_t n_points, uint32_t* d_indices) {
	if (int rc = check_batch(grid, "n2_grid_corner_indices", d_xyz, point_stride, dim_stride, n_points)) return rc;
	if (n_points == 0) return N2_OK;
	N2_REQUIRE(d_indices != nullptr, "n2_grid_corner_indices: d_indices is null");
	const uint32_t tiles = n_tiles(n_points);
	grid_indices_kernel<<<dim3(tiles * grid->tab.n_levels), dim3(GRID_BLOCK), 0, n2_stream(stream)>>>(
		grid->tab, n_points, tiles, d_xyz, point_stride, dim_stride, d_indices);
	N2_LAUNCH_CHECK();
	return N2_OK;
}

static bool uses_bucketed(const n2_grid_t* grid, uint32_t n_points);
static uint32_t bucket_groups(const n2_grid_t* grid, uint32_t level, uint32_t n_points, uint32_t tiles);

// OVERWRITE: the gradient buffer starts from zero.  The bucketed scatter writes every entry itself (with plain stores),
// so only the scatter with atomics needs the buffer cleared beforehand.
static int prepare_grads(n2_grid_t* grid, const char* fn, hipStream_t stream, n2_grad_mode mode, uint32_t n_points) {
	N2_REQUIRE(mode == N2_GRAD_IGNORE || mode == N2_GRAD_OVERWRITE || mode == N2_GRAD_ACCUMULATE, "%s: bad gradient mode %d", fn, (int)mode);
	if (mode == N2_GRAD_IGNORE) return N2_OK;
	N2_REQUIRE(grid->grads != nullptr, "%s: gradient mode %d needs a gradient buffer (n2_grid_set_params)", fn, (int)mode);
	if (mode != N2_GRAD_OVERWRITE) return N2_OK;
	if (!uses_bucketed(grid, n_points)) return n2_fill_zero_u32(stream, grid->grads, (size_t)grid->n_params * sizeof(__half));
	return N2_OK;
}

static inline uint32_t n_pair_tiles(uint32_t n_points) { return (n_points + PAIR_POINTS - 1) / PAIR_POINTS; }
static inline uint32_t n_bin_tiles(uint32_t n_points) { return (n_points + BIN_POINTS - 1) / BIN_POINTS; }

static bool bucket_supported(const n2_grid_t* grid) {
	for (uint32_t l = 0; l < grid->tab.n_levels; ++l)
		if (grid->tab.entries[l] > BKT_ENTRIES * BKT_MAX) return false;
	return true;
}
// workspace: the records' values, their keys, the tiles' bucket offsets, then one fp32 image per (bucket, group) of the
// split buckets
struct BucketCarve {
	uint64_t vals, keys, offsets, partials, total;
};
static uint32_t split_images(const n2_grid_t* grid, uint32_t n_points);
static BucketCarve bucket_carve(const n2_grid_t* grid, uint32_t max_points) {
	const uint64_t tiles = n_bin_tiles(max_points), L = grid->tab.n_levels;
	const uint64_t n_rec = L * tiles * BIN_RECORDS;
	auto up = [](uint64_t x) { return (x + 255) / 256 * 256; };
	BucketCarve c{};
	c.vals = 0;
	c.keys = c.vals + n_rec * sizeof(uint32_t);
	c.offsets = c.keys + n_rec * sizeof(uint16_t);
	c.partials = up(c.offsets + L * tiles * (BKT_MAX + 1) * sizeof(uint16_t));
	c.total = up(c.partials + (uint64_t)split_images(grid, max_points) * BKT_ENTRIES * sizeof(float2));
	return c;
}
static uint64_t bucket_ws_bytes(const n2_grid_t* grid, uint32_t max_points) { return bucket_carve(grid, max_points).total; }

// With a workspace every batch size takes the bucketed scatter, whose result does not depend on the order in which
// workgroups run; the scatter with atomics (no workspace, or more points than it was sized for) sums in arrival order.
static bool uses_bucketed(const n2_grid_t* grid, uint32_t n_points) {
	return grid->grads != nullptr && grid->ws != nullptr && n_points <= grid->ws_max_points && n_points >= 1;
}
// workgroups per bucket of a level: aim at <= ~64k records per reduce workgroup (a level holds 8 records per point)
// Entries per bucket of a level (log2).  Levels that sort pair records keep 4096-entry buckets (a pair's second entry is
// encoded against that size); the others take the largest size (a power of two, at most 4096 entries and at most BKT_MAX
// buckets) under which no bucket needs more than one workgroup: small dense levels of large batches get many small buckets
// instead of few that are split.  When even the smallest size does not get there, the buckets stay large and are split.
static uint32_t bucket_shift_for(const n2_grid_t* grid, uint32_t level, uint32_t n_points) {
	if ((grid->tab.pair_levels >> level) & 1u) return BKT_SHIFT;
	const uint32_t entries = grid->tab.entries[level];
	for (uint32_t shift = BKT_SHIFT; shift >= BKT_MIN_SHIFT; --shift) {
		const uint32_t nb = (entries + (1u << shift) - 1u) >> shift;
		if (nb > BKT_MAX) break;
		if ((uint64_t)n_points * 8 / nb <= 65536) return shift;  // (32768: scatter + 1.3 us on the training step, 16384: + 4.7)
	}
	return BKT_SHIFT;
}
static inline uint32_t level_buckets(const n2_grid_t* grid, uint32_t level, uint32_t n_points) {
	const uint32_t shift = bucket_shift_for(grid, level, n_points);
	return (grid->tab.entries[level] + (1u << shift) - 1u) >> shift;
}

static uint32_t bucket_groups(const n2_grid_t* grid, uint32_t level, uint32_t n_points, uint32_t tiles) {
	const uint32_t nb = level_buckets(grid, level, n_points);
	const uint64_t per_bucket = (uint64_t)n_points * 8 / nb;
	uint32_t groups = (uint32_t)((per_bucket + 65535) / 65536);
	if (groups > N2_CMB_MAX_GROUPS) groups = N2_CMB_MAX_GROUPS;
	if (groups > tiles) groups = tiles;
	if (groups < 1) groups = 1;
	return groups;
}

// fp32 images of all split buckets of a batch (never more for a smaller batch: the groups per bucket grow with the batch)
static uint32_t split_images(const n2_grid_t* grid, uint32_t n_points) {
	const uint32_t tiles = n_bin_tiles(n_points);
	uint32_t n = 0;
	for (uint32_t l = 0; l < grid->tab.n_levels; ++l) {
		const uint32_t nb = level_buckets(grid, l, n_points), groups = bucket_groups(grid, l, n_points, tiles);
		if (groups > 1) n += nb * groups;
	}
	return n;
}

N2_API uint64_t n2_grid_workspace_bytes(const n2_grid_t* grid, uint32_t max_points) {
	if (!grid || !bucket_supported(grid)) return 0;
	return bucket_ws_bytes(grid, max_points);
}

N2_API int n2_grid_set_workspace(n2_grid_t* grid, void* d_workspace, uint64_t n_bytes, uint32_t max_points) {
	N2_REQUIRE(grid != nullptr, "n2_grid_set_workspace: grid is null");
	if (d_workspace == nullptr) {
		grid->ws = nullptr; grid->ws_bytes = 0; grid->ws_max_points = 0;
		return N2_OK;
	}
	N2_REQUIRE(reinterpret_cast<uintptr_t>(d_workspace) % 256 == 0, "n2_grid_set_workspace: workspace must be 256-byte aligned");
	N2_REQUIRE(n_bytes >= n2_grid_workspace_bytes(grid, max_points), "n2_grid_set_workspace: %llu bytes given, %llu needed for %u points",
	           (unsigned long long)n_bytes, (unsigned long long)n2_grid_workspace_bytes(grid, max_points), max_points);
	grid->ws = reinterpret_cast<unsigned char*>(d_workspace);
	grid->ws_bytes = n_bytes;
	grid->ws_max_points = bucket_supported(grid) ? max_points : 0;
	return N2_OK;
}

// Parameter gradients through the bin + reduce kernels.  The gradient buffer has been zeroed for OVERWRITE.
static int launch_bucketed(n2_grid_t* grid, hipStream_t s, const float* d_xyz, uint32_t point_stride, uint32_t dim_stride, uint32_t n_points,
                           const __half* dL_dy, const float* v, const __half* g2, __half* dL_ddLdy, bool accumulate,
                           const uint32_t* index, uint32_t n_cols) {
	const uint32_t tiles = n_bin_tiles(n_points), L = grid->tab.n_levels;
	const bool first = dL_dy != nullptr, second = v != nullptr, out = dL_ddLdy != nullptr;
	const dim3 bd(BIN_BLOCK);
	// The records of this batch are packed as for a workspace of exactly this size (values, keys, offsets one behind the
	// other); the images of split buckets stand where the workspace's own size put them.
	const BucketCarve now = bucket_carve(grid, n_points), full = bucket_carve(grid, grid->ws_max_points);
	uint32_t* rec_vals = reinterpret_cast<uint32_t*>(grid->ws + now.vals);
	uint16_t* rec_keys = reinterpret_cast<uint16_t*>(grid->ws + now.keys);
	uint16_t* offsets = reinterpret_cast<uint16_t*>(grid->ws + now.offsets);
	float2* partials = reinterpret_cast<float2*>(grid->ws + full.partials);
	const dim3 gd(tiles * L);
	N2BucketPlan plan;
	uint32_t wg = 0, images = 0, split = 0;
	N2LevelTable tab = grid->tab;  // with this launch's bucket sizes
	for (uint32_t l = 0; l < L; ++l) {
		tab.bucket_shift[l] = (uint8_t)bucket_shift_for(grid, l, n_points);
		const uint32_t nb = level_buckets(grid, l, n_points);
		const uint32_t groups = bucket_groups(grid, l, n_points, tiles);
		plan.wg_begin[l] = wg;
		plan.n_buckets[l] = nb;
		plan.groups[l] = groups;
		plan.part_begin[l] = images;
		plan.split_begin[l] = split;
		wg += nb * groups;
		if (groups > 1) { images += nb * groups; split += nb; }
	}
	for (uint32_t l = L; l <= N2_MAX_LEVELS; ++l) plan.wg_begin[l] = wg;
	for (uint32_t l = L; l < N2_MAX_LEVELS; ++l) { plan.n_buckets[l] = 0; plan.groups[l] = 1; plan.part_begin[l] = images; }
	for (uint32_t l = L; l <= N2_MAX_LEVELS; ++l) plan.split_begin[l] = split;
#define LAUNCH(F, S, O) grid_bin_kernel<F, S, O><<<gd, bd, 0, s>>>(tab, 0u, n_points, tiles, d_xyz, point_stride, dim_stride, dL_dy, v, g2, \
                                                                   grid->params, dL_ddLdy, rec_vals, rec_keys, offsets, index, n_cols)
	if (first && second && out) LAUNCH(true, true, true);
	else if (first && second) LAUNCH(true, true, false);
	else if (second && out) LAUNCH(false, true, true);
	else if (second) LAUNCH(false, true, false);
	else LAUNCH(true, false, false);
#undef LAUNCH
	N2_LAUNCH_CHECK();
	grid_reduce_kernel<<<dim3(wg), dim3(RED_BLOCK), 0, s>>>(tab, plan, tiles, rec_vals, rec_keys, offsets, grid->grads, accumulate ? 1 : 0, partials);
	N2_LAUNCH_CHECK();
	if (split > 0) {
		N2ImageCombine cmb{};
		cmb.images = partials;
		cmb.grads = reinterpret_cast<_Float16*>(grid->grads);
		cmb.bucket_entries = BKT_ENTRIES;
		cmb.accumulate = accumulate ? 1 : 0;
		uint32_t k = 0;  // the split levels, in order
		for (uint32_t l = 0; l < L; ++l) {
			if (plan.groups[l] <= 1) continue;
			N2_REQUIRE(tab.bucket_shift[l] == BKT_SHIFT, "grid scatter: level %u splits buckets of %u entries", l, 1u << tab.bucket_shift[l]);
			cmb.split_begin[k] = plan.split_begin[l]; cmb.groups[k] = plan.groups[l]; cmb.part_begin[k] = plan.part_begin[l];
			cmb.entries[k] = grid->tab.entries[l]; cmb.offset[k] = grid->tab.offset[l];
			++k;
		}
		cmb.n_levels = k;
		for (uint32_t l = k; l <= N2_CMB_LEVELS; ++l) cmb.split_begin[l] = split;
		cmb.units = split * (BKT_ENTRIES / N2_CMB_ENTRIES);
		grid_combine_kernel<<<dim3(cmb.units), dim3(256), 0, s>>>(cmb);
		N2_LAUNCH_CHECK();
	}
	return N2_OK;
}

// One scatter pass with any combination of first-order (dL_dy) and second-order (v, g2) terms.
static int launch_scatter(n2_grid_t* grid, hipStream_t s, const float* d_xyz, uint32_t point_stride, uint32_t dim_stride, uint32_t n_points,
                          const __half* dL_dy, const float* v, const __half* g2, __half2* grads, __half* dL_ddLdy, bool accumulate,
                          const uint32_t* index = nullptr, uint32_t n_cols = 0) {
	if (grads != nullptr && uses_bucketed(grid, n_points))
		return launch_bucketed(grid, s, d_xyz, point_stride, dim_stride, n_points, dL_dy, v, g2, dL_ddLdy, accumulate, index, n_cols);
	const uint32_t tiles = n_pair_tiles(n_points);
	const dim3 gd(tiles * grid->tab.n_levels), bd(GRID_BLOCK);
	const bool first = dL_dy != nullptr, second = v != nullptr, out = dL_ddLdy != nullptr;
#define LAUNCH(F, S, O) grid_scatter_kernel<F, S, O><<<gd, bd, 0, s>>>(grid->tab, n_points, tiles, d_xyz, point_stride, dim_stride, dL_dy, v, g2, \
                                                                       grid->params, grads, dL_ddLdy, index, n_cols)
	if (first && second && out) LAUNCH(true, true, true);
	else if (first && second) LAUNCH(true, true, false);
	else if (second && out) LAUNCH(false, true, true);
	else if (second) LAUNCH(false, true, false);
	else LAUNCH(true, false, false);
#undef LAUNCH
	N2_LAUNCH_CHECK();
	return N2_OK;
}

N2_API int n2_grid_backward(n2_grid_t* grid, n2_stream_t stream, const float* d_xyz, uint32_t point_stride,
                            uint32_t dim_stride, uint32_t n_points, const n2_half* d_dL_dy, const float* d_dy_dx,
                            float* d_dL_dx, n2_grad_mode mode) {
	if (int rc = check_batch(grid, "n2_grid_backward", d_xyz, point_stride, dim_stride, n_points)) return rc;
	N2_REQUIRE(d_dL_dy != nullptr || n_points == 0, "n2_grid_backward: d_dL_dy is null");
	N2_REQUIRE(d_dL_dx == nullptr || d_dy_dx != nullptr, "n2_grid_backward: d_dL_dx needs the d_dy_dx context of the forward");
	hipStream_t s = n2_stream(stream);
	if (int rc = prepare_grads(grid, "n2_grid_backward", s, mode, n_points)) return rc;
	if (n_points == 0) return N2_OK;
	if (mode != N2_GRAD_IGNORE) {
		N2ProfScope prof(N2_PROF_GRID_BACKWARD_PARAMS, s);
		if (int rc = launch_scatter(grid, s, d_xyz, point_stride, dim_stride, n_points, reinterpret_cast<const __half*>(d_dL_dy), nullptr,
		                            nullptr, grid->grads, nullptr, mode == N2_GRAD_ACCUMULATE)) return rc;
	}
	if (d_dL_dx) {
		grid_backward_input_kernel<<<dim3(n_tiles(n_points)), dim3(GRID_BLOCK), 0, s>>>(
			n_points, grid->tab.n_levels * grid->n_features, reinterpret_cast<const __half*>(d_dL_dy), d_dy_dx, d_dL_dx);
		N2_LAUNCH_CHECK();
	}
	return N2_OK;
}

N2_API int n2_grid_backward_fused(n2_grid_t* grid, n2_stream_t stream, const float* d_xyz, uint32_t point_stride,
                                  uint32_t dim_stride, uint32_t n_points, const n2_half* d_dL_dy,
                                  const float* d_dL_ddLdx, const n2_half* d_dL_dy_second, n2_half* d_dL_ddLdy,
                                  n2_grad_mode mode) {
	if (int rc = check_batch(grid, "n2_grid_backward_fused", d_xyz, point_stride, dim_stride, n_points)) return rc;
	N2_REQUIRE((d_dL_dy && d_dL_ddLdx && d_dL_dy_second) || n_points == 0, "n2_grid_backward_fused: d_dL_dy, d_dL_ddLdx and d_dL_dy_second are required");
	N2_REQUIRE(mode == N2_GRAD_OVERWRITE || mode == N2_GRAD_ACCUMULATE, "n2_grid_backward_fused: mode must be OVERWRITE or ACCUMULATE");
	hipStream_t s = n2_stream(stream);
	if (int rc = prepare_grads(grid, "n2_grid_backward_fused", s, mode, n_points)) return rc;
	if (n_points == 0) return N2_OK;
	N2ProfScope prof(N2_PROF_GRID_BACKWARD_PARAMS, s);
	return launch_scatter(grid, s, d_xyz, point_stride, dim_stride, n_points, reinterpret_cast<const __half*>(d_dL_dy), d_dL_ddLdx,
	                      reinterpret_cast<const __half*>(d_dL_dy_second), grid->grads, reinterpret_cast<__half*>(d_dL_ddLdy),
	                      mode == N2_GRAD_ACCUMULATE);
}

int n2_grid_backward_fused_indexed(n2_grid_t* grid, n2_stream_t stream, const float* d_xyz_rows, uint32_t n_cols, const uint32_t* d_index,
                                   uint32_t n_points, const n2_half* d_dL_dy, const float* d_dL_ddLdx, const n2_half* d_dL_dy_second,
                                   n2_grad_mode mode) {
	if (d_index == nullptr) n_cols = n_points;  // the rows hold the batch itself
	if (int rc = check_batch(grid, "n2_grid_backward_fused", d_xyz_rows, 1, n_cols, n_points)) return rc;
	N2_REQUIRE((d_dL_dy && d_dL_ddLdx && d_dL_dy_second) || n_points == 0, "n2_grid_backward_fused: d_dL_dy, d_dL_ddLdx and d_dL_dy_second are required");
	N2_REQUIRE(mode == N2_GRAD_OVERWRITE || mode == N2_GRAD_ACCUMULATE, "n2_grid_backward_fused: mode must be OVERWRITE or ACCUMULATE");
	N2_REQUIRE(n_cols >= 1, "n2_grid_backward_fused: an indexed input needs at least one column");
	hipStream_t s = n2_stream(stream);
	if (int rc = prepare_grads(grid, "n2_grid_backward_fused", s, mode, n_points)) return rc;
	if (n_points == 0) return N2_OK;
	N2ProfScope prof(N2_PROF_GRID_BACKWARD_PARAMS, s);
	return launch_scatter(grid, s, d_xyz_rows, 1, n_cols, n_points, reinterpret_cast<const __half*>(d_dL_dy), d_dL_ddLdx,
	                      reinterpret_cast<const __half*>(d_dL_dy_second), grid->grads, nullptr, mode == N2_GRAD_ACCUMULATE, d_index, n_cols);
}

N2_API int n2_grid_backward_backward_input(n2_grid_t* grid, n2_stream_t stream, const float* d_xyz,
                                           uint32_t point_stride, uint32_t dim_stride, uint32_t n_points,
                                           const float* d_dL_ddLdx, const n2_half* d_dL_dy, n2_half* d_dL_ddLdy,
                                           float* d_dL_dx, n2_grad_mode mode) {
	if (int rc = check_batch(grid, "n2_grid_backward_backward_input", d_xyz, point_stride, dim_stride, n_points)) return rc;
	N2_REQUIRE((d_dL_ddLdx != nullptr && d_dL_dy != nullptr) || n_points == 0, "n2_grid_backward_backward_input: d_dL_ddLdx and d_dL_dy are required");
	hipStream_t s = n2_stream(stream);
	if (int rc = prepare_grads(grid, "n2_grid_backward_backward_input", s, mode, d_dL_dx ? 0u : n_points)) return rc;
	if (n_points == 0) return N2_OK;
	if (mode == N2_GRAD_IGNORE && !d_dL_ddLdy && !d_dL_dx) return N2_OK;
	if (d_dL_dx) {
		if (int rc = n2_fill_zero_u32(s, d_dL_dx, sizeof(float) * 3 * (size_t)n_points)) return rc;
	}
	N2ProfScope prof(N2_PROF_GRID_SECOND_ORDER, s);
	if (!d_dL_dx) {
		return launch_scatter(grid, s, d_xyz, point_stride, dim_stride, n_points, nullptr, d_dL_ddLdx, reinterpret_cast<const __half*>(d_dL_dy),
		                      mode == N2_GRAD_IGNORE ? nullptr : grid->grads, reinterpret_cast<__half*>(d_dL_ddLdy), mode == N2_GRAD_ACCUMULATE);
	}
	const uint32_t tiles = n_tiles(n_points);
	grid_bbi_kernel<<<dim3(tiles * grid->tab.n_levels), dim3(GRID_BLOCK), 0, s>>>(
		grid->tab, n_points, tiles, d_xyz, point_stride, dim_stride, d_dL_ddLdx, reinterpret_cast<const __half*>(d_dL_dy),
		grid->params, mode == N2_GRAD_IGNORE ? nullptr : grid->grads, reinterpret_cast<__half*>(d_dL_ddLdy), d_dL_dx);
	N2_LAUNCH_CHECK();
	return N2_OK;
}
