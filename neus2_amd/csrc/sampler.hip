// Training-sample generator: pixel pick, ray / unit-cube intersection and the
// march through the occupancy bitfield.  One wave per ray (see march_wave); three
// kernels: march and count, exclusive scan in ray order, emit coordinates.
//
// Sample positions are part of the bit-exact contract with the CPU oracle, so
// floating-point contraction is switched off for this file and every fused
// operation is spelled out.
#include "n2_common.h"

#pragma clang fp contract(off)

constexpr float STEP = 1.73205080757f / 1024.f;  // STEPSIZE(), src/testbed_nerf.cu:51-53
constexpr uint32_t GRIDSIZE = 128, MARCH_STEPS = 1024;
__device__ __forceinline__ uint32_t hash_u32(uint32_t seed, uint32_t ctr) {
	uint32_t x = ctr * 747796405u + seed * 2891336453u + 1u;
	x = ((x >> ((x >> 28) + 4u)) ^ x) * 277803737u;
	x = (x >> 22) ^ x;
	x ^= x >> 16; x *= 0x7feb352du; x ^= x >> 15; x *= 0x846ca68bu; x ^= x >> 16;
	return x;
}
__device__ __forceinline__ float rand01(uint32_t seed, uint32_t ray, uint32_t k) {
	return (float)(hash_u32(seed, ray * 8u + k) >> 8) * (1.0f / 16777216.0f);
}
__device__ __forceinline__ uint32_t expand_bits(uint32_t v) {
	v = (v * 0x00010001u) & 0xFF0000FFu;
	v = (v * 0x00000101u) & 0x0F00F00Fu;
	v = (v * 0x00000011u) & 0xC30C30C3u;
	v = (v * 0x00000005u) & 0x49249249u;
	return v;
}
__device__ __forceinline__ bool occupied(const uint8_t* __restrict__ bitfield, const float* pos) {
	int c[3];
#pragma unroll
	for (int d = 0; d < 3; ++d) {
		float p = pos[d] - 0.5f;
		p = p * 1.0f;
		p = p + 0.5f;
		const int i = (int)(p * (float)GRIDSIZE);
		c[d] = min(max(i, 0), (int)GRIDSIZE - 1);
	}
	const uint32_t idx = expand_bits((uint32_t)c[0]) | (expand_bits((uint32_t)c[1]) << 1) | (expand_bits((uint32_t)c[2]) << 2);
	return (bitfield[idx / 8] >> (idx % 8)) & 1;
}
__device__ __forceinline__ float to_next_voxel(const float* pos, const float* dir, const float* idir) {
	float t = 3.4e38f;
#pragma unroll
	for (int d = 0; d < 3; ++d) {
		const float p = (float)GRIDSIZE * pos[d];
		const float sgn = copysignf(1.0f, dir[d]);
		const float td = (floorf(p + 0.5f + 0.5f * sgn) - p) * idir[d];
		t = fminf(t, td);
	}
	return fmaxf(__fdiv_rn(t, (float)GRIDSIZE), 0.0f);
}

struct RaySetup {
	bool alive;
	float o[3], dir[3], idir[3], startt, target[3];
	float tmax;  // where the ray leaves the unit cube (below startt: it misses the cube)
};

// A coarse, dilated copy of the bitfield's first level, rebuilt by every sample generation: bit x + 32 y + 1024 z is set
// when any of the 4^3 cells of coarse cell (x, y, z) or of its 26 neighbours is occupied.  The march uses it to leave out,
// for certain, what cannot hold a sample: rays that pass no occupied cell at all, and the part of a ray behind the last
// occupied cell it can reach.  (In morton order the 64 cells of an aligned 4^3 block are 64 consecutive bits.)
constexpr uint32_t COARSE = 32, COARSE_WORDS = COARSE * COARSE * COARSE / 32;
__global__ void __launch_bounds__(256) sampler_coarse_kernel(const uint8_t* __restrict__ bitfield, uint32_t* __restrict__ coarse) {
	const uint32_t cell = blockIdx.x * 256u + threadIdx.x;  // x + 32 y + 1024 z
	const int x = (int)(cell % COARSE), y = (int)((cell / COARSE) % COARSE), z = (int)(cell / (COARSE * COARSE));
	const unsigned long long* blocks = reinterpret_cast<const unsigned long long*>(bitfield);
	bool any = false;
#pragma unroll
	for (int dz = -1; dz <= 1; ++dz)
#pragma unroll
		for (int dy = -1; dy <= 1; ++dy)
#pragma unroll
			for (int dx = -1; dx <= 1; ++dx) {
				const int nx = x + dx, ny = y + dy, nz = z + dz;
				// (every load is issued whatever the others return: a neighbour outside the cube reads the cell itself)
				const bool out = nx < 0 || ny < 0 || nz < 0 || nx >= (int)COARSE || ny >= (int)COARSE || nz >= (int)COARSE;
				const uint32_t ux = out ? (uint32_t)x : (uint32_t)nx, uy = out ? (uint32_t)y : (uint32_t)ny, uz = out ? (uint32_t)z : (uint32_t)nz;
				const uint32_t m = expand_bits(ux) | (expand_bits(uy) << 1) | (expand_bits(uz) << 2);
				any |= blocks[m] != 0ull;
			}
	const unsigned long long bits = __ballot(any);
	if ((threadIdx.x & 63u) == 0) { coarse[cell / 32u] = (uint32_t)bits; coarse[cell / 32u + 1u] = (uint32_t)(bits >> 32); }
}

__device__ __forceinline__ RaySetup setup_ray(uint32_t i, uint32_t n_rays, uint32_t n_rays_total, uint32_t seed,
                                              const n2_camera* __restrict__ cams, uint32_t n_images, const float* __restrict__ rgba,
                                              float bg0, float bg1, float bg2) {
	RaySetup r;
	const uint32_t img = (((i + n_rays_total) * n_images) / n_rays) % n_images;
	const n2_camera c = cams[img];
	const float u0 = rand01(seed, i, 0), u1 = rand01(seed, i, 1);
	const int px = min(max((int)(u0 * (float)c.resolution[0]), 0), (int)c.resolution[0] - 1);
	const int py = min(max((int)(u1 * (float)c.resolution[1]), 0), (int)c.resolution[1] - 1);
	const float x = __fdiv_rn((float)px + 0.5f, (float)c.resolution[0]), y = __fdiv_rn((float)py + 0.5f, (float)c.resolution[1]);
	const uint64_t off = ((uint64_t)c.pixel_offset_hi << 32) | c.pixel_offset_lo;
	const float4 pix = *reinterpret_cast<const float4*>(rgba + (off + (uint64_t)px + (uint64_t)py * c.resolution[0]) * 4);
	if (pix.x <= 0.0f && rand01(seed, i, 2) >= 0.9f) {
		r.alive = false;
		return r;
	}
	const float bg[3] = {bg0, bg1, bg2};
	const float pc[3] = {pix.x, pix.y, pix.z};
#pragma unroll
	for (int k = 0; k < 3; ++k) r.target[k] = pc[k] + (1.0f - pix.w) * bg[k];
	const float d[3] = {__fdiv_rn((x - c.principal_point[0]) * (float)c.resolution[0], c.focal_length[0]),
	                    __fdiv_rn((y - c.principal_point[1]) * (float)c.resolution[1], c.focal_length[1]), 1.0f};
	float w[3];
#pragma unroll
	for (int k = 0; k < 3; ++k) {
		w[k] = __fmaf_rn(c.xform[k * 4 + 2], d[2], __fmaf_rn(c.xform[k * 4 + 1], d[1], c.xform[k * 4 + 0] * d[0]));
		r.o[k] = c.xform[k * 4 + 3];
	}
	const float len = sqrtf(__fmaf_rn(w[2], w[2], __fmaf_rn(w[1], w[1], w[0] * w[0])));
#pragma unroll
	for (int k = 0; k < 3; ++k) { r.dir[k] = __fdiv_rn(w[k], len); r.idir[k] = __fdiv_rn(1.0f, r.dir[k]); }
	float tmin = __fdiv_rn(0.f - r.o[0], r.dir[0]), tmax = __fdiv_rn(1.f - r.o[0], r.dir[0]);
	if (tmin > tmax) { const float t = tmin; tmin = tmax; tmax = t; }
	bool hit = true;
	for (int k = 1; k < 3 && hit; ++k) {
		float a = __fdiv_rn(0.f - r.o[k], r.dir[k]), b = __fdiv_rn(1.f - r.o[k], r.dir[k]);
		if (a > b) { const float t = a; a = b; b = t; }
		if (tmin > b || a > tmax) { hit = false; break; }
		if (a > tmin) tmin = a;
		if (b < tmax) tmax = b;
	}
	if (!hit) tmin = 3.402823466e38f;
	r.tmax = hit ? tmax : -1.0f;
	tmin = fmaxf(tmin, 0.0f);
	r.startt = __fmaf_rn(STEP, rand01(seed, i, 3), tmin);
	r.alive = true;
	return r;
}

// The march of one ray, as the reference writes it: t_0 = startt, every visited step adds STEP to t; at an occupied
// step a sample is emitted, at an empty one the steps below t + to_next_voxel(pos) are skipped without being looked at;
// the ray ends at the first visited step outside the unit cube or after MARCH_STEPS samples.  One lane per ray makes
// that a chain of dependent bitfield reads (0.4 us per step, a few thousand lanes on the whole GPU).  Here a WAVE owns a
// ray and looks at 64 consecutive steps at once: every lane forms its own t, position, occupancy bit and skip target
// with the serial form's arithmetic, and the wave then replays the serial decisions on the ballots (which steps are
// visited, which emit, where the ray ends).  The result is the serial one bit for bit; the bitfield latency is paid
// once per 64 steps.  The march runs once: it records which steps emitted (64 bits per window) and the t of every
// window's first step; the coordinates are written afterwards from those, without touching the bitfield.
constexpr uint32_t WINDOWS = 17;                      // 1088 steps: a ray inside the unit cube is at most sqrt(3) long,
                                                      // i.e. MARCH_STEPS steps plus the start jitter
constexpr uint32_t RAYS_PER_BLOCK = 4;                // one wave per ray

// t of this lane's step: t_first plus `lane` additions of STEP, one at a time like the serial march.  Inside a binade
// [2^e, 2^(e+1)) every such addition moves t by the same amount d_e = (2^e + STEP) - 2^e: t is a multiple of the
// binade's ulp and STEP's remainder below that ulp rounds the same way each time (STEP has no tie in any binade
// above 2^-8), so t_k = t_0 + k d_e exactly, as long as the binade is not left.  64 steps are shorter than any binade
// from 2^-3 up, so a window crosses at most one boundary: the lanes behind it continue from the one real addition that
// crosses it with the next binade's increment.  Below 2^-3 (a camera inside the volume) the additions are done one by one.
// Must be called by all 64 lanes.
// What window_t found: with `linear` set, the t of step k of the window is window_step(w, t_first, k) for any k in 0..63.
struct WindowShape {
	bool linear;   // false: the additions were done one by one (no closed form)
	uint32_t kc;   // steps 0 .. kc-1 lie in the binade of t_first (64: all of them)
	float d1, d2, t_cross;
};
__device__ __forceinline__ float window_step(const WindowShape& w, float t_first, uint32_t k) {
	return k < w.kc ? __fmaf_rn((float)k, w.d1, t_first) : __fmaf_rn((float)(k - w.kc), w.d2, w.t_cross);
}
__device__ __forceinline__ float window_t(float t_first, uint32_t lane, WindowShape& w) {
	w.linear = t_first >= 0.125f && t_first < 1e30f;
	w.kc = 64u; w.d1 = STEP; w.d2 = STEP; w.t_cross = 3.4e38f;
	if (!w.linear) {
		float t = t_first;
		for (uint32_t a = 0; a < lane; ++a) t += STEP;
		return t;
	}
	const float lo = __uint_as_float(__float_as_uint(t_first) & 0x7F800000u), hi = lo + lo;
	w.d1 = (lo + STEP) - lo;
	w.d2 = (hi + STEP) - hi;
	const float x = __fmaf_rn((float)lane, w.d1, t_first);  // exact below hi; at or above hi only the comparison is used
	const unsigned long long below = __ballot(x < hi);       // lanes 0 .. kc-1 (lane 0 always)
	w.kc = (uint32_t)__popcll(below);
	if (w.kc == 64u) return x;
	w.t_cross = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(x), (int)w.kc - 1)) + STEP;
	return lane < w.kc ? x : __fmaf_rn((float)(lane - w.kc), w.d2, w.t_cross);
}
__device__ __forceinline__ float window_t(float t_first, uint32_t lane) {
	WindowShape w;
	return window_t(t_first, lane, w);
}

// Returns the number of samples; mask[2 w], mask[2 w + 1]: which steps of window w emitted; t_first[w]: t of its first step.
__device__ __forceinline__ uint32_t march_wave(const RaySetup& r, const uint8_t* __restrict__ bitfield, const uint32_t* __restrict__ coarse,
                                               uint32_t* __restrict__ mask, float* __restrict__ t_first_out) {
	const uint32_t lane = threadIdx.x & 63u;
	uint32_t j = 0;
	float t_first = r.startt;  // t of the window's first step
	float pending = -3.4e38f;  // steps with t below this are skipped (target of the last visited empty step)
	// Where the march may stop.  The stretch of the ray inside the cube is cut into 64 pieces, one per lane; a piece is at
	// most sqrt(3) / 64 long, less than a coarse cell (1 / 32), so every point of it lies in the coarse cell of its
	// midpoint or in a neighbour of that cell: when the dilated bit of the midpoint's cell is clear, no step of the piece is
	// occupied.  No bit set: the ray has no sample.  Else no step behind the last piece with a set bit is occupied: the
	// serial march would only walk on to the cube's far side without emitting anything, so it ends there with the same
	// samples.  (A ray outside these assumptions marches all the way.)
	float t_stop = 3.4e38f;
	if (coarse != nullptr && r.tmax > r.startt && r.startt >= 0.f && r.tmax - r.startt < 2.0f) {
		const float piece = (r.tmax - r.startt) * (1.0f / 64.0f);
		const float tm = r.startt + ((float)lane + 0.5f) * piece;
		uint32_t c[3];
#pragma unroll
		for (int k = 0; k < 3; ++k) c[k] = (uint32_t)min(max((int)((tm * r.dir[k] + r.o[k]) * (float)COARSE), 0), (int)COARSE - 1);
		const uint32_t cell = c[0] + COARSE * c[1] + COARSE * COARSE * c[2];
		const unsigned long long maybe = __ballot((coarse[cell >> 5] >> (cell & 31u)) & 1u);
		if (maybe == 0ull) return 0u;
		t_stop = r.startt + ((float)(64 - (int)__clzll((long long)maybe)) + 0.5f) * piece;
	}
	for (uint32_t w = 0; w < WINDOWS; ++w) {
		if (t_first > t_stop) break;  // nothing behind this point can emit
		WindowShape ws;
		const float t = window_t(t_first, lane, ws);
		float pos[3];
#pragma unroll
		for (int k = 0; k < 3; ++k) pos[k] = __fmaf_rn(t, r.dir[k], r.o[k]);
		const bool inside = pos[0] >= 0.f && pos[0] <= 1.f && pos[1] >= 0.f && pos[1] <= 1.f && pos[2] >= 0.f && pos[2] <= 1.f;
		const bool occ = inside && occupied(bitfield, pos);
		const float target = t + to_next_voxel(pos, r.dir, r.idir);
		const unsigned long long m_inside = __ballot(inside), m_occ = __ballot(occ);
		// replay the serial walk over this window (all values below are the same in every lane)
		unsigned long long emit = 0;
		bool done = false;
		const unsigned long long reach = __ballot(t >= pending);  // steps not skipped by the pending target
		uint32_t cur = reach ? (uint32_t)__ffsll((long long)reach) - 1u : 64u;
		// The walk without a loop.  Every lane works out the step the serial walk would visit after its own: the end of
		// its run for an occupied step, the first later step whose t reaches its target for an empty one (estimated by a
		// division, then checked against the exact t of the steps around the estimate).  Steps fall into groups that
		// share that successor; when every group's successor is the step right behind the group, the walk, wherever it
		// enters a group, leaves it for the first step of the next one: it visits every occupied step from `cur` on and
		// the first step of every empty group, and the last of those sets the pending target.  A window where that does
		// not hold (a step next to a voxel face that the two tests place differently), one that leaves the unit cube or
		// reaches the sample limit, or one without the closed form of t takes the loop below.
		bool walked = false;
		if (cur < 64u && ws.linear) {
			const unsigned long long ge = ~0ull << cur;
			if ((~m_inside & ge) == 0ull && j + (uint32_t)__popcll(m_occ & ge) < MARCH_STEPS) {
				uint32_t nxt;
				bool good = true;
				if (occ) {
					const unsigned long long rest = ~(m_occ >> lane);  // bit 64 - lane and up are set: the run ends inside the window or at its end
					nxt = lane + min((uint32_t)__ffsll((long long)rest) - 1u, 64u - lane);
				} else {
					const bool second = target >= ws.t_cross;
					const float est = second ? __fdividef(target - ws.t_cross, ws.d2) + (float)ws.kc : __fdividef(target - t_first, ws.d1);
					uint32_t k0 = (uint32_t)fminf(fmaxf(ceilf(est), 0.f), 64.f);
					if (k0 > 0u && window_step(ws, t_first, k0 - 1u) >= target) --k0;
					if (k0 < 64u && window_step(ws, t_first, k0) < target) ++k0;
					good = (k0 == 0u || window_step(ws, t_first, k0 - 1u) < target) && (k0 == 64u || window_step(ws, t_first, k0) >= target);
					nxt = max(k0, lane + 1u);  // the serial form always moves on by at least one step
				}
				const uint32_t nxt_up = (uint32_t)__shfl_down((int)nxt, 1);
				const bool occ_up = (m_occ >> ((lane + 1u) & 63u)) & 1ull;
				const bool chained = nxt == lane + 1u || (occ == occ_up && nxt == nxt_up);
				const unsigned long long bad = __ballot(lane >= cur && (!good || (lane < 63u && !chained)));
				if (bad == 0ull) {
					walked = true;
					emit = m_occ & ge;
					j += (uint32_t)__popcll(emit);
					const unsigned long long ends = __ballot(nxt == lane + 1u);
					const unsigned long long firsts = ((ends << 1) | (1ull << cur)) & ge & ~m_occ;  // visited empty steps
					if (firsts) pending = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(target), 63 - (int)__clzll((long long)firsts)));
				}
			}
		}
		while (!walked && cur < 64u) {
			if (!((m_inside >> cur) & 1ull)) { done = true; break; }
			if ((m_occ >> cur) & 1ull) {
				// a run of occupied steps: each emits and moves on by one step
				const unsigned long long rest = ~(m_occ >> cur);
				uint32_t run = rest ? (uint32_t)__ffsll((long long)rest) - 1u : 64u - cur;
				if (run > 64u - cur) run = 64u - cur;
				if (run > MARCH_STEPS - j) run = MARCH_STEPS - j;
				emit |= (run == 64u ? ~0ull : ((1ull << run) - 1ull)) << cur;
				j += run;
				cur += run;
				if (j >= MARCH_STEPS) { done = true; break; }
			} else {
				// an empty step: the next visited step is the first later one whose t reaches its target
				pending = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(target), (int)cur));
				const unsigned long long later = __ballot(t >= pending) & (cur == 63u ? 0ull : (~0ull << (cur + 1u)));
				// the serial form always moves on by at least one step
				cur = later ? (uint32_t)__ffsll((long long)later) - 1u : 64u;
			}
		}
		if (lane == 0) {
			mask[2 * w] = (uint32_t)emit;
			mask[2 * w + 1] = (uint32_t)(emit >> 32);
			t_first_out[w] = t_first;
		}
		if (done) break;
		// next window starts one step after this window's last one
		t_first = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(t), 63)) + STEP;
	}
	return j;
}

__global__ void __launch_bounds__(64 * RAYS_PER_BLOCK) sampler_count_kernel(uint32_t n_rays, uint32_t n_rays_total, uint32_t seed, const n2_camera* __restrict__ cams,
                                                            uint32_t n_images, const float* __restrict__ rgba, float bg0, float bg1, float bg2,
                                                            const uint8_t* __restrict__ bitfield, const uint32_t* __restrict__ coarse,
                                                            uint32_t* __restrict__ counts, uint32_t* __restrict__ mask, float* __restrict__ t_first,
                                                            uint32_t* __restrict__ ray_counter) {
	if (blockIdx.x == 0 && threadIdx.x == 0) *ray_counter = 0u;  // the scan kernel adds the kept rays up
	const uint32_t i = blockIdx.x * RAYS_PER_BLOCK + (threadIdx.x >> 6);
	if (i >= n_rays) return;
	const RaySetup r = setup_ray(i, n_rays, n_rays_total, seed, cams, n_images, rgba, bg0, bg1, bg2);
	const uint32_t n = r.alive ? march_wave(r, bitfield, coarse, mask + (size_t)i * 2 * WINDOWS, t_first + (size_t)i * WINDOWS) : 0u;
	if ((threadIdx.x & 63u) == 0) counts[i] = n;
}

// Sum of the counts and number of non-zero counts of each block of 1024 consecutive rays.
__global__ void __launch_bounds__(1024) sampler_block_totals_kernel(uint32_t n_rays, const uint32_t* __restrict__ counts,
                                                                    uint32_t* __restrict__ block_sum, uint32_t* __restrict__ block_nz) {
	__shared__ uint32_t ws[16], wn[16];
	const uint32_t r = blockIdx.x * 1024u + threadIdx.x;
	const uint32_t k = r < n_rays ? counts[r] : 0u;
	uint32_t sum = k, nz = k ? 1u : 0u;
#pragma unroll
	for (int o = 32; o > 0; o >>= 1) { sum += __shfl_xor(sum, o); nz += __shfl_xor(nz, o); }
	if ((threadIdx.x & 63u) == 0) { ws[threadIdx.x >> 6] = sum; wn[threadIdx.x >> 6] = nz; }
	__syncthreads();
	if (threadIdx.x == 0) {
		uint32_t a = 0, c = 0;
#pragma unroll
		for (int w = 0; w < 16; ++w) { a += ws[w]; c += wn[w]; }
		block_sum[blockIdx.x] = a;
		block_nz[blockIdx.x] = c;
	}
}

// base[i] = exclusive sum of counts; slot[i] = rank among rays that have samples and fit the budget.  One workgroup per block
// of 1024 consecutive rays: it adds up the totals of the blocks before its own and scans its own counts.  The sums never
// decrease, so once a ray with samples does not fit, no later one does: if the counts before this block fit the budget,
// every earlier ray with samples was kept; if they do not, none of this block's rays is.  The number of kept rays is added
// up over the workgroups with an integer atomic (*ray_counter was cleared by the count kernel).
__global__ void __launch_bounds__(1024) sampler_scan_kernel(uint32_t n_rays, uint32_t max_samples, const uint32_t* __restrict__ counts,
                                                            const uint32_t* __restrict__ block_sum, const uint32_t* __restrict__ block_nz,
                                                            uint32_t* __restrict__ base, uint32_t* __restrict__ slot,
                                                            uint32_t* __restrict__ ray_counter, uint32_t* __restrict__ sample_counter) {
	__shared__ uint32_t before_a[16], before_nz[16], wt_a[16], wt_b[16];
	const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
	const uint32_t r = blockIdx.x * 1024u + threadIdx.x;
	const uint32_t k = r < n_rays ? counts[r] : 0u;
	uint32_t sum = 0, nz = 0;
	for (uint32_t q = threadIdx.x; q < blockIdx.x; q += 1024u) { sum += block_sum[q]; nz += block_nz[q]; }
#pragma unroll
	for (int o = 32; o > 0; o >>= 1) { sum += __shfl_xor(sum, o); nz += __shfl_xor(nz, o); }
	uint32_t v = k;
#pragma unroll
	for (int o = 1; o < 64; o <<= 1) { const uint32_t u = __shfl_up(v, o); if (lane >= o) v += u; }
	if (lane == 63) { before_a[wave] = sum; before_nz[wave] = nz; wt_a[wave] = v; }
	__syncthreads();
	uint32_t all_before = 0, kept_before = 0, before = 0;
#pragma unroll
	for (int w = 0; w < 16; ++w) { all_before += before_a[w]; kept_before += before_nz[w]; before += w < wave ? wt_a[w] : 0u; }
	const uint32_t excl = all_before + before + v - k;
	const uint32_t keep = (k > 0 && (uint64_t)excl + k <= max_samples) ? 1u : 0u;
	uint32_t f = keep;
#pragma unroll
	for (int o = 1; o < 64; o <<= 1) { const uint32_t u = __shfl_up(f, o); if (lane >= o) f += u; }
	if (lane == 63) wt_b[wave] = f;
	__syncthreads();
	uint32_t before_b = all_before <= max_samples ? kept_before : 0u, kept_here = 0;
#pragma unroll
	for (int w = 0; w < 16; ++w) { before_b += w < wave ? wt_b[w] : 0u; kept_here += wt_b[w]; }
	if (r < n_rays) {
		base[r] = excl;
		slot[r] = keep ? before_b + f - 1u : 0xFFFFFFFFu;
	}
	if (threadIdx.x == 0 && kept_here) atomicAdd(ray_counter, kept_here);
	if (threadIdx.x == 1023 && blockIdx.x + 1 == gridDim.x) *sample_counter = excl + k;
}

// Coordinates of the samples the march marked, one wave per ray: lane l of window w is the step at t_first[w] plus l
// additions of STEP, formed exactly as in the march.
__global__ void __launch_bounds__(64 * RAYS_PER_BLOCK) sampler_emit_kernel(uint32_t n_rays, uint32_t n_rays_total, uint32_t seed, const n2_camera* __restrict__ cams,
                                                           uint32_t n_images, const float* __restrict__ rgba, float bg0, float bg1, float bg2,
                                                           const uint32_t* __restrict__ mask, const float* __restrict__ t_first,
                                                           const uint32_t* __restrict__ counts,
                                                           const uint32_t* __restrict__ base, const uint32_t* __restrict__ slot,
                                                           uint32_t* __restrict__ ray_indices, uint32_t* __restrict__ numsteps,
                                                           float* __restrict__ rgb_target, float* __restrict__ coords,
                                                           float* __restrict__ xyz_soa, uint32_t soa_pitch) {
	const uint32_t i = blockIdx.x * RAYS_PER_BLOCK + (threadIdx.x >> 6), lane = threadIdx.x & 63u;
	if (i >= n_rays) return;
	const uint32_t s = slot[i];
	if (s == 0xFFFFFFFFu) return;
	const RaySetup r = setup_ray(i, n_rays, n_rays_total, seed, cams, n_images, rgba, bg0, bg1, bg2);
	const uint32_t n = counts[i], first = base[i];
	if (lane == 0) {
		ray_indices[s] = i;
		numsteps[2 * s] = n;
		numsteps[2 * s + 1] = first;
		rgb_target[(size_t)s * 3 + 0] = r.target[0];
		rgb_target[(size_t)s * 3 + 1] = r.target[1];
		rgb_target[(size_t)s * 3 + 2] = r.target[2];
	}
	const float d0 = (r.dir[0] + 1.0f) * 0.5f, d1 = (r.dir[1] + 1.0f) * 0.5f, d2 = (r.dir[2] + 1.0f) * 0.5f;
	const uint32_t* m = mask + (size_t)i * 2 * WINDOWS;
	uint32_t j = 0;
	for (uint32_t w = 0; w < WINDOWS && j < n; ++w) {
		const unsigned long long bits = (unsigned long long)m[2 * w] | ((unsigned long long)m[2 * w + 1] << 32);
		if (bits == 0ull) continue;  // uniform: the whole wave skips the window
		const float t = window_t(t_first[(size_t)i * WINDOWS + w], lane);
		if ((bits >> lane) & 1ull) {
			const uint32_t at = first + j + (uint32_t)__popcll(bits & ((1ull << lane) - 1ull));
			float* c = coords + (size_t)at * 7;
			c[0] = __fmaf_rn(t, r.dir[0], r.o[0]);
			c[1] = __fmaf_rn(t, r.dir[1], r.o[1]);
			c[2] = __fmaf_rn(t, r.dir[2], r.o[2]);
			if (xyz_soa) {  // the positions once more as three rows: what a reader of positions alone wants
				xyz_soa[at] = c[0];
				xyz_soa[(size_t)soa_pitch + at] = c[1];
				xyz_soa[(size_t)2 * soa_pitch + at] = c[2];
			}
			c[3] = 0.0f;
			c[4] = d0; c[5] = d1; c[6] = d2;
		}
		j += (uint32_t)__popcll(bits);
	}
}

static inline uint64_t up256(uint64_t x) { return (x + 255) / 256 * 256; }

static inline uint32_t scan_blocks(uint32_t n_rays) { return (n_rays + 1023u) / 1024u; }

N2_API uint64_t n2_sampler_workspace_bytes(uint32_t max_rays) {
	return 3 * up256(4ull * max_rays) + 2 * up256(4ull * 2 * WINDOWS * max_rays) + 2 * up256(4ull * scan_blocks(max_rays)) + up256(4ull * COARSE_WORDS);
}

N2_API int n2_generate_training_samples(n2_stream_t stream, uint32_t n_rays, uint32_t n_rays_total, uint32_t seed,
                                        const n2_camera* d_cameras, uint32_t n_images, const float* d_rgba,
                                        const float background[3], const uint8_t* d_bitfield, uint32_t max_samples,
                                        uint32_t* d_ray_counter, uint32_t* d_sample_counter, uint32_t* d_ray_indices,
                                        uint32_t* d_numsteps, float* d_rgb_target, float* d_coords, void* d_workspace,
                                        uint64_t workspace_bytes) {
	return n2_generate_training_samples_rows(stream, n_rays, n_rays_total, seed, d_cameras, n_images, d_rgba, background, d_bitfield, max_samples, d_ray_counter,
	                                         d_sample_counter, d_ray_indices, d_numsteps, d_rgb_target, d_coords, d_workspace, workspace_bytes, nullptr);
}

int n2_generate_training_samples_rows(n2_stream_t stream, uint32_t n_rays, uint32_t n_rays_total, uint32_t seed,
                                      const n2_camera* d_cameras, uint32_t n_images, const float* d_rgba,
                                      const float background[3], const uint8_t* d_bitfield, uint32_t max_samples,
                                      uint32_t* d_ray_counter, uint32_t* d_sample_counter, uint32_t* d_ray_indices,
                                      uint32_t* d_numsteps, float* d_rgb_target, float* d_coords, void* d_workspace,
                                      uint64_t workspace_bytes, float* d_xyz_rows) {
	N2_REQUIRE(d_ray_counter && d_sample_counter, "n2_generate_training_samples: counters are null");
	hipStream_t s = n2_stream(stream);
	if (n_rays == 0) {
		if (int rc = n2_set_u32(s, d_ray_counter, 0u)) return rc;
		return n2_set_u32(s, d_sample_counter, 0u);
	}
	N2_REQUIRE(d_cameras && d_rgba && background && d_bitfield && d_ray_indices && d_numsteps && d_rgb_target && d_coords && d_workspace,
	           "n2_generate_training_samples: null buffer");
	N2_REQUIRE(n_images > 0, "n2_generate_training_samples: n_images must be positive");
	N2_REQUIRE(reinterpret_cast<uintptr_t>(d_rgba) % 16 == 0, "n2_generate_training_samples: d_rgba must be 16-byte aligned");
	N2_REQUIRE(workspace_bytes >= n2_sampler_workspace_bytes(n_rays), "n2_generate_training_samples: workspace of %llu bytes, %llu needed",
	           (unsigned long long)workspace_bytes, (unsigned long long)n2_sampler_workspace_bytes(n_rays));
	unsigned char* w = reinterpret_cast<unsigned char*>(d_workspace);
	uint32_t* counts = reinterpret_cast<uint32_t*>(w);
	uint32_t* base = reinterpret_cast<uint32_t*>(w + up256(4ull * n_rays));
	uint32_t* slot = reinterpret_cast<uint32_t*>(w + 2 * up256(4ull * n_rays));
	uint32_t* mask = reinterpret_cast<uint32_t*>(w + 3 * up256(4ull * n_rays));
	float* t_first = reinterpret_cast<float*>(w + 3 * up256(4ull * n_rays) + up256(4ull * 2 * WINDOWS * n_rays));
	uint32_t* block_sum = reinterpret_cast<uint32_t*>(w + 3 * up256(4ull * n_rays) + 2 * up256(4ull * 2 * WINDOWS * n_rays));
	uint32_t* block_nz = block_sum + up256(4ull * scan_blocks(n_rays)) / 4;
	uint32_t* coarse = block_nz + up256(4ull * scan_blocks(n_rays)) / 4;
	const dim3 grid((n_rays + RAYS_PER_BLOCK - 1) / RAYS_PER_BLOCK), block(64 * RAYS_PER_BLOCK);
	N2ProfScope prof(N2_PROF_SAMPLER, s);
	N2_REQUIRE(reinterpret_cast<uintptr_t>(d_bitfield) % 8 == 0, "n2_generate_training_samples: d_bitfield must be 8-byte aligned");
	sampler_coarse_kernel<<<dim3(COARSE * COARSE * COARSE / 256), dim3(256), 0, s>>>(d_bitfield, coarse);
	N2_LAUNCH_CHECK();
	sampler_count_kernel<<<grid, block, 0, s>>>(n_rays, n_rays_total, seed, d_cameras, n_images, d_rgba, background[0], background[1],
	                                            background[2], d_bitfield, coarse, counts, mask, t_first, d_ray_counter);
	N2_LAUNCH_CHECK();
	sampler_block_totals_kernel<<<dim3(scan_blocks(n_rays)), dim3(1024), 0, s>>>(n_rays, counts, block_sum, block_nz);
	N2_LAUNCH_CHECK();
	sampler_scan_kernel<<<dim3(scan_blocks(n_rays)), dim3(1024), 0, s>>>(n_rays, max_samples, counts, block_sum, block_nz, base, slot, d_ray_counter,
	                                                                 d_sample_counter);
	N2_LAUNCH_CHECK();
	sampler_emit_kernel<<<grid, block, 0, s>>>(n_rays, n_rays_total, seed, d_cameras, n_images, d_rgba, background[0], background[1],
	                                           background[2], mask, t_first, counts, base, slot, d_ray_indices, d_numsteps, d_rgb_target, d_coords,
	                                           d_xyz_rows, max_samples);
	N2_LAUNCH_CHECK();
	return N2_OK;
}
