// NeuS alpha compositing, colour loss and backward to the network outputs.
//
// One wavefront owns one ray and walks it 64 samples at a time: each lane loads
// one sample's 16 fp16 outputs (32 contiguous bytes), the transmittance before
// every sample is an exclusive product scan of (1 - alpha) across the wave,
// composited colour and the prefix the backward needs are wave reductions /
// inclusive scans.  Three kernels: forward (how many samples each ray keeps and
// its colour), an exclusive scan over rays that hands out compacted ranges in
// ray order, backward (gradients and compacted coordinates).
#include "n2_common.h"

#include <mutex>

typedef _Float16 hf;
typedef _Float16 half8 __attribute__((ext_vector_type(8)));

struct CompParams {
	float loss_scale, ek_loss_weight, anneal;
	float bg[3];
	float inv_n_rays;
	float min_step, max_step;
};

struct Sample {
	float alpha, p_div_c, iter_cos, true_cos, inv_s, dt, next_sdf;
	float rgb[3], n[3], raw[3];
};

__device__ __forceinline__ float logistic(float x) { return 1.f / (1.f + __expf(-x)); }

__device__ __forceinline__ void load_out(const hf* __restrict__ net_out, size_t s, float* o) {
	const half8 a = *reinterpret_cast<const half8*>(net_out + s * 16);
	const half8 b = *reinterpret_cast<const half8*>(net_out + s * 16 + 8);
#pragma unroll
	for (int k = 0; k < 8; ++k) { o[k] = (float)a[k]; o[8 + k] = (float)b[k]; }
}

__device__ __forceinline__ Sample eval_sample(const float* o, hf var_h, float warped_dt, const float* dir, const CompParams& c) {
	Sample s;
	s.dt = warped_dt * (c.max_step - c.min_step) + c.min_step;
#pragma unroll
	for (int k = 0; k < 3; ++k) { s.raw[k] = o[k]; s.rgb[k] = logistic(o[k]); s.n[k] = o[4 + k]; }
	s.inv_s = __expf((float)((hf)10.0f * var_h));  // product formed in half precision
	const float sdf = o[3];
	s.true_cos = dir[0] * s.n[0] + dir[1] * s.n[1] + dir[2] * s.n[2];
	const float a = fmaxf(-s.true_cos * 0.5f + 0.5f, 0.f), b = fmaxf(-s.true_cos, 0.f);
	s.iter_cos = -(a * (1.f - c.anneal) + b * c.anneal);
	s.next_sdf = sdf + s.iter_cos * s.dt * 0.5f;
	const float prev_sdf = sdf - s.iter_cos * s.dt * 0.5f;
	const float next_cdf = logistic(s.next_sdf * s.inv_s), prev_cdf = logistic(prev_sdf * s.inv_s);
	s.p_div_c = (prev_cdf - next_cdf + 1e-5f) / (prev_cdf + 1e-5f);
	s.alpha = fminf(fmaxf(s.p_div_c, 0.f), 1.f);
	return s;
}

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
	for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o);
	return v;
}
// exclusive product scan over the 64 lanes
__device__ __forceinline__ float wave_excl_prod(float v, int lane) {
#pragma unroll
	for (int o = 1; o < 64; o <<= 1) {
		const float u = __shfl_up(v, o);
		if (lane >= o) v *= u;
	}
	const float e = __shfl_up(v, 1);
	return lane == 0 ? 1.f : e;
}
__device__ __forceinline__ float wave_incl_sum(float v, int lane) {
#pragma unroll
	for (int o = 1; o < 64; o <<= 1) {
		const float u = __shfl_up(v, o);
		if (lane >= o) v += u;
	}
	return v;
}

// direction of the ray: rows 8..10 of its first sample, unwarped and normalised
__device__ __forceinline__ void ray_dir(const hf* __restrict__ net_out, size_t base, float* dir) {
	const hf* o = net_out + base * 16;
	const float x = (float)o[8] * 2.f - 1.f, y = (float)o[9] * 2.f - 1.f, z = (float)o[10] * 2.f - 1.f;
	const float len = sqrtf(x * x + y * y + z * z);
	dir[0] = x / len; dir[1] = y / len; dir[2] = z / len;
}

struct RayScratch {
	float rgb[3];
	uint32_t kept;
};

constexpr float T_EPS = 1e-4f;
constexpr int CB = 256;  // 4 rays per workgroup

// THE factor of fill_rollover_and_rescale (tcnn; called at src/testbed_nerf.cu:3908-3910 with n_elements = the target
// batch size and stride = the padded output width): a wrapped copy of an output gradient is the original times
// n_in / n_total, rows over rows, whatever the stride.  tiny-cuda-nn's source is not part of the reference tree, so this
// reading is recalled, not checked: it is the only place in the library that holds it (the CPU oracle has the same one
// function, orc_rollover_rescaled).  Two roundings, as written: the product first.
__host__ __device__ __forceinline__ float rollover_rescaled(float value, uint32_t n_in, uint32_t n_total, uint32_t stride) {
	(void)stride;
	return value * (float)n_in / (float)n_total;
}

__global__ void __launch_bounds__(CB) composite_forward_kernel(CompParams c, uint32_t n_rays, const uint32_t* __restrict__ ray_counter,
                                                               const uint32_t* __restrict__ numsteps, const hf* __restrict__ net_out,
                                                               const float* __restrict__ coords, RayScratch* __restrict__ scratch,
                                                               uint32_t* __restrict__ kept_of, uint32_t* __restrict__ kept_of_block) {
	const int lane = threadIdx.x & 63;
	const uint32_t ray = blockIdx.x * (CB / 64) + (threadIdx.x >> 6);
	const uint32_t live = ray_counter ? min(*ray_counter, n_rays) : n_rays;
	uint32_t kept = 0;
	if (ray < n_rays && ray >= live) {
		if (lane == 0) { scratch[ray] = RayScratch{{0.f, 0.f, 0.f}, 0u}; kept_of[ray] = 0u; }
	} else if (ray < n_rays) {
		const uint32_t n = numsteps[2 * ray], base = numsteps[2 * ray + 1];
		float dir[3] = {0.f, 0.f, 0.f};
		if (n > 0) ray_dir(net_out, base, dir);
		float T = 1.f, r0 = 0.f, r1 = 0.f, r2 = 0.f;
		for (uint32_t c0 = 0; c0 < n; c0 += 64) {
			const uint32_t s = c0 + lane;
			const bool valid = s < n;
			float alpha = 0.f, rgb[3] = {0.f, 0.f, 0.f};
			if (valid) {
				float o[16];
				load_out(net_out, (size_t)base + s, o);
				const Sample sm = eval_sample(o, net_out[((size_t)base + s) * 16 + 7], coords[((size_t)base + s) * 7 + 3], dir, c);
				alpha = sm.alpha; rgb[0] = sm.rgb[0]; rgb[1] = sm.rgb[1]; rgb[2] = sm.rgb[2];
			}
			const float Tb = T * wave_excl_prod(1.f - alpha, lane);
			// samples are consumed while the transmittance before them is >= 1e-4
			const unsigned long long stop = __ballot(!valid || Tb < T_EPS);
			const int n_proc = stop ? (int)__ffsll((long long)stop) - 1 : 64;
			// (samples behind the cut contribute exact zeros whatever their outputs hold: with a forward pass in depth chunks
			// those outputs were never written)
			const bool in = lane < n_proc;
			const float w = in ? alpha * Tb : 0.f;
			r0 += wave_sum(in ? w * rgb[0] : 0.f);
			r1 += wave_sum(in ? w * rgb[1] : 0.f);
			r2 += wave_sum(in ? w * rgb[2] : 0.f);
			kept += n_proc;
			if (n_proc > 0) T = __shfl(Tb * (1.f - alpha), n_proc - 1);
			if (n_proc < 64) break;
		}
		if (kept == n) { r0 += T * c.bg[0]; r1 += T * c.bg[1]; r2 += T * c.bg[2]; }
		if (lane == 0) { scratch[ray] = RayScratch{{r0, r1, r2}, kept}; kept_of[ray] = kept; }
	}
	// the workgroup's count: the backward kernel adds up a quarter as many values to place its rays in the batch
	if (kept_of_block) {
		__shared__ uint32_t wave_kept[CB / 64];
		if (lane == 0) wave_kept[threadIdx.x >> 6] = kept;
		__syncthreads();
		if (threadIdx.x == 0) {
			uint32_t sum = 0;
#pragma unroll
			for (int w = 0; w < CB / 64; ++w) sum += wave_kept[w];
			kept_of_block[blockIdx.x] = sum;
		}
	}
}

// before_of[r] = kept_of[0] + ... + kept_of[r - 1].  One workgroup per 1024 consecutive rays: it adds up the counts of all
// rays before its own (coalesced, sixteen loads in flight per thread) and scans its own 1024 counts (lane shifts, the sixteen
// wave totals through LDS).
constexpr uint32_t OFFSETS_BLOCK = 1024;
constexpr uint32_t OFFSETS_MIN_RAYS = 8192;
__global__ void __launch_bounds__(OFFSETS_BLOCK) composite_offsets_kernel(uint32_t n_rays, const uint32_t* __restrict__ kept_of,
                                                                          uint32_t* __restrict__ before_of) {
	__shared__ uint32_t wave_before[OFFSETS_BLOCK / 64], wave_total[OFFSETS_BLOCK / 64];
	const uint32_t lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
	const uint32_t first = blockIdx.x * OFFSETS_BLOCK, ray = first + threadIdx.x;
	const uint32_t own = ray < n_rays ? kept_of[ray] : 0u;
	uint32_t before = 0;
	for (uint32_t r0 = 0; r0 < first; r0 += 16 * OFFSETS_BLOCK) {
		uint32_t v[16];
#pragma unroll
		for (uint32_t u = 0; u < 16; ++u) {
			const uint32_t r = r0 + u * OFFSETS_BLOCK + threadIdx.x;
			v[u] = r < first ? kept_of[r] : 0u;
		}
#pragma unroll
		for (uint32_t u = 0; u < 16; ++u) before += v[u];
	}
#pragma unroll
	for (int o = 32; o > 0; o >>= 1) before += __shfl_xor(before, o);
	uint32_t incl = own;
#pragma unroll
	for (int o = 1; o < 64; o <<= 1) {
		const uint32_t up = __shfl_up(incl, o);
		if ((int)lane >= o) incl += up;
	}
	if (lane == 63u) { wave_before[wave] = before; wave_total[wave] = incl; }
	__syncthreads();
	uint32_t base = 0;
#pragma unroll
	for (uint32_t w = 0; w < OFFSETS_BLOCK / 64; ++w) base += wave_before[w] + (w < wave ? wave_total[w] : 0u);
	if (ray < n_rays) before_of[ray] = base + incl - own;
}

__global__ void __launch_bounds__(CB) composite_backward_kernel(CompParams c, uint32_t n_rays, uint32_t* __restrict__ numsteps,
                                                                const hf* __restrict__ net_out, const float* __restrict__ coords,
                                                                const float* __restrict__ rgb_target, const RayScratch* __restrict__ scratch,
                                                                const uint32_t* __restrict__ kept_of, uint32_t max_compacted,
                                                                uint32_t* __restrict__ counter, float* __restrict__ coords_out,
                                                                hf* __restrict__ dloss, float* __restrict__ loss, uint32_t* __restrict__ source_index,
                                                                const uint32_t* __restrict__ before_of, uint32_t pad,
                                                                const uint32_t* __restrict__ kept_of_block, const uint32_t* __restrict__ column_of) {
	// column_of (or null): where the field stored what it saved for marched sample i (a forward pass in depth chunks stores
	// the samples it evaluates side by side); source_index then names that column
	const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
	// Where this workgroup's rays start in the compacted batch: the kept samples of all rays before them, in ray order
	// (deterministic).  With a few thousand rays every workgroup adds up the counts of its predecessors itself: a few KiB
	// of L2 reads each instead of a scan kernel in between.  That work grows with the square of the ray count, so beyond
	// OFFSETS_MIN_RAYS rays composite_offsets_kernel has left the sums in before_of.
	//
	// pad: the batch is also filled up to max_compacted samples here.  With n_in = min(all kept samples, max_compacted), slot
	// j >= n_in holds a copy of slot j % n_in whose output gradient is scaled by n_in / max_compacted (fill_rollover on the
	// coordinates, fill_rollover_and_rescale on the gradients, src/testbed_nerf.cu:3908-3916): the ray that writes slot p also
	// writes slots p + n_in, p + 2 n_in, ...  That needs the count of ALL rays, which the same loop adds up.
	__shared__ uint32_t part[CB / 64], part_all[CB / 64];
	const uint32_t first = blockIdx.x * (CB / 64);
	uint32_t before = 0, all = 0;
	// eight loads in flight per lane: the last workgroups add up thousands of counts, and one dependent L2 round trip per
	// CB of them was most of this kernel's duration
	// (kept_of_block: the forward kernel's counts per workgroup of CB / 64 rays, the same workgroups as here)
	const uint32_t n_counts = before_of ? 0u : (pad ? gridDim.x : blockIdx.x);
	for (uint32_t r0 = 0; r0 < n_counts; r0 += 8 * CB) {
		uint32_t v[8];
#pragma unroll
		for (uint32_t u = 0; u < 8; ++u) {
			const uint32_t r = r0 + u * CB + threadIdx.x;
			v[u] = r < n_counts ? kept_of_block[r] : 0u;
		}
#pragma unroll
		for (uint32_t u = 0; u < 8; ++u) {
			all += v[u];
			before += r0 + u * CB + threadIdx.x < blockIdx.x ? v[u] : 0u;
		}
	}
#pragma unroll
	for (int o = 32; o > 0; o >>= 1) { before += __shfl_xor(before, o); all += __shfl_xor(all, o); }
	if (lane == 0) { part[wave] = before; part_all[wave] = all; }
	__syncthreads();
	const uint32_t ray = first + wave;
	if (ray >= n_rays) return;
	uint32_t cb = 0, total = 0;
	if (before_of) {
		cb = before_of[ray];
		if (pad) total = before_of[n_rays - 1] + kept_of[n_rays - 1];
	} else {
#pragma unroll
		for (int w = 0; w < CB / 64; ++w) { cb += part[w]; total += part_all[w]; }
		for (int w = 0; w < wave; ++w) cb += kept_of[first + w];
	}
	const uint32_t n_in = min(total, max_compacted);  // pad: the samples the batch holds before it is filled up
	const uint32_t kept = kept_of[ray];
	const uint32_t m = min(max_compacted - min(max_compacted, cb), kept);  // the batch holds max_compacted samples
	if (ray == n_rays - 1 && lane == 0) *counter = cb + kept;
	const uint32_t base = numsteps[2 * ray + 1];
	const RayScratch rs = scratch[ray];
	// Huber(0.1)/5 per channel
	float grad[3], lsum = 0.f;
#pragma unroll
	for (int k = 0; k < 3; ++k) {
		const float d = rs.rgb[k] - rgb_target[(size_t)ray * 3 + k], ad = fabsf(d);
		lsum += (ad > 0.1f ? ad - 0.05f : 5.f * d * d) / 5.f;
		grad[k] = (ad > 0.1f ? (d > 0.f ? 1.f : -1.f) : d / 0.1f) / 5.f;
	}
	__builtin_amdgcn_wave_barrier();
	if (lane == 0) {
		numsteps[2 * ray] = m;
		numsteps[2 * ray + 1] = cb;
		if (loss) loss[ray] = m == 0 ? 0.f : lsum / 3.f * c.inv_n_rays;
	}
	if (m == 0) return;
	const float loss_scale = c.loss_scale * c.inv_n_rays;
	float dir[3];
	ray_dir(net_out, base, dir);
	float T = 1.f, p0 = 0.f, p1 = 0.f, p2 = 0.f;  // transmittance and colour prefix carried between chunks
	for (uint32_t c0 = 0; c0 < m; c0 += 64) {
		const uint32_t s = c0 + lane;
		const bool valid = s < m;
		Sample sm;
		sm.alpha = 0.f;
		hf var_h = (hf)0;
		if (valid) {
			float o[16];
			load_out(net_out, (size_t)base + s, o);
			var_h = net_out[((size_t)base + s) * 16 + 7];
			sm = eval_sample(o, var_h, coords[((size_t)base + s) * 7 + 3], dir, c);
		}
		const float alpha = valid ? sm.alpha : 0.f;
		const float Tb = T * wave_excl_prod(1.f - alpha, lane);
		const float w = valid ? alpha * Tb : 0.f;
		const float Ta = Tb * (1.f - alpha);
		const float q0 = p0 + wave_incl_sum(valid ? w * sm.rgb[0] : 0.f, lane);
		const float q1 = p1 + wave_incl_sum(valid ? w * sm.rgb[1] : 0.f, lane);
		const float q2 = p2 + wave_incl_sum(valid ? w * sm.rgb[2] : 0.f, lane);
		if (valid) {
			const float dot = grad[0] * (Ta * sm.rgb[0] - (rs.rgb[0] - q0)) + grad[1] * (Ta * sm.rgb[1] - (rs.rgb[1] - q1)) +
			                  grad[2] * (Ta * sm.rgb[2] - (rs.rgb[2] - q2));
			const float dloss_dalpha = dot / (1.f - alpha + 1e-5f);
			float da_dE = 0.f, dE_dsdf = 0.f, dE_dinvs = 0.f, da_dP = 0.f, dP_dinvs = 0.f, dP_dcos = 0.f, dE_dcos = 0.f;
			if (!(sm.p_div_c <= 0.f || sm.p_div_c >= 1.f)) {
				const float P = __expf(sm.inv_s * sm.iter_cos * sm.dt);
				const float E = __expf(-sm.next_sdf * sm.inv_s);
				const float a = 1.f + E, b = 1.f + P * E, cc = 1e-5f + 1.f / (1.f + P * E);
				const float delta = a * (b * b) * (cc * cc);
				da_dE = -(P / delta - 1.f / (a * a * cc));
				da_dP = -E / delta;
				dE_dsdf = -sm.inv_s * E;
				dE_dinvs = -sm.next_sdf * E;
				dP_dinvs = P * sm.iter_cos * sm.dt;
				dP_dcos = P * sm.inv_s * sm.dt;
				dE_dcos = -sm.inv_s * E * sm.dt * 0.5f;
			}
			const float dloss_dinvs = dloss_dalpha * (da_dE * dE_dinvs + da_dP * dP_dinvs);
			const float dloss_dvar = dloss_dinvs * sm.inv_s * 10.f;
			const float dcos = sm.true_cos >= 0.f ? 0.f : 1.f;
			const float gnorm = sqrtf(sm.n[0] * sm.n[0] + sm.n[1] * sm.n[1] + sm.n[2] * sm.n[2] + 1e-6f);
			const float ek = c.ek_loss_weight * 2.f * c.loss_scale * (1.f - 1.f / gnorm);
			const float dnorm = loss_scale * dloss_dalpha * (da_dE * dE_dcos + dP_dcos * da_dP) * dcos;
			half8 lo, hi;
#pragma unroll
			for (int k = 0; k < 3; ++k) lo[k] = (hf)(loss_scale * (w * grad[k] * sm.rgb[k] * (1.f - sm.rgb[k])));
			lo[3] = (hf)(loss_scale * dloss_dalpha * da_dE * dE_dsdf);
			lo[4] = (hf)(ek * sm.n[0]); lo[5] = (hf)(ek * sm.n[1]); lo[6] = (hf)(ek * sm.n[2]);
			lo[7] = (hf)(loss_scale * dloss_dvar);
			hi[0] = (hf)(dnorm * dir[0]); hi[1] = (hf)(dnorm * dir[1]); hi[2] = (hf)(dnorm * dir[2]);
#pragma unroll
			for (int k = 3; k < 8; ++k) hi[k] = (hf)0;
			// The rows are pinned in registers here: the copies that fill the batch up are formed from these fp16 values, and a
			// second evaluation of the expressions above (which the compiler is free to contract differently) rounds to
			// another fp16 value in a few cases per million.
			{
				uint4 lb = __builtin_bit_cast(uint4, lo), hb = __builtin_bit_cast(uint4, hi);
				asm volatile("" : "+v"(lb.x), "+v"(lb.y), "+v"(lb.z), "+v"(lb.w), "+v"(hb.x), "+v"(hb.y), "+v"(hb.z), "+v"(hb.w));
				lo = __builtin_bit_cast(half8, lb); hi = __builtin_bit_cast(half8, hb);
			}
			hf* g = dloss + ((size_t)cb + s) * 16;
			*reinterpret_cast<half8*>(g) = lo;
			*reinterpret_cast<half8*>(g + 8) = hi;
			const float* ci = coords + ((size_t)base + s) * 7;
			float* co = coords_out + ((size_t)cb + s) * 7;
#pragma unroll
			for (int k = 0; k < 7; ++k) co[k] = ci[k];
			const uint32_t src_col = column_of ? column_of[base + s] : base + s;
			if (source_index) source_index[cb + s] = src_col;  // which marched sample this compacted sample is
			if (pad && n_in > 0 && n_in < max_compacted) {
				for (uint32_t j = cb + s + n_in; j < max_compacted; j += n_in) {
					half8 lo_f, hi_f;
#pragma unroll
					for (int k = 0; k < 8; ++k) {
						lo_f[k] = (hf)rollover_rescaled((float)lo[k], n_in, max_compacted, 16u);
						hi_f[k] = (hf)rollover_rescaled((float)hi[k], n_in, max_compacted, 16u);
					}
					hf* gf = dloss + (size_t)j * 16;
					*reinterpret_cast<half8*>(gf) = lo_f;
					*reinterpret_cast<half8*>(gf + 8) = hi_f;
					float* cf = coords_out + (size_t)j * 7;
#pragma unroll
					for (int k = 0; k < 7; ++k) cf[k] = ci[k];
					if (source_index) source_index[j] = src_col;
				}
			}
		}
		T = __shfl(Ta, 63);
		p0 = __shfl(q0, 63); p1 = __shfl(q1, 63); p2 = __shfl(q2, 63);
	}
}

// ----------------------------------------------------------------------------
// Forward pass in depth chunks.  The compositor consumes a ray's samples only while the transmittance before them is
// >= 1e-4 (src/testbed_nerf.cu:1562-1566); on a trained field most rays reach that point after a fraction of their
// marched samples, and everything behind it never enters loss, compaction or gradients.  The trainer can therefore
// evaluate the field in rounds: every round takes the next `chunk` samples of the rays that are still live, and between
// rounds this kernel (one thread per ray) multiplies the transmittance on over the samples just evaluated, with the
// compositor's own alpha, and retires the rays that are certainly past the cut (T < 0.5e-4: the compositor's product is
// formed in another order, which moves T by a few units in the last place, never by a factor of two; a ray that stays
// live a round too long costs work, never correctness).  For the live rays it appends the next samples to the list of
// samples to evaluate; the samples of all rounds stand side by side in that list, and column_of[marched sample] is its
// place in it (where the field stores what the backward reads).  counts[r] = samples of round r.
// ----------------------------------------------------------------------------
struct ChunkRay {
	uint32_t prev, done;  // samples [prev, done) of the ray were listed last
	float T;              // transmittance behind sample prev
	uint32_t live;
};
constexpr float CHUNK_T_EPS = 0.5f * T_EPS;
// sixteen lanes per ray, 64 rays per workgroup: every workgroup takes its places in the list with one atomic on the round's
// counter, and those atomics, all on one address, run one after the other (16 rays per workgroup: 2500 of them, 20 us)
constexpr uint32_t CHUNK_BLOCK = 1024, CHUNK_LANES = 16, CHUNK_RAYS = CHUNK_BLOCK / CHUNK_LANES;

// One ray per sixteen lanes (a row of the data-parallel lane operations): the lanes take the ray's samples sixteen at a
// time.  coords_listed receives the coordinate rows of the listed samples in list order, so that the field's kernels read
// their input without going through the list.
__global__ void __launch_bounds__(CHUNK_BLOCK) composite_chunk_kernel(CompParams c, uint32_t n_rays, const uint32_t* __restrict__ ray_counter,
                                                                      const uint32_t* __restrict__ numsteps, const hf* __restrict__ net_out,
                                                                      const float* __restrict__ coords, uint32_t round, uint32_t chunk,
                                                                      ChunkRay* __restrict__ state, uint32_t* __restrict__ counts,
                                                                      uint32_t* __restrict__ counts_other, uint32_t* __restrict__ list,
                                                                      uint32_t* __restrict__ column_of, float* __restrict__ coords_listed) {
	__shared__ uint32_t takes[CHUNK_RAYS], firsts[CHUNK_RAYS], before[CHUNK_RAYS + 1], wg_at;
	const uint32_t l = threadIdx.x % CHUNK_LANES, slot = threadIdx.x / CHUNK_LANES;
	const uint32_t ray = blockIdx.x * CHUNK_RAYS + slot;
	const uint32_t live_rays = ray_counter ? min(*ray_counter, n_rays) : n_rays;
	// the counters that the following step uses start from zero
	if (round == 0 && blockIdx.x == 0 && threadIdx.x < N2_CHUNK_MAX_ROUNDS) counts_other[threadIdx.x] = 0u;
	uint32_t begin = 0;  // samples listed by the rounds before this one
	for (uint32_t q = 0; q < round; ++q) begin += counts[q];
	ChunkRay st = {0u, 0u, 1.f, 0u};
	uint32_t n = 0, base = 0;
	if (ray < live_rays) {
		n = numsteps[2 * ray];
		base = numsteps[2 * ray + 1];
		if (round == 0) {
			st.live = n > 0 ? 1u : 0u;
		} else {
			st = state[ray];
			if (st.live) {
				float dir[3];
				ray_dir(net_out, base, dir);
				float T = st.T;
				for (uint32_t s0 = st.prev; s0 < st.done; s0 += CHUNK_LANES) {
					const uint32_t s = s0 + l;
					float keep = 1.f;
					if (s < st.done) {
						float o[16];
						load_out(net_out, (size_t)base + s, o);
						const Sample sm = eval_sample(o, net_out[((size_t)base + s) * 16 + 7], coords[((size_t)base + s) * 7 + 3], dir, c);
						keep = 1.f - sm.alpha;
					}
#pragma unroll
					for (int o = 1; o < (int)CHUNK_LANES; o <<= 1) keep *= __shfl_xor(keep, o);  // stays inside the sixteen lanes
					T *= keep;
				}
				st.T = T;
				if (!(T >= CHUNK_T_EPS) || st.done >= n) st.live = 0u;  // (a transmittance that is not a number retires the ray too)
			}
		}
	}
	const uint32_t take = st.live ? min(n - st.done, chunk) : 0u;
	// places in the list: the workgroup's 64 rays in order, one atomic per workgroup for its block of places
	if (l == 0) { takes[slot] = take; firsts[slot] = base + st.done; }
	__syncthreads();
	if (threadIdx.x < 64) {  // one wave scans the 64 counts
		static_assert(CHUNK_RAYS == 64, "one count per lane");
		const uint32_t own = takes[threadIdx.x];
		uint32_t incl = own;
#pragma unroll
		for (int o = 1; o < 64; o <<= 1) {
			const uint32_t up = __shfl_up(incl, o);
			if ((int)threadIdx.x >= o) incl += up;
		}
		const uint32_t total = __shfl(incl, 63);
		uint32_t at = 0;
		if (threadIdx.x == 0 && total) at = atomicAdd(&counts[round], total);
		before[threadIdx.x] = incl - own;
		if (threadIdx.x == 63) before[CHUNK_RAYS] = total;
		if (threadIdx.x == 0) wg_at = at;
	}
	__syncthreads();
	// The workgroup's listed samples, all threads together (a ray that lists hundreds of samples in the last round would
	// otherwise keep its sixteen lanes busy long after the others are done): sample e of the workgroup belongs to the ray r
	// with before[r] <= e < before[r + 1].  The coordinate rows go along: consecutive in the output over the whole workgroup.
	const uint32_t total = before[CHUNK_RAYS], at0 = begin + wg_at;
	auto ray_of = [&](uint32_t e) {
		uint32_t r = 0;
#pragma unroll
		for (uint32_t step = CHUNK_RAYS / 2; step > 0; step >>= 1)
			if (before[r + step] <= e) r += step;
		return r;
	};
	for (uint32_t e = threadIdx.x; e < total; e += CHUNK_BLOCK) {
		const uint32_t r = ray_of(e), id = firsts[r] + (e - before[r]);
		list[at0 + e] = id;
		column_of[id] = at0 + e;
	}
	float* to = coords_listed + (size_t)at0 * 7;
	for (uint32_t f = threadIdx.x; f < total * 7u; f += CHUNK_BLOCK) {
		const uint32_t e = f / 7u, r = ray_of(e);
		to[f] = coords[(size_t)(firsts[r] + (e - before[r])) * 7 + (f - e * 7u)];
	}
	if (ray < live_rays && l == 0) {
		st.prev = st.done;
		st.done += take;
		state[ray] = st;
	}
}

template <typename T, bool RESCALE>
__global__ void __launch_bounds__(256) fill_rollover_kernel(uint32_t n_total, uint32_t stride, const uint32_t* __restrict__ n_in_ptr,
                                                            T* __restrict__ inout) {
	const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
	const uint32_t n_in = *n_in_ptr;
	const size_t lim = (size_t)n_in * stride;
	if (n_in == 0 || i < lim || i >= (size_t)n_total * stride) return;
	T r = inout[i % lim];
	if (RESCALE) r = (T)rollover_rescaled((float)r, n_in, n_total, stride);
	inout[i] = r;
}

// ----------------------------------------------------------------------------
static inline uint64_t up256(uint64_t x) { return (x + 255) / 256 * 256; }

N2_API uint64_t n2_composite_workspace_bytes(uint32_t max_rays) {
	return up256(sizeof(RayScratch) * (uint64_t)max_rays) + 2 * up256(4ull * max_rays);
}

uint64_t n2_composite_chunk_state_bytes(uint32_t max_rays) { return up256(sizeof(ChunkRay) * (uint64_t)max_rays); }

int n2_composite_chunk_next(n2_stream_t stream, const n2_composite_config* cfg, uint32_t n_rays, const uint32_t* d_ray_counter, const uint32_t* d_numsteps,
                            const n2_half* d_network_output, const float* d_coords, uint32_t round, uint32_t chunk, void* d_state, uint32_t* d_counts,
                            uint32_t* d_counts_other, uint32_t* d_list, uint32_t* d_column_of, float* d_coords_listed) {
	N2_REQUIRE(cfg && d_numsteps && d_network_output && d_coords && d_state && d_counts && d_counts_other && d_list && d_column_of && d_coords_listed,
	           "n2_composite_chunk_next: null argument");
	N2_REQUIRE(round < N2_CHUNK_MAX_ROUNDS && chunk >= 1, "n2_composite_chunk_next: round %u of at most %u, chunk %u", round, N2_CHUNK_MAX_ROUNDS, chunk);
	if (n_rays == 0) return N2_OK;
	CompParams c;
	c.loss_scale = cfg->loss_scale; c.ek_loss_weight = cfg->ek_loss_weight; c.anneal = cfg->cos_anneal_ratio;
	c.bg[0] = cfg->background[0]; c.bg[1] = cfg->background[1]; c.bg[2] = cfg->background[2];
	c.inv_n_rays = 1.f;
	c.min_step = 1.73205080757f / 1024.f;
	c.max_step = c.min_step * 128.f;
	composite_chunk_kernel<<<dim3((n_rays + CHUNK_RAYS - 1) / CHUNK_RAYS), dim3(CHUNK_BLOCK), 0, n2_stream(stream)>>>(
		c, n_rays, d_ray_counter, d_numsteps, reinterpret_cast<const hf*>(d_network_output), d_coords, round, chunk, reinterpret_cast<ChunkRay*>(d_state),
		d_counts, d_counts_other, d_list, d_column_of, d_coords_listed);
	N2_LAUNCH_CHECK();
	return N2_OK;
}

N2_API int n2_composite_loss(n2_stream_t stream, const n2_composite_config* cfg, uint32_t n_rays,
                             const uint32_t* d_ray_counter, uint32_t* d_numsteps, const n2_half* d_network_output,
                             const float* d_coords, const float* d_rgb_target, uint32_t max_samples_compacted,
                             uint32_t* d_compacted_counter, float* d_coords_compacted, n2_half* d_dloss_doutput,
                             float* d_loss, void* d_workspace, uint64_t workspace_bytes) {
	return n2_composite_loss_indexed(stream, cfg, n_rays, d_ray_counter, d_numsteps, d_network_output, d_coords, d_rgb_target,
	                                 max_samples_compacted, d_compacted_counter, d_coords_compacted, d_dloss_doutput, d_loss, nullptr,
	                                 d_workspace, workspace_bytes);
}

// Scratch of n2_composite_loss_static: per-ray colour, kept counts and their prefix sums for up to N2_COMPOSITE_STATIC_MAX_RAYS rays, held
// by every GPU the library runs on until the process ends.  In host code the array's name stands for the symbol only;
// the device address of each GPU's copy is looked up once per device (static_scratch) and that pointer is what the
// kernels receive.
constexpr uint32_t STATIC_MAX_RAYS = N2_COMPOSITE_STATIC_MAX_RAYS;
constexpr uint64_t STATIC_BYTES = (sizeof(RayScratch) * (uint64_t)STATIC_MAX_RAYS + 255) / 256 * 256 + 2 * ((4ull * STATIC_MAX_RAYS + 255) / 256 * 256);
static __device__ __align__(256) unsigned char scratch[STATIC_BYTES];

constexpr int STATIC_MAX_DEVICES = 64;
static std::mutex g_static_lock;
static void* g_static_ptr[STATIC_MAX_DEVICES] = {};

// device address of the current device's copy of `scratch` (looked up on the first call on that device)
static int static_scratch(void** out) {
	int device = -1;
	N2_HIP(hipGetDevice(&device));
	N2_REQUIRE(device >= 0 && device < STATIC_MAX_DEVICES, "n2_composite_loss_static: device ordinal %d outside [0, %d)", device, STATIC_MAX_DEVICES);
	std::lock_guard<std::mutex> guard(g_static_lock);
	if (g_static_ptr[device] == nullptr) {
		void* p = nullptr;
		N2_HIP(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
		N2_REQUIRE(p != nullptr && reinterpret_cast<uintptr_t>(p) % 256 == 0, "n2_composite_loss_static: bad address for the scratch array");
		g_static_ptr[device] = p;
	}
	*out = g_static_ptr[device];
	return N2_OK;
}

N2_API int n2_composite_loss_static(n2_stream_t stream, const n2_composite_config* cfg, uint32_t n_rays,
                                    const uint32_t* d_ray_counter, uint32_t* d_numsteps, const n2_half* d_network_output,
                                    const float* d_coords, const float* d_rgb_target, uint32_t max_samples_compacted,
                                    uint32_t* d_compacted_counter, float* d_coords_compacted, n2_half* d_dloss_doutput,
                                    float* d_loss, uint32_t* d_source_index) {
	N2_REQUIRE(n_rays <= STATIC_MAX_RAYS, "n2_composite_loss_static: %u rays exceed the static scratch's maximum of %u (use n2_composite_loss_indexed with a workspace)",
	           n_rays, STATIC_MAX_RAYS);
	void* ws = nullptr;
	if (int rc = static_scratch(&ws)) return rc;
	return n2_composite_loss_indexed(stream, cfg, n_rays, d_ray_counter, d_numsteps, d_network_output, d_coords, d_rgb_target,
	                                 max_samples_compacted, d_compacted_counter, d_coords_compacted, d_dloss_doutput, d_loss, d_source_index,
	                                 ws, STATIC_BYTES);
}

N2_API int n2_composite_loss_indexed(n2_stream_t stream, const n2_composite_config* cfg, uint32_t n_rays,
                                     const uint32_t* d_ray_counter, uint32_t* d_numsteps, const n2_half* d_network_output,
                                     const float* d_coords, const float* d_rgb_target, uint32_t max_samples_compacted,
                                     uint32_t* d_compacted_counter, float* d_coords_compacted, n2_half* d_dloss_doutput,
                                     float* d_loss, uint32_t* d_source_index, void* d_workspace, uint64_t workspace_bytes) {
	return n2_composite_loss_filled(stream, cfg, n_rays, d_ray_counter, d_numsteps, d_network_output, d_coords, d_rgb_target, max_samples_compacted,
	                                d_compacted_counter, d_coords_compacted, d_dloss_doutput, d_loss, d_source_index, d_workspace, workspace_bytes, false);
}

int n2_composite_loss_filled(n2_stream_t stream, const n2_composite_config* cfg, uint32_t n_rays,
                             const uint32_t* d_ray_counter, uint32_t* d_numsteps, const n2_half* d_network_output,
                             const float* d_coords, const float* d_rgb_target, uint32_t max_samples_compacted,
                             uint32_t* d_compacted_counter, float* d_coords_compacted, n2_half* d_dloss_doutput,
                             float* d_loss, uint32_t* d_source_index, void* d_workspace, uint64_t workspace_bytes, bool fill, const uint32_t* d_column_of) {
	N2_REQUIRE(cfg != nullptr, "n2_composite_loss: config is null");
	N2_REQUIRE(d_compacted_counter != nullptr, "n2_composite_loss: d_compacted_counter is null");
	hipStream_t s = n2_stream(stream);
	if (n_rays == 0) return n2_set_u32(s, d_compacted_counter, 0u);
	N2_REQUIRE(d_numsteps && d_network_output && d_coords && d_rgb_target && d_coords_compacted && d_dloss_doutput && d_workspace,
	           "n2_composite_loss: null buffer");
	N2_REQUIRE(cfg->n_rays_norm > 0 && cfg->loss_scale > 0.f, "n2_composite_loss: n_rays_norm and loss_scale must be positive");
	N2_REQUIRE(workspace_bytes >= n2_composite_workspace_bytes(n_rays), "n2_composite_loss: workspace of %llu bytes, %llu needed",
	           (unsigned long long)workspace_bytes, (unsigned long long)n2_composite_workspace_bytes(n_rays));
	N2_REQUIRE(reinterpret_cast<uintptr_t>(d_network_output) % 16 == 0 && reinterpret_cast<uintptr_t>(d_dloss_doutput) % 16 == 0 &&
	           reinterpret_cast<uintptr_t>(d_workspace) % 16 == 0, "n2_composite_loss: fp16 buffers and workspace must be 16-byte aligned");
	CompParams c;
	c.loss_scale = cfg->loss_scale; c.ek_loss_weight = cfg->ek_loss_weight; c.anneal = cfg->cos_anneal_ratio;
	c.bg[0] = cfg->background[0]; c.bg[1] = cfg->background[1]; c.bg[2] = cfg->background[2];
	c.inv_n_rays = 1.f / (float)cfg->n_rays_norm;
	c.min_step = 1.73205080757f / 1024.f;  // STEPSIZE(), src/testbed_nerf.cu:51-53
	c.max_step = c.min_step * 128.f;       // * 2^(NERF_CASCADES-1), unwarp_dt :617-620
	unsigned char* w = reinterpret_cast<unsigned char*>(d_workspace);
	RayScratch* scratch = reinterpret_cast<RayScratch*>(w);
	uint32_t* kept_of = reinterpret_cast<uint32_t*>(w + up256(sizeof(RayScratch) * (uint64_t)n_rays));
	uint32_t* before_of = n_rays >= OFFSETS_MIN_RAYS ? kept_of + up256(4ull * n_rays) / 4 : nullptr;
	const dim3 grid((n_rays + CB / 64 - 1) / (CB / 64)), block(CB);
	const hf* out = reinterpret_cast<const hf*>(d_network_output);
	N2ProfScope prof(N2_PROF_COMPOSITE, s);
	// below OFFSETS_MIN_RAYS rays the second count array holds the forward kernel's counts per workgroup instead of prefix sums
	uint32_t* kept_of_block = before_of ? nullptr : kept_of + up256(4ull * n_rays) / 4;
	composite_forward_kernel<<<grid, block, 0, s>>>(c, n_rays, d_ray_counter, d_numsteps, out, d_coords, scratch, kept_of, kept_of_block);
	N2_LAUNCH_CHECK();
	if (before_of) {
		composite_offsets_kernel<<<dim3((n_rays + OFFSETS_BLOCK - 1) / OFFSETS_BLOCK), dim3(OFFSETS_BLOCK), 0, s>>>(n_rays, kept_of, before_of);
		N2_LAUNCH_CHECK();
	}
	composite_backward_kernel<<<grid, block, 0, s>>>(c, n_rays, d_numsteps, out, d_coords, d_rgb_target, scratch, kept_of, max_samples_compacted,
	                                                 d_compacted_counter, d_coords_compacted, reinterpret_cast<hf*>(d_dloss_doutput), d_loss, d_source_index,
	                                                 before_of, fill ? 1u : 0u, kept_of_block, d_column_of);
	N2_LAUNCH_CHECK();
	return N2_OK;
}

N2_API int n2_fill_rollover_f32(n2_stream_t stream, uint32_t n_total, uint32_t stride, const uint32_t* d_n_in, float* d_inout) {
	N2_REQUIRE(d_n_in && d_inout, "n2_fill_rollover_f32: null buffer");
	const size_t n = (size_t)n_total * stride;
	if (n == 0) return N2_OK;
	fill_rollover_kernel<float, false><<<dim3((uint32_t)((n + 255) / 256)), dim3(256), 0, n2_stream(stream)>>>(n_total, stride, d_n_in, d_inout);
	N2_LAUNCH_CHECK();
	return N2_OK;
}

N2_API int n2_fill_rollover_and_rescale_f16(n2_stream_t stream, uint32_t n_total, uint32_t stride, const uint32_t* d_n_in, n2_half* d_inout) {
	N2_REQUIRE(d_n_in && d_inout, "n2_fill_rollover_and_rescale_f16: null buffer");
	const size_t n = (size_t)n_total * stride;
	if (n == 0) return N2_OK;
	fill_rollover_kernel<hf, true><<<dim3((uint32_t)((n + 255) / 256)), dim3(256), 0, n2_stream(stream)>>>(n_total, stride, d_n_in,
		reinterpret_cast<hf*>(d_inout));
	N2_LAUNCH_CHECK();
	return N2_OK;
}
