// Summation of the per-workgroup partial sums (slabs) that the weight-gradient kernels of the MLPs leave behind, as a device
// function for any kernel with 256-thread workgroups: mlp.hip launches it as a kernel of its own, and the trainer's Adam
// step runs it in its first workgroups (25 MB of streaming reads inside a kernel that streams 350 MB anyway), so that a
// training step has no reduction launch.
#pragma once
#include <hip/hip_runtime.h>
#include <cstdint>

struct N2SlabReduce {
	// two parameter sets: grads (fp16) = [grads +] sum over the slabs, a unit per 32 consecutive parameters
	const float* pa; uint32_t slabs_a, params_a; _Float16* ga; int acc_a; uint32_t units_a;
	const float* pb; uint32_t slabs_b, params_b; _Float16* gb; int acc_b; uint32_t units_b;
	// one more unit (when extra_n > 0) adds up extra_n floats in a fixed order into a single fp16 value
	const float* extra; uint32_t extra_n; _Float16* extra_out; int extra_acc;
	uint32_t units;  // units_a + units_b + (extra_n > 0)
};

// Bookkeeping of a training step that rides in the optimiser's launch as one workgroup (values null: none):
// *sum_out = values[0] + ... + values[min(*n_ptr, n_max) - 1], added up in a fixed order, and copy_n words copied.
struct N2StepEpilogue {
	const float* values; const uint32_t* n_ptr; uint32_t n_max; float* sum_out;
	const uint32_t* copy_src; uint32_t* copy_dst; uint32_t copy_n;
};

// Sum of the partial images that the encoding's bucketed scatter leaves for buckets it splits over several workgroups
// (the coarsest levels of a large batch; they are levels 0 .. n_levels - 1).  Image (level, bucket, group) holds the
// bucket's bucket_entries fp32 pairs at images + (part_begin[level] + bucket * groups[level] + group) * bucket_entries.
// A unit adds up the images of 128 consecutive entries in the order of the groups and stores the fp16 gradients.
constexpr uint32_t N2_CMB_LEVELS = 32, N2_CMB_SLICES = 8, N2_CMB_ENTRIES = 128, N2_CMB_MAX_GROUPS = 32;
struct N2ImageCombine {
	const float2* images;
	_Float16* grads;                          // the encoding's gradients: entry e of level l at grads + 2 * (offset[l] + e)
	uint32_t n_levels, bucket_entries;
	uint32_t split_begin[N2_CMB_LEVELS + 1];  // split buckets in the levels below
	uint32_t groups[N2_CMB_LEVELS], part_begin[N2_CMB_LEVELS], entries[N2_CMB_LEVELS], offset[N2_CMB_LEVELS];
	int accumulate;
	uint32_t units;                           // split buckets * bucket_entries / 128 (0: nothing to do)
};

// Unit `unit` of an image combination, run by the 256 threads of a workgroup: thread (slice, quad) adds the images slice,
// slice + 8, ... of four entries (all its loads in flight at once), the eight slices meet in LDS, again in order: every
// entry is the same sum in the same order whatever runs first.  done(address of a stored fp16 gradient, its value) is
// called twice (both features) by the thread that stored an entry.  Contains one __syncthreads().
template <class Done>
__device__ __forceinline__ void n2_image_combine_unit(const N2ImageCombine& r, uint32_t unit, float2 (*part)[N2_CMB_ENTRIES], Done done) {
	const uint32_t per_bucket = r.bucket_entries / N2_CMB_ENTRIES;
	const uint32_t split = unit / per_bucket, chunk = unit % per_bucket;
	uint32_t level = 0;
	while (level + 1 < r.n_levels && split >= r.split_begin[level + 1]) ++level;
	const uint32_t bucket = split - r.split_begin[level], G = r.groups[level];
	const uint32_t quad = threadIdx.x % (256 / N2_CMB_SLICES), slice = threadIdx.x / (256 / N2_CMB_SLICES);
	const uint32_t e0 = bucket * r.bucket_entries + chunk * N2_CMB_ENTRIES;  // first entry of the unit within the level
	const float4* src = reinterpret_cast<const float4*>(r.images + ((size_t)r.part_begin[level] + (size_t)bucket * G) * r.bucket_entries +
	                                                    chunk * N2_CMB_ENTRIES + 4u * quad);
	constexpr uint32_t PER = N2_CMB_MAX_GROUPS / N2_CMB_SLICES;
	float4 lo[PER], hi[PER];
	const bool inside = e0 < r.entries[level];  // the same for the whole workgroup
#pragma unroll
	for (uint32_t u = 0; u < PER; ++u) {
		const uint32_t q = slice + N2_CMB_SLICES * u;
		if (inside && q < G) {
			lo[u] = src[(size_t)q * (r.bucket_entries / 2)];
			hi[u] = src[(size_t)q * (r.bucket_entries / 2) + 1];
		} else {
			lo[u] = hi[u] = make_float4(0.f, 0.f, 0.f, 0.f);
		}
	}
	float4 a = lo[0], b = hi[0];
#pragma unroll
	for (uint32_t u = 1; u < PER; ++u) {
		a.x += lo[u].x; a.y += lo[u].y; a.z += lo[u].z; a.w += lo[u].w;
		b.x += hi[u].x; b.y += hi[u].y; b.z += hi[u].z; b.w += hi[u].w;
	}
	part[slice][4 * quad] = make_float2(a.x, a.y);
	part[slice][4 * quad + 1] = make_float2(a.z, a.w);
	part[slice][4 * quad + 2] = make_float2(b.x, b.y);
	part[slice][4 * quad + 3] = make_float2(b.z, b.w);
	__syncthreads();
	if (threadIdx.x >= N2_CMB_ENTRIES || e0 + threadIdx.x >= r.entries[level]) return;
	_Float16* g = r.grads + 2 * ((size_t)r.offset[level] + e0 + threadIdx.x);
	float2 sum = r.accumulate ? make_float2((float)g[0], (float)g[1]) : make_float2(0.f, 0.f);
#pragma unroll
	for (uint32_t sl = 0; sl < N2_CMB_SLICES; ++sl) { sum.x += part[sl][threadIdx.x].x; sum.y += part[sl][threadIdx.x].y; }
	typedef _Float16 n2_half2v __attribute__((ext_vector_type(2)));
	const n2_half2v h = {(_Float16)sum.x, (_Float16)sum.y};
	*reinterpret_cast<n2_half2v*>(g) = h;
	done(g, h[0]);
	done(g + 1, h[1]);
}

// Unit `unit` of the plan, run by the 256 threads of a workgroup.  A unit owns 32 consecutive parameters (one 128-byte line
// of every slab): 8 lanes cover the line with 16-byte loads, 32 lane groups share the slabs, eight loads in flight per
// lane, LDS folds the groups.  n_params is a multiple of 16, so lines are never ragged.  The fp16 gradient is stored, and
// done(address of the stored gradient, its value) is called by the thread that stored it.  Contains one __syncthreads().
template <class Done>
__device__ __forceinline__ void n2_slab_reduce_unit(const N2SlabReduce& r, uint32_t unit, float (*fold)[33], Done done) {
	const uint32_t tid = threadIdx.x;
	if (unit >= r.units_a + r.units_b) {  // the extra sum
		float s = 0.f;
		for (uint32_t i = tid; i < r.extra_n; i += 256) s += r.extra[i];
#pragma unroll
		for (int o = 32; o > 0; o >>= 1) s += __shfl_xor(s, o);
		if ((tid & 63u) == 0) fold[0][tid >> 6] = s;
		__syncthreads();
		if (tid == 0) {
			const float t = (fold[0][0] + fold[0][1]) + (fold[0][2] + fold[0][3]);
			const _Float16 h = r.extra_acc ? (_Float16)((float)r.extra_out[0] + t) : (_Float16)t;
			r.extra_out[0] = h;
			done(r.extra_out, h);
		}
		return;
	}
	const bool first = unit < r.units_a;
	const float* partials = first ? r.pa : r.pb;
	const uint32_t n_slabs = first ? r.slabs_a : r.slabs_b, n_params = first ? r.params_a : r.params_b, line = first ? unit : unit - r.units_a;
	_Float16* grads = first ? r.ga : r.gb;
	const int accumulate = first ? r.acc_a : r.acc_b;
	const uint32_t q = tid & 7u, grp = tid >> 3;
	const uint32_t i = line * 32 + q * 4;
	float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
	if (i < n_params) {
		const float* p = partials + i;
		uint32_t k = grp;
		for (; k + 7 * 32 < n_slabs; k += 8 * 32) {
			float4 v[8];
#pragma unroll
			for (int u = 0; u < 8; ++u) v[u] = *reinterpret_cast<const float4*>(p + (size_t)(k + u * 32) * n_params);
#pragma unroll
			for (int u = 0; u < 8; ++u) { acc.x += v[u].x; acc.y += v[u].y; acc.z += v[u].z; acc.w += v[u].w; }
		}
		for (; k < n_slabs; k += 32) {
			const float4 v = *reinterpret_cast<const float4*>(p + (size_t)k * n_params);
			acc.x += v.x; acc.y += v.y; acc.z += v.z; acc.w += v.w;
		}
	}
	fold[grp][q * 4 + 0] = acc.x;
	fold[grp][q * 4 + 1] = acc.y;
	fold[grp][q * 4 + 2] = acc.z;
	fold[grp][q * 4 + 3] = acc.w;
	__syncthreads();
	// 8 lanes per parameter fold 4 groups each, then a shuffle tree
	const uint32_t pl = tid >> 3, part = tid & 7u;
	float t = fold[part * 4][pl] + fold[part * 4 + 1][pl] + fold[part * 4 + 2][pl] + fold[part * 4 + 3][pl];
	t += __shfl_xor(t, 1);
	t += __shfl_xor(t, 2);
	t += __shfl_xor(t, 4);
	const uint32_t o = line * 32 + pl;
	if (part == 0 && o < n_params) {
		if (accumulate) t += (float)grads[o];
		const _Float16 h = (_Float16)t;
		grads[o] = h;
		done(grads + o, h);
	}
}
