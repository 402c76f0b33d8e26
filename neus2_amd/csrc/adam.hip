// Adam step over the whole parameter vector: a pure streaming kernel.
// Four parameters per lane so that every buffer is moved with 8- or 16-byte
// accesses; parameters whose gradient is zero (most of the hash table in any
// one step) cost only the 2-byte gradient read.
#include "n2_common.h"
#include <hip/hip_ext.h>
#include "slab_reduce.h"

#include <cmath>
#include <type_traits>
#include <mutex>

typedef _Float16 hf;
typedef _Float16 half4 __attribute__((ext_vector_type(4)));

// Bias correction sqrt(1 - beta2^t) / (1 - beta1^t) for t < ADAM_TABLE, computed once per (beta1, beta2) by
// adam_table_kernel.  Two powf per parameter made the step kernel ALU bound; a (mostly uniform) table read costs nothing.
// A device holds ADAM_SLOTS such tables, one per pair of betas in use, so that optimisers with different betas (or on
// different streams) never rewrite a table another one's step is reading.
constexpr uint32_t ADAM_TABLE = 4096, ADAM_SLOTS = 4;
__device__ float g_adam_bias[ADAM_SLOTS][ADAM_TABLE];

__device__ __forceinline__ float adam_bias(float beta1, float beta2, uint32_t t) {
	return sqrtf(1.f - powf(beta2, (float)t)) / (1.f - powf(beta1, (float)t));
}
__global__ void __launch_bounds__(256) adam_table_kernel(float beta1, float beta2, uint32_t slot) {
	const uint32_t t = blockIdx.x * 256 + threadIdx.x;
	if (t < ADAM_TABLE) g_adam_bias[slot][t] = adam_bias(beta1, beta2, t);
}

// inv_loss_scale > 0: loss_scale is a power of two and multiplying by its reciprocal is the exact division
__device__ __forceinline__ bool adam_one(uint32_t i, uint32_t n_matrix, float loss_scale, float inv_loss_scale, int saturated,
                                         const n2_adam_config& c, const float* __restrict__ table, float g16, float& w, float& m1, float& m2, uint32_t& t) {
	float g = inv_loss_scale > 0.f ? g16 * inv_loss_scale : g16 / loss_scale;
	if (i >= n_matrix) {
		if (g == 0.f) return false;
	} else {
		g += c.l2_reg * w;
	}
	const float gs = g * g;
	m1 = c.beta1 * m1 + (1.f - c.beta1) * g;
	m2 = c.beta2 * m2 + (1.f - c.beta2) * gs;
	t += 1u;
	// beyond the table the factor is exactly 1 once both powers have underflowed (saturated), else it is computed
	const float bias = t < ADAM_TABLE ? table[t] : (saturated ? 1.f : adam_bias(c.beta1, c.beta2, t));
	const float lr = c.learning_rate * bias;
	w -= lr * m1 / (sqrtf(m2) + c.epsilon);
	return true;
}

// Step counters are 32 bits wide, or 16 bits saturating at 65535 (the trainer's, when both beta powers have underflowed
// long before: past the table the correction is exactly 1 then, so the count no longer matters; 4 bytes less traffic per
// touched parameter).
__device__ __forceinline__ uint32_t step_load(const uint32_t* p) { return *p; }
__device__ __forceinline__ uint32_t step_load(const uint16_t* p) { return *p; }
__device__ __forceinline__ void step_store(uint32_t* p, uint32_t t) { *p = t; }
__device__ __forceinline__ void step_store(uint16_t* p, uint32_t t) { *p = (uint16_t)min(t, 65535u); }
__device__ __forceinline__ uint4 step_load4(const uint32_t* p) { return *reinterpret_cast<const uint4*>(p); }
__device__ __forceinline__ uint4 step_load4(const uint16_t* p) {
	const ushort4 v = *reinterpret_cast<const ushort4*>(p);
	return make_uint4(v.x, v.y, v.z, v.w);
}
__device__ __forceinline__ void step_store4(uint32_t* p, uint4 t) { *reinterpret_cast<uint4*>(p) = t; }
__device__ __forceinline__ void step_store4(uint16_t* p, uint4 t) {
	*reinterpret_cast<ushort4*>(p) = make_ushort4((unsigned short)min(t.x, 65535u), (unsigned short)min(t.y, 65535u), (unsigned short)min(t.z, 65535u),
	                                              (unsigned short)min(t.w, 65535u));
}

// parameters whose gradients a slab summation produces (r.units > 0): the workgroups that run its units step them
__device__ __forceinline__ bool adam_summed(const N2SlabReduce& r, const hf* grads, uint32_t i) {
	if (r.units == 0) return false;
	const hf* g = grads + i;
	return (g >= r.ga && g < r.ga + r.params_a) || (g >= r.gb && g < r.gb + r.params_b) || (r.extra_n > 0 && g == r.extra_out);
}

template <typename StepT>
__global__ void __launch_bounds__(256) adam_step_kernel(n2_adam_config c, uint32_t n, uint32_t n_matrix, float loss_scale, float inv_loss_scale, int saturated,
                                                        uint32_t slot, const uint32_t* __restrict__ gate, float* __restrict__ master, hf* __restrict__ params, const hf* __restrict__ grads,
                                                        float* __restrict__ m1, float* __restrict__ m2, StepT* __restrict__ steps, N2SlabReduce sums,
                                                        N2StepEpilogue epi) {
	const uint32_t epi_blocks = epi.values != nullptr ? 1u : 0u;
	if (epi_blocks && blockIdx.x == 0) {
		// the caller's bookkeeping (the trainer: the loss of the step's rays and its counters), whether the step is gated or not
		__shared__ float part[4];
		const uint32_t n_val = min(*epi.n_ptr, epi.n_max);
		float s = 0.f;
		for (uint32_t i0 = 0; i0 < n_val; i0 += 16u * 256u) {  // sixteen loads in flight per thread
			float v[16];
#pragma unroll
			for (uint32_t u = 0; u < 16; ++u) {
				const uint32_t i = i0 + u * 256u + threadIdx.x;
				v[u] = i < n_val ? epi.values[i] : 0.f;
			}
#pragma unroll
			for (uint32_t u = 0; u < 16; ++u) s += v[u];
		}
#pragma unroll
		for (int o = 32; o > 0; o >>= 1) s += __shfl_xor(s, o);
		if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = s;
		__syncthreads();
		if (threadIdx.x == 0) *epi.sum_out = (part[0] + part[1]) + (part[2] + part[3]);
		if (threadIdx.x < epi.copy_n) epi.copy_dst[threadIdx.x] = epi.copy_src[threadIdx.x];
		return;
	}
	if (gate != nullptr && *gate == 0u) return;  // a step without samples leaves the parameters and the optimiser state alone
	const float* table = g_adam_bias[slot];
	const uint32_t block = blockIdx.x - epi_blocks;
	if (block < sums.units) {
		// The first workgroups add up the slabs of 32 parameters each (25 MB of streaming reads that would otherwise be a launch
		// of their own in front of this one), store the fp16 gradient and step the parameter with it.
		__shared__ float fold[32][33];
		n2_slab_reduce_unit(sums, block, fold, [&](const hf* at, hf g16) {
			const uint32_t i = (uint32_t)(at - grads);
			float w = master[i], a = m1[i], b = m2[i];
			uint32_t t = step_load(steps + i);
			if (adam_one(i, n_matrix, loss_scale, inv_loss_scale, saturated, c, table, (float)g16, w, a, b, t)) {
				master[i] = w; m1[i] = a; m2[i] = b; step_store(steps + i, t); params[i] = (hf)w;
			}
		});
		return;
	}
	const uint32_t q = (block - sums.units) * 256 + threadIdx.x;
	const uint32_t i0 = q * 4;
	if (i0 >= n) return;
	if (adam_summed(sums, grads, i0) || adam_summed(sums, grads, min(i0 + 3u, n - 1u))) {
		// a quad that touches summed parameters (the networks' weights are whole quads; the single extra value may share its
		// quad with others): one parameter at a time, leaving out the summed ones
		for (uint32_t i = i0; i < min(i0 + 4u, n); ++i) {
			if (adam_summed(sums, grads, i)) continue;
			float w = master[i], a = m1[i], b = m2[i];
			uint32_t t = step_load(steps + i);
			if (adam_one(i, n_matrix, loss_scale, inv_loss_scale, saturated, c, table, (float)grads[i], w, a, b, t)) {
				master[i] = w; m1[i] = a; m2[i] = b; step_store(steps + i, t); params[i] = (hf)w;
			}
		}
		return;
	}
	if (i0 + 4 <= n) {
		const half4 g = *reinterpret_cast<const half4*>(grads + i0);
		const bool all_zero = g[0] == (hf)0 && g[1] == (hf)0 && g[2] == (hf)0 && g[3] == (hf)0;
		if (all_zero && i0 >= n_matrix) return;  // nothing but the gradient is touched
		float4 w = *reinterpret_cast<float4*>(master + i0);
		float4 a = *reinterpret_cast<float4*>(m1 + i0);
		float4 b = *reinterpret_cast<float4*>(m2 + i0);
		uint4 t = step_load4(steps + i0);
		bool any = false;
		any |= adam_one(i0 + 0, n_matrix, loss_scale, inv_loss_scale, saturated, c, table, (float)g[0], w.x, a.x, b.x, t.x);
		any |= adam_one(i0 + 1, n_matrix, loss_scale, inv_loss_scale, saturated, c, table, (float)g[1], w.y, a.y, b.y, t.y);
		any |= adam_one(i0 + 2, n_matrix, loss_scale, inv_loss_scale, saturated, c, table, (float)g[2], w.z, a.z, b.z, t.z);
		any |= adam_one(i0 + 3, n_matrix, loss_scale, inv_loss_scale, saturated, c, table, (float)g[3], w.w, a.w, b.w, t.w);
		if (!any) return;
		*reinterpret_cast<float4*>(master + i0) = w;
		*reinterpret_cast<float4*>(m1 + i0) = a;
		*reinterpret_cast<float4*>(m2 + i0) = b;
		step_store4(steps + i0, t);
		*reinterpret_cast<half4*>(params + i0) = half4{(hf)w.x, (hf)w.y, (hf)w.z, (hf)w.w};
	} else {
		for (uint32_t i = i0; i < n; ++i) {
			float w = master[i], a = m1[i], b = m2[i];
			uint32_t t = step_load(steps + i);
			if (adam_one(i, n_matrix, loss_scale, inv_loss_scale, saturated, c, table, (float)grads[i], w, a, b, t)) {
				master[i] = w; m1[i] = a; m2[i] = b; step_store(steps + i, t); params[i] = (hf)w;
			}
		}
	}
}

bool n2_adam_counters_may_saturate(float beta1, float beta2) {
	const double small = std::ldexp(1.0, -26);
	return std::pow((double)beta1, (double)ADAM_TABLE) < small && std::pow((double)beta2, (double)ADAM_TABLE) < small;
}

N2_API int n2_adam_step(n2_stream_t stream, const n2_adam_config* config, uint32_t n_params, uint32_t n_matrix_params,
                        float loss_scale, float* d_master, n2_half* d_params, const n2_half* d_gradients, float* d_m1,
                        float* d_m2, uint32_t* d_steps) {
	return n2_adam_step_gated(stream, config, n_params, n_matrix_params, loss_scale, d_master, d_params, d_gradients, d_m1, d_m2, d_steps, 32, nullptr);
}

int n2_adam_step_gated(n2_stream_t stream, const n2_adam_config* config, uint32_t n_params, uint32_t n_matrix_params,
                       float loss_scale, float* d_master, n2_half* d_params, const n2_half* d_gradients, float* d_m1,
                       float* d_m2, void* d_steps, uint32_t steps_bits, const uint32_t* d_gate, const N2SlabReduce* sums, const N2StepEpilogue* epilogue,
                       hipEvent_t done_event) {
	N2_REQUIRE(config != nullptr, "n2_adam_step: config is null");
	if (n_params == 0) return N2_OK;
	N2_REQUIRE(d_master && d_params && d_gradients && d_m1 && d_m2 && d_steps, "n2_adam_step: null buffer");
	N2_REQUIRE(loss_scale > 0.f, "n2_adam_step: loss_scale must be positive");
	N2_REQUIRE(n_matrix_params <= n_params, "n2_adam_step: n_matrix_params %u > n_params %u", n_matrix_params, n_params);
	const uintptr_t a = reinterpret_cast<uintptr_t>(d_master) | reinterpret_cast<uintptr_t>(d_m1) | reinterpret_cast<uintptr_t>(d_m2) |
	                    reinterpret_cast<uintptr_t>(d_steps);
	N2_REQUIRE(a % 16 == 0, "n2_adam_step: fp32/uint32 buffers must be 16-byte aligned");
	N2_REQUIRE(reinterpret_cast<uintptr_t>(d_params) % 8 == 0 && reinterpret_cast<uintptr_t>(d_gradients) % 8 == 0,
	           "n2_adam_step: fp16 buffers must be 8-byte aligned");
	const uint32_t quads = (n_params + 3) / 4;
	hipStream_t s = n2_stream(stream);
	// The device's table for this pair of betas.  A new pair takes a free slot; its table is complete before any stream can
	// read it (the host waits for the kernel that fills it, once per pair).  When all slots are taken the least recently
	// used one is refilled after the whole device has gone idle, so that no step in flight still reads it.
	struct Slot { bool valid = false; float beta1 = 0.f, beta2 = 0.f; uint64_t used = 0; };
	static Slot slots[64][ADAM_SLOTS];
	static uint64_t clock = 0;
	static std::mutex lock;
	int dev = 0;
	N2_HIP(hipGetDevice(&dev));
	N2_REQUIRE(dev >= 0 && dev < 64, "n2_adam_step: device index %d not supported", dev);
	uint32_t slot = ADAM_SLOTS;
	{
		std::lock_guard<std::mutex> guard(lock);
		for (uint32_t k = 0; k < ADAM_SLOTS && slot == ADAM_SLOTS; ++k)
			if (slots[dev][k].valid && slots[dev][k].beta1 == config->beta1 && slots[dev][k].beta2 == config->beta2) slot = k;
		uint32_t victim = 0;  // a free slot if there is one, else the least recently used
		for (uint32_t k = 1; k < ADAM_SLOTS; ++k) {
			const Slot &c = slots[dev][k], &v = slots[dev][victim];
			if (v.valid && (!c.valid || c.used < v.used)) victim = k;
		}
		if (slot == ADAM_SLOTS) {
			slot = victim;
			if (slots[dev][slot].valid) N2_HIP(hipDeviceSynchronize());
			slots[dev][slot].valid = false;
			adam_table_kernel<<<dim3(ADAM_TABLE / 256), dim3(256), 0, s>>>(config->beta1, config->beta2, slot);
			N2_LAUNCH_CHECK();
			N2_HIP(hipStreamSynchronize(s));
			slots[dev][slot].valid = true; slots[dev][slot].beta1 = config->beta1; slots[dev][slot].beta2 = config->beta2;
		}
		slots[dev][slot].used = ++clock;
	}
	// 1 - beta^t == 1 in fp32 for every t past the table?
	const int saturated = n2_adam_counters_may_saturate(config->beta1, config->beta2) ? 1 : 0;
	int exp2 = 0;
	const float inv_loss_scale = (std::frexp(loss_scale, &exp2) == 0.5f && exp2 > -120 && exp2 < 120) ? 1.f / loss_scale : 0.f;
	N2ProfScope prof(N2_PROF_ADAM, s);
	N2SlabReduce plan = {};
	if (sums != nullptr && sums->units > 0) {
		plan = *sums;
		// the summed gradients must be this call's: inside d_gradients (the kernel turns their addresses into parameter numbers)
		const hf* g0 = reinterpret_cast<const hf*>(d_gradients);
		auto inside = [&](const hf* p, uint32_t count) { return count == 0 || (p >= g0 && p + count <= g0 + n_params); };
		N2_REQUIRE(inside(plan.ga, plan.params_a) && inside(plan.gb, plan.params_b) && inside(plan.extra_out, plan.extra_n > 0 ? 1u : 0u),
		           "n2_adam_step: the summed gradients do not lie inside d_gradients");
	}
	N2StepEpilogue epi = {};
	if (epilogue != nullptr && epilogue->values != nullptr) {
		epi = *epilogue;
		N2_REQUIRE(epi.n_ptr != nullptr && epi.sum_out != nullptr && epi.copy_n <= 256 && (epi.copy_n == 0 || (epi.copy_src && epi.copy_dst)),
		           "n2_adam_step: incomplete step epilogue");
	}
	const dim3 grid((quads + 255) / 256 + plan.units + (epi.values ? 1u : 0u));
	N2_REQUIRE(steps_bits == 32 || steps_bits == 16, "n2_adam_step: step counters of %u bits", steps_bits);
	N2_REQUIRE(steps_bits == 32 || saturated, "n2_adam_step: 16-bit step counters need betas whose powers underflow within %u steps", ADAM_TABLE);
	auto launch = [&](auto* steps) {
		using StepT = std::remove_pointer_t<decltype(steps)>;
		if (done_event != nullptr) {
			// the event is tied to this launch's own completion: no packet of its own behind the kernel, where an event record
			// costs the stream about 5 us before its next kernel starts
			hipExtLaunchKernelGGL(adam_step_kernel<StepT>, grid, dim3(256), 0, s, nullptr, done_event, 0, *config, n_params, n_matrix_params, loss_scale,
			                      inv_loss_scale, saturated, slot, d_gate, d_master, reinterpret_cast<hf*>(d_params), reinterpret_cast<const hf*>(d_gradients),
			                      d_m1, d_m2, steps, plan, epi);
		} else {
			adam_step_kernel<StepT><<<grid, dim3(256), 0, s>>>(*config, n_params, n_matrix_params, loss_scale, inv_loss_scale, saturated, slot, d_gate, d_master,
				reinterpret_cast<hf*>(d_params), reinterpret_cast<const hf*>(d_gradients), d_m1, d_m2, steps, plan, epi);
		}
	};
	if (steps_bits == 16) launch(static_cast<uint16_t*>(d_steps));
	else launch(static_cast<uint32_t*>(d_steps));
	N2_LAUNCH_CHECK();
	return N2_OK;
}

// Ema wrapper around the nested optimizer (configs/nerf/base.json:5-7, tcnn's EmaOptimizer): the bias-corrected
// exponential moving average of the fp16 working weights, kept in fp32 with an fp16 copy for inference.  Unlike Adam
// it touches every parameter in every step.
__global__ void __launch_bounds__(256) ema_step_kernel(uint32_t n, float decay, float debias_old, float debias_new, const hf* __restrict__ weights,
                                                       float* __restrict__ tmp, hf* __restrict__ ema) {
	const uint32_t i0 = (blockIdx.x * 256 + threadIdx.x) * 4;
	if (i0 >= n) return;
	if (i0 + 4 <= n) {
		const half4 w = *reinterpret_cast<const half4*>(weights + i0);
		float4 t = *reinterpret_cast<float4*>(tmp + i0);
		t.x = (t.x * decay * debias_old + (float)w[0] * (1.f - decay)) / debias_new;
		t.y = (t.y * decay * debias_old + (float)w[1] * (1.f - decay)) / debias_new;
		t.z = (t.z * decay * debias_old + (float)w[2] * (1.f - decay)) / debias_new;
		t.w = (t.w * decay * debias_old + (float)w[3] * (1.f - decay)) / debias_new;
		*reinterpret_cast<float4*>(tmp + i0) = t;
		*reinterpret_cast<half4*>(ema + i0) = half4{(hf)t.x, (hf)t.y, (hf)t.z, (hf)t.w};
	} else {
		for (uint32_t i = i0; i < n; ++i) {
			const float v = (tmp[i] * decay * debias_old + (float)weights[i] * (1.f - decay)) / debias_new;
			tmp[i] = v;
			ema[i] = (hf)v;
		}
	}
}

N2_API int n2_ema_step(n2_stream_t stream, uint32_t n_params, float decay, uint32_t step, const n2_half* d_weights, float* d_tmp,
                       n2_half* d_ema) {
	if (n_params == 0) return N2_OK;
	N2_REQUIRE(d_weights && d_tmp && d_ema, "n2_ema_step: null buffer");
	N2_REQUIRE(decay > 0.f && decay < 1.f, "n2_ema_step: decay %g outside (0, 1)", (double)decay);
	N2_REQUIRE(step >= 1, "n2_ema_step: step counts from 1 (the nested optimizer's step that just ran)");
	N2_REQUIRE(reinterpret_cast<uintptr_t>(d_tmp) % 16 == 0 && reinterpret_cast<uintptr_t>(d_weights) % 8 == 0 && reinterpret_cast<uintptr_t>(d_ema) % 8 == 0,
	           "n2_ema_step: buffers must be 16-byte (fp32) / 8-byte (fp16) aligned");
	const float debias_old = 1.f - (float)pow((double)decay, (double)(step - 1));
	const float debias_new = 1.f - (float)pow((double)decay, (double)step);
	const uint32_t quads = (n_params + 3) / 4;
	ema_step_kernel<<<dim3((quads + 255) / 256), dim3(256), 0, n2_stream(stream)>>>(n_params, decay, debias_old, debias_new,
		reinterpret_cast<const hf*>(d_weights), d_tmp, reinterpret_cast<hf*>(d_ema));
	N2_LAUNCH_CHECK();
	return N2_OK;
}
