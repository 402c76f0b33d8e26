// Device-side index arithmetic of the multi-resolution hash grid, shared by the stand-alone grid kernels and the
// fused field kernels: cell location, level mask and the entry index of a grid vertex.
#pragma once
#include "n2_common.h"

// ----------------------------------------------------------------------------
// device helpers
// ----------------------------------------------------------------------------

// pos = x*scale + 0.5 as one fused multiply-add, then floor: the integer cell
// and the fractional weight.  The fused form is part of the bit-exact contract
// with the CPU oracle.
__device__ __forceinline__ void n2_locate(float x, float scale, float& w, uint32_t& cell) {
	const float p = __fmaf_rn(x, scale, 0.5f);
	const float f = floorf(p);
	cell = (uint32_t)(int32_t)f;
	w = p - f;
}

// Level mask of tcnn's grid encoding: the limit is (max_level * n_output_features) / n_features_per_level in fp32
// and a level is off when level >= limit + 1e-3; the progressive mask adds level >= valid_levels.
__device__ __forceinline__ bool n2_level_masked(const N2LevelTable& tab, uint32_t level, uint32_t i) {
	if (tab.max_level_gpu == nullptr) return level >= tab.active_levels;  // uniform: the host has applied both rules
	const float limit = (tab.max_level_gpu[i] * (float)(tab.n_levels * tab.n_features)) / (float)tab.n_features;
	return (float)level >= limit + 1e-3f || level >= tab.valid_levels;
}

template <uint32_t MODE>
__device__ __forceinline__ uint32_t n2_entry(uint32_t entries, uint32_t res, uint32_t gx, uint32_t gy, uint32_t gz) {
	if (MODE == N2_LEVEL_DENSE) {
		// Positions inside [0,1]^3 never give a coordinate above res; the clamp only keeps
		// stray inputs (padding rows of a batch) inside the table.  The host has checked
		// res^3 + res^2 + res < 2*entries, so one subtraction is the modulo.
		gx = min(gx, res); gy = min(gy, res); gz = min(gz, res);
		uint32_t i = gx + gy * res + gz * res * res;
		return i >= entries ? i - entries : i;
	} else if (MODE == N2_LEVEL_HASH) {
		return (gx ^ (gy * 2654435761u) ^ (gz * 805459861u)) & (entries - 1u);
	} else if (MODE == N2_LEVEL_DENSE_MOD) {
		return (gx + gy * res + gz * res * res) % entries;
	} else {
		return (gx ^ (gy * 2654435761u) ^ (gz * 805459861u)) % entries;
	}
}


// ----------------------------------------------------------------------------
// Slopes of one (sample, level): the six values d feature_f / d x_d (before the level's scale factor) as one 16-byte
// block-float: 20-bit signed mantissas q_0..q_5 and a shared exponent e (value_i = q_i * 2^(e - 19), |value_i| < 2^e).
// The contraction of the slopes with a gradient then carries an error of 2^-20 of the largest slope, where fp16 storage
// (2^-11 of every slope) shows in the normals; fp32 storage takes 24 bytes.  A 12-byte form (15-bit mantissas, 6-bit
// exponent) is not enough: the second-order input J v of the SDF net cancels between the slopes' terms, and the weight
// gradients that follow from it then miss the oracle's by 7e-3 in relative L2.
//   word 0: q0 | q1 << 20     word 1: q1 >> 12 | q2 << 8 | q3 << 28     word 2: q3 >> 4 | q4 << 16
//   word 3: q4 >> 16 | q5 << 4 | e << 24
// ----------------------------------------------------------------------------
__device__ __forceinline__ uint4 n2_slopes_pack(const float (&v)[6]) {
	float m = 0.f;
#pragma unroll
	for (int i = 0; i < 6; ++i) m = fmaxf(m, fabsf(v[i]));
	int e = 0;
	(void)frexpf(m, &e);  // m = f * 2^e with f in [0.5, 1); 0 for m = 0
	e = min(max(e, -100), 100);
	uint32_t q[6];
#pragma unroll
	for (int i = 0; i < 6; ++i) {
		int x = (int)rintf(ldexpf(v[i], 19 - e));
		x = min(max(x, -524287), 524287);
		q[i] = (uint32_t)x & 0xFFFFFu;
	}
	uint4 w;
	w.x = q[0] | (q[1] << 20);
	w.y = (q[1] >> 12) | (q[2] << 8) | (q[3] << 28);
	w.z = (q[3] >> 4) | (q[4] << 16);
	w.w = (q[4] >> 16) | (q[5] << 4) | ((uint32_t)e << 24);
	return w;
}
// mantissas as floats and the factor 2^(e - 19) they share
__device__ __forceinline__ float n2_slopes_unpack(const uint4 w, float (&q)[6]) {
	auto sext20 = [](uint32_t x) { return (float)((int32_t)(x << 12) >> 12); };
	q[0] = sext20(w.x);
	q[1] = sext20((w.x >> 20) | (w.y << 12));
	q[2] = sext20(w.y >> 8);
	q[3] = sext20((w.y >> 28) | (w.z << 4));
	q[4] = sext20((w.z >> 16) | (w.w << 16));
	q[5] = sext20(w.w >> 4);
	return ldexpf(1.f, ((int32_t)w.w >> 24) - 19);
}
