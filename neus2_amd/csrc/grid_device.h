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

