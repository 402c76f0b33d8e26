// CPU oracle for the NeuS2 SDF-field hot path.  TEST INFRASTRUCTURE ONLY.
//
// This file is the checker that the GPU library is compared against (and the
// thing timed as the "cpu_baseline" leg of the benchmark).  It is never linked
// into, imported by, or called from the product library.
//
// It is a scalar + OpenMP fp32 restatement of the arithmetic that the
// reference reaches through its tcnn submodule (dependencies/neus2_tcnn, a
// fork of NVlabs/tiny-cuda-nn that is absent from /root/reference, no pinned
// commit) and of the in-tree glue that drives it.  Because the submodule
// source is absent, parity of the tcnn-internal parts is anchored on the
// reference's call sites, cited at each function, and on what the mathematics
// fixes (see tests/test_oracle_*.py): closed forms, scipy/torch library
// routines, autograd of an independent forward, finite differences.
//
// Parity status per function (what independent check pins it):
//   orc_grid_make_levels      closed form + published level table        pinned
//   orc_grid_indices          integer closed form, brute force           pinned
//   orc_grid_forward          scipy.ndimage.map_coordinates, invariants  pinned
//   orc_grid_backward         torch autograd of independent forward      pinned
//   orc_grid_backward_backward_input  torch double backward              pinned
//   orc_mlp_*                 torch fp64 matmul + autograd/double bwd    pinned
//   orc_sh4                   scipy.special.sph_harm_y                   pinned
//   orc_adam_step             torch.optim.Adam on dense params           pinned
//     (zero-gradient skip of non-matrix params and the per-parameter step
//      counters follow tiny-cuda-nn's published Adam; "parity unpinned"
//      against the fork, which is not in the container)
//   orc_field_*               autograd of a torch restatement of
//                             nerf_network.h's composition               pinned
//   orc_composite_*           closed-form cases + finite differences     pinned
//   orc_pcg32_*               published PCG32 outputs for seed (42, 54),
//                             advance(n) == n draws                      pinned
//     (agreement with the pcg32 class of the absent fork: parity unpinned)
//   orc_generate_grid_samples integer index closed form (bijection at full
//                             coverage), positions inside their cell     pinned
//   orc_splat_grid_max / orc_ema_grid / orc_grid_mean / orc_grid_to_bitfield
//                             numpy restatements, brute-force pooling    pinned
//   fp16 rounding order inside the reference MLP (fp16 accumulate):
//                             parity unpinned (source absent)
//
// Layout convention: every matrix is "rows x N", element (r, i) at r*N + i
// (the SoA / row-major layout the reference's grid encoding prefers,
// nerf_network.h:121-122) unless a function says otherwise.

#include <cmath>
#include <cstdint>
#include <cstring>
#include <vector>
#include <algorithm>
#ifdef _OPENMP
#include <omp.h>
#endif

#define ORC_API extern "C" __attribute__((visibility("default")))

ORC_API int orc_num_threads() {
#ifdef _OPENMP
	return omp_get_max_threads();
#else
	return 1;
#endif
}

// ---------------------------------------------------------------------------
// Hash-grid encoding (tcnn GridEncoding<T,3,2>; call sites nerf_network.h:46,
// 184-190, 234, 419-429, 534-544; config configs/nerf/base.json:29-39).
// ---------------------------------------------------------------------------

// Level geometry.  scale_l = 2^(l*log2(b))*base - 1, res_l = ceil(scale_l)+1,
// entries_l = min(round_up(res_l^3, 8), 2^log2_T); offsets are the prefix sum.
// The reference confirms the top-resolution relation at src/testbed.cu:2165-2179.
// All float steps are fp32 so that the table is identical wherever it is built.
ORC_API void orc_grid_make_levels(uint32_t n_levels, uint32_t log2_hashmap_size, uint32_t base_resolution,
                                  float per_level_scale, float* scale, uint32_t* resolution,
                                  uint32_t* entries, uint32_t* offset /* n_levels+1 */) {
	uint32_t off = 0;
	const float log2_b = std::log2(per_level_scale);
	for (uint32_t l = 0; l < n_levels; ++l) {
		const float s = exp2f((float)l * log2_b) * (float)base_resolution - 1.0f;
		const uint32_t res = (uint32_t)ceilf(s) + 1u;
		const uint32_t max_params = 0xFFFFFFFFu / 2u;
		const double cube = (double)res * (double)res * (double)res;
		uint32_t n = cube > (double)max_params ? max_params : res * res * res;
		n = (n + 7u) / 8u * 8u;
		n = std::min(n, 1u << log2_hashmap_size);
		scale[l] = s; resolution[l] = res; entries[l] = n; offset[l] = off;
		off += n;
	}
	offset[n_levels] = off;
}

struct GridDesc {
	uint32_t n_levels;
	const float* scale;
	const uint32_t* resolution;
	const uint32_t* entries;
	const uint32_t* offset;
};

static inline uint32_t grid_entry(uint32_t entries, uint32_t res, uint32_t gx, uint32_t gy, uint32_t gz) {
	// Dense index while the stride still fits in the level, else the spatial
	// hash with primes (1, 2654435761, 805459861); always reduced mod entries.
	const uint32_t g[3] = {gx, gy, gz};
	uint32_t stride = 1, index = 0;
	for (uint32_t d = 0; d < 3 && stride <= entries; ++d) {
		index += g[d] * stride;
		stride *= res;
	}
	if (entries < stride) {
		index = (gx * 1u) ^ (gy * 2654435761u) ^ (gz * 805459861u);
	}
	return index % entries;
}

static inline void pos_fract(float x, float scale, float* w, uint32_t* cell) {
	// pos = x*scale + 0.5 as ONE fused multiply-add (what nvcc emits for the
	// reference expression and what the GPU kernel uses), then floor.
	const float p = fmaf(x, scale, 0.5f);
	const float f = floorf(p);
	*cell = (uint32_t)(int32_t)f;
	*w = p - f;
}

// idx: [L][8][N] entry index (without the level offset); w: [L][3][N] fractional weights.
ORC_API void orc_grid_indices(uint32_t n_levels, const float* scale, const uint32_t* resolution, const uint32_t* entries,
                              const float* xyz, uint32_t N, uint32_t* idx, float* w) {
	#pragma omp parallel for collapse(2) schedule(static)
	for (uint32_t l = 0; l < n_levels; ++l) {
		for (uint32_t i = 0; i < N; ++i) {
			float ww[3]; uint32_t c[3];
			for (int d = 0; d < 3; ++d) pos_fract(xyz[(size_t)d * N + i], scale[l], &ww[d], &c[d]);
			for (uint32_t k = 0; k < 8; ++k) {
				idx[((size_t)l * 8 + k) * N + i] =
					grid_entry(entries[l], resolution[l], c[0] + (k & 1u), c[1] + ((k >> 1) & 1u), c[2] + ((k >> 2) & 1u));
			}
			if (w) for (int d = 0; d < 3; ++d) w[((size_t)l * 3 + d) * N + i] = ww[d];
		}
	}
}

// Forward: y[(l*2+f)][i] = sum_c weight_c * params[(offset_l + entry_c)*2 + f]
// dy_dx (optional): [(l*2+f)][i][3] fp32, = scale_l * sum over the 4 corner
// pairs of (prod of the other two weights) * (val_right - val_left).
ORC_API void orc_grid_forward(uint32_t n_levels, const float* scale, const uint32_t* resolution, const uint32_t* entries,
                              const uint32_t* offset, const float* params, const float* xyz, uint32_t N,
                              float* y, float* dy_dx) {
	#pragma omp parallel for collapse(2) schedule(static)
	for (uint32_t l = 0; l < n_levels; ++l) {
		for (uint32_t i = 0; i < N; ++i) {
			const float* P = params + (size_t)offset[l] * 2;
			float w[3]; uint32_t c[3];
			for (int d = 0; d < 3; ++d) pos_fract(xyz[(size_t)d * N + i], scale[l], &w[d], &c[d]);
			float v[8][2];
			for (uint32_t k = 0; k < 8; ++k) {
				const uint32_t e = grid_entry(entries[l], resolution[l], c[0] + (k & 1u), c[1] + ((k >> 1) & 1u), c[2] + ((k >> 2) & 1u));
				v[k][0] = P[(size_t)e * 2]; v[k][1] = P[(size_t)e * 2 + 1];
			}
			for (int f = 0; f < 2; ++f) {
				float acc = 0.f;
				for (uint32_t k = 0; k < 8; ++k) {
					float wt = 1.f;
					for (int d = 0; d < 3; ++d) wt *= ((k >> d) & 1u) ? w[d] : 1.f - w[d];
					acc += wt * v[k][f];
				}
				y[((size_t)l * 2 + f) * N + i] = acc;
				if (dy_dx) {
					for (int gd = 0; gd < 3; ++gd) {
						float g = 0.f;
						const int d1 = (gd + 1) % 3, d2 = (gd + 2) % 3;
						for (uint32_t k = 0; k < 8; ++k) {
							if ((k >> gd) & 1u) continue;  // k = left corner of the pair
							float wt = scale[l];
							wt *= ((k >> d1) & 1u) ? w[d1] : 1.f - w[d1];
							wt *= ((k >> d2) & 1u) ? w[d2] : 1.f - w[d2];
							g += wt * (v[k | (1u << gd)][f] - v[k][f]);
						}
						dy_dx[(((size_t)l * 2 + f) * N + i) * 3 + gd] = g;
					}
				}
			}
		}
	}
}

// Backward.  grad (n_params, fp32) is ACCUMULATED into (caller zeroes it for
// the reference's Overwrite mode, nerf_network.h:419-429); pass grad = null for
// the Ignore mode of the normals pass (nerf_network.h:234).
// dL_dx (optional, [3][N]) = sum_k dL_dy[k] * dy_dx[k].
ORC_API void orc_grid_backward(uint32_t n_levels, const float* scale, const uint32_t* resolution, const uint32_t* entries,
                               const uint32_t* offset, const float* params, const float* xyz, uint32_t N,
                               const float* dL_dy, float* grad, float* dL_dx) {
	if (grad) {
		#pragma omp parallel for schedule(dynamic, 1)
		for (uint32_t l = 0; l < n_levels; ++l) {
			float* G = grad + (size_t)offset[l] * 2;
			for (uint32_t i = 0; i < N; ++i) {
				float w[3]; uint32_t c[3];
				for (int d = 0; d < 3; ++d) pos_fract(xyz[(size_t)d * N + i], scale[l], &w[d], &c[d]);
				const float g0 = dL_dy[((size_t)l * 2) * N + i], g1 = dL_dy[((size_t)l * 2 + 1) * N + i];
				for (uint32_t k = 0; k < 8; ++k) {
					const uint32_t e = grid_entry(entries[l], resolution[l], c[0] + (k & 1u), c[1] + ((k >> 1) & 1u), c[2] + ((k >> 2) & 1u));
					float wt = 1.f;
					for (int d = 0; d < 3; ++d) wt *= ((k >> d) & 1u) ? w[d] : 1.f - w[d];
					G[(size_t)e * 2] += g0 * wt;
					G[(size_t)e * 2 + 1] += g1 * wt;
				}
			}
		}
	}
	if (dL_dx) {
		std::vector<float> y((size_t)n_levels * 2 * N), J((size_t)n_levels * 2 * N * 3);
		orc_grid_forward(n_levels, scale, resolution, entries, offset, params, xyz, N, y.data(), J.data());
		#pragma omp parallel for schedule(static)
		for (uint32_t i = 0; i < N; ++i) {
			float r[3] = {0, 0, 0};
			for (uint32_t k = 0; k < n_levels * 2; ++k) {
				const float g = dL_dy[(size_t)k * N + i];
				for (int d = 0; d < 3; ++d) r[d] += g * J[((size_t)k * N + i) * 3 + d];
			}
			for (int d = 0; d < 3; ++d) dL_dx[(size_t)d * N + i] = r[d];
		}
	}
}

// Second order of the input gradient (nerf_network.h:534-544).  The first
// backward computes q_d = sum_{l,f} g_{lf} * dy_{lf}/dx_d.  With v = dL/dq:
//   grad[corner c of (l,f)] += g_{lf} * scale_l * sum_d v_d * s_{c,d} * prod_{d'!=d} w_{c,d'}
//   dL_ddLdoutput[(l,f)]     = sum_d dy_{lf}/dx_d * v_d
//   dL_dinput[b]             = sum_a v_a sum_{l,f} g_{lf} d2y_{lf}/dx_a dx_b   (a != b)
// Any output pointer may be null.
ORC_API void orc_grid_backward_backward_input(uint32_t n_levels, const float* scale, const uint32_t* resolution,
                                              const uint32_t* entries, const uint32_t* offset, const float* params,
                                              const float* xyz, uint32_t N, const float* v, const float* g,
                                              float* grad, float* dL_ddLdoutput, float* dL_dinput) {
	if (dL_dinput) std::memset(dL_dinput, 0, sizeof(float) * 3 * (size_t)N);
	std::vector<float> din_lv;
	if (dL_dinput) din_lv.assign((size_t)n_levels * 3 * N, 0.f);
	#pragma omp parallel for schedule(dynamic, 1)
	for (uint32_t l = 0; l < n_levels; ++l) {
		float* G = grad ? grad + (size_t)offset[l] * 2 : nullptr;
		const float* P = params + (size_t)offset[l] * 2;
		const float sc = scale[l];
		for (uint32_t i = 0; i < N; ++i) {
			float w[3]; uint32_t c[3];
			for (int d = 0; d < 3; ++d) pos_fract(xyz[(size_t)d * N + i], sc, &w[d], &c[d]);
			const float vv[3] = {v[i], v[(size_t)N + i], v[(size_t)2 * N + i]};
			const float gg[2] = {g[((size_t)l * 2) * N + i], g[((size_t)l * 2 + 1) * N + i]};
			float out[2] = {0, 0};
			float din[3] = {0, 0, 0};
			for (uint32_t k = 0; k < 8; ++k) {
				const uint32_t e = grid_entry(entries[l], resolution[l], c[0] + (k & 1u), c[1] + ((k >> 1) & 1u), c[2] + ((k >> 2) & 1u));
				float wd[3], sd[3];
				for (int d = 0; d < 3; ++d) { wd[d] = ((k >> d) & 1u) ? w[d] : 1.f - w[d]; sd[d] = ((k >> d) & 1u) ? 1.f : -1.f; }
				// d(weight_c)/dx_d = scale * s_d * prod of other two weights
				const float dw[3] = {sc * sd[0] * wd[1] * wd[2], sc * sd[1] * wd[0] * wd[2], sc * sd[2] * wd[0] * wd[1]};
				const float coef = vv[0] * dw[0] + vv[1] * dw[1] + vv[2] * dw[2];
				const float p0 = P[(size_t)e * 2], p1 = P[(size_t)e * 2 + 1];
				if (G) { G[(size_t)e * 2] += gg[0] * coef; G[(size_t)e * 2 + 1] += gg[1] * coef; }
				out[0] += coef * p0; out[1] += coef * p1;
				if (dL_dinput) {
					// d2(weight_c)/dx_a dx_b = scale^2 s_a s_b w_third
					const float gp = gg[0] * p0 + gg[1] * p1;
					const float h01 = sc * sc * sd[0] * sd[1] * wd[2];
					const float h02 = sc * sc * sd[0] * sd[2] * wd[1];
					const float h12 = sc * sc * sd[1] * sd[2] * wd[0];
					din[0] += gp * (vv[1] * h01 + vv[2] * h02);
					din[1] += gp * (vv[0] * h01 + vv[2] * h12);
					din[2] += gp * (vv[0] * h02 + vv[1] * h12);
				}
			}
			if (dL_ddLdoutput) {
				dL_ddLdoutput[((size_t)l * 2) * N + i] = out[0];
				dL_ddLdoutput[((size_t)l * 2 + 1) * N + i] = out[1];
			}
			if (dL_dinput) for (int d = 0; d < 3; ++d) din_lv[((size_t)l * 3 + d) * N + i] = din[d];
		}
	}
	if (dL_dinput) {
		for (uint32_t l = 0; l < n_levels; ++l)
			for (size_t j = 0; j < (size_t)3 * N; ++j) dL_dinput[j] += din_lv[(size_t)l * 3 * N + j];
	}
}

// ---------------------------------------------------------------------------
// Fully fused MLP (tcnn FullyFusedMLP<T,64>; created at nerf_network.h:57,65
// from configs/nerf/base.json:40-47,63-69).  No bias, ReLU hidden activations,
// linear output.  Weights: layers concatenated, each row-major [out][in]:
//   W_0 [width][in_width], W_1..W_{H-1} [width][width], W_H [out_width][width]
// (the layout utils/mlp_weights.txt is stored in, nerf_network.h:774-803).
// hidden: [H][width][N] post-activation values.
// ---------------------------------------------------------------------------

struct MlpDesc { uint32_t in_w, width, n_hidden, out_w; };

static inline const float* mlp_layer(const MlpDesc& m, const float* W, uint32_t k, uint32_t* rows, uint32_t* cols) {
	size_t off = 0;
	for (uint32_t j = 0; j < k; ++j) off += (size_t)m.width * (j == 0 ? m.in_w : m.width);
	*rows = (k == m.n_hidden) ? m.out_w : m.width;
	*cols = (k == 0) ? m.in_w : m.width;
	return W + off;
}
static inline size_t mlp_layer_off(const MlpDesc& m, uint32_t k) {
	size_t off = 0;
	for (uint32_t j = 0; j < k; ++j) off += (size_t)m.width * (j == 0 ? m.in_w : m.width);
	return off;
}

// Round an fp32 value to the nearest fp16 (ties to even) and back: the storage
// precision of activations between layers in the reference (T = __half).
static inline float round_fp16(float f) {
	uint32_t x;
	std::memcpy(&x, &f, 4);
	const uint32_t sign = x & 0x80000000u;
	x &= 0x7FFFFFFFu;
	float out;
	if (x >= 0x7F800000u) {  // inf / nan
		out = f;
		return out;
	}
	if (x >= 0x477FF000u) {  // rounds to >= 65520 -> inf
		x = 0x7F800000u;
	} else if (x < 0x38800000u) {  // below the smallest normal half: fixed-point rounding to multiples of 2^-24
		float a;
		std::memcpy(&a, &x, 4);
		const float magic = 0.5f;  // adding 0.5 aligns the mantissa so that the ulp is 2^-24
		a = (a + magic) - magic;
		std::memcpy(&x, &a, 4);
	} else {
		const uint32_t lsb = (x >> 13) & 1u;
		x += 0xFFFu + lsb;
		x &= ~0x1FFFu;
	}
	x |= sign;
	std::memcpy(&out, &x, 4);
	return out;
}
ORC_API void orc_round_fp16(const float* in, float* out, uint32_t n) {
	for (uint32_t i = 0; i < n; ++i) out[i] = round_fp16(in[i]);
}

ORC_API uint32_t orc_mlp_n_params(uint32_t in_w, uint32_t width, uint32_t n_hidden, uint32_t out_w) {
	return width * in_w + (n_hidden - 1) * width * width + out_w * width;
}

// y = W_H relu(... relu(W_0 x)); hidden may be null (inference).
// round_hidden != 0 rounds every hidden activation to fp16 before it feeds the
// next layer, as the reference's fp16 activation storage does.
ORC_API void orc_mlp_forward(uint32_t in_w, uint32_t width, uint32_t n_hidden, uint32_t out_w, const float* W,
                             const float* x, uint32_t N, float* y, float* hidden, int round_hidden) {
	const MlpDesc m{in_w, width, n_hidden, out_w};
	#pragma omp parallel
	{
		std::vector<float> a(std::max(in_w, width)), b(std::max(out_w, width));
		#pragma omp for schedule(static)
		for (uint32_t i = 0; i < N; ++i) {
			for (uint32_t r = 0; r < in_w; ++r) a[r] = x[(size_t)r * N + i];
			for (uint32_t k = 0; k <= n_hidden; ++k) {
				uint32_t rows, cols;
				const float* Wk = mlp_layer(m, W, k, &rows, &cols);
				for (uint32_t r = 0; r < rows; ++r) {
					float s = 0.f;
					for (uint32_t c = 0; c < cols; ++c) s += Wk[(size_t)r * cols + c] * a[c];
					b[r] = (k < n_hidden) ? std::max(s, 0.f) : s;
					if (k < n_hidden && round_hidden) b[r] = round_fp16(b[r]);
				}
				if (k < n_hidden) {
					if (hidden) for (uint32_t r = 0; r < rows; ++r) hidden[((size_t)k * width + r) * N + i] = b[r];
					for (uint32_t r = 0; r < rows; ++r) a[r] = b[r];
				} else {
					for (uint32_t r = 0; r < rows; ++r) y[(size_t)r * N + i] = b[r];
				}
			}
		}
	}
}

// Backward.  dL_dx optional [in_w][N]; dW optional (n_params), ACCUMULATED
// (caller zeroes for Overwrite; null for Ignore: nerf_network.h:229,340,402,509).
ORC_API void orc_mlp_backward(uint32_t in_w, uint32_t width, uint32_t n_hidden, uint32_t out_w, const float* W,
                              const float* x, const float* hidden, const float* dL_dy, uint32_t N,
                              float* dL_dx, float* dW) {
	const MlpDesc m{in_w, width, n_hidden, out_w};
	const size_t n_params = orc_mlp_n_params(in_w, width, n_hidden, out_w);
	int nt = 1;
#ifdef _OPENMP
	nt = omp_get_max_threads();
#endif
	std::vector<std::vector<double>> dWt;
	if (dW) dWt.assign(nt, std::vector<double>(n_params, 0.0));
	#pragma omp parallel
	{
		int tid = 0;
#ifdef _OPENMP
		tid = omp_get_thread_num();
#endif
		std::vector<float> d(std::max({in_w, width, out_w})), dn(std::max({in_w, width, out_w}));
		#pragma omp for schedule(static)
		for (uint32_t i = 0; i < N; ++i) {
			for (uint32_t r = 0; r < out_w; ++r) d[r] = dL_dy[(size_t)r * N + i];
			for (int k = (int)n_hidden; k >= 0; --k) {
				uint32_t rows, cols;
				const float* Wk = mlp_layer(m, W, (uint32_t)k, &rows, &cols);
				// input of layer k
				auto in_at = [&](uint32_t c) -> float {
					return k == 0 ? x[(size_t)c * N + i] : hidden[((size_t)(k - 1) * width + c) * N + i];
				};
				if (dW) {
					double* D = dWt[tid].data() + mlp_layer_off(m, (uint32_t)k);
					for (uint32_t r = 0; r < rows; ++r) {
						if (d[r] == 0.f) continue;
						for (uint32_t c = 0; c < cols; ++c) D[(size_t)r * cols + c] += (double)d[r] * (double)in_at(c);
					}
				}
				if (k == 0 && !dL_dx) break;
				for (uint32_t c = 0; c < cols; ++c) {
					float s = 0.f;
					for (uint32_t r = 0; r < rows; ++r) s += Wk[(size_t)r * cols + c] * d[r];
					// ReLU mask of the activation that fed this layer
					if (k > 0 && !(in_at(c) > 0.f)) s = 0.f;
					dn[c] = s;
				}
				std::swap(d, dn);
			}
			if (dL_dx) for (uint32_t c = 0; c < in_w; ++c) dL_dx[(size_t)c * N + i] = d[c];
		}
	}
	if (dW) for (int t = 0; t < nt; ++t) for (size_t j = 0; j < n_params; ++j) dW[j] += (float)dWt[t][j];
}

// Second order of the input gradient (the reference fork's addition, called at
// nerf_network.h:560-571; README.md:13-19).  The first backward gives
// q = J_x^T g with J_x = W_H M_{H-1} W_{H-1} ... M_0 W_0, M_k = diag(hidden_k > 0).
// With v = dL/dq the scalar is s = g^T J_x v, and
//   a_0 = M_0 W_0 v, a_k = M_k W_k a_{k-1};  b_{H-1} = M_{H-1} W_H^T g, b_{k-1} = M_{k-1} W_k^T b_k
//   dW_0 += b_0 v^T, dW_k += b_k a_{k-1}^T, dW_H += g a_{H-1}^T
//   dL_ddLdoutput = W_H a_{H-1}          (dL_dinput is identically zero for ReLU)
ORC_API void orc_mlp_backward_backward_input(uint32_t in_w, uint32_t width, uint32_t n_hidden, uint32_t out_w,
                                             const float* W, const float* hidden, const float* v, const float* g,
                                             uint32_t N, float* dW, float* dL_ddLdoutput) {
	const MlpDesc m{in_w, width, n_hidden, out_w};
	const size_t n_params = orc_mlp_n_params(in_w, width, n_hidden, out_w);
	int nt = 1;
#ifdef _OPENMP
	nt = omp_get_max_threads();
#endif
	std::vector<std::vector<double>> dWt;
	if (dW) dWt.assign(nt, std::vector<double>(n_params, 0.0));
	#pragma omp parallel
	{
		int tid = 0;
#ifdef _OPENMP
		tid = omp_get_thread_num();
#endif
		std::vector<float> a((size_t)n_hidden * width), b((size_t)n_hidden * width);
		#pragma omp for schedule(static)
		for (uint32_t i = 0; i < N; ++i) {
			auto mask = [&](uint32_t k, uint32_t r) { return hidden[((size_t)k * width + r) * N + i] > 0.f; };
			// forward-propagate v
			for (uint32_t k = 0; k < n_hidden; ++k) {
				uint32_t rows, cols;
				const float* Wk = mlp_layer(m, W, k, &rows, &cols);
				for (uint32_t r = 0; r < rows; ++r) {
					float s = 0.f;
					for (uint32_t c = 0; c < cols; ++c) s += Wk[(size_t)r * cols + c] * (k == 0 ? v[(size_t)c * N + i] : a[(size_t)(k - 1) * width + c]);
					a[(size_t)k * width + r] = mask(k, r) ? s : 0.f;
				}
			}
			// backward-propagate g
			for (int k = (int)n_hidden - 1; k >= 0; --k) {
				uint32_t rows, cols;
				const float* Wn = mlp_layer(m, W, (uint32_t)k + 1, &rows, &cols);
				for (uint32_t c = 0; c < cols; ++c) {
					float s = 0.f;
					for (uint32_t r = 0; r < rows; ++r)
						s += Wn[(size_t)r * cols + c] * ((uint32_t)k + 1 == n_hidden ? g[(size_t)r * N + i] : b[(size_t)(k + 1) * width + r]);
					b[(size_t)k * width + c] = mask((uint32_t)k, c) ? s : 0.f;
				}
			}
			if (dW) {
				double* D = dWt[tid].data();
				for (uint32_t k = 0; k <= n_hidden; ++k) {
					uint32_t rows, cols;
					mlp_layer(m, W, k, &rows, &cols);
					double* Dk = D + mlp_layer_off(m, k);
					for (uint32_t r = 0; r < rows; ++r) {
						const float left = (k == n_hidden) ? g[(size_t)r * N + i] : b[(size_t)k * width + r];
						if (left == 0.f) continue;
						for (uint32_t c = 0; c < cols; ++c) {
							const float right = (k == 0) ? v[(size_t)c * N + i] : a[(size_t)(k - 1) * width + c];
							Dk[(size_t)r * cols + c] += (double)left * (double)right;
						}
					}
				}
			}
			if (dL_ddLdoutput) {
				uint32_t rows, cols;
				const float* Wk = mlp_layer(m, W, n_hidden, &rows, &cols);
				for (uint32_t r = 0; r < rows; ++r) {
					float s = 0.f;
					for (uint32_t c = 0; c < cols; ++c) s += Wk[(size_t)r * cols + c] * a[(size_t)(n_hidden - 1) * width + c];
					dL_ddLdoutput[(size_t)r * N + i] = s;
				}
			}
		}
	}
	if (dW) for (int t = 0; t < nt; ++t) for (size_t j = 0; j < n_params; ++j) dW[j] += (float)dWt[t][j];
}

// ---------------------------------------------------------------------------
// Direction encoding: real spherical harmonics of degree 4 (16 values) of the
// unit vector 2*d - 1 (tcnn SphericalHarmonics inside the Composite encoding,
// configs/nerf/base.json:48-62, nerf_network.h:42,251-257).
// dir: [3][N] in [0,1]; out: [16][N].
// ---------------------------------------------------------------------------
ORC_API void orc_sh4(const float* dir, uint32_t N, float* out) {
	#pragma omp parallel for schedule(static)
	for (uint32_t i = 0; i < N; ++i) {
		const float x = dir[i] * 2.f - 1.f, y = dir[(size_t)N + i] * 2.f - 1.f, z = dir[(size_t)2 * N + i] * 2.f - 1.f;
		const float xy = x * y, xz = x * z, yz = y * z, x2 = x * x, y2 = y * y, z2 = z * z;
		float o[16];
		o[0] = 0.28209479177387814f;
		o[1] = -0.48860251190291987f * y;
		o[2] = 0.48860251190291987f * z;
		o[3] = -0.48860251190291987f * x;
		o[4] = 1.0925484305920792f * xy;
		o[5] = -1.0925484305920792f * yz;
		o[6] = 0.94617469575755997f * z2 - 0.31539156525251999f;
		o[7] = -1.0925484305920792f * xz;
		o[8] = 0.54627421529603959f * x2 - 0.54627421529603959f * y2;
		o[9] = 0.59004358992664352f * y * (-3.0f * x2 + y2);
		o[10] = 2.8906114426405538f * xy * z;
		o[11] = 0.45704579946446572f * y * (1.0f - 5.0f * z2);
		o[12] = 0.3731763325901154f * z * (5.0f * z2 - 3.0f);
		o[13] = 0.45704579946446572f * x * (1.0f - 5.0f * z2);
		o[14] = 1.4453057213202769f * z * (x2 - y2);
		o[15] = 0.59004358992664352f * x * (-x2 + 3.0f * y2);
		for (int k = 0; k < 16; ++k) out[(size_t)k * N + i] = o[k];
	}
}

// ---------------------------------------------------------------------------
// Adam (tcnn Adam reached through Trainer::optimizer_step, src/testbed_nerf.cu:3498;
// hyper-parameters configs/nerf/base.json:13-26; LOSS_SCALE testbed.h:237).
// g = grad/loss_scale; params at index >= n_matrix_params whose g == 0 are
// skipped entirely (their step counter does not advance); matrix params get
// g += l2_reg*w; per-parameter step counter t drives the bias correction
// lr*sqrt(1-b2^t)/(1-b1^t); w -= lr_eff*m/(sqrt(v)+eps).
// ---------------------------------------------------------------------------
ORC_API void orc_adam_step(uint32_t n, uint32_t n_matrix_params, float loss_scale, float lr, float beta1, float beta2,
                           float eps, float l2_reg, float* w, const float* grad, float* m1, float* m2, uint32_t* steps) {
	#pragma omp parallel for schedule(static)
	for (uint32_t i = 0; i < n; ++i) {
		float g = grad[i] / loss_scale;
		if (i >= n_matrix_params) {
			if (g == 0.f) continue;
		} else {
			g += l2_reg * w[i];
		}
		const uint32_t t = ++steps[i];
		const float gs = g * g;
		const float a = m1[i] = beta1 * m1[i] + (1.f - beta1) * g;
		const float b = m2[i] = beta2 * m2[i] + (1.f - beta2) * gs;
		const float lr_eff = lr * sqrtf(1.f - powf(beta2, (float)t)) / (1.f - powf(beta1, (float)t));
		w[i] -= lr_eff * a / (sqrtf(b) + eps);
	}
}

// ---------------------------------------------------------------------------
// NeuS alpha compositing + loss + hand-derived backward, one ray at a time:
// compute_loss_kernel_train_nerf_with_global_movement, src/testbed_nerf.cu:1465-1996,
// restricted to the static path (no global movement, no envmap, no exposure /
// depth / mask supervision, Logistic colour activation, Huber(0.1)/5 loss,
// BENT_DIR 1, NORMAL_VECTORS_NORMALIZED 0).
//
// The reference allocates the compacted range of a ray with atomicAdd, so the
// order of rays in the compacted batch is a race; here the ranges are handed
// out in ray order (one of the orders the reference can produce).
//
//  numsteps   [n_rays][2] in: (samples, first sample); out: (compacted samples, compacted first)
//  net_out    [*][16]  network output per marched sample (values as stored in fp16)
//  coords     [*][7]   NerfCoordinate per marched sample
//  rgb_target [n_rays][3]
//  dloss      [max_compacted][16] out (rows 11..15 are left unset by the reference; zero here)
//  coords_out [max_compacted][7] out
//  loss       [n_rays] out: mean over channels / n_rays_norm        (testbed_nerf.cu:1717-1719)
//  counter    out: total number of samples the rays wanted to keep (may exceed max_compacted)
// ---------------------------------------------------------------------------
struct CompositeCfg {
	float loss_scale;        // LOSS_SCALE = 128, testbed.h:237
	float ek_loss_weight;    // hyperparams.ek_loss_weight
	float cos_anneal_ratio;  // nerf_network.h:1109-1118 (1 when anneal_end = 0)
	float background[3];
	uint32_t n_rays_norm;    // n_rays_per_batch: what loss and gradients are divided by (:1756)
	float min_step;          // MIN_CONE_STEPSIZE = sqrt(3)/1024 (:52-53)
	float max_step;          // MIN_CONE_STEPSIZE * 2^(NERF_CASCADES-1): unwarp_dt (:617-620)
	int exact_inv_s;         // 0: 10*variance is formed in fp16 as in the reference (:1581); 1: in fp32 (smooth, for finite differences)
};

static inline float logistic(float x) { return 1.f / (1.f + expf(-x)); }

struct SampleAlpha {
	float alpha, p_div_c, iter_cos, true_cos, inv_s, sdf, dt, next_sdf;
	float rgb[3], n[3];
};

static inline SampleAlpha sample_alpha(const float* o, float warped_dt, const float* dir, const CompositeCfg& c) {
	SampleAlpha s;
	s.dt = warped_dt * (c.max_step - c.min_step) + c.min_step;  // unwarp_dt
	for (int k = 0; k < 3; ++k) { s.rgb[k] = logistic(o[k]); s.n[k] = o[4 + k]; }
	s.inv_s = expf(c.exact_inv_s ? 10.f * o[7] : round_fp16(10.f * o[7]));  // the product is formed in fp16 (:1581)
	s.sdf = o[3];
	s.true_cos = dir[0] * s.n[0] + dir[1] * s.n[1] + dir[2] * s.n[2];
	const float a = std::max(-s.true_cos * 0.5f + 0.5f, 0.f), b = std::max(-s.true_cos, 0.f);
	s.iter_cos = -(a * (1.f - c.cos_anneal_ratio) + b * c.cos_anneal_ratio);
	s.next_sdf = s.sdf + s.iter_cos * s.dt * 0.5f;
	const float prev_sdf = s.sdf - s.iter_cos * s.dt * 0.5f;
	const float next_cdf = logistic(s.next_sdf * s.inv_s), prev_cdf = logistic(prev_sdf * s.inv_s);
	s.p_div_c = (prev_cdf - next_cdf + 1e-5f) / (prev_cdf + 1e-5f);
	s.alpha = std::min(std::max(s.p_div_c, 0.f), 1.f);
	return s;
}

ORC_API void orc_composite_loss(const CompositeCfg* cfg, uint32_t n_rays, uint32_t* numsteps, const float* net_out, const float* coords,
                                const float* rgb_target, uint32_t max_compacted, float* dloss, float* coords_out, float* loss,
                                uint32_t* counter, float* rgb_ray_out /* optional [n_rays][3] */) {
	const CompositeCfg c = *cfg;
	const float EPSILON = 1e-4f;
	std::vector<uint32_t> kept(n_rays);
	std::vector<float> rgb_ray_all((size_t)n_rays * 3);
	// first pass (:1562-1617): composite until the transmittance drops below 1e-4
	#pragma omp parallel for schedule(dynamic, 16)
	for (uint32_t i = 0; i < n_rays; ++i) {
		const uint32_t n = numsteps[2 * i], base = numsteps[2 * i + 1];
		float T = 1.f, rgb_ray[3] = {0, 0, 0}, dir[3] = {0, 0, 0};
		uint32_t j = 0;
		for (; j < n; ++j) {
			if (T < EPSILON) break;
			const float* o = net_out + (size_t)(base + j) * 16;
			if (j == 0) {  // BENT_DIR: direction carried by the first sample's output rows 8..10 (:1574-1579)
				float d[3] = {o[8] * 2.f - 1.f, o[9] * 2.f - 1.f, o[10] * 2.f - 1.f};
				const float len = sqrtf(d[0] * d[0] + d[1] * d[1] + d[2] * d[2]);
				for (int k = 0; k < 3; ++k) dir[k] = d[k] / len;
			}
			const SampleAlpha s = sample_alpha(o, coords[(size_t)(base + j) * 7 + 3], dir, c);
			const float w = s.alpha * T;
			for (int k = 0; k < 3; ++k) rgb_ray[k] += w * s.rgb[k];
			T *= (1.f - s.alpha);
		}
		if (j == n) for (int k = 0; k < 3; ++k) rgb_ray[k] += T * c.background[k];  // (:1664-1667)
		kept[i] = j;
		for (int k = 0; k < 3; ++k) rgb_ray_all[(size_t)i * 3 + k] = rgb_ray[k];
		if (rgb_ray_out) for (int k = 0; k < 3; ++k) rgb_ray_out[(size_t)i * 3 + k] = rgb_ray[k];
	}
	// compaction ranges in ray order (:1673-1679)
	std::vector<uint32_t> cbase(n_rays);
	uint64_t run = 0;
	for (uint32_t i = 0; i < n_rays; ++i) {
		cbase[i] = (uint32_t)std::min<uint64_t>(run, 0xFFFFFFFFull);
		run += kept[i];
	}
	*counter = (uint32_t)std::min<uint64_t>(run, 0xFFFFFFFFull);
	// second pass (:1767-1952)
	#pragma omp parallel for schedule(dynamic, 16)
	for (uint32_t i = 0; i < n_rays; ++i) {
		const uint32_t base = numsteps[2 * i + 1];
		const uint32_t cb = cbase[i];
		const uint32_t m = std::min(max_compacted - std::min(max_compacted, cb), kept[i]);
		numsteps[2 * i] = m;
		numsteps[2 * i + 1] = cb;
		const float* rgb_ray = &rgb_ray_all[(size_t)i * 3];
		// Huber(0.1)/5 per channel (:301-317, 1459)
		float grad[3], lsum = 0.f;
		for (int k = 0; k < 3; ++k) {
			const float d = rgb_ray[k] - rgb_target[(size_t)i * 3 + k], ad = fabsf(d), al = 0.1f;
			lsum += (ad > al ? ad - 0.5f * al : 0.5f / al * d * d) / 5.f;
			grad[k] = (ad > al ? (d > 0 ? 1.f : -1.f) : d / al) / 5.f;
		}
		if (loss) loss[i] = m == 0 ? 0.f : lsum / 3.f / (float)c.n_rays_norm;
		if (m == 0) continue;
		const float loss_scale = c.loss_scale / (float)c.n_rays_norm;
		float T = 1.f, rgb_ray2[3] = {0, 0, 0}, dir[3] = {0, 0, 0};
		for (uint32_t j = 0; j < m; ++j) {
			const float* o = net_out + (size_t)(base + j) * 16;
			if (j == 0) {
				float d[3] = {o[8] * 2.f - 1.f, o[9] * 2.f - 1.f, o[10] * 2.f - 1.f};
				const float len = sqrtf(d[0] * d[0] + d[1] * d[1] + d[2] * d[2]);
				for (int k = 0; k < 3; ++k) dir[k] = d[k] / len;
			}
			for (int k = 0; k < 7; ++k) coords_out[(size_t)(cb + j) * 7 + k] = coords[(size_t)(base + j) * 7 + k];
			const SampleAlpha s = sample_alpha(o, coords[(size_t)(base + j) * 7 + 3], dir, c);
			const float w = s.alpha * T;
			for (int k = 0; k < 3; ++k) rgb_ray2[k] += w * s.rgb[k];
			T *= (1.f - s.alpha);
			float dot = 0.f;
			for (int k = 0; k < 3; ++k) dot += grad[k] * (T * s.rgb[k] - (rgb_ray[k] - rgb_ray2[k]));
			const float dloss_dalpha = dot / (1.f - s.alpha + 1e-5f);  // mask term is zero at mask_loss_weight = 0
			float da_dE = 0, dE_dsdf = 0, dE_dinvs = 0, da_dP = 0, dP_dinvs = 0, dP_dcos = 0, dE_dcos = 0;
			if (!(s.p_div_c <= 0.f || s.p_div_c >= 1.f)) {  // (:1843-1873)
				const float P = expf(s.inv_s * s.iter_cos * s.dt);
				const float E = expf(-s.next_sdf * s.inv_s);
				const float a = 1.f + E, b = 1.f + P * E, cc = 1e-5f + 1.f / (1.f + P * E);
				const float delta = a * (b * b) * (cc * cc);
				da_dE = -(P / delta - 1.f / (a * a * cc));
				da_dP = -E / delta;
				dE_dsdf = -s.inv_s * E;
				dE_dinvs = -s.next_sdf * E;
				dP_dinvs = P * s.iter_cos * s.dt;
				dP_dcos = P * s.inv_s * s.dt;
				dE_dcos = -s.inv_s * E * s.dt * 0.5f;
			}
			const float dloss_dinvs = dloss_dalpha * (da_dE * dE_dinvs + da_dP * dP_dinvs);
			const float dloss_dvariance = dloss_dinvs * s.inv_s * 10.f;
			const float dcos_dtrue = s.true_cos >= 0.f ? 0.f : 1.f;  // the anneal ratio is ignored here (:1881-1887)
			const float gnorm = sqrtf(s.n[0] * s.n[0] + s.n[1] * s.n[1] + s.n[2] * s.n[2] + 1e-6f);
			const float ek = 1.f - 1.f / gnorm;
			const float dloss_dnormal = dloss_dalpha * (da_dE * dE_dcos + dP_dcos * da_dP) * dcos_dtrue;
			const float dloss_dsdf = dloss_dalpha * da_dE * dE_dsdf;
			float* g = dloss + (size_t)(cb + j) * 16;
			for (int k = 0; k < 3; ++k) {
				const float sg = logistic(o[k]);
				g[k] = loss_scale * (w * grad[k] * sg * (1.f - sg));
			}
			g[3] = loss_scale * dloss_dsdf;
			for (int k = 0; k < 3; ++k) g[4 + k] = c.ek_loss_weight * 2.f * c.loss_scale * ek * s.n[k];
			g[7] = loss_scale * dloss_dvariance;
			for (int k = 0; k < 3; ++k) g[8 + k] = loss_scale * dloss_dnormal * dir[k];
			for (int k = 11; k < 16; ++k) g[k] = 0.f;
		}
	}
}

// fill_rollover / fill_rollover_and_rescale (tcnn; call sites src/testbed_nerf.cu:3908-3916): pad a
// compacted batch of n_in rows (stride floats each) to n_total rows by wrapping around; the
// wrapped copies are scaled by n_in/n_total when rescale != 0.
// THE factor of fill_rollover_and_rescale: rows over rows, whatever the stride (recalled from tiny-cuda-nn, whose source
// is not in the reference tree: parity unpinned; the library's only copy is rollover_rescaled in composite.hip).
static inline float orc_rollover_rescaled(float value, uint32_t n_in, uint32_t n_total, uint32_t stride) {
	(void)stride;
	return value * (float)n_in / (float)n_total;
}
ORC_API void orc_fill_rollover(uint32_t n_total, uint32_t stride, uint32_t n_in, float* inout, int rescale) {
	if (n_in == 0 || n_in >= n_total) return;
	const size_t lim = (size_t)n_in * stride;
	for (size_t i = lim; i < (size_t)n_total * stride; ++i) {
		float r = inout[i % lim];
		if (rescale) r = orc_rollover_rescaled(r, n_in, n_total, stride);
		inout[i] = r;
	}
}

// ---------------------------------------------------------------------------
// Training-sample generator: pick a pixel per ray, march the ray through the
// 128^3 morton-ordered occupancy bitfield with the fixed step sqrt(3)/1024 and
// emit one NerfCoordinate per occupied step:
// generate_training_samples_nerf_with_global_movement, src/testbed_nerf.cu:1253-1446,
// with its helpers (:139-154, 346-368, 484-510, 614-628) and BoundingBox::ray_intersect /
// contains (bounding_box.cuh:163-221); static path (no global movement, no
// distortion, no extra dims, no error-map CDFs, cone_angle_constant = 0 as load_nerf
// sets it for aabb_scale <= 1, src/testbed_nerf.cu:3084; unit aabb).
//
// Two deliberate differences, both inside what the reference leaves open:
//  * the random numbers come from a counter-based hash instead of tcnn's pcg32
//    (absent source); draw k of ray i is hash(seed, 8*i + k);
//  * sample ranges and compact ray slots are handed out in ray order instead of
//    by atomicAdd (the reference's order is a race).
// Every floating-point step is written so that a GPU and a CPU evaluate it
// identically (explicit fmaf, no contraction): sample positions are bit-exact.
// ---------------------------------------------------------------------------
struct Camera {
	float xform[12];  // row-major 3x4 camera-to-world: [R | o]
	float focal[2], principal[2];
	uint32_t res[2];
	uint32_t pixel_offset_lo, pixel_offset_hi;  // first pixel of this image in the RGBA array
};

static inline uint32_t hash_u32(uint32_t seed, uint32_t ctr) {
	// pcg-style output permutation of a Weyl-mixed counter
	uint32_t x = ctr * 747796405u + seed * 2891336453u + 1u;
	x = ((x >> ((x >> 28) + 4u)) ^ x) * 277803737u;
	x = (x >> 22) ^ x;
	x ^= x >> 16; x *= 0x7feb352du; x ^= x >> 15; x *= 0x846ca68bu; x ^= x >> 16;
	return x;
}
static inline float rand01(uint32_t seed, uint32_t ray, uint32_t k) { return (float)(hash_u32(seed, ray * 8u + k) >> 8) * (1.0f / 16777216.0f); }

static inline uint32_t expand_bits(uint32_t v) {
	v = (v * 0x00010001u) & 0xFF0000FFu;
	v = (v * 0x00000101u) & 0x0F00F00Fu;
	v = (v * 0x00000011u) & 0xC30C30C3u;
	v = (v * 0x00000005u) & 0x49249249u;
	return v;
}
ORC_API uint32_t orc_morton3d(uint32_t x, uint32_t y, uint32_t z) { return expand_bits(x) | (expand_bits(y) << 1) | (expand_bits(z) << 2); }
ORC_API void orc_morton3d_invert(uint32_t m, uint32_t* xyz) {
	for (int d = 0; d < 3; ++d) {
		uint32_t x = (m >> d) & 0x49249249u;
		x = (x | (x >> 2)) & 0xc30c30c3u;
		x = (x | (x >> 4)) & 0x0f00f00fu;
		x = (x | (x >> 8)) & 0xff0000ffu;
		x = (x | (x >> 16)) & 0x0000ffffu;
		xyz[d] = x;
	}
}

static const float STEP = 1.73205080757f / 1024.f;  // STEPSIZE()
static const uint32_t GRIDSIZE = 128, MARCH_STEPS = 1024;

static inline bool occupied(const uint8_t* bitfield, const float* pos) {
	// cascaded_grid_idx_at(pos, mip = 0) + density_grid_occupied_at (:484-510)
	int c[3];
	for (int d = 0; d < 3; ++d) {
		float p = pos[d] - 0.5f;
		p = p * 1.0f;
		p = p + 0.5f;
		int i = (int)(p * (float)GRIDSIZE);
		c[d] = std::min(std::max(i, 0), (int)GRIDSIZE - 1);
	}
	const uint32_t idx = orc_morton3d((uint32_t)c[0], (uint32_t)c[1], (uint32_t)c[2]);
	return (bitfield[idx / 8] >> (idx % 8)) & 1;
}

static inline float to_next_voxel(const float* pos, const float* dir, const float* idir) {
	// distance_to_next_voxel at res = 128 (:346-354)
	float t = 3.4e38f;
	for (int d = 0; d < 3; ++d) {
		const float p = (float)GRIDSIZE * pos[d];
		const float sgn = copysignf(1.0f, dir[d]);
		const float td = (floorf(p + 0.5f + 0.5f * sgn) - p) * idir[d];
		t = std::min(t, td);
	}
	return std::max(t / (float)GRIDSIZE, 0.0f);
}

struct RaySetup {
	bool alive;
	float o[3], dir[3], idir[3], startt;
	float target[3];
};

static RaySetup setup_ray(uint32_t i, uint32_t n_rays, uint32_t n_rays_total, uint32_t seed, const Camera* cams, uint32_t n_images,
                          const float* rgba, const float* background) {
	RaySetup r{};
	const uint32_t img = (((i + n_rays_total) * n_images) / n_rays) % n_images;  // image_idx (:1243-1250)
	const Camera& c = cams[img];
	// nerf_random_image_pos_training with snap_to_pixel_centers (:1216-1228)
	const float u0 = rand01(seed, i, 0), u1 = rand01(seed, i, 1);
	const int px = std::min(std::max((int)(u0 * (float)c.res[0]), 0), (int)c.res[0] - 1);
	const int py = std::min(std::max((int)(u1 * (float)c.res[1]), 0), (int)c.res[1] - 1);
	const float x = ((float)px + 0.5f) / (float)c.res[0], y = ((float)py + 0.5f) / (float)c.res[1];
	const uint64_t off = ((uint64_t)c.pixel_offset_hi << 32) | c.pixel_offset_lo;
	const float* pix = rgba + (off + (uint64_t)px + (uint64_t)py * c.res[0]) * 4;
	// masked-away pixels are mostly skipped (:1300-1302)
	if (pix[0] <= 0.0f && rand01(seed, i, 2) >= 0.9f) { r.alive = false; return r; }
	for (int k = 0; k < 3; ++k) r.target[k] = pix[k] + (1.0f - pix[3]) * background[k];
	const float d[3] = {(x - c.principal[0]) * (float)c.res[0] / c.focal[0], (y - c.principal[1]) * (float)c.res[1] / c.focal[1], 1.0f};
	float w[3];
	for (int k = 0; k < 3; ++k) {
		w[k] = fmaf(c.xform[k * 4 + 2], d[2], fmaf(c.xform[k * 4 + 1], d[1], c.xform[k * 4 + 0] * d[0]));
		r.o[k] = c.xform[k * 4 + 3];
	}
	const float len = sqrtf(fmaf(w[2], w[2], fmaf(w[1], w[1], w[0] * w[0])));
	for (int k = 0; k < 3; ++k) { r.dir[k] = w[k] / len; r.idir[k] = 1.0f / r.dir[k]; }
	// BoundingBox::ray_intersect against the unit cube (bounding_box.cuh:163-210)
	float tmin = (0.f - r.o[0]) / r.dir[0], tmax = (1.f - r.o[0]) / r.dir[0];
	if (tmin > tmax) std::swap(tmin, tmax);
	bool hit = true;
	for (int k = 1; k < 3 && hit; ++k) {
		float a = (0.f - r.o[k]) / r.dir[k], b = (1.f - r.o[k]) / r.dir[k];
		if (a > b) std::swap(a, b);
		if (tmin > b || a > tmax) { hit = false; break; }
		if (a > tmin) tmin = a;
		if (b < tmax) tmax = b;
	}
	if (!hit) tmin = 3.402823466e38f;
	tmin = std::max(tmin, 0.0f);
	r.startt = fmaf(STEP, rand01(seed, i, 3), tmin);
	r.alive = true;
	return r;
}

// March; when coords != null emits up to max_emit coordinates.  Returns the number of occupied steps.
static uint32_t march(const RaySetup& r, const uint8_t* bitfield, float* coords, uint32_t max_emit) {
	uint32_t j = 0;
	float t = r.startt;
	const uint32_t limit = coords ? max_emit : MARCH_STEPS;
	while (j < limit) {
		float pos[3];
		for (int k = 0; k < 3; ++k) pos[k] = fmaf(t, r.dir[k], r.o[k]);
		if (!(pos[0] >= 0.f && pos[0] <= 1.f && pos[1] >= 0.f && pos[1] <= 1.f && pos[2] >= 0.f && pos[2] <= 1.f)) break;
		if (occupied(bitfield, pos)) {
			if (coords) {
				float* c = coords + (size_t)j * 7;
				c[0] = pos[0]; c[1] = pos[1]; c[2] = pos[2];
				c[3] = 0.0f;  // warp_dt(MIN_CONE_STEPSIZE) = 0
				for (int k = 0; k < 3; ++k) c[4 + k] = (r.dir[k] + 1.0f) * 0.5f;  // warp_direction
			}
			++j;
			t += STEP;
		} else {
			const float t_target = t + to_next_voxel(pos, r.dir, r.idir);
			do { t += STEP; } while (t < t_target);
		}
	}
	return j;
}

//  cams [n_images]; rgba fp32 [pixels][4]; bitfield 128^3/8 bytes (mip 0)
//  outputs: ray_counter, sample_counter, ray_indices [n_rays], numsteps [n_rays][2], rgb_target [n_rays][3],
//           coords [max_samples][7]
ORC_API void orc_generate_training_samples(uint32_t n_rays, uint32_t n_rays_total, uint32_t seed, const Camera* cams, uint32_t n_images,
                                           const float* rgba, const float* background, const uint8_t* bitfield, uint32_t max_samples,
                                           uint32_t* ray_counter, uint32_t* sample_counter, uint32_t* ray_indices, uint32_t* numsteps,
                                           float* rgb_target, float* coords) {
	std::vector<uint32_t> cnt(n_rays, 0);
	#pragma omp parallel for schedule(dynamic, 64)
	for (uint32_t i = 0; i < n_rays; ++i) {
		const RaySetup r = setup_ray(i, n_rays, n_rays_total, seed, cams, n_images, rgba, background);
		cnt[i] = r.alive ? march(r, bitfield, nullptr, 0) : 0;
	}
	std::vector<uint32_t> base(n_rays), slot(n_rays, 0xFFFFFFFFu);
	uint64_t run = 0;
	uint32_t rays = 0;
	for (uint32_t i = 0; i < n_rays; ++i) {
		if (cnt[i] == 0) continue;  // (:1406-1408)
		base[i] = (uint32_t)std::min<uint64_t>(run, 0xFFFFFFFFull);
		run += cnt[i];
		if ((uint64_t)base[i] + cnt[i] > max_samples) continue;  // (:1411-1414)
		slot[i] = rays++;
	}
	*ray_counter = rays;
	*sample_counter = (uint32_t)std::min<uint64_t>(run, 0xFFFFFFFFull);
	#pragma omp parallel for schedule(dynamic, 64)
	for (uint32_t i = 0; i < n_rays; ++i) {
		if (slot[i] == 0xFFFFFFFFu) continue;
		const RaySetup r = setup_ray(i, n_rays, n_rays_total, seed, cams, n_images, rgba, background);
		const uint32_t s = slot[i];
		ray_indices[s] = i;
		numsteps[2 * s] = cnt[i];
		numsteps[2 * s + 1] = base[i];
		for (int k = 0; k < 3; ++k) rgb_target[(size_t)s * 3 + k] = r.target[k];
		march(r, bitfield, coords + (size_t)base[i] * 7, cnt[i]);
	}
}

// ---------------------------------------------------------------------------
// Occupancy-grid update: update_density_grid_nerf and
// update_density_grid_mean_and_bitfield, src/testbed_nerf.cu:3286-3391, with
// their kernels (:630-660 sample generation, :662-680 max splat, :698-727 decay
// + max, :738-764 threshold to bits, :766-786 mip pooling).  The density itself
// comes from the field (NerfNetwork::density), evaluated by the caller.
//
// Random numbers: the reference passes a tcnn::pcg32 by value, skips it ahead
// by 4*i and draws four floats.  The class lives in the absent submodule; what
// is restated here is the published PCG32 (XSH-RR 64/32, M. O'Neill) in the
// form of W. Jakob's pcg32.h that tiny-cuda-nn ships: seeding, next_uint,
// next_float = bits((u >> 9) | 0x3f800000) - 1, and the O(log n) skip-ahead.
// Pinned by the generator's published first outputs for seed (42, 54) and by
// advance(n) == n draws; agreement with the fork itself is unpinned.
// ---------------------------------------------------------------------------
struct Pcg32 {
	uint64_t state, inc;
};
static const uint64_t PCG32_MULT = 0x5851f42d4c957f2dULL;

static inline uint32_t pcg32_next_uint(Pcg32& r) {
	const uint64_t old = r.state;
	r.state = old * PCG32_MULT + r.inc;
	const uint32_t xorshifted = (uint32_t)(((old >> 18u) ^ old) >> 27u);
	const uint32_t rot = (uint32_t)(old >> 59u);
	return (xorshifted >> rot) | (xorshifted << ((~rot + 1u) & 31));
}
static inline Pcg32 pcg32_seed(uint64_t initstate, uint64_t initseq) {
	Pcg32 r;
	r.state = 0u;
	r.inc = (initseq << 1u) | 1u;
	pcg32_next_uint(r);
	r.state += initstate;
	pcg32_next_uint(r);
	return r;
}
static inline float pcg32_next_float(Pcg32& r) {
	const uint32_t u = (pcg32_next_uint(r) >> 9) | 0x3f800000u;
	float f;
	memcpy(&f, &u, 4);
	return f - 1.0f;
}
static inline void pcg32_advance(Pcg32& r, uint64_t delta) {
	uint64_t cur_mult = PCG32_MULT, cur_plus = r.inc, acc_mult = 1u, acc_plus = 0u;
	while (delta > 0) {
		if (delta & 1) {
			acc_mult *= cur_mult;
			acc_plus = acc_plus * cur_mult + cur_plus;
		}
		cur_plus = (cur_mult + 1) * cur_plus;
		cur_mult *= cur_mult;
		delta /= 2;
	}
	r.state = acc_mult * r.state + acc_plus;
}

ORC_API void orc_pcg32_seed(uint64_t initstate, uint64_t initseq, uint64_t* state_inc) {
	const Pcg32 r = pcg32_seed(initstate, initseq);
	state_inc[0] = r.state; state_inc[1] = r.inc;
}
// draws n values after skipping `skip` draws; updates state_inc to the generator's state afterwards
ORC_API void orc_pcg32_draw(uint64_t* state_inc, uint64_t skip, uint32_t n, uint32_t* out_uint, float* out_float) {
	Pcg32 r{state_inc[0], state_inc[1]};
	pcg32_advance(r, skip);
	for (uint32_t i = 0; i < n; ++i) {
		if (out_float) out_float[i] = pcg32_next_float(r);
		else out_uint[i] = pcg32_next_uint(r);
	}
	state_inc[0] = r.state;
}
ORC_API void orc_pcg32_advance(uint64_t* state_inc, uint64_t delta) {
	Pcg32 r{state_inc[0], state_inc[1]};
	pcg32_advance(r, delta);
	state_inc[0] = r.state;
}

static const uint32_t GRID_CELLS = GRIDSIZE * GRIDSIZE * GRIDSIZE;

// generate_grid_samples_nerf_nonuniform (:630-660) for the unit aabb (warp_position is the identity).
//  rng      generator state {state, inc}, taken by value as in the reference
//  grid_in  n_cascades * 128^3 running densities; out: positions [n][3], indices [n]
ORC_API void orc_generate_grid_samples(uint32_t n_elements, const uint64_t* rng, uint32_t step, const float* grid_in, uint32_t n_cascades,
                                       float thresh, float* positions, uint32_t* indices) {
	#pragma omp parallel for schedule(static)
	for (uint32_t i = 0; i < n_elements; ++i) {
		Pcg32 r{rng[0], rng[1]};
		pcg32_advance(r, (uint64_t)i * 4);
		const uint32_t level = (uint32_t)(pcg32_next_float(r) * n_cascades) % n_cascades;
		uint32_t idx = 0;
		for (uint32_t j = 0; j < 10; ++j) {
			idx = ((i + step * n_elements) * 56924617u + j * 19349663u + 96925573u) % GRID_CELLS;
			idx += level * GRID_CELLS;
			if (grid_in[idx] > thresh) break;
		}
		const uint32_t pos_idx = idx % GRID_CELLS;
		uint32_t c[3];
		orc_morton3d_invert(pos_idx, c);
		const float scale = scalbnf(1.0f, (int)level);
		for (int d = 0; d < 3; ++d) {
			const float u = pcg32_next_float(r);
			positions[(size_t)i * 3 + d] = (((float)c[d] + u) / (float)GRIDSIZE - 0.5f) * scale + 0.5f;
		}
		indices[i] = idx;
	}
}

// splat_grid_samples_nerf_max_nearest_neighbor (:662-680): maximum through the unsigned bit pattern
ORC_API void orc_splat_grid_max(uint32_t n_elements, const uint32_t* indices, const float* density, float* grid_tmp) {
	for (uint32_t i = 0; i < n_elements; ++i) {
		uint32_t a, b;
		memcpy(&a, &grid_tmp[indices[i]], 4);
		memcpy(&b, &density[i], 4);
		if (b > a) memcpy(&grid_tmp[indices[i]], &b, 4);
	}
}

// ema_grid_samples_nerf (:698-727): decayed maximum; negative cells stay untouched
ORC_API void orc_ema_grid(uint32_t n_elements, float decay, float* grid, const float* grid_tmp) {
	for (uint32_t i = 0; i < n_elements; ++i) {
		const float prev = grid[i];
		grid[i] = (prev < 0.f) ? prev : fmaxf(prev * decay, grid_tmp[i]);
	}
}

// mean of max(v, 0) over the first cascade (:3383), accumulated in double
ORC_API float orc_grid_mean(const float* grid) {
	double s = 0.0;
	for (uint32_t i = 0; i < GRID_CELLS; ++i) s += (double)fmaxf(grid[i], 0.f);
	return (float)(s / GRID_CELLS);
}

// grid_to_bitfield (:738-764) over all 8 cascades and bitfield_max_pool (:766-786) for levels 1..7.
//  bitfield  8 * 128^3 / 8 bytes, level m at byte m * 128^3 / 8
ORC_API void orc_grid_to_bitfield(const float* grid, uint32_t n_cascades, float mean, float min_optical_thickness, uint8_t* bitfield) {
	const uint32_t level_bytes = GRID_CELLS / 8, n_levels = 8;
	const float thresh = std::min(min_optical_thickness, mean);
	for (uint32_t i = 0; i < level_bytes * n_levels; ++i) {
		uint8_t bits = 0;
		if (i < level_bytes * n_cascades)
			for (uint32_t j = 0; j < 8; ++j) bits |= grid[(size_t)i * 8 + j] > thresh ? (uint8_t)(1u << j) : 0;
		bitfield[i] = bits;
	}
	for (uint32_t level = 1; level < n_levels; ++level) {
		const uint8_t* prev = bitfield + (size_t)(level - 1) * level_bytes;
		uint8_t* next = bitfield + (size_t)level * level_bytes;
		for (uint32_t i = 0; i < GRID_CELLS / 64; ++i) {
			uint8_t bits = 0;
			for (uint32_t j = 0; j < 8; ++j) bits |= prev[i * 8 + j] > 0 ? (uint8_t)(1u << j) : 0;
			uint32_t c[3];
			orc_morton3d_invert(i, c);
			next[orc_morton3d(c[0] + GRIDSIZE / 8, c[1] + GRIDSIZE / 8, c[2] + GRIDSIZE / 8)] |= bits;
		}
	}
}

// ---------------------------------------------------------------------------
// Optimizer wrappers of configs/nerf/base.json:5-13 around Adam, as tiny-cuda-nn publishes them (the fork's
// copies are absent: parity with it unpinned).
//  Ema: after the nested step number t (1-based), per weight
//     tmp = (tmp * decay * (1 - decay^(t-1)) + w16 * (1 - decay)) / (1 - decay^t),  ema16 = half(tmp)
//  i.e. the bias-corrected exponential moving average of the fp16 working weights; it becomes the inference copy.
//  ExponentialDecay: after nested step t, if t >= decay_start and (t - decay_start) % decay_interval == 0 the
//  nested learning rate is multiplied by decay_base.
// ---------------------------------------------------------------------------
ORC_API void orc_ema_step(uint32_t n, float decay, uint32_t step, const float* weights16, float* tmp, float* ema16) {
	const float debias_old = 1.f - (float)std::pow((double)decay, (double)(step - 1));
	const float debias_new = 1.f - (float)std::pow((double)decay, (double)step);
	for (uint32_t i = 0; i < n; ++i) {
		const float v = (tmp[i] * decay * debias_old + weights16[i] * (1.f - decay)) / debias_new;
		tmp[i] = v;
		ema16[i] = round_fp16(v);
	}
}
ORC_API float orc_exponential_decay_lr(float base_lr, uint32_t decay_start, uint32_t decay_interval, float decay_base, uint32_t steps_done) {
	float lr = base_lr;
	for (uint32_t t = 1; t <= steps_done; ++t)
		if (t >= decay_start && (t - decay_start) % decay_interval == 0) lr *= decay_base;
	return lr;
}
