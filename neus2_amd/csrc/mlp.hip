// Fully fused 64-wide MLP for gfx950 (forward, backward, second-order
// backward_backward_input) behind the n2_mlp_* C ABI.
//
// Shape of the problem: 48->64->16 (SDF net) and 48->64->64->16 (colour net) at
// 2^18 samples are ~8-47 kflop per sample against 128+ bytes per sample of
// activations: far from the MFMA peak, so what matters is bytes, instruction
// count and occupancy.  A wave keeps a sample tile entirely in registers from
// the first layer to the last (MFMA accumulators are re-packed in place into
// the next layer's B operand), hidden activations are never written to memory
// and the backward passes recompute them from the input.  Weights live in LDS
// as ready-made MFMA operands (not in registers).  The passes that produce
// weight gradients (backward, backward + second order) are in mlp_wgrad.h:
// their batch-reduction products read row-lane operands from an LDS staging
// buffer.  The stand-alone second-order kernel here (mlp_bbi_kernel) still
// takes them from a second set of MFMAs with swapped arguments (hidden_N).
//
// MFMA tiling (v_mfma_f32_32x32x16_f16, wave64):
//   A (32 x 16, weights)      lane l holds A[l%32][8*(l/32) + 0..7]
//   B (16 x 32, activations)  lane l holds B[8*(l/32) + 0..7][l%32]
//   D (32 x 32, fp32)         lane l holds D[8*(r/4) + 4*(l/32) + r%4][l%32], r = 0..15
// A wave owns 64 consecutive samples as two 32-column tiles: tile t holds the
// samples b0 + 2*n + t, so one 4-byte load or store moves a sample pair.
// Chaining: registers r = 8*h .. 8*h+7 of a D tile are exactly one B operand for
// the K-chunk "neurons {16c+4g+0..3, 16c+8+4g+0..3}"; the weight fragments of
// the next layer are loaded with the same permutation of K.
#include "n2_common.h"

#include <new>

#include "mlp_device.h"
#include "mlp_wgrad.h"
#include "slab_reduce.h"

struct n2_mlp {
	uint32_t in_w, n_hidden, n_params;
	const hf* params;
	hf* grads;
	float* workspace;
	uint64_t workspace_bytes;
	// deferred reduction: gradient-producing calls append their slabs and one later launch sums them all
	bool deferred;
	uint32_t pending_slabs;       // slabs written since the last reduction
	n2_grad_mode pending_mode;    // mode of the first of the pending calls (later ones must accumulate)
	int dy_exponent;              // n2_mlp_set_output_gradient_exponent
	const hf* frag_image;         // n2_mlp_borrow_fragment_image (null: every workgroup builds its fragments from the weights)
};

// ----------------------------------------------------------------------------
// forward kernel
// ----------------------------------------------------------------------------
template <int IC, int NH, bool WANT_HIDDEN>
__global__ void __launch_bounds__(MLP_BLOCK, 2) mlp_forward_kernel(const hf* __restrict__ W, const hf* __restrict__ X, uint32_t N,
                                                                   hf* __restrict__ Y, int out_aos, hf* __restrict__ hidden) {
	using M = FragMap<IC, NH>;
	extern __shared__ __align__(16) unsigned char smem[];
	hf* F = reinterpret_cast<hf*>(smem);
	build_frags<IC, NH>(F, W, M::FWD_COUNT);
	const int lane = threadIdx.x & 63, n = lane & 31, g = lane >> 5;
	const uint32_t n_tiles = (N + MLP_TILE - 1) / MLP_TILE;
	const uint32_t wave_gid = blockIdx.x * (MLP_BLOCK / 64) + (threadIdx.x >> 6), n_waves = gridDim.x * (MLP_BLOCK / 64);
	for (uint32_t tile = wave_gid; tile < n_tiles; tile += n_waves) {
		const uint32_t col_raw = tile * MLP_TILE + 2 * n;
		const bool valid = col_raw < N;
		const uint32_t col = valid ? col_raw : N - 2;
		const uint32_t off4 = 4u * g * N + col;
		half8 xp[2][IC];
		load_input<IC>(X, N, col, g, xp);
		half4 keep[2];  // tile 0's output rows, held until tile 1's are known (SoA stores move sample pairs)
#pragma unroll
		for (int t = 0; t < 2; ++t) {
			half8 x[IC], h[NH][4];
			split_pairs<IC>(xp, t, x);
			hidden_S<IC, NH>(F, lane, x, h);
			float16v out = zero16();
#pragma unroll
			for (int c = 0; c < 4; ++c) out = N2_MFMA(frag(F, M::WO + c, lane), h[NH - 1][c], out);
			// registers 0..3 hold rows 4g..4g+3, registers 4..7 rows 8+4g..8+4g+3
			const half4 lo = half4{(hf)out[0], (hf)out[1], (hf)out[2], (hf)out[3]}, hi = half4{(hf)out[4], (hf)out[5], (hf)out[6], (hf)out[7]};
			if (valid) {
				if (out_aos) {
					hf* y = Y + (size_t)(col + t) * MLP_OUT;
					*reinterpret_cast<half4*>(y + 4 * g) = lo;
					*reinterpret_cast<half4*>(y + 8 + 4 * g) = hi;
				} else if (t == 0) {
					keep[0] = lo; keep[1] = hi;
				} else {
#pragma unroll
					for (int e = 0; e < 4; ++e) {
						*reinterpret_cast<half2v*>(Y + (size_t)e * N + off4) = half2v{keep[0][e], lo[e]};
						*reinterpret_cast<half2v*>(Y + (size_t)(8 + e) * N + off4) = half2v{keep[1][e], hi[e]};
					}
				}
				if (WANT_HIDDEN) {
#pragma unroll
					for (int k = 0; k < NH; ++k)
#pragma unroll
						for (int c = 0; c < 4; ++c)
#pragma unroll
							for (int e = 0; e < 8; ++e) {
								const int neuron = 16 * c + 4 * g + (e & 3) + ((e >> 2) << 3);
								hidden[((size_t)k * MLP_WIDTH + neuron) * N + col + t] = h[k][c][e];
							}
				}
			}
			tile_fence();
		}
	}
}

// ----------------------------------------------------------------------------
// weight-gradient accumulators of one wave (mlp_bbi_kernel)
// ----------------------------------------------------------------------------
// A wave with role r owns the gradient rows of neuron tile r (neurons 32r .. 32r+31):
//   gW0[nt]    : dW_0  rows 32r + drow, columns 32nt + n
//   gWh[k][nt] : dW_k+1 rows 32r + drow, columns 32nt + n
//   gWo        : dW_out rows drow (< 16), columns 32r + n
template <int IC, int NH>
struct GradAcc {
	static constexpr int IN_MT = (16 * IC + 31) / 32;
	float16v gW0[IN_MT], gWh[NH > 1 ? NH - 1 : 1][2], gWo;
	__device__ __forceinline__ void clear() {
#pragma unroll
		for (int nt = 0; nt < IN_MT; ++nt) gW0[nt] = zero16();
#pragma unroll
		for (int k = 0; k < NH - 1; ++k) { gWh[k][0] = zero16(); gWh[k][1] = zero16(); }
		gWo = zero16();
	}
	// visit every accumulator element this lane holds: fn(parameter index, value)
	template <typename Fn>
	__device__ __forceinline__ void for_each(int role, int n, int g, Fn fn) {
		constexpr int IN_W = 16 * IC;
#pragma unroll
		for (int nt = 0; nt < IN_MT; ++nt)
#pragma unroll
			for (int r = 0; r < 16; ++r)
				if (32 * nt + n < IN_W) fn((32 * role + drow(r, g)) * IN_W + 32 * nt + n, gW0[nt][r]);
#pragma unroll
		for (int k = 0; k < NH - 1; ++k)
#pragma unroll
			for (int nt = 0; nt < 2; ++nt)
#pragma unroll
				for (int r = 0; r < 16; ++r) fn(MLP_WIDTH * IN_W + k * MLP_WIDTH * MLP_WIDTH + (32 * role + drow(r, g)) * MLP_WIDTH + 32 * nt + n, gWh[k][nt][r]);
#pragma unroll
		for (int r = 0; r < 16; ++r)
			if (drow(r, g) < MLP_OUT) fn(MLP_WIDTH * IN_W + (NH - 1) * MLP_WIDTH * MLP_WIDTH + drow(r, g) * MLP_WIDTH + 32 * role + n, gWo[r]);
	}
	// Sum the four waves of a workgroup (waves 0,1 and 2,3 hold the same roles) in an fp32 LDS image
	// of the parameters and write it as this workgroup's slab.  Plain LDS stores only.
	__device__ __forceinline__ void write_slab(float* Wl, float* __restrict__ slab, int n_params, int wave, int role, int n, int g) {
		__syncthreads();  // every wave is done with the fragments the image overlays
		if (wave < 2) for_each(role, n, g, [&](int i, float v) { Wl[i] = v; });
		__syncthreads();
		if (wave >= 2) for_each(role, n, g, [&](int i, float v) { Wl[i] += v; });
		__syncthreads();
		for (int i = threadIdx.x; i < n_params; i += MLP_BLOCK) slab[i] = Wl[i];
	}
};

// ----------------------------------------------------------------------------
// backward kernel WITHOUT weight gradients (input gradient, forward + input gradient): recomputes the hidden
// activations, then
//   dL_dh_last = mask * W_out^T dL_dy ; ... ; dL_dx = W_0^T dL_dh_0
// all in registers; a wave owns 64 samples as two 32-column tiles.  (The passes that also produce weight gradients are
// mlp_wgrad_kernel, mlp_wgrad.h.)
// WANT_Y: the forward output is written as well (the recomputed hidden activations are at hand): forward and input
// gradient of the SDF net in one pass over its input.
// Register cap: amdgpu_num_vgpr counts half of the unified vector registers on this part, so 120 means 240.
// ----------------------------------------------------------------------------
template <int IC, int NH, bool WANT_Y = false>
__global__ void __launch_bounds__(MLP_BLOCK, 2) __attribute__((amdgpu_num_vgpr(120))) mlp_backward_kernel(const hf* __restrict__ W, const hf* __restrict__ X, uint32_t N,
                                                                    const hf* __restrict__ dY, int dy_aos, int unit_row,
                                                                    hf* __restrict__ dX, hf* __restrict__ Y = nullptr, int y_aos = 0,
                                                                    const uint32_t* __restrict__ x_index = nullptr, uint32_t x_cols = 0) {
	using M = FragMap<IC, NH>;
	constexpr int IN_W = 16 * IC, IN_MT = M::IN_MT;
	extern __shared__ __align__(16) unsigned char smem[];
	hf* F = reinterpret_cast<hf*>(smem);
	build_frags<IC, NH>(F, W, M::SEL);
	const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, n = lane & 31, g = lane >> 5;
	const uint32_t n_tiles = (N + MLP_TILE - 1) / MLP_TILE;
	const uint32_t slot = blockIdx.x * (MLP_BLOCK / 64) + wave, n_slots = gridDim.x * (MLP_BLOCK / 64);
	for (uint32_t tile = slot; tile < n_tiles; tile += n_slots) {
		const uint32_t col_raw = tile * MLP_TILE + 2 * n;
		const bool valid = col_raw < N;
		const uint32_t col = valid ? col_raw : N - 2;
		const uint32_t off4 = 4u * g * N + col;
		half8 xp[2][IC], dyp[2];
		// x_index: sample i of the batch is column x_index[i] of X, which has x_cols columns (the other operands are indexed by i)
		if (x_index) load_input_indexed<IC>(X, x_cols, min(x_index[col], x_cols - 1u), min(x_index[col + 1], x_cols - 1u), g, xp);
		else load_input<IC>(X, N, col, g, xp);
		outgrad_frag(dY, N, col, g, (dy_aos & 1) != 0, unit_row, dy_aos >> 8, dyp[0], dyp[1]);
		if (!valid) { dyp[0] = zero8(); dyp[1] = zero8(); }
		half8 dx_keep[IN_MT][2];  // tile 0's rows until tile 1's are known (sample-pair stores)
		half4 y_keep[2];
#pragma unroll
		for (int t = 0; t < 2; ++t) {
			half8 x[IC], h[NH][4], dh[4];
			split_pairs<IC>(xp, t, x);
			const half8 dy = dyp[t];
			hidden_S<IC, NH>(F, lane, x, h);
			if (WANT_Y) {
				float16v out = zero16();
#pragma unroll
				for (int c = 0; c < 4; ++c) out = N2_MFMA(frag(F, M::WO + c, lane), h[NH - 1][c], out);
				const half4 lo = half4{(hf)out[0], (hf)out[1], (hf)out[2], (hf)out[3]}, hi = half4{(hf)out[4], (hf)out[5], (hf)out[6], (hf)out[7]};
				if (valid) {
					if (y_aos) {
						hf* y = Y + (size_t)(col + t) * MLP_OUT;
						*reinterpret_cast<half4*>(y + 4 * g) = lo;
						*reinterpret_cast<half4*>(y + 8 + 4 * g) = hi;
					} else if (t == 0) {
						y_keep[0] = lo; y_keep[1] = hi;
					} else {
#pragma unroll
						for (int e = 0; e < 4; ++e) {
							*reinterpret_cast<half2v*>(Y + (size_t)e * N + off4) = half2v{y_keep[0][e], lo[e]};
							*reinterpret_cast<half2v*>(Y + (size_t)(8 + e) * N + off4) = half2v{y_keep[1][e], hi[e]};
						}
					}
				}
			}
			// ---- output layer ----
#pragma unroll
			for (int mt = 0; mt < 2; ++mt)
				mask_pack(N2_MFMA(frag(F, M::WOT + mt, lane), dy, zero16()), h[NH - 1][2 * mt], h[NH - 1][2 * mt + 1], dh[2 * mt], dh[2 * mt + 1]);
			// ---- hidden layers, last to first ----
#pragma unroll
			for (int k = NH - 1; k >= 1; --k) {
				half8 dprev[4];
#pragma unroll
				for (int mt = 0; mt < 2; ++mt) {
					float16v a = zero16();
#pragma unroll
					for (int c = 0; c < 4; ++c) a = N2_MFMA(frag(F, M::WHT + (k - 1) * 8 + mt * 4 + c, lane), dh[c], a);
					mask_pack(a, h[k - 1][2 * mt], h[k - 1][2 * mt + 1], dprev[2 * mt], dprev[2 * mt + 1]);
				}
#pragma unroll
				for (int c = 0; c < 4; ++c) dh[c] = dprev[c];
			}
			// ---- first layer ----
#pragma unroll
			for (int mt = 0; mt < IN_MT; ++mt) {
				float16v d = zero16();
#pragma unroll
				for (int c = 0; c < 4; ++c) d = N2_MFMA(frag(F, M::W0T + mt * 4 + c, lane), dh[c], d);
				half8 lo, hi;
				plain_pack(d, lo, hi);
				if (t == 0) {
					dx_keep[mt][0] = lo; dx_keep[mt][1] = hi;
				} else if (valid) {
#pragma unroll
					for (int e = 0; e < 8; ++e) {
						// rows 32mt + drow(e, g) and 32mt + drow(8 + e, g); the 4g part is in off4
						const int r0 = 32 * mt + 8 * (e >> 2) + (e & 3), r1 = r0 + 16;
						if (r0 + 4 * g < IN_W) *reinterpret_cast<half2v*>(dX + (size_t)r0 * N + off4) = half2v{dx_keep[mt][0][e], lo[e]};
						if (r1 + 4 * g < IN_W) *reinterpret_cast<half2v*>(dX + (size_t)r1 * N + off4) = half2v{dx_keep[mt][1][e], hi[e]};
					}
				}
			}
			tile_fence();
		}
	}
}

// ----------------------------------------------------------------------------
// second-order kernel (one hidden layer):
//   m = 1[W_0 x > 0];  a = m * (W_0 v);  b = m * (W_out^T g)
//   dW_0 += b v^T;  dW_out += g a^T;  dL_ddLdy = W_out a
// Same two-role scheme as the backward kernel.
// ----------------------------------------------------------------------------
template <int IC>
__global__ void __launch_bounds__(MLP_BLOCK, 2) mlp_bbi_kernel(const hf* __restrict__ W, const hf* __restrict__ X, uint32_t N,
                                                               const hf* __restrict__ V, const hf* __restrict__ G, int unit_row,
                                                               hf* __restrict__ dLddY, float* __restrict__ partials) {
	using M = FragMap<IC, 1>;
	constexpr int IN_W = 16 * IC, IN_MT = M::IN_MT;
	constexpr int N_PARAMS = MLP_WIDTH * IN_W + MLP_OUT * MLP_WIDTH;
	extern __shared__ __align__(16) unsigned char smem[];
	hf* F = reinterpret_cast<hf*>(smem);
	build_frags<IC, 1>(F, W, M::COUNT);
	const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, n = lane & 31, g = lane >> 5;
	const int role = __builtin_amdgcn_readfirstlane(wave & 1);
	const uint32_t n_tiles = (N + MLP_TILE - 1) / MLP_TILE;
	const uint32_t slot = (blockIdx.x * (MLP_BLOCK / 64) + wave) / 2, n_slots = gridDim.x * (MLP_BLOCK / 64) / 2;
	GradAcc<IC, 1> acc;
	acc.clear();
	for (uint32_t tile = slot; tile < n_tiles; tile += n_slots) {
		const uint32_t col_raw = tile * MLP_TILE + 2 * n;
		const bool valid = col_raw < N;
		const uint32_t col = valid ? col_raw : N - 2;
		const uint32_t off4 = 4u * g * N + col;
		half8 xp[2][IC], vp[2][IC], gp[2];
		load_input<IC>(X, N, col, g, xp);
		load_input<IC>(V, N, col, g, vp);
		outgrad_frag(G, N, col, g, false, unit_row, MLP_OUT, gp[0], gp[1]);
		if (!valid) {
			gp[0] = zero8(); gp[1] = zero8();
#pragma unroll
			for (int c = 0; c < IC; ++c) { vp[0][c] = zero8(); vp[1][c] = zero8(); }
		}
		half4 keep[2];
#pragma unroll
		for (int t = 0; t < 2; ++t) {
			half8 x[IC], v[IC], h[1][4];
			split_pairs<IC>(xp, t, x);
			split_pairs<IC>(vp, t, v);
			const half8 gg = gp[t];
			if (partials) {
				half8 hN[2], aN[2], bN[2], gN[2];
				hidden_N<IC, 1>(F, lane, 0, role, x, h, hN);  // the mask of neuron tile `role`, neuron-lane form
				float16v a = zero16();
#pragma unroll
				for (int c = 0; c < IC; ++c) a = N2_MFMA(v[c], frag(F, M::W0 + role * IC + c, lane), a);
				mask_pack(a, hN[0], hN[1], aN[0], aN[1]);
				mask_pack(N2_MFMA(gg, frag(F, M::WOT + role, lane), zero16()), hN[0], hN[1], bN[0], bN[1]);
				plain_pack(N2_MFMA(gg, frag(F, M::ID, lane), zero16()), gN[0], gN[1]);
				acc.gWo = N2_MFMA(gN[0], aN[0], acc.gWo);
				acc.gWo = N2_MFMA(gN[1], aN[1], acc.gWo);
#pragma unroll
				for (int nt = 0; nt < IN_MT; ++nt) {
					half8 vN[2];
					input_N<IC, 1>(F, lane, nt, v, vN);
					acc.gW0[nt] = N2_MFMA(bN[0], vN[0], acc.gW0[nt]);
					acc.gW0[nt] = N2_MFMA(bN[1], vN[1], acc.gW0[nt]);
				}
			}
			if (dLddY && role == 0) {
				hidden_S<IC, 1>(F, lane, x, h);
				half8 a[4];
#pragma unroll
				for (int mt = 0; mt < 2; ++mt) {
					float16v d = zero16();
#pragma unroll
					for (int c = 0; c < IC; ++c) d = N2_MFMA(frag(F, M::W0 + mt * IC + c, lane), v[c], d);
					mask_pack(d, h[0][2 * mt], h[0][2 * mt + 1], a[2 * mt], a[2 * mt + 1]);
				}
				float16v out = zero16();
#pragma unroll
				for (int c = 0; c < 4; ++c) out = N2_MFMA(frag(F, M::WO + c, lane), a[c], out);
				const half4 lo = half4{(hf)out[0], (hf)out[1], (hf)out[2], (hf)out[3]}, hi = half4{(hf)out[4], (hf)out[5], (hf)out[6], (hf)out[7]};
				if (t == 0) {
					keep[0] = lo; keep[1] = hi;
				} else if (valid) {
#pragma unroll
					for (int e = 0; e < 4; ++e) {
						*reinterpret_cast<half2v*>(dLddY + (size_t)e * N + off4) = half2v{keep[0][e], lo[e]};
						*reinterpret_cast<half2v*>(dLddY + (size_t)(8 + e) * N + off4) = half2v{keep[1][e], hi[e]};
					}
				}
			}
			tile_fence();
		}
	}
	if (partials) acc.write_slab(reinterpret_cast<float*>(smem), partials + (size_t)blockIdx.x * N_PARAMS, N_PARAMS, wave, role, n, g);
}

// grads (fp16) = [grads +] sum over slabs: n2_slab_reduce_unit (slab_reduce.h), one unit per workgroup.
__global__ void __launch_bounds__(256) mlp_reduce_units_kernel(N2SlabReduce r) {
	__shared__ float fold[32][33];
	n2_slab_reduce_unit(r, blockIdx.x, fold, [](const hf*, hf) {});
}

// ----------------------------------------------------------------------------
// host side
// ----------------------------------------------------------------------------
N2_API int n2_mlp_create(uint32_t in_width, uint32_t n_hidden_layers, n2_mlp_t** out) {
	N2_REQUIRE(out != nullptr, "n2_mlp_create: out is null");
	*out = nullptr;
	if (in_width % 16 != 0 || in_width < 16 || in_width > 64) {
		n2_set_error("n2_mlp_create: in_width %u must be a multiple of 16 in [16, 64]", in_width);
		return N2_ERR_UNSUPPORTED;
	}
	if (n_hidden_layers < 1 || n_hidden_layers > 2) {
		n2_set_error("n2_mlp_create: n_hidden_layers %u not in {1, 2}", n_hidden_layers);
		return N2_ERR_UNSUPPORTED;
	}
	n2_mlp* m = new (std::nothrow) n2_mlp();
	N2_REQUIRE(m != nullptr, "n2_mlp_create: out of host memory");
	m->in_w = in_width;
	m->n_hidden = n_hidden_layers;
	m->n_params = MLP_WIDTH * in_width + (n_hidden_layers - 1) * MLP_WIDTH * MLP_WIDTH + MLP_OUT * MLP_WIDTH;
	m->params = nullptr;
	m->grads = nullptr;
	m->workspace = nullptr;
	m->workspace_bytes = 0;
	m->deferred = false;
	m->pending_slabs = 0;
	m->pending_mode = N2_GRAD_IGNORE;
	*out = m;
	return N2_OK;
}
N2_API void n2_mlp_destroy(n2_mlp_t* mlp) { delete mlp; }
const n2_half* n2_mlp_params(const n2_mlp_t* mlp) { return reinterpret_cast<const n2_half*>(mlp->params); }
uint32_t n2_mlp_hidden_layers(const n2_mlp_t* mlp) { return mlp->n_hidden; }
N2_API uint32_t n2_mlp_n_params(const n2_mlp_t* mlp) { return mlp ? mlp->n_params : 0; }
N2_API uint32_t n2_mlp_input_width(const n2_mlp_t* mlp) { return mlp ? mlp->in_w : 0; }
N2_API uint32_t n2_mlp_output_width(const n2_mlp_t* mlp) { return mlp ? MLP_OUT : 0; }
constexpr uint32_t MLP_SLAB_SETS = 2;  // a backward and a second-order pass may be pending at the same time
N2_API uint64_t n2_mlp_workspace_bytes(const n2_mlp_t* mlp) {
	return mlp ? (uint64_t)MLP_SLAB_SETS * MLP_MAX_SLABS * mlp->n_params * sizeof(float) : 0;
}

N2_API int n2_mlp_set_params(n2_mlp_t* mlp, const n2_half* d_params, n2_half* d_gradients) {
	N2_REQUIRE(mlp != nullptr, "n2_mlp_set_params: mlp is null");
	N2_REQUIRE(d_params != nullptr, "n2_mlp_set_params: d_params is null");
	N2_REQUIRE(reinterpret_cast<uintptr_t>(d_params) % 16 == 0, "n2_mlp_set_params: d_params must be 16-byte aligned");
	N2_REQUIRE(reinterpret_cast<uintptr_t>(d_gradients) % 16 == 0, "n2_mlp_set_params: d_gradients must be 16-byte aligned");
	mlp->params = reinterpret_cast<const hf*>(d_params);
	mlp->grads = reinterpret_cast<hf*>(d_gradients);
	return N2_OK;
}

N2_API int n2_mlp_set_workspace(n2_mlp_t* mlp, void* d_workspace, uint64_t n_bytes) {
	N2_REQUIRE(mlp != nullptr, "n2_mlp_set_workspace: mlp is null");
	N2_REQUIRE(d_workspace == nullptr || n_bytes >= n2_mlp_workspace_bytes(mlp), "n2_mlp_set_workspace: %llu bytes given, %llu needed",
	           (unsigned long long)n_bytes, (unsigned long long)n2_mlp_workspace_bytes(mlp));
	N2_REQUIRE(reinterpret_cast<uintptr_t>(d_workspace) % 16 == 0, "n2_mlp_set_workspace: workspace must be 16-byte aligned");
	mlp->workspace = reinterpret_cast<float*>(d_workspace);
	mlp->workspace_bytes = d_workspace ? n_bytes : 0;
	return N2_OK;
}

static int check_mlp_batch(const n2_mlp_t* mlp, const char* fn, const void* d_input, uint32_t n) {
	N2_REQUIRE(mlp != nullptr, "%s: mlp is null", fn);
	N2_REQUIRE(mlp->params != nullptr, "%s: n2_mlp_set_params has not been called", fn);
	N2_REQUIRE(n % 8 == 0, "%s: batch size %u is not a multiple of 8", fn, n);
	N2_REQUIRE(n <= (1u << 28), "%s: batch size %u exceeds 2^28 (per-lane offsets are 32-bit)", fn, n);
	N2_REQUIRE(d_input != nullptr || n == 0, "%s: d_input is null", fn);
	N2_REQUIRE(reinterpret_cast<uintptr_t>(d_input) % 16 == 0, "%s: d_input must be 16-byte aligned", fn);
	return N2_OK;
}

// workgroups of a launch: every wave (or pair of waves when two roles share a tile) takes 64-sample
// tiles in a grid-stride loop; never more than two workgroups per CU, which build the weight fragments once
static inline uint32_t stream_grid(uint32_t n, uint32_t waves_per_tile) {
	const uint32_t tiles = (n + MLP_TILE - 1) / MLP_TILE;
	const uint32_t tiles_per_block = (MLP_BLOCK / 64) / waves_per_tile;
	const uint32_t blocks = (tiles + tiles_per_block - 1) / tiles_per_block;
	return blocks < (uint32_t)MLP_MAX_SLABS ? blocks : (uint32_t)MLP_MAX_SLABS;
}
static inline size_t frag_bytes(int n_frags) { return (size_t)n_frags * 64 * 16; }
// workgroups of the weight-gradient kernels: rounds of 128 samples in a grid-stride loop, two workgroups per CU
static inline uint32_t wgrad_grid(uint32_t n) {
	const uint32_t rounds = (n + WG_SAMPLES - 1) / WG_SAMPLES;
	return rounds < (uint32_t)MLP_MAX_SLABS ? rounds : (uint32_t)MLP_MAX_SLABS;
}
uint32_t n2_mlp_wgrad_blocks(uint32_t n) { return wgrad_grid(n); }

#define MLP_DISPATCH(in_w, n_hidden, CALL)                                            \
	do {                                                                              \
		const uint32_t key_ = ((in_w) / 16) * 10 + (n_hidden);                        \
		switch (key_) {                                                               \
			case 11: { CALL(1, 1); } break;                                           \
			case 12: { CALL(1, 2); } break;                                           \
			case 21: { CALL(2, 1); } break;                                           \
			case 22: { CALL(2, 2); } break;                                           \
			case 31: { CALL(3, 1); } break;                                           \
			case 32: { CALL(3, 2); } break;                                           \
			case 41: { CALL(4, 1); } break;                                           \
			case 42: { CALL(4, 2); } break;                                           \
			default: n2_set_error("mlp: unsupported shape"); return N2_ERR_UNSUPPORTED; \
		}                                                                             \
	} while (0)

N2_API int n2_mlp_forward(n2_mlp_t* mlp, n2_stream_t stream, const n2_half* d_input, uint32_t n, n2_half* d_output,
                          n2_layout out_layout, n2_half* d_hidden) {
	if (int rc = check_mlp_batch(mlp, "n2_mlp_forward", d_input, n)) return rc;
	if (n == 0) return N2_OK;
	N2_REQUIRE(d_output != nullptr, "n2_mlp_forward: d_output is null");
	N2_REQUIRE(out_layout == N2_LAYOUT_SOA || out_layout == N2_LAYOUT_AOS, "n2_mlp_forward: bad layout %d", (int)out_layout);
	N2_REQUIRE(reinterpret_cast<uintptr_t>(d_output) % 16 == 0 && reinterpret_cast<uintptr_t>(d_hidden) % 16 == 0,
	           "n2_mlp_forward: outputs must be 16-byte aligned");
	const dim3 grid(stream_grid(n, 1)), block(MLP_BLOCK);
	N2ProfScope prof(N2_PROF_MLP_FORWARD, n2_stream(stream));
#define CALL(IC, NH)                                                                                                     \
	do {                                                                                                                 \
		if (d_hidden)                                                                                                    \
			mlp_forward_kernel<IC, NH, true><<<grid, block, frag_bytes(FragMap<IC, NH>::FWD_COUNT), n2_stream(stream)>>>(mlp->params, \
				reinterpret_cast<const hf*>(d_input), n, reinterpret_cast<hf*>(d_output), out_layout == N2_LAYOUT_AOS ? 1 : 0, reinterpret_cast<hf*>(d_hidden)); \
		else                                                                                                             \
			mlp_forward_kernel<IC, NH, false><<<grid, block, frag_bytes(FragMap<IC, NH>::FWD_COUNT), n2_stream(stream)>>>(mlp->params, \
				reinterpret_cast<const hf*>(d_input), n, reinterpret_cast<hf*>(d_output), out_layout == N2_LAYOUT_AOS ? 1 : 0, nullptr); \
	} while (0)
	MLP_DISPATCH(mlp->in_w, mlp->n_hidden, CALL);
#undef CALL
	N2_LAUNCH_CHECK();
	return N2_OK;
}

// where the next gradient-producing kernel writes its slabs
static float* next_slabs(n2_mlp_t* mlp) { return mlp->workspace + (size_t)mlp->pending_slabs * mlp->n_params; }

static void slab_set(N2SlabReduce& r, bool second, const n2_mlp_t* mlp, uint32_t n_slabs, n2_grad_mode mode) {
	const uint32_t units = (mlp->n_params + 31) / 32;
	if (!second) { r.pa = mlp->workspace; r.slabs_a = n_slabs; r.params_a = mlp->n_params; r.ga = mlp->grads; r.acc_a = mode == N2_GRAD_ACCUMULATE ? 1 : 0; r.units_a = units; }
	else { r.pb = mlp->workspace; r.slabs_b = n_slabs; r.params_b = mlp->n_params; r.gb = mlp->grads; r.acc_b = mode == N2_GRAD_ACCUMULATE ? 1 : 0; r.units_b = units; }
	r.units = r.units_a + r.units_b + (r.extra_n > 0 ? 1u : 0u);
}

int n2_slab_reduce_launch(n2_stream_t stream, const N2SlabReduce& r) {
	if (r.units == 0) return N2_OK;
	mlp_reduce_units_kernel<<<dim3(r.units), dim3(256), 0, n2_stream(stream)>>>(r);
	N2_LAUNCH_CHECK();
	return N2_OK;
}

static int reduce_now(n2_mlp_t* mlp, hipStream_t s, uint32_t n_slabs, n2_grad_mode mode) {
	N2SlabReduce r = {};
	slab_set(r, false, mlp, n_slabs, mode);
	return n2_slab_reduce_launch(reinterpret_cast<n2_stream_t>(s), r);
}

// a kernel has just written n_slabs slabs at next_slabs(mlp)
static int reduce_partials(n2_mlp_t* mlp, hipStream_t s, uint32_t n_slabs, n2_grad_mode mode) {
	if (!mlp->deferred) return reduce_now(mlp, s, n_slabs, mode);
	if (mlp->pending_slabs == 0) mlp->pending_mode = mode;
	mlp->pending_slabs += n_slabs;
	return N2_OK;
}

// a gradient-producing call may run: room for its slabs, and a mode that can be folded into what is pending
static int check_pending(n2_mlp_t* mlp, const char* fn, uint32_t n_slabs, n2_grad_mode mode) {
	if (!mlp->deferred || mode == N2_GRAD_IGNORE) return N2_OK;
	N2_REQUIRE(mlp->pending_slabs == 0 || mode == N2_GRAD_ACCUMULATE, "%s: with deferred reduction only ACCUMULATE can follow a pending gradient pass", fn);
	N2_REQUIRE(mlp->pending_slabs + n_slabs <= MLP_SLAB_SETS * (uint32_t)MLP_MAX_SLABS, "%s: too many gradient passes pending (call n2_mlp_reduce_deferred)", fn);
	return N2_OK;
}

void n2_mlp_drop_pending(n2_mlp_t* mlp) {
	if (mlp) mlp->pending_slabs = 0;
}

N2_API int n2_mlp_set_deferred_reduction(n2_mlp_t* mlp, int enable) {
	N2_REQUIRE(mlp != nullptr, "n2_mlp_set_deferred_reduction: mlp is null");
	N2_REQUIRE(mlp->pending_slabs == 0, "n2_mlp_set_deferred_reduction: gradient passes are pending");
	mlp->deferred = enable != 0;
	return N2_OK;
}

void n2_mlp_borrow_fragment_image(n2_mlp_t* mlp, const n2_half* image) { mlp->frag_image = reinterpret_cast<const hf*>(image); }
uint32_t n2_mlp_fragment_image_bytes(uint32_t in_w, uint32_t n_hidden) {
	if (in_w == 48 && n_hidden == 2) return (uint32_t)frag_bytes(FragMap<3, 2>::SEL);
	if (in_w == 48 && n_hidden == 1) return (uint32_t)frag_bytes(FragMap<3, 1>::SEL);
	return 0;
}

N2_API int n2_mlp_set_output_gradient_exponent(n2_mlp_t* mlp, int exponent) {
	N2_REQUIRE(mlp != nullptr, "n2_mlp_set_output_gradient_exponent: mlp is null");
	N2_REQUIRE(exponent >= -14 && exponent <= 14, "n2_mlp_set_output_gradient_exponent: exponent %d outside [-14, 14]", exponent);
	mlp->dy_exponent = exponent;
	return N2_OK;
}

N2_API int n2_colour_gradient_exponent(float loss_scale, uint32_t n_rays) {
	if (!(loss_scale > 0.f) || n_rays == 0) return 0;
	int k = 0;
	// largest k with loss_scale / n_rays * 2^k <= 16
	while (k < 14 && ldexpf(loss_scale / (float)n_rays, k + 1) <= 16.f) ++k;
	return k;
}

N2_API int n2_mlp_reduce_deferred(n2_mlp_t* a, n2_mlp_t* b, n2_stream_t stream) { return n2_mlp_reduce_deferred_sum(a, b, stream, nullptr, 0, nullptr, 0); }

int n2_mlp_reduce_deferred_plan(n2_mlp_t* a, n2_mlp_t* b, const float* d_parts, uint32_t n_parts, n2_half* d_sum, int accumulate, N2SlabReduce* out) {
	N2_REQUIRE(out != nullptr, "n2_mlp_reduce_deferred: plan is null");
	N2SlabReduce r = {};
	if (n_parts > 0) { r.extra = d_parts; r.extra_n = n_parts; r.extra_out = reinterpret_cast<hf*>(d_sum); r.extra_acc = accumulate; r.units = 1; }
	bool second = false;
	n2_mlp_t* nets[2] = {a, b};
	for (n2_mlp_t* m : nets) {
		if (m == nullptr || m->pending_slabs == 0) continue;
		slab_set(r, second, m, m->pending_slabs, m->pending_mode);
		m->pending_slabs = 0;
		second = true;
	}
	*out = r;
	return N2_OK;
}

int n2_mlp_reduce_deferred_sum(n2_mlp_t* a, n2_mlp_t* b, n2_stream_t stream, const float* d_parts, uint32_t n_parts, n2_half* d_sum, int accumulate) {
	N2_REQUIRE(a != nullptr, "n2_mlp_reduce_deferred: mlp is null");
	N2SlabReduce r;
	if (int rc = n2_mlp_reduce_deferred_plan(a, b, d_parts, n_parts, d_sum, accumulate, &r)) return rc;
	return n2_slab_reduce_launch(stream, r);
}

static int check_grad_mode(const n2_mlp_t* mlp, const char* fn, n2_grad_mode mode) {
	N2_REQUIRE(mode == N2_GRAD_IGNORE || mode == N2_GRAD_OVERWRITE || mode == N2_GRAD_ACCUMULATE, "%s: bad gradient mode %d", fn, (int)mode);
	if (mode != N2_GRAD_IGNORE) {
		N2_REQUIRE(mlp->grads != nullptr, "%s: gradient mode %d needs a gradient buffer (n2_mlp_set_params)", fn, (int)mode);
		N2_REQUIRE(mlp->workspace != nullptr, "%s: gradient mode %d needs a workspace (n2_mlp_set_workspace)", fn, (int)mode);
	}
	return N2_OK;
}

template <typename K>
static int allow_lds(K kernel, size_t bytes) {
	if (bytes > 48 * 1024) N2_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes));
	return N2_OK;
}

// unit_row >= 0: dL_doutput is the constant e_{unit_row} and d_dL_doutput is not read
static int mlp_backward_impl(n2_mlp_t* mlp, n2_stream_t stream, const n2_half* d_input, uint32_t n,
                             const n2_half* d_dL_doutput, n2_layout dL_layout, int unit_row, n2_half* d_dL_dinput, n2_grad_mode mode,
                             n2_half* d_output = nullptr, n2_layout out_layout = N2_LAYOUT_SOA, uint32_t dy_rows = MLP_OUT,
                             const uint32_t* x_index = nullptr, uint32_t x_cols = 0, bool dx_out_and_normal_only = false,
                             const N2FieldPrepTail* tail = nullptr) {
	if (int rc = check_mlp_batch(mlp, "n2_mlp_backward", d_input, n)) return rc;
	if (int rc = check_grad_mode(mlp, "n2_mlp_backward", mode)) return rc;
	N2_REQUIRE(dL_layout == N2_LAYOUT_SOA || dL_layout == N2_LAYOUT_AOS, "n2_mlp_backward: bad layout %d", (int)dL_layout);
	N2_REQUIRE(d_dL_doutput != nullptr || n == 0 || unit_row >= 0, "n2_mlp_backward: d_dL_doutput is null");
	N2_REQUIRE(reinterpret_cast<uintptr_t>(d_dL_doutput) % 16 == 0 && reinterpret_cast<uintptr_t>(d_dL_dinput) % 16 == 0,
	           "n2_mlp_backward: buffers must be 16-byte aligned");
	hipStream_t s = n2_stream(stream);
	const bool want_dw = mode != N2_GRAD_IGNORE, want_dx = d_dL_dinput != nullptr;
	N2_REQUIRE(!want_dw || unit_row < 0, "n2_mlp_backward: a constant output gradient goes with mode IGNORE");
	if (n == 0) {
		if (mode == N2_GRAD_OVERWRITE) return n2_fill_zero_u32(s, mlp->grads, mlp->n_params * sizeof(hf));
		return N2_OK;
	}
	if (!want_dw && !want_dx) return N2_OK;
	const uint32_t blocks = want_dw ? wgrad_grid(n) : stream_grid(n, 1);
	if (int rc = check_pending(mlp, "n2_mlp_backward", blocks, mode)) return rc;
	const hf* X = reinterpret_cast<const hf*>(d_input);
	const hf* dY = reinterpret_cast<const hf*>(d_dL_doutput);
	hf* dX = reinterpret_cast<hf*>(d_dL_dinput);
	const int aos = (dL_layout == N2_LAYOUT_AOS ? 1 : 0) | ((int)dy_rows << 8);  // layout flag and the number of rows in use
	const float dy_gain = ldexpf(1.f, mlp->dy_exponent), dy_gain_inv = ldexpf(1.f, -mlp->dy_exponent);
	N2ProfScope prof(N2_PROF_MLP_BACKWARD, s);
#define LAUNCH(IC, NH)                                                                                              \
	do {                                                                                                            \
		const size_t lds = frag_bytes(FragMap<IC, NH>::SEL);                                                        \
		if (int rc = allow_lds(mlp_backward_kernel<IC, NH>, lds)) return rc;                                        \
		mlp_backward_kernel<IC, NH><<<dim3(blocks), dim3(MLP_BLOCK), lds, s>>>(mlp->params, X, n, dY, aos, unit_row, dX, nullptr, 0, x_index, x_cols); \
	} while (0)
#define LAUNCH_W(IC, NH, DX)                                                                                        \
	do {                                                                                                            \
		const size_t lds = mlp_wgrad_lds<IC, NH, false>();                                                          \
		if (int rc = allow_lds(mlp_wgrad_kernel<IC, NH, DX, false>, lds)) return rc;                                \
		mlp_wgrad_kernel<IC, NH, DX, false><<<dim3(blocks), dim3(MLP_BLOCK), lds, s>>>(mlp->params, X, n, dY, aos & 1, (int)dy_rows, dX, \
			next_slabs(mlp), nullptr, nullptr, -1, x_index, x_cols, dy_gain, dy_gain_inv, mlp->frag_image);                            \
	} while (0)
	// the field's colour net (48 inputs, two hidden layers): only the rows the field reads are stored
	N2_REQUIRE(tail == nullptr || (want_dx && want_dw && dx_out_and_normal_only && mlp->in_w == 48 && mlp->n_hidden == 2 && (aos & 1) && dy_rows <= 8),
	           "n2_mlp_backward: the field's tail goes with the colour net's launch (48 inputs, two hidden layers, AoS output gradient)");
	if (want_dx && want_dw && dx_out_and_normal_only && mlp->in_w == 48 && mlp->n_hidden == 2) {
		if (tail) {
			WgFieldPrepTail t{*tail};
			const size_t lds = mlp_wgrad_lds<3, 2, false>();
			if (int rc = allow_lds(mlp_wgrad_kernel<3, 2, WG_DX_OUT_AND_NORMAL, false, WgFieldPrepTail>, lds)) return rc;
			mlp_wgrad_kernel<3, 2, WG_DX_OUT_AND_NORMAL, false, WgFieldPrepTail><<<dim3(blocks), dim3(MLP_BLOCK), lds, s>>>(mlp->params, X, n, dY, aos & 1,
				(int)dy_rows, dX, next_slabs(mlp), nullptr, nullptr, -1, x_index, x_cols, dy_gain, dy_gain_inv, mlp->frag_image, t);
		} else {
			LAUNCH_W(3, 2, WG_DX_OUT_AND_NORMAL);
		}
		N2_LAUNCH_CHECK();
		return reduce_partials(mlp, s, blocks, mode);
	}
#define LAUNCH_Y(IC, NH)                                                                                            \
	do {                                                                                                            \
		const size_t lds = frag_bytes(FragMap<IC, NH>::SEL);                                                        \
		if (int rc = allow_lds(mlp_backward_kernel<IC, NH, true>, lds)) return rc;                                  \
		mlp_backward_kernel<IC, NH, true><<<dim3(blocks), dim3(MLP_BLOCK), lds, s>>>(mlp->params, X, n, dY, aos, unit_row, dX, \
			reinterpret_cast<hf*>(d_output), out_layout == N2_LAYOUT_AOS ? 1 : 0);                                  \
	} while (0)
#define CALL(IC, NH)                                   \
	do {                                               \
		if (d_output) LAUNCH_Y(IC, NH);                        \
		else if (want_dx && want_dw) LAUNCH_W(IC, NH, WG_DX_ALL);   \
		else if (want_dx) LAUNCH(IC, NH);                      \
		else LAUNCH_W(IC, NH, WG_DX_NONE);                     \
	} while (0)
	MLP_DISPATCH(mlp->in_w, mlp->n_hidden, CALL);
#undef CALL
#undef LAUNCH
#undef LAUNCH_W
#undef LAUNCH_Y
	N2_LAUNCH_CHECK();
	if (want_dw) return reduce_partials(mlp, s, blocks, mode);
	return N2_OK;
}

N2_API int n2_mlp_forward_and_input_gradient(n2_mlp_t* mlp, n2_stream_t stream, uint32_t dim, const n2_half* d_input, uint32_t n,
                                             n2_half* d_output, n2_layout out_layout, n2_half* d_dinput) {
	N2_REQUIRE(dim < (uint32_t)MLP_OUT, "n2_mlp_forward_and_input_gradient: output dimension %u out of range", dim);
	N2_REQUIRE((d_output != nullptr && d_dinput != nullptr) || n == 0, "n2_mlp_forward_and_input_gradient: null output");
	N2_REQUIRE(out_layout == N2_LAYOUT_SOA || out_layout == N2_LAYOUT_AOS, "n2_mlp_forward_and_input_gradient: bad layout %d", (int)out_layout);
	N2_REQUIRE(reinterpret_cast<uintptr_t>(d_output) % 16 == 0, "n2_mlp_forward_and_input_gradient: d_output must be 16-byte aligned");
	return mlp_backward_impl(mlp, stream, d_input, n, nullptr, N2_LAYOUT_SOA, (int)dim, d_dinput, N2_GRAD_IGNORE, d_output, out_layout);
}

N2_API int n2_mlp_backward(n2_mlp_t* mlp, n2_stream_t stream, const n2_half* d_input, uint32_t n,
                           const n2_half* d_dL_doutput, n2_layout dL_layout, n2_half* d_dL_dinput, n2_grad_mode mode) {
	return mlp_backward_impl(mlp, stream, d_input, n, d_dL_doutput, dL_layout, -1, d_dL_dinput, mode);
}

N2_API int n2_mlp_backward_rows(n2_mlp_t* mlp, n2_stream_t stream, const n2_half* d_input, uint32_t n, const n2_half* d_dL_doutput,
                                n2_layout dL_layout, uint32_t n_rows, n2_half* d_dL_dinput, n2_grad_mode mode) {
	N2_REQUIRE(n_rows >= 1 && n_rows <= (uint32_t)MLP_OUT, "n2_mlp_backward_rows: n_rows %u outside [1, %d]", n_rows, MLP_OUT);
	return mlp_backward_impl(mlp, stream, d_input, n, d_dL_doutput, dL_layout, -1, d_dL_dinput, mode, nullptr, N2_LAYOUT_SOA, n_rows);
}

int n2_mlp_backward_rows_indexed(n2_mlp_t* mlp, n2_stream_t stream, const n2_half* d_input, uint32_t n_cols, const uint32_t* d_index, uint32_t n,
                                 const n2_half* d_dL_doutput, n2_layout dL_layout, uint32_t n_rows, n2_half* d_dL_dinput, n2_grad_mode mode,
                                 bool dx_out_and_normal_only, const N2FieldPrepTail* tail) {
	N2_REQUIRE(n_rows >= 1 && n_rows <= (uint32_t)MLP_OUT, "n2_mlp_backward_rows: n_rows %u outside [1, %d]", n_rows, MLP_OUT);
	N2_REQUIRE(d_index == nullptr || n_cols >= 1, "n2_mlp_backward_rows: an indexed input needs at least one column");
	return mlp_backward_impl(mlp, stream, d_input, n, d_dL_doutput, dL_layout, -1, d_dL_dinput, mode, nullptr, N2_LAYOUT_SOA, n_rows, d_index, n_cols,
	                         dx_out_and_normal_only, tail);
}

N2_API int n2_mlp_input_gradient(n2_mlp_t* mlp, n2_stream_t stream, uint32_t dim, const n2_half* d_input, uint32_t n,
                                 n2_half* d_dinput) {
	N2_REQUIRE(dim < (uint32_t)MLP_OUT, "n2_mlp_input_gradient: output dimension %u out of range", dim);
	N2_REQUIRE(d_dinput != nullptr || n == 0, "n2_mlp_input_gradient: d_dinput is null");
	return mlp_backward_impl(mlp, stream, d_input, n, nullptr, N2_LAYOUT_SOA, (int)dim, d_dinput, N2_GRAD_IGNORE);
}

N2_API int n2_mlp_backward_and_second_order(n2_mlp_t* mlp, n2_stream_t stream, const n2_half* d_input, uint32_t n,
                                            const n2_half* d_dL_doutput, n2_layout dL_layout, n2_half* d_dL_dinput,
                                            const n2_half* d_dL_ddLdinput, const n2_half* d_second_dL_doutput, n2_grad_mode mode) {
	return n2_mlp_backward_and_second_order_indexed(mlp, stream, d_input, 0, nullptr, n, d_dL_doutput, dL_layout, d_dL_dinput, d_dL_ddLdinput,
	                                                d_second_dL_doutput, mode, false);
}

int n2_mlp_backward_and_second_order_indexed(n2_mlp_t* mlp, n2_stream_t stream, const n2_half* d_input, uint32_t n_cols, const uint32_t* d_index,
                                             uint32_t n, const n2_half* d_dL_doutput, n2_layout dL_layout, n2_half* d_dL_dinput,
                                             const n2_half* d_dL_ddLdinput, const n2_half* d_second_dL_doutput, n2_grad_mode mode,
                                             bool dx_encoding_only) {
	const char* fn = "n2_mlp_backward_and_second_order";
	N2_REQUIRE(d_index == nullptr || n_cols >= 1, "%s: an indexed input needs at least one column", fn);
	if (int rc = check_mlp_batch(mlp, fn, d_input, n)) return rc;
	if (int rc = check_grad_mode(mlp, fn, mode)) return rc;
	N2_REQUIRE(mode != N2_GRAD_IGNORE, "%s: the merged pass exists for its weight gradients (mode must be OVERWRITE or ACCUMULATE)", fn);
	if (mlp->n_hidden != 1) {
		n2_set_error("%s: implemented for one hidden layer (got %u)", fn, mlp->n_hidden);
		return N2_ERR_UNSUPPORTED;
	}
	N2_REQUIRE(dL_layout == N2_LAYOUT_SOA || dL_layout == N2_LAYOUT_AOS, "%s: bad layout %d", fn, (int)dL_layout);
	N2_REQUIRE((d_dL_doutput != nullptr && d_dL_dinput != nullptr && d_dL_ddLdinput != nullptr) || n == 0,
	           "%s: d_dL_doutput, d_dL_dinput and d_dL_ddLdinput are required", fn);
	N2_REQUIRE(reinterpret_cast<uintptr_t>(d_dL_doutput) % 16 == 0 && reinterpret_cast<uintptr_t>(d_dL_dinput) % 16 == 0 &&
	           reinterpret_cast<uintptr_t>(d_dL_ddLdinput) % 16 == 0 && reinterpret_cast<uintptr_t>(d_second_dL_doutput) % 16 == 0,
	           "%s: buffers must be 16-byte aligned", fn);
	hipStream_t s = n2_stream(stream);
	if (n == 0) {
		if (mode == N2_GRAD_OVERWRITE) return n2_fill_zero_u32(s, mlp->grads, mlp->n_params * sizeof(hf));
		return N2_OK;
	}
	const uint32_t blocks = wgrad_grid(n);
	if (int rc = check_pending(mlp, fn, blocks, mode)) return rc;
	const int aos = dL_layout == N2_LAYOUT_AOS ? 1 : 0;
	const int unit_row2 = d_second_dL_doutput == nullptr ? 0 : -1;
	N2ProfScope prof(N2_PROF_MLP_BACKWARD, s);
	if (dx_encoding_only && mlp->in_w == 48) {
		// the field's SDF net: only the encoding's rows of dL/dinput are stored
		const size_t lds = mlp_wgrad_lds<3, 1, true>();
		if (int rc = allow_lds(mlp_wgrad_kernel<3, 1, WG_DX_ENCODING, true>, lds)) return rc;
		mlp_wgrad_kernel<3, 1, WG_DX_ENCODING, true><<<dim3(blocks), dim3(MLP_BLOCK), lds, s>>>(mlp->params,
			reinterpret_cast<const hf*>(d_input), n, reinterpret_cast<const hf*>(d_dL_doutput), aos, MLP_OUT,
			reinterpret_cast<hf*>(d_dL_dinput), next_slabs(mlp), reinterpret_cast<const hf*>(d_dL_ddLdinput),
			reinterpret_cast<const hf*>(d_second_dL_doutput), unit_row2, d_index, n_cols, 1.f, 1.f, mlp->frag_image);
		N2_LAUNCH_CHECK();
		return reduce_partials(mlp, s, blocks, mode);
	}
	switch (mlp->in_w / 16) {
#define CASE(IC)                                                                                                           \
	case IC: {                                                                                                             \
		const size_t lds = mlp_wgrad_lds<IC, 1, true>();                                                                   \
		if (int rc = allow_lds(mlp_wgrad_kernel<IC, 1, WG_DX_ALL, true>, lds)) return rc;                                  \
		mlp_wgrad_kernel<IC, 1, WG_DX_ALL, true><<<dim3(blocks), dim3(MLP_BLOCK), lds, s>>>(mlp->params,                   \
			reinterpret_cast<const hf*>(d_input), n, reinterpret_cast<const hf*>(d_dL_doutput), aos, MLP_OUT,              \
			reinterpret_cast<hf*>(d_dL_dinput), next_slabs(mlp), reinterpret_cast<const hf*>(d_dL_ddLdinput),              \
			reinterpret_cast<const hf*>(d_second_dL_doutput), unit_row2, d_index, n_cols, 1.f, 1.f, mlp->frag_image);                       \
		break;                                                                                                             \
	}
		CASE(1) CASE(2) CASE(3) CASE(4)
#undef CASE
		default: n2_set_error("mlp: unsupported shape"); return N2_ERR_UNSUPPORTED;
	}
	N2_LAUNCH_CHECK();
	return reduce_partials(mlp, s, blocks, mode);
}

N2_API int n2_mlp_backward_backward_input(n2_mlp_t* mlp, n2_stream_t stream, const n2_half* d_input, uint32_t n,
                                          const n2_half* d_dL_ddLdinput, const n2_half* d_dL_doutput,
                                          n2_half* d_dL_ddLdoutput, n2_grad_mode mode) {
	if (int rc = check_mlp_batch(mlp, "n2_mlp_backward_backward_input", d_input, n)) return rc;
	if (int rc = check_grad_mode(mlp, "n2_mlp_backward_backward_input", mode)) return rc;
	if (mlp->n_hidden != 1) {
		n2_set_error("n2_mlp_backward_backward_input: implemented for one hidden layer (got %u)", mlp->n_hidden);
		return N2_ERR_UNSUPPORTED;
	}
	N2_REQUIRE(d_dL_ddLdinput != nullptr || n == 0, "n2_mlp_backward_backward_input: d_dL_ddLdinput is required");
	const int unit_row = d_dL_doutput == nullptr ? 0 : -1;
	N2_REQUIRE(reinterpret_cast<uintptr_t>(d_dL_ddLdinput) % 16 == 0 && reinterpret_cast<uintptr_t>(d_dL_doutput) % 16 == 0 &&
	           reinterpret_cast<uintptr_t>(d_dL_ddLdoutput) % 16 == 0, "n2_mlp_backward_backward_input: buffers must be 16-byte aligned");
	hipStream_t s = n2_stream(stream);
	const bool want_dw = mode != N2_GRAD_IGNORE;
	if (n == 0) {
		if (mode == N2_GRAD_OVERWRITE) return n2_fill_zero_u32(s, mlp->grads, mlp->n_params * sizeof(hf));
		return N2_OK;
	}
	if (!want_dw && !d_dL_ddLdoutput) return N2_OK;
	const uint32_t blocks = stream_grid(n, 2);
	if (int rc = check_pending(mlp, "n2_mlp_backward_backward_input", blocks, mode)) return rc;
	N2ProfScope prof(N2_PROF_MLP_SECOND_ORDER, s);
	switch (mlp->in_w / 16) {
#define CASE(IC)                                                                                                           \
	case IC:                                                                                                               \
		if (int rc = allow_lds(mlp_bbi_kernel<IC>, frag_bytes(FragMap<IC, 1>::COUNT))) return rc;                          \
		mlp_bbi_kernel<IC><<<dim3(blocks), dim3(MLP_BLOCK), frag_bytes(FragMap<IC, 1>::COUNT), s>>>(mlp->params, reinterpret_cast<const hf*>(d_input), n, \
			reinterpret_cast<const hf*>(d_dL_ddLdinput), reinterpret_cast<const hf*>(d_dL_doutput), unit_row,              \
			reinterpret_cast<hf*>(d_dL_ddLdoutput), want_dw ? next_slabs(mlp) : nullptr);                                  \
		break;
		CASE(1) CASE(2) CASE(3) CASE(4)
#undef CASE
		default: n2_set_error("mlp: unsupported shape"); return N2_ERR_UNSUPPORTED;
	}
	N2_LAUNCH_CHECK();
	if (want_dw) return reduce_partials(mlp, s, blocks, mode);
	return N2_OK;
}
