// Fully fused 64-wide MLP for gfx950 (forward, backward, second-order
// backward_backward_input) behind the n2_mlp_* C ABI.
//
// Shape of the problem: 48->64->16 (SDF net) and 48->64->64->16 (colour net) at
// 2^18 samples are ~8-16 kflop per sample against 128+ bytes per sample of
// activations, so every kernel here is bound by HBM, not by MFMA.  The design
// therefore minimises bytes: a wave keeps a 64-sample tile entirely in
// registers from the first layer to the last (MFMA accumulators are re-packed
// in place into the next layer's B operand), hidden activations are never
// written to memory, and the backward passes recompute them from the input.
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

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef _Float16 half4 __attribute__((ext_vector_type(4)));
typedef _Float16 half2v __attribute__((ext_vector_type(2)));
typedef float float16v __attribute__((ext_vector_type(16)));
typedef _Float16 hf;

#define N2_MFMA(a, b, c) __builtin_amdgcn_mfma_f32_32x32x16_f16((a), (b), (c), 0, 0, 0)

constexpr int MLP_WIDTH = 64;
constexpr int MLP_OUT = 16;
constexpr int MLP_BLOCK = 256;      // 4 waves
constexpr int MLP_TILE = 64;        // samples per wave iteration
constexpr int MLP_MAX_SLABS = 256;  // workgroups of the weight-gradient kernels
constexpr int STAGE_LD = 72;        // halves per staged row: 64 samples + 8 pad (keeps 16-byte alignment)

struct n2_mlp {
	uint32_t in_w, n_hidden, n_params;
	const hf* params;
	hf* grads;
	float* workspace;
	uint64_t workspace_bytes;
};

// ----------------------------------------------------------------------------
// fragment loaders (weights live in global memory, a few KB, L1/L2 resident)
// ----------------------------------------------------------------------------
// rows of W as A operand, natural K order: K-chunk c covers inputs 16c .. 16c+15
__device__ __forceinline__ half8 wfrag_natural(const hf* W, int ld, int row, int c, int g) {
	return *reinterpret_cast<const half8*>(W + row * ld + 16 * c + 8 * g);
}
// rows of W as A operand, chained K order (input comes from a D tile)
__device__ __forceinline__ half8 wfrag_chained(const hf* W, int ld, int row, int c, int g) {
	const half4 lo = *reinterpret_cast<const half4*>(W + row * ld + 16 * c + 4 * g);
	const half4 hi = *reinterpret_cast<const half4*>(W + row * ld + 16 * c + 8 + 4 * g);
	return half8{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
}
// rows of W^T as A operand (A[m][k] = W[k][m]), natural K order over W's rows
__device__ __forceinline__ half8 wTfrag_natural(const hf* W, int ld, int m, int c, int g, int n_rows) {
	half8 f;
#pragma unroll
	for (int e = 0; e < 8; ++e) {
		const int k = 16 * c + 8 * g + e;
		f[e] = (k < n_rows) ? W[k * ld + m] : (hf)0;
	}
	return f;
}
// rows of W^T as A operand, chained K order over W's rows
__device__ __forceinline__ half8 wTfrag_chained(const hf* W, int ld, int m, int c, int g) {
	half8 f;
#pragma unroll
	for (int e = 0; e < 8; ++e) {
		const int k = 16 * c + 4 * g + (e & 3) + ((e >> 2) << 3);
		f[e] = W[k * ld + m];
	}
	return f;
}

// B operands of both sample tiles for K-chunk c from an SoA matrix (rows x N):
// rows 16c + 8g + e, sample pair at column `col` (even, already clamped).
__device__ __forceinline__ void bfrag_soa(const hf* __restrict__ M, size_t N, uint32_t col, int c, int g, int n_rows,
                                          half8& t0, half8& t1) {
#pragma unroll
	for (int e = 0; e < 8; ++e) {
		const int k = 16 * c + 8 * g + e;
		half2v v = {(hf)0, (hf)0};
		if (k < n_rows) v = *reinterpret_cast<const half2v*>(M + (size_t)k * N + col);
		t0[e] = v[0];
		t1[e] = v[1];
	}
}

// ReLU + fp16 rounding of a D tile into the two chained B operands it holds
__device__ __forceinline__ void relu_pack(const float16v& d, half8& lo, half8& hi) {
#pragma unroll
	for (int e = 0; e < 8; ++e) {
		lo[e] = (hf)fmaxf(d[e], 0.f);
		hi[e] = (hf)fmaxf(d[8 + e], 0.f);
	}
}
// masked (by the sign of a saved activation) fp16 rounding of a D tile
__device__ __forceinline__ void mask_pack(const float16v& d, const half8& act_lo, const half8& act_hi, half8& lo, half8& hi) {
#pragma unroll
	for (int e = 0; e < 8; ++e) {
		lo[e] = (act_lo[e] > (hf)0) ? (hf)d[e] : (hf)0;
		hi[e] = (act_hi[e] > (hf)0) ? (hf)d[8 + e] : (hf)0;
	}
}

__device__ __forceinline__ float16v zero16() {
	float16v z;
#pragma unroll
	for (int r = 0; r < 16; ++r) z[r] = 0.f;
	return z;
}

// row index inside a 32-row D tile held in register r by lane group g
__device__ __forceinline__ int drow(int r, int g) { return 8 * (r >> 2) + 4 * g + (r & 3); }

// Write both sample tiles of a chained operand set (4 chunks = 64 neurons) to a
// staging matrix [64][STAGE_LD] so that rows can be re-read along the batch.
__device__ __forceinline__ void stage_sync() {
	// staging buffers are private to a wave: order its LDS writes and reads
	__builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
	__builtin_amdgcn_wave_barrier();
	__builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}
__device__ __forceinline__ void stage_store(hf* S, const half8 (&f)[2][4], int n, int g) {
	stage_sync();
#pragma unroll
	for (int c = 0; c < 4; ++c) {
#pragma unroll
		for (int e = 0; e < 8; ++e) {
			const int neuron = 16 * c + 4 * g + (e & 3) + ((e >> 2) << 3);
			*reinterpret_cast<half2v*>(S + neuron * STAGE_LD + 2 * n) = half2v{f[0][c][e], f[1][c][e]};
		}
	}
}
// A operand along the batch: row `row` of a staged matrix, samples 16c + 8g + 0..7
__device__ __forceinline__ half8 stage_frag(const hf* S, int row, int c, int g) {
	return *reinterpret_cast<const half8*>(S + row * STAGE_LD + 16 * c + 8 * g);
}
// B operand along the batch from an SoA global matrix: row `row`, samples b0 + 16c + 8g + 0..7
__device__ __forceinline__ half8 batch_frag_soa(const hf* __restrict__ M, size_t N, uint32_t b0, int row, int n_rows, int c, int g) {
	const uint32_t col = b0 + 16 * c + 8 * g;
	half8 z;
#pragma unroll
	for (int e = 0; e < 8; ++e) z[e] = (hf)0;
	if (row < n_rows && col < N) z = *reinterpret_cast<const half8*>(M + (size_t)row * N + col);
	return z;
}
// the constant matrix e_{unit_row} 1^T restricted to valid samples
__device__ __forceinline__ half8 batch_frag_unit(size_t N, uint32_t b0, int row, int unit_row, int c, int g) {
	const uint32_t col = b0 + 16 * c + 8 * g;
	half8 z;
#pragma unroll
	for (int e = 0; e < 8; ++e) z[e] = (row == unit_row && col < N) ? (hf)1 : (hf)0;
	return z;
}
__device__ __forceinline__ half8 batch_frag_aos16(const hf* __restrict__ M, size_t N, uint32_t b0, int row, int c, int g) {
	half8 z;
#pragma unroll
	for (int e = 0; e < 8; ++e) {
		const uint32_t col = b0 + 16 * c + 8 * g + e;
		z[e] = (row < MLP_OUT && col < N) ? M[(size_t)col * MLP_OUT + row] : (hf)0;
	}
	return z;
}

// 16-row operand (network output gradient) as B operand of both tiles, K = 16
__device__ __forceinline__ void outgrad_frag(const hf* __restrict__ dY, size_t N, uint32_t col, int g, bool aos, int unit_row, half8& t0, half8& t1) {
	if (unit_row >= 0) {
		// dL_dy = e_{unit_row} for every sample: nothing is read
#pragma unroll
		for (int e = 0; e < 8; ++e) t0[e] = t1[e] = (8 * g + e == unit_row) ? (hf)1 : (hf)0;
	} else if (aos) {
		t0 = *reinterpret_cast<const half8*>(dY + (size_t)col * MLP_OUT + 8 * g);
		t1 = *reinterpret_cast<const half8*>(dY + (size_t)(col + 1) * MLP_OUT + 8 * g);
	} else {
		bfrag_soa(dY, N, col, 0, g, MLP_OUT, t0, t1);
	}
}

// Store rows [0, n_rows) of D tiles (both sample tiles) of a 32*MT-row result to an SoA matrix.
template <int MT>
__device__ __forceinline__ void store_soa(hf* __restrict__ M, size_t N, uint32_t col, bool valid, const float16v (&d)[2][MT],
                                          int g, int n_rows) {
	if (!valid) return;
#pragma unroll
	for (int mt = 0; mt < MT; ++mt) {
#pragma unroll
		for (int r = 0; r < 16; ++r) {
			const int row = 32 * mt + drow(r, g);
			if (row < n_rows) *reinterpret_cast<half2v*>(M + (size_t)row * N + col) = half2v{(hf)d[0][mt][r], (hf)d[1][mt][r]};
		}
	}
}

// ----------------------------------------------------------------------------
// weights of one network in registers
// ----------------------------------------------------------------------------
template <int IN_CHUNKS, int N_HIDDEN>
struct FwdWeights {
	half8 w0[2][IN_CHUNKS];
	half8 wh[N_HIDDEN > 1 ? N_HIDDEN - 1 : 1][2][4];
	half8 wo[4];
	__device__ __forceinline__ void load(const hf* W, int n, int g) {
		constexpr int IN_W = 16 * IN_CHUNKS;
#pragma unroll
		for (int mt = 0; mt < 2; ++mt)
#pragma unroll
			for (int c = 0; c < IN_CHUNKS; ++c) w0[mt][c] = wfrag_natural(W, IN_W, 32 * mt + n, c, g);
		const hf* Wk = W + MLP_WIDTH * IN_W;
#pragma unroll
		for (int k = 0; k < N_HIDDEN - 1; ++k) {
#pragma unroll
			for (int mt = 0; mt < 2; ++mt)
#pragma unroll
				for (int c = 0; c < 4; ++c) wh[k][mt][c] = wfrag_chained(Wk, MLP_WIDTH, 32 * mt + n, c, g);
			Wk += MLP_WIDTH * MLP_WIDTH;
		}
#pragma unroll
		for (int c = 0; c < 4; ++c) {
			half8 z;
#pragma unroll
			for (int e = 0; e < 8; ++e) z[e] = (hf)0;
			wo[c] = (n < MLP_OUT) ? wfrag_chained(Wk, MLP_WIDTH, n, c, g) : z;
		}
	}
};

// Forward through the hidden layers for one 64-sample tile: fills h[k][t][c]
// (post-activation, fp16, chained operand form) for every hidden layer k.
template <int IN_CHUNKS, int N_HIDDEN>
__device__ __forceinline__ void forward_hidden(const FwdWeights<IN_CHUNKS, N_HIDDEN>& w, const half8 (&x)[2][IN_CHUNKS],
                                               half8 (&h)[N_HIDDEN][2][4]) {
#pragma unroll
	for (int t = 0; t < 2; ++t) {
#pragma unroll
		for (int mt = 0; mt < 2; ++mt) {
			float16v acc = zero16();
#pragma unroll
			for (int c = 0; c < IN_CHUNKS; ++c) acc = N2_MFMA(w.w0[mt][c], x[t][c], acc);
			relu_pack(acc, h[0][t][2 * mt], h[0][t][2 * mt + 1]);
		}
	}
#pragma unroll
	for (int k = 1; k < N_HIDDEN; ++k) {
#pragma unroll
		for (int t = 0; t < 2; ++t) {
#pragma unroll
			for (int mt = 0; mt < 2; ++mt) {
				float16v acc = zero16();
#pragma unroll
				for (int c = 0; c < 4; ++c) acc = N2_MFMA(w.wh[k - 1][mt][c], h[k - 1][t][c], acc);
				relu_pack(acc, h[k][t][2 * mt], h[k][t][2 * mt + 1]);
			}
		}
	}
}

template <int IN_CHUNKS>
__device__ __forceinline__ void load_input(const hf* __restrict__ X, size_t N, uint32_t col, int g, half8 (&x)[2][IN_CHUNKS]) {
#pragma unroll
	for (int c = 0; c < IN_CHUNKS; ++c) bfrag_soa(X, N, col, c, g, 16 * IN_CHUNKS, x[0][c], x[1][c]);
}

// ----------------------------------------------------------------------------
// forward kernel
// ----------------------------------------------------------------------------
template <int IN_CHUNKS, int N_HIDDEN>
__global__ void __launch_bounds__(MLP_BLOCK) mlp_forward_kernel(const hf* __restrict__ W, const hf* __restrict__ X, uint32_t N,
                                                                hf* __restrict__ Y, int out_aos, hf* __restrict__ hidden) {
	const int lane = threadIdx.x & 63, n = lane & 31, g = lane >> 5;
	const uint32_t n_tiles = (N + MLP_TILE - 1) / MLP_TILE;
	const uint32_t wave_gid = blockIdx.x * (MLP_BLOCK / 64) + (threadIdx.x >> 6), n_waves = gridDim.x * (MLP_BLOCK / 64);
	FwdWeights<IN_CHUNKS, N_HIDDEN> w;
	w.load(W, n, g);
	for (uint32_t tile = wave_gid; tile < n_tiles; tile += n_waves) {
		const uint32_t b0 = tile * MLP_TILE, col_raw = b0 + 2 * n;
		const bool valid = col_raw < N;
		const uint32_t col = valid ? col_raw : N - 2;
		half8 x[2][IN_CHUNKS];
		load_input<IN_CHUNKS>(X, N, col, g, x);
		half8 h[N_HIDDEN][2][4];
		forward_hidden<IN_CHUNKS, N_HIDDEN>(w, x, h);
		float16v out[2][1];
#pragma unroll
		for (int t = 0; t < 2; ++t) {
			out[t][0] = zero16();
#pragma unroll
			for (int c = 0; c < 4; ++c) out[t][0] = N2_MFMA(w.wo[c], h[N_HIDDEN - 1][t][c], out[t][0]);
		}
		if (out_aos) {
			if (valid) {
				// rows 4g..4g+3 (r = 0..3) and 8+4g..8+4g+3 (r = 4..7) of each sample
#pragma unroll
				for (int t = 0; t < 2; ++t) {
					hf* y = Y + (size_t)(col + t) * MLP_OUT;
					*reinterpret_cast<half4*>(y + 4 * g) = half4{(hf)out[t][0][0], (hf)out[t][0][1], (hf)out[t][0][2], (hf)out[t][0][3]};
					*reinterpret_cast<half4*>(y + 8 + 4 * g) = half4{(hf)out[t][0][4], (hf)out[t][0][5], (hf)out[t][0][6], (hf)out[t][0][7]};
				}
			}
		} else {
			store_soa<1>(Y, N, col, valid, out, g, MLP_OUT);
		}
		if (hidden && valid) {
#pragma unroll
			for (int k = 0; k < N_HIDDEN; ++k)
#pragma unroll
				for (int c = 0; c < 4; ++c)
#pragma unroll
					for (int e = 0; e < 8; ++e) {
						const int neuron = 16 * c + 4 * g + (e & 3) + ((e >> 2) << 3);
						*reinterpret_cast<half2v*>(hidden + ((size_t)k * MLP_WIDTH + neuron) * N + col) = half2v{h[k][0][c][e], h[k][1][c][e]};
					}
		}
	}
}

// ----------------------------------------------------------------------------
// weight-gradient accumulation helpers
// ----------------------------------------------------------------------------
// acc[mt][nt] += A_staged(64 rows) x B^T over the 64 samples of the tile.
// B comes from a second staged matrix.
template <int NT>
__device__ __forceinline__ void outer_staged(float16v (&acc)[2][NT], const hf* SA, const hf* SB, int n, int g) {
	stage_sync();
#pragma unroll
	for (int c = 0; c < 4; ++c) {
		half8 a[2], b[NT];
#pragma unroll
		for (int mt = 0; mt < 2; ++mt) a[mt] = stage_frag(SA, 32 * mt + n, c, g);
#pragma unroll
		for (int nt = 0; nt < NT; ++nt) b[nt] = stage_frag(SB, 32 * nt + n, c, g);
#pragma unroll
		for (int mt = 0; mt < 2; ++mt)
#pragma unroll
			for (int nt = 0; nt < NT; ++nt) acc[mt][nt] = N2_MFMA(a[mt], b[nt], acc[mt][nt]);
	}
}
// B comes straight from an SoA global matrix with n_rows valid rows.
template <int NT>
__device__ __forceinline__ void outer_global(float16v (&acc)[2][NT], const hf* SA, const hf* __restrict__ M, size_t N, uint32_t b0,
                                             int n_rows, bool aos16, int unit_row, int n, int g) {
	stage_sync();
#pragma unroll
	for (int c = 0; c < 4; ++c) {
		half8 a[2], b[NT];
#pragma unroll
		for (int mt = 0; mt < 2; ++mt) a[mt] = stage_frag(SA, 32 * mt + n, c, g);
#pragma unroll
		for (int nt = 0; nt < NT; ++nt)
			b[nt] = unit_row >= 0 ? batch_frag_unit(N, b0, 32 * nt + n, unit_row, c, g)
			      : aos16 ? batch_frag_aos16(M, N, b0, 32 * nt + n, c, g) : batch_frag_soa(M, N, b0, 32 * nt + n, n_rows, c, g);
#pragma unroll
		for (int mt = 0; mt < 2; ++mt)
#pragma unroll
			for (int nt = 0; nt < NT; ++nt) acc[mt][nt] = N2_MFMA(a[mt], b[nt], acc[mt][nt]);
	}
}

// Add a wave's D tiles (rows = 64 "left" indices, cols = 32*NT "right" indices)
// into the workgroup's fp32 LDS image of a weight matrix.
// transposed = false: left is the weight's row (out), right its column (in): W[left*ld + right]
// transposed = true : left is the column, right the row:                   W[right*ld + left]
template <int NT>
__device__ __forceinline__ void flush_acc(float* Wl, int ld, bool transposed, int n_right, const float16v (&acc)[2][NT], int n, int g) {
#pragma unroll
	for (int mt = 0; mt < 2; ++mt)
#pragma unroll
		for (int nt = 0; nt < NT; ++nt) {
			const int right = 32 * nt + n;
			if (right >= n_right) continue;
#pragma unroll
			for (int r = 0; r < 16; ++r) {
				const int left = 32 * mt + drow(r, g);
				atomicAdd(&Wl[transposed ? right * ld + left : left * ld + right], acc[mt][nt][r]);
			}
		}
}

// ----------------------------------------------------------------------------
// backward kernel: recomputes the hidden activations, then
//   dL_dh_last = mask * W_out^T dL_dy ; ... ; dL_dx = W_0^T dL_dh_0
//   dW_out = dL_dy h_last^T ; dW_k = dL_dh_k h_{k-1}^T ; dW_0 = dL_dh_0 x^T
// Weight gradients are summed per workgroup in fp32 and written to one slab of
// `partials` per workgroup; a second tiny kernel reduces the slabs.
// ----------------------------------------------------------------------------
template <int IN_CHUNKS, int N_HIDDEN, bool WANT_DX, bool WANT_DW>
__global__ void __launch_bounds__(MLP_BLOCK) mlp_backward_kernel(const hf* __restrict__ W, const hf* __restrict__ X, uint32_t N,
                                                                 const hf* __restrict__ dY, int dy_aos, int unit_row,
                                                                 hf* __restrict__ dX, float* __restrict__ partials) {
	constexpr int IN_W = 16 * IN_CHUNKS;
	constexpr int IN_MT = (IN_W + 31) / 32;
	constexpr int N_PARAMS = MLP_WIDTH * IN_W + (N_HIDDEN - 1) * MLP_WIDTH * MLP_WIDTH + MLP_OUT * MLP_WIDTH;
	extern __shared__ __align__(16) unsigned char smem[];
	const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, n = lane & 31, g = lane >> 5;
	const uint32_t n_tiles = (N + MLP_TILE - 1) / MLP_TILE;
	const uint32_t wave_gid = blockIdx.x * (MLP_BLOCK / 64) + wave, n_waves = gridDim.x * (MLP_BLOCK / 64);
	hf* SA = reinterpret_cast<hf*>(smem) + (size_t)wave * 2 * MLP_WIDTH * STAGE_LD;
	hf* SB = SA + MLP_WIDTH * STAGE_LD;

	FwdWeights<IN_CHUNKS, N_HIDDEN> w;
	w.load(W, n, g);
	// transposed weights for the data path
	const hf* W_out = W + MLP_WIDTH * IN_W + (N_HIDDEN - 1) * MLP_WIDTH * MLP_WIDTH;
	half8 woT[2];
#pragma unroll
	for (int mt = 0; mt < 2; ++mt) woT[mt] = wTfrag_natural(W_out, MLP_WIDTH, 32 * mt + n, 0, g, MLP_OUT);
	half8 whT[N_HIDDEN > 1 ? N_HIDDEN - 1 : 1][2][4];
#pragma unroll
	for (int k = 0; k < N_HIDDEN - 1; ++k)
#pragma unroll
		for (int mt = 0; mt < 2; ++mt)
#pragma unroll
			for (int c = 0; c < 4; ++c) whT[k][mt][c] = wTfrag_chained(W + MLP_WIDTH * IN_W + k * MLP_WIDTH * MLP_WIDTH, MLP_WIDTH, 32 * mt + n, c, g);
	half8 w0T[IN_MT][4];
	if (WANT_DX) {
#pragma unroll
		for (int mt = 0; mt < IN_MT; ++mt)
#pragma unroll
			for (int c = 0; c < 4; ++c) {
				half8 z;
#pragma unroll
				for (int e = 0; e < 8; ++e) z[e] = (hf)0;
				w0T[mt][c] = (32 * mt + n < IN_W) ? wTfrag_chained(W, IN_W, 32 * mt + n, c, g) : z;
			}
	}

	float16v gW0[2][IN_MT], gWh[N_HIDDEN > 1 ? N_HIDDEN - 1 : 1][2][2], gWo[2][1];
	if (WANT_DW) {
#pragma unroll
		for (int mt = 0; mt < 2; ++mt) {
#pragma unroll
			for (int nt = 0; nt < IN_MT; ++nt) gW0[mt][nt] = zero16();
#pragma unroll
			for (int k = 0; k < N_HIDDEN - 1; ++k) { gWh[k][mt][0] = zero16(); gWh[k][mt][1] = zero16(); }
			gWo[mt][0] = zero16();
		}
	}

	for (uint32_t tile = wave_gid; tile < n_tiles; tile += n_waves) {
		const uint32_t b0 = tile * MLP_TILE, col_raw = b0 + 2 * n;
		const bool valid = col_raw < N;
		const uint32_t col = valid ? col_raw : N - 2;
		half8 x[2][IN_CHUNKS];
		load_input<IN_CHUNKS>(X, N, col, g, x);
		half8 h[N_HIDDEN][2][4];
		forward_hidden<IN_CHUNKS, N_HIDDEN>(w, x, h);
		half8 dy[2];
		outgrad_frag(dY, N, col, g, dy_aos != 0, unit_row, dy[0], dy[1]);
		if (!valid) {
#pragma unroll
			for (int e = 0; e < 8; ++e) { dy[0][e] = (hf)0; dy[1][e] = (hf)0; }
		}
		// dL_dh of the last hidden layer
		half8 dh[2][4];
#pragma unroll
		for (int t = 0; t < 2; ++t)
#pragma unroll
			for (int mt = 0; mt < 2; ++mt) {
				float16v acc = N2_MFMA(woT[mt], dy[t], zero16());
				mask_pack(acc, h[N_HIDDEN - 1][t][2 * mt], h[N_HIDDEN - 1][t][2 * mt + 1], dh[t][2 * mt], dh[t][2 * mt + 1]);
			}
		if (WANT_DW) {
			// dW_out^T [neuron][o] += h_last dY^T
			stage_store(SA, h[N_HIDDEN - 1], n, g);
			outer_global<1>(gWo, SA, dY, N, b0, MLP_OUT, dy_aos != 0, unit_row, n, g);
		}
#pragma unroll
		for (int k = N_HIDDEN - 1; k >= 1; --k) {
			if (WANT_DW) {
				// dW_k [out][in] += dh_k h_{k-1}^T
				stage_store(SA, dh, n, g);
				stage_store(SB, h[k - 1], n, g);
				outer_staged<2>(gWh[k - 1], SA, SB, n, g);
			}
			half8 dprev[2][4];
#pragma unroll
			for (int t = 0; t < 2; ++t)
#pragma unroll
				for (int mt = 0; mt < 2; ++mt) {
					float16v acc = zero16();
#pragma unroll
					for (int c = 0; c < 4; ++c) acc = N2_MFMA(whT[k - 1][mt][c], dh[t][c], acc);
					mask_pack(acc, h[k - 1][t][2 * mt], h[k - 1][t][2 * mt + 1], dprev[t][2 * mt], dprev[t][2 * mt + 1]);
				}
#pragma unroll
			for (int t = 0; t < 2; ++t)
#pragma unroll
				for (int c = 0; c < 4; ++c) dh[t][c] = dprev[t][c];
		}
		if (WANT_DW) {
			// dW_0 [neuron][input] += dh_0 x^T
			stage_store(SA, dh, n, g);
			outer_global<IN_MT>(gW0, SA, X, N, b0, IN_W, false, -1, n, g);
		}
		if (WANT_DX) {
			float16v dx[2][IN_MT];
#pragma unroll
			for (int t = 0; t < 2; ++t)
#pragma unroll
				for (int mt = 0; mt < IN_MT; ++mt) {
					dx[t][mt] = zero16();
#pragma unroll
					for (int c = 0; c < 4; ++c) dx[t][mt] = N2_MFMA(w0T[mt][c], dh[t][c], dx[t][mt]);
				}
			store_soa<IN_MT>(dX, N, col, valid, dx, g, IN_W);
		}
	}

	if (WANT_DW) {
		__syncthreads();
		float* Wl = reinterpret_cast<float*>(smem);
		for (int i = threadIdx.x; i < N_PARAMS; i += MLP_BLOCK) Wl[i] = 0.f;
		__syncthreads();
		flush_acc<IN_MT>(Wl, IN_W, false, IN_W, gW0, n, g);
#pragma unroll
		for (int k = 0; k < N_HIDDEN - 1; ++k) flush_acc<2>(Wl + MLP_WIDTH * IN_W + k * MLP_WIDTH * MLP_WIDTH, MLP_WIDTH, false, MLP_WIDTH, gWh[k], n, g);
		flush_acc<1>(Wl + MLP_WIDTH * IN_W + (N_HIDDEN - 1) * MLP_WIDTH * MLP_WIDTH, MLP_WIDTH, true, MLP_OUT, gWo, n, g);
		__syncthreads();
		float* slab = partials + (size_t)blockIdx.x * N_PARAMS;
		for (int i = threadIdx.x; i < N_PARAMS; i += MLP_BLOCK) slab[i] = Wl[i];
	}
}

// ----------------------------------------------------------------------------
// second-order kernel (one hidden layer):
//   m = 1[W_0 x > 0];  a = m * (W_0 v);  b = m * (W_out^T g)
//   dW_0 += b v^T;  dW_out += g a^T;  dL_ddLdy = W_out a
// ----------------------------------------------------------------------------
template <int IN_CHUNKS>
__global__ void __launch_bounds__(MLP_BLOCK) mlp_bbi_kernel(const hf* __restrict__ W, const hf* __restrict__ X, uint32_t N,
                                                            const hf* __restrict__ V, const hf* __restrict__ G, int unit_row,
                                                            hf* __restrict__ dLddY, float* __restrict__ partials) {
	constexpr int IN_W = 16 * IN_CHUNKS;
	constexpr int IN_MT = (IN_W + 31) / 32;
	constexpr int N_PARAMS = MLP_WIDTH * IN_W + MLP_OUT * MLP_WIDTH;
	extern __shared__ __align__(16) unsigned char smem[];
	const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, n = lane & 31, g = lane >> 5;
	const uint32_t n_tiles = (N + MLP_TILE - 1) / MLP_TILE;
	const uint32_t wave_gid = blockIdx.x * (MLP_BLOCK / 64) + wave, n_waves = gridDim.x * (MLP_BLOCK / 64);
	hf* SA = reinterpret_cast<hf*>(smem) + (size_t)wave * 2 * MLP_WIDTH * STAGE_LD;

	FwdWeights<IN_CHUNKS, 1> w;
	w.load(W, n, g);
	const hf* W_out = W + MLP_WIDTH * IN_W;
	half8 woT[2];
#pragma unroll
	for (int mt = 0; mt < 2; ++mt) woT[mt] = wTfrag_natural(W_out, MLP_WIDTH, 32 * mt + n, 0, g, MLP_OUT);
	float16v gW0[2][IN_MT], gWo[2][1];
#pragma unroll
	for (int mt = 0; mt < 2; ++mt) {
#pragma unroll
		for (int nt = 0; nt < IN_MT; ++nt) gW0[mt][nt] = zero16();
		gWo[mt][0] = zero16();
	}
	for (uint32_t tile = wave_gid; tile < n_tiles; tile += n_waves) {
		const uint32_t b0 = tile * MLP_TILE, col_raw = b0 + 2 * n;
		const bool valid = col_raw < N;
		const uint32_t col = valid ? col_raw : N - 2;
		half8 x[2][IN_CHUNKS], v[2][IN_CHUNKS], gg[2];
		load_input<IN_CHUNKS>(X, N, col, g, x);
		load_input<IN_CHUNKS>(V, N, col, g, v);
		outgrad_frag(G, N, col, g, false, unit_row, gg[0], gg[1]);
		if (!valid) {
#pragma unroll
			for (int e = 0; e < 8; ++e) {
				gg[0][e] = (hf)0; gg[1][e] = (hf)0;
#pragma unroll
				for (int c = 0; c < IN_CHUNKS; ++c) { v[0][c][e] = (hf)0; v[1][c][e] = (hf)0; }
			}
		}
		half8 h[1][2][4];
		forward_hidden<IN_CHUNKS, 1>(w, x, h);
		half8 a[2][4], b[2][4];
#pragma unroll
		for (int t = 0; t < 2; ++t)
#pragma unroll
			for (int mt = 0; mt < 2; ++mt) {
				float16v acc = zero16();
#pragma unroll
				for (int c = 0; c < IN_CHUNKS; ++c) acc = N2_MFMA(w.w0[mt][c], v[t][c], acc);
				mask_pack(acc, h[0][t][2 * mt], h[0][t][2 * mt + 1], a[t][2 * mt], a[t][2 * mt + 1]);
				float16v accb = N2_MFMA(woT[mt], gg[t], zero16());
				mask_pack(accb, h[0][t][2 * mt], h[0][t][2 * mt + 1], b[t][2 * mt], b[t][2 * mt + 1]);
			}
		if (partials) {
			stage_store(SA, b, n, g);
			outer_global<IN_MT>(gW0, SA, V, N, b0, IN_W, false, -1, n, g);
			stage_store(SA, a, n, g);
			outer_global<1>(gWo, SA, G, N, b0, MLP_OUT, false, unit_row, n, g);
		}
		if (dLddY) {
			float16v out[2][1];
#pragma unroll
			for (int t = 0; t < 2; ++t) {
				out[t][0] = zero16();
#pragma unroll
				for (int c = 0; c < 4; ++c) out[t][0] = N2_MFMA(w.wo[c], a[t][c], out[t][0]);
			}
			store_soa<1>(dLddY, N, col, valid, out, g, MLP_OUT);
		}
	}
	if (partials) {
		__syncthreads();
		float* Wl = reinterpret_cast<float*>(smem);
		for (int i = threadIdx.x; i < N_PARAMS; i += MLP_BLOCK) Wl[i] = 0.f;
		__syncthreads();
		flush_acc<IN_MT>(Wl, IN_W, false, IN_W, gW0, n, g);
		flush_acc<1>(Wl + MLP_WIDTH * IN_W, MLP_WIDTH, true, MLP_OUT, gWo, n, g);
		__syncthreads();
		float* slab = partials + (size_t)blockIdx.x * N_PARAMS;
		for (int i = threadIdx.x; i < N_PARAMS; i += MLP_BLOCK) slab[i] = Wl[i];
	}
}

// grads (fp16) = [grads +] sum over slabs.  16 parameters x 16 slab groups per workgroup: every
// lane adds up n_slabs/16 partial sums (coalesced across the 16 parameters), LDS folds the groups.
__global__ void __launch_bounds__(256) mlp_reduce_partials_kernel(const float* __restrict__ partials, uint32_t n_slabs, uint32_t n_params,
                                                                  hf* __restrict__ grads, int accumulate) {
	__shared__ float fold[16][17];
	const uint32_t pl = threadIdx.x & 15, grp = threadIdx.x >> 4;
	const uint32_t i = blockIdx.x * 16 + pl;
	float s = 0.f;
	if (i < n_params)
		for (uint32_t k = grp; k < n_slabs; k += 16) s += partials[(size_t)k * n_params + i];
	fold[grp][pl] = s;
	__syncthreads();
	if (grp == 0 && i < n_params) {
		float t = 0.f;
#pragma unroll
		for (int k = 0; k < 16; ++k) t += fold[k][pl];
		if (accumulate) t += (float)grads[i];
		grads[i] = (hf)t;
	}
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
	*out = m;
	return N2_OK;
}
N2_API void n2_mlp_destroy(n2_mlp_t* mlp) { delete mlp; }
N2_API uint32_t n2_mlp_n_params(const n2_mlp_t* mlp) { return mlp ? mlp->n_params : 0; }
N2_API uint32_t n2_mlp_input_width(const n2_mlp_t* mlp) { return mlp ? mlp->in_w : 0; }
N2_API uint32_t n2_mlp_output_width(const n2_mlp_t* mlp) { return mlp ? MLP_OUT : 0; }
N2_API uint64_t n2_mlp_workspace_bytes(const n2_mlp_t* mlp) { return mlp ? (uint64_t)MLP_MAX_SLABS * mlp->n_params * sizeof(float) : 0; }

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
	N2_REQUIRE(n <= (1u << 30), "%s: batch size %u exceeds 2^30", fn, n);
	N2_REQUIRE(d_input != nullptr || n == 0, "%s: d_input is null", fn);
	N2_REQUIRE(reinterpret_cast<uintptr_t>(d_input) % 16 == 0, "%s: d_input must be 16-byte aligned", fn);
	return N2_OK;
}

static inline uint32_t stream_grid(uint32_t n, uint32_t max_blocks) {
	const uint32_t tiles = (n + MLP_TILE - 1) / MLP_TILE;
	const uint32_t blocks = (tiles + (MLP_BLOCK / 64) - 1) / (MLP_BLOCK / 64);
	return blocks < max_blocks ? blocks : max_blocks;
}

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
	const dim3 grid(stream_grid(n, 2048)), block(MLP_BLOCK);
	N2ProfScope prof(N2_PROF_MLP_FORWARD, n2_stream(stream));
#define CALL(IC, NH)                                                                                                     \
	mlp_forward_kernel<IC, NH><<<grid, block, 0, n2_stream(stream)>>>(mlp->params, reinterpret_cast<const hf*>(d_input), n, \
		reinterpret_cast<hf*>(d_output), out_layout == N2_LAYOUT_AOS ? 1 : 0, reinterpret_cast<hf*>(d_hidden))
	MLP_DISPATCH(mlp->in_w, mlp->n_hidden, CALL);
#undef CALL
	N2_LAUNCH_CHECK();
	return N2_OK;
}

static int reduce_partials(n2_mlp_t* mlp, hipStream_t s, uint32_t n_slabs, n2_grad_mode mode) {
	mlp_reduce_partials_kernel<<<dim3((mlp->n_params + 15) / 16), dim3(256), 0, s>>>(mlp->workspace, n_slabs, mlp->n_params,
		mlp->grads, mode == N2_GRAD_ACCUMULATE ? 1 : 0);
	N2_LAUNCH_CHECK();
	return N2_OK;
}

static int check_grad_mode(const n2_mlp_t* mlp, const char* fn, n2_grad_mode mode) {
	N2_REQUIRE(mode == N2_GRAD_IGNORE || mode == N2_GRAD_OVERWRITE || mode == N2_GRAD_ACCUMULATE, "%s: bad gradient mode %d", fn, (int)mode);
	if (mode != N2_GRAD_IGNORE) {
		N2_REQUIRE(mlp->grads != nullptr, "%s: gradient mode %d needs a gradient buffer (n2_mlp_set_params)", fn, (int)mode);
		N2_REQUIRE(mlp->workspace != nullptr, "%s: gradient mode %d needs a workspace (n2_mlp_set_workspace)", fn, (int)mode);
	}
	return N2_OK;
}

static constexpr size_t STAGE_BYTES = (size_t)(MLP_BLOCK / 64) * 2 * MLP_WIDTH * STAGE_LD * sizeof(hf);

template <typename K>
static int allow_lds(K kernel, size_t bytes) {
	if (bytes > 48 * 1024) N2_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes));
	return N2_OK;
}

// unit_row >= 0: dL_doutput is the constant e_{unit_row} and d_dL_doutput is not read
static int mlp_backward_impl(n2_mlp_t* mlp, n2_stream_t stream, const n2_half* d_input, uint32_t n,
                             const n2_half* d_dL_doutput, n2_layout dL_layout, int unit_row, n2_half* d_dL_dinput, n2_grad_mode mode) {
	if (int rc = check_mlp_batch(mlp, "n2_mlp_backward", d_input, n)) return rc;
	if (int rc = check_grad_mode(mlp, "n2_mlp_backward", mode)) return rc;
	N2_REQUIRE(dL_layout == N2_LAYOUT_SOA || dL_layout == N2_LAYOUT_AOS, "n2_mlp_backward: bad layout %d", (int)dL_layout);
	N2_REQUIRE(d_dL_doutput != nullptr || n == 0 || unit_row >= 0, "n2_mlp_backward: d_dL_doutput is null");
	N2_REQUIRE(reinterpret_cast<uintptr_t>(d_dL_doutput) % 16 == 0 && reinterpret_cast<uintptr_t>(d_dL_dinput) % 16 == 0,
	           "n2_mlp_backward: buffers must be 16-byte aligned");
	hipStream_t s = n2_stream(stream);
	const bool want_dw = mode != N2_GRAD_IGNORE, want_dx = d_dL_dinput != nullptr;
	if (n == 0) {
		if (mode == N2_GRAD_OVERWRITE) return n2_fill_zero_u32(s, mlp->grads, mlp->n_params * sizeof(hf));
		return N2_OK;
	}
	if (!want_dw && !want_dx) return N2_OK;
	const uint32_t blocks = stream_grid(n, want_dw ? MLP_MAX_SLABS : 2048);
	const size_t lds_stage = want_dw ? STAGE_BYTES : 0;
	const size_t lds = want_dw ? (lds_stage > mlp->n_params * sizeof(float) ? lds_stage : mlp->n_params * sizeof(float)) : 0;
	const hf* X = reinterpret_cast<const hf*>(d_input);
	const hf* dY = reinterpret_cast<const hf*>(d_dL_doutput);
	hf* dX = reinterpret_cast<hf*>(d_dL_dinput);
	const int aos = dL_layout == N2_LAYOUT_AOS ? 1 : 0;
	N2ProfScope prof(N2_PROF_MLP_BACKWARD, s);
#define LAUNCH(IC, NH, DX, DW)                                                                                      \
	do {                                                                                                            \
		if (int rc = allow_lds(mlp_backward_kernel<IC, NH, DX, DW>, lds)) return rc;                                \
		mlp_backward_kernel<IC, NH, DX, DW><<<dim3(blocks), dim3(MLP_BLOCK), lds, s>>>(mlp->params, X, n, dY, aos, unit_row, dX, mlp->workspace); \
	} while (0)
#define CALL(IC, NH)                                   \
	do {                                               \
		if (want_dx && want_dw) LAUNCH(IC, NH, true, true);    \
		else if (want_dx) LAUNCH(IC, NH, true, false);         \
		else LAUNCH(IC, NH, false, true);                      \
	} while (0)
	MLP_DISPATCH(mlp->in_w, mlp->n_hidden, CALL);
#undef CALL
#undef LAUNCH
	N2_LAUNCH_CHECK();
	if (want_dw) return reduce_partials(mlp, s, blocks, mode);
	return N2_OK;
}

N2_API int n2_mlp_backward(n2_mlp_t* mlp, n2_stream_t stream, const n2_half* d_input, uint32_t n,
                           const n2_half* d_dL_doutput, n2_layout dL_layout, n2_half* d_dL_dinput, n2_grad_mode mode) {
	return mlp_backward_impl(mlp, stream, d_input, n, d_dL_doutput, dL_layout, -1, d_dL_dinput, mode);
}

N2_API int n2_mlp_input_gradient(n2_mlp_t* mlp, n2_stream_t stream, uint32_t dim, const n2_half* d_input, uint32_t n,
                                 n2_half* d_dinput) {
	N2_REQUIRE(dim < (uint32_t)MLP_OUT, "n2_mlp_input_gradient: output dimension %u out of range", dim);
	N2_REQUIRE(d_dinput != nullptr || n == 0, "n2_mlp_input_gradient: d_dinput is null");
	return mlp_backward_impl(mlp, stream, d_input, n, nullptr, N2_LAYOUT_SOA, (int)dim, d_dinput, N2_GRAD_IGNORE);
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
	const uint32_t blocks = stream_grid(n, MLP_MAX_SLABS);
	const size_t lds = STAGE_BYTES > mlp->n_params * sizeof(float) ? STAGE_BYTES : mlp->n_params * sizeof(float);
	N2ProfScope prof(N2_PROF_MLP_SECOND_ORDER, s);
	switch (mlp->in_w / 16) {
#define CASE(IC)                                                                                                           \
	case IC:                                                                                                               \
		if (int rc = allow_lds(mlp_bbi_kernel<IC>, lds)) return rc;                                                        \
		mlp_bbi_kernel<IC><<<dim3(blocks), dim3(MLP_BLOCK), lds, s>>>(mlp->params, reinterpret_cast<const hf*>(d_input), n, \
			reinterpret_cast<const hf*>(d_dL_ddLdinput), reinterpret_cast<const hf*>(d_dL_doutput), unit_row,              \
			reinterpret_cast<hf*>(d_dL_ddLdoutput), want_dw ? mlp->workspace : nullptr);                                   \
		break;
		CASE(1) CASE(2) CASE(3) CASE(4)
#undef CASE
		default: n2_set_error("mlp: unsupported shape"); return N2_ERR_UNSUPPORTED;
	}
	N2_LAUNCH_CHECK();
	if (want_dw) return reduce_partials(mlp, s, blocks, mode);
	return N2_OK;
}
