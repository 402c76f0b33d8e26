// Device-side building blocks of the fully fused 64-wide MLP kernels: MFMA operand layouts, fragment loaders,
// packing / ReLU / mask helpers and the weight fragments kept in LDS.  Shared by the stand-alone MLP kernels and
// the fused field kernels.
//
// MFMA tiling (v_mfma_f32_32x32x16_f16, wave64):
//   A (32 x 16, weights)      lane l holds A[l%32][8*(l/32) + 0..7]
//   B (16 x 32, activations)  lane l holds B[8*(l/32) + 0..7][l%32]
//   D (32 x 32, fp32)         lane l holds D[8*(r/4) + 4*(l/32) + r%4][l%32], r = 0..15
// Chaining: registers r = 8*h .. 8*h+7 of a D tile are exactly one B operand for the K-chunk
// "rows {16c+4g+0..3, 16c+8+4g+0..3}" (c = h); weight fragments of the next layer are loaded with the same
// permutation of K ("chained" order).
#pragma once
#include "n2_common.h"

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef _Float16 half4v __attribute__((ext_vector_type(4)));
typedef _Float16 half4 __attribute__((ext_vector_type(4)));
typedef _Float16 half2v __attribute__((ext_vector_type(2)));
typedef float float16v __attribute__((ext_vector_type(16)));
typedef _Float16 hf;

#define N2_MFMA(a, b, c) __builtin_amdgcn_mfma_f32_32x32x16_f16((a), (b), (c), 0, 0, 0)

constexpr int MLP_WIDTH = 64;
constexpr int MLP_OUT = 16;
constexpr int MLP_BLOCK = 256;      // 4 waves
constexpr int MLP_TILE = 64;        // samples per wave iteration
constexpr int MLP_MAX_SLABS = 512;  // workgroups of the weight-gradient kernels (two per CU)

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

// B operands of both sample tiles for K-chunk c from an SoA matrix (rows x N): rows 16c + 8g + e,
// sample pair at column `col`.  off8 = 8*g*N + col is the only per-lane part of the address; the
// row part is uniform, so every load is "scalar base + one shared 32-bit lane offset".
__device__ __forceinline__ void bfrag_soa(const hf* __restrict__ M, uint32_t N, uint32_t off8, int c, int n_rows, half8& t0, half8& t1) {
#pragma unroll
	for (int e = 0; e < 8; ++e) {
		half2v v = {(hf)0, (hf)0};
		if (16 * c + e < n_rows) v = *reinterpret_cast<const half2v*>(M + (size_t)(16 * c + e) * N + off8);
		t0[e] = v[0];
		t1[e] = v[1];
	}
}

typedef short short8 __attribute__((ext_vector_type(8)));
typedef uint32_t uint4v __attribute__((ext_vector_type(4)));
// fp16 rounding of eight D-tile registers starting at `base`, as four two-element conversions
typedef float float2v __attribute__((ext_vector_type(2)));
__device__ __forceinline__ half8 round8(const float16v& d, int base) {
	uint4v r;
#pragma unroll
	for (int w = 0; w < 4; ++w) {
		const float2v p = {d[base + 2 * w], d[base + 2 * w + 1]};
		r[w] = __builtin_bit_cast(uint32_t, __builtin_convertvector(p, half2v));
	}
	return __builtin_bit_cast(half8, r);
}
// ReLU of rounded values as a packed 16-bit integer max with 0: every negative half (the sign bit makes it a negative
// integer, -0 included) becomes +0, positive halves keep their bits.  relu(round(x)) == round(relu(x)).
__device__ __forceinline__ half8 relu8(half8 v) {
	const short8 z = {0, 0, 0, 0, 0, 0, 0, 0};
	return __builtin_bit_cast(half8, __builtin_elementwise_max(__builtin_bit_cast(short8, v), z));
}
// v where the saved activation is > 0, else 0.  Activations come out of relu8, so as 16-bit integers they are 0 or
// positive and (0 - a) >> 15 (arithmetic) is all ones exactly for a > 0: two packed 16-bit instructions per pair.  The
// empty asm statement between them only hides the subtraction's result from the optimiser, which otherwise turns the
// expression back into one compare and select per element; it emits no instruction, so every register write comes
// from an instruction whose hazards the compiler tracks (a real instruction inside an asm block is not covered by its
// wait-state insertion: placed right behind an MFMA whose destination registers it reuses, its result is overwritten).
typedef short short2v __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint32_t positive_mask2(uint32_t act_pair) {
	short2v d = (short2v){0, 0} - __builtin_bit_cast(short2v, act_pair);
	asm("" : "+v"(d));
	d = d >> (short2v){15, 15};
	return __builtin_bit_cast(uint32_t, d);
}
__device__ __forceinline__ half8 mask8(half8 v, half8 act) {
	const uint4v a = __builtin_bit_cast(uint4v, act);
	uint4v x = __builtin_bit_cast(uint4v, v);
#pragma unroll
	for (int w = 0; w < 4; ++w) x[w] &= positive_mask2(a[w]);
	return __builtin_bit_cast(half8, x);
}
// ReLU + fp16 rounding of a D tile into the two chained B operands it holds
__device__ __forceinline__ void relu_pack(const float16v& d, half8& lo, half8& hi) {
	lo = relu8(round8(d, 0));
	hi = relu8(round8(d, 8));
}
// masked (by the sign of a saved activation) fp16 rounding of a D tile
__device__ __forceinline__ void mask_pack(const float16v& d, const half8& act_lo, const half8& act_hi, half8& lo, half8& hi) {
	lo = mask8(round8(d, 0), act_lo);
	hi = mask8(round8(d, 8), act_hi);
}

__device__ __forceinline__ float16v zero16() {
	float16v z;
#pragma unroll
	for (int r = 0; r < 16; ++r) z[r] = 0.f;
	return z;
}

// row index inside a 32-row D tile held in register r by lane group g
__device__ __forceinline__ int drow(int r, int g) { return 8 * (r >> 2) + 4 * g + (r & 3); }

// 16-row operand (network output gradient) as B operand of both tiles, K = 16
// rows >= n_rows of the operand count as zero (n_rows = 16: all rows are read)
__device__ __forceinline__ void outgrad_frag(const hf* __restrict__ dY, size_t N, uint32_t col, int g, bool aos, int unit_row, int n_rows, half8& t0,
                                             half8& t1) {
	if (unit_row >= 0) {
		// dL_dy = e_{unit_row} for every sample: nothing is read
#pragma unroll
		for (int e = 0; e < 8; ++e) t0[e] = t1[e] = (8 * g + e == unit_row) ? (hf)1 : (hf)0;
	} else if (aos) {
		t0 = *reinterpret_cast<const half8*>(dY + (size_t)col * MLP_OUT + 8 * g);
		t1 = *reinterpret_cast<const half8*>(dY + (size_t)(col + 1) * MLP_OUT + 8 * g);
	} else {
		bfrag_soa(dY, (uint32_t)N, 8u * g * (uint32_t)N + col, 0, MLP_OUT, t0, t1);
	}
	if (unit_row < 0 && n_rows < MLP_OUT) {
#pragma unroll
		for (int e = 0; e < 8; ++e)
			if (8 * g + e >= n_rows) { t0[e] = (hf)0; t1[e] = (hf)0; }
	}
}

// natural-K input operands of both sample tiles of a wave's 64 samples
template <int IC>
__device__ __forceinline__ void load_input(const hf* __restrict__ X, size_t N, uint32_t col, int g, half8 (&x)[2][IC]) {
#pragma unroll
	for (int c = 0; c < IC; ++c) bfrag_soa(X, (uint32_t)N, 8u * g * (uint32_t)N + col, c, 16 * IC, x[0][c], x[1][c]);
}

// the same operands when the wave's samples are columns s0 (tile 0) and s1 (tile 1) of a matrix with n_src columns:
// the row part of every address is uniform (a scalar base), the lane part two 32-bit byte offsets
template <int IC>
__device__ __forceinline__ void load_input_indexed(const hf* __restrict__ X, uint32_t n_src, uint32_t s0, uint32_t s1, int g, half8 (&x)[2][IC]) {
	const uint32_t b0 = (8u * g * n_src + s0) * 2u, b1 = (8u * g * n_src + s1) * 2u;
#pragma unroll
	for (int c = 0; c < IC; ++c)
#pragma unroll
		for (int e = 0; e < 8; ++e) {
			const char* row = reinterpret_cast<const char*>(X + (size_t)(16 * c + e) * n_src);
			x[0][c][e] = *reinterpret_cast<const hf*>(row + b0);
			x[1][c][e] = *reinterpret_cast<const hf*>(row + b1);
		}
}

// ----------------------------------------------------------------------------
// Weight fragments in LDS.
// A workgroup builds every MFMA operand the kernels need once, in "fragment
// form": fragment f is 64 lanes x 16 bytes at F + f*512 halves, so a wave reads
// an operand with one conflict-free 16-byte LDS load per lane.  Keeping the
// weights out of the register file is what lets two workgroups share a CU.
// ----------------------------------------------------------------------------
template <int IC, int NH>
struct FragMap {
	static constexpr int IN_W = 16 * IC, IN_MT = (IN_W + 31) / 32;
	static constexpr int W0 = 0;                      // [mt][c]    W_0 rows 32mt+n, natural K            (A of the sample-lane chain)
	static constexpr int WH = W0 + 2 * IC;            // [k][mt][c] hidden weights, chained K
	static constexpr int WO = WH + (NH - 1) * 8;      // [c]        W_out rows n < 16, chained K
	static constexpr int FWD_COUNT = WO + 4;
	static constexpr int WOT = FWD_COUNT;             // [mt]       W_out^T rows 32mt+n, K = 16 outputs
	static constexpr int WHT = WOT + 2;               // [k][mt][c] hidden weights transposed, chained K
	static constexpr int W0T = WHT + (NH - 1) * 8;    // [mt][c]    W_0^T rows 32mt+n (< IN_W), chained K
	static constexpr int SEL = W0T + IN_MT * 4;       // [c]        selects input rows 16c.. into feature tile c/2
	static constexpr int ID = SEL + IC;               //            16 x 32 identity
	static constexpr int COUNT = ID + 1;
};

__device__ __forceinline__ half8 zero8() {
	half8 z;
#pragma unroll
	for (int e = 0; e < 8; ++e) z[e] = (hf)0;
	return z;
}

// what lane l holds of fragment f
template <int IC, int NH>
__device__ __forceinline__ half8 mlp_frag_value(const hf* __restrict__ W, int f, int l) {
	using M = FragMap<IC, NH>;
	const hf* W_hid = W + MLP_WIDTH * M::IN_W;
	const hf* W_out = W_hid + (NH - 1) * MLP_WIDTH * MLP_WIDTH;
	{
		const int n = l & 31, g = l >> 5;
		half8 v = zero8();
		if (f < M::WH) {
			v = wfrag_natural(W, M::IN_W, 32 * (f / IC) + n, f % IC, g);
		} else if (f < M::WO) {
			const int q = f - M::WH;
			v = wfrag_chained(W_hid + (q >> 3) * MLP_WIDTH * MLP_WIDTH, MLP_WIDTH, 32 * ((q >> 2) & 1) + n, q & 3, g);
		} else if (f < M::WOT) {
			if (n < MLP_OUT) v = wfrag_chained(W_out, MLP_WIDTH, n, f - M::WO, g);
		} else if (f < M::WHT) {
			v = wTfrag_natural(W_out, MLP_WIDTH, 32 * (f - M::WOT) + n, 0, g, MLP_OUT);
		} else if (f < M::W0T) {
			const int q = f - M::WHT;
			v = wTfrag_chained(W_hid + (q >> 3) * MLP_WIDTH * MLP_WIDTH, MLP_WIDTH, 32 * ((q >> 2) & 1) + n, q & 3, g);
		} else if (f < M::SEL) {
			const int q = f - M::W0T, m = 32 * (q >> 2) + n;
			if (m < M::IN_W) v = wTfrag_chained(W, M::IN_W, m, q & 3, g);
		} else if (f < M::ID) {
			const int c = f - M::SEL;
#pragma unroll
			for (int e = 0; e < 8; ++e) v[e] = (16 * c + 8 * g + e == 32 * (c >> 1) + n) ? (hf)1 : (hf)0;
		} else {
#pragma unroll
			for (int e = 0; e < 8; ++e) v[e] = (8 * g + e == n) ? (hf)1 : (hf)0;
		}
		return v;
	}
}
template <int IC, int NH>
__device__ __forceinline__ void build_frags(hf* F, const hf* __restrict__ W, int count) {
	for (int idx = threadIdx.x; idx < count * 64; idx += MLP_BLOCK) *reinterpret_cast<half8*>(F + (size_t)idx * 8) = mlp_frag_value<IC, NH>(W, idx >> 6, idx & 63);
	__syncthreads();
}
// the same fragments from an image that another launch has built in global memory (count KiB)
__device__ __forceinline__ void load_frags(hf* F, const hf* __restrict__ image, int count) {
	for (int idx = threadIdx.x; idx < count * 64; idx += MLP_BLOCK) *reinterpret_cast<half8*>(F + (size_t)idx * 8) = *reinterpret_cast<const half8*>(image + (size_t)idx * 8);
	__syncthreads();
}

// Ends one 32-sample tile: keeps the compiler from interleaving two tiles and from hoisting the
// (loop-invariant) fragment loads into registers, which is exactly the register pressure to avoid.
__device__ __forceinline__ void tile_fence() {
	__builtin_amdgcn_sched_barrier(0);
	asm volatile("" ::: "memory");
}
__device__ __forceinline__ half8 frag(const hf* F, int f, int lane) { return *reinterpret_cast<const half8*>(F + f * 512 + lane * 8); }

// fp16 rounding of a D tile into its two chained operands (no activation)
__device__ __forceinline__ void plain_pack(const float16v& d, half8& lo, half8& hi) {
#pragma unroll
	for (int e = 0; e < 8; ++e) {
		lo[e] = (hf)d[e];
		hi[e] = (hf)d[8 + e];
	}
}

// A register set that is the B operand of a matrix X (K x 32 samples, lane = sample) is at the same
// time the A operand of X^T.  Swapping the two MFMA arguments of D = W X therefore yields
// D^T = X^T W^T: the same activations with lane = neuron and the 32 samples along the registers.
// Packed, a D^T tile is directly an operand of the batch-reduction products dW = dh h^T
// (K = samples), so the weight gradients need no transposition through memory.

// hidden layers, sample-lane form, for one 32-sample tile
template <int IC, int NH>
__device__ __forceinline__ void hidden_S(const hf* F, int lane, const half8 (&x)[IC], half8 (&h)[NH][4]) {
	using M = FragMap<IC, NH>;
#pragma unroll
	for (int mt = 0; mt < 2; ++mt) {
		float16v acc = zero16();
#pragma unroll
		for (int c = 0; c < IC; ++c) acc = N2_MFMA(frag(F, M::W0 + mt * IC + c, lane), x[c], acc);
		relu_pack(acc, h[0][2 * mt], h[0][2 * mt + 1]);
	}
#pragma unroll
	for (int k = 1; k < NH; ++k)
#pragma unroll
		for (int mt = 0; mt < 2; ++mt) {
			float16v acc = zero16();
#pragma unroll
			for (int c = 0; c < 4; ++c) acc = N2_MFMA(frag(F, M::WH + (k - 1) * 8 + mt * 4 + c, lane), h[k - 1][c], acc);
			relu_pack(acc, h[k][2 * mt], h[k][2 * mt + 1]);
		}
}
// neuron-lane form of neuron tile nt of hidden layer k (k = 0: from the input, else from layer k-1 in sample-lane form)
template <int IC, int NH>
__device__ __forceinline__ void hidden_N(const hf* F, int lane, int k, int nt, const half8 (&x)[IC], const half8 (&h)[NH][4], half8 (&out)[2]) {
	using M = FragMap<IC, NH>;
	float16v acc = zero16();
	if (k == 0) {
#pragma unroll
		for (int c = 0; c < IC; ++c) acc = N2_MFMA(x[c], frag(F, M::W0 + nt * IC + c, lane), acc);
	} else {
#pragma unroll
		for (int c = 0; c < 4; ++c) acc = N2_MFMA(h[k - 1][c], frag(F, M::WH + (k - 1) * 8 + nt * 4 + c, lane), acc);
	}
	relu_pack(acc, out[0], out[1]);
}
// input rows of feature tile nt in feature-lane form (exact: products with 0 and 1)
template <int IC, int NH>
__device__ __forceinline__ void input_N(const hf* F, int lane, int nt, const half8 (&x)[IC], half8 (&out)[2]) {
	using M = FragMap<IC, NH>;
	float16v acc = zero16();
#pragma unroll
	for (int c = 0; c < IC; ++c)
		if ((c >> 1) == nt) acc = N2_MFMA(x[c], frag(F, M::SEL + c, lane), acc);
	plain_pack(acc, out[0], out[1]);
}

template <int IC>
__device__ __forceinline__ void split_pairs(const half8 (&p)[2][IC], int t, half8 (&x)[IC]) {
#pragma unroll
	for (int c = 0; c < IC; ++c) x[c] = p[t][c];
}

