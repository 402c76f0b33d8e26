// Backward pass of the fully fused 64-wide MLP WITH weight gradients (and, for one hidden layer, the second-order pass
// riding along): every wave runs the forward and the data-gradient chain for its OWN 32 samples only, and the batch
// reductions dW = dh h^T take their operands from LDS, where the four waves of a workgroup leave the activations and
// their gradients of 128 samples.
//
// The chain produces matrices in sample-lane form (lane = sample, registers = rows); a product over samples needs
// them in row-lane form (lane = row, registers = 8 consecutive samples), for both operands.  The staging buffer is laid
// out as quads, S[quad q][sample s] = rows 4q .. 4q+3 of sample s (8 bytes): a lane writes the rows it holds with 8-byte
// stores, and ds_read_b64_tr_b16 hands a row-lane its samples: in every group of 16 lanes, lane i receives as element j
// the (i % 4)-th 16-bit value of what lane i / 4 + 4 j of the group addressed.  With lane a + 4 j' of a group addressing
// quad qb + a of sample k + j', lane i gets row 4 qb + i for the samples k .. k+3: two such reads are one MFMA operand
// (32 rows x 16 samples).  A quad row is 128 x 8 + 32 bytes, so the four quads of a read fall on different banks.
//
// Stages of a round (a stage = write, barrier, products, barrier), two hidden layers:  {dy, h1} -> dW_out,
// {dh1, h0} -> dW_1, {dh0, x} -> dW_0; one hidden layer with the second-order pass:  {dy, h, g, a} -> dW_out,
// {dh, x} -> dW_0, {b, v} -> dW_0.  The weight-gradient tiles (32 x 32) of a matrix are dealt to the four waves; where a
// matrix has two tiles only, the waves split the samples or the two products.  Each wave then holds 48 accumulator
// registers instead of 128, and no activation is computed twice.
#pragma once
#include "grid_device.h"
#include "mlp_device.h"

constexpr int WG_SAMPLES = 128;              // samples per workgroup round (4 waves x 32)
constexpr int WG_QP = WG_SAMPLES * 8 + 32;   // bytes per quad row of the staging buffer

typedef short short4v __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) short4v* lds_short4_ptr;

// staging writes: v holds 8 rows of the lane's sample; `at` = S + quad offset of the rows' block + the lane's part
// natural row order (rows 8 g + e of a 16-row chunk):  lane part = s * 8 + 2 g * WG_QP, quads q, q + 1
__device__ __forceinline__ void stage_natural(unsigned char* at, const half8& v) {
	const uint4v w = __builtin_bit_cast(uint4v, v);
	*reinterpret_cast<uint2*>(at) = make_uint2(w[0], w[1]);
	*reinterpret_cast<uint2*>(at + WG_QP) = make_uint2(w[2], w[3]);
}
// chained row order (rows 4 g + 0..3 and 8 + 4 g + 0..3 of a 16-row chunk):  lane part = s * 8 + g * WG_QP, quads q, q + 2
__device__ __forceinline__ void stage_chained(unsigned char* at, const half8& v) {
	const uint4v w = __builtin_bit_cast(uint4v, v);
	*reinterpret_cast<uint2*>(at) = make_uint2(w[0], w[1]);
	*reinterpret_cast<uint2*>(at + 2 * WG_QP) = make_uint2(w[2], w[3]);
}
// row-lane MFMA operand: rows 4 qb .. 4 qb + 31, samples 16 kc .. 16 kc + 15 of the round; tr = S + the lane's part
// ((4 (G & 1) + (l & 3)) * WG_QP + (8 (G >> 1) + ((l & 15) >> 2)) * 8, G = l / 16)
__device__ __forceinline__ half8 row_operand(const unsigned char* tr, int qb, int kc) {
	const unsigned char* p = tr + qb * WG_QP + kc * 128;
	const short4v lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_short4_ptr)(p));
	const short4v hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_short4_ptr)(p + 32));
	const short8 v = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
	return __builtin_bit_cast(half8, v);
}
// acc += A B^T over the sample chunks [kc0, kc0 + NK): A = rows of quad base qa, B = rows of quad base qb
template <int NK>
__device__ __forceinline__ void wgrad_tile(const unsigned char* tr, int qa, int qb, int kc0, float16v& acc) {
#pragma unroll
	for (int k = 0; k < NK; ++k) acc = N2_MFMA(row_operand(tr, qa, kc0 + k), row_operand(tr, qb, kc0 + k), acc);
}

// input operands (natural K order) of one 32-sample tile; column `col` of a matrix with n_cols columns
template <int IC>
__device__ __forceinline__ void load_tile_rows(const hf* __restrict__ X, uint32_t n_cols, uint32_t col, int g, half8 (&x)[IC]) {
	const uint32_t b = (8u * g * n_cols + col) * 2u;
#pragma unroll
	for (int c = 0; c < IC; ++c)
#pragma unroll
		for (int e = 0; e < 8; ++e) x[c][e] = *reinterpret_cast<const hf*>(reinterpret_cast<const char*>(X + (size_t)(16 * c + e) * n_cols) + b);
}

// Which rows of dL/dinput a launch stores: all of them, or only those its caller reads (rows that differ between the two
// halves of a wave turn into a predicate on the half, rows nobody reads cost no instruction)
enum : int {
	WG_DX_NONE = 0,
	WG_DX_ALL = 1,
	WG_DX_OUT_AND_NORMAL = 2,  // rows 0..15 and 35..37: the field's colour net (gradient of the SDF net's output and of the normal)
	WG_DX_ENCODING = 3         // rows 3..34: the field's SDF net (gradient of the encoding; positions are not optimised)
};
__device__ __forceinline__ constexpr bool wg_dx_row(int mode, int row, int in_w) {
	return row < in_w && (mode == WG_DX_ALL || (mode == WG_DX_OUT_AND_NORMAL && (row < 16 || (row >= 35 && row < 38))) ||
	                      (mode == WG_DX_ENCODING && row >= 3 && row < 35));
}

// A tail: work on the same samples that rides along with a launch.  The field hangs the preparation of its SDF net's
// backward on the colour net's kernel (N2FieldPrepTail, n2_common.h): that work streams 256 bytes of slopes per sample, and
// inside this kernel, whose waves wait for barriers and matrix results half of their time, it costs less than as a launch
// of its own between the two networks' kernels.
struct WgNoTail {
	static constexpr bool active = false;
};
// With the tail, the launch also takes the field's layouts: X holds a column's first N2_RGB_IN_PITCH values side by side
// (column c at X + N2_RGB_IN_PITCH c), and rows 0..15 of dL/dinput are written the same way (16 values per column, dX + 16 c); nothing else of
// dL/dinput is stored.
struct WgFieldPrepTail {
	static constexpr bool active = true;
	N2FieldPrepTail a;
};

template <int IC, int NH, int WANT_DX, bool SECOND, class Tail = WgNoTail>
__global__ void __launch_bounds__(MLP_BLOCK, 2) mlp_wgrad_kernel(const hf* __restrict__ W, const hf* __restrict__ X, uint32_t N, const hf* __restrict__ dY,
                                                                 int dy_aos, int dy_rows, hf* __restrict__ dX, float* __restrict__ partials,
                                                                 const hf* __restrict__ V, const hf* __restrict__ G2, int unit_row2,
                                                                 const uint32_t* __restrict__ x_index, uint32_t x_cols, float dy_gain, float dy_gain_inv,
                                                                 const hf* __restrict__ frag_image, const Tail tail = Tail()) {
	static_assert(!SECOND || NH == 1, "the second-order pass needs one hidden layer");
	static_assert(!Tail::active || (IC == 3 && NH == 2 && WANT_DX == WG_DX_OUT_AND_NORMAL), "the field's tail goes with the colour net");
	// dy_gain = 2^k, dy_gain_inv = 2^-k (first-order launches only).  The output gradient is multiplied by 2^k when it is
	// loaded and everything the launch hands on (dL/dinput, the weight-gradient slab) by 2^-k in fp32, so the chain between
	// them, whose matrices are rounded to fp16 for the matrix cores, works on values 2^k larger: an output gradient in the
	// subnormal range of fp16 (a loss scale of 128 over thousands of rays puts the colour rows there: steps of 6e-8 on values
	// near 2e-6) then loses nothing, the products with a power of two being exact.  2^0 leaves every value as it is.
	const float gain_inv = SECOND ? 1.f : dy_gain_inv;
	using M = FragMap<IC, NH>;
	constexpr int IN_W = 16 * IC, IN_MT = M::IN_MT;
	constexpr int N_PARAMS = MLP_WIDTH * IN_W + (NH - 1) * MLP_WIDTH * MLP_WIDTH + MLP_OUT * MLP_WIDTH;
	extern __shared__ __align__(16) unsigned char smem[];
	hf* F = reinterpret_cast<hf*>(smem);
	unsigned char* S = smem + (size_t)M::SEL * 1024;  // staging buffer behind the fragments
	// (frag_image: the fragments as a launch in front of this one has left them in global memory, M::SEL KiB; null: built here)
	if (frag_image) load_frags(F, frag_image, M::SEL);
	else build_frags<IC, NH>(F, W, M::SEL);
	const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, n = lane & 31, g = lane >> 5;
	const int mt = __builtin_amdgcn_readfirstlane(wave >> 1), nt = __builtin_amdgcn_readfirstlane(wave & 1);
	const uint32_t s_local = 32u * wave + n;
	unsigned char* const st_nat = S + s_local * 8u + 2u * g * WG_QP;
	unsigned char* const st_ch = S + s_local * 8u + (uint32_t)g * WG_QP;
	const int G = lane >> 4;
	const unsigned char* const tr = S + (4 * (G & 1) + (lane & 3)) * WG_QP + (8 * (G >> 1) + ((lane & 15) >> 2)) * 8;
	float16v gW0 = zero16(), gWh = zero16(), gWo = zero16();
	float var_acc = 0.f;  // tail: this lane's part of the variance gradient
	const uint32_t n_rounds = (N + WG_SAMPLES - 1) / WG_SAMPLES;
	for (uint32_t round = blockIdx.x; round < n_rounds; round += gridDim.x) {
		const uint32_t col_raw = round * WG_SAMPLES + s_local;
		const bool valid = col_raw < N;
		const uint32_t col = valid ? col_raw : N - 1u;
		// ---- the chain of this wave's 32 samples ----
		half8 x[IC], dy, h[NH][4];
		const uint32_t col_src = x_index ? min(x_index[col], x_cols - 1u) : col;  // the sample's column in X
		if constexpr (Tail::active) {
			// the field keeps the colour net's input sample-major (N2_RGB_IN_PITCH values per column, the rows behind them
			// are the padding's zeros): an operand is one 16-byte load
#pragma unroll
			for (int c = 0; c < IC; ++c)
				x[c] = 16 * c + 8 * g < (int)N2_RGB_IN_PITCH ? *reinterpret_cast<const half8*>(X + (size_t)col_src * N2_RGB_IN_PITCH + 16 * c + 8 * g) : zero8();
		} else {
			load_tile_rows<IC>(X, x_index ? x_cols : N, col_src, g, x);
		}
		if (dy_aos) {
			dy = *reinterpret_cast<const half8*>(dY + (size_t)col * MLP_OUT + 8 * g);
		} else {
#pragma unroll
			for (int e = 0; e < 8; ++e) dy[e] = dY[(size_t)(8 * g + e) * N + col];
		}
		const half8 dy_all = dy;  // tail: all 16 rows of the output gradient
#pragma unroll
		for (int e = 0; e < 8; ++e)
			if (!valid || 8 * g + e >= dy_rows) dy[e] = (hf)0;
		if constexpr (!SECOND) {
			const hf gain = (hf)dy_gain;
#pragma unroll
			for (int e = 0; e < 8; ++e) dy[e] = dy[e] * gain;
		}
		hidden_S<IC, NH>(F, lane, x, h);
		half8 dh[NH][4];
#pragma unroll
		for (int t = 0; t < 2; ++t)
			mask_pack(N2_MFMA(frag(F, M::WOT + t, lane), dy, zero16()), h[NH - 1][2 * t], h[NH - 1][2 * t + 1], dh[NH - 1][2 * t], dh[NH - 1][2 * t + 1]);
#pragma unroll
		for (int k = NH - 1; k >= 1; --k)
#pragma unroll
			for (int t = 0; t < 2; ++t) {
				float16v a = zero16();
#pragma unroll
				for (int c = 0; c < 4; ++c) a = N2_MFMA(frag(F, M::WHT + (k - 1) * 8 + t * 4 + c, lane), dh[k][c], a);
				mask_pack(a, h[k - 1][2 * t], h[k - 1][2 * t + 1], dh[k - 1][2 * t], dh[k - 1][2 * t + 1]);
			}
		hf dn[2] = {(hf)0, (hf)0};  // tail: g = 0: row 35; g = 1: rows 36, 37 of dL/dinput
		if (WANT_DX != WG_DX_NONE) {
#pragma unroll
			for (int t = 0; t < IN_MT; ++t) {
				float16v d = zero16();
#pragma unroll
				for (int c = 0; c < 4; ++c) d = N2_MFMA(frag(F, M::W0T + t * 4 + c, lane), dh[0][c], d);
#pragma unroll
				for (int r = 0; r < 16; ++r) d[r] *= gain_inv;
				if constexpr (Tail::active) {
					// row 0 also takes the direct gradient of the SDF output (row 3 of dL/doutput); rows 35..37 are dL/dnormal
					if (t == 0 && g == 0) d[0] = (float)((hf)d[0] + dy_all[3]);
					if (t == 1) { dn[0] = (hf)(g == 0 ? d[3] : d[0]); dn[1] = (hf)d[1]; }
					// rows 0..15 go out sample-major (16 values per column, the SDF net's output gradient): the lane holds
					// rows 4 g .. 4 g + 3 and 8 + 4 g .. 8 + 4 g + 3; rows 35..37 stay in registers (dn)
					if (t == 0 && valid) {
						const half4v lo = {(hf)d[0], (hf)d[1], (hf)d[2], (hf)d[3]}, hi = {(hf)d[4], (hf)d[5], (hf)d[6], (hf)d[7]};
						hf* o = dX + (size_t)col * MLP_OUT + 4 * g;
						*reinterpret_cast<half4v*>(o) = lo;
						*reinterpret_cast<half4v*>(o + 8) = hi;
					}
				}
				if (!Tail::active && valid) {
#pragma unroll
					for (int r = 0; r < 16; ++r) {
						const int row = 32 * t + 8 * (r >> 2) + (r & 3);  // + 4 g
						const bool lo = wg_dx_row(WANT_DX, row, IN_W), hi = wg_dx_row(WANT_DX, row + 4, IN_W);
						if (lo && hi) dX[(size_t)(row + 4 * g) * N + col] = (hf)d[r];
						else if (lo) { if (g == 0) dX[(size_t)row * N + col] = (hf)d[r]; }
						else if (hi) { if (g == 1) dX[(size_t)(row + 4) * N + col] = (hf)d[r]; }
					}
				}
			}
		}
		half8 v[IC], gg, sa[4], sb[4];
		if constexpr (SECOND) {
			load_tile_rows<IC>(V, N, col, g, v);
			if (unit_row2 >= 0) {
#pragma unroll
				for (int e = 0; e < 8; ++e) gg[e] = (8 * g + e == unit_row2) ? (hf)1 : (hf)0;
			} else {
#pragma unroll
				for (int e = 0; e < 8; ++e) gg[e] = G2[(size_t)(8 * g + e) * N + col];
			}
			if (!valid) {
				gg = zero8();
#pragma unroll
				for (int c = 0; c < IC; ++c) v[c] = zero8();
			}
			// a = m * (W_0 v),  b = m * (W_out^T g); m = the sign of the hidden layer
#pragma unroll
			for (int t = 0; t < 2; ++t) {
				float16v a = zero16();
#pragma unroll
				for (int c = 0; c < IC; ++c) a = N2_MFMA(frag(F, M::W0 + t * IC + c, lane), v[c], a);
				mask_pack(a, h[0][2 * t], h[0][2 * t + 1], sa[2 * t], sa[2 * t + 1]);
				mask_pack(N2_MFMA(frag(F, M::WOT + t, lane), gg, zero16()), h[0][2 * t], h[0][2 * t + 1], sb[2 * t], sb[2 * t + 1]);
			}
		}
		// ---- stage 1: dW_out = dy h_last^T (+ g a^T) ----
		// quads: dy 0..3 | h_last 4..19 | g 20..23 | a 24..39
		stage_natural(st_nat, dy);
#pragma unroll
		for (int c = 0; c < 4; ++c) stage_chained(st_ch + (4 + 4 * c) * WG_QP, h[NH - 1][c]);
		if constexpr (SECOND) {
			stage_natural(st_nat + 20 * WG_QP, gg);
#pragma unroll
			for (int c = 0; c < 4; ++c) stage_chained(st_ch + (24 + 4 * c) * WG_QP, sa[c]);
		}
		__syncthreads();
		if constexpr (SECOND) {
			// waves 0, 1: dy h^T; waves 2, 3: g a^T; column tile nt, all samples
			if (mt == 0) wgrad_tile<8>(tr, 0, 4 + 8 * nt, 0, gWo);
			else wgrad_tile<8>(tr, 20, 24 + 8 * nt, 0, gWo);
		} else {
			// column tile nt, samples of half mt
			wgrad_tile<4>(tr, 0, 4 + 8 * nt, 4 * mt, gWo);
		}
		__syncthreads();
		// ---- hidden matrices: dW_k = dh_k h_{k-1}^T ----
#pragma unroll
		for (int k = NH - 1; k >= 1; --k) {
#pragma unroll
			for (int c = 0; c < 4; ++c) {
				stage_chained(st_ch + (4 * c) * WG_QP, dh[k][c]);
				stage_chained(st_ch + (16 + 4 * c) * WG_QP, h[k - 1][c]);
			}
			__syncthreads();
			wgrad_tile<8>(tr, 8 * mt, 16 + 8 * nt, 0, gWh);
			__syncthreads();
		}
		// ---- first matrix: dW_0 = dh_0 x^T (+ b v^T) ----
		// quads: dh_0 (b) 0..15 | x (v) 16..16+4 IC-1; a column tile that the input does not fill reads what lies behind
		// (stale values of an earlier stage), which only reaches accumulator columns that are never written out
#pragma unroll
		for (int c = 0; c < 4; ++c) stage_chained(st_ch + (4 * c) * WG_QP, dh[0][c]);
#pragma unroll
		for (int c = 0; c < IC; ++c) stage_natural(st_nat + (16 + 4 * c) * WG_QP, x[c]);
		uint4 sl[Tail::active ? 8 : 1];
		if constexpr (Tail::active) {
			// the slopes of this lane's 8 levels (level 4 (j / 2) + 2 g + j % 2), in flight during the last products
#pragma unroll
			for (int j = 0; j < 8; ++j) {
				const uint32_t level = 4u * (j >> 1) + 2u * g + (j & 1);
				sl[j] = reinterpret_cast<const uint4*>(tail.a.slopes)[(size_t)(2u * level < tail.a.enc_w ? level : 0u) * tail.a.n_src + col_src];
			}
		}
		__syncthreads();
		if (nt < IN_MT) wgrad_tile<8>(tr, 8 * mt, 16 + 8 * nt, 0, gW0);
		__syncthreads();
		if constexpr (Tail::active) {
			// dL/dnormal = row 35..37 of dL/dinput + rows 4..6 of dL/doutput / ek_batch + rows 8..10 of dL/doutput; its pieces
			// sit in the two halves of the wave: g = 0 holds dn[0] and rows 4..6, g = 1 holds dn[0..1] (rows 36, 37) and rows 8..10
			auto pk = [](hf a, hf b) { return (uint32_t)__builtin_bit_cast(unsigned short, a) | ((uint32_t)__builtin_bit_cast(unsigned short, b) << 16); };
			auto lo16 = [](uint32_t w) { return (float)__builtin_bit_cast(hf, (unsigned short)(w & 0xFFFFu)); };
			auto hi16 = [](uint32_t w) { return (float)__builtin_bit_cast(hf, (unsigned short)(w >> 16)); };
			const uint32_t m0 = g == 0 ? pk(dn[0], dy_all[4]) : pk(dn[0], dn[1]);
			const uint32_t m1 = g == 0 ? pk(dy_all[5], dy_all[6]) : pk(dy_all[0], dy_all[1]);
			const uint32_t m2 = g == 0 ? 0u : pk(dy_all[2], (hf)0);
			const uint32_t o0 = (uint32_t)__shfl_xor((int)m0, 32), o1 = (uint32_t)__shfl_xor((int)m1, 32), o2 = (uint32_t)__shfl_xor((int)m2, 32);
			const uint32_t a0 = g == 0 ? m0 : o0, a1 = g == 0 ? m1 : o1;             // what the lower half holds
			const uint32_t b0 = g == 0 ? o0 : m0, b1 = g == 0 ? o1 : m1, b2 = g == 0 ? o2 : m2;  // what the upper half holds
			float vv[3] = {lo16(a0), lo16(b0), hi16(b0)};
			const float r4[3] = {hi16(a0), lo16(a1), hi16(a1)}, r8[3] = {lo16(b1), hi16(b1), lo16(b2)};
#pragma unroll
			for (int d = 0; d < 3; ++d) {
				vv[d] += r4[d] / tail.a.ek_batch;
				vv[d] += r8[d];
			}
			if (valid) {
				if (g == 0) {
					var_acc += (float)dy_all[7];
#pragma unroll
					for (int d = 0; d < 3; ++d) {
						tail.a.v[(size_t)d * N + col] = vv[d];
						reinterpret_cast<hf*>(tail.a.d_density_in)[(size_t)d * N + col] = (hf)vv[d];
					}
				}
				// rows 3.. of the SDF net's second-order input: the encoding's dL_ddLdoutput = J v
#pragma unroll
				for (int j = 0; j < 8; ++j) {
					const uint32_t level = 4u * (j >> 1) + 2u * g + (j & 1);
					if (2u * level < tail.a.enc_w) {
						float m[6];
						const float unit = n2_slopes_unpack(sl[j], m) * tail.a.scale[level];
						hf* o = reinterpret_cast<hf*>(tail.a.d_density_in) + (size_t)(3 + 2 * level) * N + col;
						o[0] = (hf)((m[0] * vv[0] + m[1] * vv[1] + m[2] * vv[2]) * unit);
						o[N] = (hf)((m[3] * vv[0] + m[4] * vv[1] + m[5] * vv[2]) * unit);
					}
				}
			}
		}
		if constexpr (SECOND) {
#pragma unroll
			for (int c = 0; c < 4; ++c) stage_chained(st_ch + (4 * c) * WG_QP, sb[c]);
#pragma unroll
			for (int c = 0; c < IC; ++c) stage_natural(st_nat + (16 + 4 * c) * WG_QP, v[c]);
			__syncthreads();
			if (nt < IN_MT) wgrad_tile<8>(tr, 8 * mt, 16 + 8 * nt, 0, gW0);
			__syncthreads();
		}
	}
	// ---- the workgroup's slab: an fp32 image of the parameters in LDS, summed over the waves that share a tile ----
	float* Wl = reinterpret_cast<float*>(smem);
	__syncthreads();  // every wave is done with the fragments the image overlays
	if (nt < IN_MT) {
#pragma unroll
		for (int r = 0; r < 16; ++r)
			if (32 * nt + n < IN_W) Wl[(32 * mt + drow(r, g)) * IN_W + 32 * nt + n] = gW0[r] * gain_inv;
	}
	if (NH > 1) {
#pragma unroll
		for (int r = 0; r < 16; ++r) Wl[MLP_WIDTH * IN_W + (32 * mt + drow(r, g)) * MLP_WIDTH + 32 * nt + n] = gWh[r] * gain_inv;
	}
	constexpr int OFF_O = MLP_WIDTH * IN_W + (NH - 1) * MLP_WIDTH * MLP_WIDTH;
	if (mt == 0) {
#pragma unroll
		for (int r = 0; r < 16; ++r)
			if (drow(r, g) < MLP_OUT) Wl[OFF_O + drow(r, g) * MLP_WIDTH + 32 * nt + n] = gWo[r] * gain_inv;
	}
	__syncthreads();
	if (mt == 1) {
#pragma unroll
		for (int r = 0; r < 16; ++r)
			if (drow(r, g) < MLP_OUT) Wl[OFF_O + drow(r, g) * MLP_WIDTH + 32 * nt + n] += gWo[r] * gain_inv;
	}
	__syncthreads();
	float* slab = partials + (size_t)blockIdx.x * N_PARAMS;
	for (int i = threadIdx.x; i < N_PARAMS; i += MLP_BLOCK) slab[i] = Wl[i];
	if constexpr (Tail::active) {
		// the workgroup's part of the variance gradient (row 7 of dL/doutput), summed in a fixed order
#pragma unroll
		for (int o = 32; o > 0; o >>= 1) var_acc += __shfl_xor(var_acc, o);
		__syncthreads();
		if (lane == 0) Wl[wave] = var_acc;
		__syncthreads();
		if (threadIdx.x == 0) tail.a.var_part[blockIdx.x] = (Wl[0] + Wl[1]) + (Wl[2] + Wl[3]);
	}
}

// dynamic LDS of the kernel: fragments, then the staging buffer (40 quad rows with the second-order pass, else 32)
template <int IC, int NH, bool SECOND>
constexpr size_t mlp_wgrad_lds() {
	return (size_t)FragMap<IC, NH>::SEL * 1024 + (size_t)(SECOND ? 40 : 32) * WG_QP;
}
