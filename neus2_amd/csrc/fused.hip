// Fused forward of the NeuS field for gfx950 (counterpart of NerfNetwork::forward_impl, nerf_network.h:132-315, and of
// NerfNetwork::sdf / density, :643-726).
//
// Training forward = two kernels.
//  * field_gather_kernel walks the grid LEVEL-MAJOR (one workgroup = one level x 256 samples, all workgroups of a
//    level next to each other in time), so that the level being read (<= 2 MiB) stays resident in every L2; a
//    sample-major walk touches all 24 MiB of tables at once and three of five L2 requests miss.  It writes the
//    features into the SDF net's input rows and the level's slopes (the Jacobian of the encoding without the level's
//    scale factor) as a 16-byte block-float per sample and level (n2_slopes_pack), against 24 bytes of fp32.
//  * field_fused_forward_kernel then takes 32 samples per wave through everything else without touching memory in
//    between: SDF net forward, the gradient of its first output w.r.t. its input, the normal (that gradient contracted
//    with the slopes), the direction encoding, the colour net and the 16 output rows.
// Inference (sdf / density) is the second kernel alone with the gather inside it: positions that arrive in lattice or
// near-lattice order hit cached lines whatever the order of the levels.
//
// Layout of the network kernel.  Lane (n, g), n = lane % 32, g = lane / 32, works for sample b0 + n.  In the MFMA
// layouts (see mlp_device.h) lane (n, g)
// holds, of a B operand in chained order, the rows {16c + 4g + 0..3, 16c + 8 + 4g + 0..3} of chunk c, and of a D tile
// the rows {8q + 4g + 0..3}, q = 0..3.  With the encoding's features as rows 0..31 of the SDF net's input (row
// 2 l + f for feature f of level l; the three centred coordinates follow as rows 32..34) both sets are the levels
//     l(j, g) = 4 (j / 2) + 2 g + j % 2,   j = 0..7,
// so a lane loads (or gathers) exactly those eight levels of its sample: the features are its B operand registers,
// the rows of d sdf / d encoding come back to it in the D tile of the input-gradient product, and the contraction
// with the slopes it holds (normal = J^T g) is lane-local up to one exchange between the two halves of the wave.  The permutation of the input rows is folded into the weight fragments, which are built once per
// workgroup in LDS.
#include "n2_common.h"

#include "grid_device.h"
#include "mlp_device.h"

constexpr int FF_BLOCK = 256;  // 4 waves
constexpr uint32_t FF_LEVELS = 16;  // levels the lane layout covers

// fragment numbers (64 lanes x 16 bytes each)
enum : int {
	S_W0 = 0,    // [mt][c]  SDF net W_0 rows 32 mt + n; c = 0, 1: feature rows in chained order, c = 2: centred coordinates
	S_WO = 6,    // [c]      SDF net W_out rows n < 16, chained K
	FF_SDF_COUNT = 10,
	S_W0T = 10,  // [mt][c]  SDF net W_0^T, row = internal input row 32 mt + n, chained K over the neurons
	S_DH = 18,   // [c]      row 0 of W_out as a chained B operand (every column the same): d sdf / d hidden before the mask
	C_W0 = 22,   // [mt][c]  colour net W_0 rows 32 mt + n; c = 0 chained (SDF-net outputs), c = 1, 2 natural
	C_WH = 28,   // [mt][c]  colour net hidden matrix, chained K
	C_WO = 36,   // [c]      colour net W_out rows n < 16, chained K
	FF_COUNT = 40
};

// per-level constants as the kernel reads them: one 16-byte LDS entry per level
struct FusedLevels {
	float scale[FF_LEVELS];
	uint32_t res[FF_LEVELS], entries[FF_LEVELS], offset[FF_LEVELS];  // offset in entries
	uint32_t hash_mask;      // bit l: level l is hashed (power-of-two table), else dense
	uint32_t active_levels;  // levels >= this are switched off (or do not exist)
};

struct FusedArgs {
	FusedLevels lv;
	const __half2* table;   // grid parameters
	const hf* sdf_w;        // SDF net weights: W_0 [64][sdf_in_w], W_out [16][64]
	const hf* rgb_w;        // colour net weights: W_0 [64][48], W_1 [64][64], W_out [16][64]
	const hf* variance;
	uint32_t sdf_in_w, enc_w;
	float sdf_bias;
	uint32_t N;
	const uint32_t* live;   // or null: only samples below min(*live, N) are evaluated (N stays the column count of the matrices)
	// A listed pass (full field only; list null: off) evaluates the samples begin .. begin + counts[round] of the
	// coordinates, begin = counts[0] + ... + counts[round - 1]: sample c writes row list[c] of the output, and everything
	// the backward reads is stored at column c.
	const uint32_t* list;
	const uint32_t* counts;
	uint32_t round, n_levels;
	// full field: the weight fragments of the network kernel as one image in global memory (FF_COUNT KiB; null: every
	// workgroup builds them from the weights).  The gather launch in front of the network kernel writes it.
	hf* frags;
	const float* pos;       // coordinate d of sample i at pos[i * ps + d * ds]; null: sample i is point lat.first + i of a lattice
	uint32_t ps, ds;
	N2Lattice lat;
	const float* coords;    // full field: [N][7] NerfCoordinate (direction at 4..6)
	// full field: what the backward pass reads, and the output
	hf* sdf_in;             // [sdf_in_w][N]  rows 0..2 centred coordinates, 3.. features
	float* xyz_rows;        // [3][N]
	uint4* slopes;          // [n_levels][N]: d feature / d position of each level (2 x 3 values, see n2_slopes_pack), without the level's scale
	hf* dsdf_din;           // [sdf_in_w][N]
	hf* rgb_in;             // [N][N2_RGB_IN_PITCH]: sample-major
	hf* output;             // [N][16]
	// SDF only
	hf* sdf_out;            // [16][N] or null
	float* row0;            // [row0_n] fp32 copy of row 0 of the first row0_n samples, or null
	uint32_t row0_n;
	int density;            // row 0 becomes the logistic density
};

__device__ __forceinline__ hf h_or_zero(const hf* W, bool ok, size_t at) { return ok ? W[at] : (hf)0; }

// internal input row of the SDF net -> column of W_0 (or -1): rows 0..31 are features, 32..34 the coordinates
__device__ __forceinline__ int sdf_col(int row, uint32_t enc_w) {
	if (row < 32) return (uint32_t)row < enc_w ? 3 + row : -1;
	return row < 35 ? row - 32 : -1;
}
__device__ __forceinline__ int chained_k(int c, int g, int e) { return 16 * c + 4 * g + (e & 3) + ((e >> 2) << 3); }

// lane l's 16 bytes of fragment f
__device__ __forceinline__ half8 fused_frag_value(const FusedArgs& a, int f, int l) {
	const hf* W0s = a.sdf_w;
	const int ld_s = (int)a.sdf_in_w;
	const hf* W1s = W0s + MLP_WIDTH * ld_s;
	const hf* W0c = a.rgb_w;
	const hf* Whc = W0c + MLP_WIDTH * 48;
	const hf* Woc = Whc + MLP_WIDTH * MLP_WIDTH;
	{
		const int n = l & 31, g = l >> 5;
		half8 v = zero8();
		if (f < S_WO) {
			const int mt = f / 3, c = f % 3, row = 32 * mt + n;
#pragma unroll
			for (int e = 0; e < 8; ++e) {
				const int col = c < 2 ? sdf_col(chained_k(c, g, e), a.enc_w) : sdf_col(32 + 8 * g + e, a.enc_w);
				v[e] = h_or_zero(W0s, col >= 0, (size_t)row * ld_s + (col >= 0 ? col : 0));
			}
		} else if (f < S_W0T) {
			if (n < MLP_OUT) v = wfrag_chained(W1s, MLP_WIDTH, n, f - S_WO, g);
		} else if (f < S_DH) {
			const int q = f - S_W0T, mt = q >> 2, c = q & 3, col = sdf_col(32 * mt + n, a.enc_w);
#pragma unroll
			for (int e = 0; e < 8; ++e) v[e] = h_or_zero(W0s, col >= 0, (size_t)chained_k(c, g, e) * ld_s + (col >= 0 ? col : 0));
		} else if (f < C_W0) {
#pragma unroll
			for (int e = 0; e < 8; ++e) v[e] = W1s[chained_k(f - S_DH, g, e)];
		} else if (f < C_WH) {
			const int q = f - C_W0, mt = q / 3, c = q % 3;
			v = c == 0 ? wfrag_chained(W0c, 48, 32 * mt + n, 0, g) : wfrag_natural(W0c, 48, 32 * mt + n, c, g);
		} else if (f < C_WO) {
			const int q = f - C_WH;
			v = wfrag_chained(Whc, MLP_WIDTH, 32 * (q >> 2) + n, q & 3, g);
		} else {
			if (n < MLP_OUT) v = wfrag_chained(Woc, MLP_WIDTH, n, f - C_WO, g);
		}
		return v;
	}
}

__device__ __forceinline__ void build_fused_frags(hf* F, const FusedArgs& a, int count) {
	for (int idx = threadIdx.x; idx < count * 64; idx += FF_BLOCK) *reinterpret_cast<half8*>(F + (size_t)idx * 8) = fused_frag_value(a, idx >> 6, idx & 63);
	__syncthreads();
}
// the same fragments copied from the image a gather launch left in global memory: 16 consecutive bytes per lane instead
// of two-byte picks all over the weight matrices (5 to 7 us of a network launch went into those)
__device__ __forceinline__ void load_fused_frags(hf* F, const hf* __restrict__ image, int count) {
	for (int idx = threadIdx.x; idx < count * 64; idx += FF_BLOCK) *reinterpret_cast<half8*>(F + (size_t)idx * 8) = *reinterpret_cast<const half8*>(image + (size_t)idx * 8);
	__syncthreads();
}
// Workgroups FRAG_BLOCKS .. of a gather launch (behind those that gather) write the image: the network kernel's fragments,
// then those of the backward's weight-gradient kernels (colour net: FragMap<3, 2>; SDF net with 48 inputs: FragMap<3, 1>).
constexpr uint32_t BWD_RGB_FRAGS = FragMap<3, 2>::SEL, BWD_SDF_FRAGS = FragMap<3, 1>::SEL;
static_assert(FF_COUNT * 1024 == N2_FUSED_FRAG_FORWARD && BWD_RGB_FRAGS * 1024 == N2_FUSED_FRAG_RGB && BWD_SDF_FRAGS * 1024 == N2_FUSED_FRAG_SDF,
              "the image's parts as n2_common.h sizes them");
constexpr uint32_t FG_BLOCK = 256;  // threads of a gather workgroup (128: the gather 1.8 us shorter, the step 5 us longer; 512: +2 / +5; 1024: +11 / +11)
constexpr uint32_t FRAG_BLOCKS = ((FF_COUNT + BWD_RGB_FRAGS + BWD_SDF_FRAGS) * 64 + FG_BLOCK - 1) / FG_BLOCK;
__device__ __forceinline__ void write_frag_image(const FusedArgs& a, uint32_t block) {
	const uint32_t idx = block * FG_BLOCK + threadIdx.x;
	half8* at = reinterpret_cast<half8*>(a.frags) + idx;
	if (idx < (uint32_t)FF_COUNT * 64u) {
		*at = fused_frag_value(a, (int)(idx >> 6), (int)(idx & 63u));
	} else if (idx < (FF_COUNT + BWD_RGB_FRAGS) * 64u) {
		const uint32_t i = idx - FF_COUNT * 64u;
		*at = mlp_frag_value<3, 2>(a.rgb_w, (int)(i >> 6), (int)(i & 63u));
	} else if (idx < (FF_COUNT + BWD_RGB_FRAGS + BWD_SDF_FRAGS) * 64u && a.sdf_in_w == 48u) {
		const uint32_t i = idx - (FF_COUNT + BWD_RGB_FRAGS) * 64u;
		*at = mlp_frag_value<3, 1>(a.sdf_w, (int)(i >> 6), (int)(i & 63u));
	}
}

// ----------------------------------------------------------------------------
// gather of one (sample, level) item
// ----------------------------------------------------------------------------
struct LaneLevel {
	float scale;
	uint32_t res, entries, offset;  // offset in entries
	bool hashed;
};

// byte offsets of the 8 corner entries in the table (corner k: +1 on dimension d iff bit d of k is set)
template <int KIND>  // 0: every lane dense, 1: every lane hashed, 2: mixed
__device__ __forceinline__ void corner_offsets(const LaneLevel& L, const uint32_t (&c)[3], uint32_t (&boff)[8]) {
	uint32_t hx[2], hyz[4], dx[2], dyz[4];
	if (KIND != 0) {
		const uint32_t mask = L.entries - 1u;
		const uint32_t y0 = c[1] * 2654435761u, y1 = y0 + 2654435761u, z0 = c[2] * 805459861u, z1 = z0 + 805459861u;
		hyz[0] = (y0 ^ z0) & mask; hyz[1] = (y1 ^ z0) & mask; hyz[2] = (y0 ^ z1) & mask; hyz[3] = (y1 ^ z1) & mask;
		hx[0] = c[0] & mask; hx[1] = (c[0] + 1u) & mask;
	}
	if (KIND != 1) {
		const uint32_t r = L.res;
		dx[0] = min(c[0], r); dx[1] = min(c[0] + 1u, r);
		const uint32_t y0 = min(c[1], r) * r, y1 = min(c[1] + 1u, r) * r, z0 = min(c[2], r) * r * r, z1 = min(c[2] + 1u, r) * r * r;
		dyz[0] = y0 + z0; dyz[1] = y1 + z0; dyz[2] = y0 + z1; dyz[3] = y1 + z1;
	}
#pragma unroll
	for (int k = 0; k < 8; ++k) {
		uint32_t ih = 0, id = 0;
		if (KIND != 0) ih = hx[k & 1] ^ hyz[k >> 1];
		if (KIND != 1) {
			id = dx[k & 1] + dyz[k >> 1];
			id = min(id, id - L.entries);  // one conditional subtraction stands in for the modulo (unsigned wrap-around)
		}
		const uint32_t i = KIND == 0 ? id : KIND == 1 ? ih : (L.hashed ? ih : id);
		boff[k] = (L.offset + i) << 2;
	}
}

struct Item {
	uint32_t raw[8];
	float w[3];
	float scale;  // 0 for a switched-off level
};

// J: the lane's step; its level is l = 4 (J / 2) + 2 g + J % 2.  LV: the level constants in LDS.
template <int J>
__device__ __forceinline__ void item_fetch(const uint4* LV, uint32_t hash_mask, uint32_t active, const __half2* __restrict__ table, int g,
                                           const float (&p)[3], Item& it) {
	constexpr int lo = 4 * (J >> 1) + (J & 1), hi = lo + 2;
	const uint4 q = LV[lo + 2 * g];
	LaneLevel L;
	L.scale = __uint_as_float(q.x); L.res = q.y; L.entries = q.z; L.offset = q.w;
	L.hashed = g ? ((hash_mask >> hi) & 1u) : ((hash_mask >> lo) & 1u);
	const bool off = (uint32_t)(lo + 2 * g) >= active;
	uint32_t c[3], boff[8];
#pragma unroll
	for (int d = 0; d < 3; ++d) n2_locate(p[d], L.scale, it.w[d], c[d]);
	it.scale = off ? 0.f : L.scale;
	const bool h_lo = (hash_mask >> lo) & 1u, h_hi = (hash_mask >> hi) & 1u;  // wave-uniform
	if (h_lo && h_hi) corner_offsets<1>(L, c, boff);
	else if (!h_lo && !h_hi) corner_offsets<0>(L, c, boff);
	else corner_offsets<2>(L, c, boff);
	const char* base = reinterpret_cast<const char*>(table);
#pragma unroll
	for (int k = 0; k < 8; ++k) {
		if (off) boff[k] = 0;  // a switched-off level reads entry 0 and ignores it
		it.raw[k] = *reinterpret_cast<const uint32_t*>(base + boff[k]);
	}
}

__device__ __forceinline__ float2 h2f(uint32_t raw) {
	const half2v h = __builtin_bit_cast(half2v, raw);
	return make_float2((float)h[0], (float)h[1]);
}

// trilinear value and (with WANT_J) Jacobian of both features of one level
template <bool WANT_J>
__device__ __forceinline__ void item_finish(const Item& it, float (&feat)[2], float (&J)[2][3]) {
	float2 v[8];
#pragma unroll
	for (int k = 0; k < 8; ++k) v[k] = h2f(it.raw[k]);
	const float wx = it.w[0], wy = it.w[1], wz = it.w[2], ux = 1.f - wx, uy = 1.f - wy, uz = 1.f - wz;
	const float w00 = uy * uz, w10 = wy * uz, w01 = uy * wz, w11 = wy * wz;
	float s[2][2], ty[2][2], tz[2][2];  // [x plane][feature]
#pragma unroll
	for (int b = 0; b < 2; ++b) {
		const float2 a0 = v[b], a1 = v[b + 2], a2 = v[b + 4], a3 = v[b + 6];
		s[b][0] = fmaf(w00, a0.x, fmaf(w10, a1.x, fmaf(w01, a2.x, w11 * a3.x)));
		s[b][1] = fmaf(w00, a0.y, fmaf(w10, a1.y, fmaf(w01, a2.y, w11 * a3.y)));
		if (WANT_J) {
			ty[b][0] = fmaf(uz, a1.x - a0.x, wz * (a3.x - a2.x));
			ty[b][1] = fmaf(uz, a1.y - a0.y, wz * (a3.y - a2.y));
			tz[b][0] = fmaf(uy, a2.x - a0.x, wy * (a3.x - a1.x));
			tz[b][1] = fmaf(uy, a2.y - a0.y, wy * (a3.y - a1.y));
		}
	}
	const float sc = it.scale, on = it.scale != 0.f ? 1.f : 0.f;
#pragma unroll
	for (int f = 0; f < 2; ++f) {
		feat[f] = fmaf(ux, s[0][f], wx * s[1][f]) * on;
		if (WANT_J) {
			J[f][0] = (s[1][f] - s[0][f]) * sc;
			J[f][1] = fmaf(ux, ty[0][f], wx * ty[1][f]) * sc;
			J[f][2] = fmaf(ux, tz[0][f], wx * tz[1][f]) * sc;
		}
	}
}

// degree-4 real spherical harmonics of the direction 2 d - 1 (tcnn's SphericalHarmonics encoding, nerf_network.h:251-257)
__device__ __forceinline__ void sh4(float x, float y, float z, float* o) {
	const float xy = x * y, xz = x * z, yz = y * z, x2 = x * x, y2 = y * y, z2 = z * z;
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
}

// ----------------------------------------------------------------------------
// level-major gather: features into the SDF net's input rows, slopes as fp16
// ----------------------------------------------------------------------------

// FULL: positions from the [N][7] coordinates, slopes and the coordinate rows are written; else positions with the
// strides (ps, ds) and the feature rows only (inference on points in no particular order).
// one (sample, level) item: the sample's coordinates are row `src` of the input, what it writes goes to column i
template <bool FULL>
__device__ __forceinline__ void gather_item(const FusedArgs& a, uint32_t level, uint32_t i, uint32_t src) {
	const uint32_t N = a.N;
	// (full field: the positions from the coordinate rows, or from three rows of their own when the caller has them: a wave
	// then reads two lines per coordinate instead of fourteen)
	const bool rows = FULL && a.pos == nullptr;
	const float* q = rows ? a.coords + (size_t)src * 7 : a.pos + (size_t)src * a.ps;
	const size_t qs = rows ? 1 : a.ds;
	const float p[3] = {q[0], q[qs], q[2 * qs]};
	if (FULL && level == 0) {
#pragma unroll
		for (int d = 0; d < 3; ++d) {
			a.sdf_in[(size_t)d * N + i] = (hf)p[d] - (hf)0.5f;
			a.xyz_rows[(size_t)d * N + i] = p[d];
		}
	}
	float feat[2] = {0.f, 0.f}, J[2][3] = {{0.f, 0.f, 0.f}, {0.f, 0.f, 0.f}};
	if (level < a.lv.active_levels) {  // a switched-off level: zero features, zero slopes
		LaneLevel L;
		L.scale = a.lv.scale[level]; L.res = a.lv.res[level]; L.entries = a.lv.entries[level]; L.offset = a.lv.offset[level];
		L.hashed = (a.lv.hash_mask >> level) & 1u;
		Item it;
		uint32_t c[3], boff[8];
#pragma unroll
		for (int d = 0; d < 3; ++d) n2_locate(p[d], L.scale, it.w[d], c[d]);
		it.scale = 1.f;  // slopes are stored without the level's scale factor
		const char* base = reinterpret_cast<const char*>(a.table);
		if (L.hashed) corner_offsets<1>(L, c, boff);
		else corner_offsets<0>(L, c, boff);
#pragma unroll
		for (int k = 0; k < 8; ++k) it.raw[k] = *reinterpret_cast<const uint32_t*>(base + boff[k]);
		item_finish<FULL>(it, feat, J);
	}
	a.sdf_in[(size_t)(3 + 2 * level) * N + i] = (hf)feat[0];
	a.sdf_in[(size_t)(4 + 2 * level) * N + i] = (hf)feat[1];
	if (FULL) {
		const float six[6] = {J[0][0], J[0][1], J[0][2], J[1][0], J[1][1], J[1][2]};
		a.slopes[(size_t)level * N + i] = n2_slopes_pack(six);
	}
}

// first column and number of samples of a listed pass
__device__ __forceinline__ void listed_range(const FusedArgs& a, uint32_t& begin, uint32_t& count) {
	begin = 0;
	for (uint32_t q = 0; q < a.round; ++q) begin += a.counts[q];
	count = min(a.counts[a.round], a.N - min(begin, a.N));
}

// The listed pass: the number of samples is known on the device only.  The launch has est_tiles workgroups per level, level-
// major like the other kernel's; workgroup t of a level takes the tiles t, t + est_tiles, ...: any estimate gives the right
// result, a good one gives every workgroup one tile.  (A fixed number of workgroups that walk all items by a stride is
// 1.6 times slower beside the trainer's sample generator: its waves keep some of them from starting until others have
// finished their whole share.)
__global__ void __launch_bounds__(FG_BLOCK) field_gather_list_kernel(const FusedArgs a, uint32_t est_tiles) {
	__builtin_amdgcn_s_setprio(3);
	const uint32_t level = blockIdx.x / est_tiles;
	if (level >= a.n_levels) {  // the network kernel's weight fragments (round 0 only)
		write_frag_image(a, blockIdx.x - a.n_levels * est_tiles);
		return;
	}
	uint32_t begin, count;
	listed_range(a, begin, count);
	const uint32_t tiles = (count + FG_BLOCK - 1) / FG_BLOCK;
	for (uint32_t tile = blockIdx.x - level * est_tiles; tile < tiles; tile += est_tiles) {
		const uint32_t j = tile * FG_BLOCK + threadIdx.x;
		if (j < count) gather_item<true>(a, level, begin + j, begin + j);
	}
}

template <bool FULL>
__global__ void __launch_bounds__(FG_BLOCK) field_gather_kernel(const FusedArgs a, uint32_t tiles) {
	// level-major workgroup ids: the workgroups that run at one time work on one or two levels, whose tables stay in every
	// L2.  The launch is bound by the L2s' request rate: 10 M requests for the training step's 2.6e5 ray-ordered samples
	// (four lines per sample on every level whose cells are smaller than the marching step), 63 % of them hits.  Measured on
	// that workload and dropped: whole levels dealt to XCDs by a cost plan (the launch then fetches a third of the 278 MiB,
	// but takes 9 to 20 us longer with every cost model tried), one 8- or 16-byte load per pair of x neighbours instead of
	// two 4-byte loads (+12 us), a pair of lanes per sample so that the x neighbours' line is looked up once (+2 us), loads of
	// the hashed levels that bypass the L1 (agent- or system-scope: +27 us, the x neighbour's line is then requested twice and
	// a request is no cheaper) or carry the non-temporal hint (no change).
	// Staging the coarse levels in LDS has nothing to win: with all caches cold, levels 0..2 together add 2 us to the launch
	// and the five dense levels 4 us, against 5 to 6 us for each of the fine hashed levels and 19 us for reading the
	// positions and writing 320 bytes of features and slopes per sample.
	// The trainer's sample generator runs beside this kernel on a second stream: where a wave of each is ready on a SIMD, this
	// one issues first (the generator has the rest of the step to finish; measured 4 us on the forward, 2 us on the step).
	__builtin_amdgcn_s_setprio(3);
	const uint32_t level = blockIdx.x / tiles, tile = blockIdx.x - level * tiles;
	if (FULL && level >= a.n_levels) {  // the workgroups behind the last level: the network kernel's weight fragments
		write_frag_image(a, blockIdx.x - a.n_levels * tiles);
		return;
	}
	const uint32_t i = tile * FG_BLOCK + threadIdx.x;
	if (i >= a.N || (a.live && i >= *a.live)) return;
	gather_item<FULL>(a, level, i, i);
}

// ----------------------------------------------------------------------------
// the network kernel: a wave takes 32 samples per pass, lane (n, g) works for sample b0 + n on the levels l(j, g).
// GATHER: the features come from the table (inference on points in lattice order); else from the rows the gather kernel wrote.
// ----------------------------------------------------------------------------
template <bool FULL, bool GATHER>
__global__ void __launch_bounds__(FF_BLOCK, 2) field_fused_forward_kernel(const FusedArgs a) {
	static_assert(!(FULL && GATHER), "the full forward reads the gather kernel's rows");
	extern __shared__ __align__(16) unsigned char smem[];
	hf* F = reinterpret_cast<hf*>(smem);
	uint4* LV = reinterpret_cast<uint4*>(smem + (size_t)(FULL ? FF_COUNT : FF_SDF_COUNT) * 1024);
	// FULL: each wave's staging area for the colour net's input (32 samples)
	unsigned char* const stage = smem + (size_t)(FULL ? FF_COUNT : FF_SDF_COUNT) * 1024 + FF_LEVELS * sizeof(uint4) + (threadIdx.x >> 6) * (32 * 2 * N2_RGB_IN_PITCH);
	if (threadIdx.x < FF_LEVELS)
		LV[threadIdx.x] = make_uint4(__float_as_uint(a.lv.scale[threadIdx.x]), a.lv.res[threadIdx.x], a.lv.entries[threadIdx.x], a.lv.offset[threadIdx.x]);
	if (FULL && a.frags) load_fused_frags(F, a.frags, FF_COUNT);
	else build_fused_frags(F, a, FULL ? FF_COUNT : FF_SDF_COUNT);
	const int lane = threadIdx.x & 63, n = lane & 31, g = lane >> 5;
	const uint32_t N = a.N, hash_mask = a.lv.hash_mask, active = a.lv.active_levels;
	uint32_t n_live = a.live ? min(*a.live, N) : N, col0 = 0;
	if (FULL && a.list) listed_range(a, col0, n_live);  // a listed pass: columns col0 .. col0 + n_live
	const uint32_t n_tiles = (n_live + 31u) / 32u;
	const uint32_t wave_gid = blockIdx.x * (FF_BLOCK / 64) + (threadIdx.x >> 6), n_waves = gridDim.x * (FF_BLOCK / 64);
	// (Loading a wave's next tile while the current one is computed, into the registers the current operands have left, was
	// measured on the full forward: no change; neither did three workgroups per CU at 168 registers, which spills.)
	for (uint32_t tile = wave_gid; tile < n_tiles; tile += n_waves) {
		const uint32_t col_raw = tile * 32u + n;
		const bool valid = col_raw < n_live;
		const uint32_t col = col0 + (valid ? col_raw : n_live - 1u);
		const uint32_t dst = (FULL && a.list) ? a.list[col] : col;  // the sample's row in the output
		half8 xs[3];               // SDF net input, B operands
		float p[3], dir[3] = {0.f, 0.f, 0.f};
		uint4 slope[8];            // FULL: the slopes of the lane's 8 levels as stored
		if (GATHER) {
			if (a.pos) {
				const float* q = a.pos + (size_t)col * a.ps;
#pragma unroll
				for (int d = 0; d < 3; ++d) p[d] = q[(size_t)d * a.ds];
			} else {
				// lattice point (x, y, z), x fastest: (c / res) * extent + corner, each step rounded on its own (the positions are
				// part of a bit-exact contract); points behind the lattice's end sit at the centre
				const uint32_t idx = a.lat.first + col;
				const uint32_t c[3] = {idx % a.lat.res[0], (idx / a.lat.res[0]) % a.lat.res[1], idx / (a.lat.res[0] * a.lat.res[1])};
#pragma unroll
				for (int d = 0; d < 3; ++d)
					p[d] = idx < a.lat.total ? __fadd_rn(__fmul_rn(__fmul_rn((float)c[d], a.lat.inv_res[d]), a.lat.extent[d]), a.lat.corner[d]) : 0.5f;
			}
			// the lane's 8 levels, the next level's loads in flight while one is finished
			Item cur, nxt;
			float unused[2][3];
			item_fetch<0>(LV, hash_mask, active, a.table, g, p, cur);
#define FF_STEP(J)                                                                           \
			if (J < 7) item_fetch<(J < 7 ? J + 1 : 0)>(LV, hash_mask, active, a.table, g, p, nxt); \
			{                                                                                \
				float feat[2];                                                               \
				item_finish<false>(cur, feat, unused);                                       \
				xs[J >> 2][2 * (J & 3)] = (hf)feat[0];                                       \
				xs[J >> 2][2 * (J & 3) + 1] = (hf)feat[1];                                   \
			}                                                                                \
			cur = nxt;                                                                       \
			__builtin_amdgcn_sched_barrier(0);
			FF_STEP(0) FF_STEP(1) FF_STEP(2) FF_STEP(3) FF_STEP(4) FF_STEP(5) FF_STEP(6) FF_STEP(7)
#undef FF_STEP
		} else {
			if (FULL) {
				const float* q = a.coords + (size_t)col * 7;
#pragma unroll
				for (int d = 0; d < 3; ++d) { p[d] = q[d]; dir[d] = q[4 + d]; }
			} else {
				const float* q = a.pos + (size_t)col * a.ps;
#pragma unroll
				for (int d = 0; d < 3; ++d) p[d] = q[(size_t)d * a.ds];
			}
#pragma unroll
			for (int j = 0; j < 8; ++j) {
				const uint32_t level = 4u * (j >> 1) + 2u * g + (j & 1);
				// levels the grid does not have read level 0's rows and are ignored (their weights are zero)
				const uint32_t lr = 2u * level < a.enc_w ? level : 0u;
				xs[j >> 2][2 * (j & 3)] = a.sdf_in[(size_t)(3 + 2 * lr) * N + col];
				xs[j >> 2][2 * (j & 3) + 1] = a.sdf_in[(size_t)(4 + 2 * lr) * N + col];
				if (FULL) slope[j] = a.slopes[(size_t)lr * N + col];
			}
		}
		xs[2] = zero8();
		if (g == 0) {
#pragma unroll
			for (int d = 0; d < 3; ++d) xs[2][d] = (hf)p[d] - (hf)0.5f;
		}
		const size_t off4 = (size_t)4u * g * N + col;
		// ---- SDF net ----
		half8 h[4];
#pragma unroll
		for (int mt = 0; mt < 2; ++mt) {
			float16v acc = zero16();
#pragma unroll
			for (int c = 0; c < 3; ++c) acc = N2_MFMA(frag(F, S_W0 + mt * 3 + c, lane), xs[c], acc);
			relu_pack(acc, h[2 * mt], h[2 * mt + 1]);
		}
		float16v out = zero16();
#pragma unroll
		for (int c = 0; c < 4; ++c) out = N2_MFMA(frag(F, S_WO + c, lane), h[c], out);
		half8 y = round8(out, 0);  // rows 4g .. 4g+3 and 8+4g .. 8+4g+3
		if (!FULL) {
			if (g == 0) {
				hf s = y[0] + (hf)a.sdf_bias;
				if (a.density) {
					const hf is = (hf)__expf((float)(a.variance[0] * (hf)10.0f));
					const hf x = s * is;
					const hf sig = (hf)(1.0f / (1.0f + __expf(-(float)x)));
					s = is * sig * ((hf)1.0f - sig);
				}
				y[0] = s;
				if (a.row0 && col_raw < a.row0_n) a.row0[col] = (float)s;
			}
			if (a.sdf_out && valid) {
#pragma unroll
				for (int e = 0; e < 4; ++e) {
					a.sdf_out[(size_t)e * N + off4] = y[e];
					a.sdf_out[(size_t)(8 + e) * N + off4] = y[4 + e];
				}
			}
			tile_fence();
			continue;
		}
		// ---- d sdf / d input: dh = mask * W_out[0, :], dX = W_0^T dh ----
		half8 dh[4];
#pragma unroll
		for (int c = 0; c < 4; ++c) dh[c] = mask8(frag(F, S_DH + c, lane), h[c]);
		float16v dx0 = zero16(), dx1 = zero16();
#pragma unroll
		for (int c = 0; c < 4; ++c) dx0 = N2_MFMA(frag(F, S_W0T + c, lane), dh[c], dx0);
#pragma unroll
		for (int c = 0; c < 4; ++c) dx1 = N2_MFMA(frag(F, S_W0T + 4 + c, lane), dh[c], dx1);
		// register r of dx0 is feature r % 2 of the lane's level step r / 2; registers 0..2 of dx1 (g = 0) the coordinates
		const half8 g_lo = round8(dx0, 0), g_hi = round8(dx0, 8);
		const hf gx[3] = {(hf)dx1[0], (hf)dx1[1], (hf)dx1[2]};
		float nrm[3];
#pragma unroll
		for (int d = 0; d < 3; ++d) nrm[d] = g == 0 ? (float)gx[d] : 0.f;
#pragma unroll
		for (int j = 0; j < 8; ++j) {
			const uint32_t level = 4u * (j >> 1) + 2u * g + (j & 1);
			const float sc = 2u * level < a.enc_w ? __uint_as_float(LV[level].x) : 0.f;
			float q[6];
			const float unit = n2_slopes_unpack(slope[j], q) * sc;
			const float g0 = (float)(j < 4 ? g_lo[2 * j] : g_hi[2 * j - 8]) * unit, g1 = (float)(j < 4 ? g_lo[2 * j + 1] : g_hi[2 * j - 7]) * unit;
#pragma unroll
			for (int d = 0; d < 3; ++d) nrm[d] = fmaf(g0, q[d], fmaf(g1, q[3 + d], nrm[d]));
		}
#pragma unroll
		for (int d = 0; d < 3; ++d) nrm[d] += __shfl_xor(nrm[d], 32);
		const hf hn[3] = {(hf)nrm[0], (hf)nrm[1], (hf)nrm[2]};
		// ---- colour net input: SDF-net outputs | SH of the direction | position, normal ----
		float sh[16];
		sh4(dir[0] * 2.f - 1.f, dir[1] * 2.f - 1.f, dir[2] * 2.f - 1.f, sh);
		half8 xc[3];
		xc[0] = y;
		{
			// both halves are formed and one is picked value by value: picking between sh[e] and sh[8 + e] inside the
			// conversion turns into an index that depends on the lane, and the array then lives in scratch memory
			half8 lo8, hi8;
#pragma unroll
			for (int e = 0; e < 8; ++e) { lo8[e] = (hf)sh[e]; hi8[e] = (hf)sh[8 + e]; }
			const uint4 lo = __builtin_bit_cast(uint4, lo8), hi = __builtin_bit_cast(uint4, hi8);
			xc[1] = __builtin_bit_cast(half8, make_uint4(g ? hi.x : lo.x, g ? hi.y : lo.y, g ? hi.z : lo.z, g ? hi.w : lo.w));
		}
		xc[2] = zero8();
		if (g == 0) {
#pragma unroll
			for (int d = 0; d < 3; ++d) { xc[2][d] = (hf)p[d]; xc[2][3 + d] = hn[d]; }
		}
		{
			// The colour net's input goes out sample-major for the backward pass (N2_RGB_IN_PITCH = 40 values per sample: rows
			// 38, 39 zero, rows 40..47 of the padded input left out): the wave's 32 samples are 2560 consecutive bytes.  A
			// lane's registers are runs of 4 and 8 rows of its sample; stored from there, every 16 bytes would be a write
			// request of their own.  Through LDS (80 bytes per sample: the 16-byte writes of 16 lanes fall on different
			// banks) the wave writes whole lines.
			unsigned char* sp = stage + n * (2 * N2_RGB_IN_PITCH);
			*reinterpret_cast<half4v*>(sp + 8 * g) = half4v{y[0], y[1], y[2], y[3]};
			*reinterpret_cast<half4v*>(sp + 16 + 8 * g) = half4v{y[4], y[5], y[6], y[7]};
			*reinterpret_cast<half8*>(sp + 32 + 16 * g) = xc[1];
			if (g == 0) *reinterpret_cast<half8*>(sp + 64) = xc[2];
			__builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
			__builtin_amdgcn_wave_barrier();
			__builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
			const uint32_t chunks = 5u * min(32u, n_live - tile * 32u);  // 16-byte chunks of the tile's samples
			unsigned char* out = reinterpret_cast<unsigned char*>(a.rgb_in) + ((size_t)col0 + (size_t)tile * 32u) * (2u * N2_RGB_IN_PITCH);
#pragma unroll
			for (int i = 0; i < 3; ++i) {
				const uint32_t k = (uint32_t)lane + 64u * i;
				if (k < chunks) *reinterpret_cast<uint4*>(out + (size_t)k * 16u) = *reinterpret_cast<const uint4*>(stage + k * 16u);
			}
		}
		if (valid) {
			// (rows 0..2 of d sdf / d input, gx, have no reader behind this kernel)
#pragma unroll
			for (int r = 0; r < 16; ++r) {
				const uint32_t level = 4u * (r >> 2) + 2u * g + ((r >> 1) & 1);
				if (2u * level < a.enc_w) a.dsdf_din[(size_t)(3 + 2 * level + (r & 1)) * N + col] = r < 8 ? g_lo[r] : g_hi[r - 8];
			}
		}
		half8 h0[4], h1[4];
#pragma unroll
		for (int mt = 0; mt < 2; ++mt) {
			float16v acc = zero16();
#pragma unroll
			for (int c = 0; c < 3; ++c) acc = N2_MFMA(frag(F, C_W0 + mt * 3 + c, lane), xc[c], acc);
			relu_pack(acc, h0[2 * mt], h0[2 * mt + 1]);
		}
#pragma unroll
		for (int mt = 0; mt < 2; ++mt) {
			float16v acc = zero16();
#pragma unroll
			for (int c = 0; c < 4; ++c) acc = N2_MFMA(frag(F, C_WH + mt * 4 + c, lane), h0[c], acc);
			relu_pack(acc, h1[2 * mt], h1[2 * mt + 1]);
		}
		float16v co = zero16();
#pragma unroll
		for (int c = 0; c < 4; ++c) co = N2_MFMA(frag(F, C_WO + c, lane), h1[c], co);
		// ---- output rows: r g b | sdf + bias | normal | variance | direction | colour-net rows 11..15 ----
		half4 lo = half4{(hf)co[0], (hf)co[1], (hf)co[2], (hf)co[3]}, hi = half4{(hf)co[4], (hf)co[5], (hf)co[6], (hf)co[7]};
		if (g == 0) {
			lo[3] = y[0] + (hf)a.sdf_bias;
			hi[0] = (hf)dir[0]; hi[1] = (hf)dir[1]; hi[2] = (hf)dir[2];
		} else {
			lo[0] = hn[0]; lo[1] = hn[1]; lo[2] = hn[2]; lo[3] = a.variance[0];
		}
		if (valid) {
			hf* o = a.output + (size_t)dst * MLP_OUT;
			*reinterpret_cast<half4*>(o + 4 * g) = lo;
			*reinterpret_cast<half4*>(o + 8 + 4 * g) = hi;
		}
		tile_fence();
	}
}

// ----------------------------------------------------------------------------
// host side
// ----------------------------------------------------------------------------
bool n2_fused_supported(const N2LevelTable& tab, uint32_t sdf_hidden_layers, uint32_t rgb_hidden_layers) {
	if (tab.n_levels > FF_LEVELS || tab.n_features != 2 || sdf_hidden_layers != 1 || rgb_hidden_layers != 2) return false;
	if (tab.max_level_gpu != nullptr) return false;  // per-point level masks take the unfused path
	for (uint32_t l = 0; l < tab.n_levels; ++l)
		if (tab.mode[l] != N2_LEVEL_DENSE && tab.mode[l] != N2_LEVEL_HASH) return false;
	return true;
}

template <bool FULL>
static void launch_gather(const FusedArgs& a, const N2LevelTable& tab, hipStream_t s) {
	const uint32_t tiles = (a.N + FG_BLOCK - 1) / FG_BLOCK;
	field_gather_kernel<FULL><<<dim3(tiles * tab.n_levels + (FULL && a.frags ? FRAG_BLOCKS : 0u)), dim3(FG_BLOCK), 0, s>>>(a, tiles);
}

static uint32_t fused_grid(uint32_t n) {
	const uint32_t tiles = (n + 31u) / 32u, blocks = (tiles + 3u) / 4u;
	return blocks < 512u ? blocks : 512u;
}
static size_t fused_lds(int n_frags, bool staged = false) {
	return (size_t)n_frags * 1024 + FF_LEVELS * sizeof(uint4) + (staged ? (size_t)(FF_BLOCK / 64) * 32 * 2 * N2_RGB_IN_PITCH : 0);
}

static FusedArgs fused_base(const N2FusedNets& nets, uint32_t n) {
	FusedArgs a{};
	const N2LevelTable& tab = *nets.tab;
	const uint32_t active = tab.active_levels < tab.n_levels ? tab.active_levels : tab.n_levels;
	for (uint32_t l = 0; l < FF_LEVELS; ++l) {
		const bool have = l < tab.n_levels;  // levels the table does not have read as switched off
		a.lv.scale[l] = have ? tab.scale[l] : 1.f;
		a.lv.res[l] = have ? tab.resolution[l] : 1u;
		a.lv.entries[l] = have ? tab.entries[l] : 8u;
		a.lv.offset[l] = have ? tab.offset[l] : 0u;
		if (have && tab.mode[l] == N2_LEVEL_HASH) a.lv.hash_mask |= 1u << l;
	}
	a.lv.active_levels = active;
	a.table = nets.table;
	a.sdf_w = reinterpret_cast<const hf*>(nets.sdf_w);
	a.rgb_w = reinterpret_cast<const hf*>(nets.rgb_w);
	a.variance = reinterpret_cast<const hf*>(nets.variance);
	a.sdf_in_w = nets.sdf_in_w;
	a.enc_w = tab.n_levels * 2;
	a.n_levels = tab.n_levels;
	a.sdf_bias = nets.sdf_bias;
	a.N = n;
	a.live = nullptr;
	a.list = nullptr;
	a.counts = nullptr;
	a.round = 0;
	a.frags = nullptr;
	return a;
}

int n2_fused_field_forward(const N2FusedNets& nets, hipStream_t s, const float* d_coords, uint32_t n, n2_half* sdf_in, float* xyz_rows,
                           void* slopes, n2_half* dsdf_din, n2_half* rgb_in, n2_half* d_output, const uint32_t* d_live, const uint32_t* d_list,
                           const uint32_t* d_counts, uint32_t round, uint32_t est_samples, const float* d_xyz_soa) {
	FusedArgs a = fused_base(nets, n);
	if (d_xyz_soa) { a.pos = d_xyz_soa; a.ps = 1; a.ds = n; }
	a.live = d_live;
	a.list = d_list;
	a.counts = d_counts;
	a.round = round;
	a.frags = reinterpret_cast<hf*>(nets.frag_image);
	a.coords = d_coords;
	a.sdf_in = reinterpret_cast<hf*>(sdf_in);
	a.xyz_rows = xyz_rows;
	a.slopes = reinterpret_cast<uint4*>(slopes);
	a.dsdf_din = reinterpret_cast<hf*>(dsdf_din);
	a.rgb_in = reinterpret_cast<hf*>(rgb_in);
	a.output = reinterpret_cast<hf*>(d_output);
	if (d_list) {
		// est_samples: the caller's estimate of this round's sample count (it only sizes the launches)
		const uint32_t est = est_samples < 1u ? 1u : (est_samples > n ? n : est_samples);
		const uint32_t est_tiles = (est + FG_BLOCK - 1) / FG_BLOCK;
		field_gather_list_kernel<<<dim3(est_tiles * a.n_levels + (a.frags && round == 0 ? FRAG_BLOCKS : 0u)), dim3(FG_BLOCK), 0, s>>>(a, est_tiles);
		N2_LAUNCH_CHECK();
		// one 32-sample tile per wave where the estimate holds (the weight fragments come as a copy, so small workgroups are cheap)
		const uint32_t blocks = (est + 127u) / 128u;
		field_fused_forward_kernel<true, false><<<dim3(blocks < 2048u ? blocks : 2048u), dim3(FF_BLOCK), fused_lds(FF_COUNT, true), s>>>(a);
		N2_LAUNCH_CHECK();
		return N2_OK;
	}
	{
		N2ProfScope prof(N2_PROF_FIELD_GATHER, s);
		launch_gather<true>(a, *nets.tab, s);
	}
	N2_LAUNCH_CHECK();
	field_fused_forward_kernel<true, false><<<dim3(fused_grid(n)), dim3(FF_BLOCK), fused_lds(FF_COUNT, true), s>>>(a);
	N2_LAUNCH_CHECK();
	return N2_OK;
}

int n2_fused_field_sdf(const N2FusedNets& nets, hipStream_t s, const float* d_xyz, uint32_t ps, uint32_t ds, uint32_t n, n2_half* d_out_soa,
                       float* d_row0, bool density, n2_half* sdf_in, uint32_t row0_n, const N2Lattice* lattice) {
	FusedArgs a = fused_base(nets, n);
	a.pos = d_xyz; a.ps = ps; a.ds = ds;
	if (lattice) {
		if (d_xyz != nullptr || sdf_in != nullptr) { n2_set_error("n2_fused_field_sdf: lattice points are generated in the one-launch form only"); return N2_ERR_INVALID_ARGUMENT; }
		a.lat = *lattice;
	}
	a.sdf_out = reinterpret_cast<hf*>(d_out_soa);
	a.row0 = d_row0;
	a.row0_n = row0_n < n ? row0_n : n;
	a.density = density ? 1 : 0;
	if (sdf_in == nullptr) {
		field_fused_forward_kernel<false, true><<<dim3(fused_grid(n)), dim3(FF_BLOCK), fused_lds(FF_SDF_COUNT), s>>>(a);
		N2_LAUNCH_CHECK();
		return N2_OK;
	}
	// points in no particular order: a sample-major walk would touch all tables at once, so the features are gathered level
	// by level into the network's input rows first
	a.sdf_in = reinterpret_cast<hf*>(sdf_in);
	launch_gather<false>(a, *nets.tab, s);
	N2_LAUNCH_CHECK();
	field_fused_forward_kernel<false, false><<<dim3(fused_grid(n)), dim3(FF_BLOCK), fused_lds(FF_SDF_COUNT), s>>>(a);
	N2_LAUNCH_CHECK();
	return N2_OK;
}
