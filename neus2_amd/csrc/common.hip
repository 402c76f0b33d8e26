// Error reporting, version string and small utility kernels.
#include "n2_common.h"

static thread_local char g_err[512] = "";

void n2_set_error(const char* fmt, ...) {
	va_list ap;
	va_start(ap, fmt);
	vsnprintf(g_err, sizeof(g_err), fmt, ap);
	va_end(ap);
}

N2_API const char* n2_last_error(void) { return g_err; }
N2_API const char* n2_version(void) { return "neus2_amd 0.1 gfx950"; }

__global__ void __launch_bounds__(256) n2_fill_zero_kernel(uint4* __restrict__ p16, size_t n16, uint8_t* __restrict__ tail, uint32_t n_tail) {
	const size_t stride = (size_t)gridDim.x * blockDim.x;
	for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n16; i += stride) p16[i] = make_uint4(0, 0, 0, 0);
	if (blockIdx.x == 0 && threadIdx.x < n_tail) tail[threadIdx.x] = 0;
}

int n2_fill_zero_u32(hipStream_t stream, void* d_ptr, size_t n_bytes) {
	if (n_bytes == 0) return N2_OK;
	if (reinterpret_cast<uintptr_t>(d_ptr) % 16 != 0) {
		n2_set_error("zero fill needs a 16-byte aligned buffer");
		return N2_ERR_INVALID_ARGUMENT;
	}
	const size_t n16 = n_bytes / 16;
	const uint32_t n_tail = (uint32_t)(n_bytes % 16);
	size_t blocks = (n16 + 255) / 256;
	if (blocks > 4096) blocks = 4096;
	if (blocks == 0) blocks = 1;
	n2_fill_zero_kernel<<<dim3((uint32_t)blocks), dim3(256), 0, stream>>>(
		reinterpret_cast<uint4*>(d_ptr), n16, reinterpret_cast<uint8_t*>(d_ptr) + n16 * 16, n_tail);
	N2_LAUNCH_CHECK();
	return N2_OK;
}

__global__ void n2_set_u32_kernel(uint32_t* p, uint32_t v) { *p = v; }

int n2_set_u32(hipStream_t stream, uint32_t* d_ptr, uint32_t value) {
	n2_set_u32_kernel<<<dim3(1), dim3(1), 0, stream>>>(d_ptr, value);
	N2_LAUNCH_CHECK();
	return N2_OK;
}

// ---------------------------------------------------------------------------
// event timing
// ---------------------------------------------------------------------------
#include <vector>

namespace {
struct ProfState {
	bool enabled = false;
	uint32_t mask = 0xFFFFFFFFu;                  // ids that are timed while enabled
	uint32_t period = 1;                          // every period-th launch of an id is timed
	uint32_t seen[N2_PROF_COUNT] = {};
	std::vector<hipEvent_t> pool;                 // recycled events
	std::vector<hipEvent_t> pending[N2_PROF_COUNT];  // begin/end pairs, not yet read
	float total_ms[N2_PROF_COUNT] = {};
	uint32_t launches[N2_PROF_COUNT] = {};
	hipEvent_t open_begin[N2_PROF_COUNT] = {};
};
ProfState g_prof;

hipEvent_t prof_take() {
	if (!g_prof.pool.empty()) {
		hipEvent_t e = g_prof.pool.back();
		g_prof.pool.pop_back();
		return e;
	}
	hipEvent_t e = nullptr;
	if (hipEventCreate(&e) != hipSuccess) return nullptr;
	return e;
}

void prof_collect(int id) {
	auto& v = g_prof.pending[id];
	for (size_t i = 0; i + 1 < v.size(); i += 2) {
		float ms = 0.f;
		if (hipEventSynchronize(v[i + 1]) == hipSuccess && hipEventElapsedTime(&ms, v[i], v[i + 1]) == hipSuccess) {
			g_prof.total_ms[id] += ms;
			g_prof.launches[id] += 1;
		}
		g_prof.pool.push_back(v[i]);
		g_prof.pool.push_back(v[i + 1]);
	}
	v.clear();
}
}  // namespace

void n2_prof_begin(int id, hipStream_t stream) {
	if (!g_prof.enabled || !((g_prof.mask >> id) & 1u)) return;
	if (g_prof.seen[id]++ % g_prof.period != 0) return;
	hipEvent_t e = prof_take();
	if (!e) return;
	(void)hipEventRecord(e, stream);
	g_prof.open_begin[id] = e;
}

void n2_prof_end(int id, hipStream_t stream) {
	if (!g_prof.enabled || !g_prof.open_begin[id]) return;
	hipEvent_t e = prof_take();
	if (!e) return;
	(void)hipEventRecord(e, stream);
	g_prof.pending[id].push_back(g_prof.open_begin[id]);
	g_prof.pending[id].push_back(e);
	g_prof.open_begin[id] = nullptr;
	if (g_prof.pending[id].size() >= 8192) prof_collect(id);  // bound the number of live events
}

N2_API int n2_profile_enable(int enable) {
	g_prof.enabled = enable != 0;
	return N2_OK;
}

N2_API int n2_profile_select(uint32_t id_mask) {
	g_prof.mask = id_mask;
	return N2_OK;
}

N2_API int n2_profile_set_period(uint32_t every) {
	N2_REQUIRE(every >= 1, "n2_profile_set_period: the period must be at least 1");
	g_prof.period = every;
	for (int id = 0; id < N2_PROF_COUNT; ++id) g_prof.seen[id] = 0;
	return N2_OK;
}

N2_API int n2_profile_read(n2_prof_id id, float* total_ms, uint32_t* launches) {
	N2_REQUIRE((int)id >= 0 && (int)id < N2_PROF_COUNT, "n2_profile_read: bad id %d", (int)id);
	prof_collect((int)id);
	if (total_ms) *total_ms = g_prof.total_ms[id];
	if (launches) *launches = g_prof.launches[id];
	return N2_OK;
}

N2_API int n2_profile_reset(void) {
	for (int id = 0; id < N2_PROF_COUNT; ++id) {
		prof_collect(id);
		g_prof.total_ms[id] = 0.f;
		g_prof.launches[id] = 0;
	}
	return N2_OK;
}
