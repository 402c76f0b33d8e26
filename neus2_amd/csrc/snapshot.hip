// Snapshot files: the reference stores its network configuration plus a
// "snapshot" object as MessagePack (nlohmann::json::to_msgpack of
// m_network_config; Testbed::save_snapshot / load_snapshot,
// src/testbed.cu:3134-3244).  Layout of the "snapshot" object:
//   n_params, params_type ("__half" | "float"), params_binary        Trainer::serialize
//   optimizer { nested... }                                           only with optimizer state
//   density_grid_size (128), density_grid_binary (fp16 cells)         :3144-3152
//   nerf { aabb_scale, rgb { rays_per_batch, measured_batch_size,
//          measured_batch_size_before_compaction } }                  :3154, 3160-3163
//   training_step, loss                                               :3157-3158
// Binary members are MessagePack "bin" items (nlohmann's binary_t).  The member names of the optimizer object
// (Ema > ExponentialDecay > Adam nesting, "first_moments_binary" ...) follow tiny-cuda-nn's published serializers;
// the fork's own copies are not in the reference tree.
//
// This file holds a small MessagePack writer and reader (the subset JSON maps onto), the host logic of
// save / open / read, and the fp32 <-> fp16 conversion kernels for the density grid and the parameters.
#include "n2_common.h"

#include <cstdlib>
#include <cstring>
#include <new>
#include <string>
#include <vector>

typedef _Float16 hf;

// ---------------------------------------------------------------------------
// MessagePack writer
// ---------------------------------------------------------------------------
namespace {

struct Writer {
	std::vector<uint8_t> buf;
	void byte(uint8_t b) { buf.push_back(b); }
	void be(uint64_t v, int n) { for (int i = n - 1; i >= 0; --i) buf.push_back((uint8_t)(v >> (8 * i))); }
	void raw(const void* p, size_t n) { const uint8_t* b = (const uint8_t*)p; buf.insert(buf.end(), b, b + n); }
	void map(uint32_t n) {
		if (n < 16) byte(0x80 | n); else if (n < 65536) { byte(0xde); be(n, 2); } else { byte(0xdf); be(n, 4); }
	}
	void str(const char* s) {
		const size_t n = strlen(s);
		if (n < 32) byte(0xa0 | (uint8_t)n); else if (n < 256) { byte(0xd9); be(n, 1); } else if (n < 65536) { byte(0xda); be(n, 2); } else { byte(0xdb); be(n, 4); }
		raw(s, n);
	}
	void uint(uint64_t v) {
		if (v < 128) byte((uint8_t)v); else if (v < 256) { byte(0xcc); be(v, 1); } else if (v < 65536) { byte(0xcd); be(v, 2); }
		else if (v < (1ull << 32)) { byte(0xce); be(v, 4); } else { byte(0xcf); be(v, 8); }
	}
	// nlohmann writes a number as float32 when that is exact, else as float64
	void real(double d) {
		const float f = (float)d;
		if ((double)f == d) { uint32_t u; memcpy(&u, &f, 4); byte(0xca); be(u, 4); }
		else { uint64_t u; memcpy(&u, &d, 8); byte(0xcb); be(u, 8); }
	}
	void bin_header(uint64_t n) {
		if (n < 256) { byte(0xc4); be(n, 1); } else if (n < 65536) { byte(0xc5); be(n, 2); } else { byte(0xc6); be(n, 4); }
	}
};

// ---------------------------------------------------------------------------
// MessagePack reader: a cursor over the file image; values are skipped or decoded in place
// ---------------------------------------------------------------------------
struct Reader {
	const uint8_t* p;
	const uint8_t* end;
	bool ok = true;

	bool need(size_t n) { if ((size_t)(end - p) < n) { ok = false; return false; } return true; }
	uint64_t be(int n) {
		if (!need(n)) return 0;
		uint64_t v = 0;
		for (int i = 0; i < n; ++i) v = (v << 8) | *p++;
		return v;
	}
	uint8_t peek() { return need(1) ? *p : 0xc1; }

	// containers: returns the element count (pairs for maps), or false if the next item is something else
	bool map(uint32_t& n) {
		const uint8_t t = peek();
		if ((t & 0xf0) == 0x80) { ++p; n = t & 0x0f; return true; }
		if (t == 0xde) { ++p; n = (uint32_t)be(2); return ok; }
		if (t == 0xdf) { ++p; n = (uint32_t)be(4); return ok; }
		return false;
	}
	bool array(uint32_t& n) {
		const uint8_t t = peek();
		if ((t & 0xf0) == 0x90) { ++p; n = t & 0x0f; return true; }
		if (t == 0xdc) { ++p; n = (uint32_t)be(2); return ok; }
		if (t == 0xdd) { ++p; n = (uint32_t)be(4); return ok; }
		return false;
	}
	bool str(std::string& s) {
		const uint8_t t = peek();
		size_t n;
		if ((t & 0xe0) == 0xa0) { ++p; n = t & 0x1f; }
		else if (t == 0xd9) { ++p; n = be(1); } else if (t == 0xda) { ++p; n = be(2); } else if (t == 0xdb) { ++p; n = be(4); }
		else return false;
		if (!ok || !need(n)) return false;
		s.assign((const char*)p, n);
		p += n;
		return true;
	}
	bool bin(const uint8_t*& data, uint64_t& n) {
		const uint8_t t = peek();
		if (t == 0xc4) { ++p; n = be(1); } else if (t == 0xc5) { ++p; n = be(2); } else if (t == 0xc6) { ++p; n = be(4); }
		else return false;
		if (!ok || !need(n)) return false;
		data = p;
		p += n;
		return true;
	}
	// any number as double (and whether it was an integer)
	bool number(double& d) {
		const uint8_t t = peek();
		if (t < 0x80) { ++p; d = t; return true; }
		if (t >= 0xe0) { ++p; d = (int8_t)t; return true; }
		switch (t) {
			case 0xcc: ++p; d = (double)be(1); return ok;
			case 0xcd: ++p; d = (double)be(2); return ok;
			case 0xce: ++p; d = (double)be(4); return ok;
			case 0xcf: ++p; d = (double)be(8); return ok;
			case 0xd0: ++p; d = (double)(int8_t)be(1); return ok;
			case 0xd1: ++p; d = (double)(int16_t)be(2); return ok;
			case 0xd2: ++p; d = (double)(int32_t)be(4); return ok;
			case 0xd3: ++p; d = (double)(int64_t)be(8); return ok;
			case 0xca: { ++p; const uint32_t u = (uint32_t)be(4); float f; memcpy(&f, &u, 4); d = f; return ok; }
			case 0xcb: { ++p; const uint64_t u = be(8); memcpy(&d, &u, 8); return ok; }
			default: return false;
		}
	}
	void skip() {
		if (!ok) return;
		uint32_t n;
		std::string s;
		const uint8_t* b;
		uint64_t len;
		double d;
		const uint8_t t = peek();
		if (!ok) return;
		if (map(n)) { for (uint32_t i = 0; i < 2 * n && ok; ++i) skip(); return; }
		if (array(n)) { for (uint32_t i = 0; i < n && ok; ++i) skip(); return; }
		if (str(s) || bin(b, len) || number(d)) return;
		if (t == 0xc0 || t == 0xc2 || t == 0xc3) { ++p; return; }
		// ext types: fixext 1..16, ext 8/16/32
		if (t >= 0xd4 && t <= 0xd8) { ++p; const size_t m = (size_t)1 << (t - 0xd4); if (need(1 + m)) p += 1 + m; return; }
		if (t >= 0xc7 && t <= 0xc9) { ++p; const uint64_t m = be(1 << (t - 0xc7)); if (ok && need(1 + m)) p += 1 + m; return; }
		ok = false;
	}
};

struct BinRef {
	const uint8_t* data = nullptr;
	uint64_t bytes = 0;
};

}  // namespace

struct n2_snapshot {
	std::vector<uint8_t> file;
	n2_snapshot_info info;
	BinRef params, density, m1, m2, steps, ema;
};

// ---------------------------------------------------------------------------
// conversion kernels
// ---------------------------------------------------------------------------
__global__ void __launch_bounds__(256) snap_f32_to_f16_kernel(uint64_t n, const float* __restrict__ in, hf* __restrict__ out) {
	const uint64_t i = (uint64_t)blockIdx.x * 256 + threadIdx.x;
	if (i < n) out[i] = (hf)in[i];
}
__global__ void __launch_bounds__(256) snap_f16_to_f32_kernel(uint64_t n, const hf* __restrict__ in, float* __restrict__ out) {
	const uint64_t i = (uint64_t)blockIdx.x * 256 + threadIdx.x;
	if (i < n) out[i] = (float)in[i];
}
static inline dim3 sgrid(uint64_t n) { return dim3((uint32_t)((n + 255) / 256)); }

// ---------------------------------------------------------------------------
// save
// ---------------------------------------------------------------------------
static int append_device_bin(Writer& w, const void* d_ptr, uint64_t bytes) {
	N2_REQUIRE(bytes < (1ull << 32), "n2_snapshot_save: a binary member of %llu bytes exceeds MessagePack's 4 GiB limit", (unsigned long long)bytes);
	w.bin_header(bytes);
	const size_t at = w.buf.size();
	w.buf.resize(at + bytes);
	if (bytes) N2_HIP(hipMemcpy(w.buf.data() + at, d_ptr, bytes, hipMemcpyDeviceToHost));
	return N2_OK;
}

N2_API int n2_snapshot_save(const char* path, const n2_snapshot_desc* d, n2_stream_t stream) {
	N2_REQUIRE(path != nullptr && d != nullptr, "n2_snapshot_save: null argument");
	N2_REQUIRE(d->d_params != nullptr && d->n_params > 0, "n2_snapshot_save: no parameters");
	N2_REQUIRE(d->density_grid_cells == 0 || (d->d_density_grid != nullptr && d->d_scratch != nullptr && d->scratch_bytes >= 2 * d->density_grid_cells),
	           "n2_snapshot_save: the density grid needs a device scratch of 2 bytes per cell");
	const bool opt = d->include_optimizer_state != 0;
	N2_REQUIRE(!opt || (d->d_first_moments && d->d_second_moments && d->d_param_steps), "n2_snapshot_save: optimizer state requested but its buffers are null");
	hipStream_t s = n2_stream(stream);
	// the caller's configuration: an encoded MessagePack map whose entries become the top-level entries
	uint32_t n_config = 0;
	const uint8_t* config_body = nullptr;
	size_t config_body_bytes = 0;
	if (d->config_msgpack && d->config_bytes) {
		Reader r{d->config_msgpack, d->config_msgpack + d->config_bytes};
		N2_REQUIRE(r.map(n_config), "n2_snapshot_save: config_msgpack is not a MessagePack map");
		config_body = r.p;
		for (uint32_t i = 0; i < n_config && r.ok; ++i) {
			std::string key;
			N2_REQUIRE(r.str(key), "n2_snapshot_save: config_msgpack has a non-string key");
			N2_REQUIRE(key != "snapshot", "n2_snapshot_save: config_msgpack already holds a snapshot");
			r.skip();
		}
		N2_REQUIRE(r.ok && r.p == r.end, "n2_snapshot_save: config_msgpack is truncated or has trailing bytes");
		config_body_bytes = (size_t)(r.p - config_body);
	}
	Writer w;
	w.map(n_config + 1);
	if (config_body_bytes) w.raw(config_body, config_body_bytes);
	w.str("snapshot");
	w.map(opt ? 9u : 8u);
	w.str("n_params"); w.uint(d->n_params);
	w.str("params_type"); w.str("__half");
	w.str("params_binary");
	if (int rc = append_device_bin(w, d->d_params, 2ull * d->n_params)) return rc;
	if (opt) {
		// Ema { nested: ExponentialDecay { nested: Adam {...} } } as the configuration nests them
		w.str("optimizer");
		const bool ema = d->d_ema_weights != nullptr;
		if (ema) {
			w.map(2);
			w.str("ema_weights_binary");
			if (int rc = append_device_bin(w, d->d_ema_weights, 4ull * d->n_params)) return rc;
			w.str("nested");
		}
		w.map(1);
		w.str("nested");
		w.map(5);
		w.str("current_step"); w.uint(d->optimizer_steps);
		w.str("base_learning_rate"); w.real((double)d->learning_rate);
		w.str("first_moments_binary");
		if (int rc = append_device_bin(w, d->d_first_moments, 4ull * d->n_params)) return rc;
		w.str("second_moments_binary");
		if (int rc = append_device_bin(w, d->d_second_moments, 4ull * d->n_params)) return rc;
		w.str("param_steps_binary");
		N2_REQUIRE(d->param_steps_bits == 0 || d->param_steps_bits == 16 || d->param_steps_bits == 32, "n2_snapshot_save: step counters of %u bits", d->param_steps_bits);
		if (d->param_steps_bits == 16) {
			// the file holds 32-bit counters
			std::vector<uint16_t> narrow(d->n_params);
			N2_HIP(hipMemcpy(narrow.data(), d->d_param_steps, 2ull * d->n_params, hipMemcpyDeviceToHost));
			w.bin_header(4ull * d->n_params);
			const size_t at = w.buf.size();
			w.buf.resize(at + 4ull * d->n_params);
			for (uint32_t i = 0; i < d->n_params; ++i) {
				const uint32_t v = narrow[i];
				std::memcpy(w.buf.data() + at + 4ull * i, &v, 4);
			}
		} else if (int rc = append_device_bin(w, d->d_param_steps, 4ull * d->n_params)) return rc;
	}
	w.str("density_grid_size"); w.uint(128);
	w.str("density_grid_binary");
	if (d->density_grid_cells) {
		snap_f32_to_f16_kernel<<<sgrid(d->density_grid_cells), dim3(256), 0, s>>>(d->density_grid_cells, d->d_density_grid, reinterpret_cast<hf*>(d->d_scratch));
		N2_LAUNCH_CHECK();
		N2_HIP(hipStreamSynchronize(s));
	}
	if (int rc = append_device_bin(w, d->d_scratch, 2ull * d->density_grid_cells)) return rc;
	w.str("nerf");
	w.map(2);
	w.str("aabb_scale"); w.uint(d->aabb_scale);
	w.str("rgb");
	w.map(3);
	w.str("rays_per_batch"); w.uint(d->rays_per_batch);
	w.str("measured_batch_size"); w.uint(d->measured_batch_size);
	w.str("measured_batch_size_before_compaction"); w.uint(d->measured_batch_size_before_compaction);
	w.str("training_step"); w.uint(d->training_step);
	w.str("loss"); w.real((double)d->loss);
	FILE* f = fopen(path, "wb");
	N2_REQUIRE(f != nullptr, "n2_snapshot_save: cannot open '%s' for writing", path);
	const size_t written = fwrite(w.buf.data(), 1, w.buf.size(), f);
	const int closed = fclose(f);
	N2_REQUIRE(written == w.buf.size() && closed == 0, "n2_snapshot_save: short write to '%s'", path);
	return N2_OK;
}

// ---------------------------------------------------------------------------
// open / read
// ---------------------------------------------------------------------------
// walks the optimizer object down its "nested" chain and picks up the members it knows
static void parse_optimizer(Reader& r, n2_snapshot* sn) {
	uint32_t n;
	if (!r.map(n)) { r.skip(); return; }
	for (uint32_t i = 0; i < n && r.ok; ++i) {
		std::string key;
		if (!r.str(key)) { r.ok = false; return; }
		double d;
		if (key == "nested") parse_optimizer(r, sn);
		else if (key == "current_step" && r.number(d)) sn->info.optimizer_steps = (uint32_t)d;
		else if (key == "base_learning_rate" && r.number(d)) sn->info.learning_rate = (float)d;
		else if (key == "first_moments_binary" && r.bin(sn->m1.data, sn->m1.bytes)) {}
		else if (key == "second_moments_binary" && r.bin(sn->m2.data, sn->m2.bytes)) {}
		else if (key == "param_steps_binary" && r.bin(sn->steps.data, sn->steps.bytes)) {}
		else if (key == "ema_weights_binary" && r.bin(sn->ema.data, sn->ema.bytes)) {}
		else r.skip();
	}
}

static int parse_snapshot(n2_snapshot* sn, const char* path) {
	Reader r{sn->file.data(), sn->file.data() + sn->file.size()};
	uint32_t n_top;
	N2_REQUIRE(r.map(n_top), "n2_snapshot_open: '%s' is not a MessagePack map", path);
	bool found = false;
	bool params_float = false, have_type = false;
	for (uint32_t i = 0; i < n_top && r.ok; ++i) {
		std::string key;
		N2_REQUIRE(r.str(key), "n2_snapshot_open: '%s' has a non-string key", path);
		if (key != "snapshot") { r.skip(); continue; }
		found = true;
		uint32_t n;
		N2_REQUIRE(r.map(n), "n2_snapshot_open: the snapshot member of '%s' is not a map", path);
		for (uint32_t j = 0; j < n && r.ok; ++j) {
			std::string k;
			N2_REQUIRE(r.str(k), "n2_snapshot_open: '%s' has a non-string key", path);
			double d;
			std::string sv;
			if (k == "n_params" && r.number(d)) sn->info.n_params = (uint32_t)d;
			else if (k == "params_type" && r.str(sv)) { have_type = true; params_float = (sv == "float"); N2_REQUIRE(params_float || sv == "__half", "n2_snapshot_open: unknown params_type '%s'", sv.c_str()); }
			else if (k == "params_binary" && r.bin(sn->params.data, sn->params.bytes)) {}
			else if (k == "density_grid_size" && r.number(d)) sn->info.density_grid_size = (uint32_t)d;
			else if (k == "density_grid_binary" && r.bin(sn->density.data, sn->density.bytes)) {}
			else if (k == "training_step" && r.number(d)) sn->info.training_step = (uint32_t)d;
			else if (k == "loss" && r.number(d)) sn->info.loss = (float)d;
			else if (k == "optimizer") { sn->info.has_optimizer_state = 1; parse_optimizer(r, sn); }
			else if (k == "nerf") {
				uint32_t m;
				if (!r.map(m)) { r.skip(); continue; }
				for (uint32_t a = 0; a < m && r.ok; ++a) {
					std::string nk;
					N2_REQUIRE(r.str(nk), "n2_snapshot_open: '%s' has a non-string key", path);
					if (nk == "aabb_scale" && r.number(d)) sn->info.aabb_scale = (uint32_t)d;
					else if (nk == "rgb") {
						uint32_t q;
						if (!r.map(q)) { r.skip(); continue; }
						for (uint32_t b = 0; b < q && r.ok; ++b) {
							std::string rk;
							N2_REQUIRE(r.str(rk), "n2_snapshot_open: '%s' has a non-string key", path);
							if (rk == "rays_per_batch" && r.number(d)) sn->info.rays_per_batch = (uint32_t)d;
							else if (rk == "measured_batch_size" && r.number(d)) sn->info.measured_batch_size = (uint32_t)d;
							else if (rk == "measured_batch_size_before_compaction" && r.number(d)) sn->info.measured_batch_size_before_compaction = (uint32_t)d;
							else r.skip();
						}
					} else r.skip();
				}
			} else r.skip();
		}
	}
	N2_REQUIRE(r.ok, "n2_snapshot_open: '%s' is truncated or malformed", path);
	// load_snapshot: "does not contain a snapshot" (src/testbed.cu:3181-3184)
	N2_REQUIRE(found, "n2_snapshot_open: file '%s' does not contain a snapshot", path);
	N2_REQUIRE(sn->params.data != nullptr && have_type, "n2_snapshot_open: '%s' has no parameters", path);
	sn->info.params_are_fp32 = params_float ? 1 : 0;
	const uint64_t elem = params_float ? 4 : 2;
	N2_REQUIRE(sn->params.bytes == elem * sn->info.n_params, "n2_snapshot_open: params_binary holds %llu bytes, n_params %u of %llu bytes each were announced",
	           (unsigned long long)sn->params.bytes, sn->info.n_params, (unsigned long long)elem);
	sn->info.density_grid_cells = sn->density.bytes / 2;
	if (sn->info.has_optimizer_state) {
		const uint64_t want = 4ull * sn->info.n_params;
		const bool full = sn->m1.bytes == want && sn->m2.bytes == want && sn->steps.bytes == want;
		if (!full) sn->info.has_optimizer_state = 0;  // an optimizer object this build cannot map onto Adam's buffers
		sn->info.has_ema_weights = (sn->ema.bytes == want) ? 1 : 0;
	}
	return N2_OK;
}

N2_API int n2_snapshot_open(const char* path, n2_snapshot_t** out, n2_snapshot_info* info) {
	N2_REQUIRE(path != nullptr && out != nullptr, "n2_snapshot_open: null argument");
	*out = nullptr;
	FILE* f = fopen(path, "rb");
	N2_REQUIRE(f != nullptr, "n2_snapshot_open: cannot open '%s'", path);
	n2_snapshot* sn = new (std::nothrow) n2_snapshot();
	if (!sn) { fclose(f); n2_set_error("n2_snapshot_open: out of host memory"); return N2_ERR_INVALID_ARGUMENT; }
	memset(&sn->info, 0, sizeof(sn->info));
	fseek(f, 0, SEEK_END);
	const long size = ftell(f);
	fseek(f, 0, SEEK_SET);
	bool read_ok = size >= 0;
	if (read_ok) {
		sn->file.resize((size_t)size);
		read_ok = fread(sn->file.data(), 1, (size_t)size, f) == (size_t)size;
	}
	fclose(f);
	if (!read_ok) { delete sn; n2_set_error("n2_snapshot_open: cannot read '%s'", path); return N2_ERR_INVALID_ARGUMENT; }
	const int rc = parse_snapshot(sn, path);
	if (rc != N2_OK) { delete sn; return rc; }
	if (info) *info = sn->info;
	*out = sn;
	return N2_OK;
}

N2_API void n2_snapshot_close(n2_snapshot_t* snapshot) { delete snapshot; }

N2_API int n2_snapshot_read(n2_snapshot_t* sn, n2_stream_t stream, const n2_snapshot_targets* t) {
	N2_REQUIRE(sn != nullptr && t != nullptr, "n2_snapshot_read: null argument");
	hipStream_t s = n2_stream(stream);
	const uint64_t n = sn->info.n_params;
	std::vector<uint16_t> narrow_steps;  // lives until the stream has been waited for
	if (t->d_master || t->d_params) {
		N2_REQUIRE(t->n_params == n, "n2_snapshot_read: the snapshot holds %llu parameters, the model has %u", (unsigned long long)n, t->n_params);
		N2_REQUIRE(t->d_scratch != nullptr && t->scratch_bytes >= sn->params.bytes, "n2_snapshot_read: the parameters need %llu bytes of device scratch",
		           (unsigned long long)sn->params.bytes);
		N2_HIP(hipMemcpyAsync(t->d_scratch, sn->params.data, sn->params.bytes, hipMemcpyHostToDevice, s));
		if (sn->info.params_are_fp32) {
			if (t->d_master) N2_HIP(hipMemcpyAsync(t->d_master, t->d_scratch, 4 * n, hipMemcpyDeviceToDevice, s));
			if (t->d_params) { snap_f32_to_f16_kernel<<<sgrid(n), dim3(256), 0, s>>>(n, reinterpret_cast<const float*>(t->d_scratch), reinterpret_cast<hf*>(t->d_params)); N2_LAUNCH_CHECK(); }
		} else {
			if (t->d_params) N2_HIP(hipMemcpyAsync(t->d_params, t->d_scratch, 2 * n, hipMemcpyDeviceToDevice, s));
			if (t->d_master) { snap_f16_to_f32_kernel<<<sgrid(n), dim3(256), 0, s>>>(n, reinterpret_cast<const hf*>(t->d_scratch), t->d_master); N2_LAUNCH_CHECK(); }
		}
		N2_HIP(hipStreamSynchronize(s));  // the scratch is reused below
	}
	if (t->d_density_grid) {
		// load_snapshot: "Incompatible grid size." / "Incompatible number of grid cascades." (src/testbed.cu:3194-3196, 3227-3231)
		N2_REQUIRE(sn->info.density_grid_size == 128, "n2_snapshot_read: incompatible grid size %u", sn->info.density_grid_size);
		N2_REQUIRE(sn->info.density_grid_cells == t->density_grid_cells || sn->info.density_grid_cells == 0,
		           "n2_snapshot_read: incompatible number of grid cascades (%llu cells in the file, %llu expected)",
		           (unsigned long long)sn->info.density_grid_cells, (unsigned long long)t->density_grid_cells);
		if (sn->info.density_grid_cells) {
			N2_REQUIRE(t->d_scratch != nullptr && t->scratch_bytes >= sn->density.bytes, "n2_snapshot_read: the density grid needs %llu bytes of device scratch",
			           (unsigned long long)sn->density.bytes);
			N2_HIP(hipMemcpyAsync(t->d_scratch, sn->density.data, sn->density.bytes, hipMemcpyHostToDevice, s));
			snap_f16_to_f32_kernel<<<sgrid(sn->info.density_grid_cells), dim3(256), 0, s>>>(sn->info.density_grid_cells, reinterpret_cast<const hf*>(t->d_scratch), t->d_density_grid);
			N2_LAUNCH_CHECK();
			N2_HIP(hipStreamSynchronize(s));
		}
	}
	if (t->d_first_moments || t->d_second_moments || t->d_param_steps) {
		N2_REQUIRE(sn->info.has_optimizer_state, "n2_snapshot_read: the snapshot holds no optimizer state");
		N2_REQUIRE(t->n_params == n, "n2_snapshot_read: the snapshot holds %llu parameters, the model has %u", (unsigned long long)n, t->n_params);
		if (t->d_first_moments) N2_HIP(hipMemcpyAsync(t->d_first_moments, sn->m1.data, 4 * n, hipMemcpyHostToDevice, s));
		if (t->d_second_moments) N2_HIP(hipMemcpyAsync(t->d_second_moments, sn->m2.data, 4 * n, hipMemcpyHostToDevice, s));
		N2_REQUIRE(t->param_steps_bits == 0 || t->param_steps_bits == 16 || t->param_steps_bits == 32, "n2_snapshot_read: step counters of %u bits", t->param_steps_bits);
		if (t->d_param_steps && t->param_steps_bits == 16) {
			narrow_steps.resize(n);
			for (uint64_t i = 0; i < n; ++i) {
				uint32_t v;
				std::memcpy(&v, sn->steps.data + 4 * i, 4);
				narrow_steps[i] = (uint16_t)(v < 65535u ? v : 65535u);
			}
			N2_HIP(hipMemcpyAsync(t->d_param_steps, narrow_steps.data(), 2 * n, hipMemcpyHostToDevice, s));
		} else if (t->d_param_steps) {
			N2_HIP(hipMemcpyAsync(t->d_param_steps, sn->steps.data, 4 * n, hipMemcpyHostToDevice, s));
		}
	}
	if (t->d_ema_weights) {
		N2_REQUIRE(sn->info.has_ema_weights, "n2_snapshot_read: the snapshot holds no Ema weights");
		N2_HIP(hipMemcpyAsync(t->d_ema_weights, sn->ema.data, 4 * n, hipMemcpyHostToDevice, s));
	}
	N2_HIP(hipStreamSynchronize(s));
	return N2_OK;
}
