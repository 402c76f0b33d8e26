// One training step on one GPU: sample generation, field forward over all
// marched samples, compositing / loss / compaction, roll-over to the target
// batch size, field forward + backward (first and second order), Adam.
// Everything is enqueued on the caller's stream, without host synchronisation,
// except that the sample generator of the FOLLOWING step (which depends only on
// the scene and the seed) may run ahead on a stream the trainer owns, into the
// other of two sample sets, while this step's field kernels occupy the GPU.
#include "n2_common.h"
#include "slab_reduce.h"


#include <cstring>
#include <new>

typedef _Float16 hf;

struct n2_trainer {
	n2_trainer_config cfg;
	n2_field_t* field;
	uint32_t n_params, n_matrix_params;
	unsigned char* ws;
	// parameters and optimiser state
	float* master;
	hf* params;
	hf* grads;
	float* m1;
	float* m2;
	void* steps;              // per-parameter step counters, steps_bits wide
	uint32_t steps_bits;
	float* ema_tmp;   // fp32 moving average of the fp16 weights (null without the Ema wrapper)
	hf* ema;          // its fp16 copy: the inference parameters
	uint32_t optimizer_steps;  // nested optimizer steps taken so far
	uint32_t ema_steps;        // steps the moving average has taken since it was last (re)started
	uint32_t training_step;    // m_training_step: steps taken so far, the clock of the encoding's progressive level mask
	// per-step buffers; everything the sample generator writes exists twice
	struct SampleSet {
		float* coords;            // [max_samples][7]
		float* xyz_rows;          // [3][n_inference of the generation]: the positions once more, as rows
		bool has_rows;            // the last generation into this set wrote them
		uint32_t* numsteps;       // [max_rays][2]
		uint32_t* ray_indices;    // [max_rays]
		float* rgb_target;        // [max_rays][3]
		uint32_t* counters;       // [0] live rays, [1] marched samples
		void* ws_sampler;
	} sets[2];
	hf* mlp_out;              // [max(max_samples, target)][16]
	hf* dloss;                // [target][16]
	float* coords_compacted;  // [target][7]
	uint32_t* src_index;      // [target] marched sample behind every compacted sample
	float* ray_loss;          // [max_rays]
	uint32_t* counters;       // [0] live rays, [1] marched samples, [2] compacted samples (+ [4] as float: loss)
	void* ws_composite;
	uint64_t ws_sampler_bytes, ws_composite_bytes;
	// forward pass in depth chunks (n2_trainer_set_depth_chunks)
	uint32_t chunk_size, chunk_rounds;
	uint32_t chunk_estimate[N2_CHUNK_MAX_ROUNDS];  // samples per round as last measured by the caller (0: not known)
	uint32_t chunk_parity;    // which of the two counter sets the next chunked step uses
	bool last_chunked;        // the last step ran in depth chunks
	uint32_t* chunk_list;     // [max_samples] marched samples in the order of their evaluation
	uint32_t* chunk_column;   // [max_samples] inverse map
	float* chunk_coords;      // [max_samples][7] coordinate rows in list order
	uint32_t* chunk_counts;   // [2][N2_CHUNK_MAX_ROUNDS]
	void* chunk_state;
	void* ws_field;
	// scene
	const n2_camera* cameras;
	uint32_t n_images;
	const float* rgba;
	const uint8_t* bitfield;
	uint32_t n_rays_total;
	// sample generation running ahead of the step that uses it
	hipStream_t side;
	bool ev_main_from_adam;   // ev_main stands for the completion of the last step's Adam launch
	hipEvent_t ev_main, ev_ready;
	bool pf_valid;
	bool view_taken;          // n2_trainer_last_step_view since the last step: the caller may have enqueued readers of the sample set
	hipStream_t last_stream;  // stream of the last step
	uint32_t pf_set, pf_n_rays, pf_n_inference, pf_seed, pf_ray_base;
	uint32_t last_set;
};

struct TrainerCarve {
	uint64_t master, params, grads, m1, m2, steps, ema_tmp, ema, coords[2], xyz_rows[2], mlp_out, dloss, coords_compacted, src_index, numsteps[2], ray_indices[2], rgb_target[2],
		set_counters[2], ray_loss, counters, chunk_counts, chunk_list, chunk_column, chunk_state, chunk_coords, ws_sampler[2], ws_composite, ws_field, total;
};

static inline uint64_t a256(uint64_t x) { return (x + 255) / 256 * 256; }

static int make_field(const n2_trainer_config* cfg, n2_field_t** f) { return n2_field_create(&cfg->field, f); }

static TrainerCarve trainer_carve(const n2_trainer_config* cfg, const n2_field_t* f) {
	TrainerCarve c{};
	uint64_t o = 0;
	auto take = [&](uint64_t bytes) { const uint64_t at = o; o = a256(o + bytes); return at; };
	const uint64_t np = n2_field_n_params(f), T = cfg->target_batch_size, S = cfg->max_samples, R = cfg->max_rays_per_batch;
	c.master = take(4 * np);
	c.params = take(2 * np);
	c.grads = take(2 * np);
	c.m1 = take(4 * np);
	c.m2 = take(4 * np);
	c.steps = take((n2_adam_counters_may_saturate(cfg->adam.beta1, cfg->adam.beta2) ? 2 : 4) * np);
	const bool ema = cfg->ema_decay > 0.f;
	c.ema_tmp = take(ema ? 4 * np : 0);
	c.ema = take(ema ? 2 * np : 0);
	for (int i = 0; i < 2; ++i) c.coords[i] = take(28 * S);
	for (int i = 0; i < 2; ++i) c.xyz_rows[i] = take(12 * S);
	c.mlp_out = take(32 * (S > T ? S : T));
	c.dloss = take(32 * T);
	c.coords_compacted = take(28 * T);
	c.src_index = take(4 * T);
	for (int i = 0; i < 2; ++i) {
		c.numsteps[i] = take(8 * R);
		c.ray_indices[i] = take(4 * R);
		c.rgb_target[i] = take(12 * R);
		c.set_counters[i] = take(64);
	}
	c.ray_loss = take(4 * R);
	c.counters = take(64);
	c.chunk_counts = take(2 * N2_CHUNK_MAX_ROUNDS * sizeof(uint32_t));
	c.chunk_list = take(4 * S);
	c.chunk_column = take(4 * S);
	c.chunk_state = take(n2_composite_chunk_state_bytes((uint32_t)R));
	c.chunk_coords = take(28 * S);
	for (int i = 0; i < 2; ++i) c.ws_sampler[i] = take(n2_sampler_workspace_bytes((uint32_t)R));
	c.ws_composite = take(n2_composite_workspace_bytes((uint32_t)R));
	c.ws_field = take(n2_field_workspace_bytes(f, (uint32_t)(S > T ? S : T), (uint32_t)T));
	c.total = o;
	return c;
}

static int check_cfg(const n2_trainer_config* cfg, const char* fn) {
	N2_REQUIRE(cfg != nullptr, "%s: config is null", fn);
	N2_REQUIRE(cfg->target_batch_size >= 8 && cfg->target_batch_size % 8 == 0, "%s: target_batch_size %u must be a positive multiple of 8", fn,
	           cfg->target_batch_size);
	N2_REQUIRE(cfg->max_samples >= cfg->target_batch_size && cfg->max_samples % 8 == 0, "%s: max_samples %u must be a multiple of 8 and >= target_batch_size", fn,
	           cfg->max_samples);
	N2_REQUIRE(cfg->max_rays_per_batch >= 1, "%s: max_rays_per_batch must be positive", fn);
	N2_REQUIRE(cfg->loss_scale > 0.f, "%s: loss_scale must be positive", fn);
	N2_REQUIRE(cfg->ema_decay >= 0.f && cfg->ema_decay < 1.f, "%s: ema_decay %g outside [0, 1)", fn, (double)cfg->ema_decay);
	return N2_OK;
}

N2_API uint64_t n2_trainer_workspace_bytes(const n2_trainer_config* cfg) {
	if (check_cfg(cfg, "n2_trainer_workspace_bytes") != N2_OK) return 0;
	n2_field_t* f = nullptr;
	if (make_field(cfg, &f) != N2_OK) return 0;
	const uint64_t total = trainer_carve(cfg, f).total;
	n2_field_destroy(f);
	return total;
}

__global__ void __launch_bounds__(256) trainer_cast_params_kernel(uint32_t n, const float* __restrict__ master, hf* __restrict__ params) {
	const uint32_t i = blockIdx.x * 256 + threadIdx.x;
	if (i < n) params[i] = (hf)master[i];
}

N2_API int n2_trainer_create(const n2_trainer_config* cfg, void* d_workspace, uint64_t workspace_bytes, n2_trainer_t** out) {
	N2_REQUIRE(out != nullptr, "n2_trainer_create: out is null");
	*out = nullptr;
	if (int rc = check_cfg(cfg, "n2_trainer_create")) return rc;
	N2_REQUIRE(d_workspace != nullptr && reinterpret_cast<uintptr_t>(d_workspace) % 256 == 0, "n2_trainer_create: workspace must be non-null and 256-byte aligned");
	n2_trainer* t = new (std::nothrow) n2_trainer();
	N2_REQUIRE(t != nullptr, "n2_trainer_create: out of host memory");
	*t = n2_trainer{};
	t->cfg = *cfg;
	int rc = make_field(cfg, &t->field);
	if (rc != N2_OK) { delete t; return rc; }
	const TrainerCarve c = trainer_carve(cfg, t->field);
	if (workspace_bytes < c.total) {
		n2_set_error("n2_trainer_create: %llu bytes given, %llu needed", (unsigned long long)workspace_bytes, (unsigned long long)c.total);
		n2_field_destroy(t->field);
		delete t;
		return N2_ERR_INVALID_ARGUMENT;
	}
	unsigned char* b = reinterpret_cast<unsigned char*>(d_workspace);
	t->ws = b;
	t->n_params = n2_field_n_params(t->field);
	uint32_t offs[5];
	n2_field_param_offsets(t->field, offs);
	t->n_matrix_params = offs[2];
	t->master = reinterpret_cast<float*>(b + c.master);
	t->params = reinterpret_cast<hf*>(b + c.params);
	t->grads = reinterpret_cast<hf*>(b + c.grads);
	t->m1 = reinterpret_cast<float*>(b + c.m1);
	t->m2 = reinterpret_cast<float*>(b + c.m2);
	t->steps = b + c.steps;
	t->steps_bits = n2_adam_counters_may_saturate(cfg->adam.beta1, cfg->adam.beta2) ? 16u : 32u;
	t->ema_tmp = cfg->ema_decay > 0.f ? reinterpret_cast<float*>(b + c.ema_tmp) : nullptr;
	t->ema = cfg->ema_decay > 0.f ? reinterpret_cast<hf*>(b + c.ema) : nullptr;
	t->optimizer_steps = 0;
	t->ema_steps = 0;
	t->training_step = 0;
	for (int i = 0; i < 2; ++i) {
		t->sets[i].coords = reinterpret_cast<float*>(b + c.coords[i]);
		t->sets[i].xyz_rows = reinterpret_cast<float*>(b + c.xyz_rows[i]);
		t->sets[i].numsteps = reinterpret_cast<uint32_t*>(b + c.numsteps[i]);
		t->sets[i].ray_indices = reinterpret_cast<uint32_t*>(b + c.ray_indices[i]);
		t->sets[i].rgb_target = reinterpret_cast<float*>(b + c.rgb_target[i]);
		t->sets[i].counters = reinterpret_cast<uint32_t*>(b + c.set_counters[i]);
		t->sets[i].ws_sampler = b + c.ws_sampler[i];
	}
	t->mlp_out = reinterpret_cast<hf*>(b + c.mlp_out);
	t->dloss = reinterpret_cast<hf*>(b + c.dloss);
	t->coords_compacted = reinterpret_cast<float*>(b + c.coords_compacted);
	t->src_index = reinterpret_cast<uint32_t*>(b + c.src_index);
	t->ray_loss = reinterpret_cast<float*>(b + c.ray_loss);
	t->counters = reinterpret_cast<uint32_t*>(b + c.counters);
	t->chunk_counts = reinterpret_cast<uint32_t*>(b + c.chunk_counts);
	t->chunk_list = reinterpret_cast<uint32_t*>(b + c.chunk_list);
	t->chunk_column = reinterpret_cast<uint32_t*>(b + c.chunk_column);
	t->chunk_state = b + c.chunk_state;
	t->chunk_coords = reinterpret_cast<float*>(b + c.chunk_coords);
	t->ws_sampler_bytes = c.ws_sampler[1] - c.ws_sampler[0];
	t->ws_composite = b + c.ws_composite;
	t->ws_composite_bytes = c.ws_field - c.ws_composite;
	t->ws_field = b + c.ws_field;
	const uint32_t S = cfg->max_samples > cfg->target_batch_size ? cfg->max_samples : cfg->target_batch_size;
	rc = n2_field_set_params(t->field, reinterpret_cast<const n2_half*>(t->params), reinterpret_cast<n2_half*>(t->grads));
	if (rc == N2_OK) rc = n2_field_set_workspace(t->field, t->ws_field, c.total - c.ws_field, S, cfg->target_batch_size);
	// optimiser state, gradients, counters and every per-step buffer start at zero (padding rows of a
	// batch are then valid positions with zero gradient)
	if (rc == N2_OK) rc = n2_fill_zero_u32(nullptr, b + c.grads, c.coords[0] - c.grads);
	if (rc == N2_OK) rc = n2_fill_zero_u32(nullptr, b + c.coords[0], c.ws_sampler[0] - c.coords[0]);
	if (rc == N2_OK && hipStreamSynchronize(nullptr) != hipSuccess) { n2_set_error("n2_trainer_create: workspace initialisation failed"); rc = N2_ERR_HIP; }
	if (rc == N2_OK && cfg->prefetch_samples) {
		// default priority on purpose: the stream only has to run beside the caller's, not ahead of it.  The two events order
		// kernels of this GPU only (the host never waits on them), so they skip the system-scope fence: 2.5 us per step
		if (hipStreamCreateWithFlags(&t->side, hipStreamNonBlocking) != hipSuccess ||
		    hipEventCreateWithFlags(&t->ev_main, hipEventDisableTiming | hipEventDisableSystemFence) != hipSuccess ||
		    hipEventCreateWithFlags(&t->ev_ready, hipEventDisableTiming | hipEventDisableSystemFence) != hipSuccess) {
			n2_set_error("n2_trainer_create: cannot create the sample-generation stream");
			rc = N2_ERR_HIP;
		}
	}
	if (rc != N2_OK) {
		n2_trainer_destroy(t);
		return rc;
	}
	*out = t;
	return N2_OK;
}

N2_API void n2_trainer_destroy(n2_trainer_t* t) {
	if (!t) return;
	if (t->side) { (void)hipStreamSynchronize(t->side); (void)hipStreamDestroy(t->side); }
	if (t->ev_main) (void)hipEventDestroy(t->ev_main);
	if (t->ev_ready) (void)hipEventDestroy(t->ev_ready);
	n2_field_destroy(t->field);
	delete t;
}

N2_API int n2_trainer_buffers(n2_trainer_t* t, float** d_master, n2_half** d_params, n2_half** d_gradients, uint32_t* n_params) {
	N2_REQUIRE(t != nullptr, "n2_trainer_buffers: trainer is null");
	if (d_master) *d_master = t->master;
	if (d_params) *d_params = reinterpret_cast<n2_half*>(t->params);
	if (d_gradients) *d_gradients = reinterpret_cast<n2_half*>(t->grads);
	if (n_params) *n_params = t->n_params;
	return N2_OK;
}

N2_API int n2_trainer_sync_params(n2_trainer_t* t, n2_stream_t stream) {
	N2_REQUIRE(t != nullptr, "n2_trainer_sync_params: trainer is null");
	trainer_cast_params_kernel<<<dim3((t->n_params + 255) / 256), dim3(256), 0, n2_stream(stream)>>>(t->n_params, t->master, t->params);
	N2_LAUNCH_CHECK();
	return N2_OK;
}

N2_API n2_field_t* n2_trainer_field(n2_trainer_t* t) { return t ? t->field : nullptr; }

N2_API int n2_trainer_set_scene(n2_trainer_t* t, const n2_camera* d_cameras, uint32_t n_images, const float* d_rgba, const uint8_t* d_bitfield) {
	N2_REQUIRE(t != nullptr, "n2_trainer_set_scene: trainer is null");
	N2_REQUIRE(d_cameras && d_rgba && d_bitfield && n_images > 0, "n2_trainer_set_scene: null scene buffer or no images");
	// a sample generation that is still running ahead reads the previous scene
	if (t->side) N2_HIP(hipStreamSynchronize(t->side));
	t->pf_valid = false;
	t->cameras = d_cameras; t->n_images = n_images; t->rgba = d_rgba; t->bitfield = d_bitfield;
	return N2_OK;
}

N2_API int n2_trainer_invalidate_prefetch(n2_trainer_t* t) {
	N2_REQUIRE(t != nullptr, "n2_trainer_invalidate_prefetch: trainer is null");
	if (t->side) N2_HIP(hipStreamSynchronize(t->side));
	t->pf_valid = false;
	return N2_OK;
}

N2_API int n2_trainer_step(n2_trainer_t* t, n2_stream_t stream, uint32_t n_rays, uint32_t n_inference, uint32_t seed) {
	N2_REQUIRE(t != nullptr, "n2_trainer_step: trainer is null");
	N2_REQUIRE(t->cameras != nullptr, "n2_trainer_step: n2_trainer_set_scene has not been called");
	N2_REQUIRE(n_rays >= 1 && n_rays <= t->cfg.max_rays_per_batch, "n2_trainer_step: n_rays %u outside [1, %u]", n_rays, t->cfg.max_rays_per_batch);
	N2_REQUIRE(n_inference % 8 == 0 && n_inference <= t->cfg.max_samples, "n2_trainer_step: n_inference %u must be a multiple of 8 and <= %u",
	           n_inference, t->cfg.max_samples);
	hipStream_t s = n2_stream(stream);
	const uint32_t T = t->cfg.target_batch_size;
	uint32_t* compacted_counter = t->counters + 2;
	// progressive level mask: the encoding is told the number of training steps taken so far before every step
	// (Testbed::train, src/testbed.cu:2641-2647)
	if (int rc = n2_grid_set_training_step(n2_field_encoding(t->field), t->training_step)) return rc;
	// the colour rows of dL/doutput are at most 0.05 * loss_scale / n_rays: the colour net's backward lifts them out of
	// fp16's subnormal range by an exact power of two
	if (int rc = n2_field_set_colour_gradient_exponent(t->field, n2_colour_gradient_exponent(t->cfg.loss_scale, n_rays))) return rc;
	// A step in depth rounds reads its positions from the rounds' lists: the generator then leaves the rows out (on a trained
	// field it writes three times the samples, beside the forward's first round)
	const bool want_rows = !(t->chunk_rounds >= 2 && !t->cfg.recompute_training_forward);
	auto sample = [&](n2_trainer::SampleSet& set, hipStream_t on, uint32_t ray_base, uint32_t sd) {
		set.has_rows = want_rows;
		// rays -> marched samples (capacity n_inference: rays that do not fit are dropped, as when max_samples is reached)
		// (the positions also as three rows of n_inference floats, for the field's gather)
		return n2_generate_training_samples_rows(reinterpret_cast<n2_stream_t>(on), n_rays, ray_base, sd, t->cameras, t->n_images, t->rgba,
		                                         t->cfg.composite.background, t->bitfield, n_inference, set.counters, set.counters + 1, set.ray_indices,
		                                         set.numsteps, set.rgb_target, set.coords, set.ws_sampler, t->ws_sampler_bytes, want_rows ? set.xyz_rows : nullptr);
	};
	// the following step's samples on the side stream, assuming the same ray count and the next seed
	bool main_event_is_last_step = false;
	auto prefetch = [&](uint32_t cur_set) -> int {
		t->pf_valid = false;
		// The generator overwrites the other sample set, which the previous step's kernels read: it waits for that step's
		// last launch, whose completion is ev_main (no packet on s).  When anything else may have been enqueued on s since
		// (the first step, a step that missed its prefetch: the caller has changed the scene, the bitfield or the
		// arguments), the event is recorded here, behind everything on s.
		if (!main_event_is_last_step) N2_HIP(hipEventRecord(t->ev_main, s));
		N2_HIP(hipStreamWaitEvent(t->side, t->ev_main, 0));
		if (int rc = sample(t->sets[1u - cur_set], t->side, t->n_rays_total, seed + 1)) return rc;
		N2_HIP(hipEventRecord(t->ev_ready, t->side));
		t->pf_valid = true; t->pf_set = 1u - cur_set; t->pf_n_rays = n_rays; t->pf_n_inference = n_inference; t->pf_seed = seed + 1; t->pf_ray_base = t->n_rays_total;
		return N2_OK;
	};
	uint32_t cur;
	if (t->side) {
		const bool hit = t->pf_valid && t->pf_n_rays == n_rays && t->pf_n_inference == n_inference && t->pf_seed == seed && t->pf_ray_base == t->n_rays_total;
		if (hit) {
			cur = t->pf_set;
			// ev_main stands for the last step's Adam launch: enough unless the caller may have put readers of that step's
			// buffers on the stream since (it asked for the view), or this step runs on another stream
			main_event_is_last_step = t->ev_main_from_adam && !t->view_taken && s == t->last_stream;
			N2_HIP(hipStreamWaitEvent(s, t->ev_ready, 0));
		} else {
			// a generation that ran ahead with other arguments is abandoned (it stays ordered on the side stream)
			cur = t->pf_valid ? 1u - t->pf_set : 1u - t->last_set;
			if (int rc = sample(t->sets[cur], s, t->n_rays_total, seed)) return rc;
		}
		t->n_rays_total += n_rays;
		if (int rc = prefetch(cur)) return rc;
	} else {
		cur = 0;
		if (int rc = sample(t->sets[0], s, t->n_rays_total, seed)) return rc;
		t->n_rays_total += n_rays;
	}
	t->last_set = cur;
	t->view_taken = false;
	t->last_stream = s;
	const n2_trainer::SampleSet& set = t->sets[cur];
	const uint32_t* ray_counter = set.counters;
	n2_composite_config cc = t->cfg.composite;
	cc.n_rays_norm = n_rays;
	cc.loss_scale = t->cfg.loss_scale;
	const bool chunked = t->chunk_rounds >= 2 && !t->cfg.recompute_training_forward;

	if (chunked) {
		// the field over the marched samples in depth chunks: only what lies in front of the rays' cuts (and at most a chunk
		// behind them) is evaluated
		uint32_t* counts = t->chunk_counts + N2_CHUNK_MAX_ROUNDS * t->chunk_parity;
		uint32_t* counts_other = t->chunk_counts + N2_CHUNK_MAX_ROUNDS * (1u - t->chunk_parity);
		t->chunk_parity ^= 1u;
		for (uint32_t round = 0; round < t->chunk_rounds; ++round) {
			const uint32_t chunk = round + 1 == t->chunk_rounds ? 0xFFFFFFFFu : t->chunk_size;
			if (int rc = n2_composite_chunk_next(stream, &cc, n_rays, ray_counter, set.numsteps, reinterpret_cast<const n2_half*>(t->mlp_out), set.coords, round, chunk,
			                                     t->chunk_state, counts, counts_other, t->chunk_list, t->chunk_column, t->chunk_coords)) return rc;
			// the launches are sized by what the caller measured on earlier steps (with a margin), else by the most a round can hold
			const uint64_t most = round + 1 == t->chunk_rounds ? n_inference : (uint64_t)n_rays * t->chunk_size;
			uint64_t est = t->chunk_estimate[round] ? (uint64_t)t->chunk_estimate[round] * 9 / 8 + 1024 : most;
			if (est > most) est = most;
			if (est > n_inference) est = n_inference;
			if (int rc = n2_field_forward_listed(t->field, stream, t->chunk_coords, n_inference, t->chunk_list, counts, round, (uint32_t)est,
			                                     reinterpret_cast<n2_half*>(t->mlp_out))) return rc;
		}
	} else {
		// field over every marched sample: the window of n_inference samples, of which the generator filled set.counters[1]
		if (int rc = n2_field_forward_live(t->field, stream, set.coords, n_inference, set.counters + 1, reinterpret_cast<n2_half*>(t->mlp_out), set.has_rows ? set.xyz_rows : nullptr)) return rc;
	}
	t->last_chunked = chunked;
	// compositing, loss, gradients w.r.t. the outputs, compaction
	// (the compacted batch comes back filled up to exactly T samples: fill_rollover_and_rescale on the output gradients,
	// fill_rollover on the coordinates, src/testbed_nerf.cu:3908-3916)
	if (int rc = n2_composite_loss_filled(stream, &cc, n_rays, ray_counter, set.numsteps, reinterpret_cast<const n2_half*>(t->mlp_out), set.coords,
	                                      set.rgb_target, T, compacted_counter, t->coords_compacted, reinterpret_cast<n2_half*>(t->dloss),
	                                      t->ray_loss, t->src_index, t->ws_composite, t->ws_composite_bytes, true, chunked ? t->chunk_column : nullptr)) return rc;
	// forward + backward on the compacted batch, then the optimiser.  Every compacted sample is one of the marched
	// samples the field has just been evaluated on: unless asked to run the field again, the activations saved for it
	// are selected instead (the same values, a fraction of the work).
	if (t->cfg.recompute_training_forward) {
		if (int rc = n2_field_forward(t->field, stream, t->coords_compacted, T, reinterpret_cast<n2_half*>(t->mlp_out))) return rc;
	} else {
		if (int rc = n2_field_select_borrow(t->field, t->src_index, n_inference, T)) return rc;
	}
	// the summation of the networks' weight-gradient slabs rides in the optimiser's kernel instead of taking a launch
	N2SlabReduce sums;
	if (int rc = n2_field_backward_deferred(t->field, stream, t->coords_compacted, T, reinterpret_cast<const n2_half*>(t->dloss), T, N2_GRAD_OVERWRITE, &sums)) return rc;
	// a step whose rays kept no sample (counter 2 is zero) must not apply the previous step's gradients again.  The step's
	// bookkeeping rides along: the sum of the live rays' losses (counter 4, as a float) and the sample set's counters
	N2StepEpilogue epi{};
	epi.values = t->ray_loss; epi.n_ptr = ray_counter; epi.n_max = n_rays; epi.sum_out = reinterpret_cast<float*>(t->counters) + 4;
	epi.copy_src = set.counters; epi.copy_dst = t->counters; epi.copy_n = 2;
	if (int rc = n2_adam_step_gated(stream, &t->cfg.adam, t->n_params, t->n_matrix_params, t->cfg.loss_scale, t->master, reinterpret_cast<n2_half*>(t->params),
	                                reinterpret_cast<const n2_half*>(t->grads), t->m1, t->m2, t->steps, t->steps_bits, compacted_counter, &sums, &epi,
	                                t->side ? t->ev_main : nullptr)) return rc;
	t->ev_main_from_adam = t->side != nullptr;
	t->optimizer_steps += 1;
	t->training_step += 1;
	if (t->ema) {
		t->ema_steps += 1;
		return n2_ema_step(stream, t->n_params, t->cfg.ema_decay, t->ema_steps, reinterpret_cast<const n2_half*>(t->params), t->ema_tmp,
		                   reinterpret_cast<n2_half*>(t->ema));
	}
	return N2_OK;
}

N2_API int n2_trainer_set_depth_chunks(n2_trainer_t* t, uint32_t chunk_size, uint32_t n_rounds) {
	N2_REQUIRE(t != nullptr, "n2_trainer_set_depth_chunks: trainer is null");
	N2_REQUIRE(n_rounds <= N2_CHUNK_MAX_ROUNDS, "n2_trainer_set_depth_chunks: %u rounds, at most %u", n_rounds, N2_CHUNK_MAX_ROUNDS);
	N2_REQUIRE(n_rounds < 2 || chunk_size >= 1, "n2_trainer_set_depth_chunks: chunk_size must be positive");
	t->chunk_size = chunk_size;
	t->chunk_rounds = n_rounds < 2 ? 0u : n_rounds;
	for (uint32_t r = 0; r < N2_CHUNK_MAX_ROUNDS; ++r) t->chunk_estimate[r] = 0;
	return N2_OK;
}

N2_API int n2_trainer_set_depth_chunk_estimates(n2_trainer_t* t, const uint32_t* samples_per_round, uint32_t n_rounds) {
	N2_REQUIRE(t != nullptr && (samples_per_round != nullptr || n_rounds == 0), "n2_trainer_set_depth_chunk_estimates: null argument");
	N2_REQUIRE(n_rounds <= N2_CHUNK_MAX_ROUNDS, "n2_trainer_set_depth_chunk_estimates: %u rounds, at most %u", n_rounds, N2_CHUNK_MAX_ROUNDS);
	for (uint32_t r = 0; r < N2_CHUNK_MAX_ROUNDS; ++r) t->chunk_estimate[r] = r < n_rounds ? samples_per_round[r] : 0u;
	return N2_OK;
}

N2_API int n2_trainer_set_learning_rate(n2_trainer_t* t, float learning_rate) {
	N2_REQUIRE(t != nullptr, "n2_trainer_set_learning_rate: trainer is null");
	N2_REQUIRE(learning_rate >= 0.f, "n2_trainer_set_learning_rate: negative learning rate");
	t->cfg.adam.learning_rate = learning_rate;
	return N2_OK;
}

N2_API int n2_trainer_optimizer_state(n2_trainer_t* t, n2_trainer_optimizer_buffers* out) {
	N2_REQUIRE(t != nullptr && out != nullptr, "n2_trainer_optimizer_state: null argument");
	out->first_moments = t->m1;
	out->second_moments = t->m2;
	out->param_steps = t->steps;
	out->param_steps_bits = t->steps_bits;
	out->ema_weights = t->ema_tmp;
	out->inference_params = reinterpret_cast<n2_half*>(t->ema ? t->ema : t->params);
	out->optimizer_steps = t->optimizer_steps;
	out->learning_rate = t->cfg.adam.learning_rate;
	return N2_OK;
}

__global__ void __launch_bounds__(256) trainer_restart_ema_kernel(uint32_t n, const hf* __restrict__ params, float* __restrict__ tmp, hf* __restrict__ ema) {
	const uint32_t i = blockIdx.x * 256 + threadIdx.x;
	if (i < n) { tmp[i] = (float)params[i]; ema[i] = params[i]; }
}

N2_API int n2_trainer_restart_ema(n2_trainer_t* t, n2_stream_t stream, uint32_t ema_steps) {
	N2_REQUIRE(t != nullptr, "n2_trainer_restart_ema: trainer is null");
	t->ema_steps = ema_steps;
	if (t->ema == nullptr || ema_steps != 0) return N2_OK;
	trainer_restart_ema_kernel<<<dim3((t->n_params + 255) / 256), dim3(256), 0, n2_stream(stream)>>>(t->n_params, t->params, t->ema_tmp, t->ema);
	N2_LAUNCH_CHECK();
	return N2_OK;
}

N2_API int n2_trainer_set_training_step(n2_trainer_t* t, uint32_t step) {
	N2_REQUIRE(t != nullptr, "n2_trainer_set_training_step: trainer is null");
	t->training_step = step;
	return n2_grid_set_training_step(n2_field_encoding(t->field), step);
}

N2_API int n2_trainer_set_optimizer_steps(n2_trainer_t* t, uint32_t steps) {
	N2_REQUIRE(t != nullptr, "n2_trainer_set_optimizer_steps: trainer is null");
	t->optimizer_steps = steps;
	return N2_OK;
}

N2_API int n2_trainer_last_step_view(n2_trainer_t* t, n2_trainer_step_view* out) {
	N2_REQUIRE(t != nullptr && out != nullptr, "n2_trainer_last_step_view: null argument");
	const n2_trainer::SampleSet& set = t->sets[t->last_set];
	t->view_taken = true;
	out->coords = set.coords;
	out->numsteps = set.numsteps;
	out->rgb_target = set.rgb_target;
	out->ray_indices = set.ray_indices;
	out->network_output = reinterpret_cast<const n2_half*>(t->mlp_out);
	out->coords_compacted = t->coords_compacted;
	out->dloss_doutput = reinterpret_cast<const n2_half*>(t->dloss);
	out->source_index = t->src_index;
	out->evaluated_samples = t->last_chunked ? t->chunk_list : nullptr;
	out->evaluated_counts = t->last_chunked ? t->chunk_counts + N2_CHUNK_MAX_ROUNDS * (1u - t->chunk_parity) : nullptr;
	return N2_OK;
}

N2_API int n2_trainer_read_counters(n2_trainer_t* t, n2_stream_t stream, uint32_t* rays, uint32_t* samples, uint32_t* compacted, float* loss) {
	N2_REQUIRE(t != nullptr, "n2_trainer_read_counters: trainer is null");
	uint32_t host[8] = {};
	N2_HIP(hipMemcpyAsync(host, t->counters, sizeof(host), hipMemcpyDeviceToHost, n2_stream(stream)));
	N2_HIP(hipStreamSynchronize(n2_stream(stream)));
	if (rays) *rays = host[0];
	if (samples) *samples = host[1];
	if (compacted) *compacted = host[2];
	if (loss) { float f; memcpy(&f, &host[4], 4); *loss = f; }
	return N2_OK;
}
