// neus2_amd.hpp - header-only C++ shim over the C ABI (neus2_amd.h) that keeps the method names,
// argument order and error behaviour of the tcnn-style interface the reference programs against:
//   tcnn::Encoding<T>   (GridEncoding created at nerf_network.h:46)
//   tcnn::Network<T>    (FullyFusedMLP created at nerf_network.h:57, 65)
//   NerfNetwork<T>      (include/neural-graphics-primitives/nerf_network.h)
// Differences a caller has to know about:
//   * Matrices are non-owning views (pointer + shape + layout); nothing here allocates device memory.
//     Where tcnn takes temporaries from its stream-ordered arena, the caller hands in a buffer
//     (set_workspace, and the Jacobian buffer of GridEncoding::forward).
//   * T is fixed to IEEE binary16, passed as n2::half_t (uint16_t storage).
//   * Streams are hipStream_t passed as void*.
//   * Failures throw std::runtime_error with the library's message, like CUDA_CHECK_THROW in the reference.
#ifndef NEUS2_AMD_HPP
#define NEUS2_AMD_HPP

#include <cstddef>
#include <cstdint>
#include <memory>
#include <stdexcept>
#include <string>

#include "neus2_amd.h"

namespace n2 {

using half_t = n2_half;
using stream_t = n2_stream_t;

inline void check(int status, const char* what) {
	if (status != N2_OK) throw std::runtime_error(std::string(what) + ": " + n2_last_error());
}

// tcnn::EGradientMode
enum class GradientMode : int { Ignore = N2_GRAD_IGNORE, Overwrite = N2_GRAD_OVERWRITE, Accumulate = N2_GRAD_ACCUMULATE };

// tcnn::MatrixLayout.  RowMajor / SoA: element (r, i) at r * n + i.  ColumnMajor / AoS: at i * stride + r.
enum class MatrixLayout : int { RowMajor = 0, SoA = 0, ColumnMajor = 1, AoS = 1 };
constexpr MatrixLayout RM = MatrixLayout::RowMajor, CM = MatrixLayout::ColumnMajor, SoA = MatrixLayout::SoA, AoS = MatrixLayout::AoS;

// tcnn::GPUMatrixDynamic<T> as a view: m rows (features), n columns (batch).
template <typename T>
class GPUMatrixDynamic {
public:
	GPUMatrixDynamic() = default;
	GPUMatrixDynamic(T* data, uint32_t m, uint32_t n, MatrixLayout layout = CM, uint32_t stride = 0)
		: m_data(data), m_rows(m), m_cols(n), m_layout(layout), m_stride(stride ? stride : (layout == CM ? m : n)) {}
	T* data() const { return m_data; }
	uint32_t m() const { return m_rows; }
	uint32_t rows() const { return m_rows; }
	uint32_t n() const { return m_cols; }
	uint32_t cols() const { return m_cols; }
	uint32_t stride() const { return m_stride; }
	MatrixLayout layout() const { return m_layout; }
	// rows [offset, offset + n_rows) as a view with the same stride (common_operation.cuh's slice_rows)
	GPUMatrixDynamic<T> slice_rows(uint32_t offset, uint32_t n_rows) const {
		if (offset + n_rows > m_rows) throw std::runtime_error("slice_rows: out of range");
		T* p = m_layout == CM ? m_data + offset : m_data + (size_t)offset * m_stride;
		return GPUMatrixDynamic<T>(p, n_rows, m_cols, m_layout, m_stride);
	}
private:
	T* m_data = nullptr;
	uint32_t m_rows = 0, m_cols = 0;
	MatrixLayout m_layout = CM;
	uint32_t m_stride = 0;
};

// tcnn::Context
struct Context {
	virtual ~Context() = default;
};

namespace detail {
// position strides of a 3-row fp32 matrix as n2_grid_* wants them
inline void position_strides(const GPUMatrixDynamic<float>& in, uint32_t& point_stride, uint32_t& dim_stride) {
	if (in.m() < 3) throw std::runtime_error("positions need at least 3 rows");
	if (in.layout() == CM) { point_stride = in.stride(); dim_stride = 1; }
	else { point_stride = 1; dim_stride = in.stride(); }
}
template <typename T>
inline void require_soa(const GPUMatrixDynamic<T>& mat, uint32_t rows, uint32_t n, const char* what) {
	if (mat.layout() != SoA || mat.m() != rows || mat.n() != n || mat.stride() != n)
		throw std::runtime_error(std::string(what) + ": expected a dense SoA (row-major) matrix of " + std::to_string(rows) + " x " + std::to_string(n));
}
}  // namespace detail

// ---------------------------------------------------------------------------------------------
// tcnn::GridEncoding<__half, 3, 2> (HashGrid)
// ---------------------------------------------------------------------------------------------
class GridEncoding {
public:
	GridEncoding(uint32_t n_levels, uint32_t n_features_per_level, uint32_t log2_hashmap_size, uint32_t base_resolution,
	             float per_level_scale) {
		check(n2_grid_create(n_levels, n_features_per_level, log2_hashmap_size, base_resolution, per_level_scale, &m_grid), "GridEncoding");
	}
	~GridEncoding() { n2_grid_destroy(m_grid); }
	GridEncoding(const GridEncoding&) = delete;
	GridEncoding& operator=(const GridEncoding&) = delete;

	uint32_t input_width() const { return 3; }
	uint32_t output_width() const { return n2_grid_output_width(m_grid); }
	uint32_t padded_output_width() const { return n2_grid_output_width(m_grid); }
	uint32_t required_input_alignment() const { return 1; }
	size_t n_params() const { return n2_grid_n_params(m_grid); }
	MatrixLayout preferred_output_layout() const { return SoA; }
	n2_grid_t* handle() const { return m_grid; }

	// Encoding::set_params(params, inference_params, backward_params, gradients): one fp16 copy serves all three roles
	void set_params(half_t* params, half_t* /*inference_params*/, half_t* /*backward_params*/, half_t* gradients) {
		check(n2_grid_set_params(m_grid, params, gradients), "GridEncoding::set_params");
	}
	// level mask (GridEncoding::set_max_level / set_max_level_gpu, Encoding::set_training_step)
	void set_max_level(float value) { check(n2_grid_set_max_level(m_grid, value), "GridEncoding::set_max_level"); }
	void set_max_level_gpu(const float* d_value) { check(n2_grid_set_max_level_gpu(m_grid, d_value), "GridEncoding::set_max_level_gpu"); }
	void set_progressive(float base_valid_level_scale, float valid_level_scale, uint32_t base_training_step) {
		check(n2_grid_set_progressive(m_grid, base_valid_level_scale, valid_level_scale, base_training_step), "GridEncoding::set_progressive");
	}
	void set_training_step(int training_step) {
		check(n2_grid_set_training_step(m_grid, training_step < 0 ? 0u : (uint32_t)training_step), "GridEncoding::set_training_step");
	}
	// scratch of the parameter-gradient scatter (tcnn: arena temporaries)
	size_t workspace_bytes(uint32_t max_points) const { return n2_grid_workspace_bytes(m_grid, max_points); }
	void set_workspace(void* d_workspace, size_t n_bytes, uint32_t max_points) {
		check(n2_grid_set_workspace(m_grid, d_workspace, n_bytes, max_points), "GridEncoding::set_workspace");
	}

	struct ForwardContext : Context {
		float* dy_dx = nullptr;  // fp32 [output_width][N][3]
	};

	// Encoding::forward(stream, input, &output, use_inference_params, prepare_input_gradients).
	// d_dy_dx: caller-owned buffer of output_width * N * 3 floats, required when prepare_input_gradients is set.
	std::unique_ptr<Context> forward(stream_t stream, const GPUMatrixDynamic<float>& input, GPUMatrixDynamic<half_t>* output,
	                                 bool /*use_inference_params*/ = false, bool prepare_input_gradients = false, float* d_dy_dx = nullptr) {
		if (!output) throw std::runtime_error("GridEncoding::forward: output is required");
		if (prepare_input_gradients && !d_dy_dx) throw std::runtime_error("GridEncoding::forward: prepare_input_gradients needs a Jacobian buffer");
		uint32_t ps, ds;
		detail::position_strides(input, ps, ds);
		detail::require_soa(*output, output_width(), input.n(), "GridEncoding::forward output");
		check(n2_grid_forward(m_grid, stream, input.data(), ps, ds, input.n(), output->data(), prepare_input_gradients ? d_dy_dx : nullptr),
		      "GridEncoding::forward");
		auto ctx = std::make_unique<ForwardContext>();
		ctx->dy_dx = prepare_input_gradients ? d_dy_dx : nullptr;
		return ctx;
	}

	// Encoding::backward(stream, ctx, input, output, dL_doutput, &dL_dinput, use_inference_params, mode)
	void backward(stream_t stream, const Context& ctx, const GPUMatrixDynamic<float>& input, const GPUMatrixDynamic<half_t>& /*output*/,
	              const GPUMatrixDynamic<half_t>& dL_doutput, GPUMatrixDynamic<float>* dL_dinput = nullptr,
	              bool /*use_inference_params*/ = false, GradientMode mode = GradientMode::Overwrite) {
		const auto& fc = static_cast<const ForwardContext&>(ctx);
		uint32_t ps, ds;
		detail::position_strides(input, ps, ds);
		detail::require_soa(dL_doutput, output_width(), input.n(), "GridEncoding::backward dL_doutput");
		if (dL_dinput) detail::require_soa(*dL_dinput, 3, input.n(), "GridEncoding::backward dL_dinput");
		check(n2_grid_backward(m_grid, stream, input.data(), ps, ds, input.n(), dL_doutput.data(), fc.dy_dx,
		                       dL_dinput ? dL_dinput->data() : nullptr, (n2_grad_mode)mode), "GridEncoding::backward");
	}

	// Encoding::backward_backward_input(stream, ctx, input, dL_ddLdinput, dL_doutput, &dL_ddLdoutput, &dL_dinput,
	//                                   use_inference_params, mode), nerf_network.h:534-544
	void backward_backward_input(stream_t stream, const Context& /*ctx*/, const GPUMatrixDynamic<float>& input,
	                             const GPUMatrixDynamic<float>& dL_ddLdinput, const GPUMatrixDynamic<half_t>& dL_doutput,
	                             GPUMatrixDynamic<half_t>* dL_ddLdoutput = nullptr, GPUMatrixDynamic<float>* dL_dinput = nullptr,
	                             bool /*use_inference_params*/ = false, GradientMode mode = GradientMode::Overwrite) {
		uint32_t ps, ds;
		detail::position_strides(input, ps, ds);
		detail::require_soa(dL_ddLdinput, 3, input.n(), "GridEncoding::backward_backward_input dL_ddLdinput");
		detail::require_soa(dL_doutput, output_width(), input.n(), "GridEncoding::backward_backward_input dL_doutput");
		if (dL_ddLdoutput) detail::require_soa(*dL_ddLdoutput, output_width(), input.n(), "GridEncoding::backward_backward_input dL_ddLdoutput");
		if (dL_dinput) detail::require_soa(*dL_dinput, 3, input.n(), "GridEncoding::backward_backward_input dL_dinput");
		check(n2_grid_backward_backward_input(m_grid, stream, input.data(), ps, ds, input.n(), dL_ddLdinput.data(), dL_doutput.data(),
		                                      dL_ddLdoutput ? dL_ddLdoutput->data() : nullptr, dL_dinput ? dL_dinput->data() : nullptr,
		                                      (n2_grad_mode)mode), "GridEncoding::backward_backward_input");
	}

private:
	n2_grid_t* m_grid = nullptr;
};

// ---------------------------------------------------------------------------------------------
// tcnn::FullyFusedMLP<__half, 64>: ReLU hidden layers, 16 linear outputs, no bias
// ---------------------------------------------------------------------------------------------
class FullyFusedMLP {
public:
	FullyFusedMLP(uint32_t input_width, uint32_t n_hidden_layers) {
		check(n2_mlp_create(input_width, n_hidden_layers, &m_mlp), "FullyFusedMLP");
	}
	~FullyFusedMLP() { n2_mlp_destroy(m_mlp); }
	FullyFusedMLP(const FullyFusedMLP&) = delete;
	FullyFusedMLP& operator=(const FullyFusedMLP&) = delete;

	uint32_t input_width() const { return n2_mlp_input_width(m_mlp); }
	uint32_t output_width() const { return n2_mlp_output_width(m_mlp); }
	uint32_t padded_output_width() const { return n2_mlp_output_width(m_mlp); }
	uint32_t required_input_alignment() const { return 16; }
	size_t n_params() const { return n2_mlp_n_params(m_mlp); }
	n2_mlp_t* handle() const { return m_mlp; }

	void set_params(half_t* params, half_t* /*inference_params*/, half_t* /*backward_params*/, half_t* gradients) {
		check(n2_mlp_set_params(m_mlp, params, gradients), "FullyFusedMLP::set_params");
	}
	size_t workspace_bytes() const { return n2_mlp_workspace_bytes(m_mlp); }
	void set_workspace(void* d_workspace, size_t n_bytes) { check(n2_mlp_set_workspace(m_mlp, d_workspace, n_bytes), "FullyFusedMLP::set_workspace"); }

	// Network::forward / inference_mixed_precision: SoA input; the output may be SoA (16 x N) or AoS (N x 16).
	// The hidden activations are recomputed by the backward passes, so the context is empty.
	std::unique_ptr<Context> forward(stream_t stream, const GPUMatrixDynamic<half_t>& input, GPUMatrixDynamic<half_t>* output,
	                                 bool /*use_inference_params*/ = false, bool /*prepare_input_gradients*/ = false) {
		inference_mixed_precision(stream, input, *output);
		return std::make_unique<Context>();
	}
	void inference_mixed_precision(stream_t stream, const GPUMatrixDynamic<half_t>& input, GPUMatrixDynamic<half_t>& output,
	                               bool /*use_inference_params*/ = true) {
		detail::require_soa(input, input_width(), input.n(), "FullyFusedMLP input");
		check(n2_mlp_forward(m_mlp, stream, input.data(), input.n(), output.data(), out_layout(output, input.n()), nullptr), "FullyFusedMLP::forward");
	}
	void backward(stream_t stream, const Context& /*ctx*/, const GPUMatrixDynamic<half_t>& input, const GPUMatrixDynamic<half_t>& /*output*/,
	              const GPUMatrixDynamic<half_t>& dL_doutput, GPUMatrixDynamic<half_t>* dL_dinput = nullptr,
	              bool /*use_inference_params*/ = false, GradientMode mode = GradientMode::Overwrite) {
		detail::require_soa(input, input_width(), input.n(), "FullyFusedMLP input");
		if (dL_dinput) detail::require_soa(*dL_dinput, input_width(), input.n(), "FullyFusedMLP::backward dL_dinput");
		check(n2_mlp_backward(m_mlp, stream, input.data(), input.n(), dL_doutput.data(), out_layout(dL_doutput, input.n()),
		                      dL_dinput ? dL_dinput->data() : nullptr, (n2_grad_mode)mode), "FullyFusedMLP::backward");
	}
	// Network::input_gradient(stream, dim, input, d_dinput), nerf_network.h:229
	void input_gradient(stream_t stream, uint32_t dim, const GPUMatrixDynamic<half_t>& input, GPUMatrixDynamic<half_t>& d_dinput) {
		detail::require_soa(input, input_width(), input.n(), "FullyFusedMLP input");
		detail::require_soa(d_dinput, input_width(), input.n(), "FullyFusedMLP::input_gradient d_dinput");
		check(n2_mlp_input_gradient(m_mlp, stream, dim, input.data(), input.n(), d_dinput.data()), "FullyFusedMLP::input_gradient");
	}
	// Network::backward_backward_input, nerf_network.h:560-571.  dL_doutput == nullptr: the first backward ran with e_0.
	void backward_backward_input(stream_t stream, const Context& /*ctx*/, const GPUMatrixDynamic<half_t>& input,
	                             const GPUMatrixDynamic<half_t>& dL_ddLdinput, const GPUMatrixDynamic<half_t>* dL_doutput,
	                             GPUMatrixDynamic<half_t>* dL_ddLdoutput = nullptr, GPUMatrixDynamic<half_t>* /*dL_dinput*/ = nullptr,
	                             bool /*use_inference_params*/ = false, GradientMode mode = GradientMode::Overwrite) {
		detail::require_soa(input, input_width(), input.n(), "FullyFusedMLP input");
		detail::require_soa(dL_ddLdinput, input_width(), input.n(), "FullyFusedMLP::backward_backward_input dL_ddLdinput");
		if (dL_doutput) detail::require_soa(*dL_doutput, output_width(), input.n(), "FullyFusedMLP::backward_backward_input dL_doutput");
		if (dL_ddLdoutput) detail::require_soa(*dL_ddLdoutput, output_width(), input.n(), "FullyFusedMLP::backward_backward_input dL_ddLdoutput");
		check(n2_mlp_backward_backward_input(m_mlp, stream, input.data(), input.n(), dL_ddLdinput.data(), dL_doutput ? dL_doutput->data() : nullptr,
		                                     dL_ddLdoutput ? dL_ddLdoutput->data() : nullptr, (n2_grad_mode)mode),
		      "FullyFusedMLP::backward_backward_input");
	}
	// backward(mode) and backward_backward_input(nullptr, nullptr, Accumulate) of the same input in one pass
	// (nerf_network.h:402 and :560-571 on the SDF net).  second_dL_doutput == nullptr: e_0.
	void backward_and_second_order(stream_t stream, const GPUMatrixDynamic<half_t>& input, const GPUMatrixDynamic<half_t>& dL_doutput,
	                               GPUMatrixDynamic<half_t>& dL_dinput, const GPUMatrixDynamic<half_t>& dL_ddLdinput,
	                               const GPUMatrixDynamic<half_t>* second_dL_doutput = nullptr, GradientMode mode = GradientMode::Overwrite) {
		detail::require_soa(input, input_width(), input.n(), "FullyFusedMLP input");
		detail::require_soa(dL_dinput, input_width(), input.n(), "FullyFusedMLP::backward_and_second_order dL_dinput");
		detail::require_soa(dL_ddLdinput, input_width(), input.n(), "FullyFusedMLP::backward_and_second_order dL_ddLdinput");
		if (second_dL_doutput) detail::require_soa(*second_dL_doutput, output_width(), input.n(), "FullyFusedMLP::backward_and_second_order second dL_doutput");
		check(n2_mlp_backward_and_second_order(m_mlp, stream, input.data(), input.n(), dL_doutput.data(), out_layout(dL_doutput, input.n()),
		                                       dL_dinput.data(), dL_ddLdinput.data(), second_dL_doutput ? second_dL_doutput->data() : nullptr,
		                                       (n2_grad_mode)mode), "FullyFusedMLP::backward_and_second_order");
	}

private:
	n2_layout out_layout(const GPUMatrixDynamic<half_t>& mat, uint32_t n) const {
		if (mat.m() != output_width() || mat.n() != n) throw std::runtime_error("FullyFusedMLP: output-side matrix must be 16 x N");
		if (mat.layout() == SoA && mat.stride() == n) return N2_LAYOUT_SOA;
		if (mat.layout() == AoS && mat.stride() == output_width()) return N2_LAYOUT_AOS;
		throw std::runtime_error("FullyFusedMLP: output-side matrix must be dense");
	}
	n2_mlp_t* m_mlp = nullptr;
};

// ---------------------------------------------------------------------------------------------
// NerfNetwork<__half> of the reference (static scene): input 7 x N column-major NerfCoordinate batch,
// output 16 x N column-major (src/testbed_nerf.cu:3771-3777)
// ---------------------------------------------------------------------------------------------
class NerfNetwork {
public:
	explicit NerfNetwork(const n2_field_config& config) { check(n2_field_create(&config, &m_field), "NerfNetwork"); }
	~NerfNetwork() { n2_field_destroy(m_field); }
	NerfNetwork(const NerfNetwork&) = delete;
	NerfNetwork& operator=(const NerfNetwork&) = delete;

	uint32_t input_width() const { return 7; }
	uint32_t padded_output_width() const { return 16; }
	size_t n_params() const { return n2_field_n_params(m_field); }
	n2_field_t* handle() const { return m_field; }
	void set_params(half_t* params, half_t* /*inference_params*/, half_t* /*backward_params*/, half_t* gradients) {
		check(n2_field_set_params(m_field, params, gradients), "NerfNetwork::set_params");
	}
	size_t workspace_bytes(uint32_t max_batch, uint32_t max_batch_backward) const { return n2_field_workspace_bytes(m_field, max_batch, max_batch_backward); }
	void set_workspace(void* d_workspace, size_t n_bytes, uint32_t max_batch, uint32_t max_batch_backward) {
		check(n2_field_set_workspace(m_field, d_workspace, n_bytes, max_batch, max_batch_backward), "NerfNetwork::set_workspace");
	}

	// forward_impl (nerf_network.h:132-315); the context lives in the workspace until the next forward
	std::unique_ptr<Context> forward(stream_t stream, const GPUMatrixDynamic<float>& input, GPUMatrixDynamic<half_t>* output,
	                                 bool /*use_inference_params*/ = false, bool /*prepare_input_gradients*/ = false) {
		require_coords(input);
		require_out(*output, input.n());
		check(n2_field_forward(m_field, stream, input.data(), input.n(), output->data()), "NerfNetwork::forward");
		return std::make_unique<Context>();
	}
	// backward_impl (nerf_network.h:317-641) incl. the second-order eikonal passes
	void backward(stream_t stream, const Context& /*ctx*/, const GPUMatrixDynamic<float>& input, const GPUMatrixDynamic<half_t>& /*output*/,
	              const GPUMatrixDynamic<half_t>& dL_doutput, GPUMatrixDynamic<float>* /*dL_dinput*/ = nullptr,
	              bool /*use_inference_params*/ = false, GradientMode mode = GradientMode::Overwrite, uint32_t ek_batch_size = 0) {
		require_coords(input);
		require_out(dL_doutput, input.n());
		check(n2_field_backward(m_field, stream, input.data(), input.n(), dL_doutput.data(), ek_batch_size ? ek_batch_size : input.n(), (n2_grad_mode)mode),
		      "NerfNetwork::backward");
	}
	// sdf / density (nerf_network.h:643-726): positions in, 16 x N row-major out (row 0 used)
	void sdf(stream_t stream, const GPUMatrixDynamic<float>& input, GPUMatrixDynamic<half_t>& output) { field_sdf(stream, input, output, false); }
	void density(stream_t stream, const GPUMatrixDynamic<float>& input, GPUMatrixDynamic<half_t>& output) { field_sdf(stream, input, output, true); }

private:
	static void require_coords(const GPUMatrixDynamic<float>& in) {
		if (in.layout() != CM || in.m() != 7 || in.stride() != 7) throw std::runtime_error("NerfNetwork: input must be a dense 7 x N column-major coordinate batch");
	}
	static void require_out(const GPUMatrixDynamic<half_t>& mat, uint32_t n) {
		if (mat.layout() != CM || mat.m() != 16 || mat.n() != n || mat.stride() != 16) throw std::runtime_error("NerfNetwork: output-side matrix must be dense 16 x N column-major");
	}
	void field_sdf(stream_t stream, const GPUMatrixDynamic<float>& input, GPUMatrixDynamic<half_t>& output, bool density) {
		uint32_t ps, ds;
		detail::position_strides(input, ps, ds);
		detail::require_soa(output, 16, input.n(), "NerfNetwork::sdf output");
		check((density ? n2_field_density : n2_field_sdf)(m_field, stream, input.data(), ps, ds, input.n(), output.data()), "NerfNetwork::sdf");
	}
	n2_field_t* m_field = nullptr;
};

}  // namespace n2

#endif  // NEUS2_AMD_HPP
