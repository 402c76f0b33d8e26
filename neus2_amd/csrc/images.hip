// Training images: 8-bit sRGB RGBA as the loader decodes it -> linear, alpha-premultiplied fp32 RGBA as the ray
// generator reads it.  NerfDataset::set_training_image with convert_rgba32 (src/nerf_loader.cu:59-81, 758-792) followed
// by the Byte branch of read_rgba (common_device.cuh:635-655) and srgb_to_linear (:31-37), done once per image
// instead of once per pixel access.
#include "n2_common.h"

__device__ __forceinline__ float n2_srgb_to_linear(float srgb) {
	return srgb <= 0.04045f ? srgb / 12.92f : powf((srgb + 0.055f) / 1.055f, 2.4f);
}

__global__ void __launch_bounds__(256) convert_rgba8_kernel(uint64_t n_pixels, const uint32_t* __restrict__ in, float4* __restrict__ out,
                                                            int white_transparent, int black_transparent, uint32_t mask_color) {
	const uint64_t i = (uint64_t)blockIdx.x * 256 + threadIdx.x;
	if (i >= n_pixels) return;
	uint32_t px = in[i];
	uint32_t r = px & 0xFFu, g = (px >> 8) & 0xFFu, b = (px >> 16) & 0xFFu, a = px >> 24;
	if (white_transparent && r == 255 && g == 255 && b == 255) a = 0;
	if (black_transparent && r == 0 && g == 0 && b == 0) a = 0;
	px = r | (g << 8) | (b << 16) | (a << 24);
	if (mask_color != 0 && mask_color == px) px = 0x00FF00FFu;  // masked pixels become "hot pink", alpha 0 ...
	if (px == 0x00FF00FFu) {                                     // ... which reads back as -1: the pixel is skipped
		out[i] = make_float4(-1.f, -1.f, -1.f, -1.f);
		return;
	}
	const float alpha = (float)a * (1.0f / 255.0f);
	out[i] = make_float4(n2_srgb_to_linear((float)r * (1.0f / 255.0f)) * alpha, n2_srgb_to_linear((float)g * (1.0f / 255.0f)) * alpha,
	                     n2_srgb_to_linear((float)b * (1.0f / 255.0f)) * alpha, alpha);
}

N2_API int n2_convert_rgba8(n2_stream_t stream, uint64_t n_pixels, const uint8_t* d_rgba8, float* d_rgba, int white_transparent,
                            int black_transparent, uint32_t mask_color) {
	if (n_pixels == 0) return N2_OK;
	N2_REQUIRE(d_rgba8 != nullptr && d_rgba != nullptr, "n2_convert_rgba8: null buffer");
	N2_REQUIRE(reinterpret_cast<uintptr_t>(d_rgba8) % 4 == 0 && reinterpret_cast<uintptr_t>(d_rgba) % 16 == 0,
	           "n2_convert_rgba8: input must be 4-byte and output 16-byte aligned");
	N2_REQUIRE(n_pixels < (1ull << 40), "n2_convert_rgba8: too many pixels");
	convert_rgba8_kernel<<<dim3((uint32_t)((n_pixels + 255) / 256)), dim3(256), 0, n2_stream(stream)>>>(
		n_pixels, reinterpret_cast<const uint32_t*>(d_rgba8), reinterpret_cast<float4*>(d_rgba), white_transparent, black_transparent, mask_color);
	N2_LAUNCH_CHECK();
	return N2_OK;
}
