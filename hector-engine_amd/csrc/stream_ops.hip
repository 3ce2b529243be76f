// Two small operations on whole rows of the residual stream's width:
//   he_depth_mix   the stream that goes on after a layer as a weighted sum of the embedding's output and
//                  of every layer's result so far
//   he_gated_add   out = a + sigmoid(x . g) * b, one number a row in front of b
#include "common.h"
#include "hector_kernels.h"

// kept: fp32 [n or more][count] (plane j at j * plane elements): planes 0 .. n - 2 hold the earlier results.
// resid (fp32 [count]) holds the newest result: it is stored as plane n - 1, and resid becomes
// sum_j coeffs[j] * plane_j, added in ascending j.
__global__ __launch_bounds__(256) void depth_mix_kernel(float* __restrict__ resid, float* __restrict__ kept,
                                                        int64_t plane, const void* __restrict__ coeffs, int c_dtype,
                                                        int n, int64_t count) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= count) return;
  const float newest = resid[i];
  kept[(int64_t)(n - 1) * plane + i] = newest;
  float acc = 0.f;
  for (int j = 0; j + 1 < n; ++j) acc = fmaf(load_param(coeffs, j, c_dtype), kept[(int64_t)j * plane + i], acc);
  resid[i] = fmaf(load_param(coeffs, n - 1, c_dtype), newest, acc);
}

extern "C" int he_depth_mix(void* resid_f32, void* kept_f32, int64_t plane, const void* coeffs, int c_dtype, int n,
                            int64_t count, void* stream) {
  HE_REQUIRE(n >= 1 && count >= 0 && plane >= count, "he_depth_mix: bad sizes n=%d", n);
  HE_REQUIRE(c_dtype == HE_BF16 || c_dtype == HE_F32, "he_depth_mix: unknown dtype %d", c_dtype);
  if (count == 0) return 0;
  const int64_t blocks = (count + 255) / 256;
  depth_mix_kernel<<<(unsigned)blocks, 256, 0, (hipStream_t)stream>>>((float*)resid_f32, (float*)kept_f32, plane, coeffs,
                                                                      c_dtype, n, count);
  return he_check_launch("he_depth_mix");
}

// out[r, :] = a[r, :] + sigmoid(sum_i x[r, i] * g[i]) * b[r, :]; x [rows, Dx], a, b, out [rows, D]; the sum in fp32.
template <typename T>
__global__ __launch_bounds__(256) void gated_add_kernel(T* __restrict__ out, const T* __restrict__ a,
                                                        const T* __restrict__ b, const T* __restrict__ x,
                                                        const void* __restrict__ g, int g_dtype, int D, int Dx) {
  __shared__ float scratch[16];
  const int64_t row = blockIdx.x;
  float dot = 0.f;
  for (int i = threadIdx.x; i < Dx; i += blockDim.x) dot = fmaf(to_float(x[row * Dx + i]), load_param(g, i, g_dtype), dot);
  dot = block_sum(dot, scratch);
  const float w = 1.f / (1.f + expf(-dot));
  for (int i = threadIdx.x; i < D; i += blockDim.x)
    out[row * D + i] = from_float<T>(fmaf(w, to_float(b[row * D + i]), to_float(a[row * D + i])));
}

extern "C" int he_gated_add(void* out, const void* a, const void* b, const void* x, const void* g, int g_dtype,
                            int rows, int D, int Dx, int dtype, void* stream) {
  HE_REQUIRE(rows >= 0 && D > 0 && Dx > 0, "he_gated_add: bad sizes");
  HE_REQUIRE((dtype == HE_BF16 || dtype == HE_F32) && (g_dtype == HE_BF16 || g_dtype == HE_F32), "he_gated_add: unknown dtype");
  if (rows == 0) return 0;
  const int threads = D >= 1024 ? 256 : (D >= 256 ? 128 : 64);
  hipStream_t s = (hipStream_t)stream;
  if (dtype == HE_BF16)
    gated_add_kernel<bf16_t><<<rows, threads, 0, s>>>((bf16_t*)out, (const bf16_t*)a, (const bf16_t*)b, (const bf16_t*)x, g, g_dtype, D, Dx);
  else
    gated_add_kernel<float><<<rows, threads, 0, s>>>((float*)out, (const float*)a, (const float*)b, (const float*)x, g, g_dtype, D, Dx);
  return he_check_launch("he_gated_add");
}
