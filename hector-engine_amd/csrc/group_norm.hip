// Norms over parts of a row, all in fp32:
//   he_add_group_normed  a branch output that is normed in equal consecutive groups before it joins the
//                        residual stream, and what the next reader wants of the new stream
//   he_polynorm          a N(z) + b N(z^2) + c N(z^3) + e over a row, N the division by the root mean square
//   he_qk_head_norm      q and k heads normed by one gain vector a kind, the un-normed k copied as value
#include "common.h"
#include "hector_kernels.h"

// resid[r, :] += delta_scale * gn(delta[r, :]) (delta given), where gn(x) cuts x into `groups` equal
// consecutive parts, divides each by sqrt(mean(part^2) + eps) and multiplies the whole by weight; then, with
// out given, out[r, :] = next_weight ? gn'(resid[r, :]) with (next_weight, next_groups, next_eps) : resid[r, :].
// One workgroup of four wavefronts a row; a wavefront takes whole groups, so a group's sum is a chain in
// each lane and one butterfly, and no group waits for another.
template <typename TD, typename TO>
__global__ __launch_bounds__(256) void add_group_normed_kernel(
    float* __restrict__ resid, const TD* __restrict__ delta, const void* __restrict__ weight, int w_dtype, int groups,
    float eps, float delta_scale, TO* __restrict__ out, const void* __restrict__ next_weight, int next_groups,
    float next_eps, int D) {
  const int64_t row = blockIdx.x;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, waves = blockDim.x >> 6;
  float* r = resid + row * D;
  if (delta != nullptr) {
    const TD* d = delta + row * D;
    const int width = D / groups;
    for (int g = wave; g < groups; g += waves) {
      const int c0 = g * width;
      float ss = 0.f;
      for (int i = lane; i < width; i += 64) {
        const float x = to_float(d[c0 + i]);
        ss = fmaf(x, x, ss);
      }
      const float inv = delta_scale / sqrtf(wave_sum(ss) / (float)width + eps);
      for (int i = lane; i < width; i += 64) {
        const float x = to_float(d[c0 + i]);
        const float v = fmaf(x * inv, load_param(weight, c0 + i, w_dtype), r[c0 + i]);
        r[c0 + i] = v;
        if (out != nullptr && next_weight == nullptr) out[row * D + c0 + i] = from_float<TO>(v);
      }
    }
    if (out == nullptr || next_weight == nullptr) return;
    __syncthreads();      // the next norm's groups may be other lanes' elements
  }
  if (out == nullptr) return;
  if (next_weight == nullptr) {
    for (int i = threadIdx.x; i < D; i += blockDim.x) out[row * D + i] = from_float<TO>(r[i]);
    return;
  }
  const int width = D / next_groups;
  for (int g = wave; g < next_groups; g += waves) {
    const int c0 = g * width;
    float ss = 0.f;
    for (int i = lane; i < width; i += 64) ss = fmaf(r[c0 + i], r[c0 + i], ss);
    const float inv = 1.f / sqrtf(wave_sum(ss) / (float)width + next_eps);
    for (int i = lane; i < width; i += 64)
      out[row * D + c0 + i] = from_float<TO>(r[c0 + i] * inv * load_param(next_weight, c0 + i, w_dtype));
  }
}

extern "C" int he_add_group_normed(void* resid_f32, const void* delta, int delta_dtype, const void* weight,
                                   int w_dtype, int groups, float eps, float delta_scale, void* out, int out_dtype,
                                   const void* next_weight, int next_groups, float next_eps, int rows, int D,
                                   void* stream) {
  HE_REQUIRE(rows >= 0 && D > 0, "he_add_group_normed: bad sizes rows=%d D=%d", rows, D);
  HE_REQUIRE(delta == nullptr || (weight != nullptr && groups > 0 && D % groups == 0),
             "he_add_group_normed: %d groups do not divide the width %d", groups, D);
  HE_REQUIRE(next_weight == nullptr || (next_groups > 0 && D % next_groups == 0),
             "he_add_group_normed: %d groups do not divide the width %d", next_groups, D);
  HE_REQUIRE(w_dtype == HE_F32 || w_dtype == HE_BF16, "he_add_group_normed: bad weight dtype");
  HE_REQUIRE((delta == nullptr || delta_dtype == HE_F32 || delta_dtype == HE_BF16) &&
                 (out == nullptr || out_dtype == HE_F32 || out_dtype == HE_BF16),
             "he_add_group_normed: unknown dtype");
  if (rows == 0 || (delta == nullptr && out == nullptr)) return 0;
  hipStream_t s = (hipStream_t)stream;
  const int threads = D / (groups > 0 ? groups : 1) >= 256 || groups >= 4 ? 256 : (groups >= 2 ? 128 : 64);
#define GN_LAUNCH(TD, TO)                                                                                          \
  add_group_normed_kernel<TD, TO><<<rows, threads, 0, s>>>((float*)resid_f32, (const TD*)delta, weight, w_dtype,  \
                                                           groups, eps, delta_scale, (TO*)out, next_weight,        \
                                                           next_groups, next_eps, D)
  const bool db = delta != nullptr && delta_dtype == HE_BF16, ob = out != nullptr && out_dtype == HE_BF16;
  if (db && ob) GN_LAUNCH(bf16_t, bf16_t);
  else if (db) GN_LAUNCH(bf16_t, float);
  else if (ob) GN_LAUNCH(float, bf16_t);
  else GN_LAUNCH(float, float);
#undef GN_LAUNCH
  return he_check_launch("he_add_group_normed");
}

// out[r, i] = a z / rms(z) + b z^2 / rms(z^2) + c z^3 / rms(z^3) + e over the W values z of row r, with
// rms(x) = sqrt(mean(x^2) + eps) and the four numbers (a, b, c, e) in `numbers`. out may be x itself.
template <typename T>
__global__ __launch_bounds__(1024) void polynorm_kernel(T* out, const T* x,
                                                        const void* __restrict__ numbers, int n_dtype, int W, float eps) {
  __shared__ float scratch[16];
  const int64_t row = blockIdx.x;
  const T* z = x + row * W;
  float s2 = 0.f, s4 = 0.f, s6 = 0.f;
  for (int i = threadIdx.x; i < W; i += blockDim.x) {
    const float v = to_float(z[i]);
    const float v2 = v * v;
    s2 += v2;
    s4 = fmaf(v2, v2, s4);
    s6 = fmaf(v2 * v, v2 * v, s6);
  }
  s2 = block_sum(s2, scratch);
  __syncthreads();
  s4 = block_sum(s4, scratch);
  __syncthreads();
  s6 = block_sum(s6, scratch);
  const float a = load_param(numbers, 0, n_dtype) / sqrtf(s2 / (float)W + eps);
  const float b = load_param(numbers, 1, n_dtype) / sqrtf(s4 / (float)W + eps);
  const float c = load_param(numbers, 2, n_dtype) / sqrtf(s6 / (float)W + eps);
  const float e = load_param(numbers, 3, n_dtype);
  for (int i = threadIdx.x; i < W; i += blockDim.x) {
    const float v = to_float(z[i]);
    out[row * W + i] = from_float<T>(fmaf(a, v, fmaf(b, v * v, fmaf(c, v * v * v, e))));
  }
}

extern "C" int he_polynorm(void* out, const void* x, const void* numbers, int n_dtype, int rows, int W, float eps,
                           int dtype, void* stream) {
  HE_REQUIRE(rows >= 0 && W > 0, "he_polynorm: bad sizes rows=%d W=%d", rows, W);
  HE_REQUIRE((dtype == HE_BF16 || dtype == HE_F32) && (n_dtype == HE_BF16 || n_dtype == HE_F32), "he_polynorm: unknown dtype");
  if (rows == 0) return 0;
  // few rows: a row's elements over as many threads as a workgroup has; many rows fill the chip anyway
  const int threads = rows <= 64 && W >= 8192 ? 1024 : rows <= 64 && W >= 4096 ? 512 : W >= 1024 ? 256 : (W >= 256 ? 128 : 64);
  hipStream_t s = (hipStream_t)stream;
  if (dtype == HE_BF16)
    polynorm_kernel<bf16_t><<<rows, threads, 0, s>>>((bf16_t*)out, (const bf16_t*)x, numbers, n_dtype, W, eps);
  else
    polynorm_kernel<float><<<rows, threads, 0, s>>>((float*)out, (const float*)x, numbers, n_dtype, W, eps);
  return he_check_launch("he_polynorm");
}

// Rows [q heads | k heads] of `in`, in_stride elements apart, to rows [q heads | k heads | v heads] of out: every
// q head (H of them, d wide) is divided by its root mean square and multiplied by q_w [d], every k head (G of
// them) likewise with k_w; with copy_v the k head as it was before the norm becomes the v head. out may be in.
// One wavefront a (row, head).
template <typename T>
__global__ __launch_bounds__(256) void qk_head_norm_kernel(T* __restrict__ out, int64_t out_stride, const T* in, int64_t in_stride,
                                                            const void* __restrict__ q_w, const void* __restrict__ k_w,
                                                            int w_dtype, int H, int G, int d, float eps, int copy_v,
                                                            int rows) {
  const int lane = threadIdx.x & 63;
  const int64_t unit = (int64_t)blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
  if (unit >= (int64_t)rows * (H + G)) return;
  const int64_t row = unit / (H + G);
  const int head = (int)(unit % (H + G));
  const T* x = in + row * in_stride + (int64_t)head * d;
  T* o = out + row * out_stride + (int64_t)head * d;
  const void* w = head < H ? q_w : k_w;
  float ss = 0.f;
  for (int i = lane; i < d; i += 64) {
    const float v = to_float(x[i]);
    ss = fmaf(v, v, ss);
  }
  const float inv = 1.f / sqrtf(wave_sum(ss) / (float)d + eps);
  T* vcol = o + (int64_t)G * d;     // the v head behind the k heads
  for (int i = lane; i < d; i += 64) {
    const T raw = x[i];
    if (copy_v && head >= H) vcol[i] = raw;
    o[i] = from_float<T>(to_float(raw) * inv * load_param(w, i, w_dtype));
  }
}

extern "C" int he_qk_head_norm(void* out, int64_t out_stride, const void* in, int64_t in_stride, const void* q_w, const void* k_w, int w_dtype, int H, int G,
                               int d, float eps, int copy_v, int rows, int dtype, void* stream) {
  HE_REQUIRE(rows >= 0 && H > 0 && G >= 0 && d > 0 && out_stride >= (int64_t)(H + G + (copy_v ? G : 0)) * d &&
                 in_stride >= (int64_t)(H + G) * d,
             "he_qk_head_norm: bad sizes H=%d G=%d d=%d", H, G, d);
  HE_REQUIRE((dtype == HE_BF16 || dtype == HE_F32) && (w_dtype == HE_BF16 || w_dtype == HE_F32), "he_qk_head_norm: unknown dtype");
  if (rows == 0) return 0;
  const int64_t units = (int64_t)rows * (H + G);
  const int blocks = (int)((units + 3) / 4);
  hipStream_t s = (hipStream_t)stream;
  if (dtype == HE_BF16)
    qk_head_norm_kernel<bf16_t><<<blocks, 256, 0, s>>>((bf16_t*)out, out_stride, (const bf16_t*)in, in_stride, q_w, k_w, w_dtype, H, G, d, eps, copy_v, rows);
  else
    qk_head_norm_kernel<float><<<blocks, 256, 0, s>>>((float*)out, out_stride, (const float*)in, in_stride, q_w, k_w, w_dtype, H, G, d, eps, copy_v, rows);
  return he_check_launch("he_qk_head_norm");
}
