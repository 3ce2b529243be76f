// What a latent attention needs around the shared attention kernels. Its keys and values are one latent
// vector c a token (plus one rotated key part shared by all heads); a head's own key part is W_uk,h c and
// its value W_uv,h c. Because q . (W_uk,h c) = (W_uk,h^T q) . c, the cache keeps [rotated part | c] as the
// one key of a token and c as its value, the queries are taken through W_uk,h^T, and a head's attention
// result over the latents goes through W_uv,h afterwards: two products per head.
//   he_head_product   out[r, h, :] = x[r, h, :] W_h for a matrix a head
//   he_latent_pack    the rows [q heads | key | value] as the rotation and cache-write kernel reads them
#include "common.h"
#include "hector_kernels.h"

#define HP_ROWS 8
#define HP_KCHUNK 256
// out[r, h, n] = sum_k x[r, h, k] * w[h, k, n] in fp32: k in chunks of HP_KCHUNK; inside a chunk each of the
// workgroup's four wavefronts takes a quarter of the k (a chain of multiply-adds in ascending k, eight weight loads
// in flight), the four sums meet in wavefront order, and the chunks' sums are added in chunk order: one order a
// row whatever else the step holds. x at x_row / x_head element strides, out likewise; w [H][K][N]. A workgroup
// takes HP_ROWS rows of one head and 64 neighbouring n; the rows' x values are staged in LDS a chunk at a time.
template <typename T, typename TW>
__global__ __launch_bounds__(256) void head_product_kernel(T* __restrict__ out, int64_t o_row, int64_t o_head,
                                                           const T* __restrict__ x, int64_t x_row, int64_t x_head,
                                                           const TW* __restrict__ w, int rows, int K, int N) {
  __shared__ float xs[HP_ROWS][HP_KCHUNK];
  __shared__ float part[4][HP_ROWS][64];
  const int h = blockIdx.y;
  const int64_t r0 = (int64_t)blockIdx.z * HP_ROWS;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int n = blockIdx.x * 64 + lane;
  const int nc = min(n, N - 1);            // a lane beyond N reads the last column and stores nothing
  const TW* wh = w + (int64_t)h * K * N;
  float total[HP_ROWS];
#pragma unroll
  for (int r = 0; r < HP_ROWS; ++r) total[r] = 0.f;
  for (int k0 = 0; k0 < K; k0 += HP_KCHUNK) {
    const int kc = min(HP_KCHUNK, K - k0);
    __syncthreads();
    for (int i = threadIdx.x; i < HP_ROWS * kc; i += blockDim.x) {
      const int r = i / kc, k = i % kc;
      xs[r][k] = r0 + r < rows ? to_float(x[(r0 + r) * x_row + h * x_head + k0 + k]) : 0.f;
    }
    __syncthreads();
    const int per = (kc + 3) / 4;
    const int ka = wave * per, kb = min(kc, ka + per);
    float acc[HP_ROWS];
#pragma unroll
    for (int r = 0; r < HP_ROWS; ++r) acc[r] = 0.f;
    for (int k = ka; k < kb; k += 8) {
      float wv[8];
#pragma unroll
      for (int u = 0; u < 8; ++u) wv[u] = to_float(wh[(int64_t)(k0 + min(k + u, kb - 1)) * N + nc]);
#pragma unroll
      for (int u = 0; u < 8; ++u)
        if (k + u < kb) {
#pragma unroll
          for (int r = 0; r < HP_ROWS; ++r) acc[r] = fmaf(xs[r][k + u], wv[u], acc[r]);
        }
    }
#pragma unroll
    for (int r = 0; r < HP_ROWS; ++r) part[wave][r][lane] = acc[r];
    __syncthreads();
    if (wave == 0) {
#pragma unroll
      for (int r = 0; r < HP_ROWS; ++r)
        total[r] += ((part[0][r][lane] + part[1][r][lane]) + part[2][r][lane]) + part[3][r][lane];
    }
  }
  if (wave != 0 || n >= N) return;
#pragma unroll
  for (int r = 0; r < HP_ROWS; ++r)
    if (r0 + r < rows) out[(r0 + r) * o_row + h * o_head + n] = from_float<T>(total[r]);
}

extern "C" int he_head_product(void* out, int64_t o_row, int64_t o_head, const void* x, int64_t x_row, int64_t x_head,
                               const void* w, int w_dtype, int rows, int H, int K, int N, int dtype, void* stream) {
  HE_REQUIRE(rows >= 0 && H > 0 && K > 0 && N > 0 && H <= 65535, "he_head_product: bad sizes H=%d K=%d N=%d", H, K, N);
  HE_REQUIRE((dtype == HE_BF16 || dtype == HE_F32) && (w_dtype == HE_BF16 || w_dtype == HE_F32), "he_head_product: unknown dtype");
  if (rows == 0) return 0;
  const int threads = 256;
  const dim3 grid((N + 63) / 64, H, (rows + HP_ROWS - 1) / HP_ROWS);
  HE_REQUIRE(grid.z <= 65535, "he_head_product: %d rows are too many for one launch", rows);
  hipStream_t s = (hipStream_t)stream;
#define HP_LAUNCH(T, TW)                                                                                    \
  head_product_kernel<T, TW><<<grid, threads, 0, s>>>((T*)out, o_row, o_head, (const T*)x, x_row, x_head, \
                                                      (const TW*)w, rows, K, N)
  if (dtype == HE_BF16 && w_dtype == HE_BF16) {
    HP_LAUNCH(bf16_t, bf16_t);
  } else if (dtype == HE_BF16) {
    HP_LAUNCH(bf16_t, float);
  } else if (w_dtype == HE_BF16) {
    HP_LAUNCH(float, bf16_t);
  } else {
    HP_LAUNCH(float, float);
  }
#undef HP_LAUNCH
  return he_check_launch("he_head_product");
}

// qkv [rows][H * (r + rank) + (r + rank) + rank]: head h's columns are [r rotated dims | rank]; the rank part is
// written by he_head_product. This kernel fills the rest: a head's rotated dims from q [rows][H][d + r] (its last r
// columns), the key [rotated part | c] and the value c from `down` [rows][rank + r] (c first) at down_stride.
template <typename T>
__global__ __launch_bounds__(256) void latent_pack_kernel(T* __restrict__ qkv, const T* __restrict__ q,
                                                          const T* __restrict__ down, int64_t down_stride, int rows, int H,
                                                          int d, int r, int rank) {
  const int per_row = H * r + r + 2 * rank;
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= (int64_t)rows * per_row) return;
  const int64_t row = i / per_row;
  int c = (int)(i % per_row);
  const int hd = r + rank;
  T* o = qkv + row * ((int64_t)(H + 1) * hd + rank);
  if (c < H * r) {
    const int h = c / r, u = c % r;
    o[h * hd + u] = q[(row * H + h) * (int64_t)(d + r) + d + u];
    return;
  }
  c -= H * r;
  const T* dn = down + row * down_stride;
  if (c < r) o[H * hd + c] = dn[rank + c];
  else if (c < r + rank) o[H * hd + c] = dn[c - r];
  else o[(H + 1) * hd + (c - r - rank)] = dn[c - r - rank];
}

extern "C" int he_latent_pack(void* qkv, const void* q, const void* down, int64_t down_stride, int rows, int H, int d,
                              int r, int rank, int dtype, void* stream) {
  HE_REQUIRE(rows >= 0 && H > 0 && d >= 0 && r >= 0 && rank > 0 && down_stride >= rank + r, "he_latent_pack: bad sizes");
  HE_REQUIRE(dtype == HE_BF16 || dtype == HE_F32, "he_latent_pack: unknown dtype %d", dtype);
  if (rows == 0) return 0;
  const int64_t total = (int64_t)rows * (H * r + r + 2 * rank);
  const unsigned blocks = (unsigned)((total + 255) / 256);
  hipStream_t s = (hipStream_t)stream;
  if (dtype == HE_BF16)
    latent_pack_kernel<bf16_t><<<blocks, 256, 0, s>>>((bf16_t*)qkv, (const bf16_t*)q, (const bf16_t*)down, down_stride, rows, H, d, r, rank);
  else
    latent_pack_kernel<float><<<blocks, 256, 0, s>>>((float*)qkv, (const float*)q, (const float*)down, down_stride, rows, H, d, r, rank);
  return he_check_launch("he_latent_pack");
}
