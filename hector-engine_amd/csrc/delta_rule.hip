// The gated delta rule: a matrix S [d, e] per head that is carried from token to token. Per token, with
// q and k of d dims (shared by the heads of a group), v of e dims, a write strength beta and a decay g:
//     q <- q / sqrt(sum(q^2) + unit_eps) * q_scale,   k <- k / sqrt(sum(k^2) + unit_eps)
//     beta = sigmoid(b),   g = exp(-exp(A_log_h) * softplus(a + dt_bias_h))
//     S <- g S;   u = beta (v - S^T k);   S <- S + k u^T;   o = S^T q
// so the read-out sees the token's own write. Everything here is fp32 but the loads of q, k and v.
//
// One wavefront a (sequence, head, tile of value dims). A value dim's column of S is held by NG
// neighbouring lanes, KPT key dims each (NG a power of two, KPT 8 to 32 in steps of 8, NG * KPT >= d):
// the two sums over the key dims (S^T k and S^T q) are a chain of multiply-adds in a lane and a butterfly
// over the NG lanes, the same order for every token however the rows were cut into steps, so that a
// sequence's results do not depend on the cut. A sequence's S lies in its row of the state area as
// [head][value dim][NG * KPT]: each lane's share is contiguous.
#include "common.h"
#include "hector_kernels.h"

__device__ __forceinline__ float dr_softplus(float z) { return z > 20.f ? z : log1pf(expf(z)); }

static void dr_plan(int d, int* ng, int* kpt) {
  for (int g = 1; g <= 64; g <<= 1) {
    const int per = ((d + g - 1) / g + 7) / 8 * 8;
    if (per <= 32) {
      *ng = g;
      *kpt = per;
      return;
    }
  }
  *ng = 0;
  *kpt = 0;
}

extern "C" int64_t he_delta_state_floats(int H, int d, int e) {
  int ng, kpt;
  dr_plan(d, &ng, &kpt);
  return (int64_t)H * e * ng * kpt;
}

template <typename T, int KPT>
__global__ __launch_bounds__(64) void delta_scan_kernel(
    float* __restrict__ y, const T* __restrict__ q_in, const T* __restrict__ k_in, const T* __restrict__ v_in,
    int64_t in_stride, const float* __restrict__ ba, const void* __restrict__ a_log, const void* __restrict__ dt_bias,
    int w_dtype, uint8_t* __restrict__ state, int64_t state_stride, int64_t state_offset,
    const int32_t* __restrict__ cu_seqlens, const int32_t* __restrict__ seq_slot, int H, int G, int d, int e, int NG,
    float q_scale, float unit_eps) {
  const int seq = blockIdx.x, h = blockIdx.y;
  const int slot = seq_slot[seq];
  if (slot < 0) return;
  const int r0 = cu_seqlens[seq], r1 = cu_seqlens[seq + 1];
  if (r1 <= r0) return;
  const int lane = threadIdx.x;
  const int g_lane = lane & (NG - 1);
  const int per_block = 64 / NG;                       // value dims of this wavefront
  const int j = blockIdx.z * per_block + lane / NG;    // this lane's value dim
  const bool has = j < e;
  const int kv = h / (H / G);                          // the head's q/k group
  const int i0 = g_lane * KPT;                         // first key dim of this lane
  float* S_row = reinterpret_cast<float*>(state + (int64_t)slot * state_stride + state_offset) +
                 (((int64_t)h * e + (has ? j : 0)) * NG + g_lane) * KPT;
  float S[KPT];
#pragma unroll
  for (int i = 0; i < KPT; ++i) S[i] = has ? S_row[i] : 0.f;
  const float rate = expf(load_param(a_log, h, w_dtype));
  const float bias = load_param(dt_bias, h, w_dtype);
  const T* qp = q_in + (int64_t)kv * d + i0;
  const T* kp = k_in + (int64_t)kv * d + i0;
  const T* vp = v_in + (int64_t)h * e + (has ? j : 0);

  // the loads of the next token are issued before this token's chain of sums
  float kq[KPT], qq[KPT], vv, bb, aa;
  auto fetch = [&](int64_t r) {
#pragma unroll
    for (int i = 0; i < KPT; ++i) {
      const bool in = i0 + i < d;
      kq[i] = in ? to_float(kp[r * in_stride + i]) : 0.f;
      qq[i] = in ? to_float(qp[r * in_stride + i]) : 0.f;
    }
    vv = to_float(vp[r * in_stride]);
    bb = ba[r * 2 * H + h];
    aa = ba[r * 2 * H + H + h];
  };
  fetch(r0);
  for (int64_t r = r0; r < r1; ++r) {
    float k[KPT], q[KPT];
    float ssk = 0.f, ssq = 0.f;
#pragma unroll
    for (int i = 0; i < KPT; ++i) {
      k[i] = kq[i];
      q[i] = qq[i];
      ssk = fmaf(k[i], k[i], ssk);
      ssq = fmaf(q[i], q[i], ssq);
    }
    const float v = vv;
    const float beta = 1.f / (1.f + expf(-bb));
    const float decay = expf(-rate * dr_softplus(aa + bias));
    if (r + 1 < r1) fetch(r + 1);
    for (int m = NG >> 1; m >= 1; m >>= 1) {
      ssk += __shfl_xor(ssk, m);
      ssq += __shfl_xor(ssq, m);
    }
    const float kn = 1.f / sqrtf(ssk + unit_eps);
    const float qn = q_scale / sqrtf(ssq + unit_eps);
    float dot = 0.f;
#pragma unroll
    for (int i = 0; i < KPT; ++i) {
      k[i] *= kn;
      q[i] *= qn;
      S[i] *= decay;
      dot = fmaf(S[i], k[i], dot);
    }
    for (int m = NG >> 1; m >= 1; m >>= 1) dot += __shfl_xor(dot, m);
    const float u = beta * (v - dot);
    float o = 0.f;
#pragma unroll
    for (int i = 0; i < KPT; ++i) {
      S[i] = fmaf(k[i], u, S[i]);
      o = fmaf(S[i], q[i], o);
    }
    for (int m = NG >> 1; m >= 1; m >>= 1) o += __shfl_xor(o, m);
    if (has && g_lane == 0) y[r * ((int64_t)H * e) + (int64_t)h * e + j] = o;
  }
  if (has) {
#pragma unroll
    for (int i = 0; i < KPT; ++i) S_row[i] = S[i];
  }
}

extern "C" int he_delta_scan(void* y_f32, const void* q, const void* k, const void* v, int64_t in_stride,
                             const void* ba_f32, const void* a_log, const void* dt_bias, int w_dtype, void* state,
                             int64_t state_stride, int64_t state_offset, const void* cu_seqlens, const void* seq_slot,
                             int rows, int num_seqs, int H, int G, int d, int e, float q_scale, float unit_eps,
                             int dtype, void* stream) {
  HE_REQUIRE(rows >= 0 && num_seqs >= 0 && H > 0 && G > 0 && H % G == 0 && d > 0 && e > 0,
             "he_delta_scan: bad sizes H=%d G=%d d=%d e=%d", H, G, d, e);
  HE_REQUIRE(dtype == HE_BF16 || dtype == HE_F32, "he_delta_scan: unknown dtype %d", dtype);
  HE_REQUIRE(w_dtype == HE_BF16 || w_dtype == HE_F32, "he_delta_scan: unknown parameter dtype %d", w_dtype);
  int ng, kpt;
  dr_plan(d, &ng, &kpt);
  HE_REQUIRE(ng > 0, "he_delta_scan: key width %d above 2048", d);
  HE_REQUIRE(state != nullptr && state_offset % 16 == 0 && state_stride % 4 == 0 &&
                 state_stride >= state_offset + 4 * he_delta_state_floats(H, d, e),
             "he_delta_scan: the state row is too short");
  if (rows == 0 || num_seqs == 0) return 0;
  const int per_block = 64 / ng;
  const dim3 grid(num_seqs, H, (e + per_block - 1) / per_block);
  HE_REQUIRE(grid.y <= 65535 && grid.z <= 65535, "he_delta_scan: too many heads or value tiles for one launch");
  hipStream_t s = (hipStream_t)stream;
#define DR_LAUNCH(T, KPT)                                                                                           \
  delta_scan_kernel<T, KPT><<<grid, 64, 0, s>>>((float*)y_f32, (const T*)q, (const T*)k, (const T*)v, in_stride,      \
                                                (const float*)ba_f32, a_log, dt_bias, w_dtype, (uint8_t*)state,      \
                                                state_stride, state_offset, (const int32_t*)cu_seqlens,              \
                                                (const int32_t*)seq_slot, H, G, d, e, ng, q_scale, unit_eps)
#define DR_BY_KPT(T)                    \
  if (kpt == 8) DR_LAUNCH(T, 8);        \
  else if (kpt == 16) DR_LAUNCH(T, 16); \
  else if (kpt == 24) DR_LAUNCH(T, 24); \
  else DR_LAUNCH(T, 32)
  if (dtype == HE_BF16) {
    DR_BY_KPT(bf16_t);
  } else {
    DR_BY_KPT(float);
  }
#undef DR_BY_KPT
#undef DR_LAUNCH
  return he_check_launch("he_delta_scan");
}
