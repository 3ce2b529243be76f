// The gated delta rule: a matrix S [d, e] per head that is carried from token to token. Per token, with
// q and k of d dims (shared by the heads of a group), v of e dims, a write strength beta and a decay g:
//     q <- q / sqrt(sum(q^2) + unit_eps) * q_scale,   k <- k / sqrt(sum(k^2) + unit_eps)
//     beta = sigmoid(b),   g = exp(-exp(A_log_h) * softplus(a + dt_bias_h))
//     S <- g S;   u = beta (v - S^T k);   S <- S + k u^T;   o = S^T q
// so the read-out sees the token's own write. Everything here is fp32 but the loads of q, k and v.
//
// Two launches. he_delta_prepare (inside he_delta_scan) forms, row by row and in parallel, what does not
// depend on the state: the unit vectors k and q as fp32 (padded with zeros to the lanes' shares), and per
// head beta, g and k . q. The scan then walks a sequence's rows with one wavefront a (sequence, head, tile
// of value dims). A value dim's column of S is held by NG neighbouring lanes, KPT key dims each (NG a power
// of two, KPT 8 to 32 in steps of 8, NG * KPT >= d, the smallest such product and then the most lanes).
// With the old S, both sums over the key dims are formed side by side, a = S^T k and b = S^T q (a chain
// of multiply-adds in a lane, then a butterfly over the NG lanes, inside a row of 16 lanes by lane
// permutations), and then
//     u = beta (v - g a),   o = g b + u (k . q),   S <- g S + k u^T,
// which is the recurrence above with the read-out written in terms of the old S: the write is off the path
// from one token's sums to its output. The rows' k, q and scalars are staged in LDS a block of 8 rows at a
// time, the next block's loads in flight while this block is walked. Every token's sums are formed in one
// order however the rows were cut into steps, so a sequence's results do not depend on the cut. A
// sequence's S lies in its row of the state area as [head][value dim][NG * KPT]: each lane's share is
// contiguous.
#include "common.h"
#include "hector_kernels.h"

__device__ __forceinline__ float dr_softplus(float z) { return z > 20.f ? z : log1pf(expf(z)); }

#define DR_ROWS 8          // rows of a block staged in LDS
#define DR_MAX_DP 256      // padded key width up to which the staged kernel runs

static void dr_plan(int d, int* ng, int* kpt) {
  int best = 0, best_pad = 0;
  for (int g = 1; g <= 64; g <<= 1) {
    const int per = ((d + g - 1) / g + 7) / 8 * 8;
    if (per > 32) continue;
    if (best == 0 || g * per < best_pad || (g * per == best_pad && g <= 16)) {
      best = g;
      best_pad = g * per;
      *kpt = per;
    }
  }
  *ng = best;
  if (best == 0) *kpt = 0;
}

extern "C" int64_t he_delta_state_floats(int H, int d, int e) {
  int ng, kpt;
  dr_plan(d, &ng, &kpt);
  return (int64_t)H * e * ng * kpt;
}

// floats of the prepared rows: [rows][G][k | q] of the padded key width, then [rows][H][4]
extern "C" int64_t he_delta_workspace_floats(int rows, int H, int G, int d) {
  int ng, kpt;
  dr_plan(d, &ng, &kpt);
  return (int64_t)rows * G * 2 * ng * kpt + (int64_t)rows * H * 4;
}

// One wavefront a (row, group): the group's k and q to unit length (q times q_scale), zeros beyond d; for the
// heads of the group (lane i < H / G: head g H/G + i) beta, g and k . q.
template <typename T>
__global__ __launch_bounds__(256) void delta_prepare_kernel(
    float* __restrict__ kq_out, float* __restrict__ head_out, const T* __restrict__ q_in, const T* __restrict__ k_in,
    int64_t in_stride, const float* __restrict__ ba, const void* __restrict__ a_log, const void* __restrict__ dt_bias,
    int w_dtype, int rows, int H, int G, int d, int DP, float q_scale, float unit_eps) {
  const int lane = threadIdx.x & 63;
  const int64_t unit = (int64_t)blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
  if (unit >= (int64_t)rows * G) return;
  const int64_t row = unit / G;
  const int g = (int)(unit % G);
  const T* qp = q_in + row * in_stride + (int64_t)g * d;
  const T* kp = k_in + row * in_stride + (int64_t)g * d;
  float ssk = 0.f, ssq = 0.f;
  for (int i = lane; i < d; i += 64) {
    const float kv = to_float(kp[i]), qv = to_float(qp[i]);
    ssk = fmaf(kv, kv, ssk);
    ssq = fmaf(qv, qv, ssq);
  }
  const float kn = 1.f / sqrtf(wave_sum(ssk) + unit_eps);
  const float qn = q_scale / sqrtf(wave_sum(ssq) + unit_eps);
  float* out = kq_out + unit * 2 * DP;
  float dot = 0.f;
  for (int i = lane; i < DP; i += 64) {
    const float kv = i < d ? to_float(kp[i]) * kn : 0.f;
    const float qv = i < d ? to_float(qp[i]) * qn : 0.f;
    out[i] = kv;
    out[DP + i] = qv;
    dot = fmaf(kv, qv, dot);
  }
  dot = wave_sum(dot);
  const int per = H / G;
  for (int i = lane; i < per; i += 64) {
    const int h = g * per + i;
    const float beta = 1.f / (1.f + expf(-ba[row * 2 * H + h]));
    const float decay = expf(-expf(load_param(a_log, h, w_dtype)) *
                             dr_softplus(ba[row * 2 * H + H + h] + load_param(dt_bias, h, w_dtype)));
    reinterpret_cast<float4*>(head_out)[row * H + h] = make_float4(beta, decay, dot, 0.f);
  }
}

__device__ __forceinline__ float dr_group_sum(float v, int NG) {
  if (NG >= 2) v += lane_xor1(v);
  if (NG >= 4) v += lane_xor2(v);
  if (NG >= 8) v += lane_xor4(v);
  if (NG >= 16) v += lane_xor8(v);
  if (NG >= 32) v = xor16_sum(v);
  if (NG >= 64) v = xor32_sum(v);
  return v;
}

// What a lane moves of the block that begins at row T0: its float4 of the rows' k | q, a row's scalars (lanes below
// DR_ROWS; rows beyond the sequence get beta 0, g 1: they leave S as it is), and its own value dim of every row.
// Rows beyond the sequence read its last row.
#define DR_FETCH(T0)                                                                                     \
  {                                                                                                      \
    _Pragma("unroll") for (int i = 0; i < NLD; ++i) {                                                    \
      const int f = min(lane + 64 * i, BLOCK_F4 - 1);                                                    \
      const int t = f / ROW_F4, c = f - t * ROW_F4;                                                      \
      const float4 w = kq4[((int64_t)min((T0) + t, r1 - 1) * G + kv) * ROW_F4 + c];                      \
      ld[4 * i] = w.x, ld[4 * i + 1] = w.y, ld[4 * i + 2] = w.z, ld[4 * i + 3] = w.w;                    \
    }                                                                                                    \
    const int tr = (T0) + min(lane, DR_ROWS - 1);                                                        \
    const float4 w = head4[(int64_t)min(tr, r1 - 1) * H + h];                                            \
    sc_beta = tr >= r1 ? 0.f : w.x, sc_g = tr >= r1 ? 1.f : w.y, sc_kq = tr >= r1 ? 0.f : w.z;           \
    _Pragma("unroll") for (int t = 0; t < DR_ROWS; ++t)                                                  \
        ld_v[t] = to_float(vp[(int64_t)min((T0) + t, r1 - 1) * in_stride]);                              \
  }

template <typename T, int KPT, int NG>
__global__ __launch_bounds__(64) void delta_scan_kernel(
    float* __restrict__ y, const float* __restrict__ kq_in, const float* __restrict__ head_in,
    const T* __restrict__ v_in, int64_t in_stride, uint8_t* __restrict__ state, int64_t state_stride,
    int64_t state_offset, const int32_t* __restrict__ cu_seqlens, const int32_t* __restrict__ seq_slot, int H, int G,
    int e) {
  constexpr int DP = NG * KPT;
  constexpr int ROW_F4 = DP / 2;                       // float4 of one row's k | q
  constexpr int BLOCK_F4 = DR_ROWS * ROW_F4;
  constexpr int NLD = (BLOCK_F4 + 63) / 64;            // float4 a lane moves per block
  constexpr int PER_BLOCK = 64 / NG;                   // value dims of this wavefront
  __shared__ float4 kq_s[BLOCK_F4];
  __shared__ float4 sc_s[DR_ROWS];
  const int seq = blockIdx.x, h = blockIdx.y;
  const int slot = seq_slot[seq];
  if (slot < 0) return;
  const int r0 = cu_seqlens[seq], r1 = cu_seqlens[seq + 1];
  if (r1 <= r0) return;
  const int lane = threadIdx.x;
  const int g_lane = lane & (NG - 1);
  const int j = blockIdx.z * PER_BLOCK + lane / NG;    // this lane's value dim
  const bool has = j < e;
  const int kv = h / (H / G);                          // the head's q/k group
  float* S_row = reinterpret_cast<float*>(state + (int64_t)slot * state_stride + state_offset) +
                 (((int64_t)h * e + (has ? j : 0)) * NG + g_lane) * KPT;
  float S[KPT];
#pragma unroll
  for (int i = 0; i < KPT; ++i) S[i] = has ? S_row[i] : 0.f;
  const T* vp = v_in + (int64_t)h * e + (has ? j : 0);
  const float4* kq4 = reinterpret_cast<const float4*>(kq_in);
  const float4* head4 = reinterpret_cast<const float4*>(head_in);
  float* yp = y + (int64_t)h * e + (has ? j : 0);
  const int64_t y_stride = (int64_t)H * e;

  float ld[4 * NLD], sc_beta, sc_g, sc_kq;
  float ld_v[DR_ROWS];
  DR_FETCH(r0)
  for (int t0 = r0; t0 < r1; t0 += DR_ROWS) {
    __syncthreads();        // the block before has been walked
#pragma unroll
    for (int i = 0; i < NLD; ++i)
      if (BLOCK_F4 % 64 == 0 || lane + 64 * i < BLOCK_F4)
        kq_s[lane + 64 * i] = make_float4(ld[4 * i], ld[4 * i + 1], ld[4 * i + 2], ld[4 * i + 3]);
    if (lane < DR_ROWS) sc_s[lane] = make_float4(sc_beta, sc_g, sc_kq, 0.f);
    float vs[DR_ROWS];
#pragma unroll
    for (int t = 0; t < DR_ROWS; ++t) vs[t] = ld_v[t];
    __syncthreads();
    if (t0 + DR_ROWS < r1) DR_FETCH(t0 + DR_ROWS)
    const int n = r1 - t0;
#pragma unroll
    for (int t = 0; t < DR_ROWS; ++t) {
      const float4 sc = sc_s[t];                       // beta, g, k . q
      const float4* kr = kq_s + t * ROW_F4 + g_lane * (KPT / 4);
      const float4* qr = kr + ROW_F4 / 2;
      float k[KPT], q[KPT];
#pragma unroll
      for (int i = 0; i < KPT / 4; ++i) {
        const float4 a = kr[i], b = qr[i];
        k[4 * i] = a.x, k[4 * i + 1] = a.y, k[4 * i + 2] = a.z, k[4 * i + 3] = a.w;
        q[4 * i] = b.x, q[4 * i + 1] = b.y, q[4 * i + 2] = b.z, q[4 * i + 3] = b.w;
      }
      float sk = 0.f, sq = 0.f;
#pragma unroll
      for (int i = 0; i < KPT; ++i) {
        sk = fmaf(S[i], k[i], sk);
        sq = fmaf(S[i], q[i], sq);
      }
      sk = dr_group_sum(sk, NG);
      sq = dr_group_sum(sq, NG);
      const float u = sc.x * (vs[t] - sc.y * sk);
      const float o = fmaf(sc.y, sq, u * sc.z);
#pragma unroll
      for (int i = 0; i < KPT; ++i) S[i] = fmaf(k[i], u, sc.y * S[i]);
      if (has && g_lane == 0 && t < n) yp[(int64_t)(t0 + t) * y_stride] = o;
    }
  }
  if (has) {
#pragma unroll
    for (int i = 0; i < KPT; ++i) S_row[i] = S[i];
  }
}
#undef DR_FETCH

// The same walk without staging, for key widths beyond DR_MAX_DP: a lane reads its own share of a row's prepared
// k and q, one row ahead.
template <typename T, int KPT>
__global__ __launch_bounds__(64) void delta_scan_direct_kernel(
    float* __restrict__ y, const float* __restrict__ kq_in, const float* __restrict__ head_in,
    const T* __restrict__ v_in, int64_t in_stride, uint8_t* __restrict__ state, int64_t state_stride,
    int64_t state_offset, const int32_t* __restrict__ cu_seqlens, const int32_t* __restrict__ seq_slot, int H, int G,
    int e, int NG) {
  const int seq = blockIdx.x, h = blockIdx.y;
  const int slot = seq_slot[seq];
  if (slot < 0) return;
  const int r0 = cu_seqlens[seq], r1 = cu_seqlens[seq + 1];
  if (r1 <= r0) return;
  const int lane = threadIdx.x;
  const int g_lane = lane & (NG - 1);
  const int per_block = 64 / NG;
  const int j = blockIdx.z * per_block + lane / NG;
  const bool has = j < e;
  const int kv = h / (H / G);
  const int DP = NG * KPT;
  float* S_row = reinterpret_cast<float*>(state + (int64_t)slot * state_stride + state_offset) +
                 (((int64_t)h * e + (has ? j : 0)) * NG + g_lane) * KPT;
  float S[KPT];
#pragma unroll
  for (int i = 0; i < KPT; ++i) S[i] = has ? S_row[i] : 0.f;
  const T* vp = v_in + (int64_t)h * e + (has ? j : 0);
  const float4* head4 = reinterpret_cast<const float4*>(head_in);
  float kn[KPT], qn[KPT], vn;
  float4 scn;
  auto fetch = [&](int64_t r) {
    const float* kr = kq_in + (r * G + kv) * 2 * DP + g_lane * KPT;
#pragma unroll
    for (int i = 0; i < KPT; ++i) {
      kn[i] = kr[i];
      qn[i] = kr[DP + i];
    }
    vn = to_float(vp[r * in_stride]);
    scn = head4[r * H + h];
  };
  fetch(r0);
  for (int64_t r = r0; r < r1; ++r) {
    float k[KPT], q[KPT];
#pragma unroll
    for (int i = 0; i < KPT; ++i) k[i] = kn[i], q[i] = qn[i];
    const float v = vn;
    const float4 sc = scn;
    if (r + 1 < r1) fetch(r + 1);
    float sk = 0.f, sq = 0.f;
#pragma unroll
    for (int i = 0; i < KPT; ++i) {
      sk = fmaf(S[i], k[i], sk);
      sq = fmaf(S[i], q[i], sq);
    }
    sk = dr_group_sum(sk, NG);
    sq = dr_group_sum(sq, NG);
    const float u = sc.x * (v - sc.y * sk);
    const float o = fmaf(sc.y, sq, u * sc.z);
#pragma unroll
    for (int i = 0; i < KPT; ++i) S[i] = fmaf(k[i], u, sc.y * S[i]);
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
                             void* workspace_f32, int64_t workspace_floats, int dtype, void* stream) {
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
  const int64_t need = he_delta_workspace_floats(rows, H, G, d);
  HE_REQUIRE(workspace_f32 != nullptr && workspace_floats >= need && ((uintptr_t)workspace_f32 & 15) == 0,
             "he_delta_scan: workspace of %lld floats (16-byte aligned), need %lld", (long long)workspace_floats,
             (long long)need);
  if (rows == 0 || num_seqs == 0) return 0;
  hipStream_t s = (hipStream_t)stream;
  const int DP = ng * kpt;
  float* kq_ws = (float*)workspace_f32;
  float* head_ws = kq_ws + (int64_t)rows * G * 2 * DP;
  const int64_t units = (int64_t)rows * G;
  const unsigned pblocks = (unsigned)((units + 3) / 4);
  if (dtype == HE_BF16)
    delta_prepare_kernel<bf16_t><<<pblocks, 256, 0, s>>>(kq_ws, head_ws, (const bf16_t*)q, (const bf16_t*)k, in_stride,
                                                         (const float*)ba_f32, a_log, dt_bias, w_dtype, rows, H, G, d, DP,
                                                         q_scale, unit_eps);
  else
    delta_prepare_kernel<float><<<pblocks, 256, 0, s>>>(kq_ws, head_ws, (const float*)q, (const float*)k, in_stride,
                                                        (const float*)ba_f32, a_log, dt_bias, w_dtype, rows, H, G, d, DP,
                                                        q_scale, unit_eps);
  int rc = he_check_launch("he_delta_scan (prepare)");
  if (rc) return rc;
  const int per_block = 64 / ng;
  const dim3 grid(num_seqs, H, (e + per_block - 1) / per_block);
  HE_REQUIRE(grid.y <= 65535 && grid.z <= 65535, "he_delta_scan: too many heads or value tiles for one launch");
#define DR_ARGS(T)                                                                                          \
  (float*)y_f32, kq_ws, head_ws, (const T*)v, in_stride, (uint8_t*)state, state_stride, state_offset,       \
      (const int32_t*)cu_seqlens, (const int32_t*)seq_slot, H, G, e
#define DR_STAGED(T, KPT, NG)           \
  if (kpt == KPT && ng == NG) {         \
    delta_scan_kernel<T, KPT, NG><<<grid, 64, 0, s>>>(DR_ARGS(T)); \
    launched = true;                    \
  }
#define DR_STAGED_ALL(T)                                                                                         \
  DR_STAGED(T, 8, 1) DR_STAGED(T, 8, 2) DR_STAGED(T, 8, 4) DR_STAGED(T, 8, 8) DR_STAGED(T, 8, 16)                  \
  DR_STAGED(T, 16, 16) DR_STAGED(T, 24, 1) DR_STAGED(T, 24, 2) DR_STAGED(T, 24, 4) DR_STAGED(T, 24, 8)
#define DR_DIRECT(T)                                                                   \
  if (kpt == 8) delta_scan_direct_kernel<T, 8><<<grid, 64, 0, s>>>(DR_ARGS(T), ng);        \
  else if (kpt == 16) delta_scan_direct_kernel<T, 16><<<grid, 64, 0, s>>>(DR_ARGS(T), ng); \
  else if (kpt == 24) delta_scan_direct_kernel<T, 24><<<grid, 64, 0, s>>>(DR_ARGS(T), ng); \
  else delta_scan_direct_kernel<T, 32><<<grid, 64, 0, s>>>(DR_ARGS(T), ng)
  bool launched = false;
  if (DP <= DR_MAX_DP) {
    if (dtype == HE_BF16) {
      DR_STAGED_ALL(bf16_t)
    } else {
      DR_STAGED_ALL(float)
    }
  }
  if (!launched) {      // wider keys, or a split of the key dims the staged kernel is not built for
    if (dtype == HE_BF16) {
      DR_DIRECT(bf16_t);
    } else {
      DR_DIRECT(float);
    }
  }
#undef DR_DIRECT
#undef DR_STAGED_ALL
#undef DR_STAGED
#undef DR_ARGS
  return he_check_launch("he_delta_scan");
}
