// Kernels of a state-space mixer (a selective scan with a short causal convolution in front and a
// gated, grouped RMS norm behind), over the packed rows of a step. What a sequence carries from step
// to step lives in its row of the cache's state area, in fp32: the last K-1 inputs of the
// convolution, [K-1][C], and then the state of the scan, he_ssm_state_floats() floats in the order the
// scan's threads hold them. Everything that enters the recurrence is fp32.
#include "common.h"
#include "hector_kernels.h"

__device__ __forceinline__ float ss_silu(float z) { return z / (1.f + expf(-z)); }
__device__ __forceinline__ float ss_softplus(float z) { return z > 20.f ? z : log1pf(expf(z)); }

// ---- causal convolution per channel ---------------------------------------------------------
// out[row, c] = silu(bias[c] + sum_j taps[c, j] * u[pos - (K-1) + j, c]): the last tap weighs the
// row's own input (bias null: none; act 0: the sum as it is, without silu). Inputs before the step's first row of the sequence come from the carried inputs
// (zeros at a sequence's start). SINGLE: every sequence brings one row, and the thread that computed
// (row, c) also moves the carried inputs on; otherwise conv_carry_kernel does that afterwards.
template <typename T, bool SINGLE>
__global__ void conv_taps_kernel(T* __restrict__ out, const T* __restrict__ x, int64_t x_stride,
                                 const void* __restrict__ taps, const void* __restrict__ bias, int w_dtype,
                                 uint8_t* __restrict__ state, int64_t state_stride,
                                 const int32_t* __restrict__ positions, const int32_t* __restrict__ row_seq,
                                 const int32_t* __restrict__ seq_slot, const int32_t* __restrict__ seq_start,
                                 int C, int K, int act) {
  const int64_t row = blockIdx.y;
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  if (c >= C) return;
  const int seq = row_seq[row];
  const int slot = seq < 0 ? -1 : seq_slot[seq];
  if (slot < 0) {   // a padding row stays finite
    out[row * (int64_t)C + c] = from_float<T>(0.f);
    return;
  }
  const int before = positions[row] - seq_start[seq];   // rows of the same sequence ahead of this one in the step
  float* hist = reinterpret_cast<float*>(state + (int64_t)slot * state_stride);
  float acc = bias ? load_param(bias, c, w_dtype) : 0.f;
  for (int j = 0; j < K; ++j) {
    const int back = K - 1 - j;
    float u;
    if (back <= before)
      u = to_float(x[(row - back) * x_stride + c]);
    else
      u = hist[(int64_t)(K - 1 - (back - before)) * C + c];
    acc = fmaf(load_param(taps, (int64_t)c * K + j, w_dtype), u, acc);
  }
  out[row * (int64_t)C + c] = from_float<T>(act ? ss_silu(acc) : acc);
  if (SINGLE) {
    for (int i = 0; i + 2 < K; ++i) hist[(int64_t)i * C + c] = hist[(int64_t)(i + 1) * C + c];
    if (K > 1) hist[(int64_t)(K - 2) * C + c] = to_float(x[row * x_stride + c]);
  }
}

// The carried inputs after a step: the last K-1 inputs of the sequence, from its new rows and, where
// those are fewer, from what was carried before. One thread owns (sequence, channel).
template <typename T>
__global__ void conv_carry_kernel(const T* __restrict__ x, int64_t x_stride, uint8_t* __restrict__ state,
                                  int64_t state_stride, const int32_t* __restrict__ cu_seqlens,
                                  const int32_t* __restrict__ seq_slot, int C, int K) {
  const int seq = blockIdx.y;
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  if (c >= C) return;
  const int slot = seq_slot[seq];
  if (slot < 0) return;
  const int end = cu_seqlens[seq + 1];
  const int n = end - cu_seqlens[seq];
  if (n <= 0) return;
  float* hist = reinterpret_cast<float*>(state + (int64_t)slot * state_stride);
  // entry i comes from entry i + n or from a new row: entries are read before they are written
  for (int i = 0; i < K - 1; ++i) {
    const int back = K - 1 - i;
    hist[(int64_t)i * C + c] = back <= n ? to_float(x[(int64_t)(end - back) * x_stride + c])
                                         : hist[(int64_t)(i + n) * C + c];
  }
}

extern "C" int he_conv_state(void* out, const void* x, int64_t x_stride, const void* taps, const void* bias,
                             int w_dtype, void* state, int64_t state_stride, const void* positions,
                             const void* row_seq, const void* seq_slot, const void* seq_start,
                             const void* cu_seqlens, int rows, int num_seqs, int C, int K, int all_single,
                             int act, int dtype, void* stream) {
  HE_REQUIRE(rows >= 0 && num_seqs >= 0 && C > 0 && K >= 1 && K <= 64, "he_conv_state: bad sizes rows=%d C=%d K=%d", rows,
             C, K);
  HE_REQUIRE(dtype == HE_BF16 || dtype == HE_F32, "he_conv_state: unknown dtype %d", dtype);
  HE_REQUIRE(state != nullptr && state_stride >= (int64_t)(K - 1) * C * 4 && state_stride % 4 == 0,
             "he_conv_state: the state row is too short for %d x %d carried inputs", K - 1, C);
  if (rows == 0) return 0;
  hipStream_t s = (hipStream_t)stream;
  const int threads = C >= 256 ? 256 : 64;
  const dim3 grid((C + threads - 1) / threads, rows);
#define CONV_LAUNCH(T, SINGLE)                                                                          \
  conv_taps_kernel<T, SINGLE><<<grid, threads, 0, s>>>(                                                 \
      (T*)out, (const T*)x, x_stride, taps, bias, w_dtype, (uint8_t*)state, state_stride,               \
      (const int32_t*)positions, (const int32_t*)row_seq, (const int32_t*)seq_slot, (const int32_t*)seq_start, C, K, act)
  if (dtype == HE_BF16) {
    if (all_single) CONV_LAUNCH(bf16_t, true); else CONV_LAUNCH(bf16_t, false);
  } else {
    if (all_single) CONV_LAUNCH(float, true); else CONV_LAUNCH(float, false);
  }
#undef CONV_LAUNCH
  int st = he_check_launch("he_conv_state");
  if (st || all_single || num_seqs == 0 || K == 1) return st;
  const dim3 cgrid((C + threads - 1) / threads, num_seqs);
  if (dtype == HE_BF16)
    conv_carry_kernel<bf16_t><<<cgrid, threads, 0, s>>>((const bf16_t*)x, x_stride, (uint8_t*)state, state_stride,
                                                        (const int32_t*)cu_seqlens, (const int32_t*)seq_slot, C, K);
  else
    conv_carry_kernel<float><<<cgrid, threads, 0, s>>>((const float*)x, x_stride, (uint8_t*)state, state_stride,
                                                       (const int32_t*)cu_seqlens, (const int32_t*)seq_slot, C, K);
  return he_check_launch("he_conv_state (carry)");
}

// ---- selective scan ---------------------------------------------------------------------------
// Per head r (its B and C vectors are those of group r / (R / Q)) and token t:
//   dt = softplus(dt_in + dt_bias_r),  S <- exp(-exp(A_log_r) dt) S + dt B x^T,  y = S^T C + D_r x
// with S [N][P] carried in fp32. A thread holds NPT neighbouring state dims of one value dim p; the NG
// threads of a p are neighbouring lanes, and their partial sums of y meet in a butterfly whose order
// does not depend on the step. A workgroup takes PB value dims of one (sequence, head) and walks the
// sequence's rows in order; what a token brings (its B and C, the x of the workgroup's value dims,
// its step size and decay, which one thread a token computes) is staged through LDS a tile of tokens
// at a time, the next tile's loads in flight while this one is computed. In the state area the
// workgroup's share of S lies in the order its threads load it, 16 bytes a lane: [i / 4][thread][i % 4].
#define SS_PRE 16      // values a thread fetches for the next tile
// state dims a thread holds. Measured at 64 heads of 64 with a state of 128, one prompt of 2,048 tokens: 0.93 ms
// with 8 (a wavefront a SIMD), 1.20 ms with 4 (two a SIMD, but every workgroup stages all of B and C for half as
// many value dims)
static inline int ss_npt(int N) { return N <= 512 ? 8 : 16; }
static inline int ss_groups(int N) {
  const int npt = ss_npt(N);
  int ng = 1;
  while (ng * npt < N) ng *= 2;
  return ng;
}
static inline int ss_pb(int N, int P) {
  const int most = 256 / ss_groups(N);
  return P < most ? P : most;
}

// TRIM: the tile is a small part of what the threads could stage (a one-token step), and the loops over a
// thread's values end early. They are uniform branches, but behind branches the compiler waits for every load in
// flight, so the long tiles of a prompt run without them.
template <typename T, int NPT, bool TRIM>
__global__ __launch_bounds__(256) void ssm_scan_kernel(
    float* __restrict__ y, const T* __restrict__ xbc, const T* __restrict__ dt_in, int64_t dt_stride,
    const void* __restrict__ dt_bias, const void* __restrict__ a_log, const void* __restrict__ d_skip, int w_dtype,
    uint8_t* __restrict__ state, int64_t state_stride, int64_t state_offset, const int32_t* __restrict__ cu_seqlens,
    const int32_t* __restrict__ seq_slot, int R, int Q, int N, int P, int NG, int PB, int TT) {
  extern __shared__ float4 ss_lds4[];
  float* lds = reinterpret_cast<float*>(ss_lds4);
  const int seq = blockIdx.z, r = blockIdx.y;
  const int slot = seq_slot[seq];
  if (slot < 0) return;
  const int t0 = cu_seqlens[seq], t1 = cu_seqlens[seq + 1];
  if (t1 <= t0) return;
  const int tid = threadIdx.x, threads = blockDim.x;
  const int ng = tid % NG;
  const bool own = tid < PB * NG;                       // the thread holds a share of the state
  const int pl = own ? tid / NG : 0;
  const int p0 = blockIdx.x * PB;
  const bool live = own && p0 + pl < P;
  const int n0 = ng * NPT;
  const int Npad = NG * NPT;
  const int W = (2 * Npad + PB + 2 + 3) & ~3;           // floats a token takes in LDS: B, C, x, dt, decay
  const int inner = R * P;
  const int C = inner + 2 * Q * N;
  const int q = r / (R / Q);
  const int share = PB * NG * NPT;                      // floats of the workgroup's part of S
  float* S = reinterpret_cast<float*>(state + (int64_t)slot * state_stride + state_offset) +
             ((int64_t)r * gridDim.x + blockIdx.x) * share;
  float s[NPT];
#pragma unroll
  for (int i4 = 0; i4 < NPT / 4; ++i4) {
    const float4 v = own ? *reinterpret_cast<const float4*>(S + ((int64_t)i4 * PB * NG + tid) * 4) : make_float4(0, 0, 0, 0);
    s[4 * i4] = v.x, s[4 * i4 + 1] = v.y, s[4 * i4 + 2] = v.z, s[4 * i4 + 3] = v.w;
  }
  const float a = -expf(load_param(a_log, r, w_dtype));
  const float dk = load_param(d_skip, r, w_dtype);
  const float db = load_param(dt_bias, r, w_dtype);
  const int tile_floats = TT * W;
  // What thread `tid` stages of a tile does not change from tile to tile: value k is token tok_of[k]'s float
  // idx % W, which comes from column col[k] of the token's row of xbc (B, C, x), is padding (a zero), or is not
  // this loop's (the two floats of a token's step size and decay: threads 0 .. 2 TT - 1 bring those). The loads
  // carry no branch, so that a tile's loads go out together and stay in flight while the tile before is
  // computed; they are turned into values when they are written to LDS.
  enum { SS_SKIP = 0, SS_ZERO = 1, SS_VALUE = 2 };
  int col[SS_PRE], tok_of[SS_PRE];
  unsigned kinds = 0;                                  // two bits a value
#pragma unroll
  for (int k = 0; k < SS_PRE; ++k) {
    col[k] = 0, tok_of[k] = 0;
    if (TRIM && k * threads >= tile_floats) break;
    const int idx = tid + k * threads;
    const int tt = idx / W, j = idx - tt * W;
    int kind = SS_SKIP, c = 0;
    if (idx < tile_floats && j < 2 * Npad + PB) {
      kind = SS_ZERO;
      if (j < Npad) {
        if (j < N) kind = SS_VALUE, c = inner + q * N + j;
      } else if (j < 2 * Npad) {
        if (j - Npad < N) kind = SS_VALUE, c = inner + (Q + q) * N + (j - Npad);
      } else if (p0 + (j - 2 * Npad) < P) {
        kind = SS_VALUE, c = r * P + p0 + (j - 2 * Npad);
      }
    }
    col[k] = c;
    tok_of[k] = kind == SS_VALUE ? tt : 0;
    kinds |= (unsigned)kind << (2 * k);
  }
  T pre[SS_PRE], pre_dt;
  auto fetch = [&](int first) {
    const int last = t1 - 1 - first;                   // tokens beyond the sequence's rows read its last row
    const T* base = xbc + (int64_t)first * C;
#pragma unroll
    for (int k = 0; k < SS_PRE; ++k) {
      if (TRIM && k * threads >= tile_floats) break;
      pre[k] = base[min(tok_of[k], last) * C + col[k]];
    }
    pre_dt = dt_in[(int64_t)(first + min(min(tid >> 1, TT - 1), last)) * dt_stride + r];
  };
  auto put = [&](int buf) {
    float* dst = lds + buf * tile_floats;
#pragma unroll
    for (int k = 0; k < SS_PRE; ++k) {
      if (TRIM && k * threads >= tile_floats) break;
      const int kind = (kinds >> (2 * k)) & 3;
      if (kind != SS_SKIP) dst[tid + k * threads] = kind == SS_ZERO ? 0.f : to_float(pre[k]);
    }
    if (tid < 2 * TT) {
      const float dt = ss_softplus(to_float(pre_dt) + db);
      dst[(tid >> 1) * W + 2 * Npad + PB + (tid & 1)] = (tid & 1) ? expf(a * dt) : dt;
    }
  };
  fetch(t0);
  put(0);
  __syncthreads();
  int buf = 0;
  for (int first = t0; first < t1; first += TT, buf ^= 1) {
    const bool more = first + TT < t1;
    if (more) fetch(first + TT);
    const int count = min(TT, t1 - first);
    const float* mine = lds + buf * tile_floats + n0;                  // the thread's own B values of the tile's first token
    const float* shared = lds + buf * tile_floats + 2 * Npad;          // x of the value dims, then dt and decay
    float* ytile = y + (int64_t)first * inner + r * P + p0 + pl;
    // two tokens a turn: their values are read from LDS together, their sums of y meet side by side. A turn
    // whose second token lies beyond the rows runs it with decay 1 and step 0, which leaves S as it is.
    for (int tt = 0; tt < count; tt += 2) {
      const bool two = tt + 1 < count;
      const int ta = tt * W, tb = (two ? tt + 1 : tt) * W;
      float4 ba[NPT / 4], ca[NPT / 4], bb[NPT / 4], cb[NPT / 4];
#pragma unroll
      for (int i4 = 0; i4 < NPT / 4; ++i4) {
        ba[i4] = *reinterpret_cast<const float4*>(mine + ta + 4 * i4);
        ca[i4] = *reinterpret_cast<const float4*>(mine + ta + Npad + 4 * i4);
        bb[i4] = *reinterpret_cast<const float4*>(mine + tb + 4 * i4);
        cb[i4] = *reinterpret_cast<const float4*>(mine + tb + Npad + 4 * i4);
      }
      const float xa = shared[ta + pl], xb = shared[tb + pl];
      const float dta = shared[ta + PB], dtb = two ? shared[tb + PB] : 0.f;
      const float da = shared[ta + PB + 1], dbb = two ? shared[tb + PB + 1] : 1.f;
      const float dtxa = dta * xa, dtxb = dtb * xb;
      float acca = 0.f, accb = 0.f;
#pragma unroll
      for (int i4 = 0; i4 < NPT / 4; ++i4) {
        const float b[4] = {ba[i4].x, ba[i4].y, ba[i4].z, ba[i4].w}, c[4] = {ca[i4].x, ca[i4].y, ca[i4].z, ca[i4].w};
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          s[4 * i4 + e] = fmaf(da, s[4 * i4 + e], dtxa * b[e]);
          acca = fmaf(s[4 * i4 + e], c[e], acca);
        }
      }
#pragma unroll
      for (int i4 = 0; i4 < NPT / 4; ++i4) {
        const float b[4] = {bb[i4].x, bb[i4].y, bb[i4].z, bb[i4].w}, c[4] = {cb[i4].x, cb[i4].y, cb[i4].z, cb[i4].w};
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          s[4 * i4 + e] = fmaf(dbb, s[4 * i4 + e], dtxb * b[e]);
          accb = fmaf(s[4 * i4 + e], c[e], accb);
        }
      }
      // the NG neighbouring lanes of a value dim: through the vector ALU's own lane exchanges (every lane
      // of the wavefront runs this loop, which they require)
      if (NG > 1) acca += lane_xor1(acca), accb += lane_xor1(accb);
      if (NG > 2) acca += lane_xor2(acca), accb += lane_xor2(accb);
      if (NG > 4) acca += lane_xor4(acca), accb += lane_xor4(accb);
      if (NG > 8) acca += lane_xor8(acca), accb += lane_xor8(accb);
      if (NG > 16) acca = xor16_sum(acca), accb = xor16_sum(accb);
      if (NG > 32) acca = xor32_sum(acca), accb = xor32_sum(accb);
      if (ng == 0 && live) {
        ytile[(int64_t)tt * inner] = fmaf(dk, xa, acca);
        if (two) ytile[(int64_t)(tt + 1) * inner] = fmaf(dk, xb, accb);
      }
    }
    if (more) put(buf ^ 1);
    __syncthreads();
  }
  if (own) {
#pragma unroll
    for (int i4 = 0; i4 < NPT / 4; ++i4)
      *reinterpret_cast<float4*>(S + ((int64_t)i4 * PB * NG + tid) * 4) =
          make_float4(s[4 * i4], s[4 * i4 + 1], s[4 * i4 + 2], s[4 * i4 + 3]);
  }
}

extern "C" int64_t he_ssm_state_floats(int R, int P, int N) {
  if (R <= 0 || P <= 0 || N <= 0) return 0;
  const int PB = ss_pb(N, P);
  return (int64_t)R * ((P + PB - 1) / PB) * PB * ss_groups(N) * ss_npt(N);
}

extern "C" int he_ssm_scan(void* y_f32, const void* xbc, const void* dt_in, int64_t dt_stride, const void* dt_bias,
                           const void* a_log, const void* d_skip, int w_dtype, void* state, int64_t state_stride,
                           int64_t state_offset, const void* cu_seqlens, const void* seq_slot, int rows, int num_seqs,
                           int max_q_len, int R, int Q, int N, int P, int dtype, void* stream) {
  HE_REQUIRE(rows >= 0 && num_seqs >= 0 && R > 0 && Q > 0 && N > 0 && P > 0 && R % Q == 0,
             "he_ssm_scan: bad sizes R=%d Q=%d N=%d P=%d", R, Q, N, P);
  HE_REQUIRE(N <= 1024, "he_ssm_scan: state size %d above 1024", N);
  HE_REQUIRE(dtype == HE_BF16 || dtype == HE_F32, "he_ssm_scan: unknown dtype %d", dtype);
  HE_REQUIRE(state != nullptr && state_offset % 16 == 0 && state_stride % 16 == 0 &&
                 state_stride >= state_offset + 4 * he_ssm_state_floats(R, P, N),
             "he_ssm_scan: the state row is too short or not aligned");
  if (rows == 0 || num_seqs == 0) return 0;
  const int NG = ss_groups(N);
  const int PB = ss_pb(N, P);
  const int threads = (PB * NG + 63) / 64 * 64;
  const int W = (2 * NG * ss_npt(N) + PB + 2 + 3) & ~3;
  int TT = SS_PRE * threads / W;
  TT = TT < 1 ? 1 : (TT > 16 ? 16 : TT);
  if (max_q_len > 0 && TT > max_q_len) TT = max_q_len;      // no sequence brings more rows than that
  HE_REQUIRE(W <= SS_PRE * threads, "he_ssm_scan: a token's %d values do not fit a tile", W);
  if (2 * TT > threads) TT = threads / 2;               // a thread a token brings its step size, another its decay
  const size_t lds_bytes = (size_t)2 * TT * W * sizeof(float);
  const dim3 grid((P + PB - 1) / PB, R, num_seqs);
  hipStream_t s = (hipStream_t)stream;
  const bool trim = TT * W <= (SS_PRE / 2) * threads;
#define SCAN_LAUNCH(T, NPT)                                                                                       \
  if (trim) SCAN_LAUNCH_(T, NPT, true); else SCAN_LAUNCH_(T, NPT, false)
#define SCAN_LAUNCH_(T, NPT, TRIM)                                                                                \
  ssm_scan_kernel<T, NPT, TRIM><<<grid, threads, lds_bytes, s>>>(                                                       \
      (float*)y_f32, (const T*)xbc, (const T*)dt_in, dt_stride, dt_bias, a_log, d_skip, w_dtype, (uint8_t*)state, \
      state_stride, state_offset, (const int32_t*)cu_seqlens, (const int32_t*)seq_slot, R, Q, N, P, NG, PB, TT)
  const int npt = ss_npt(N);
  if (dtype == HE_BF16) {
    if (npt == 8) { SCAN_LAUNCH(bf16_t, 8); } else { SCAN_LAUNCH(bf16_t, 16); }
  } else {
    if (npt == 8) { SCAN_LAUNCH(float, 8); } else { SCAN_LAUNCH(float, 16); }
  }
#undef SCAN_LAUNCH
#undef SCAN_LAUNCH_
  return he_check_launch("he_ssm_scan");
}

// ---- gated, grouped RMS norm ------------------------------------------------------------------
// gate_after 0:  out[row, c] = v / sqrt(mean over c's part of v^2 + eps) * weight[c], v = y[row, c] * silu(z[row, c]):
// the product with silu(z) is formed first and normalised afterwards, each of the `parts` equal stretches of
// a row by a root mean square of its own.
// gate_after 1:  out[row, c] = y / sqrt(mean over c's part of y^2 + eps) * weight[c] * sigmoid(z[row, c]) * out_scale:
// the stretch is normalised as it is and the gate, a sigmoid, multiplies the result. One workgroup a (row, part).
template <typename T>
__global__ void gated_group_norm_kernel(T* __restrict__ out, const float* __restrict__ y, const T* __restrict__ z,
                                        int64_t z_stride, const void* __restrict__ weight, int w_dtype, int W,
                                        int parts, float eps, int gate_after, float out_scale) {
  __shared__ float scratch[16];
  const int64_t row = blockIdx.y;
  const int width = W / parts;
  const int c0 = blockIdx.x * width;
  float sq = 0.f;
  for (int i = threadIdx.x; i < width; i += blockDim.x) {
    float v = y[row * W + c0 + i];
    if (!gate_after) v *= ss_silu(to_float(z[row * z_stride + c0 + i]));
    sq = fmaf(v, v, sq);
  }
  const float total = block_sum(sq, scratch);
  const float inv = 1.f / sqrtf(total / (float)width + eps);
  for (int i = threadIdx.x; i < width; i += blockDim.x) {
    const float g = to_float(z[row * z_stride + c0 + i]);
    float v = y[row * W + c0 + i];
    if (!gate_after) {
      v = v * ss_silu(g) * inv * load_param(weight, c0 + i, w_dtype);
    } else {
      v = v * inv * load_param(weight, c0 + i, w_dtype) * (out_scale / (1.f + expf(-g)));
      if (gate_after == 2) v *= g;      // silu(g) = g * sigmoid(g)
    }
    out[row * W + c0 + i] = from_float<T>(v);
  }
}

extern "C" int he_gated_group_norm(void* out, const void* y_f32, const void* z, int64_t z_stride, const void* weight,
                                   int w_dtype, int rows, int W, int parts, float eps, int gate_after, float out_scale,
                                   int dtype, void* stream) {
  HE_REQUIRE(rows >= 0 && W > 0 && parts > 0 && W % parts == 0, "he_gated_group_norm: bad sizes W=%d parts=%d", W, parts);
  HE_REQUIRE(dtype == HE_BF16 || dtype == HE_F32, "he_gated_group_norm: unknown dtype %d", dtype);
  if (rows == 0) return 0;
  const int width = W / parts;
  const int threads = width >= 1024 ? 256 : (width >= 256 ? 128 : 64);
  const dim3 grid(parts, rows);
  hipStream_t s = (hipStream_t)stream;
  if (dtype == HE_BF16)
    gated_group_norm_kernel<bf16_t><<<grid, threads, 0, s>>>((bf16_t*)out, (const float*)y_f32, (const bf16_t*)z, z_stride,
                                                             weight, w_dtype, W, parts, eps, gate_after, out_scale);
  else
    gated_group_norm_kernel<float><<<grid, threads, 0, s>>>((float*)out, (const float*)y_f32, (const float*)z, z_stride,
                                                            weight, w_dtype, W, parts, eps, gate_after, out_scale);
  return he_check_launch("he_gated_group_norm");
}
