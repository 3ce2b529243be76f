// A matrix memory per head that is carried from token to token (the mLSTM recurrence):
//   m_t = max(f_t + m_(t-1), i_t)
//   S_t = exp(f_t + m_(t-1) - m_t) S_(t-1) + exp(i_t - m_t) k_t v_t^T      (dk x dv)
//   n_t = exp(f_t + m_(t-1) - m_t) n_(t-1) + exp(i_t - m_t) k_t            (dk)
//   y_t = S_t^T q_t / (max(|n_t . q_t|, exp(-m_t)) + 1e-6)
// with i_t and f_t the logarithms of the input and forget gates. S, n and m start at zero and live in
// 32-bit floats in the sequence's row of the cache's state area; everything here is fp32 arithmetic, only
// q, k and v are read in the activation dtype.
#include "common.h"
#include "hector_kernels.h"

#define MM_NPT 8   // key dims of S a thread holds for its value dim

static int mm_groups(int dk) {
  int ng = 1;
  while (ng * MM_NPT < dk) ng *= 2;
  return ng;
}
static int mm_pb(int dk, int dv) {
  const int pb = 256 / mm_groups(dk);
  return dv < pb ? dv : (pb < 1 ? 1 : pb);
}

extern "C" int64_t he_mlstm_state_floats(int H, int dk, int dv) {
  if (H <= 0 || dk <= 0 || dv <= 0) return 0;
  const int64_t dkp = (int64_t)mm_groups(dk) * MM_NPT;
  const int pb = mm_pb(dk, dv);
  const int64_t tiles = (dv + pb - 1) / pb;
  // S as [H][dv][dkp]; then, for every (head, tile of value dims), that workgroup's own copy of n (dkp) and m (1 of 4)
  return (int64_t)H * dv * dkp + (int64_t)H * tiles * (dkp + 4);
}

// The logarithms of the two gates from their pre-activations x (biases added here):
//   i = cap tanh((x_i + b_i) / cap),   f = logsigmoid(cap tanh((x_f + b_f) / cap));   cap <= 0: no bound.
// x: fp32 [rows, 2 H] (the i columns, then the f columns); out the same shape.
__global__ void mlstm_gates_kernel(float* __restrict__ out, const float* __restrict__ x, const void* __restrict__ bias,
                                   int b_dtype, int64_t n, int H, float cap) {
  const int64_t i = blockIdx.x * (int64_t)blockDim.x + threadIdx.x;
  if (i >= n) return;
  const int c = (int)(i % (2 * H));
  float z = x[i] + (bias ? load_param(bias, c, b_dtype) : 0.f);
  if (cap > 0.f) z = cap * tanhf(z / cap);
  if (c >= H) z = fminf(z, 0.f) - log1pf(expf(-fabsf(z)));
  out[i] = z;
}

extern "C" int he_mlstm_gates(void* out_f32, const void* x_f32, const void* bias, int bias_dtype, int rows, int H,
                              float cap, void* stream) {
  HE_REQUIRE(rows >= 0 && H > 0, "he_mlstm_gates: bad sizes rows=%d H=%d", rows, H);
  if (rows == 0) return 0;
  const int64_t n = (int64_t)rows * 2 * H;
  mlstm_gates_kernel<<<(int)((n + 255) / 256), 256, 0, (hipStream_t)stream>>>((float*)out_f32, (const float*)x_f32, bias,
                                                                              bias_dtype, n, H, cap);
  return he_check_launch("he_mlstm_gates");
}

template <typename T>
__device__ __forceinline__ void mm_load8(float* dst, const T* p, int have, bool vec) {
  if (sizeof(T) == 2 && vec) {
    const uint4 v = *reinterpret_cast<const uint4*>(p);
    const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      dst[2 * j] = __uint_as_float(w[j] << 16);
      dst[2 * j + 1] = __uint_as_float(w[j] & 0xffff0000u);
    }
  } else if (sizeof(T) == 4 && vec) {
    const float4 a = *reinterpret_cast<const float4*>(p);
    const float4 b = *reinterpret_cast<const float4*>((const float*)p + 4);
    dst[0] = a.x; dst[1] = a.y; dst[2] = a.z; dst[3] = a.w;
    dst[4] = b.x; dst[5] = b.y; dst[6] = b.z; dst[7] = b.w;
  } else {
#pragma unroll
    for (int e = 0; e < MM_NPT; ++e) dst[e] = e < have ? to_float(p[e]) : 0.f;
  }
}

// One workgroup a (tile of value dims, head, sequence). Thread (c, j) holds the MM_NPT key dims j of value
// dim c of S, and its own copy of those dims of n; the NG threads of a value dim are neighbouring lanes.
// (n and m are the same in every tile of a head: the same operations in the same order.)
// The rows of a sequence are walked in order, the operands of the next row asked for while this one is
// computed. The sums of a row do not depend on how the rows were cut into steps.
template <typename T>
__global__ void mlstm_scan_kernel(float* __restrict__ y, const T* __restrict__ q, const T* __restrict__ k,
                                  const T* __restrict__ v, int64_t in_stride, const float* __restrict__ gates,
                                  uint8_t* __restrict__ state, int64_t state_stride, int64_t state_offset,
                                  const int32_t* __restrict__ cu_seqlens, const int32_t* __restrict__ seq_slot, int H,
                                  int dk, int dv, int NG, int PB, float q_scale, int vec) {
  const int seq = blockIdx.z, h = blockIdx.y;
  const int slot = seq_slot[seq];
  const int r0 = cu_seqlens[seq], r1 = cu_seqlens[seq + 1];
  if (slot < 0 || r0 >= r1) return;
  const int c = threadIdx.x / NG, j = threadIdx.x % NG;
  const int col = blockIdx.x * PB + c;
  const bool active = c < PB && col < dv;
  const int colc = active ? col : 0;
  const int dkp = NG * MM_NPT;
  const int d0 = j * MM_NPT;
  const int have = dk - d0 < 0 ? 0 : (dk - d0 > MM_NPT ? MM_NPT : dk - d0);
  const bool full = vec && have == MM_NPT;
  float* st = reinterpret_cast<float*>(state + (int64_t)slot * state_stride + state_offset);
  float* sp = st + ((int64_t)h * dv + colc) * dkp + d0;
  // n and m are kept once a workgroup: each carries them on for itself, whenever it runs
  float* aux = st + (int64_t)H * dv * dkp + ((int64_t)h * gridDim.x + blockIdx.x) * (dkp + 4);
  float* np = aux + d0;
  float* mp = aux + dkp;
  float S[MM_NPT], nn[MM_NPT];
  {
    const float4 a = *reinterpret_cast<const float4*>(sp), b = *reinterpret_cast<const float4*>(sp + 4);
    S[0] = a.x; S[1] = a.y; S[2] = a.z; S[3] = a.w; S[4] = b.x; S[5] = b.y; S[6] = b.z; S[7] = b.w;
    const float4 e = *reinterpret_cast<const float4*>(np), f = *reinterpret_cast<const float4*>(np + 4);
    nn[0] = e.x; nn[1] = e.y; nn[2] = e.z; nn[3] = e.w; nn[4] = f.x; nn[5] = f.y; nn[6] = f.z; nn[7] = f.w;
  }
  float m = *mp;
  const int dlo = have > 0 ? d0 : 0;     // a thread without key dims reads the row's first ones and drops them
  float qn[MM_NPT], kn[MM_NPT], vn, ign, fgn;
  {
    const int64_t at = (int64_t)r0 * in_stride;
    mm_load8(qn, q + at + (int64_t)h * dk + dlo, have, full);
    mm_load8(kn, k + at + (int64_t)h * dk + dlo, have, full);
    vn = to_float(v[at + (int64_t)h * dv + colc]);
    ign = gates[(int64_t)r0 * 2 * H + h];
    fgn = gates[(int64_t)r0 * 2 * H + H + h];
  }
  for (int r = r0; r < r1; ++r) {
    float qc[MM_NPT], kc[MM_NPT];
#pragma unroll
    for (int e = 0; e < MM_NPT; ++e) {
      qc[e] = have > 0 ? qn[e] * q_scale : 0.f;
      kc[e] = have > 0 ? kn[e] : 0.f;
    }
    const float vc = vn, ig = ign, fg = fgn;
    {
      const int rn = r + 1 < r1 ? r + 1 : r;
      const int64_t at = (int64_t)rn * in_stride;
      mm_load8(qn, q + at + (int64_t)h * dk + dlo, have, full);
      mm_load8(kn, k + at + (int64_t)h * dk + dlo, have, full);
      vn = to_float(v[at + (int64_t)h * dv + colc]);
      ign = gates[(int64_t)rn * 2 * H + h];
      fgn = gates[(int64_t)rn * 2 * H + H + h];
    }
    const float mn = fmaxf(fg + m, ig);
    const float a = expf(fg + m - mn), b = expf(ig - mn);
    m = mn;
    float py = 0.f, pn = 0.f;
#pragma unroll
    for (int e = 0; e < MM_NPT; ++e) {
      const float bk = b * kc[e];
      S[e] = fmaf(a, S[e], bk * vc);
      nn[e] = fmaf(a, nn[e], bk);
      py = fmaf(S[e], qc[e], py);
      pn = fmaf(nn[e], qc[e], pn);
    }
    for (int off = NG >> 1; off > 0; off >>= 1) {
      py += __shfl_xor(py, off);
      pn += __shfl_xor(pn, off);
    }
    if (active && j == 0) y[(int64_t)r * H * dv + (int64_t)h * dv + col] = py / (fmaxf(fabsf(pn), expf(-m)) + 1e-6f);
  }
  if (active) {
    *reinterpret_cast<float4*>(sp) = make_float4(S[0], S[1], S[2], S[3]);
    *reinterpret_cast<float4*>(sp + 4) = make_float4(S[4], S[5], S[6], S[7]);
  }
  if (c == 0) {
    *reinterpret_cast<float4*>(np) = make_float4(nn[0], nn[1], nn[2], nn[3]);
    *reinterpret_cast<float4*>(np + 4) = make_float4(nn[4], nn[5], nn[6], nn[7]);
    if (j == 0) *mp = m;
  }
}

extern "C" int he_mlstm_scan(void* y_f32, const void* q, const void* k, const void* v, int64_t in_stride,
                             const void* gates_f32, void* state, int64_t state_stride, int64_t state_offset,
                             const void* cu_seqlens, const void* seq_slot, int rows, int num_seqs, int H, int dk, int dv,
                             float q_scale, int dtype, void* stream) {
  HE_REQUIRE(rows >= 0 && num_seqs >= 0 && H > 0 && dk > 0 && dv > 0, "he_mlstm_scan: bad sizes H=%d dk=%d dv=%d", H, dk, dv);
  HE_REQUIRE(dk <= 512, "he_mlstm_scan: key size %d above 512", dk);
  HE_REQUIRE(dtype == HE_BF16 || dtype == HE_F32, "he_mlstm_scan: unknown dtype %d", dtype);
  HE_REQUIRE(state != nullptr && state_offset % 16 == 0 && state_stride % 16 == 0 &&
                 state_stride >= state_offset + 4 * he_mlstm_state_floats(H, dk, dv),
             "he_mlstm_scan: the state row is too short or not aligned");
  if (rows == 0 || num_seqs == 0) return 0;
  const int NG = mm_groups(dk), PB = mm_pb(dk, dv);
  const int threads = (PB * NG + 63) / 64 * 64;
  const int esz = dtype == HE_BF16 ? 2 : 4;
  // whole 16-byte (bf16) or 32-byte (fp32) loads of a thread's key dims: every row and head starts aligned
  const int vec = dk % MM_NPT == 0 && (in_stride * esz) % 16 == 0 && (((uintptr_t)q | (uintptr_t)k) & 15) == 0;
  const dim3 grid((dv + PB - 1) / PB, H, num_seqs);
  hipStream_t s = (hipStream_t)stream;
  if (dtype == HE_BF16)
    mlstm_scan_kernel<bf16_t><<<grid, threads, 0, s>>>((float*)y_f32, (const bf16_t*)q, (const bf16_t*)k, (const bf16_t*)v,
                                                       in_stride, (const float*)gates_f32, (uint8_t*)state, state_stride,
                                                       state_offset, (const int32_t*)cu_seqlens, (const int32_t*)seq_slot,
                                                       H, dk, dv, NG, PB, q_scale, vec);
  else
    mlstm_scan_kernel<float><<<grid, threads, 0, s>>>((float*)y_f32, (const float*)q, (const float*)k, (const float*)v,
                                                      in_stride, (const float*)gates_f32, (uint8_t*)state, state_stride,
                                                      state_offset, (const int32_t*)cu_seqlens, (const int32_t*)seq_slot,
                                                      H, dk, dv, NG, PB, q_scale, vec);
  return he_check_launch("he_mlstm_scan");
}
