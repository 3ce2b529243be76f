// Row-wise kernels without reductions: embedding gather into the fp32 residual
// stream, row gather, gated activation (SiLU(gate) * up) and the materialising
// residual add.
#include "common.h"
#include "hector_kernels.h"

// out[t, :] = table[ids[t], :] * scale as fp32 (scale 1: the row as it is); an id outside
// [0, V) gives a zero row (reference: kernels/linear.cu:36-69).
template <typename T>
__global__ void embedding_kernel(float* __restrict__ out, const T* __restrict__ table,
                                 const int32_t* __restrict__ ids, int D, int V, float scale) {
  const int64_t t = blockIdx.x;
  const int id = ids[t];
  float* o = out + t * (int64_t)D;
  if (id < 0 || id >= V) {
    for (int i = threadIdx.x; i < D; i += blockDim.x) o[i] = 0.f;
    return;
  }
  const T* row = table + (int64_t)id * D;
  if (sizeof(T) == 2 && (D & 7) == 0 && (((uintptr_t)table | (uintptr_t)out) & 15) == 0) {
    // eight elements a thread and turn: one 16-byte load, two 16-byte stores
    for (int i = 8 * threadIdx.x; i < D; i += 8 * blockDim.x) {
      const uint4 v = *reinterpret_cast<const uint4*>(reinterpret_cast<const uint16_t*>(row) + i);
      const uint32_t w[4] = {v.x, v.y, v.z, v.w};
      float f[8];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        f[2 * j] = __uint_as_float(w[j] << 16) * scale;
        f[2 * j + 1] = __uint_as_float(w[j] & 0xffff0000u) * scale;
      }
      *reinterpret_cast<float4*>(o + i) = make_float4(f[0], f[1], f[2], f[3]);
      *reinterpret_cast<float4*>(o + i + 4) = make_float4(f[4], f[5], f[6], f[7]);
    }
    return;
  }
  for (int i = threadIdx.x; i < D; i += blockDim.x) o[i] = to_float(row[i]) * scale;
}

extern "C" int he_embedding(void* out_f32, const void* table, const void* ids, int rows, int D,
                            int V, int table_dtype, float scale, void* stream) {
  HE_REQUIRE(rows >= 0 && D > 0 && V > 0, "he_embedding: bad sizes rows=%d D=%d V=%d", rows, D, V);
  if (rows == 0) return 0;
  const int threads = D >= 1024 ? 256 : (D >= 256 ? 128 : 64);
  hipStream_t s = (hipStream_t)stream;
  if (table_dtype == HE_BF16)
    embedding_kernel<bf16_t><<<rows, threads, 0, s>>>((float*)out_f32, (const bf16_t*)table,
                                                      (const int32_t*)ids, D, V, scale);
  else if (table_dtype == HE_F32)
    embedding_kernel<float><<<rows, threads, 0, s>>>((float*)out_f32, (const float*)table,
                                                     (const int32_t*)ids, D, V, scale);
  else
    HE_REQUIRE(false, "he_embedding: unknown dtype %d", table_dtype);
  return he_check_launch("he_embedding");
}

// out[r, :] = src[rows[r], :]; a negative row index gives a zero row.
__global__ void gather_rows_f32_kernel(float* __restrict__ out, const float* __restrict__ src,
                                       const int32_t* __restrict__ rows, int D, int n_src) {
  const int64_t r = blockIdx.x;
  const int idx = rows[r];
  float* o = out + r * (int64_t)D;
  if (idx < 0 || idx >= n_src) {
    for (int i = threadIdx.x; i < D; i += blockDim.x) o[i] = 0.f;
    return;
  }
  const float* in = src + (int64_t)idx * D;
  if ((D & 3) == 0 && (((uintptr_t)src | (uintptr_t)out) & 15) == 0) {
    for (int i = 4 * threadIdx.x; i < D; i += 4 * blockDim.x)
      *reinterpret_cast<float4*>(o + i) = *reinterpret_cast<const float4*>(in + i);
    return;
  }
  for (int i = threadIdx.x; i < D; i += blockDim.x) o[i] = in[i];
}

extern "C" int he_gather_rows_f32(void* out, const void* src, const void* rows, int n_out, int D,
                                  int n_src, void* stream) {
  HE_REQUIRE(n_out >= 0 && D > 0 && n_src >= 0, "he_gather_rows_f32: bad sizes");
  if (n_out == 0) return 0;
  gather_rows_f32_kernel<<<n_out, 256, 0, (hipStream_t)stream>>>(
      (float*)out, (const float*)src, (const int32_t*)rows, D, n_src);
  return he_check_launch("he_gather_rows_f32");
}

// resid[r, :] += scale * delta[r, :], the residual sum in fp32 (scale 1: the plain sum).
template <typename T>
__global__ void residual_add_kernel(float* __restrict__ resid, const T* __restrict__ delta,
                                    int64_t n, float scale) {
  int64_t i = blockIdx.x * (int64_t)blockDim.x + threadIdx.x;
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (; i < n; i += stride) resid[i] += scale * to_float(delta[i]);
}

extern "C" int he_residual_add(void* resid_f32, const void* delta, int64_t n, int delta_dtype,
                               float scale, void* stream) {
  HE_REQUIRE(n >= 0, "he_residual_add: bad size");
  if (n == 0) return 0;
  int64_t blocks = (n + 255) / 256;
  if (blocks > 65535) blocks = 65535;
  hipStream_t s = (hipStream_t)stream;
  if (delta_dtype == HE_BF16)
    residual_add_kernel<bf16_t><<<(int)blocks, 256, 0, s>>>((float*)resid_f32,
                                                            (const bf16_t*)delta, n, scale);
  else if (delta_dtype == HE_F32)
    residual_add_kernel<float><<<(int)blocks, 256, 0, s>>>((float*)resid_f32, (const float*)delta,
                                                           n, scale);
  else
    HE_REQUIRE(false, "he_residual_add: unknown dtype %d", delta_dtype);
  return he_check_launch("he_residual_add");
}

// out[r, i] = silu(gate[r, i]) * up[r, i] with x = [rows, 2I],
// silu(z) = z / (1 + exp(-z)) in fp32 (reference: kernels/activations.cu:19-21,183-198).
// CLAMPED: the gated activation with its constants (common.h: he_gated_act).
// Column layout of x: gate then up (x[r, i], x[r, I + i]); or interleaved, as the
// fused gate||up weight of the MFMA path lays its rows out: gate i at column 2i,
// its up at 2i + 1.
// With splits > 0, x is the fp32 K slices [splits][rows][2I] of the gate||up product,
// added here in the order of the slice index.
template <typename T, typename TI, bool CLAMPED>
__global__ void silu_mul_kernel(T* __restrict__ out, const TI* __restrict__ x, int64_t rows,
                                int I, int interleaved, int splits, GatedAct act) {
  const int64_t n = rows * (int64_t)I;
  const int64_t split_stride = rows * 2 * (int64_t)I;
  int64_t i = blockIdx.x * (int64_t)blockDim.x + threadIdx.x;
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (; i < n; i += stride) {
    const int64_t r = i / I;
    const int c = (int)(i - r * I);
    const int gc = interleaved ? 2 * c : c;
    const int uc = interleaved ? gc + 1 : I + c;
    const TI* row = x + r * 2 * (int64_t)I;
    float g = to_float(row[gc]), u = to_float(row[uc]);
    for (int s = 1; s < splits; ++s) {
      g += to_float(row[s * split_stride + gc]);
      u += to_float(row[s * split_stride + uc]);
    }
    const float y = he_gated_act<CLAMPED>(g, u, act);
    out[i] = from_float<T>(y);
  }
}

// bf16, eight outputs per thread, I a multiple of 8: eight consecutive gates and their ups are
// two runs of 16 bytes, or, interleaved, one run of 32 bytes of (gate, up) pairs.
template <bool CLAMPED>
__global__ void silu_mul_vec_kernel(uint16_t* __restrict__ out, const uint16_t* __restrict__ x,
                                    int64_t rows, int I, int interleaved, GatedAct act) {
  const int64_t n8 = rows * (int64_t)(I >> 3);
  int64_t i = blockIdx.x * (int64_t)blockDim.x + threadIdx.x;
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  const int per_row = I >> 3;
  for (; i < n8; i += stride) {
    const int64_t r = i / per_row;
    const int c = (int)(i - r * per_row) << 3;
    const uint16_t* row = x + r * 2 * (int64_t)I;
    uint32_t o[4];
    if (interleaved) {
      const uint4 a = *reinterpret_cast<const uint4*>(row + 2 * c);
      const uint4 b = *reinterpret_cast<const uint4*>(row + 2 * c + 8);
      const uint32_t w[8] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};   // (gate, up) a word
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const float g0 = __uint_as_float(w[2 * j] << 16), u0 = __uint_as_float(w[2 * j] & 0xffff0000u);
        const float g1 = __uint_as_float(w[2 * j + 1] << 16), u1 = __uint_as_float(w[2 * j + 1] & 0xffff0000u);
        o[j] = pack2_bf16(he_gated_act<CLAMPED>(g0, u0, act), he_gated_act<CLAMPED>(g1, u1, act));
      }
    } else {
      const uint4 g4 = *reinterpret_cast<const uint4*>(row + c);
      const uint4 u4 = *reinterpret_cast<const uint4*>(row + I + c);
      const uint32_t gw[4] = {g4.x, g4.y, g4.z, g4.w}, uw[4] = {u4.x, u4.y, u4.z, u4.w};
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const float g0 = __uint_as_float(gw[j] << 16), g1 = __uint_as_float(gw[j] & 0xffff0000u);
        const float u0 = __uint_as_float(uw[j] << 16), u1 = __uint_as_float(uw[j] & 0xffff0000u);
        o[j] = pack2_bf16(he_gated_act<CLAMPED>(g0, u0, act), he_gated_act<CLAMPED>(g1, u1, act));
      }
    }
    *reinterpret_cast<uint4*>(out + r * (int64_t)I + c) = make_uint4(o[0], o[1], o[2], o[3]);
  }
}

template <bool CLAMPED>
static int gated_act_launch(void* out, const void* gate_up, int rows, int I, int interleaved, int splits,
                            int dtype, GatedAct act, hipStream_t s) {
  const int64_t n = (int64_t)rows * I;
  int64_t blocks = (n + 255) / 256;
  if (blocks > 65535 * 4) blocks = 65535 * 4;
  if (splits == 0 && dtype == HE_BF16 && (I & 7) == 0 &&
      ((((uintptr_t)out) | ((uintptr_t)gate_up)) & 15) == 0) {
    const int64_t n8 = n >> 3;
    int64_t vb = (n8 + 255) / 256;
    if (vb > 65535 * 4) vb = 65535 * 4;
    silu_mul_vec_kernel<CLAMPED><<<(int)vb, 256, 0, s>>>((uint16_t*)out, (const uint16_t*)gate_up, rows, I,
                                                         interleaved, act);
  } else if (splits > 0) {  // fp32 partial sums in
    if (dtype == HE_BF16)
      silu_mul_kernel<bf16_t, float, CLAMPED><<<(int)blocks, 256, 0, s>>>(
          (bf16_t*)out, (const float*)gate_up, rows, I, interleaved, splits, act);
    else
      silu_mul_kernel<float, float, CLAMPED><<<(int)blocks, 256, 0, s>>>(
          (float*)out, (const float*)gate_up, rows, I, interleaved, splits, act);
  } else if (dtype == HE_BF16) {
    silu_mul_kernel<bf16_t, bf16_t, CLAMPED><<<(int)blocks, 256, 0, s>>>(
        (bf16_t*)out, (const bf16_t*)gate_up, rows, I, interleaved, 1, act);
  } else {
    silu_mul_kernel<float, float, CLAMPED><<<(int)blocks, 256, 0, s>>>((float*)out, (const float*)gate_up,
                                                                       rows, I, interleaved, 1, act);
  }
  return he_check_launch("he_gated_act");
}

// out = act(gate) * up over gate||up columns as he_silu_mul takes them, with
// gate' = min(gate, limit), up' = clamp(up, -limit, limit) (limit <= 0: neither is bounded),
// out = gate' * sigmoid(alpha * gate') * (up' + up_shift). alpha 1, no limit and no shift is SiLU(gate) * up.
extern "C" int he_gated_act(void* out, const void* gate_up, int rows, int I, int interleaved, int splits,
                            int dtype, float alpha, float limit, float up_shift, void* stream) {
  HE_REQUIRE(rows >= 0 && I > 0, "he_gated_act: bad sizes rows=%d I=%d", rows, I);
  HE_REQUIRE(splits >= 0 && splits <= 64, "he_gated_act: bad slice count %d", splits);
  HE_REQUIRE(dtype == HE_BF16 || dtype == HE_F32, "he_gated_act: unknown dtype %d", dtype);
  if (rows == 0) return 0;
  GatedAct act;
  act.alpha = alpha;
  act.limit = limit > 0.f ? limit : INFINITY;
  act.shift = up_shift;
  if (alpha == 1.f && !(limit > 0.f) && up_shift == 0.f)
    return gated_act_launch<false>(out, gate_up, rows, I, interleaved, splits, dtype, act, (hipStream_t)stream);
  return gated_act_launch<true>(out, gate_up, rows, I, interleaved, splits, dtype, act, (hipStream_t)stream);
}

extern "C" int he_silu_mul(void* out, const void* gate_up, int rows, int I, int interleaved,
                           int splits, int dtype, void* stream) {
  return he_gated_act(out, gate_up, rows, I, interleaved, splits, dtype, 1.f, 0.f, 0.f, stream);
}

// ---- activations and gates of one input -----------------------------------------------------------
// kind 0: relu(x)^2; 1: gelu with tanh, 0.5 x (1 + tanh(sqrt(2/pi) (x + 0.044715 x^3))); 2: silu; 3: relu
#define HE_ACT_RELU2 0
#define HE_ACT_GELU_TANH 1
#define HE_ACT_SILU 2
#define HE_ACT_RELU 3
__device__ __forceinline__ float he_unary(float x, int kind) {
  if (kind == HE_ACT_RELU2) {
    const float r = fmaxf(x, 0.f);
    return r * r;
  }
  if (kind == HE_ACT_GELU_TANH) return 0.5f * x * (1.f + tanhf(0.7978845608028654f * (x + 0.044715f * x * x * x)));
  if (kind == HE_ACT_SILU) return x / (1.f + expf(-x));
  return fmaxf(x, 0.f);
}

// out[i] = act(x[i]), in place when out == x
template <typename T>
__global__ void unary_act_kernel(T* out, const T* x, int64_t n, int kind) {
  int64_t i = blockIdx.x * (int64_t)blockDim.x + threadIdx.x;
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (; i < n; i += stride) out[i] = from_float<T>(he_unary(to_float(x[i]), kind));
}

// The same over whole 16-byte pieces (8 bf16 or 4 fp32 a lane and turn); the launcher gives the rest to the kernel above.
template <typename T>
__global__ void unary_act_pieces_kernel(T* out, const T* x, int64_t pieces, int kind) {
  constexpr int VE = 16 / sizeof(T);
  int64_t i = blockIdx.x * (int64_t)blockDim.x + threadIdx.x;
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (; i < pieces; i += stride) {
    const uint4 v = reinterpret_cast<const uint4*>(x)[i];
    const uint32_t w[4] = {v.x, v.y, v.z, v.w};
    uint32_t o[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      if (VE == 8) {
        const float lo = he_unary(__uint_as_float(w[u] << 16), kind), hi = he_unary(__uint_as_float(w[u] & 0xffff0000u), kind);
        o[u] = (uint32_t)float_to_bf16_bits(lo) | ((uint32_t)float_to_bf16_bits(hi) << 16);
      } else {
        o[u] = __float_as_uint(he_unary(__uint_as_float(w[u]), kind));
      }
    }
    reinterpret_cast<uint4*>(out)[i] = make_uint4(o[0], o[1], o[2], o[3]);
  }
}

extern "C" int he_unary_act(void* out, const void* x, int64_t n, int kind, int dtype, void* stream) {
  HE_REQUIRE(n >= 0 && kind >= 0 && kind <= 3, "he_unary_act: bad size or kind %d", kind);
  HE_REQUIRE(dtype == HE_BF16 || dtype == HE_F32, "he_unary_act: unknown dtype %d", dtype);
  if (n == 0) return 0;
  hipStream_t s = (hipStream_t)stream;
  const int ve = dtype == HE_BF16 ? 8 : 4;
  int64_t done = 0;
  if ((((uintptr_t)out | (uintptr_t)x) & 15) == 0 && n >= ve) {
    const int64_t pieces = n / ve;
    int64_t blocks = (pieces + 255) / 256;
    if (blocks > 65535) blocks = 65535;
    if (dtype == HE_BF16) unary_act_pieces_kernel<bf16_t><<<(int)blocks, 256, 0, s>>>((bf16_t*)out, (const bf16_t*)x, pieces, kind);
    else unary_act_pieces_kernel<float><<<(int)blocks, 256, 0, s>>>((float*)out, (const float*)x, pieces, kind);
    done = pieces * ve;
    if (done == n) return he_check_launch("he_unary_act");
  }
  const int64_t rest = n - done;
  int64_t blocks = (rest + 255) / 256;
  if (blocks > 65535) blocks = 65535;
  const int esz = dtype == HE_BF16 ? 2 : 4;
  void* o = (char*)out + done * esz;
  const void* xi = (const char*)x + done * esz;
  if (dtype == HE_BF16) unary_act_kernel<bf16_t><<<(int)blocks, 256, 0, s>>>((bf16_t*)o, (const bf16_t*)xi, rest, kind);
  else unary_act_kernel<float><<<(int)blocks, 256, 0, s>>>((float*)o, (const float*)xi, rest, kind);
  return he_check_launch("he_unary_act");
}

// out[r, j] = act(x[r, j]) * table[ids[r], offset + j] for j < W: a gate of the stream's own values on a
// stretch of a token's row of a second embedding table (row length table_width). A bad id gives zeros.
template <typename T, typename TT>
__global__ void token_gate_kernel(T* __restrict__ out, const T* __restrict__ x, const TT* __restrict__ table,
                                  const int32_t* __restrict__ ids, int rows, int W, int table_width, int offset, int V,
                                  int kind) {
  const int64_t i = blockIdx.x * (int64_t)blockDim.x + threadIdx.x;
  if (i >= (int64_t)rows * W) return;
  const int r = (int)(i / W), j = (int)(i % W);
  const int id = ids[r];
  float e = 0.f;
  if (id >= 0 && id < V) e = to_float(table[(int64_t)id * table_width + offset + j]);
  out[i] = from_float<T>(he_unary(to_float(x[i]), kind) * e);
}

extern "C" int he_token_gate(void* out, const void* x, const void* table, const void* ids, int rows, int W,
                             int table_width, int offset, int V, int kind, int dtype, int table_dtype, void* stream) {
  HE_REQUIRE(rows >= 0 && W > 0 && offset >= 0 && offset + W <= table_width && V > 0 && kind >= 0 && kind <= 3,
             "he_token_gate: bad sizes W=%d offset=%d table_width=%d", W, offset, table_width);
  HE_REQUIRE((dtype == HE_BF16 || dtype == HE_F32) && (table_dtype == HE_BF16 || table_dtype == HE_F32),
             "he_token_gate: unknown dtype");
  if (rows == 0) return 0;
  const int64_t n = (int64_t)rows * W;
  const int blocks = (int)((n + 255) / 256);
  hipStream_t s = (hipStream_t)stream;
#define TG_LAUNCH(T, TT)                                                                                          \
  token_gate_kernel<T, TT><<<blocks, 256, 0, s>>>((T*)out, (const T*)x, (const TT*)table, (const int32_t*)ids, rows, W, \
                                                  table_width, offset, V, kind)
  if (dtype == HE_BF16 && table_dtype == HE_BF16) TG_LAUNCH(bf16_t, bf16_t);
  else if (dtype == HE_BF16) TG_LAUNCH(bf16_t, float);
  else if (table_dtype == HE_BF16) TG_LAUNCH(float, bf16_t);
  else TG_LAUNCH(float, float);
#undef TG_LAUNCH
  return he_check_launch("he_token_gate");
}

// x[r, h * hd + d] *= sigmoid(gate[r * gate_stride + h * vd + d]) * scale for d < vd (the values of a head;
// its padding up to hd is left as it is): an output gate, element by element, on concatenated heads.
template <typename T>
__global__ void sigmoid_gate_kernel(T* __restrict__ x, const T* __restrict__ gate, int64_t gate_stride, int rows, int H,
                                    int hd, int vd, float scale) {
  const int64_t i = blockIdx.x * (int64_t)blockDim.x + threadIdx.x;
  const int64_t per = (int64_t)H * vd;
  if (i >= rows * per) return;
  const int64_t r = i / per;
  const int c = (int)(i % per), h = c / vd, d = c % vd;
  const float g = to_float(gate[r * gate_stride + c]);
  const int64_t at = r * H * hd + (int64_t)h * hd + d;
  x[at] = from_float<T>(to_float(x[at]) * scale / (1.f + expf(-g)));
}

extern "C" int he_sigmoid_gate(void* x, const void* gate, int64_t gate_stride, int rows, int H, int hd, int vd,
                               float scale, int dtype, void* stream) {
  HE_REQUIRE(rows >= 0 && H > 0 && vd > 0 && hd >= vd && gate_stride >= (int64_t)H * vd, "he_sigmoid_gate: bad sizes");
  HE_REQUIRE(dtype == HE_BF16 || dtype == HE_F32, "he_sigmoid_gate: unknown dtype %d", dtype);
  if (rows == 0) return 0;
  const int64_t n = (int64_t)rows * H * vd;
  const int blocks = (int)((n + 255) / 256);
  hipStream_t s = (hipStream_t)stream;
  if (dtype == HE_BF16)
    sigmoid_gate_kernel<bf16_t><<<blocks, 256, 0, s>>>((bf16_t*)x, (const bf16_t*)gate, gate_stride, rows, H, hd, vd, scale);
  else
    sigmoid_gate_kernel<float><<<blocks, 256, 0, s>>>((float*)x, (const float*)gate, gate_stride, rows, H, hd, vd, scale);
  return he_check_launch("he_sigmoid_gate");
}

// out[i] = sa * a[i] + sb * b[i], the sum formed in fp32 (two branches that read the same input, each with its weight)
template <typename T>
__global__ void scaled_sum_kernel(T* out, const T* a, const T* b, int64_t n, float sa, float sb) {
  int64_t i = blockIdx.x * (int64_t)blockDim.x + threadIdx.x;
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (; i < n; i += stride) out[i] = from_float<T>(fmaf(sa, to_float(a[i]), sb * to_float(b[i])));
}

extern "C" int he_scaled_sum(void* out, const void* a, const void* b, int64_t n, float sa, float sb, int dtype,
                             void* stream) {
  HE_REQUIRE(n >= 0, "he_scaled_sum: bad size");
  HE_REQUIRE(dtype == HE_BF16 || dtype == HE_F32, "he_scaled_sum: unknown dtype %d", dtype);
  if (n == 0) return 0;
  int64_t blocks = (n + 255) / 256;
  if (blocks > 65535) blocks = 65535;
  hipStream_t s = (hipStream_t)stream;
  if (dtype == HE_BF16)
    scaled_sum_kernel<bf16_t><<<(int)blocks, 256, 0, s>>>((bf16_t*)out, (const bf16_t*)a, (const bf16_t*)b, n, sa, sb);
  else
    scaled_sum_kernel<float><<<(int)blocks, 256, 0, s>>>((float*)out, (const float*)a, (const float*)b, n, sa, sb);
  return he_check_launch("he_scaled_sum");
}
