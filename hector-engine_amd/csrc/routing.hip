// A token's choice among experts, the experts' gated activation weighted by that choice, and the
// combination of the two score maps of a differential attention head.
#include "common.h"
#include "hector_kernels.h"

#define ROUTE_MAX_EXPERTS 1024

// (value, index) maximum over the wavefront; among equal values the lowest index wins
__device__ __forceinline__ void wave_argmax(float& v, int& i) {
  for (int m = 32; m >= 1; m >>= 1) {
    const float ov = __shfl_xor(v, m);
    const int oi = __shfl_xor(i, m);
    if (ov > v || (ov == v && oi < i)) {
      v = ov;
      i = oi;
    }
  }
}

// One wavefront a row. logits [rows][E] fp32, or, with x and router given, the router's product itself:
// logits[e] = sum_i x[row][i] * router[e][i] in fp32 (router fp32 [E][D]; a lane adds its elements i = lane,
// lane + 64, ... in that order, the lanes' sums meet in the wavefront's butterfly: one fixed order a row,
// whatever else the step holds). s = softmax(logits) over all E outputs; the choice is made
// on c = s + correction: the E outputs are cut into `groups` equal runs of neighbours, each run ranked by the
// largest c it holds; outside the `keep` best runs every c is replaced by -inf, and the `top` largest c that
// are left are chosen. The weight of a chosen output is s * scale (s, not c; the weights are not made to sum
// to one). The last E - real outputs are experts without weights whose result is the input
// itself: their weights are added up in column `real` of dense. dense [rows][real + 1] holds the
// weight of every expert (0 where not chosen); ids / weights [rows][top] list the chosen ones.
#define ROUTE_WAVES 8
__global__ __launch_bounds__(64 * ROUTE_WAVES) void route_kernel(
    float* __restrict__ dense, int32_t* __restrict__ ids, float* __restrict__ weights, const float* __restrict__ logits,
    const void* __restrict__ x, int x_dtype, const float* __restrict__ router, int D,
    const void* __restrict__ correction, int c_dtype, int E, int real, int groups, int keep, int top, float scale,
    int normalize) {
  __shared__ float s_sh[ROUTE_MAX_EXPERTS];
  __shared__ float c_sh[ROUTE_MAX_EXPERTS];
  __shared__ float d_sh[ROUTE_MAX_EXPERTS + 1];
  __shared__ float g_sh[ROUTE_MAX_EXPERTS];
  __shared__ float z[ROUTE_MAX_EXPERTS];
  const int64_t row = blockIdx.x;
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  // The first wavefront makes the choice; with x given, all of them form the logits first, each the outputs
  // e = wave, wave + 8, ...: four elements a lane and turn, four sums a lane that meet in index order.
  const bool lead = wave == 0;
  if (x != nullptr) {
    const bool vec = (D & 3) == 0 && ((uintptr_t)x & 15) == 0 && ((uintptr_t)router & 15) == 0;
    for (int e = wave; e < E; e += ROUTE_WAVES) {
      const float* w = router + (int64_t)e * D;
      float a0 = 0.f, a1 = 0.f, a2 = 0.f, a3 = 0.f;
      if (vec && x_dtype == HE_BF16) {
        const uint2* xr = reinterpret_cast<const uint2*>((const uint16_t*)x + row * D);
#pragma unroll 4
        for (int i = lane; i < (D >> 2); i += 64) {
          const uint2 xv = xr[i];
          const float4 wv = reinterpret_cast<const float4*>(w)[i];
          a0 = fmaf(__uint_as_float(xv.x << 16), wv.x, a0);
          a1 = fmaf(__uint_as_float(xv.x & 0xffff0000u), wv.y, a1);
          a2 = fmaf(__uint_as_float(xv.y << 16), wv.z, a2);
          a3 = fmaf(__uint_as_float(xv.y & 0xffff0000u), wv.w, a3);
        }
      } else if (vec) {
        const float4* xr = reinterpret_cast<const float4*>((const float*)x + row * D);
#pragma unroll 4
        for (int i = lane; i < (D >> 2); i += 64) {
          const float4 xv = xr[i];
          const float4 wv = reinterpret_cast<const float4*>(w)[i];
          a0 = fmaf(xv.x, wv.x, a0);
          a1 = fmaf(xv.y, wv.y, a1);
          a2 = fmaf(xv.z, wv.z, a2);
          a3 = fmaf(xv.w, wv.w, a3);
        }
      } else {
        for (int i = lane; i < D; i += 64) {
          const float xv = x_dtype == HE_BF16 ? bf16_bits_to_float(((const uint16_t*)x)[row * D + i])
                                              : ((const float*)x)[row * D + i];
          a0 = fmaf(xv, w[i], a0);
        }
      }
      const float acc = wave_sum((a0 + a1) + (a2 + a3));
      if (lane == 0) z[e] = acc;
    }
  } else if (lead) {
    for (int e = lane; e < E; e += 64) z[e] = logits[row * E + e];
  }
  __syncthreads();
  // from here on the first wavefront works; the others only keep the barriers' count
  if (lead) {
    float mx = -INFINITY;
    for (int e = lane; e < E; e += 64) mx = fmaxf(mx, z[e]);
    mx = wave_max(mx);
    float sum = 0.f;
    for (int e = lane; e < E; e += 64) {
      const float v = expf(z[e] - mx);
      s_sh[e] = v;
      sum += v;
    }
    sum = wave_sum(sum);
    const float inv = 1.f / sum;
    for (int e = lane; e < E; e += 64) {
      const float s = s_sh[e] * inv;
      s_sh[e] = s;
      c_sh[e] = s + (correction ? load_param(correction, e, c_dtype) : 0.f);
    }
    for (int e = lane; e <= real; e += 64) d_sh[e] = 0.f;
  }
  __syncthreads();
  const int size = E / groups;
  if (keep < groups) {
    if (lead) {
      for (int g = lane; g < groups; g += 64) {
        float best = -INFINITY;
        for (int i = 0; i < size; ++i) best = fmaxf(best, c_sh[g * size + i]);
        g_sh[g] = best;
      }
    }
    __syncthreads();
    // the `keep` best groups are marked by +inf in g_sh, then the others' outputs are masked
    for (int k = 0; k < keep; ++k) {
      float v = -INFINITY;
      int idx = 0x7fffffff;
      if (lead) {
        for (int g = lane; g < groups; g += 64) {
          const float gv = g_sh[g];
          if (gv != INFINITY && (gv > v || (gv == v && g < idx))) {
            v = gv;
            idx = g;
          }
        }
        wave_argmax(v, idx);
      }
      __syncthreads();
      if (lead && lane == 0 && idx < groups) g_sh[idx] = INFINITY;
      __syncthreads();
    }
    if (lead) {
      for (int e = lane; e < E; e += 64)
        if (g_sh[e / size] != INFINITY) c_sh[e] = -INFINITY;
    }
    __syncthreads();
  }
  float chosen_sum = 0.f;     // lane 0 of the first wavefront: the chosen outputs' scores, added in the order of the choice
  for (int k = 0; k < top; ++k) {
    float v = -INFINITY;
    int idx = 0x7fffffff;
    if (lead) {
      for (int e = lane; e < E; e += 64) {
        const float cv = c_sh[e];
        // a chosen output is marked by NaN, which no comparison takes
        if (cv > v || (cv == v && e < idx)) {
          v = cv;
          idx = e;
        }
      }
      wave_argmax(v, idx);
    }
    __syncthreads();
    if (lead && lane == 0) {
      const bool found = idx < E;
      const int e = found ? idx : 0;
      const float w = found ? s_sh[e] * scale : 0.f;
      if (found) {
        c_sh[e] = NAN;
        d_sh[e < real ? e : real] += w;
        chosen_sum += s_sh[e];
      }
      ids[row * top + k] = found ? e : -1;
      weights[row * top + k] = w;
    }
    __syncthreads();
  }
  if (lead) {
    // normalize: the chosen outputs' weights are made to sum to `scale` (the softmax over the chosen logits alone)
    const float norm = normalize ? 1.f / __shfl(chosen_sum, 0) : 1.f;
    for (int e = lane; e <= real; e += 64) dense[row * (real + 1) + e] = normalize ? d_sh[e] * norm : d_sh[e];
    if (normalize)
      for (int k = lane; k < top; k += 64) weights[row * top + k] *= norm;
  }
}

extern "C" int he_route_tokens(void* dense_f32, void* ids_i32, void* weights_f32, const void* logits_f32,
                               const void* x, int x_dtype, const void* router_f32, int D,
                               const void* correction, int c_dtype, int rows, int E, int real, int groups, int keep,
                               int top, float scale, int normalize, void* stream) {
  HE_REQUIRE((logits_f32 != nullptr) != (x != nullptr), "he_route_tokens: give the logits, or the rows and the router");
  HE_REQUIRE(x == nullptr || (router_f32 != nullptr && D > 0 && (x_dtype == HE_BF16 || x_dtype == HE_F32)),
             "he_route_tokens: the router's matrix is missing");
  HE_REQUIRE(rows >= 0 && E > 0 && E <= ROUTE_MAX_EXPERTS && real >= 0 && real <= E,
             "he_route_tokens: bad sizes E=%d real=%d (at most %d outputs)", E, real, ROUTE_MAX_EXPERTS);
  HE_REQUIRE(groups > 0 && E % groups == 0 && keep > 0 && keep <= groups,
             "he_route_tokens: %d outputs do not form %d equal groups of which %d are kept", E, groups, keep);
  HE_REQUIRE(top > 0 && top <= keep * (E / groups), "he_route_tokens: %d chosen of %d kept outputs", top,
             keep * (E / groups));
  if (rows == 0) return 0;
  route_kernel<<<rows, 64 * ROUTE_WAVES, 0, (hipStream_t)stream>>>((float*)dense_f32, (int32_t*)ids_i32, (float*)weights_f32,
                                                     (const float*)logits_f32, x, x_dtype, (const float*)router_f32, D,
                                                     correction, c_dtype, E, real, groups, keep, top, scale, normalize);
  return he_check_launch("he_route_tokens");
}

// out [rows][real * I + extra]: column e * I + i = act(gate, up) * dense[row][e] with gate and up the
// columns 2 (e I + i) and 2 (e I + i) + 1 of gate_up (a fused weight whose rows alternate gate and up),
// act as he_gated_act; the last `extra` columns = dense[row][real] * h[row][:] (the share of the
// experts whose result is their input). A product over these columns with the experts' down
// matrices side by side (and an identity block for the extra columns) is the weighted sum of the
// chosen experts' results.
template <typename T, bool CLAMPED>
__global__ void routed_act_kernel(T* __restrict__ out, const T* __restrict__ gate_up, const float* __restrict__ dense,
                                  const T* __restrict__ h, int real, int I, int extra, GatedAct act) {
  const int64_t row = blockIdx.y;
  const int cols = real * I + extra;
  const int j = blockIdx.x * blockDim.x + threadIdx.x;
  if (j >= cols) return;
  const float* d = dense + row * (real + 1);
  float v;
  if (j < real * I) {
    const float w = d[j / I];
    const T* gu = gate_up + row * (int64_t)(2 * real * I) + 2 * j;
    // an expert that was not chosen gives exact zeros, whatever its rows hold
    v = w == 0.f ? 0.f : he_gated_act<CLAMPED>(to_float(gu[0]), to_float(gu[1]), act) * w;
  } else {
    const float w = d[real];
    v = w == 0.f ? 0.f : w * to_float(h[row * (int64_t)extra + (j - real * I)]);
  }
  out[row * (int64_t)cols + j] = from_float<T>(v);
}

// The same for bf16 rows, eight columns a thread (16-byte loads and stores): needs I and extra in multiples of 8.
template <bool CLAMPED>
__global__ void routed_act_vec_kernel(uint16_t* __restrict__ out, const uint16_t* __restrict__ gate_up,
                                      const float* __restrict__ dense, const uint16_t* __restrict__ h, int real, int I,
                                      int extra, GatedAct act) {
  const int64_t row = blockIdx.y;
  const int cols = real * I + extra;
  const int j = 8 * (blockIdx.x * blockDim.x + threadIdx.x);
  if (j >= cols) return;
  const float* d = dense + row * (real + 1);
  float v[8];
  if (j < real * I) {
    const float w = d[j / I];
    const uint4* gu = reinterpret_cast<const uint4*>(gate_up + row * (int64_t)(2 * real * I) + 2 * j);
    const uint4 lo = gu[0], hi = gu[1];
    const uint32_t pairs[8] = {lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};      // (gate, up) a word
#pragma unroll
    for (int i = 0; i < 8; ++i)
      v[i] = w == 0.f ? 0.f
                      : he_gated_act<CLAMPED>(__uint_as_float(pairs[i] << 16), __uint_as_float(pairs[i] & 0xffff0000u), act) * w;
  } else {
    const float w = d[real];
    const uint4 raw = *reinterpret_cast<const uint4*>(h + row * (int64_t)extra + (j - real * I));
    const uint32_t words[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      v[2 * i] = w == 0.f ? 0.f : w * __uint_as_float(words[i] << 16);
      v[2 * i + 1] = w == 0.f ? 0.f : w * __uint_as_float(words[i] & 0xffff0000u);
    }
  }
  *reinterpret_cast<uint4*>(out + row * (int64_t)cols + j) =
      make_uint4(pack2_bf16(v[0], v[1]), pack2_bf16(v[2], v[3]), pack2_bf16(v[4], v[5]), pack2_bf16(v[6], v[7]));
}

extern "C" int he_routed_act(void* out, const void* gate_up, const void* dense_f32, const void* h, int rows, int real,
                             int I, int extra, int dtype, float alpha, float limit, float up_shift, void* stream) {
  HE_REQUIRE(rows >= 0 && real >= 0 && I > 0 && extra >= 0 && (int64_t)real * I + extra > 0, "he_routed_act: bad sizes");
  HE_REQUIRE(extra == 0 || h != nullptr, "he_routed_act: the input rows are missing");
  HE_REQUIRE(dtype == HE_BF16 || dtype == HE_F32, "he_routed_act: unknown dtype %d", dtype);
  if (rows == 0) return 0;
  const int cols = real * I + extra;
  const dim3 grid((cols + 255) / 256, rows);
  hipStream_t s = (hipStream_t)stream;
  const bool clamped = limit > 0.f || alpha != 1.f || up_shift != 0.f;
  const GatedAct act = {alpha, limit > 0.f ? limit : INFINITY, up_shift};
  if (dtype == HE_BF16 && I % 8 == 0 && extra % 8 == 0 &&
      ((((uintptr_t)out) | ((uintptr_t)gate_up) | ((uintptr_t)h)) & 15) == 0) {
    const dim3 vgrid((cols / 8 + 255) / 256, rows);
    if (clamped)
      routed_act_vec_kernel<true><<<vgrid, 256, 0, s>>>((uint16_t*)out, (const uint16_t*)gate_up, (const float*)dense_f32,
                                                        (const uint16_t*)h, real, I, extra, act);
    else
      routed_act_vec_kernel<false><<<vgrid, 256, 0, s>>>((uint16_t*)out, (const uint16_t*)gate_up, (const float*)dense_f32,
                                                         (const uint16_t*)h, real, I, extra, act);
    return he_check_launch("he_routed_act");
  }
#define ACT_LAUNCH(T, CL)                                                                                      \
  routed_act_kernel<T, CL><<<grid, 256, 0, s>>>((T*)out, (const T*)gate_up, (const float*)dense_f32, (const T*)h, real, \
                                                I, extra, act)
  if (dtype == HE_BF16) {
    if (clamped) ACT_LAUNCH(bf16_t, true); else ACT_LAUNCH(bf16_t, false);
  } else {
    if (clamped) ACT_LAUNCH(float, true); else ACT_LAUNCH(float, false);
  }
#undef ACT_LAUNCH
  return he_check_launch("he_routed_act");
}

// ---- the chosen experts alone, for steps of very few rows ---------------------------------------
// Where a step's rows choose fewer experts than there are, the two products over all experts read weights
// nobody asked for. These two kernels walk only the chosen experts' rows of the same fused matrices (bf16):
// a wavefront an output, the lanes along K with 16-byte loads, sums in fp32.
__device__ __forceinline__ float dot8_bf16(const uint4& a, const uint4& b, float acc) {
  const uint32_t x[4] = {a.x, a.y, a.z, a.w}, y[4] = {b.x, b.y, b.z, b.w};
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    acc = fmaf(__uint_as_float(x[i] << 16), __uint_as_float(y[i] << 16), acc);
    acc = fmaf(__uint_as_float(x[i] & 0xffff0000u), __uint_as_float(y[i] & 0xffff0000u), acc);
  }
  return acc;
}

// h[(row, k), i] = weight[row, k] * act(gate . x[row], up . x[row]) with gate and up the rows 2 (e I + i) and
// 2 (e I + i) + 1 of gate_up [2 real I][D], e = ids[row, k]; zeros where e is no expert with weights.
template <bool CLAMPED>
__global__ __launch_bounds__(256) void chosen_gate_up_kernel(uint16_t* __restrict__ h, const uint16_t* __restrict__ x,
                                                             const uint16_t* __restrict__ gate_up,
                                                             const int32_t* __restrict__ ids,
                                                             const float* __restrict__ weights, int top, int real, int I,
                                                             int D, GatedAct act) {
  const int lane = threadIdx.x & 63;
  const int i = blockIdx.x * 4 + (threadIdx.x >> 6);
  const int64_t rk = blockIdx.y;                 // row * top + k
  if (i >= I) return;
  const int e = ids[rk];
  const int64_t row = rk / top;
  float g = 0.f, u = 0.f;
  if (e >= 0 && e < real) {
    const uint16_t* wg = gate_up + ((int64_t)e * I + i) * 2 * D;
    const uint16_t* xr = x + row * D;
#pragma unroll 4
    for (int c = lane * 8; c < D; c += 512) {
      const uint4 xv = *reinterpret_cast<const uint4*>(xr + c);
      g = dot8_bf16(*reinterpret_cast<const uint4*>(wg + c), xv, g);
      u = dot8_bf16(*reinterpret_cast<const uint4*>(wg + D + c), xv, u);
    }
  }
  g = wave_sum(g);
  u = wave_sum(u);
  if (lane == 0) {
    const float v = (e >= 0 && e < real) ? he_gated_act<CLAMPED>(g, u, act) * weights[rk] : 0.f;
    h[rk * I + i] = float_to_bf16_bits(v);
  }
}

// out[row, d] = sum over the row's chosen experts e of down[d][e I ..] . h[(row, k)] + dense[row][real] * x[row, d]
// (down [D][ldw]: the experts' matrices side by side; the last term is the identity experts' share).
__global__ __launch_bounds__(256) void chosen_down_kernel(uint16_t* __restrict__ out, const uint16_t* __restrict__ h,
                                                          const uint16_t* __restrict__ x, const uint16_t* __restrict__ down,
                                                          int64_t ldw, const int32_t* __restrict__ ids,
                                                          const float* __restrict__ dense, int top, int real, int I,
                                                          int D) {
  const int lane = threadIdx.x & 63;
  const int d = blockIdx.x * 4 + (threadIdx.x >> 6);
  const int64_t row = blockIdx.y;
  if (d >= D) return;
  float acc = 0.f;
  for (int k = 0; k < top; ++k) {
    const int e = ids[row * top + k];
    if (e < 0 || e >= real) continue;
    const uint16_t* w = down + (int64_t)d * ldw + (int64_t)e * I;
    const uint16_t* hr = h + (row * top + k) * I;
#pragma unroll 4
    for (int c = lane * 8; c < I; c += 512)
      acc = dot8_bf16(*reinterpret_cast<const uint4*>(w + c), *reinterpret_cast<const uint4*>(hr + c), acc);
  }
  acc = wave_sum(acc);
  if (lane == 0)
    out[row * D + d] = float_to_bf16_bits(fmaf(dense[row * (real + 1) + real], bf16_bits_to_float(x[row * D + d]), acc));
}

extern "C" int he_chosen_experts(void* out, void* h_scratch, const void* x, const void* gate_up, const void* down,
                                 int64_t ldw, const void* ids_i32, const void* weights_f32, const void* dense_f32,
                                 int rows, int top, int real, int I, int D, float alpha, float limit, float up_shift,
                                 void* stream) {
  HE_REQUIRE(rows >= 0 && top > 0 && real > 0 && I > 0 && D > 0, "he_chosen_experts: bad sizes");
  HE_REQUIRE(I % 8 == 0 && D % 8 == 0 && ldw % 8 == 0 && ldw >= (int64_t)real * I,
             "he_chosen_experts: I=%d, D=%d and the down matrix's row stride must be multiples of 8", I, D);
  HE_REQUIRE(((((uintptr_t)out) | ((uintptr_t)h_scratch) | ((uintptr_t)x) | ((uintptr_t)gate_up) | ((uintptr_t)down)) & 15) == 0,
             "he_chosen_experts: pointers must be 16-byte aligned");
  HE_REQUIRE((int64_t)rows * top <= 65535, "he_chosen_experts: too many rows");
  if (rows == 0) return 0;
  hipStream_t s = (hipStream_t)stream;
  const bool clamped = limit > 0.f || alpha != 1.f || up_shift != 0.f;
  const GatedAct act = {alpha, limit > 0.f ? limit : INFINITY, up_shift};
  const dim3 grid_up((I + 3) / 4, rows * top);
  if (clamped)
    chosen_gate_up_kernel<true><<<grid_up, 256, 0, s>>>((uint16_t*)h_scratch, (const uint16_t*)x, (const uint16_t*)gate_up,
                                                        (const int32_t*)ids_i32, (const float*)weights_f32, top, real, I,
                                                        D, act);
  else
    chosen_gate_up_kernel<false><<<grid_up, 256, 0, s>>>((uint16_t*)h_scratch, (const uint16_t*)x, (const uint16_t*)gate_up,
                                                         (const int32_t*)ids_i32, (const float*)weights_f32, top, real, I,
                                                         D, act);
  int st = he_check_launch("he_chosen_experts (gate, up)");
  if (st) return st;
  chosen_down_kernel<<<dim3((D + 3) / 4, rows), 256, 0, s>>>((uint16_t*)out, (const uint16_t*)h_scratch, (const uint16_t*)x,
                                                             (const uint16_t*)down, ldw, (const int32_t*)ids_i32,
                                                             (const float*)dense_f32, top, real, I, D);
  return he_check_launch("he_chosen_experts (down)");
}

// Differential attention's last step. attn [rows][2 H][hd] holds, for kv head g and its R = H / G
// query heads, first the R outputs of score map 1 and then the R outputs of map 2 (head order
// [g][map][r]); out [rows][H][vd], head h = g R + r:
//   o = a1 - lambda a2;  out = o / sqrt(mean(o^2) + eps) * post
// over the vd values of a head (no learned gain). One wavefront a (row, head).
template <typename T>
__global__ __launch_bounds__(64) void diff_heads_kernel(T* __restrict__ out, const T* __restrict__ attn, int H, int G,
                                                        int hd, int vd, float lambda, float post, float eps) {
  const int64_t row = blockIdx.y;
  const int h = blockIdx.x;
  const int R = H / G;
  const int g = h / R, r = h - g * R;
  const T* a1 = attn + (row * 2 * H + (int64_t)(2 * g) * R + r) * hd;
  const T* a2 = a1 + (int64_t)R * hd;
  float sq = 0.f;
  for (int i = threadIdx.x; i < vd; i += 64) {
    const float o = fmaf(-lambda, to_float(a2[i]), to_float(a1[i]));
    sq = fmaf(o, o, sq);
  }
  sq = wave_sum(sq);
  const float mul = post / sqrtf(sq / (float)vd + eps);
  T* dst = out + (row * H + h) * vd;
  for (int i = threadIdx.x; i < vd; i += 64) {
    const float o = fmaf(-lambda, to_float(a2[i]), to_float(a1[i]));
    dst[i] = from_float<T>(o * mul);
  }
}

extern "C" int he_diff_heads(void* out, const void* attn, int rows, int H, int G, int hd, int vd, float lambda,
                             float post, float eps, int dtype, void* stream) {
  HE_REQUIRE(rows >= 0 && H > 0 && G > 0 && H % G == 0 && vd > 0 && vd <= hd, "he_diff_heads: bad sizes H=%d G=%d hd=%d vd=%d",
             H, G, hd, vd);
  HE_REQUIRE(dtype == HE_BF16 || dtype == HE_F32, "he_diff_heads: unknown dtype %d", dtype);
  if (rows == 0) return 0;
  const dim3 grid(H, rows);
  hipStream_t s = (hipStream_t)stream;
  if (dtype == HE_BF16)
    diff_heads_kernel<bf16_t><<<grid, 64, 0, s>>>((bf16_t*)out, (const bf16_t*)attn, H, G, hd, vd, lambda, post, eps);
  else
    diff_heads_kernel<float><<<grid, 64, 0, s>>>((float*)out, (const float*)attn, H, G, hd, vd, lambda, post, eps);
  return he_check_launch("he_diff_heads");
}
