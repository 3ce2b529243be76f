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
__device__ __forceinline__ float mm_gate_log(float z, float cap, bool forget) {
  if (cap > 0.f) z = cap * tanhf(z / cap);
  if (forget) z = fminf(z, 0.f) - log1pf(expf(-fabsf(z)));
  return z;
}

__global__ void mlstm_gates_kernel(float* __restrict__ out, const float* __restrict__ x, const void* __restrict__ bias,
                                   int b_dtype, int64_t n, int H, float cap) {
  const int64_t i = blockIdx.x * (int64_t)blockDim.x + threadIdx.x;
  if (i >= n) return;
  const int c = (int)(i % (2 * H));
  out[i] = mm_gate_log(x[i] + (bias ? load_param(bias, c, b_dtype) : 0.f), cap, c >= H);
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

#define MM_TB 32      // rows of a sequence staged in LDS at a time (fewer where the keys are wide)
#define MM_MAXV 4     // 16-byte pieces of q and k a thread asks for ahead of a block
#define MM_MAXS 8     // values a thread asks for ahead of a block
#define MM_ROWS 4     // rows of a block walked together

// Rows a block stages: at most MM_TB, q and k of a block within 48 KB of LDS, and, where the block's operands are asked
// for a block ahead, no more than the threads can hold in their registers.
static int mm_block_rows(int dk, int dv, int threads, int pieces_per_row) {
  const int dkp = mm_groups(dk) * MM_NPT, PB = mm_pb(dk, dv);
  int tb = MM_TB;
  if (tb > 6144 / dkp) tb = 6144 / dkp;
  if (pieces_per_row > 0) {
    if (tb > MM_MAXV * threads / pieces_per_row) tb = MM_MAXV * threads / pieces_per_row;
    if (tb > MM_MAXS * threads / PB) tb = MM_MAXS * threads / PB;
    if (tb > threads / 2) tb = threads / 2;
  }
  return tb;       // 0: the threads cannot hold one row (the caller then stages without asking ahead)
}

template <int CTRL>
__device__ __forceinline__ float mm_dpp_add(float v) {
  return v + __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xf, 0xf, true));
}

// The sum of v over the NG neighbouring lanes of a value dim (NG a power of two up to 64), in every one of them:
// pairs, quads, halves of 16 and rows of 16 by lane permutations inside a row, the rest by exchanges across rows.
__device__ __forceinline__ float mm_group_sum(float v, int NG) {
  if (NG >= 2) v = mm_dpp_add<0xB1>(v);      // lanes 1,0,3,2 of a quad
  if (NG >= 4) v = mm_dpp_add<0x4E>(v);      // lanes 2,3,0,1 of a quad
  if (NG >= 8) v = mm_dpp_add<0x141>(v);     // a half row of 8 mirrored
  if (NG >= 16) v = mm_dpp_add<0x140>(v);    // a row of 16 mirrored
  if (NG >= 32) v += __shfl_xor(v, 16);
  if (NG >= 64) v += __shfl_xor(v, 32);
  return v;
}

typedef uint32_t mm_piece __attribute__((ext_vector_type(4)));     // 16 bytes of a row, as they are loaded

template <typename T>
__device__ __forceinline__ void mm_unpack(float* dst, const mm_piece& v) {
  if (sizeof(T) == 2) {
    const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      dst[2 * j] = __uint_as_float(w[j] << 16);
      dst[2 * j + 1] = __uint_as_float(w[j] & 0xffff0000u);
    }
  } else {
    dst[0] = __uint_as_float(v.x); dst[1] = __uint_as_float(v.y); dst[2] = __uint_as_float(v.z); dst[3] = __uint_as_float(v.w);
  }
}

// One workgroup a (tile of value dims, head, sequence). Thread (c, j) holds the MM_NPT key dims j of value
// dim c of S, and its own copy of those dims of n; the NG threads of a value dim are neighbouring lanes.
// (n and m are the same in every tile of a head: the same operations in the same order.)
// The rows of a sequence are walked in order, a block of TB rows at a time from LDS: the block's q (scaled), k,
// the tile's values and the head's gates are put there as 32-bit floats by all threads together, and with AHEAD the
// next block's are asked for before this block is computed and put there after it, so that the walk does not wait
// for memory. The running maximum and the exponentials of a block's rows are formed before its rows are walked (one
// thread a row), and a row's answer is divided after the block, when the rows are written: the walk itself is the
// products and sums of S and n. The sums of a row do not depend on how the rows were cut into steps or blocks.
template <typename T, bool AHEAD>
__global__ void __launch_bounds__(256) mlstm_scan_kernel(float* __restrict__ y, const T* __restrict__ q, const T* __restrict__ k,
                                  const T* __restrict__ v, int64_t in_stride, const float* __restrict__ gates,
                                  uint8_t* __restrict__ state, int64_t state_stride, int64_t state_offset,
                                  const int32_t* __restrict__ cu_seqlens, const int32_t* __restrict__ seq_slot, int H,
                                  int dk, int dv, int NG, int PB, int TB, float q_scale, int raw_gates,
                                  const void* __restrict__ gate_bias, int bias_dtype, float cap) {
  extern __shared__ float mm_lds[];
  constexpr int VE = 16 / sizeof(T);            // elements of a 16-byte piece
  const int seq = blockIdx.z, h = blockIdx.y;
  const int slot = seq_slot[seq];
  const int r0 = cu_seqlens[seq], r1 = cu_seqlens[seq + 1];
  if (slot < 0 || r0 >= r1) return;
  const int t = threadIdx.x, threads = blockDim.x;
  const int c = t / NG, j = t % NG;
  const int col0 = blockIdx.x * PB;
  const int col = col0 + c;
  const bool active = c < PB && col < dv;
  const int colc = active ? col : 0;
  const int cl = c < PB ? c : 0;                 // the thread's column of the tile's values in LDS
  const int dkp = NG * MM_NPT;
  const int d0 = j * MM_NPT;
  float* qs = mm_lds;                            // [TB][dkp], key dims past dk are zero
  float* ks = qs + TB * dkp;                     // [TB][dkp]
  float* vs = ks + TB * dkp;                     // [TB][PB]
  float* gs = vs + TB * PB;                      // [TB][2]: the logarithms of the input and forget gates
  float* ys = gs + 2 * TB;                       // [TB][PB]: S^T q of the block's rows
  float* ps = ys + TB * PB;                      // [TB]: n . q of the block's rows
  float* cs = ps + TB;                           // [TB][3] the rows' two decays and floor, then m after the block
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
  if (dk != dkp) {       // the key dims past dk stay zero from here on
    for (int i = t; i < 2 * TB * dkp; i += threads) mm_lds[i] = 0.f;
    __syncthreads();
  }

  const int vq = dk / VE;                        // AHEAD: 16-byte pieces of a row's q (and of its k)
  const int tile = dv - col0 < PB ? dv - col0 : PB;      // value dims of this tile
  mm_piece rqk[MM_MAXV];
  uint32_t rv[MM_MAXS];        // a value's bits as a 32-bit float's
  float rg = 0.f;

  // AHEAD: which piece of a block's q and k, and which of its values, a thread moves is the same in every block:
  // the row inside the block, where it is read (from the block's first row) and where it lies in LDS, formed once
  int qk_row[MM_MAXV], qk_src[MM_MAXV], qk_dst[MM_MAXV], v_row[MM_MAXS], v_src[MM_MAXS], v_dst[MM_MAXS];
  if (AHEAD) {
#pragma unroll
    for (int n = 0; n < MM_MAXV; ++n) {
      const int id = t + n * threads;
      const int row = id / (2 * vq), w = id % (2 * vq);
      qk_row[n] = row < TB ? row : MM_TB;                         // MM_TB: none
      qk_src[n] = row * (int)in_stride + h * dk + (w % vq) * VE;  // in q, or in k for the pieces behind a row's q
      qk_dst[n] = (w < vq ? 0 : TB * dkp) + row * dkp + (w % vq) * VE;
    }
#pragma unroll
    for (int n = 0; n < MM_MAXS; ++n) {
      const int id = t + n * threads;
      const int row = id / tile, x = id % tile;
      v_row[n] = row < TB ? row : MM_TB;
      v_src[n] = row * (int)in_stride + h * dv + col0 + x;
      v_dst[n] = row * PB + x;
    }
  }
  // raw_gates: `gates` holds the pre-activations, and their logarithms are formed here as he_mlstm_gates forms them
  auto gate = [&](float x, int which) {
    if (!raw_gates) return x;
    return mm_gate_log(x + (gate_bias ? load_param(gate_bias, which * H + h, bias_dtype) : 0.f), cap, which == 1);
  };
  auto ask = [&](int rb, int nt) {
    const int64_t base = (int64_t)rb * in_stride;
#pragma unroll
    for (int n = 0; n < MM_MAXV; ++n)
      if (qk_row[n] < nt) rqk[n] = *reinterpret_cast<const mm_piece*>((qk_dst[n] < TB * dkp ? q : k) + base + qk_src[n]);
#pragma unroll
    for (int n = 0; n < MM_MAXS; ++n)
      if (v_row[n] < nt)
        rv[n] = sizeof(T) == 2 ? (uint32_t)*reinterpret_cast<const uint16_t*>(v + base + v_src[n]) << 16
                               : *reinterpret_cast<const uint32_t*>(v + base + v_src[n]);
    if (t < 2 * nt) rg = gates[(int64_t)(rb + t / 2) * 2 * H + (t % 2) * H + h];
  };
  // AHEAD: what ask() fetched into LDS
  auto put = [&](int nt) {
#pragma unroll
    for (int n = 0; n < MM_MAXV; ++n) {
      if (qk_row[n] < nt) {
        float e[VE];
        mm_unpack<T>(e, rqk[n]);
        const float sc = qk_dst[n] < TB * dkp ? q_scale : 1.f;
#pragma unroll
        for (int x = 0; x < VE; ++x) mm_lds[qk_dst[n] + x] = e[x] * sc;
      }
    }
#pragma unroll
    for (int n = 0; n < MM_MAXS; ++n)
      if (v_row[n] < nt) vs[v_dst[n]] = __uint_as_float(rv[n]);
    if (t < 2 * nt) gs[t] = gate(rg, t % 2);
  };
  // without AHEAD: the same, element by element and straight into LDS
  auto stage = [&](int rb, int nt) {
    for (int id = t; id < nt * 2 * dk; id += threads) {
      const int row = id / (2 * dk), w = id % (2 * dk);
      const int64_t at = (int64_t)(rb + row) * in_stride + (int64_t)h * dk;
      if (w < dk) qs[row * dkp + w] = to_float(q[at + w]) * q_scale;
      else ks[row * dkp + w - dk] = to_float(k[at + w - dk]);
    }
    for (int id = t; id < nt * tile; id += threads)
      vs[(id / tile) * PB + id % tile] = to_float(v[(int64_t)(rb + id / tile) * in_stride + (int64_t)h * dv + col0 + id % tile]);
    for (int id = t; id < 2 * nt; id += threads) gs[id] = gate(gates[(int64_t)(rb + id / 2) * 2 * H + (id % 2) * H + h], id % 2);
  };

  {
    const int nt = r1 - r0 < TB ? r1 - r0 : TB;
    if (AHEAD) { ask(r0, nt); put(nt); } else stage(r0, nt);
  }
  __syncthreads();
  for (int rb = r0; rb < r1; rb += TB) {
    const int nt = r1 - rb < TB ? r1 - rb : TB;
    const int next = r1 - rb - TB < TB ? r1 - rb - TB : TB;      // rows of the block after this one (<= 0: none)
    // The block's decays: thread `row` walks the maxima from the block's first row to its own (additions and
    // maxima only), then forms its row's three exponentials; the row loop below has none left.
    if (t < 64) {
      // (every lane of the first wave walks all rows, with their gates loaded beforehand, and keeps its own row's pair)
      float mr = m, before = m, mine = m;
#pragma unroll
      for (int row = 0; row < MM_TB; ++row) {
        const int r = row < nt ? row : nt - 1;
        const float up = fmaxf(gs[2 * r + 1] + mr, gs[2 * r]);
        before = row == t ? mr : before;
        mr = row < nt ? up : mr;
        mine = row == t ? mr : mine;
      }
      if (t < nt) {
        cs[3 * t] = expf(gs[2 * t + 1] + before - mine);      // on S and n as they were
        cs[3 * t + 1] = expf(gs[2 * t] - mine);               // on the row's k v^T and k
        cs[3 * t + 2] = expf(-mine);                          // the floor of the denominator
      }
      if (t == 0) cs[3 * TB] = mr;
    }
    __syncthreads();
    m = cs[3 * TB];
    if (AHEAD && next > 0) ask(rb + TB, next);
    // Four rows at a time: their loads come first, S and n go through the four rows in order (the only chain from
    // row to row is one multiply-add per element), and the eight sums over the lanes of a value dim are formed
    // side by side, so that no step waits for the one before it.
    for (int row = 0; row < nt; row += MM_ROWS) {
      float py[MM_ROWS], pn[MM_ROWS], qc[MM_ROWS][MM_NPT], kc[MM_ROWS][MM_NPT], vc[MM_ROWS], a[MM_ROWS], b[MM_ROWS];
#pragma unroll
      for (int u = 0; u < MM_ROWS; ++u) {
        const int r = row + u < nt ? row + u : nt - 1;          // rows past the block's end repeat its last row and are dropped
        const float4 q0 = *reinterpret_cast<const float4*>(qs + r * dkp + d0), q1 = *reinterpret_cast<const float4*>(qs + r * dkp + d0 + 4);
        const float4 k0 = *reinterpret_cast<const float4*>(ks + r * dkp + d0), k1 = *reinterpret_cast<const float4*>(ks + r * dkp + d0 + 4);
        qc[u][0] = q0.x; qc[u][1] = q0.y; qc[u][2] = q0.z; qc[u][3] = q0.w; qc[u][4] = q1.x; qc[u][5] = q1.y; qc[u][6] = q1.z; qc[u][7] = q1.w;
        kc[u][0] = k0.x; kc[u][1] = k0.y; kc[u][2] = k0.z; kc[u][3] = k0.w; kc[u][4] = k1.x; kc[u][5] = k1.y; kc[u][6] = k1.z; kc[u][7] = k1.w;
        vc[u] = vs[r * PB + cl];
        a[u] = cs[3 * r];
        b[u] = cs[3 * r + 1];
      }
#pragma unroll
      for (int u = 0; u < MM_ROWS; ++u) {
        if (row + u < nt) {
          float y0 = 0.f, y1 = 0.f, n0 = 0.f, n1 = 0.f;
#pragma unroll
          for (int e = 0; e < MM_NPT; e += 2) {
            const float bk0 = b[u] * kc[u][e], bk1 = b[u] * kc[u][e + 1];
            S[e] = fmaf(a[u], S[e], bk0 * vc[u]);
            S[e + 1] = fmaf(a[u], S[e + 1], bk1 * vc[u]);
            nn[e] = fmaf(a[u], nn[e], bk0);
            nn[e + 1] = fmaf(a[u], nn[e + 1], bk1);
            y0 = fmaf(S[e], qc[u][e], y0);
            y1 = fmaf(S[e + 1], qc[u][e + 1], y1);
            n0 = fmaf(nn[e], qc[u][e], n0);
            n1 = fmaf(nn[e + 1], qc[u][e + 1], n1);
          }
          py[u] = y0 + y1;
          pn[u] = n0 + n1;
        } else {
          py[u] = pn[u] = 0.f;
        }
      }
#pragma unroll
      for (int u = 0; u < MM_ROWS; ++u) {
        py[u] = mm_group_sum(py[u], NG);
        pn[u] = mm_group_sum(pn[u], NG);
      }
#pragma unroll
      for (int u = 0; u < MM_ROWS; ++u) {
        if (row + u < nt) {
          if (j == 0 && c < PB) ys[(row + u) * PB + c] = py[u];
          if (t == 0) ps[row + u] = pn[u];
        }
      }
    }
    __syncthreads();
    if (AHEAD) {
#pragma unroll
      for (int n = 0; n < MM_MAXS; ++n) {
        const int row = v_row[n];
        if (row < nt)
          y[(int64_t)(rb + row) * H * dv + (int64_t)h * dv + col0 + v_dst[n] - row * PB] =
              ys[v_dst[n]] / (fmaxf(fabsf(ps[row]), cs[3 * row + 2]) + 1e-6f);
      }
    } else {
      for (int id = t; id < nt * tile; id += threads) {
        const int row = id / tile;
        y[(int64_t)(rb + row) * H * dv + (int64_t)h * dv + col0 + id % tile] =
            ys[row * PB + id % tile] / (fmaxf(fabsf(ps[row]), cs[3 * row + 2]) + 1e-6f);
      }
    }
    if (next > 0) {
      if (AHEAD) put(next); else stage(rb + TB, next);
    }
    __syncthreads();
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

template <typename T>
__device__ __forceinline__ void mm_load8(float* dst, const T* p, int have, bool vec) {
  if (vec && sizeof(T) == 2) {
    mm_unpack<T>(dst, *reinterpret_cast<const mm_piece*>(p));
  } else if (vec) {
    mm_unpack<T>(dst, *reinterpret_cast<const mm_piece*>(p));
    mm_unpack<T>(dst + 4, *reinterpret_cast<const mm_piece*>((const float*)p + 4));
  } else {
#pragma unroll
    for (int e = 0; e < MM_NPT; ++e) dst[e] = e < have ? to_float(p[e]) : 0.f;
  }
}

// Steps that bring every sequence one row: the same workgroups and threads, without the staging. A thread reads its
// own key dims of q and k, its value and the head's gates straight from memory and forms the row's exponentials
// itself; every product and sum is the one the kernel above forms, in the same order, so a row's result has the
// same bits whichever of the two ran it.
template <typename T>
__global__ void __launch_bounds__(256) mlstm_step_kernel(float* __restrict__ y, const T* __restrict__ q, const T* __restrict__ k,
                                                         const T* __restrict__ v, int64_t in_stride,
                                                         const float* __restrict__ gates, uint8_t* __restrict__ state,
                                                         int64_t state_stride, int64_t state_offset,
                                                         const int32_t* __restrict__ cu_seqlens,
                                                         const int32_t* __restrict__ seq_slot, int H, int dk, int dv, int NG,
                                                         int PB, float q_scale, int vec, int raw_gates,
                                                         const void* __restrict__ gate_bias, int bias_dtype, float cap) {
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
  const int dlo = have > 0 ? d0 : 0;     // a thread without key dims reads the row's first ones and drops them
  float* st = reinterpret_cast<float*>(state + (int64_t)slot * state_stride + state_offset);
  float* sp = st + ((int64_t)h * dv + colc) * dkp + d0;
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
  for (int r = r0; r < r1; ++r) {
    float qc[MM_NPT], kc[MM_NPT];
    const int64_t at = (int64_t)r * in_stride;
    mm_load8(qc, q + at + (int64_t)h * dk + dlo, have, full);
    mm_load8(kc, k + at + (int64_t)h * dk + dlo, have, full);
#pragma unroll
    for (int e = 0; e < MM_NPT; ++e) {
      qc[e] = have > 0 ? qc[e] * q_scale : 0.f;
      kc[e] = have > 0 ? kc[e] : 0.f;
    }
    const float vc = to_float(v[at + (int64_t)h * dv + colc]);
    float ig = gates[(int64_t)r * 2 * H + h], fg = gates[(int64_t)r * 2 * H + H + h];
    if (raw_gates) {
      ig = mm_gate_log(ig + (gate_bias ? load_param(gate_bias, h, bias_dtype) : 0.f), cap, false);
      fg = mm_gate_log(fg + (gate_bias ? load_param(gate_bias, H + h, bias_dtype) : 0.f), cap, true);
    }
    const float mn = fmaxf(fg + m, ig);
    const float a = expf(fg + m - mn), b = expf(ig - mn);
    m = mn;
    float y0 = 0.f, y1 = 0.f, n0 = 0.f, n1 = 0.f;
#pragma unroll
    for (int e = 0; e < MM_NPT; e += 2) {
      const float bk0 = b * kc[e], bk1 = b * kc[e + 1];
      S[e] = fmaf(a, S[e], bk0 * vc);
      S[e + 1] = fmaf(a, S[e + 1], bk1 * vc);
      nn[e] = fmaf(a, nn[e], bk0);
      nn[e + 1] = fmaf(a, nn[e + 1], bk1);
      y0 = fmaf(S[e], qc[e], y0);
      y1 = fmaf(S[e + 1], qc[e + 1], y1);
      n0 = fmaf(nn[e], qc[e], n0);
      n1 = fmaf(nn[e + 1], qc[e + 1], n1);
    }
    const float py = mm_group_sum(y0 + y1, NG), pn = mm_group_sum(n0 + n1, NG);
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
                             float q_scale, int dtype, int raw_gates, const void* gate_bias, int bias_dtype, float cap,
                             void* stream) {
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
  // whole 16-byte pieces of a row's q and k: every row and head starts aligned
  const int ve = 16 / esz;
  const bool vec = dk % ve == 0 && in_stride < (1 << 24) && (in_stride * esz) % 16 == 0 && (((uintptr_t)q | (uintptr_t)k) & 15) == 0;
  const dim3 grid((dv + PB - 1) / PB, H, num_seqs);
  hipStream_t s = (hipStream_t)stream;
  if (rows <= num_seqs) {       // no sequence brings more than a row, or the few that do are walked row by row
#define MM_STEP(T)                                                                                                       \
  mlstm_step_kernel<T><<<grid, threads, 0, s>>>((float*)y_f32, (const T*)q, (const T*)k, (const T*)v, in_stride,          \
                                                (const float*)gates_f32, (uint8_t*)state, state_stride, state_offset,    \
                                                (const int32_t*)cu_seqlens, (const int32_t*)seq_slot, H, dk, dv, NG, PB,  \
                                                q_scale, (int)vec, raw_gates, gate_bias, bias_dtype, cap)
    if (dtype == HE_BF16) MM_STEP(bf16_t); else MM_STEP(float);
#undef MM_STEP
    return he_check_launch("he_mlstm_scan");
  }
  int TB = vec ? mm_block_rows(dk, dv, threads, 2 * dk / ve) : 0;
  const bool ahead = TB > 0;
  if (!ahead) TB = mm_block_rows(dk, dv, threads, 0);
  if (rows < TB) TB = rows;        // a step of few rows stages no more than it has
  const size_t lds = sizeof(float) * ((size_t)2 * TB * NG * MM_NPT + (size_t)2 * TB * PB + 6 * TB + 4);
  HE_REQUIRE(TB >= 1 && lds <= 64 * 1024, "he_mlstm_scan: a block of %d rows needs %zu bytes of LDS", TB, lds);
#define MM_LAUNCH(T, AHEAD)                                                                                              \
  mlstm_scan_kernel<T, AHEAD><<<grid, threads, lds, s>>>((float*)y_f32, (const T*)q, (const T*)k, (const T*)v, in_stride, \
                                                         (const float*)gates_f32, (uint8_t*)state, state_stride,         \
                                                         state_offset, (const int32_t*)cu_seqlens,                       \
                                                         (const int32_t*)seq_slot, H, dk, dv, NG, PB, TB, q_scale, \
                                                         raw_gates, gate_bias, bias_dtype, cap)
  if (dtype == HE_BF16) {
    if (ahead) MM_LAUNCH(bf16_t, true); else MM_LAUNCH(bf16_t, false);
  } else {
    if (ahead) MM_LAUNCH(float, true); else MM_LAUNCH(float, false);
  }
#undef MM_LAUNCH
  return he_check_launch("he_mlstm_scan");
}
