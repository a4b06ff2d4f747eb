// Linear attention with one fixed decay per head ("lightning attention") and a carried fp32 state.
//
// Per head, with keys / queries of size D, values of size V and a decay 0 <= lambda <= 1:
//
//   S_t = lambda S_{t-1} + k_t v_t^T   [D, V]          o_t = S_t^T q_t
//
// q, k and v are columns of one projection; an activation (SiLU) is applied to them on the way in, in fp32, so the
// activated operands never pass through 16 bits. State slots [slots, heads, D, V] live in device memory between
// steps: a row whose first token has position 0 starts from S = 0 whatever its slot held before; a row with a
// negative slot is skipped (its outputs are zero).
//
// `lightning_scan_kernel`: token by token, one workgroup of four waves per (row, head, 64 value columns); wave r keeps
// a quarter of the rows of S in registers (lane c: column c).
// `lightning_chunk_kernel`: prompt portions, chunks of 64 tokens on the fp32 matrix cores (MFMA 16x16x4):
//
//   o_t   = lambda^(t+1) S_prev^T q_t + sum_{s <= t} lambda^(t-s) (q_t . k_s) v_s            t, s inside the chunk
//   S_new = lambda^L S_prev + sum_s lambda^(L-1-s) k_s v_s^T                                  L tokens in the chunk
//
// Every power has a non-negative exponent, so nothing overflows and nothing is divided.
// `lightning_out_kernel`: RMS norm over ALL heads' read-outs of a token together, weight, sigmoid gate.
#include "common.hpp"

namespace {

template <typename T> DEVINL float ldf(const T* p, size_t i);
template <> DEVINL float ldf<bf16_t>(const bf16_t* p, size_t i) { return bf2f(p[i]); }
template <> DEVINL float ldf<float>(const float* p, size_t i) { return p[i]; }
template <typename T> DEVINL void stf(T* p, size_t i, float v);
template <> DEVINL void stf<bf16_t>(bf16_t* p, size_t i, float v) { p[i] = f2bf(v); }
template <> DEVINL void stf<float>(float* p, size_t i, float v) { p[i] = v; }

DEVINL float act_in(float x, int act) { return act ? x / (1.f + expf(-x)) : x; }

constexpr int TC = 8;  // tokens staged per step of the loop
constexpr int RW = 4;  // waves of a workgroup

template <typename T, int DP>
__global__ void __launch_bounds__(64 * RW) lightning_scan_kernel(
    const T* __restrict__ proj, int64_t row_stride, int q_off, int k_off, int v_off, const float* __restrict__ decay,
    const int* __restrict__ cu_q, const int* __restrict__ first_pos, const int* __restrict__ state_slots,
    float* __restrict__ S, float* __restrict__ obuf, int NH, int D, int V, int act) {
  constexpr int DQ = DP / RW;
  __shared__ float kq[TC][2][DP];
  __shared__ float hpart[RW][TC][64];
  const int b = blockIdx.x, hd = blockIdx.y, tid = threadIdx.x, lane = tid & 63, r = tid >> 6;
  const int col = blockIdx.z * 64 + lane;
  const bool has = col < V;
  const int slot = state_slots[b];
  const int t_lo = cu_q[b], t_hi = cu_q[b + 1];
  if (slot < 0) {
    if (r == 0)
      for (int t = t_lo; t < t_hi; ++t)
        if (has) obuf[((size_t)t * NH + hd) * V + col] = 0.f;
    return;
  }
  if (t_hi <= t_lo) return;
  const bool fresh = first_pos[b] == 0;
  const float lam = decay[hd];
  const size_t sbase = ((size_t)slot * NH + hd) * D;
  const int d0 = r * DQ;
  float s[DQ];
#pragma unroll
  for (int d = 0; d < DQ; ++d) s[d] = (!fresh && has && d0 + d < D) ? S[(sbase + d0 + d) * V + col] : 0.f;
  for (int tb = t_lo; tb < t_hi; tb += TC) {
    const int nt = min(TC, t_hi - tb);
    __syncthreads();  // the step before is finished with kq and the partials
    for (int i = tid; i < TC * DP; i += 64 * RW) {
      const int d = i % DP, tt = i / DP;
      const bool live = tt < nt && d < D;
      const T* row = proj + (size_t)(tb + min(tt, nt - 1)) * row_stride;
      kq[tt][0][d] = live ? act_in(ldf<T>(row, k_off + hd * D + d), act) : 0.f;
      kq[tt][1][d] = live ? act_in(ldf<T>(row, q_off + hd * D + d), act) : 0.f;
    }
    float vv[TC];
#pragma unroll
    for (int tt = 0; tt < TC; ++tt)
      vv[tt] = (tt < nt && has) ? act_in(ldf<T>(proj + (size_t)(tb + tt) * row_stride, v_off + hd * V + col), act) : 0.f;
    __syncthreads();
#pragma unroll
    for (int tt = 0; tt < TC; ++tt) {
      if (tt < nt) {
        float hacc = 0.f;
#pragma unroll
        for (int d = 0; d < DQ; ++d) {
          s[d] = lam * s[d] + vv[tt] * kq[tt][0][d0 + d];
          hacc += s[d] * kq[tt][1][d0 + d];
        }
        hpart[r][tt][lane] = hacc;
      }
    }
    __syncthreads();
#pragma unroll
    for (int tt = 0; tt < TC; ++tt) {
      if (tt < nt && (tt % RW) == r && has) {
        float hsum = 0.f;
#pragma unroll
        for (int w = 0; w < RW; ++w) hsum += hpart[w][tt][lane];
        obuf[((size_t)(tb + tt) * NH + hd) * V + col] = hsum;
      }
    }
  }
  if (has) {
#pragma unroll
    for (int d = 0; d < DQ; ++d)
      if (d0 + d < D) S[(sbase + d0 + d) * V + col] = s[d];
  }
}

constexpr int CL = 64;
template <typename T, int DP>
__global__ void __launch_bounds__(256) lightning_chunk_kernel(
    const T* __restrict__ proj, int64_t row_stride, int q_off, int k_off, int v_off, const float* __restrict__ decay,
    const int* __restrict__ cu_q, const int* __restrict__ first_pos, const int* __restrict__ state_slots,
    float* __restrict__ S, float* __restrict__ obuf, int NH, int D, int V, int act) {
  constexpr int QS = DP + 4, CS = CL + 4;
  extern __shared__ float cl[];
  float* Sst = cl;                 // [DP][CS] state slice
  float* Qs = Sst + DP * CS;       // [CL][QS]
  float* Ks = Qs + CL * QS;        // [CL][QS]
  float* Vs = Ks + CL * QS;        // [CL][CS] values of this column slice
  float* Ps = Vs + CL * CS;        // [CL][CS] decayed q.k
  float* pw = Ps + CL * CS;        // [CL + 1] powers of the decay
  const int b = blockIdx.x, hd = blockIdx.y, tid = threadIdx.x, lane = tid & 63, w = tid >> 6;
  const int r16 = lane & 15, quad = lane >> 4, col0 = blockIdx.z * 64;
  const int slot = state_slots[b];
  const int t_lo = cu_q[b], t_hi = cu_q[b + 1];
  if (slot < 0) {
    for (int i = tid; i < (t_hi - t_lo) * 64; i += 256) {
      const int t = t_lo + i / 64, c = col0 + i % 64;
      if (c < V) obuf[((size_t)t * NH + hd) * V + c] = 0.f;
    }
    return;
  }
  if (t_hi <= t_lo) return;
  const bool fresh = first_pos[b] == 0;
  const size_t sbase = ((size_t)slot * NH + hd) * D;
  for (int i = tid; i < DP * 64; i += 256) {
    const int d = i / 64, c = i % 64;
    Sst[d * CS + c] = (!fresh && d < D && col0 + c < V) ? S[(sbase + d) * V + col0 + c] : 0.f;
  }
  {
    const float l2 = log2f(decay[hd]);  // lambda = 0: -inf, and every power but the zeroth is 0
    for (int j = tid; j <= CL; j += 256) pw[j] = j == 0 ? 1.f : exp2f((float)j * l2);
  }

  // 16-byte loads of a chunk's operands, fetched into registers one chunk ahead so that their latency runs under the
  // matrix work of the chunk before (rows and offsets that are multiples of a vector, key size = its padded size)
  constexpr int VE = 16 / (int)sizeof(T);                 // elements per vector
  constexpr int NKQ = CL * DP / VE / 256;                 // vectors per thread of K (and of Q)
  constexpr int NVV = CL * 64 / VE / 256;                 // vectors per thread of V
  const bool vec = D == DP && row_stride % VE == 0 && q_off % VE == 0 && k_off % VE == 0 && v_off % VE == 0 &&
                   V % VE == 0 && (reinterpret_cast<uintptr_t>(proj) & 15) == 0;
  u32x4 rk[NKQ], rq[NKQ], rv[NVV];
  auto fetch = [&](int tb) {
    const int nt = min(CL, t_hi - tb);
#pragma unroll
    for (int j = 0; j < NKQ; ++j) {
      const int e = (tid + 256 * j) * VE, d = e % DP, tt = e / DP;
      const T* row = proj + (size_t)(tb + min(tt, nt - 1)) * row_stride;
      rk[j] = *reinterpret_cast<const u32x4*>(row + k_off + hd * D + d);
      rq[j] = *reinterpret_cast<const u32x4*>(row + q_off + hd * D + d);
    }
#pragma unroll
    for (int j = 0; j < NVV; ++j) {
      const int e = (tid + 256 * j) * VE, c = e % 64, tt = e / 64;
      const T* row = proj + (size_t)(tb + min(tt, nt - 1)) * row_stride;
      rv[j] = (col0 + c < V) ? *reinterpret_cast<const u32x4*>(row + v_off + hd * V + col0 + c) : (u32x4){0u, 0u, 0u, 0u};
    }
  };
  auto unpack = [&](u32x4 r, float* dst, bool live) {  // VE activated values (zeros for rows past the chunk's end)
    if (sizeof(T) == 2) {
      const bf16x8 x = __builtin_bit_cast(bf16x8, r);
#pragma unroll
      for (int e = 0; e < 8; ++e) dst[e] = live ? act_in(bf2f(x[e]), act) : 0.f;
    } else {
      const f32x4 x = __builtin_bit_cast(f32x4, r);
#pragma unroll
      for (int e = 0; e < 4; ++e) dst[e] = live ? act_in(x[e], act) : 0.f;
    }
  };
  if (vec) fetch(t_lo);

  for (int tb = t_lo; tb < t_hi; tb += CL) {
    const int nt = min(CL, t_hi - tb);
    __syncthreads();  // the chunk before is done with the staged operands
    if (vec) {
#pragma unroll
      for (int j = 0; j < NKQ; ++j) {
        const int e = (tid + 256 * j) * VE, d = e % DP, tt = e / DP;
        unpack(rk[j], Ks + tt * QS + d, tt < nt);
        unpack(rq[j], Qs + tt * QS + d, tt < nt);
      }
#pragma unroll
      for (int j = 0; j < NVV; ++j) {
        const int e = (tid + 256 * j) * VE, c = e % 64, tt = e / 64;
        unpack(rv[j], Vs + tt * CS + c, tt < nt && col0 + c < V);
      }
      if (tb + CL < t_hi) fetch(tb + CL);
    } else {
#pragma unroll 8
      for (int i = tid; i < CL * DP; i += 256) {
        const int d = i % DP, tt = i / DP;
        const bool live = tt < nt && d < D;
        const T* row = proj + (size_t)(tb + min(tt, nt - 1)) * row_stride;
        Ks[tt * QS + d] = live ? act_in(ldf<T>(row, k_off + hd * D + d), act) : 0.f;
        Qs[tt * QS + d] = live ? act_in(ldf<T>(row, q_off + hd * D + d), act) : 0.f;
      }
#pragma unroll 8
      for (int i = tid; i < CL * 64; i += 256) {
        const int c = i % 64, tt = i / 64;
        Vs[tt * CS + c] = (tt < nt && col0 + c < V)
                              ? act_in(ldf<T>(proj + (size_t)(tb + tt) * row_stride, v_off + hd * V + col0 + c), act) : 0.f;
      }
    }
    __syncthreads();
    // ---- P[t][s] = lambda^(t-s) (q_t . k_s) for s <= t; rows of wave w: t = 16 w + ..
    {
      f32x4 c[4];
#pragma unroll
      for (int cb = 0; cb < 4; ++cb) c[cb] = (f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll 4
      for (int kk = 0; kk < DP / 4; ++kk) {
        const float a = Qs[(16 * w + r16) * QS + 4 * kk + quad];
#pragma unroll
        for (int cb = 0; cb < 4; ++cb)
          if (cb <= w) c[cb] = __builtin_amdgcn_mfma_f32_16x16x4f32(a, Ks[(16 * cb + r16) * QS + 4 * kk + quad], c[cb], 0, 0, 0);
      }
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int t = 16 * w + 4 * quad + i;
#pragma unroll
        for (int cb = 0; cb < 4; ++cb) {
          const int sidx = 16 * cb + r16;
          Ps[t * CS + sidx] = (cb <= w && sidx <= t) ? c[cb][i] * pw[t - sidx] : 0.f;
        }
      }
    }
    __syncthreads();
    // ---- read-out of wave w's tokens: lambda^(t+1) (q_t S_prev) + P V
    {
      f32x4 acc[4];
#pragma unroll
      for (int cb = 0; cb < 4; ++cb) acc[cb] = (f32x4){0.f, 0.f, 0.f, 0.f};
      const float e_row = pw[16 * w + r16 + 1];  // the A operand's row is token 16 w + r16
#pragma unroll 4
      for (int kk = 0; kk < DP / 4; ++kk) {
        const float a = Qs[(16 * w + r16) * QS + 4 * kk + quad] * e_row;
#pragma unroll
        for (int cb = 0; cb < 4; ++cb)
          acc[cb] = __builtin_amdgcn_mfma_f32_16x16x4f32(a, Sst[(4 * kk + quad) * CS + 16 * cb + r16], acc[cb], 0, 0, 0);
      }
      for (int kk = 0; kk < 4 * (w + 1); ++kk) {
        const float a = Ps[(16 * w + r16) * CS + 4 * kk + quad];
#pragma unroll
        for (int cb = 0; cb < 4; ++cb)
          acc[cb] = __builtin_amdgcn_mfma_f32_16x16x4f32(a, Vs[(4 * kk + quad) * CS + 16 * cb + r16], acc[cb], 0, 0, 0);
      }
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int t = 16 * w + 4 * quad + i;
        if (t < nt) {
          const size_t th = (size_t)(tb + t) * NH + hd;
#pragma unroll
          for (int cb = 0; cb < 4; ++cb) {
            const int c = col0 + 16 * cb + r16;
            if (c < V) obuf[th * V + c] = acc[cb][i];
          }
        }
      }
    }
    __syncthreads();  // every read of the old state is done
    // ---- state to the end of the chunk's nt tokens
    {
      const float dec = pw[nt];
      for (int rb = w; rb < DP / 16; rb += 4) {
        f32x4 acc[4];
#pragma unroll
        for (int cb = 0; cb < 4; ++cb) acc[cb] = (f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll 4
        for (int kk = 0; kk < CL / 4; ++kk) {
          const int sidx = 4 * kk + quad;
          const float a = Ks[sidx * QS + 16 * rb + r16];
          const float ws = sidx < nt ? pw[nt - 1 - sidx] : 0.f;
#pragma unroll
          for (int cb = 0; cb < 4; ++cb)
            acc[cb] = __builtin_amdgcn_mfma_f32_16x16x4f32(a, ws * Vs[sidx * CS + 16 * cb + r16], acc[cb], 0, 0, 0);
        }
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
          for (int cb = 0; cb < 4; ++cb) {
            float* p = Sst + (16 * rb + 4 * quad + i) * CS + 16 * cb + r16;
            *p = dec * *p + acc[cb][i];
          }
      }
    }
  }
  __syncthreads();
  for (int i = tid; i < DP * 64; i += 256) {
    const int d = i / 64, c = i % 64;
    if (d < D && col0 + c < V) S[(sbase + d) * V + col0 + c] = Sst[d * CS + c];
  }
}

// y = o / rms(o over all heads' columns) * w * sigmoid(gate); one workgroup per token
template <typename T>
__global__ void __launch_bounds__(256) lightning_out_kernel(const float* __restrict__ obuf, const T* __restrict__ gate,
                                                             int64_t gate_stride, const T* __restrict__ w,
                                                             T* __restrict__ out, int64_t out_stride, int N, float eps) {
  __shared__ float red[16];
  const size_t t = blockIdx.x;
  const float* o = obuf + t * (size_t)N;
  float ss = 0.f;
  for (int i = threadIdx.x; i < N; i += 256) ss += o[i] * o[i];
  ss = block_sum(ss, red);
  const float r = 1.f / sqrtf(ss / (float)N + eps);
  for (int i = threadIdx.x; i < N; i += 256) {
    const float g = ldf<T>(gate, t * gate_stride + i);
    stf<T>(out, t * out_stride + i, o[i] * r * ldf<T>(w, i) / (1.f + expf(-g)));
  }
}


// The same for rows that are multiples of 4 at aligned addresses: 16-byte loads of the read-out, 8- / 16-byte loads and
// stores of gate and result (the weight may sit anywhere in a flat parameter buffer: element loads).
template <typename T>
__global__ void __launch_bounds__(256) lightning_out_vec_kernel(const float* __restrict__ obuf, const T* __restrict__ gate,
                                                                 int64_t gate_stride, const T* __restrict__ w,
                                                                 T* __restrict__ out, int64_t out_stride, int N,
                                                                 float eps) {
  __shared__ float red[16];
  const size_t t = blockIdx.x;
  const float* o = obuf + t * (size_t)N;
  float ss = 0.f;
  for (int i = 4 * threadIdx.x; i < N; i += 1024) {
    const f32x4 v = *reinterpret_cast<const f32x4*>(o + i);
    ss += v[0] * v[0] + v[1] * v[1] + v[2] * v[2] + v[3] * v[3];
  }
  ss = block_sum(ss, red);
  const float r = 1.f / sqrtf(ss / (float)N + eps);
  for (int i = 4 * threadIdx.x; i < N; i += 1024) {
    const f32x4 v = *reinterpret_cast<const f32x4*>(o + i);
    float g[4], y[4];
    if (sizeof(T) == 2) {
      const bf16x4 gv = *reinterpret_cast<const bf16x4*>(reinterpret_cast<const bf16_t*>(gate) + t * gate_stride + i);
#pragma unroll
      for (int e = 0; e < 4; ++e) g[e] = bf2f(gv[e]);
    } else {
      const f32x4 gv = *reinterpret_cast<const f32x4*>(reinterpret_cast<const float*>(gate) + t * gate_stride + i);
#pragma unroll
      for (int e = 0; e < 4; ++e) g[e] = gv[e];
    }
#pragma unroll
    for (int e = 0; e < 4; ++e) y[e] = v[e] * r * ldf<T>(w, i + e) / (1.f + expf(-g[e]));
    if (sizeof(T) == 2)
      *reinterpret_cast<bf16x4*>(reinterpret_cast<bf16_t*>(out) + t * out_stride + i) =
          (bf16x4){f2bf(y[0]), f2bf(y[1]), f2bf(y[2]), f2bf(y[3])};
    else
      *reinterpret_cast<f32x4*>(reinterpret_cast<float*>(out) + t * out_stride + i) = (f32x4){y[0], y[1], y[2], y[3]};
  }
}

}  // namespace

// proj rows hold (at q_off / k_off / v_off) NH query heads of D, NH key heads of D, NH value heads of V; act = 1:
// SiLU on all three. decay [NH] fp32. S [slots, NH, D, V] fp32; obuf [T, NH, V] fp32.
extern "C" int areal_lightning_scan(const void* proj, int64_t row_stride, int q_off, int k_off, int v_off,
                                    const float* decay, const int* cu_q, const int* first_pos, const int* state_slots,
                                    float* S, float* obuf, int B, int NH, int D, int V, int max_q, int act, int dt,
                                    hipStream_t st) {
  if (B == 0) return 0;
  if (D > 256 || D <= 0 || V <= 0) return -1;
  const dim3 grid(B, NH, (V + 63) / 64);
  if (max_q >= 16 && D <= 128) {
#define CHUNK(TT, DPV)                                                                                             \
  do {                                                                                                             \
    const size_t lds = sizeof(float) * ((size_t)DPV * (CL + 4) + 2 * (size_t)CL * (DPV + 4) + 2 * (size_t)CL * (CL + 4) + \
                                        CL + 1);                                                                   \
    static bool raised = false;                                                                                    \
    if (!raised && lds > 64 * 1024) {                                                                              \
      HIP_RET(hipFuncSetAttribute((const void*)lightning_chunk_kernel<TT, DPV>,                                    \
                                  hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024));                        \
      raised = true;                                                                                               \
    }                                                                                                              \
    hipLaunchKernelGGL((lightning_chunk_kernel<TT, DPV>), grid, dim3(256), lds, st, (const TT*)proj, row_stride,   \
                       q_off, k_off, v_off, decay, cu_q, first_pos, state_slots, S, obuf, NH, D, V, act);          \
  } while (0)
#define PICKC(TT)                      \
  do {                                 \
    if (D <= 32) CHUNK(TT, 32);        \
    else if (D <= 64) CHUNK(TT, 64);   \
    else CHUNK(TT, 128);               \
  } while (0)
    if (dt == 0) PICKC(bf16_t);
    else PICKC(float);
#undef PICKC
#undef CHUNK
    return (int)hipGetLastError();
  }
#define LAUNCH(TT, DPV)                                                                                           \
  hipLaunchKernelGGL((lightning_scan_kernel<TT, DPV>), grid, dim3(64 * RW), 0, st, (const TT*)proj, row_stride,   \
                     q_off, k_off, v_off, decay, cu_q, first_pos, state_slots, S, obuf, NH, D, V, act)
#define PICK(TT)                        \
  do {                                  \
    if (D <= 32) LAUNCH(TT, 32);        \
    else if (D <= 64) LAUNCH(TT, 64);   \
    else if (D <= 128) LAUNCH(TT, 128); \
    else LAUNCH(TT, 256);               \
  } while (0)
  if (dt == 0) PICK(bf16_t);
  else PICK(float);
#undef PICK
#undef LAUNCH
  return (int)hipGetLastError();
}

// obuf [T, N] fp32 (N = heads x V), gate rows of N with gate_stride, w [N]; out rows of N with out_stride
extern "C" int areal_lightning_out(const float* obuf, const void* gate, int64_t gate_stride, const void* w, void* out,
                                   int64_t out_stride, int T, int N, float eps, int dt, hipStream_t st) {
  if (T == 0) return 0;
  const uintptr_t al = dt == 0 ? 8 : 16;
  if (N % 4 == 0 && gate_stride % 4 == 0 && out_stride % 4 == 0 && ((uintptr_t)obuf % 16) == 0 &&
      ((uintptr_t)gate % al) == 0 && ((uintptr_t)out % al) == 0) {
    if (dt == 0)
      hipLaunchKernelGGL(lightning_out_vec_kernel<bf16_t>, dim3(T), dim3(256), 0, st, obuf, (const bf16_t*)gate,
                         gate_stride, (const bf16_t*)w, (bf16_t*)out, out_stride, N, eps);
    else
      hipLaunchKernelGGL(lightning_out_vec_kernel<float>, dim3(T), dim3(256), 0, st, obuf, (const float*)gate,
                         gate_stride, (const float*)w, (float*)out, out_stride, N, eps);
    return (int)hipGetLastError();
  }
  if (dt == 0)
    hipLaunchKernelGGL(lightning_out_kernel<bf16_t>, dim3(T), dim3(256), 0, st, obuf, (const bf16_t*)gate, gate_stride,
                       (const bf16_t*)w, (bf16_t*)out, out_stride, N, eps);
  else
    hipLaunchKernelGGL(lightning_out_kernel<float>, dim3(T), dim3(256), 0, st, obuf, (const float*)gate, gate_stride,
                       (const float*)w, (float*)out, out_stride, N, eps);
  return (int)hipGetLastError();
}
