// Gated linear attention: a matrix state per head whose rows (one per key channel) decay by a data-dependent factor.
//
//   alpha_t = sigmoid(z_t)^(1 / tau) = exp(-softplus(-z_t) / tau)        z_t: one logit per head and key channel
//   S_t     = diag(alpha_t) S_(t-1) + k_t v_t^T      [D, V]              o_t = S_t^T (q_t * q_scale)
//   y_t     = o_t / rms(o_t over V) * w * silu(g_t)                      per head; w [V] is shared by the heads
//
// q, k, v and g are columns of one projection (storage type T); z arrives as fp32 logits (plus a bias in T), and the
// decays, the state, the read-out and the norm are fp32. State slots [slots, heads, D, V] live in device memory
// between steps: a row whose first token has position 0 starts from S = 0 whatever its slot held before; a row with a
// negative slot is skipped (its outputs are zero).
//
// `gla_scan_kernel`: token by token, one workgroup of four waves per (row, head, 64 value columns); wave r keeps a
// quarter of the rows of S in registers (lane c: column c). Keys, queries and decays of 8 tokens are staged ahead.
// `gla_chunk_kernel`: prompt portions in chunks of 16 tokens. With b_t = sum_{u <= t} ln alpha_u (per channel, from the
// chunk's start; every b <= 0):
//
//   o_t   = (q_t * exp(b_t))^T S_prev + sum_{s <= t} A[t, s] v_s,     A[t, s] = sum_d q_t[d] k_s[d] exp(b_t[d] - b_s[d])
//   S_new = diag(exp(b_L)) S_prev + sum_s (k_s * exp(b_L - b_s)) v_s^T
//
// Every exponent is <= 0: nothing overflows whatever the decays are, and nothing is divided.
// `gla_out_kernel`: per-head RMS norm of the read-out, weight, SiLU gate.
#include "common.hpp"

namespace {

template <typename T> DEVINL float ldf(const T* p, size_t i);
template <> DEVINL float ldf<bf16_t>(const bf16_t* p, size_t i) { return bf2f(p[i]); }
template <> DEVINL float ldf<float>(const float* p, size_t i) { return p[i]; }
template <typename T> DEVINL void stf(T* p, size_t i, float v);
template <> DEVINL void stf<bf16_t>(bf16_t* p, size_t i, float v) { p[i] = f2bf(v); }
template <> DEVINL void stf<float>(float* p, size_t i, float v) { p[i] = v; }

// ln sigmoid(z) / tau
DEVINL float log_decay(float z, float inv_tau) { return -(fmaxf(-z, 0.f) + log1pf(expf(-fabsf(z)))) * inv_tau; }

constexpr int TC = 8;  // tokens staged per step of the loop
constexpr int RW = 4;  // waves of a workgroup

template <typename T, int DP>
__global__ void __launch_bounds__(64 * RW) gla_scan_kernel(
    const T* __restrict__ proj, int64_t row_stride, int q_off, int k_off, int v_off, const float* __restrict__ z,
    int64_t z_stride, const T* __restrict__ z_bias, float inv_tau, float q_scale, const int* __restrict__ cu_q,
    const int* __restrict__ first_pos, const int* __restrict__ state_slots, float* __restrict__ S,
    float* __restrict__ obuf, int NH, int D, int V) {
  constexpr int DQ = DP / RW;
  __shared__ float kqa[TC][3][DP];
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
  const size_t sbase = ((size_t)slot * NH + hd) * D;
  const int d0 = r * DQ;
  float s[DQ];
#pragma unroll
  for (int d = 0; d < DQ; ++d) s[d] = (!fresh && has && d0 + d < D) ? S[(sbase + d0 + d) * V + col] : 0.f;
  for (int tb = t_lo; tb < t_hi; tb += TC) {
    const int nt = min(TC, t_hi - tb);
    __syncthreads();  // the step before is finished with the staged operands and the partials
    for (int i = tid; i < TC * DP; i += 64 * RW) {
      const int d = i % DP, tt = i / DP;
      const bool live = tt < nt && d < D;
      const size_t tok = (size_t)(tb + min(tt, nt - 1));
      const T* row = proj + tok * row_stride;
      kqa[tt][0][d] = live ? ldf<T>(row, k_off + hd * D + d) : 0.f;
      kqa[tt][1][d] = live ? ldf<T>(row, q_off + hd * D + d) * q_scale : 0.f;
      kqa[tt][2][d] = live ? expf(log_decay(z[tok * z_stride + hd * D + d] + (z_bias ? ldf<T>(z_bias, hd * D + d) : 0.f),
                                            inv_tau))
                           : 1.f;
    }
    float vv[TC];
#pragma unroll
    for (int tt = 0; tt < TC; ++tt)
      vv[tt] = (tt < nt && has) ? ldf<T>(proj + (size_t)(tb + tt) * row_stride, v_off + hd * V + col) : 0.f;
    __syncthreads();
#pragma unroll
    for (int tt = 0; tt < TC; ++tt) {
      if (tt < nt) {
        float hacc = 0.f;
#pragma unroll
        for (int d = 0; d < DQ; ++d) {
          s[d] = kqa[tt][2][d0 + d] * s[d] + vv[tt] * kqa[tt][0][d0 + d];
          hacc += s[d] * kqa[tt][1][d0 + d];
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

// Prompt portions: chunks of CT tokens, in two launches. Whatever does not depend on the state is formed for all
// chunks at once by `gla_prep_kernel` (one workgroup per (chunk, row, head), thousands of them): the per-channel log
// decays summed along the chunk's tokens (b_t), q_t * exp(b_t), k_s * exp(b_L - b_s), exp(b_L), and the lower triangle
// A[t, s] = sum_d q_t[d] k_s[d] exp(b_t[d] - b_s[d]), pair by pair so that every exponent is <= 0. `gla_chunk_kernel`
// then walks a row's chunks in order with nothing but matrix products on the fp32 matrix cores (MFMA 16x16x4): the
// read-out q~ S_prev + A V (wave w owns 16 of the workgroup's 64 value columns) and the state's move to the chunk's end
// diag(exp(b_L)) S_prev + k~^T V (every fourth block of 16 state rows a wave). The next chunk's operands are fetched
// into registers under the matrix work.
constexpr int CT = 16;

// bf16 storage: v_exp_f32 (relative error ~1e-6, far below the storage's); fp32 storage: the library's exp
template <typename T> DEVINL float exp_le0(float x) { return sizeof(T) == 2 ? __expf(x) : expf(x); }

template <typename T, int DP>
__global__ void __launch_bounds__(256) gla_prep_kernel(
    const T* __restrict__ proj, int64_t row_stride, int q_off, int k_off, const float* __restrict__ z, int64_t z_stride,
    const T* __restrict__ z_bias, float inv_tau, float q_scale, const int* __restrict__ cu_q,
    const int* __restrict__ state_slots, float* __restrict__ qd, float* __restrict__ kd, float* __restrict__ el,
    float* __restrict__ abuf, int NH, int D) {
  constexpr int QS = DP + 1;  // odd stride: the pair loop's 16 key rows fall on different banks
  __shared__ float Qr[CT * QS], Kr[CT * QS], Bs[CT * QS];
  const int b = blockIdx.y, hd = blockIdx.z, tid = threadIdx.x;
  const int t_lo = cu_q[b], t_hi = cu_q[b + 1], tb = t_lo + CT * blockIdx.x;
  if (tb >= t_hi || state_slots[b] < 0) return;
  const int nt = min(CT, t_hi - tb);
  for (int i = tid; i < CT * DP; i += 256) {
    const int d = i % DP, tt = i / DP;
    const bool live = tt < nt && d < D;
    const size_t tok = (size_t)(tb + min(tt, nt - 1));
    const T* row = proj + tok * row_stride;
    const int dc = min(d, D - 1);
    Kr[tt * QS + d] = live ? ldf<T>(row, k_off + hd * D + dc) : 0.f;
    Qr[tt * QS + d] = live ? ldf<T>(row, q_off + hd * D + dc) * q_scale : 0.f;
    // rows past the chunk's end and padding channels do not decay
    Bs[tt * QS + d] = live ? log_decay(z[tok * z_stride + hd * D + dc] + (z_bias ? ldf<T>(z_bias, hd * D + dc) : 0.f), inv_tau)
                           : 0.f;
  }
  __syncthreads();
  if (tid < DP) {  // running sums along the chunk's tokens, one channel a thread
    float run = 0.f;
#pragma unroll
    for (int tt = 0; tt < CT; ++tt) {
      run += Bs[tt * QS + tid];
      Bs[tt * QS + tid] = run;
    }
  }
  __syncthreads();
  const size_t N = (size_t)NH * D;
  for (int i = tid; i < CT * DP; i += 256) {
    const int d = i % DP, tt = i / DP;
    if (tt < nt && d < D) {
      const float bt = Bs[tt * QS + d], bl = Bs[(nt - 1) * QS + d];
      qd[(size_t)(tb + tt) * N + hd * D + d] = Qr[tt * QS + d] * exp_le0<T>(bt);
      kd[(size_t)(tb + tt) * N + hd * D + d] = Kr[tt * QS + d] * exp_le0<T>(bl - bt);
      if (tt == 0) el[(size_t)tb * N + hd * D + d] = exp_le0<T>(bl);
    }
  }
  {  // the chunk's own pairs: thread (t, s), s <= t
    const int t = tid / CT, sx = tid % CT;
    float a0 = 0.f, a1 = 0.f;
    if (sx <= t && t < nt) {
      const float *qt = Qr + t * QS, *ks = Kr + sx * QS, *bt = Bs + t * QS, *bs = Bs + sx * QS;
#pragma unroll 4
      for (int d = 0; d < DP; d += 2) {
        a0 += qt[d] * ks[d] * exp_le0<T>(bt[d] - bs[d]);
        a1 += qt[d + 1] * ks[d + 1] * exp_le0<T>(bt[d + 1] - bs[d + 1]);
      }
    }
    if (t < nt) abuf[((size_t)(tb + t) * NH + hd) * CT + sx] = a0 + a1;
  }
}

template <int DP>
__global__ void __launch_bounds__(256) gla_chunk_kernel(
    const float* __restrict__ qd, const float* __restrict__ kd, const float* __restrict__ el,
    const float* __restrict__ abuf, const void* __restrict__ proj, int64_t row_stride, int v_off, int bf16_storage,
    const int* __restrict__ cu_q, const int* __restrict__ first_pos, const int* __restrict__ state_slots,
    float* __restrict__ S, float* __restrict__ obuf, int NH, int D, int V) {
  constexpr int QS = DP + 4, CS = 64 + 4, AS = CT + 1;
  constexpr int NE = CT * DP / 256, NV = CT * 64 / 256;  // elements per thread of q~ / k~, and of v
  extern __shared__ float cl[];
  float* Sst = cl;               // [DP][CS] state slice
  float* Qd = Sst + DP * CS;     // [CT][QS] q * q_scale * exp(b_t)
  float* Kd = Qd + CT * QS;      // [CT][QS] k * exp(b_L - b_t)
  float* Vs = Kd + CT * QS;      // [CT][CS]
  float* As = Vs + CT * CS;      // [CT][AS]
  float* Es = As + CT * AS;      // [DP] exp(b_L)
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
  const size_t sbase = ((size_t)slot * NH + hd) * D, N = (size_t)NH * D;
  for (int i = tid; i < DP * 64; i += 256) {
    const int d = i / 64, c = i % 64;
    Sst[d * CS + c] = (!fresh && d < D && col0 + c < V) ? S[(sbase + d) * V + col0 + c] : 0.f;
  }
  float rq[NE], rk[NE], rv[NV], ra, re = 1.f;
  auto fetch = [&](int tb) {
    const int nt = min(CT, t_hi - tb);
#pragma unroll
    for (int j = 0; j < NE; ++j) {
      const int i = tid + 256 * j, d = i % DP, tt = i / DP;
      const bool live = tt < nt && d < D;
      const size_t at = (size_t)(tb + min(tt, nt - 1)) * N + hd * D + min(d, D - 1);
      rq[j] = live ? qd[at] : 0.f;
      rk[j] = live ? kd[at] : 0.f;
    }
#pragma unroll
    for (int j = 0; j < NV; ++j) {
      const int i = tid + 256 * j, c = i % 64, tt = i / 64;
      const size_t at = (size_t)(tb + min(tt, nt - 1)) * row_stride + v_off + hd * V + min(col0 + c, V - 1);
      const float x = bf16_storage ? bf2f(reinterpret_cast<const bf16_t*>(proj)[at]) : reinterpret_cast<const float*>(proj)[at];
      rv[j] = (tt < nt && col0 + c < V) ? x : 0.f;
    }
    {
      const int t = tid / CT, sx = tid % CT;
      ra = (t < nt && sx <= t) ? abuf[((size_t)(tb + t) * NH + hd) * CT + sx] : 0.f;
    }
    if (tid < DP) re = tid < D ? el[(size_t)tb * N + hd * D + tid] : 1.f;
  };
  fetch(t_lo);
  for (int tb = t_lo; tb < t_hi; tb += CT) {
    const int nt = min(CT, t_hi - tb);
    __syncthreads();  // the chunk before is done with the staged operands
#pragma unroll
    for (int j = 0; j < NE; ++j) {
      const int i = tid + 256 * j, d = i % DP, tt = i / DP;
      Qd[tt * QS + d] = rq[j];
      Kd[tt * QS + d] = rk[j];
    }
#pragma unroll
    for (int j = 0; j < NV; ++j) {
      const int i = tid + 256 * j;
      Vs[(i / 64) * CS + i % 64] = rv[j];
    }
    As[(tid / CT) * AS + tid % CT] = ra;
    if (tid < DP) Es[tid] = re;
    if (tb + CT < t_hi) fetch(tb + CT);
    __syncthreads();
    {  // read-out: rows = the chunk's tokens, columns 16 w .. 16 w + 15 of the slice; two accumulation chains
      f32x4 acc = {0.f, 0.f, 0.f, 0.f}, acc2 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll 8
      for (int kk = 0; kk < DP / 4; kk += 2) {
        acc = __builtin_amdgcn_mfma_f32_16x16x4f32(Qd[r16 * QS + 4 * kk + quad], Sst[(4 * kk + quad) * CS + 16 * w + r16],
                                                   acc, 0, 0, 0);
        acc2 = __builtin_amdgcn_mfma_f32_16x16x4f32(Qd[r16 * QS + 4 * kk + 4 + quad],
                                                    Sst[(4 * kk + 4 + quad) * CS + 16 * w + r16], acc2, 0, 0, 0);
      }
#pragma unroll
      for (int kk = 0; kk < CT / 4; kk += 2) {
        acc = __builtin_amdgcn_mfma_f32_16x16x4f32(As[r16 * AS + 4 * kk + quad], Vs[(4 * kk + quad) * CS + 16 * w + r16],
                                                   acc, 0, 0, 0);
        acc2 = __builtin_amdgcn_mfma_f32_16x16x4f32(As[r16 * AS + 4 * kk + 4 + quad],
                                                    Vs[(4 * kk + 4 + quad) * CS + 16 * w + r16], acc2, 0, 0, 0);
      }
      acc += acc2;
      const int c = col0 + 16 * w + r16;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int t = 4 * quad + i;
        if (t < nt && c < V) obuf[((size_t)(tb + t) * NH + hd) * V + c] = acc[i];
      }
    }
    __syncthreads();  // every read of the old state is done
    for (int rb = w; rb < DP / 16; rb += 4) {  // state to the end of the chunk's nt tokens
      f32x4 acc[4];
#pragma unroll
      for (int cb = 0; cb < 4; ++cb) acc[cb] = (f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int kk = 0; kk < CT / 4; ++kk) {
        const float a = Kd[(4 * kk + quad) * QS + 16 * rb + r16];
#pragma unroll
        for (int cb = 0; cb < 4; ++cb)
          acc[cb] = __builtin_amdgcn_mfma_f32_16x16x4f32(a, Vs[(4 * kk + quad) * CS + 16 * cb + r16], acc[cb], 0, 0, 0);
      }
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int d = 16 * rb + 4 * quad + i;
        const float dec = Es[d];
#pragma unroll
        for (int cb = 0; cb < 4; ++cb) {
          float* p = Sst + d * CS + 16 * cb + r16;
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

// One wave per (token, head): y = o / rms(o over V) * w * silu(gate)
template <typename T>
__global__ void __launch_bounds__(256) gla_out_kernel(const float* __restrict__ obuf, const T* __restrict__ gate,
                                                      int64_t gate_stride, const T* __restrict__ w, T* __restrict__ out,
                                                      int64_t n_rows, int NH, int V, float eps) {
  const int lane = threadIdx.x & 63;
  const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= n_rows) return;
  const int64_t t = row / NH;
  const int hd = (int)(row % NH);
  const float* o = obuf + row * V;
  float ss = 0.f;
  for (int i = lane; i < V; i += 64) ss += o[i] * o[i];
  const float r = 1.f / sqrtf(wave_sum(ss) / (float)V + eps);
  for (int i = lane; i < V; i += 64) {
    const float g = ldf<T>(gate, t * gate_stride + hd * V + i);
    stf<T>(out, row * V + i, o[i] * r * ldf<T>(w, i) * (g / (1.f + expf(-g))));
  }
}

}  // namespace

// proj rows hold (at q_off / k_off / v_off) NH query heads of D, NH key heads of D, NH value heads of V. z fp32 rows of
// NH D decay logits (z_stride apart), z_bias [NH D] in the storage type or null. S [slots, NH, D, V] fp32; obuf
// [T, NH, V] fp32. scratch: T (3 NH D + 16 NH) floats for the chunked form (rows of 16 tokens and more, D <= 128), or
// null: token by token.
extern "C" int areal_gla_scan(const void* proj, int64_t row_stride, int q_off, int k_off, int v_off, const float* z,
                              int64_t z_stride, const void* z_bias, float tau, float q_scale, const int* cu_q,
                              const int* first_pos, const int* state_slots, float* S, float* obuf, float* scratch, int T,
                              int B, int NH, int D, int V, int max_q, int dt, hipStream_t st) {
  if (B == 0) return 0;
  if (D > 256 || D <= 0 || V <= 0 || !(tau > 0.f)) return -1;
  const dim3 grid(B, NH, (V + 63) / 64);
  const float inv_tau = 1.f / tau;
  if (max_q >= CT && D <= 128 && scratch) {
    // scratch: q~ | k~ | exp(b_L) as [T, NH D] each, then A as [T, NH, CT]
    const size_t N = (size_t)NH * D;
    float *qd = scratch, *kd = qd + (size_t)T * N, *el = kd + (size_t)T * N, *ab = el + (size_t)T * N;
    const dim3 pgrid((max_q + CT - 1) / CT, B, NH);
#define CHUNK(TT, DPV)                                                                                              \
  do {                                                                                                              \
    const size_t lds = sizeof(float) * ((size_t)DPV * 68 + 2 * (size_t)CT * (DPV + 4) + (size_t)CT * 68 + CT * (CT + 1) + DPV); \
    static bool raised = false;                                                                                     \
    if (!raised && lds > 64 * 1024) {                                                                               \
      HIP_RET(hipFuncSetAttribute((const void*)gla_chunk_kernel<DPV>, hipFuncAttributeMaxDynamicSharedMemorySize,   \
                                  160 * 1024));                                                                     \
      raised = true;                                                                                                \
    }                                                                                                               \
    hipLaunchKernelGGL((gla_prep_kernel<TT, DPV>), pgrid, dim3(256), 0, st, (const TT*)proj, row_stride, q_off, k_off, \
                       z, z_stride, (const TT*)z_bias, inv_tau, q_scale, cu_q, state_slots, qd, kd, el, ab, NH, D);  \
    hipLaunchKernelGGL((gla_chunk_kernel<DPV>), grid, dim3(256), lds, st, qd, kd, el, ab, proj, row_stride, v_off,  \
                       dt == 0 ? 1 : 0, cu_q, first_pos, state_slots, S, obuf, NH, D, V);                           \
  } while (0)
#define PICKC(TT)                    \
  do {                               \
    if (D <= 32) CHUNK(TT, 32);      \
    else if (D <= 64) CHUNK(TT, 64); \
    else CHUNK(TT, 128);             \
  } while (0)
    if (dt == 0) PICKC(bf16_t);
    else PICKC(float);
#undef PICKC
#undef CHUNK
    return (int)hipGetLastError();
  }
#define LAUNCH(TT, DPV)                                                                                          \
  hipLaunchKernelGGL((gla_scan_kernel<TT, DPV>), grid, dim3(64 * RW), 0, st, (const TT*)proj, row_stride, q_off,  \
                     k_off, v_off, z, z_stride, (const TT*)z_bias, inv_tau, q_scale, cu_q, first_pos, state_slots, S, \
                     obuf, NH, D, V)
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

// obuf [T, NH, V] fp32, gate rows of NH V with gate_stride, w [V]; out [T, NH V] contiguous
extern "C" int areal_gla_out(const float* obuf, const void* gate, int64_t gate_stride, const void* w, void* out, int T,
                             int NH, int V, float eps, int dt, hipStream_t st) {
  if (T == 0) return 0;
  const int64_t n = (int64_t)T * NH;
  const dim3 grid((unsigned)((n + 3) / 4));
  if (dt == 0)
    hipLaunchKernelGGL(gla_out_kernel<bf16_t>, grid, dim3(256), 0, st, obuf, (const bf16_t*)gate, gate_stride,
                       (const bf16_t*)w, (bf16_t*)out, n, NH, V, eps);
  else
    hipLaunchKernelGGL(gla_out_kernel<float>, grid, dim3(256), 0, st, obuf, (const float*)gate, gate_stride,
                       (const float*)w, (float*)out, n, NH, V, eps);
  return (int)hipGetLastError();
}
