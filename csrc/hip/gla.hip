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
// [T, NH, V] fp32.
extern "C" int areal_gla_scan(const void* proj, int64_t row_stride, int q_off, int k_off, int v_off, const float* z,
                              int64_t z_stride, const void* z_bias, float tau, float q_scale, const int* cu_q,
                              const int* first_pos, const int* state_slots, float* S, float* obuf, int B, int NH, int D,
                              int V, int max_q, int dt, hipStream_t st) {
  if (B == 0) return 0;
  if (D > 256 || D <= 0 || V <= 0 || !(tau > 0.f)) return -1;
  const dim3 grid(B, NH, (V + 63) / 64);
  const float inv_tau = 1.f / tau;
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
