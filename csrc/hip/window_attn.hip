// Causal sliding-window attention over the paged cache whose scores are shaped before the softmax:
//
//   s_g(i, j)  = (q_g(i) . k_c(g)(j)) * scale                      c(g) = g / (H / G): grouped key/value heads
//   s_g       <- cap * tanh(s_g / cap)                             (cap > 0; otherwise left as it is)
//   s_g       <- s_g - slope_g * (i - j),  slope_g = 2^(-slope_exp * (g + 1) / H)     (slope_exp = 0: no bias)
//   s_g       <- s_g - r1_g * ln(1 + r2_g * (i - j))              (r1 / r2 given: a learned logarithmic distance penalty)
//   t_h        = sum_g M[h, g] s_g                                 head mixing (M = null: t_h = s_h)
//   visible:     0 <= i - j < window, or j <= i and j < keep_first    (window <= 0: every earlier key; the first
//                keep_first tokens of a sequence stay visible to every later query, at their true positions)
//   p_h(j)     = exp(t_h(j)) / (sink + sum_j' exp(t_h(j')))        sink = 1: a key of score 0 that has no value
//   o_h(i)     = sum_j p_h(j) v_c(h)(j)  [* sigmoid(gate_h(i)) when a gate is given: one number per head and token, or
//                one per head, token and value channel (`gate_elem`)]
//
// Scores, weights and the accumulation run in fp32 whatever the storage type T (bf16 / fp32) of q, the caches
// and the output. Because the heads are mixed before the softmax, one workgroup owns ALL heads of a tile of BQ
// queries: per 32-key page it forms the H raw score tiles in LDS, mixes them, updates the running maximum /
// denominator of every (head, query) row and accumulates p.v into LDS-resident fp32 accumulators.
//
// The same kernel serves prompt portions (tiles of BQ queries, grid x = tiles, y = rows of the batch) and
// decoding (BQ = 1, grid z = splits of the visible key range whose partial results `window_attn_combine` merges);
// bf16 prompt portions of the common head sizes take the matrix-core kernel further down instead.
// Queries of row b are the LAST cu_q[b+1] - cu_q[b] positions of its context of ctx_len[b] tokens.
//
// Cache layout: K [pages, G, 32, D], V [pages, G, 32, Dv], token-major inside a page.
#include "common.hpp"

namespace {

constexpr int PAGE = 32;

template <typename T> DEVINL float ldf(const T* p, size_t i);
template <> DEVINL float ldf<bf16_t>(const bf16_t* p, size_t i) { return bf2f(p[i]); }
template <> DEVINL float ldf<float>(const float* p, size_t i) { return p[i]; }
template <typename T> DEVINL void stf(T* p, size_t i, float v);
template <> DEVINL void stf<bf16_t>(bf16_t* p, size_t i, float v) { p[i] = f2bf(v); }
template <> DEVINL void stf<float>(float* p, size_t i, float v) { p[i] = v; }

// Per token: RMS norm of every query head (-> q_out) and key head (-> K cache) over its D elements with a weight
// vector shared by the heads, values copied into the V cache. `proj` rows hold q heads | k heads | v heads (and may
// be longer: row_stride). slots[t] = page * 32 + offset, negative: nothing is cached for this token.
template <typename T>
__global__ void __launch_bounds__(256) qk_norm_cache_write_kernel(
    const T* __restrict__ proj, int64_t row_stride, const T* __restrict__ qw, const T* __restrict__ kw,
    const int64_t* __restrict__ slots, T* __restrict__ q_out, T* __restrict__ kcache, T* __restrict__ vcache, int H,
    int G, int D, int V, float eps) {
  const int t = blockIdx.x;
  const T* row = proj + (size_t)t * row_stride;
  const int64_t slot = slots[t];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const size_t page = slot >= 0 ? (size_t)(slot / PAGE) : 0;
  const int off = slot >= 0 ? (int)(slot % PAGE) : 0;
  for (int u = wave; u < H + G; u += 4) {
    const T* src = row + (size_t)u * D;
    float ss = 0.f;
    for (int d = lane; d < D; d += 64) {
      const float x = ldf<T>(src, d);
      ss += x * x;
    }
    ss = wave_sum(ss);
    const float r = 1.f / sqrtf(ss / (float)D + eps);
    if (u < H) {
      T* dst = q_out + ((size_t)t * H + u) * D;
      for (int d = lane; d < D; d += 64) stf<T>(dst, d, ldf<T>(src, d) * r * (qw ? ldf<T>(qw, d) : 1.f));
    } else if (slot >= 0) {
      T* dst = kcache + ((page * G + (u - H)) * PAGE + off) * D;
      for (int d = lane; d < D; d += 64) stf<T>(dst, d, ldf<T>(src, d) * r * (kw ? ldf<T>(kw, d) : 1.f));
    }
  }
  if (slot >= 0) {
    const T* vsrc = row + (size_t)(H + G) * D;
    for (int i = threadIdx.x; i < G * V; i += 256) {
      const int c = i / V, v = i % V;
      vcache[((page * G + c) * PAGE + off) * V + v] = vsrc[i];
    }
  }
}

// Per token: rotate the first R coordinates of every query and key head by the token's position (neighbouring
// coordinates (2i, 2i + 1) form a pair; table rows hold R / 2 cosines, then R / 2 sines, already multiplied by
// whatever factor the rotation carries), then divide the head by its root mean square over D (no weight). Queries go
// to q_out, keys into the K cache. Values: v <- (1 - lam) v + lam v_first when `v_first` is given (rows of G V values of
// the same tokens, from the layer whose values are shared), then into the V cache.
template <typename T>
__global__ void __launch_bounds__(256) rot_norm_cache_write_kernel(
    const T* __restrict__ proj, int64_t row_stride, const int* __restrict__ positions, const float* __restrict__ table,
    int n_pos, int R, const int64_t* __restrict__ slots, const T* __restrict__ v_first, int64_t vf_stride,
    const T* __restrict__ lam_p, T* __restrict__ q_out, T* __restrict__ kcache, T* __restrict__ vcache, int H, int G,
    int D, int V, float eps, int v_transposed) {
  const int t = blockIdx.x;
  const T* row = proj + (size_t)t * row_stride;
  const int64_t slot = slots[t];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const size_t page = slot >= 0 ? (size_t)(slot / PAGE) : 0;
  const int off = slot >= 0 ? (int)(slot % PAGE) : 0;
  const int pos = min(max(positions[t], 0), n_pos - 1);
  const float* cs = table + (size_t)pos * R;
  const int half = R / 2;
  // grid y spreads a token's heads over workgroups (one head a wave when there are enough of them)
  for (int u = blockIdx.y * 4 + wave; u < H + G; u += 4 * gridDim.y) {
    if (u >= H && slot < 0) continue;
    const T* src = row + (size_t)u * D;
    T* dst = u < H ? q_out + ((size_t)t * H + u) * D : kcache + ((page * G + (u - H)) * PAGE + off) * D;
    // units of work: pairs below R, single coordinates from R on
    const int units = half + (D - R);
    float ss = 0.f;
    for (int i = lane; i < units; i += 64) {
      if (i < half) {
        const float a = ldf<T>(src, 2 * i), b = ldf<T>(src, 2 * i + 1), c = cs[i], s = cs[half + i];
        const float x = a * c - b * s, y = b * c + a * s;
        ss += x * x + y * y;
      } else {
        const float x = ldf<T>(src, R + i - half);
        ss += x * x;
      }
    }
    ss = wave_sum(ss);
    const float r = 1.f / sqrtf(ss / (float)D + eps);
    for (int i = lane; i < units; i += 64) {
      if (i < half) {
        const float a = ldf<T>(src, 2 * i), b = ldf<T>(src, 2 * i + 1), c = cs[i], s = cs[half + i];
        stf<T>(dst, 2 * i, (a * c - b * s) * r);
        stf<T>(dst, 2 * i + 1, (b * c + a * s) * r);
      } else {
        stf<T>(dst, R + i - half, ldf<T>(src, R + i - half) * r);
      }
    }
  }
  if (slot >= 0) {
    const T* vsrc = row + (size_t)(H + G) * D;
    const float lam = v_first ? ldf<T>(lam_p, 0) : 0.f;
    for (int i = blockIdx.y * 256 + threadIdx.x; i < G * V; i += 256 * gridDim.y) {
      const int c = i / V, v = i % V;
      float x = ldf<T>(vsrc, i);
      if (v_first) x = (1.f - lam) * x + lam * ldf<T>(v_first, (size_t)t * vf_stride + i);
      // V pages are [G][32][V], or [G][V][32] (a channel's 32 tokens side by side) for the kernels that want V^T
      stf<T>(vcache, v_transposed ? ((page * G + c) * V + v) * PAGE + off : ((page * G + c) * PAGE + off) * V + v, x);
    }
  }
}

// The same for bf16 rows whose head sizes, strides and addresses are multiples of 8 elements (head size <= 512):
// sixteen lanes a head, every lane 8 consecutive coordinates (four rotation pairs) per 16-byte load, the head's
// rotated values kept in registers between the sum of squares and the scaling. Values move as 16-byte vectors too.
template <int NV>
__global__ void __launch_bounds__(256) rot_norm_cache_write_vec_kernel(
    const bf16_t* __restrict__ proj, int64_t row_stride, const int* __restrict__ positions,
    const float* __restrict__ table, int n_pos, int R, const int64_t* __restrict__ slots,
    const bf16_t* __restrict__ v_first, int64_t vf_stride, const bf16_t* __restrict__ lam_p, bf16_t* __restrict__ q_out,
    bf16_t* __restrict__ kcache, bf16_t* __restrict__ vcache, int H, int G, int D, int V, float eps, int v_transposed) {
  const int t = blockIdx.x;
  const bf16_t* row = proj + (size_t)t * row_stride;
  const int64_t slot = slots[t];
  const int l16 = threadIdx.x & 15, grp = threadIdx.x >> 4;
  const size_t page = slot >= 0 ? (size_t)(slot / PAGE) : 0;
  const int off = slot >= 0 ? (int)(slot % PAGE) : 0;
  const int pos = min(max(positions[t], 0), n_pos - 1);
  const float* cs = table + (size_t)pos * R;
  const int half = R / 2;
  const int u = blockIdx.y * 16 + grp;
  if (u < H + G && (u < H || slot >= 0)) {
    const bf16_t* src = row + (size_t)u * D;
    bf16_t* dst = u < H ? q_out + ((size_t)t * H + u) * D : kcache + ((page * G + (u - H)) * PAGE + off) * D;
    float x[NV][8];
    float ss = 0.f;
#pragma unroll
    for (int j = 0; j < NV; ++j) {
      const int d0 = 8 * (l16 + 16 * j);
      if (d0 < D) {
        const bf16x8 raw = ld8(src + d0);
#pragma unroll
        for (int e = 0; e < 8; e += 2) {
          const float a = bf2f(raw[e]), b = bf2f(raw[e + 1]);
          const int pi = (d0 + e) >> 1;
          if (pi < half) {
            const float c = cs[pi], sn = cs[half + pi];
            x[j][e] = a * c - b * sn;
            x[j][e + 1] = b * c + a * sn;
          } else {
            x[j][e] = a;
            x[j][e + 1] = b;
          }
          ss += x[j][e] * x[j][e] + x[j][e + 1] * x[j][e + 1];
        }
      }
    }
#pragma unroll
    for (int o = 8; o > 0; o >>= 1) ss += __shfl_xor(ss, o, 64);
    const float r = 1.f / sqrtf(ss / (float)D + eps);
#pragma unroll
    for (int j = 0; j < NV; ++j) {
      const int d0 = 8 * (l16 + 16 * j);
      if (d0 < D) {
        bf16x8 o8;
#pragma unroll
        for (int e = 0; e < 8; ++e) o8[e] = f2bf(x[j][e] * r);
        st8(dst + d0, o8);
      }
    }
  }
  if (slot >= 0) {
    const bf16_t* vsrc = row + (size_t)(H + G) * D;
    const float lam = v_first ? bf2f(lam_p[0]) : 0.f;
    for (int i = 8 * (blockIdx.y * 256 + threadIdx.x); i < G * V; i += 8 * 256 * gridDim.y) {
      const int c = i / V, v = i % V;
      bf16x8 raw = ld8(vsrc + i);
      if (v_first) {
        const bf16x8 f = ld8(v_first + (size_t)t * vf_stride + i);
#pragma unroll
        for (int e = 0; e < 8; ++e) raw[e] = f2bf((1.f - lam) * bf2f(raw[e]) + lam * bf2f(f[e]));
      }
      if (v_transposed) {
#pragma unroll
        for (int e = 0; e < 8; ++e) vcache[((page * G + c) * V + v + e) * PAGE + off] = raw[e];
      } else {
        st8(vcache + ((page * G + c) * PAGE + off) * V + v, raw);
      }
    }
  }
}

// Per token: queries and keys as they are (queries -> q_out, keys -> K cache); every value head divided by its root
// mean square over its V elements (no weight; `v_norm` = 0: copied) -> V cache. One head a wave, a token's heads
// spread over grid y.
template <typename T>
__global__ void __launch_bounds__(256) qkv_vnorm_cache_write_kernel(
    const T* __restrict__ proj, int64_t row_stride, const int64_t* __restrict__ slots, T* __restrict__ q_out,
    T* __restrict__ kcache, T* __restrict__ vcache, int H, int G, int D, int V, float eps, int v_norm,
    int v_transposed) {
  const int t = blockIdx.x;
  const T* row = proj + (size_t)t * row_stride;
  const int64_t slot = slots[t];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const size_t page = slot >= 0 ? (size_t)(slot / PAGE) : 0;
  const int off = slot >= 0 ? (int)(slot % PAGE) : 0;
  for (int u = blockIdx.y * 4 + wave; u < H + 2 * G; u += 4 * gridDim.y) {
    if (u < H) {
      if (q_out)
        for (int d = lane; d < D; d += 64) q_out[((size_t)t * H + u) * D + d] = row[(size_t)u * D + d];
    } else if (slot < 0) {
      continue;
    } else if (u < H + G) {
      T* dst = kcache + ((page * G + (u - H)) * PAGE + off) * D;
      for (int d = lane; d < D; d += 64) dst[d] = row[(size_t)u * D + d];
    } else {
      const int c = u - H - G;
      const T* src = row + (size_t)(H + G) * D + (size_t)c * V;
      // V pages are [G][32][V], or [G][V][32] (a channel's 32 tokens side by side) for the kernels that want V^T
      T* dst = v_transposed ? vcache + (page * G + c) * V * PAGE + off : vcache + ((page * G + c) * PAGE + off) * V;
      const int dstep = v_transposed ? PAGE : 1;
      float r = 1.f;
      if (v_norm) {
        float ss = 0.f;
        for (int d = lane; d < V; d += 64) {
          const float x = ldf<T>(src, d);
          ss += x * x;
        }
        r = 1.f / sqrtf(wave_sum(ss) / (float)V + eps);
      }
      for (int d = lane; d < V; d += 64) stf<T>(dst, (size_t)d * dstep, v_norm ? ldf<T>(src, d) * r : ldf<T>(src, d));
    }
  }
}

// x[t, i] *= sigmoid(gate[t, i]) over rows of n elements (x contiguous, gate rows gate_stride apart)
template <typename T>
__global__ void __launch_bounds__(256) sigmoid_gate_rows_kernel(T* __restrict__ x, const T* __restrict__ gate,
                                                                int64_t gate_stride, int64_t rows, int n) {
  const int64_t total = rows * n;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < total; i += (int64_t)gridDim.x * 256) {
    const int64_t t = i / n;
    const float g = ldf<T>(gate, t * gate_stride + (i - t * n));
    stf<T>(x, i, ldf<T>(x, i) / (1.f + expf(-g)));
  }
}

struct AttnShape {
  int H, G, D, V, BQ;
  // LDS layout in floats
  DEVINL int rows() const { return H * BQ; }
  __host__ __device__ size_t floats() const {
    return (size_t)H * BQ * D + (size_t)H * BQ * V + 2 * (size_t)H * BQ * PAGE + (size_t)PAGE * (D + 1) +
           (size_t)PAGE * V + 3 * (size_t)H * BQ + (size_t)H * H;
  }
};

template <typename T>
__global__ void __launch_bounds__(256) window_attn_kernel(
    const T* __restrict__ q, const T* __restrict__ kcache, const T* __restrict__ vcache,
    const int* __restrict__ block_tables, int max_pages, const int* __restrict__ cu_q,
    const int* __restrict__ ctx_len, const T* __restrict__ mix, const T* __restrict__ gate, int64_t gate_stride,
    int gate_elem, const T* __restrict__ r1, const T* __restrict__ r2,
    T* __restrict__ out, float* __restrict__ part_acc, float* __restrict__ part_ml, AttnShape sh, float scale, float softcap, float slope_exp, int window, int keep, int sink,
    int nsplit) {
  extern __shared__ float lds[];
  const int H = sh.H, G = sh.G, D = sh.D, V = sh.V, BQ = sh.BQ;
  const int b = blockIdx.y, split = blockIdx.z, tid = threadIdx.x;
  const int q0 = cu_q[b], qlen = cu_q[b + 1] - q0;
  const int t0 = blockIdx.x * BQ;
  if (t0 >= qlen) return;
  const int nq = min(BQ, qlen - t0);
  const int ctx = ctx_len[b];
  const int pos0 = ctx - qlen + t0;  // position of the tile's first query
  const int R = H * BQ, rep = H / G;
  float* qs = lds;                       // [H][BQ][D]
  float* acc = qs + (size_t)R * D;       // [H][BQ][V]
  float* S1 = acc + (size_t)R * V;       // [H][BQ][32] shaped scores per head
  float* S2 = S1 + (size_t)R * PAGE;     // [H][BQ][32] mixed scores, then weights
  float* Kt = S2 + (size_t)R * PAGE;     // [32][D + 1]
  float* Vt = Kt + PAGE * (D + 1);       // [32][V]
  float* mrow = Vt + PAGE * V;           // [R] running maximum
  float* lrow = mrow + R;                // [R] running denominator
  float* corr = lrow + R;                // [R] rescale factor of the page in flight
  float* mixs = corr + R;                // [H][H]

  for (int i = tid; i < R * D; i += 256) {
    const int d = i % D, r = i / D, qi = r % BQ, g = r / BQ;
    qs[i] = qi < nq ? ldf<T>(q, ((size_t)(q0 + t0 + qi) * H + g) * D + d) : 0.f;
  }
  for (int i = tid; i < R * V; i += 256) acc[i] = 0.f;
  const bool with_sink = sink && split == 0;
  for (int i = tid; i < R; i += 256) {
    mrow[i] = with_sink ? 0.f : -1e30f;
    lrow[i] = with_sink ? 1.f : 0.f;
  }
  if (mix)
    for (int i = tid; i < H * H; i += 256) mixs[i] = ldf<T>(mix, i);

  // visible keys of the tile: [j_lo, j_hi) and the kept first ones; pages [0, p_keep) and [p_lo, p_hi), this split's
  // share of them
  const int j_hi = pos0 + nq;
  const int j_lo = window > 0 ? max(0, pos0 - window + 1) : 0;
  const int p_lo = j_lo / PAGE, p_hi = (j_hi + PAGE - 1) / PAGE;
  const int p_keep = min((max(keep, 0) + PAGE - 1) / PAGE, p_lo);
  const int n_pages = p_keep + p_hi - p_lo;
  const int per = (n_pages + nsplit - 1) / nsplit;
  const int my_lo = split * per, my_hi = min(n_pages, my_lo + per);

  for (int pi = my_lo; pi < my_hi; ++pi) {
    const int pg = pi < p_keep ? pi : p_lo + pi - p_keep;
    const size_t page = (size_t)block_tables[(size_t)b * max_pages + pg];
    const int jb = pg * PAGE;
    // ---- shaped scores of every head
    for (int c = 0; c < G; ++c) {
      __syncthreads();  // Kt free (and, at the first page, the tile set-up visible)
      const T* kp = kcache + ((page * G + c) * PAGE) * D;
      if (sizeof(T) == 2 && D % 8 == 0) {  // 16-byte loads
        for (int i = tid; i < PAGE * D / 8; i += 256) {
          const bf16x8 x = ld8(reinterpret_cast<const bf16_t*>(kp) + 8 * i);
          float* dst = Kt + (8 * i / D) * (D + 1) + (8 * i) % D;
#pragma unroll
          for (int e = 0; e < 8; ++e) dst[e] = bf2f(x[e]);
        }
      } else {
        for (int i = tid; i < PAGE * D; i += 256) Kt[(i / D) * (D + 1) + i % D] = ldf<T>(kp, i);
      }
      __syncthreads();
      for (int e = tid; e < rep * BQ * PAGE; e += 256) {
        const int kj = e % PAGE, r = e / PAGE, qi = r % BQ, g = c * rep + r / BQ;
        const float* qv = qs + ((size_t)g * BQ + qi) * D;
        const float* kv = Kt + kj * (D + 1);
        float s = 0.f;
        for (int d = 0; d < D; ++d) s += qv[d] * kv[d];
        s *= scale;
        if (softcap > 0.f) s = softcap * tanhf(s / softcap);
        if (slope_exp != 0.f) s -= exp2f(-slope_exp * (float)(g + 1) / (float)H) * (float)(pos0 + qi - (jb + kj));
        if (r1) s -= ldf<T>(r1, g) * log1pf(ldf<T>(r2, g) * (float)max(pos0 + qi - (jb + kj), 0));
        S1[((size_t)g * BQ + qi) * PAGE + kj] = s;
      }
    }
    __syncthreads();
    // ---- mix the heads, mask
    for (int e = tid; e < R * PAGE; e += 256) {
      const int kj = e % PAGE, r = e / PAGE, qi = r % BQ, h = r / BQ;
      float s;
      if (mix) {
        s = 0.f;
        for (int g = 0; g < H; ++g) s += mixs[h * H + g] * S1[((size_t)g * BQ + qi) * PAGE + kj];
      } else {
        s = S1[e];
      }
      const int dist = pos0 + qi - (jb + kj);
      const bool ok = qi < nq && dist >= 0 && (window <= 0 || dist < window || jb + kj < keep);
      S2[e] = ok ? s : -INFINITY;
    }
    __syncthreads();
    // ---- running maximum / denominator per (head, query) row: 32 lanes a row
    for (int r = tid >> 5; r < R; r += 8) {
      const float s = S2[(size_t)r * PAGE + (tid & 31)];
      float mx = s;
#pragma unroll
      for (int o = 16; o > 0; o >>= 1) mx = fmaxf(mx, __shfl_xor(mx, o, 64));
      const float m_old = mrow[r], m_new = fmaxf(m_old, mx);
      const float p = expf(s - m_new);
      float sum = p;
#pragma unroll
      for (int o = 16; o > 0; o >>= 1) sum += __shfl_xor(sum, o, 64);
      S2[(size_t)r * PAGE + (tid & 31)] = p;
      if ((tid & 31) == 0) {
        const float cf = expf(m_old - m_new);
        corr[r] = cf;
        lrow[r] = lrow[r] * cf + sum;
        mrow[r] = m_new;
      }
    }
    // ---- weights x values
    for (int c = 0; c < G; ++c) {
      __syncthreads();  // Vt free; weights and corr visible
      const T* vp = vcache + ((page * G + c) * PAGE) * V;
      if (sizeof(T) == 2 && V % 8 == 0) {
        for (int i = tid; i < PAGE * V / 8; i += 256) {
          const bf16x8 x = ld8(reinterpret_cast<const bf16_t*>(vp) + 8 * i);
          const bool live = jb + (8 * i) / V < j_hi;
#pragma unroll
          for (int e = 0; e < 8; ++e) Vt[8 * i + e] = live ? bf2f(x[e]) : 0.f;
        }
      } else {
        for (int i = tid; i < PAGE * V; i += 256) Vt[i] = (jb + i / V < j_hi) ? ldf<T>(vp, i) : 0.f;
      }
      __syncthreads();
      for (int o = tid; o < rep * BQ * V; o += 256) {
        const int v = o % V, rr = o / V;
        const int r = c * rep * BQ + rr;  // (head, query) row: heads of this group are consecutive
        const float* pw = S2 + (size_t)r * PAGE;
        float a = acc[(size_t)r * V + v] * corr[r];
#pragma unroll 8
        for (int kj = 0; kj < PAGE; ++kj) a += pw[kj] * Vt[kj * V + v];
        acc[(size_t)r * V + v] = a;
      }
    }
  }
  __syncthreads();
  for (int o = tid; o < R * V; o += 256) {
    const int v = o % V, r = o / V, qi = r % BQ, h = r / BQ;
    if (qi >= nq) continue;
    const size_t tok = (size_t)(q0 + t0 + qi);
    if (nsplit == 1) {
      const float l = lrow[r];
      float val = l > 0.f ? acc[o] / l : 0.f;
      if (gate) val /= 1.f + expf(-ldf<T>(gate, tok * gate_stride + (gate_elem ? h * V + v : h)));
      stf<T>(out, (tok * H + h) * V + v, val);
    } else {
      part_acc[((tok * nsplit + split) * H + h) * V + v] = acc[o];
      if (v == 0) {
        part_ml[((tok * nsplit + split) * H + h) * 2] = mrow[r];
        part_ml[((tok * nsplit + split) * H + h) * 2 + 1] = lrow[r];
      }
    }
  }
}

// ------------------------------------------------------------------------------------------------------------------
// Matrix-core version for bf16 prompt portions (head sizes 64 / 128). One workgroup = 16 queries x all heads (up to 16;
// without head mixing more heads are split into groups of whole key/value heads over grid z), H / HPW waves, wave w owning heads w HPW .. w HPW + HPW - 1. Per 32-key page:
//   stage   K of every key/value head -> LDS [G][32][D + 8], V transposed -> LDS [G][V][32 + 8]
//   scores  per owned head: q (registers) x K^T, bf16 MFMA 16x16x32 with fp32 accumulation; scale, cap, distance bias
//           in fp32 -> LDS SM[head][query][key] (fp32)
//   mix     fp32 MFMA 16x16x4: M [16 x 16, zero padded] x SM[all heads][query, 16 keys]; a wave takes queries
//           w, w + waves, ...; mask, running maximum / denominator per (head, query) in LDS; the weight p (fp32) goes
//           back into its 4-byte slot of SM as the pair (bf16(p), bf16(p - bf16(p)))
//   p.v     per owned head: bf16 MFMA over the (hi, lo) pairs as 32 k-slots against the value rows taken twice: the
//           product carries 16 bits of p's mantissa (the values themselves are bf16), fp32 accumulation
template <int HPW, int DK, int VT_, int MAXT>
__global__ void __launch_bounds__(MAXT) window_attn_mfma_kernel(
    const bf16_t* __restrict__ q, const bf16_t* __restrict__ kcache, const bf16_t* __restrict__ vcache,
    const int* __restrict__ block_tables, int max_pages, const int* __restrict__ cu_q,
    const int* __restrict__ ctx_len, const bf16_t* __restrict__ mix, const bf16_t* __restrict__ gate,
    int64_t gate_stride, int gate_elem, const bf16_t* __restrict__ r1, const bf16_t* __restrict__ r2,
    bf16_t* __restrict__ out, int Hall, int Gall, int H, float scale, float softcap,
    float slope_exp, int window, int keep, int sink) {
  constexpr int D = DK * 32, V = VT_ * 16, KS = D + 8, VS = PAGE + 8, SS = PAGE + 4;
  // this workgroup's heads: hbase .. hbase + H - 1 of Hall (several groups only without head mixing), and their G
  // key/value heads from c0 on
  const int rep = Hall / Gall, hbase = blockIdx.z * H, c0 = hbase / rep, G = H / rep;
  extern __shared__ __attribute__((aligned(16))) char smem[];
  unsigned* SM = reinterpret_cast<unsigned*>(smem);                      // [16][16][SS] 4-byte slots
  bf16_t* KT = reinterpret_cast<bf16_t*>(smem + 16 * 16 * SS * 4);       // [G][32][KS]
  bf16_t* VTt = KT + (size_t)G * PAGE * KS;                              // [G][V][VS]
  float* mS = reinterpret_cast<float*>(VTt + (size_t)G * V * VS);        // [16][16]
  float* lS = mS + 256;
  float* cS = lS + 256;
  float* Tm = cS + 256;                                                  // [16][16]
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, nthr = blockDim.x, NW = nthr >> 6;
  const int r16 = lane & 15, quad = lane >> 4;
  const int b = blockIdx.y;

  const int q0 = cu_q[b], qlen = cu_q[b + 1] - q0, t0 = blockIdx.x * 16;
  if (t0 >= qlen) return;
  const int nq = min(16, qlen - t0), ctx = ctx_len[b], pos0 = ctx - qlen + t0;

  for (int i = tid; i < 16 * 16 * SS; i += nthr) SM[i] = 0u;
  for (int i = tid; i < 256; i += nthr) {
    mS[i] = sink ? 0.f : -1e30f;
    lS[i] = sink ? 1.f : 0.f;
    cS[i] = 1.f;
    const int h = i >> 4, g = i & 15;
    Tm[i] = (h < H && g < H) ? (mix ? bf2f(mix[h * H + g]) : (h == g ? 1.f : 0.f)) : 0.f;
  }
  bf16x8 qf[HPW][DK];
  f32x4 acc[HPW][VT_];
  float slope[HPW], lr1[HPW], lr2[HPW];
#pragma unroll
  for (int hh = 0; hh < HPW; ++hh) {
    const int h = wave * HPW + hh;
    slope[hh] = slope_exp != 0.f ? exp2f(-slope_exp * (float)(hbase + h + 1) / (float)Hall) : 0.f;
    lr1[hh] = r1 ? bf2f(r1[hbase + h]) : 0.f;
    lr2[hh] = r1 ? bf2f(r2[hbase + h]) : 0.f;
#pragma unroll
    for (int ks = 0; ks < DK; ++ks) {
      if (r16 < nq) qf[hh][ks] = ld8(q + ((size_t)(q0 + t0 + r16) * Hall + hbase + h) * D + 32 * ks + 8 * quad);
      else qf[hh][ks] = (bf16x8){0, 0, 0, 0, 0, 0, 0, 0};
    }
#pragma unroll
    for (int vt = 0; vt < VT_; ++vt) acc[hh][vt] = (f32x4){0.f, 0.f, 0.f, 0.f};
  }
  const int j_hi = pos0 + nq;
  const int j_lo = window > 0 ? max(0, pos0 - window + 1) : 0;
  const int p_lo = j_lo / PAGE, p_hi = (j_hi + PAGE - 1) / PAGE;
  const int p_keep = min((max(keep, 0) + PAGE - 1) / PAGE, p_lo);  // pages of kept first tokens below the window's
  const float inv_cap = softcap > 0.f ? 1.f / softcap : 0.f;

  for (int pi = 0; pi < p_keep + p_hi - p_lo; ++pi) {
    const int pg = pi < p_keep ? pi : p_lo + pi - p_keep;
    const size_t page = (size_t)block_tables[(size_t)b * max_pages + pg];
    const int jb = pg * PAGE;
    __syncthreads();  // the page before is consumed (first time: the set-up above is visible)
    for (int i = tid; i < G * PAGE * (D / 8); i += nthr) {
      const int dv = i % (D / 8), key = (i / (D / 8)) % PAGE, c = i / (PAGE * (D / 8));
      st8(KT + ((size_t)c * PAGE + key) * KS + 8 * dv, ld8(kcache + ((page * Gall + c0 + c) * PAGE + key) * D + 8 * dv));
    }
    for (int i = tid; i < G * PAGE * (V / 8); i += nthr) {
      const int key = i % PAGE, vv = (i / PAGE) % (V / 8), c = i / (PAGE * (V / 8));
      bf16x8 x = ld8(vcache + ((page * Gall + c0 + c) * PAGE + key) * V + 8 * vv);
      const bool live = jb + key < j_hi;  // rows past the tile's last key may hold anything: they must not reach p.v
#pragma unroll
      for (int e = 0; e < 8; ++e) VTt[((size_t)c * V + 8 * vv + e) * VS + key] = live ? x[e] : (bf16_t)0.f;
    }
    __syncthreads();
    // ---- shaped scores of the owned heads
#pragma unroll
    for (int hh = 0; hh < HPW; ++hh) {
      const int h = wave * HPW + hh, c = h / rep;
      f32x4 c0 = {0.f, 0.f, 0.f, 0.f}, c1 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int ks = 0; ks < DK; ++ks) {
        const bf16x8 b0 = ld8(KT + ((size_t)c * PAGE + r16) * KS + 32 * ks + 8 * quad);
        const bf16x8 b1 = ld8(KT + ((size_t)c * PAGE + 16 + r16) * KS + 32 * ks + 8 * quad);
        c0 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(qf[hh][ks], b0, c0, 0, 0, 0);
        c1 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(qf[hh][ks], b1, c1, 0, 0, 0);
      }
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int qi = 4 * quad + i;
#pragma unroll
        for (int half = 0; half < 2; ++half) {
          float sc = (half ? c1[i] : c0[i]) * scale;
          if (softcap > 0.f) {
            const float e = __expf(2.f * fminf(fmaxf(sc * inv_cap, -15.f), 15.f));
            sc = softcap * ((e - 1.f) / (e + 1.f));
          }
          sc -= slope[hh] * (float)(pos0 + qi - (jb + 16 * half + r16));
          if (r1) sc -= lr1[hh] * __logf(1.f + lr2[hh] * (float)max(pos0 + qi - (jb + 16 * half + r16), 0));
          SM[((size_t)h * 16 + qi) * SS + 16 * half + r16] = __float_as_uint(sc);
        }
      }
    }
    __syncthreads();
    // ---- mix the heads (fp32 matrix cores), mask, running softmax statistics, weights back into SM
    for (int qi = wave; qi < 16; qi += NW) {
      f32x4 m0 = {0.f, 0.f, 0.f, 0.f}, m1 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int kk = 0; kk < 4; ++kk) {
        const float a = Tm[r16 * 16 + 4 * kk + quad];
        const float b0 = __uint_as_float(SM[((size_t)(4 * kk + quad) * 16 + qi) * SS + r16]);
        const float b1 = __uint_as_float(SM[((size_t)(4 * kk + quad) * 16 + qi) * SS + 16 + r16]);
        m0 = __builtin_amdgcn_mfma_f32_16x16x4f32(a, b0, m0, 0, 0, 0);
        m1 = __builtin_amdgcn_mfma_f32_16x16x4f32(a, b1, m1, 0, 0, 0);
      }
      const int d0 = pos0 + qi - (jb + r16), d1 = d0 - 16;
      const bool ok0 = qi < nq && d0 >= 0 && (window <= 0 || d0 < window || jb + r16 < keep);
      const bool ok1 = qi < nq && d1 >= 0 && (window <= 0 || d1 < window || jb + 16 + r16 < keep);
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int h = 4 * quad + i;
        const float s0 = ok0 ? m0[i] : -INFINITY, s1 = ok1 ? m1[i] : -INFINITY;
        float mx = fmaxf(s0, s1);
#pragma unroll
        for (int o = 8; o > 0; o >>= 1) mx = fmaxf(mx, __shfl_xor(mx, o, 64));
        const float m_old = mS[h * 16 + qi], m_new = fmaxf(m_old, mx);
        const float p0 = __expf(s0 - m_new), p1 = __expf(s1 - m_new);
        float sum = p0 + p1;
#pragma unroll
        for (int o = 8; o > 0; o >>= 1) sum += __shfl_xor(sum, o, 64);
        if (h < H) {
          const bf16_t h0 = f2bf(p0), h1 = f2bf(p1);
          const bf16_t l0 = f2bf(p0 - bf2f(h0)), l1 = f2bf(p1 - bf2f(h1));
          SM[((size_t)h * 16 + qi) * SS + r16] = (unsigned)__builtin_bit_cast(unsigned short, h0) |
                                                 ((unsigned)__builtin_bit_cast(unsigned short, l0) << 16);
          SM[((size_t)h * 16 + qi) * SS + 16 + r16] = (unsigned)__builtin_bit_cast(unsigned short, h1) |
                                                      ((unsigned)__builtin_bit_cast(unsigned short, l1) << 16);
          if (r16 == 0) {
            const float cf = __expf(m_old - m_new);
            cS[h * 16 + qi] = cf;
            lS[h * 16 + qi] = lS[h * 16 + qi] * cf + sum;
            mS[h * 16 + qi] = m_new;
          }
        }
      }
    }
    __syncthreads();
    // ---- weights x values of the owned heads
#pragma unroll
    for (int hh = 0; hh < HPW; ++hh) {
      const int h = wave * HPW + hh, c = h / rep;
      f32x4 cf;
#pragma unroll
      for (int i = 0; i < 4; ++i) cf[i] = cS[h * 16 + 4 * quad + i];
#pragma unroll
      for (int vt = 0; vt < VT_; ++vt) acc[hh][vt] *= cf;
#pragma unroll
      for (int kb = 0; kb < 2; ++kb) {
        const bf16x8 a = *reinterpret_cast<const bf16x8*>(SM + ((size_t)h * 16 + r16) * SS + 16 * kb + 4 * quad);
#pragma unroll
        for (int vt = 0; vt < VT_; ++vt) {
          const bf16x4 v4 =
              *reinterpret_cast<const bf16x4*>(VTt + ((size_t)c * V + 16 * vt + r16) * VS + 16 * kb + 4 * quad);
          const bf16x8 bb = {v4[0], v4[0], v4[1], v4[1], v4[2], v4[2], v4[3], v4[3]};
          acc[hh][vt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, bb, acc[hh][vt], 0, 0, 0);
        }
      }
    }
  }
  __syncthreads();
#pragma unroll
  for (int hh = 0; hh < HPW; ++hh) {
    const int h = wave * HPW + hh;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int qi = 4 * quad + i;
      if (qi >= nq) continue;
      const size_t tok = (size_t)(q0 + t0 + qi);
      const float l = lS[h * 16 + qi];
      float f = l > 0.f ? 1.f / l : 0.f;
      if (gate && !gate_elem) f /= 1.f + expf(-bf2f(gate[tok * gate_stride + hbase + h]));
#pragma unroll
      for (int vt = 0; vt < VT_; ++vt) {
        float val = acc[hh][vt][i] * f;
        if (gate && gate_elem) val /= 1.f + expf(-bf2f(gate[tok * gate_stride + (size_t)(hbase + h) * V + 16 * vt + r16]));
        out[(tok * Hall + hbase + h) * V + 16 * vt + r16] = f2bf(val);
      }
    }
  }
}

size_t mfma_lds_bytes(int G, int D, int V) {
  return (size_t)16 * 16 * (PAGE + 4) * 4 + (size_t)G * PAGE * (D + 8) * 2 + (size_t)G * V * (PAGE + 8) * 2 + 4 * 256 * 4;
}
int mfma_heads_per_wave(int H) { return (H % 4 == 0 && H >= 16) ? 4 : ((H % 2 == 0 && H >= 8) ? 2 : 1); }
// Heads per workgroup: all of them when the heads' scores are mixed; otherwise the largest group of at most 16 heads
// that holds whole key/value heads and divides the head count (0: none).
int mfma_head_group(int H, int G, bool mixed) {
  if (H < 1 || G < 1 || H % G != 0) return 0;
  if (mixed || H <= 16) return H <= 16 ? H : 0;
  const int rep = H / G;
  for (int hb = 16; hb >= 1; --hb)
    if (H % hb == 0 && hb % rep == 0) return hb;
  return 0;
}
bool mfma_usable(int H, int G, int D, int V, bool mixed) {
  if ((D != 64 && D != 128) || (V != 32 && V != 64 && V != 128)) return false;
  const int hb = mfma_head_group(H, G, mixed);
  if (hb < 1 || hb / mfma_heads_per_wave(hb) > 8) return false;
  return mfma_lds_bytes(hb / (H / G), D, V) <= 160 * 1024;
}

template <int HPW, int MAXT>
int launch_mfma(dim3 grid, int nthr, size_t lds, hipStream_t st, const bf16_t* q, const bf16_t* kc, const bf16_t* vc,
                const int* bt, int max_pages, const int* cu_q, const int* ctx_len, const bf16_t* mix,
                const bf16_t* gate, int64_t gate_stride, int gate_elem, const bf16_t* r1, const bf16_t* r2, bf16_t* out,
                int Hall, int Gall, int H, int D, int V, float scale, float softcap, float slope_exp, int window,
                int keep, int sink) {
#define MFMA_CASE(DKV, VTV)                                                                                        \
  do {                                                                                                             \
    static bool raised = false; /* once per kernel: no attribute call inside a stream capture later */            \
    if (!raised) {                                                                                                 \
      HIP_RET(hipFuncSetAttribute((const void*)window_attn_mfma_kernel<HPW, DKV, VTV, MAXT>,                       \
                                  hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024));                        \
      raised = true;                                                                                               \
    }                                                                                                              \
    hipLaunchKernelGGL((window_attn_mfma_kernel<HPW, DKV, VTV, MAXT>), grid, dim3(nthr), lds, st, q, kc, vc, bt,   \
                       max_pages, cu_q, ctx_len, mix, gate, gate_stride, gate_elem, r1, r2, out, Hall, Gall, H,    \
                       scale, softcap, slope_exp, window, keep, sink);                                             \
  } while (0)
  if (D == 64 && V == 32) MFMA_CASE(2, 2);
  else if (D == 64 && V == 64) MFMA_CASE(2, 4);
  else if (D == 64 && V == 128) MFMA_CASE(2, 8);
  else if (D == 128 && V == 32) MFMA_CASE(4, 2);
  else if (D == 128 && V == 64) MFMA_CASE(4, 4);
  else MFMA_CASE(4, 8);
#undef MFMA_CASE
  return (int)hipGetLastError();
}

// one workgroup per (token, head): thread v merges the splits' partial sums of value column v
template <typename T>
__global__ void __launch_bounds__(128) window_attn_combine_kernel(const float* __restrict__ part_acc,
                                                                   const float* __restrict__ part_ml,
                                                                   const T* __restrict__ gate, int64_t gate_stride,
                                                                   int gate_elem, T* __restrict__ out, int H, int V,
                                                                   int nsplit) {
  const size_t tok = blockIdx.x;
  const int h = blockIdx.y;
  float M = -1e30f;
  for (int s = 0; s < nsplit; ++s) M = fmaxf(M, part_ml[((tok * nsplit + s) * H + h) * 2]);
  float den = 0.f;
  for (int s = 0; s < nsplit; ++s)
    den += expf(part_ml[((tok * nsplit + s) * H + h) * 2] - M) * part_ml[((tok * nsplit + s) * H + h) * 2 + 1];
  float f = den > 0.f ? 1.f / den : 0.f;
  if (gate && !gate_elem) f /= 1.f + expf(-ldf<T>(gate, tok * gate_stride + h));
  for (int v = threadIdx.x; v < V; v += 128) {
    float num = 0.f;
    for (int s = 0; s < nsplit; ++s)
      num += expf(part_ml[((tok * nsplit + s) * H + h) * 2] - M) * part_acc[((tok * nsplit + s) * H + h) * V + v];
    num *= f;
    if (gate && gate_elem) num /= 1.f + expf(-ldf<T>(gate, tok * gate_stride + (size_t)h * V + v));
    stf<T>(out, (tok * H + h) * V + v, num);
  }
}

}  // namespace

extern "C" int areal_qk_norm_cache_write(const void* proj, int64_t row_stride, const void* qw, const void* kw,
                                         const int64_t* slots, void* q_out, void* kcache, void* vcache, int T, int H,
                                         int G, int D, int V, float eps, int dt, hipStream_t st) {
  if (T == 0) return 0;
  if (dt == 0)
    hipLaunchKernelGGL(qk_norm_cache_write_kernel<bf16_t>, dim3(T), dim3(256), 0, st, (const bf16_t*)proj, row_stride,
                       (const bf16_t*)qw, (const bf16_t*)kw, slots, (bf16_t*)q_out, (bf16_t*)kcache, (bf16_t*)vcache,
                       H, G, D, V, eps);
  else
    hipLaunchKernelGGL(qk_norm_cache_write_kernel<float>, dim3(T), dim3(256), 0, st, (const float*)proj, row_stride,
                       (const float*)qw, (const float*)kw, slots, (float*)q_out, (float*)kcache, (float*)vcache, H, G,
                       D, V, eps);
  return (int)hipGetLastError();
}

// proj rows: q heads | k heads | v heads from the pointer on. table fp32 [n_pos, R]; v_first / lam null: values as they are.
extern "C" int areal_rot_norm_cache_write(const void* proj, int64_t row_stride, const int* positions, const float* table,
                                          int n_pos, int R, const int64_t* slots, const void* v_first, int64_t vf_stride,
                                          const void* lam, void* q_out, void* kcache, void* vcache, int T, int H, int G,
                                          int D, int V, float eps, int v_transposed, int dt, hipStream_t st) {
  if (T == 0) return 0;
  if (R < 0 || R > D || R % 2 != 0 || n_pos < 1 || (v_first && !lam)) return -1;
  if (dt == 0 && D % 8 == 0 && V % 8 == 0 && D <= 512 && row_stride % 8 == 0 && ((uintptr_t)proj % 16) == 0 &&
      (!v_first || (vf_stride % 8 == 0 && ((uintptr_t)v_first % 16) == 0))) {
    const dim3 vgrid(T, (H + G + 15) / 16);
#define VEC(NVV)                                                                                                    \
  hipLaunchKernelGGL(rot_norm_cache_write_vec_kernel<NVV>, vgrid, dim3(256), 0, st, (const bf16_t*)proj, row_stride, \
                     positions, table, n_pos, R, slots, (const bf16_t*)v_first, vf_stride, (const bf16_t*)lam,       \
                     (bf16_t*)q_out, (bf16_t*)kcache, (bf16_t*)vcache, H, G, D, V, eps, v_transposed)
    if (D <= 128) VEC(1);
    else if (D <= 256) VEC(2);
    else VEC(4);
#undef VEC
    return (int)hipGetLastError();
  }
  // a head a wave: a token's heads are spread over grid y
  const dim3 grid(T, (H + G + 3) / 4);
  if (dt == 0)
    hipLaunchKernelGGL(rot_norm_cache_write_kernel<bf16_t>, grid, dim3(256), 0, st, (const bf16_t*)proj, row_stride,
                       positions, table, n_pos, R, slots, (const bf16_t*)v_first, vf_stride, (const bf16_t*)lam,
                       (bf16_t*)q_out, (bf16_t*)kcache, (bf16_t*)vcache, H, G, D, V, eps, v_transposed);
  else
    hipLaunchKernelGGL(rot_norm_cache_write_kernel<float>, grid, dim3(256), 0, st, (const float*)proj, row_stride,
                       positions, table, n_pos, R, slots, (const float*)v_first, vf_stride, (const float*)lam,
                       (float*)q_out, (float*)kcache, (float*)vcache, H, G, D, V, eps, v_transposed);
  return (int)hipGetLastError();
}

// proj rows: q heads | k heads | v heads from the pointer on; nothing is rotated or normed but (v_norm) the values
extern "C" int areal_qkv_vnorm_cache_write(const void* proj, int64_t row_stride, const int64_t* slots, void* q_out,
                                           void* kcache, void* vcache, int T, int H, int G, int D, int V, float eps,
                                           int v_norm, int v_transposed, int dt, hipStream_t st) {
  if (T == 0) return 0;
  const dim3 grid(T, (H + 2 * G + 3) / 4);
  if (dt == 0)
    hipLaunchKernelGGL(qkv_vnorm_cache_write_kernel<bf16_t>, grid, dim3(256), 0, st, (const bf16_t*)proj, row_stride,
                       slots, (bf16_t*)q_out, (bf16_t*)kcache, (bf16_t*)vcache, H, G, D, V, eps, v_norm, v_transposed);
  else
    hipLaunchKernelGGL(qkv_vnorm_cache_write_kernel<float>, grid, dim3(256), 0, st, (const float*)proj, row_stride,
                       slots, (float*)q_out, (float*)kcache, (float*)vcache, H, G, D, V, eps, v_norm, v_transposed);
  return (int)hipGetLastError();
}

// x [rows, n] contiguous <- x * sigmoid(gate), gate rows gate_stride apart
extern "C" int areal_sigmoid_gate_rows(void* x, const void* gate, int64_t gate_stride, int64_t rows, int n, int dt,
                                       hipStream_t st) {
  if (rows == 0 || n == 0) return 0;
  const int64_t total = rows * n;
  const dim3 grid((unsigned)((total + 1023) / 1024 < 4096 ? (total + 1023) / 1024 : 4096));
  if (dt == 0)
    hipLaunchKernelGGL(sigmoid_gate_rows_kernel<bf16_t>, grid, dim3(256), 0, st, (bf16_t*)x, (const bf16_t*)gate,
                       gate_stride, rows, n);
  else
    hipLaunchKernelGGL(sigmoid_gate_rows_kernel<float>, grid, dim3(256), 0, st, (float*)x, (const float*)gate,
                       gate_stride, rows, n);
  return (int)hipGetLastError();
}

// Largest query tile (16, 8, 4, 2, 1) whose LDS footprint fits the workgroup limit; 0 if even one query does not.
extern "C" int areal_window_attn_tile(int H, int G, int D, int V, int want) {
  for (int bq = want; bq >= 1; bq >>= 1) {
    AttnShape sh{H, G, D, V, bq};
    if (sh.floats() * sizeof(float) <= 156 * 1024) return bq;
  }
  return 0;
}

// B rows; row b's queries are tokens cu_q[b] .. cu_q[b+1] of q [T, H, D]; max_q = longest row. nsplit > 1 needs
// part_acc [T, nsplit, H, V] and part_ml [T, nsplit, H, 2] (fp32) and is meant for single-query rows.
extern "C" int areal_window_attn(const void* q, const void* kcache, const void* vcache, const int* block_tables,
                                 int max_pages, const int* cu_q, const int* ctx_len, const void* mix, const void* gate,
                                 int64_t gate_stride, int gate_elem, const void* r1, const void* r2, void* out,
                                 float* part_acc, float* part_ml, int B, int max_q, int T, int H, int G, int D, int V,
                                 int bq, float scale, float softcap, float slope_exp, int window, int keep, int sink,
                                 int nsplit, int dt, int matrix_cores, hipStream_t st) {
  if (B == 0 || T == 0) return 0;
  if (G <= 0 || H % G != 0 || bq <= 0 || nsplit < 1 || (r1 == nullptr) != (r2 == nullptr)) return -1;
  if (matrix_cores && dt == 0 && nsplit == 1 && max_q > 1 && mfma_usable(H, G, D, V, mix != nullptr)) {
    const int hb = mfma_head_group(H, G, mix != nullptr);
    const int hpw = mfma_heads_per_wave(hb), nthr = 64 * (hb / hpw);
    const dim3 mgrid((max_q + 15) / 16, B, H / hb);
    const size_t mlds = mfma_lds_bytes(hb / (H / G), D, V);
#define MFMA_ARGS                                                                                                  \
  mgrid, nthr, mlds, st, (const bf16_t*)q, (const bf16_t*)kcache, (const bf16_t*)vcache, block_tables, max_pages,   \
      cu_q, ctx_len, (const bf16_t*)mix, (const bf16_t*)gate, gate_stride, gate_elem, (const bf16_t*)r1,            \
      (const bf16_t*)r2, (bf16_t*)out, H, G, hb, D, V, scale, softcap, slope_exp, window, keep, sink
    if (hpw == 4) return launch_mfma<4, 256>(MFMA_ARGS);
    if (hpw == 2) return launch_mfma<2, 512>(MFMA_ARGS);
    return launch_mfma<1, 512>(MFMA_ARGS);
#undef MFMA_ARGS
  }
  AttnShape sh{H, G, D, V, bq};
  const size_t lds = sh.floats() * sizeof(float);
  if (lds > 160 * 1024) return -2;
  if (nsplit > 1 && (!part_acc || !part_ml)) return -3;
  const dim3 grid((max_q + bq - 1) / bq, B, nsplit);
#define LAUNCH(TT)                                                                                                   \
  do {                                                                                                               \
    static size_t allowed = 64 * 1024; /* raised once per size: no attribute call inside a stream capture */         \
    if (lds > allowed) {                                                                                             \
      HIP_RET(hipFuncSetAttribute((const void*)window_attn_kernel<TT>, hipFuncAttributeMaxDynamicSharedMemorySize,   \
                                  160 * 1024));                                                                      \
      allowed = 160 * 1024;                                                                                          \
    }                                                                                                                \
    hipLaunchKernelGGL(window_attn_kernel<TT>, grid, dim3(256), lds, st, (const TT*)q, (const TT*)kcache,            \
                       (const TT*)vcache, block_tables, max_pages, cu_q, ctx_len, (const TT*)mix, (const TT*)gate,   \
                       gate_stride, gate_elem, (const TT*)r1, (const TT*)r2, (TT*)out, part_acc, part_ml, sh, scale, \
                       softcap, slope_exp, window, keep, sink, nsplit);                                             \
    if (nsplit > 1)                                                                                                  \
      hipLaunchKernelGGL(window_attn_combine_kernel<TT>, dim3(T, H), dim3(128), 0, st, part_acc, part_ml,           \
                         (const TT*)gate, gate_stride, gate_elem, (TT*)out, H, V, nsplit);                          \
  } while (0)
  if (dt == 0) LAUNCH(bf16_t);
  else LAUNCH(float);
#undef LAUNCH
  return (int)hipGetLastError();
}
