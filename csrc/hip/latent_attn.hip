// Attention through a shared low-rank latent over a paged cache of [c | r] rows (c: R latent numbers, r: P rotary
// key numbers shared by all heads; token-major pages of 32).
//
//   latent_prep   per token: RMS norm (times weight) of the query latent -> cq, of the key/value latent -> cache c;
//                 the rotary key part rotated at the token's position -> cache r
//   latent_attn   s_h(i, j) = scale * (q~_h(i) . c(j) + rot_i(q^r_h(i)) . r(j)),  visible: 0 <= i - j < window
//                 o~_h(i)   = sum_j softmax_j(s_h(i, .)) c(j)   [* sigmoid(gate_h(i))]
//                 q~ are the queries already carried into latent space (absorbed key expansion); the rotary query
//                 part arrives unrotated (the last P entries of every head of q) and is rotated here.
//
// All heads read the same keys, and the values are the first R entries of the keys: a workgroup owns a tile of BQ
// queries x a group of HG heads, stages each 32-key page ONCE in LDS and uses it for both products. Scores, weights
// and the accumulation are fp32 whatever the storage type T (bf16 / fp32).
//
// The same kernel serves prompt portions (grid x = query tiles x head groups, y = rows of the batch) and decoding
// (BQ = 1, grid z = splits of the visible key range whose partial results `latent_attn_combine` merges).
// Queries of row b are the LAST cu_q[b+1] - cu_q[b] positions of its context of ctx_len[b] tokens.
// Rotation: pairs (i, i + P/2), or (`neighbours`) pairs (2i, 2i + 1) of the projection's columns; table [n_pos][P] =
// cos | sin of position * frequency. Rotated neighbour pairs are stored (cache) and scored (query) in the order
// first members | second members: a dot product does not see a permutation applied to both of its sides.
// `sink` (one logit per head, or null): a key without a value whose exp(sink_h) counts once in the denominator.
#include "common.hpp"

namespace {

constexpr int PAGE = 32;

template <typename T> DEVINL float ldf(const T* p, size_t i);
template <> DEVINL float ldf<bf16_t>(const bf16_t* p, size_t i) { return bf2f(p[i]); }
template <> DEVINL float ldf<float>(const float* p, size_t i) { return p[i]; }
template <typename T> DEVINL void stf(T* p, size_t i, float v);
template <> DEVINL void stf<bf16_t>(bf16_t* p, size_t i, float v) { p[i] = f2bf(v); }
template <> DEVINL void stf<float>(float* p, size_t i, float v) { p[i] = v; }

// One workgroup per token; wave 0: query latent, wave 1: key/value latent, wave 2: rotary key part.
template <typename T>
__global__ void __launch_bounds__(256) latent_prep_kernel(
    const T* __restrict__ proj, int64_t row_stride, const T* __restrict__ qw, const T* __restrict__ cw,
    const int* __restrict__ positions, const int64_t* __restrict__ slots, const float* __restrict__ table, int n_pos,
    T* __restrict__ cq, T* __restrict__ cache, int Q, int R, int P, float eps, int neighbours) {
  const int t = blockIdx.x, lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const T* row = proj + (size_t)t * row_stride;
  const int64_t slot = slots[t];
  T* dst = slot >= 0 ? cache + (size_t)slot * (R + P) : nullptr;  // slot = page * 32 + offset
  if (wave == 0) {
    if (Q <= 0) return;
    float ss = 0.f;
    for (int i = lane; i < Q; i += 64) {
      const float x = ldf<T>(row, i);
      ss += x * x;
    }
    const float r = 1.f / sqrtf(wave_sum(ss) / (float)Q + eps);
    for (int i = lane; i < Q; i += 64) stf<T>(cq, (size_t)t * Q + i, ldf<T>(row, i) * r * ldf<T>(qw, i));
  } else if (wave == 1) {
    if (!dst) return;
    float ss = 0.f;
    for (int i = lane; i < R; i += 64) {
      const float x = ldf<T>(row, Q + i);
      ss += x * x;
    }
    const float r = 1.f / sqrtf(wave_sum(ss) / (float)R + eps);
    for (int i = lane; i < R; i += 64) stf<T>(dst, i, ldf<T>(row, Q + i) * r * ldf<T>(cw, i));
  } else if (wave == 2) {
    if (!dst) return;
    const int pos = min(max(positions[t], 0), n_pos - 1);
    const float* cs = table + (size_t)pos * P;
    const int half = P / 2;
    for (int i = lane; i < half; i += 64) {
      const float u = ldf<T>(row, Q + R + (neighbours ? 2 * i : i));
      const float v = ldf<T>(row, Q + R + (neighbours ? 2 * i + 1 : half + i));
      const float c = cs[i], s = cs[half + i];
      stf<T>(dst, R + i, u * c - v * s);
      stf<T>(dst, R + half + i, v * c + u * s);
    }
  }
}

struct LatentShape {
  int H, HG, D, P, R, BQ;
  __host__ __device__ int rows() const { return HG * BQ; }
  __host__ __device__ int ks() const { return R + P + 1; }  // padded key row: conflict-free column walks
  __host__ __device__ size_t floats() const {
    return (size_t)rows() * (R + P) + (size_t)rows() * R + (size_t)rows() * PAGE + (size_t)PAGE * ks() + 3 * (size_t)rows();
  }
};

template <typename T>
__global__ void __launch_bounds__(256) latent_attn_kernel(
    const T* __restrict__ q, int64_t q_stride, const T* __restrict__ q_lat, const T* __restrict__ cache,
    const int* __restrict__ block_tables, int max_pages, const int* __restrict__ cu_q,
    const int* __restrict__ ctx_len, const float* __restrict__ table, int n_pos, int neighbours,
    const T* __restrict__ sink, const T* __restrict__ gate,
    int64_t gate_stride, T* __restrict__ out, float* __restrict__ part_acc, float* __restrict__ part_ml,
    LatentShape sh, float scale, int window, int nsplit) {
  extern __shared__ float lds[];
  const int H = sh.H, HG = sh.HG, D = sh.D, P = sh.P, R = sh.R, BQ = sh.BQ, KW = R + P, KS = sh.ks();
  const int tid = threadIdx.x;
  const int n_groups = (H + HG - 1) / HG;
  const int tile = blockIdx.x / n_groups, h0 = (blockIdx.x % n_groups) * HG;
  const int nh = min(HG, H - h0);
  const int b = blockIdx.y, split = blockIdx.z;
  const int q0 = cu_q[b], qlen = cu_q[b + 1] - q0;
  const int t0 = tile * BQ;
  if (t0 >= qlen) return;
  const int nq = min(BQ, qlen - t0);
  const int ctx = ctx_len[b];
  const int pos0 = ctx - qlen + t0;  // position of the tile's first query
  const int NR = HG * BQ;            // (head, query) rows: r = hh * BQ + qi
  float* qs = lds;                        // [NR][KW]
  float* acc = qs + (size_t)NR * KW;      // [NR][R]
  float* S = acc + (size_t)NR * R;        // [NR][32]
  float* Kt = S + (size_t)NR * PAGE;      // [32][KS]
  float* mrow = Kt + (size_t)PAGE * KS;   // [NR]
  float* lrow = mrow + NR;
  float* corr = lrow + NR;

  const int half = P / 2;
  for (int i = tid; i < NR * KW; i += 256) {
    const int d = i % KW, r = i / KW, qi = r % BQ, hh = r / BQ;
    float v = 0.f;
    if (qi < nq && hh < nh) {
      const size_t tok = (size_t)(q0 + t0 + qi);
      if (d < R) {
        v = ldf<T>(q_lat, (tok * H + h0 + hh) * R + d);
      } else {
        const int e = d - R, pi = e < half ? e : e - half;
        const T* qr = q + tok * q_stride + (size_t)(h0 + hh) * (D + P) + D;
        const float* cs = table + (size_t)min(max(pos0 + qi, 0), n_pos - 1) * P;
        const float u = ldf<T>(qr, neighbours ? 2 * pi : pi), w = ldf<T>(qr, neighbours ? 2 * pi + 1 : half + pi);
        const float c = cs[pi], s = cs[half + pi];
        v = e < half ? u * c - w * s : w * c + u * s;
      }
    }
    qs[i] = v;
  }
  for (int i = tid; i < NR * R; i += 256) acc[i] = 0.f;
  for (int i = tid; i < NR; i += 256) {
    const int hh = i / BQ;
    const bool with_sink = sink && split == 0 && hh < nh;
    mrow[i] = with_sink ? ldf<T>(sink, h0 + hh) : -1e30f;
    lrow[i] = with_sink ? 1.f : 0.f;
  }

  // visible keys of the tile: [j_lo, j_hi); pages [p_lo, p_hi), this split's share of them
  const int j_hi = pos0 + nq;
  const int j_lo = window > 0 ? max(0, pos0 - window + 1) : 0;
  const int p_lo = j_lo / PAGE, p_hi = (j_hi + PAGE - 1) / PAGE;
  const int per = (p_hi - p_lo + nsplit - 1) / nsplit;
  const int my_lo = p_lo + split * per, my_hi = min(p_hi, my_lo + per);

  for (int pg = my_lo; pg < my_hi; ++pg) {
    const size_t page = (size_t)block_tables[(size_t)b * max_pages + pg];
    const int jb = pg * PAGE;
    __syncthreads();  // Kt free (and, at the first page, the tile set-up visible)
    const T* kp = cache + page * PAGE * KW;
    if (sizeof(T) == 2 && KW % 8 == 0) {  // 16-byte loads
      for (int i = tid; i < PAGE * KW / 8; i += 256) {
        const int key = (8 * i) / KW;
        const bf16x8 x = ld8(reinterpret_cast<const bf16_t*>(kp) + 8 * i);
        float* dst = Kt + key * KS + (8 * i) % KW;
        const bool live = jb + key < j_hi;  // rows past the last key may hold anything
#pragma unroll
        for (int e = 0; e < 8; ++e) dst[e] = live ? bf2f(x[e]) : 0.f;
      }
    } else {
      for (int i = tid; i < PAGE * KW; i += 256)
        Kt[(i / KW) * KS + i % KW] = (jb + i / KW < j_hi) ? ldf<T>(kp, i) : 0.f;
    }
    __syncthreads();
    // ---- scores
    for (int e = tid; e < NR * PAGE; e += 256) {
      const int kj = e % PAGE, r = e / PAGE, qi = r % BQ, hh = r / BQ;
      const float* qv = qs + (size_t)r * KW;
      const float* kv = Kt + kj * KS;
      float s = 0.f;
      for (int d = 0; d < KW; ++d) s += qv[d] * kv[d];
      const int dist = pos0 + qi - (jb + kj);
      const bool ok = qi < nq && hh < nh && dist >= 0 && (window <= 0 || dist < window);
      S[e] = ok ? s * scale : -INFINITY;
    }
    __syncthreads();
    // ---- running maximum / denominator per (head, query) row: 32 lanes a row
    for (int r = tid >> 5; r < NR; r += 8) {
      const float s = S[(size_t)r * PAGE + (tid & 31)];
      float mx = s;
#pragma unroll
      for (int o = 16; o > 0; o >>= 1) mx = fmaxf(mx, __shfl_xor(mx, o, 64));
      const float m_old = mrow[r], m_new = fmaxf(m_old, mx);
      const float p = expf(s - m_new);
      float sum = p;
#pragma unroll
      for (int o = 16; o > 0; o >>= 1) sum += __shfl_xor(sum, o, 64);
      S[(size_t)r * PAGE + (tid & 31)] = p;
      if ((tid & 31) == 0) {
        corr[r] = expf(m_old - m_new);
        lrow[r] = lrow[r] * corr[r] + sum;
        mrow[r] = m_new;
      }
    }
    __syncthreads();
    // ---- weights x latents (the first R entries of the staged keys)
    for (int o = tid; o < NR * R; o += 256) {
      const int v = o % R, r = o / R;
      const float* pw = S + (size_t)r * PAGE;
      float a = acc[o] * corr[r];
#pragma unroll 8
      for (int kj = 0; kj < PAGE; ++kj) a += pw[kj] * Kt[kj * KS + v];
      acc[o] = a;
    }
  }
  __syncthreads();
  for (int o = tid; o < NR * R; o += 256) {
    const int v = o % R, r = o / R, qi = r % BQ, hh = r / BQ;
    if (qi >= nq || hh >= nh) continue;
    const size_t tok = (size_t)(q0 + t0 + qi);
    const int h = h0 + hh;
    if (nsplit == 1) {
      const float l = lrow[r];
      float val = l > 0.f ? acc[o] / l : 0.f;
      if (gate) val /= 1.f + expf(-ldf<T>(gate, tok * gate_stride + h));
      stf<T>(out, (tok * H + h) * R + v, val);
    } else {
      part_acc[((tok * nsplit + split) * H + h) * R + v] = acc[o];
      if (v == 0) {
        part_ml[((tok * nsplit + split) * H + h) * 2] = mrow[r];
        part_ml[((tok * nsplit + split) * H + h) * 2 + 1] = lrow[r];
      }
    }
  }
}

// ------------------------------------------------------------------------------------------------------------------
// Matrix-core version for bf16. The 16 rows of a matrix-core tile are
//   prompt portions (DEC = false): 16 queries of ONE head; a workgroup = 16 queries x a group of heads;
//   decoding        (DEC = true):  the 16 heads of a head group of ONE query; grid z = splits of the key range.
// RS waves share a tile's rows: each computes the scores (cheap beside p.c) and owns R / RS of the output columns,
// which keeps the fp32 accumulators of large latents in registers. Per 32-key page:
//   stage   the page's [c | r] rows -> LDS KT [32][KW + 8] (bf16), and the latent part transposed -> VT [R][32 + 4]
//   scores  rows (registers: absorbed query | rotated rotary part, bf16) x KT^T, bf16 MFMA 16x16x32 with fp32
//           accumulation; scale and mask in fp32; running maximum / denominator of the 16 rows in registers (a row's
//           keys sit in the 16 lanes of one quad); the weight p (fp32) goes into the wave's own LDS tile as the pair
//           (bf16(p), bf16(p - bf16(p)))
//   p.c     bf16 MFMA over the (hi, lo) pairs as 32 k-slots against the latent columns taken twice: the product
//           carries 16 bits of p's mantissa (the latents themselves are bf16), fp32 accumulation in registers
// KW32 = (R + P) / 32 k-steps of the scores, R16 = R / 16 output tiles.
template <int KW32, int R16, int RS, bool DEC>
__global__ void __launch_bounds__(DEC ? 256 : 512) latent_attn_mfma_kernel(
    const bf16_t* __restrict__ q, int64_t q_stride, const bf16_t* __restrict__ q_lat, const bf16_t* __restrict__ cache,
    const int* __restrict__ block_tables, int max_pages, const int* __restrict__ cu_q,
    const int* __restrict__ ctx_len, const float* __restrict__ table, int n_pos, int neighbours,
    const bf16_t* __restrict__ sink, const bf16_t* __restrict__ gate,
    int64_t gate_stride, bf16_t* __restrict__ out, float* __restrict__ part_acc, float* __restrict__ part_ml, int H,
    int HG, int D, float scale, int window, int nsplit) {
  constexpr int KW = KW32 * 32, R = R16 * 16, P = KW - R, KS = KW + 8, VS = PAGE + 4, SS = PAGE + 4, NT = R16 / RS;
  constexpr int NB = (!DEC && KW32 >= 18) ? 3 : 4;  // the largest prompt instance has no registers to spare
  static_assert(R16 % RS == 0, "output tiles split evenly over the waves of a row tile");
  extern __shared__ __attribute__((aligned(16))) char smem[];
  bf16_t* KT = reinterpret_cast<bf16_t*>(smem);                  // [32][KS]
  bf16_t* VT = KT + (size_t)PAGE * KS;                           // [R][VS]
  unsigned* PM = reinterpret_cast<unsigned*>(VT + (size_t)R * VS);  // [waves][16][SS] 4-byte slots
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, nthr = blockDim.x;
  const int r16 = lane & 15, quad = lane >> 4;
  const int part = wave % RS, slot = wave / RS;
  const int b = blockIdx.y, split = DEC ? blockIdx.z : 0;
  const int q0 = cu_q[b], qlen = cu_q[b + 1] - q0, ctx = ctx_len[b];
  // rows of this wave's tile: (token, head) of row r, how many rows are real, position of row r's query
  int t0, hbase, nrows, pos0;
  if (DEC) {
    if (qlen < 1) return;
    t0 = 0;
    hbase = blockIdx.x * 16;
    nrows = min(16, H - hbase);
    pos0 = ctx - 1;
  } else {
    const int n_groups = (H + HG - 1) / HG;
    t0 = (blockIdx.x / n_groups) * 16;
    if (t0 >= qlen) return;
    hbase = (blockIdx.x % n_groups) * HG + slot;
    nrows = hbase < H ? min(16, qlen - t0) : 0;  // waves past the last head only help staging
    pos0 = ctx - qlen + t0;
  }
  auto row_tok = [&](int r) -> size_t { return (size_t)(q0 + (DEC ? 0 : t0 + r)); };
  auto row_head = [&](int r) -> int { return DEC ? hbase + r : hbase; };
  auto row_pos = [&](int r) -> int { return DEC ? pos0 : pos0 + r; };
  // decoding: the four waves of the tile compute the same weights; one tile holds them (written by the first wave)
  unsigned* pm = PM + (size_t)(DEC ? 0 : wave) * 16 * SS;

  bf16x8 qf[KW32];
  f32x4 acc[NT];
  float mrow[4], lrow[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int r = 4 * quad + i;
    const bool with_sink = sink && split == 0 && r < nrows;
    mrow[i] = with_sink ? bf2f(sink[row_head(r)]) : -1e30f;
    lrow[i] = with_sink ? 1.f : 0.f;
  }
#pragma unroll
  for (int vt = 0; vt < NT; ++vt) acc[vt] = (f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int ks = 0; ks < KW32; ++ks) {
    qf[ks] = (bf16x8){0, 0, 0, 0, 0, 0, 0, 0};
    if (r16 < nrows) {
      const size_t tok = row_tok(r16);
      const int h = row_head(r16), d = 32 * ks + 8 * quad;
      if (d < R) {
        qf[ks] = ld8(q_lat + (tok * H + h) * R + d);
      } else {  // rotary part: entry e pairs with e +- P/2
        constexpr int half = P / 2;
        const int e = d - R, pi = e < half ? e : e - half;
        const bf16_t* qr = q + tok * q_stride + (size_t)h * (D + P) + D;
        bf16x8 u, w;
        if (neighbours) {  // 16 consecutive columns hold the 8 pairs
          const bf16x8 x0 = ld8(qr + 2 * pi), x1 = ld8(qr + 2 * pi + 8);
          u = (bf16x8){x0[0], x0[2], x0[4], x0[6], x1[0], x1[2], x1[4], x1[6]};
          w = (bf16x8){x0[1], x0[3], x0[5], x0[7], x1[1], x1[3], x1[5], x1[7]};
        } else {
          u = ld8(qr + pi);
          w = ld8(qr + half + pi);
        }
        const float* cs = table + (size_t)min(max(row_pos(r16), 0), n_pos - 1) * P;
#pragma unroll
        for (int k = 0; k < 8; ++k) {
          const float c = cs[pi + k], sn = cs[half + pi + k], uu = bf2f(u[k]), ww = bf2f(w[k]);
          qf[ks][k] = f2bf(e < half ? uu * c - ww * sn : ww * c + uu * sn);
        }
      }
    }
  }
  // visible keys of the tile: [j_lo, j_hi); pages [p_lo, p_hi), this split's share of them
  const int j_hi = DEC ? ctx : pos0 + min(16, qlen - t0);
  const int j_lo = window > 0 ? max(0, pos0 - window + 1) : 0;
  const int p_lo = j_lo / PAGE, p_hi = (j_hi + PAGE - 1) / PAGE;
  const int per = (p_hi - p_lo + nsplit - 1) / nsplit;
  const int my_lo = p_lo + split * per, my_hi = min(p_hi, my_lo + per);

  // Decoding (256 threads): the NEXT page's rows are fetched into registers while this page is worked on, and its
  // page number one step earlier still, so a workgroup's walk over its pages is not a chain of memory latencies.
  constexpr int CH = PAGE * (KW / 8), NL = (CH + 255) / 256;
  bf16x8 pre[DEC ? NL : 1];
  int page_next = 0;
  auto fetch = [&](int page) {
    const bf16_t* kp = cache + (size_t)page * PAGE * KW;
#pragma unroll
    for (int u = 0; u < NL; ++u) {
      const int i = tid + u * 256;
      if (i < CH) pre[u] = ld8(kp + (size_t)(i / (KW / 8)) * KW + 8 * (i % (KW / 8)));
    }
  };
  if (DEC && my_lo < my_hi) {
    fetch(block_tables[(size_t)b * max_pages + my_lo]);
    if (my_lo + 1 < my_hi) page_next = block_tables[(size_t)b * max_pages + my_lo + 1];
  }
  for (int pg = my_lo; pg < my_hi; ++pg) {
    const int jb = pg * PAGE;
    __syncthreads();  // the page before is consumed
    if (DEC) {
#pragma unroll
      for (int u = 0; u < NL; ++u) {
        const int i = tid + u * 256;
        if (i < CH) {
          const int dv = i % (KW / 8), key = i / (KW / 8);
          if (jb + key >= j_hi) pre[u] = (bf16x8){0, 0, 0, 0, 0, 0, 0, 0};  // rows past the last key may hold anything
          st8(KT + (size_t)key * KS + 8 * dv, pre[u]);
        }
      }
      if (pg + 1 < my_hi) {
        fetch(page_next);
        if (pg + 2 < my_hi) page_next = block_tables[(size_t)b * max_pages + pg + 2];
      }
    } else {
      const bf16_t* kp = cache + (size_t)block_tables[(size_t)b * max_pages + pg] * PAGE * KW;
      // NB 16-byte loads of a thread are in flight before the first goes to LDS
      for (int i0 = tid; i0 < CH; i0 += NB * nthr) {
        bf16x8 x[NB];
#pragma unroll
        for (int u = 0; u < NB; ++u) {
          const int i = i0 + u * nthr;
          if (i < CH) x[u] = ld8(kp + (size_t)(i / (KW / 8)) * KW + 8 * (i % (KW / 8)));
        }
#pragma unroll
        for (int u = 0; u < NB; ++u) {
          const int i = i0 + u * nthr;
          if (i < CH) {
            const int dv = i % (KW / 8), key = i / (KW / 8);
            if (jb + key >= j_hi) x[u] = (bf16x8){0, 0, 0, 0, 0, 0, 0, 0};  // rows past the last key may hold anything
            st8(KT + (size_t)key * KS + 8 * dv, x[u]);
          }
        }
      }
    }
    __syncthreads();
    // the latent part once more, transposed, for p.c: a thread takes two neighbouring keys and 8 columns and stores
    // 4-byte key pairs; consecutive lanes take consecutive key pairs, so a wave's stores spread over the banks
    // (walking the columns instead puts a whole wave on one bank)
    for (int i = tid; i < (PAGE / 2) * (R / 8); i += nthr) {
      const int kp2 = i % (PAGE / 2), dv = i / (PAGE / 2);
      const bf16x8 x0 = ld8(KT + (size_t)(2 * kp2) * KS + 8 * dv), x1 = ld8(KT + (size_t)(2 * kp2 + 1) * KS + 8 * dv);
#pragma unroll
      for (int e = 0; e < 8; ++e)
        *reinterpret_cast<bf16x2*>(VT + (size_t)(8 * dv + e) * VS + 2 * kp2) = (bf16x2){x0[e], x1[e]};
    }
    if (nrows > 0) {
      f32x4 c0 = {0.f, 0.f, 0.f, 0.f}, c1 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int ks = 0; ks < KW32; ++ks) {
        const bf16x8 b0 = ld8(KT + (size_t)r16 * KS + 32 * ks + 8 * quad);
        const bf16x8 b1 = ld8(KT + (size_t)(16 + r16) * KS + 32 * ks + 8 * quad);
        c0 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(qf[ks], b0, c0, 0, 0, 0);
        c1 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(qf[ks], b1, c1, 0, 0, 0);
      }
      f32x4 cf;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int r = 4 * quad + i;
        const int d0 = row_pos(r) - (jb + r16), d1 = d0 - 16;
        const bool ok0 = r < nrows && d0 >= 0 && (window <= 0 || d0 < window);
        const bool ok1 = r < nrows && d1 >= 0 && (window <= 0 || d1 < window);
        const float s0 = ok0 ? c0[i] * scale : -INFINITY, s1 = ok1 ? c1[i] * scale : -INFINITY;
        float mx = fmaxf(s0, s1);
#pragma unroll
        for (int o = 8; o > 0; o >>= 1) mx = fmaxf(mx, __shfl_xor(mx, o, 64));
        const float m_new = fmaxf(mrow[i], mx);
        const float p0 = __expf(s0 - m_new), p1 = __expf(s1 - m_new);
        float sum = p0 + p1;
#pragma unroll
        for (int o = 8; o > 0; o >>= 1) sum += __shfl_xor(sum, o, 64);
        cf[i] = __expf(mrow[i] - m_new);
        lrow[i] = lrow[i] * cf[i] + sum;
        mrow[i] = m_new;
        if (!DEC || part == 0) {
          const bf16_t h0 = f2bf(p0), h1 = f2bf(p1);
          const bf16_t l0 = f2bf(p0 - bf2f(h0)), l1 = f2bf(p1 - bf2f(h1));
          pm[r * SS + r16] = (unsigned)__builtin_bit_cast(unsigned short, h0) |
                             ((unsigned)__builtin_bit_cast(unsigned short, l0) << 16);
          pm[r * SS + 16 + r16] = (unsigned)__builtin_bit_cast(unsigned short, h1) |
                                  ((unsigned)__builtin_bit_cast(unsigned short, l1) << 16);
        }
      }
#pragma unroll
      for (int vt = 0; vt < NT; ++vt) acc[vt] *= cf;
    }
    __syncthreads();  // the wave's weights are in its tile
    if (nrows > 0) {
#pragma unroll
      for (int kb = 0; kb < 2; ++kb) {
        const bf16x8 a = *reinterpret_cast<const bf16x8*>(pm + r16 * SS + 16 * kb + 4 * quad);
#pragma unroll
        for (int vt = 0; vt < NT; ++vt) {
          const bf16x4 v4 = *reinterpret_cast<const bf16x4*>(VT + (size_t)(16 * (part * NT + vt) + r16) * VS + 16 * kb +
                                                             4 * quad);
          const bf16x8 bb = {v4[0], v4[0], v4[1], v4[1], v4[2], v4[2], v4[3], v4[3]};
          acc[vt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, bb, acc[vt], 0, 0, 0);
        }
      }
    }
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int r = 4 * quad + i;
    if (r >= nrows) continue;
    const size_t tok = row_tok(r);
    const int h = row_head(r);
    if (!DEC || nsplit == 1) {
      float f = lrow[i] > 0.f ? 1.f / lrow[i] : 0.f;
      if (gate) f /= 1.f + expf(-bf2f(gate[tok * gate_stride + h]));
#pragma unroll
      for (int vt = 0; vt < NT; ++vt) out[(tok * H + h) * R + 16 * (part * NT + vt) + r16] = f2bf(acc[vt][i] * f);
    } else {
      float* pa = part_acc + ((tok * nsplit + split) * H + h) * (size_t)R;
#pragma unroll
      for (int vt = 0; vt < NT; ++vt) pa[16 * (part * NT + vt) + r16] = acc[vt][i];
      if (part == 0 && r16 == 0) {
        part_ml[((tok * nsplit + split) * H + h) * 2] = mrow[i];
        part_ml[((tok * nsplit + split) * H + h) * 2 + 1] = lrow[i];
      }
    }
  }
}

size_t mfma_lds_bytes(int R, int P, int waves) {
  return (size_t)PAGE * (R + P + 8) * 2 + (size_t)R * (PAGE + 4) * 2 + (size_t)waves * 16 * (PAGE + 4) * 4;
}

// Shapes the matrix-core kernel is instantiated for: (latent size, rotary size), unrotated key size D.
bool mfma_usable(int R, int P, int D, int64_t q_stride) {
  if (D % 8 != 0 || q_stride % 8 != 0) return false;  // 16-byte loads of the rotary query part
  return (R == 512 && P == 64) || (R == 256 && (P == 64 || P == 32)) || (R == 128 && (P == 64 || P == 32)) ||
         (R == 64 && (P == 64 || P == 32));
}

struct MfmaArgs {
  const bf16_t *q, *q_lat, *cache;
  int64_t q_stride;
  int neighbours;
  const bf16_t* sink;
  const int* bt;
  int max_pages;
  const int *cu_q, *ctx_len;
  const float* table;
  int n_pos;
  const bf16_t* gate;
  int64_t gate_stride;
  bf16_t* out;
  float *part_acc, *part_ml;
  int H, D;
  float scale;
  int window, nsplit;
};

template <int KW32, int R16, int RS, bool DEC>
int launch_mfma(dim3 grid, int nthr, int hg, hipStream_t st, const MfmaArgs& a) {
  static bool raised = false;  // once per kernel: no attribute call inside a stream capture later
  if (!raised) {
    HIP_RET(hipFuncSetAttribute((const void*)latent_attn_mfma_kernel<KW32, R16, RS, DEC>,
                                hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024));
    raised = true;
  }
  const size_t lds = mfma_lds_bytes(R16 * 16, KW32 * 32 - R16 * 16, DEC ? 1 : nthr / 64);
  hipLaunchKernelGGL((latent_attn_mfma_kernel<KW32, R16, RS, DEC>), grid, dim3(nthr), lds, st, a.q, a.q_stride, a.q_lat,
                     a.cache, a.bt, a.max_pages, a.cu_q, a.ctx_len, a.table, a.n_pos, a.neighbours, a.sink, a.gate,
                     a.gate_stride, a.out, a.part_acc,
                     a.part_ml, a.H, hg, a.D, a.scale, a.window, a.nsplit);
  return (int)hipGetLastError();
}

// Prompt portions: RS waves per head (2 for the largest latent, so that the accumulators stay in registers), up to
// 8 waves a workgroup. Decoding: 4 waves on the 16 heads of a head group.
template <bool DEC>
int dispatch_mfma(int R, int P, int B, int max_q, hipStream_t st, const MfmaArgs& a) {
#define GO(KW32, R16, RS)                                                                      \
  do {                                                                                         \
    if (DEC) {                                                                                 \
      const dim3 grid((a.H + 15) / 16, B, a.nsplit);                                           \
      return launch_mfma<KW32, R16, 4, true>(grid, 256, 16, st, a);                            \
    }                                                                                          \
    const int hg = a.H < 8 / RS ? a.H : 8 / RS, n_groups = (a.H + hg - 1) / hg;                \
    const dim3 grid(((max_q + 15) / 16) * n_groups, B, 1);                                     \
    return launch_mfma<KW32, R16, RS, false>(grid, 64 * hg * RS, hg, st, a);                   \
  } while (0)
  if (R == 512) GO(18, 32, 2);
  if (R == 256 && P == 64) GO(10, 16, 1);
  if (R == 256) GO(9, 16, 1);
  if (R == 128 && P == 64) GO(6, 8, 1);
  if (R == 128) GO(5, 8, 1);
  if (P == 64) GO(4, 4, 1);
  GO(3, 4, 1);
#undef GO
}

// Merge of the key-range splits of one (token, head): grid (T, H). The splits' weights exp(m_s - m) (times gate / l)
// are formed once in LDS; every thread then sums its columns over the splits with independent loads.
template <typename T>
__global__ void __launch_bounds__(128) latent_attn_combine_kernel(const float* __restrict__ part_acc,
                                                                  const float* __restrict__ part_ml,
                                                                  const T* __restrict__ gate, int64_t gate_stride,
                                                                  T* __restrict__ out, int H, int R, int nsplit) {
  __shared__ float wsp[64];  // nsplit <= 64
  const size_t tok = blockIdx.x;
  const int h = blockIdx.y;
  if (threadIdx.x < 64) {
    const int s = threadIdx.x;
    const float ms = s < nsplit ? part_ml[((tok * nsplit + s) * H + h) * 2] : -1e30f;
    const float ls = s < nsplit ? part_ml[((tok * nsplit + s) * H + h) * 2 + 1] : 0.f;
    const float m = wave_max(ms);
    const float w = s < nsplit ? expf(ms - m) : 0.f;
    const float l = wave_sum(ls * w);
    float g = 1.f;
    if (gate) g = 1.f / (1.f + expf(-ldf<T>(gate, tok * gate_stride + h)));
    wsp[s] = l > 0.f ? w * g / l : 0.f;
  }
  __syncthreads();
  const float* base = part_acc + (tok * nsplit * H + h) * (size_t)R;
  const size_t step = (size_t)H * R;
  for (int v = threadIdx.x; v < R; v += 128) {
    float a = 0.f;
#pragma unroll 4
    for (int s = 0; s < nsplit; ++s) a += wsp[s] * base[s * step + v];
    stf<T>(out, (tok * H + h) * R + v, a);
  }
}

// Query tile and head group of a launch: the largest tile (up to `want` queries) x group that fits the LDS limit,
// preferring whole-head launches (the staged keys are shared by all heads of the group).
bool pick_shape(int H, int D, int P, int R, int want, LatentShape* out) {
  for (int hg = H; hg >= 1; hg = (hg + 1) / 2) {
    for (int bq = want; bq >= 1; bq >>= 1) {
      LatentShape sh{H, hg, D, P, R, bq};
      if (sh.floats() * sizeof(float) <= 156 * 1024) {
        *out = sh;
        return true;
      }
    }
    if (hg == 1) break;
  }
  return false;
}

}  // namespace

extern "C" int areal_latent_prep(const void* proj, int64_t row_stride, const void* qw, const void* cw,
                                 const int* positions, const int64_t* slots, const float* table, int n_pos, void* cq,
                                 void* cache, int T, int Q, int R, int P, float eps, int neighbours, int dt,
                                 hipStream_t st) {
  if (T == 0) return 0;
  if (P % 2 || n_pos < 1) return -1;
  if (dt == 0)
    hipLaunchKernelGGL(latent_prep_kernel<bf16_t>, dim3(T), dim3(256), 0, st, (const bf16_t*)proj, row_stride,
                       (const bf16_t*)qw, (const bf16_t*)cw, positions, slots, table, n_pos, (bf16_t*)cq,
                       (bf16_t*)cache, Q, R, P, eps, neighbours);
  else
    hipLaunchKernelGGL(latent_prep_kernel<float>, dim3(T), dim3(256), 0, st, (const float*)proj, row_stride,
                       (const float*)qw, (const float*)cw, positions, slots, table, n_pos, (float*)cq, (float*)cache,
                       Q, R, P, eps, neighbours);
  return (int)hipGetLastError();
}

// B rows; row b's queries are tokens cu_q[b] .. cu_q[b+1]; max_q = longest row. nsplit > 1 needs part_acc
// [T, nsplit, H, R] and part_ml [T, nsplit, H, 2] (fp32) and is meant for single-query rows.
extern "C" int areal_latent_attn(const void* q, int64_t q_stride, const void* q_lat, const void* cache,
                                 const int* block_tables, int max_pages, const int* cu_q, const int* ctx_len,
                                 const float* table, int n_pos, int neighbours, const void* sink, const void* gate, int64_t gate_stride, void* out, float* part_acc, float* part_ml,
                                 int B, int max_q, int T, int H, int D, int P, int R, float scale, int window,
                                 int nsplit, int dt, int matrix_cores, hipStream_t st) {
  if (B == 0 || T == 0) return 0;
  if (H < 1 || R < 1 || P % 2 || nsplit < 1 || nsplit > 64 || n_pos < 1) return -1;
  if (nsplit > 1 && (!part_acc || !part_ml)) return -3;
  if (matrix_cores && dt == 0 && mfma_usable(R, P, D, q_stride) && ((uintptr_t)q % 16) == 0 &&
      (max_q > 1 ? nsplit == 1 : true)) {
    const MfmaArgs a{(const bf16_t*)q, (const bf16_t*)q_lat, (const bf16_t*)cache, q_stride, neighbours,
                     (const bf16_t*)sink, block_tables, max_pages, cu_q,
                     ctx_len, table, n_pos, (const bf16_t*)gate, gate_stride, (bf16_t*)out, part_acc, part_ml, H, D,
                     scale, window, nsplit};
    if (max_q > 1) return dispatch_mfma<false>(R, P, B, max_q, st, a);
    const int e = dispatch_mfma<true>(R, P, B, 1, st, a);
    if (e == 0 && nsplit > 1)
      hipLaunchKernelGGL(latent_attn_combine_kernel<bf16_t>, dim3(T, H), dim3(128), 0, st, part_acc, part_ml,
                         (const bf16_t*)gate, gate_stride, (bf16_t*)out, H, R, nsplit);
    return e ? e : (int)hipGetLastError();
  }
  int want = 1;
  while (want < 8 && want < max_q) want <<= 1;
  LatentShape sh;
  if (!pick_shape(H, D, P, R, want, &sh)) return -2;
  const size_t lds = sh.floats() * sizeof(float);
  const int n_groups = (H + sh.HG - 1) / sh.HG;
  const dim3 grid(((max_q + sh.BQ - 1) / sh.BQ) * n_groups, B, nsplit);
#define LAUNCH(TT)                                                                                                  \
  do {                                                                                                              \
    static size_t allowed = 64 * 1024; /* raised once: no attribute call inside a stream capture */                 \
    if (lds > allowed) {                                                                                            \
      HIP_RET(hipFuncSetAttribute((const void*)latent_attn_kernel<TT>, hipFuncAttributeMaxDynamicSharedMemorySize,  \
                                  160 * 1024));                                                                     \
      allowed = 160 * 1024;                                                                                         \
    }                                                                                                               \
    hipLaunchKernelGGL(latent_attn_kernel<TT>, grid, dim3(256), lds, st, (const TT*)q, q_stride, (const TT*)q_lat,  \
                       (const TT*)cache, block_tables, max_pages, cu_q, ctx_len, table, n_pos, neighbours,          \
                       (const TT*)sink, (const TT*)gate, gate_stride, (TT*)out, part_acc, part_ml, sh, scale, window, nsplit);                        \
    if (nsplit > 1)                                                                                                 \
      hipLaunchKernelGGL(latent_attn_combine_kernel<TT>, dim3(T, H), dim3(128), 0, st, part_acc, part_ml,           \
                         (const TT*)gate, gate_stride, (TT*)out, H, R, nsplit);                                     \
  } while (0)
  if (dt == 0) LAUNCH(bf16_t);
  else LAUNCH(float);
#undef LAUNCH
  return (int)hipGetLastError();
}
