// Parallel blocks on an fp32 residual stream: both sublayers of a layer read ONE norm of the stream and their outputs
// are added together,
//
//   h = x / sqrt(mean(x^2) + eps) * w;     x <- x + a(h) + b(h)
//
// `sum_norm_kernel` does the closing sum of one layer and the opening norm of the next in one pass over the row
// (x += y1 + y2 in place; h in fp32 and / or the compute type); with no y it is the plain norm.
// `embed_scale_kernel`: x = E[token] * scale as the fp32 stream.  `glu_rows_kernel`: act(gate) * up over rows that hold
// gate | up side by side (rows may be a column range of a wider matrix);  `relu2_rows_kernel`: max(z, 0)^2.
#include "common.hpp"

namespace {

template <typename T> DEVINL float ldf(const T* p, size_t i);
template <> DEVINL float ldf<bf16_t>(const bf16_t* p, size_t i) { return bf2f(p[i]); }
template <> DEVINL float ldf<float>(const float* p, size_t i) { return p[i]; }
template <typename T> DEVINL void stf(T* p, size_t i, float v);
template <> DEVINL void stf<bf16_t>(bf16_t* p, size_t i, float v) { p[i] = f2bf(v); }
template <> DEVINL void stf<float>(float* p, size_t i, float v) { p[i] = v; }

template <typename T>
__global__ void __launch_bounds__(256) sum_norm_kernel(float* __restrict__ x, const T* __restrict__ y1,
                                                        const T* __restrict__ y2, const T* __restrict__ w,
                                                        float* __restrict__ o32, T* __restrict__ oc, int W, float eps) {
  __shared__ float red[16];
  const size_t base = (size_t)blockIdx.x * W;
  float ss = 0.f;
  for (int i = threadIdx.x; i < W; i += 256) {
    float z = x[base + i];
    if (y1) {
      float add = ldf<T>(y1, base + i);
      if (y2) add += ldf<T>(y2, base + i);
      z += add;
      x[base + i] = z;
    }
    ss += z * z;
  }
  if (!w) return;
  ss = block_sum(ss, red);
  const float r = 1.f / sqrtf(ss / (float)W + eps);
  for (int i = threadIdx.x; i < W; i += 256) {
    const float h = x[base + i] * r * ldf<T>(w, i);  // the thread re-reads what it wrote itself
    if (o32) o32[base + i] = h;
    if (oc) stf<T>(oc, base + i, h);
  }
}

template <typename T> DEVINL f32x4 ld4(const T* p, size_t i);
template <> DEVINL f32x4 ld4<bf16_t>(const bf16_t* p, size_t i) {
  const bf16x4 v = *reinterpret_cast<const bf16x4*>(p + i);
  return (f32x4){bf2f(v[0]), bf2f(v[1]), bf2f(v[2]), bf2f(v[3])};
}
template <> DEVINL f32x4 ld4<float>(const float* p, size_t i) { return *reinterpret_cast<const f32x4*>(p + i); }
template <typename T> DEVINL void st4(T* p, size_t i, f32x4 v);
template <> DEVINL void st4<bf16_t>(bf16_t* p, size_t i, f32x4 v) {
  *reinterpret_cast<bf16x4*>(p + i) = (bf16x4){f2bf(v[0]), f2bf(v[1]), f2bf(v[2]), f2bf(v[3])};
}
template <> DEVINL void st4<float>(float* p, size_t i, f32x4 v) { *reinterpret_cast<f32x4*>(p + i) = v; }

// The same for rows of up to 1024 NV elements that are multiples of 4: the row stays in registers between the sum of
// squares and the scaling, and moves as 8- / 16-byte vectors.
template <typename T, int NV>
__global__ void __launch_bounds__(256) sum_norm_vec_kernel(float* __restrict__ x, const T* __restrict__ y1,
                                                            const T* __restrict__ y2, const T* __restrict__ w,
                                                            float* __restrict__ o32, T* __restrict__ oc, int W, float eps) {
  __shared__ float red[16];
  const size_t base = (size_t)blockIdx.x * W;
  f32x4 z[NV];
  float ss = 0.f;
#pragma unroll
  for (int v = 0; v < NV; ++v) {
    const int i = 4 * (threadIdx.x + 256 * v);
    if (i < W) {
      z[v] = *reinterpret_cast<const f32x4*>(x + base + i);
      if (y1) {
        z[v] += ld4<T>(y1, base + i);
        if (y2) z[v] += ld4<T>(y2, base + i);
        *reinterpret_cast<f32x4*>(x + base + i) = z[v];
      }
      ss += z[v][0] * z[v][0] + z[v][1] * z[v][1] + z[v][2] * z[v][2] + z[v][3] * z[v][3];
    }
  }
  if (!w) return;
  ss = block_sum(ss, red);
  const float r = 1.f / sqrtf(ss / (float)W + eps);
#pragma unroll
  for (int v = 0; v < NV; ++v) {
    const int i = 4 * (threadIdx.x + 256 * v);
    if (i < W) {
      // the weight may sit anywhere in a flat parameter buffer: element loads
      const f32x4 h = z[v] * r * (f32x4){ldf<T>(w, i), ldf<T>(w, i + 1), ldf<T>(w, i + 2), ldf<T>(w, i + 3)};
      if (o32) *reinterpret_cast<f32x4*>(o32 + base + i) = h;
      if (oc) st4<T>(oc, base + i, h);
    }
  }
}

template <typename T>
__global__ void __launch_bounds__(256) embed_scale_kernel(const int64_t* __restrict__ tokens, const T* __restrict__ embed,
                                                           float* __restrict__ out, int W, int vocab, float scale) {
  const size_t t = blockIdx.x;
  int64_t tok = tokens[t];
  tok = tok < 0 ? 0 : (tok >= vocab ? vocab - 1 : tok);
  for (int i = threadIdx.x; i < W; i += 256) out[t * W + i] = ldf<T>(embed, (size_t)tok * W + i) * scale;
}

// act 0: SiLU, 1: tanh-GELU
template <typename T>
__global__ void __launch_bounds__(256) glu_rows_kernel(const T* __restrict__ gu, int64_t row_stride, T* __restrict__ out,
                                                        int64_t n, int F, int act) {
  const int64_t total = n * F;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < total; i += (int64_t)gridDim.x * 256) {
    const int64_t r = i / F;
    const int c = (int)(i % F);
    const float g = ldf<T>(gu, r * row_stride + c), u = ldf<T>(gu, r * row_stride + F + c);
    float a;
    if (act == 0) a = g / (1.f + expf(-g));
    else a = 0.5f * g * (1.f + tanhf(0.7978845608028654f * (g + 0.044715f * g * g * g)));
    stf<T>(out, i, a * u);
  }
}

template <typename T>
__global__ void __launch_bounds__(256) relu2_rows_kernel(const T* __restrict__ z, int64_t row_stride, T* __restrict__ out,
                                                          int64_t n, int F) {
  const int64_t total = n * F;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < total; i += (int64_t)gridDim.x * 256) {
    const float v = fmaxf(ldf<T>(z, (i / F) * row_stride + i % F), 0.f);
    stf<T>(out, i, v * v);
  }
}

// z[t, e] = x[t, :] . w[e, :] + b[e]: fp32 input rows (a norm's fp32 output), weights in the storage type, fp32 sums.
// For few tokens (decoding; large batches go to the fp32 library product): one wave per (token, weight row). VEC: rows
// that are multiples of 4 with 8- / 16-byte aligned weights move as vectors, eight loads of a lane in flight.
template <typename T, bool VEC>
__global__ void __launch_bounds__(256) router_logits_kernel(const float* __restrict__ x, const T* __restrict__ w,
                                                             const T* __restrict__ bias, float* __restrict__ z, int W,
                                                             int E) {
  const int t = blockIdx.x, lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int u = blockIdx.y * 4 + wave;
  if (u >= E) return;
  const T* wr = w + (size_t)u * W;
  const float* xr = x + (size_t)t * W;
  float s = 0.f;
  if (VEC) {
#pragma unroll 8
    for (int i = 4 * lane; i < W; i += 256) {
      const f32x4 a = *reinterpret_cast<const f32x4*>(xr + i), b = ld4<T>(wr, i);
      s += a[0] * b[0] + a[1] * b[1] + a[2] * b[2] + a[3] * b[3];
    }
  } else {
#pragma unroll 8
    for (int i = lane; i < W; i += 64) s += xr[i] * ldf<T>(wr, i);
  }
  s = wave_sum(s);
  if (lane == 0) z[(size_t)t * E + u] = s + (bias ? ldf<T>(bias, u) : 0.f);
}

// bf16 rows whose width, stride and addresses are multiples of 8 elements: 16-byte loads and stores, 8 outputs a thread.
// GLU = true: act(gate) * up (act 0: SiLU, 1: tanh-GELU); false: max(z, 0)^2.
template <bool GLU>
__global__ void __launch_bounds__(256) act_rows_vec_kernel(const bf16_t* __restrict__ in, int64_t row_stride,
                                                            bf16_t* __restrict__ out, int64_t n, int F, int act) {
  const int fv = F / 8;
  const int64_t total = n * fv;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < total; i += (int64_t)gridDim.x * 256) {
    const int64_t r = i / fv;
    const int c = 8 * (int)(i % fv);
    const bf16x8 g = ld8(in + r * row_stride + c);
    bf16x8 o;
    if (GLU) {
      const bf16x8 u = ld8(in + r * row_stride + F + c);
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const float x = bf2f(g[e]);
        const float a = act == 0 ? x / (1.f + expf(-x))
                                 : 0.5f * x * (1.f + tanhf(0.7978845608028654f * (x + 0.044715f * x * x * x)));
        o[e] = f2bf(a * bf2f(u[e]));
      }
    } else {
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const float x = fmaxf(bf2f(g[e]), 0.f);
        o[e] = f2bf(x * x);
      }
    }
    st8(out + r * (int64_t)F + c, o);
  }
}

bool rows_vec_ok(const void* in, int64_t row_stride, const void* out, int F, int dt) {
  return dt == 0 && F % 8 == 0 && row_stride % 8 == 0 && ((uintptr_t)in % 16) == 0 && ((uintptr_t)out % 16) == 0;
}

int blocks_for(int64_t total) { return (int)((total + 255) / 256 < 65535 * 8 ? (total + 255) / 256 : 65535 * 8); }

}  // namespace

// x fp32 [T, W] (+= y1 + y2 in place when y1 is given; y2 needs y1); w null: no norm is produced.
extern "C" int areal_sum_norm(float* x, const void* y1, const void* y2, const void* w, float* o32, void* oc, int T, int W,
                              float eps, int dt, hipStream_t st) {
  if (T == 0) return 0;
  if (y2 && !y1) return -1;
  if (W % 4 == 0 && W <= 4096) {
#define VEC(TT, NVV)                                                                                                \
  hipLaunchKernelGGL((sum_norm_vec_kernel<TT, NVV>), dim3(T), dim3(256), 0, st, x, (const TT*)y1, (const TT*)y2,     \
                     (const TT*)w, o32, (TT*)oc, W, eps)
    if (dt == 0) {
      if (W <= 1024) VEC(bf16_t, 1);
      else if (W <= 2048) VEC(bf16_t, 2);
      else VEC(bf16_t, 4);
    } else {
      if (W <= 1024) VEC(float, 1);
      else if (W <= 2048) VEC(float, 2);
      else VEC(float, 4);
    }
#undef VEC
    return (int)hipGetLastError();
  }
  if (dt == 0)
    hipLaunchKernelGGL(sum_norm_kernel<bf16_t>, dim3(T), dim3(256), 0, st, x, (const bf16_t*)y1, (const bf16_t*)y2,
                       (const bf16_t*)w, o32, (bf16_t*)oc, W, eps);
  else
    hipLaunchKernelGGL(sum_norm_kernel<float>, dim3(T), dim3(256), 0, st, x, (const float*)y1, (const float*)y2,
                       (const float*)w, o32, (float*)oc, W, eps);
  return (int)hipGetLastError();
}

extern "C" int areal_embed_scale(const int64_t* tokens, const void* embed, float* out, int T, int W, int vocab,
                                 float scale, int dt, hipStream_t st) {
  if (T == 0) return 0;
  if (dt == 0)
    hipLaunchKernelGGL(embed_scale_kernel<bf16_t>, dim3(T), dim3(256), 0, st, tokens, (const bf16_t*)embed, out, W,
                       vocab, scale);
  else
    hipLaunchKernelGGL(embed_scale_kernel<float>, dim3(T), dim3(256), 0, st, tokens, (const float*)embed, out, W, vocab,
                       scale);
  return (int)hipGetLastError();
}

extern "C" int areal_glu_rows(const void* gu, int64_t row_stride, void* out, int64_t n, int F, int act, int dt,
                              hipStream_t st) {
  if (n == 0 || F == 0) return 0;
  if (rows_vec_ok(gu, row_stride, out, F, dt)) {
    hipLaunchKernelGGL(act_rows_vec_kernel<true>, dim3(blocks_for(n * F / 8)), dim3(256), 0, st, (const bf16_t*)gu,
                       row_stride, (bf16_t*)out, n, F, act);
    return (int)hipGetLastError();
  }
  const int nb = blocks_for(n * F);
  if (dt == 0)
    hipLaunchKernelGGL(glu_rows_kernel<bf16_t>, dim3(nb), dim3(256), 0, st, (const bf16_t*)gu, row_stride, (bf16_t*)out,
                       n, F, act);
  else
    hipLaunchKernelGGL(glu_rows_kernel<float>, dim3(nb), dim3(256), 0, st, (const float*)gu, row_stride, (float*)out, n,
                       F, act);
  return (int)hipGetLastError();
}

extern "C" int areal_relu2_rows(const void* z, int64_t row_stride, void* out, int64_t n, int F, int dt, hipStream_t st) {
  if (n == 0 || F == 0) return 0;
  if (rows_vec_ok(z, row_stride, out, F, dt)) {
    hipLaunchKernelGGL(act_rows_vec_kernel<false>, dim3(blocks_for(n * F / 8)), dim3(256), 0, st, (const bf16_t*)z,
                       row_stride, (bf16_t*)out, n, F, 0);
    return (int)hipGetLastError();
  }
  const int nb = blocks_for(n * F);
  if (dt == 0)
    hipLaunchKernelGGL(relu2_rows_kernel<bf16_t>, dim3(nb), dim3(256), 0, st, (const bf16_t*)z, row_stride, (bf16_t*)out,
                       n, F);
  else
    hipLaunchKernelGGL(relu2_rows_kernel<float>, dim3(nb), dim3(256), 0, st, (const float*)z, row_stride, (float*)out, n,
                       F);
  return (int)hipGetLastError();
}

// x fp32 [T, W], w [E, W] and bias [E] (or null) in the storage type -> z fp32 [T, E]
extern "C" int areal_router_logits(const float* x, const void* w, const void* bias, float* z, int T, int W, int E, int dt,
                                   hipStream_t st) {
  if (T == 0 || E == 0) return 0;
  const bool vec = W % 4 == 0 && ((uintptr_t)w % (dt == 0 ? 8 : 16)) == 0 && ((uintptr_t)x % 16) == 0;
  const dim3 grid(T, (E + 3) / 4);
#define LAUNCH(TT, VV)                                                                                            \
  hipLaunchKernelGGL((router_logits_kernel<TT, VV>), grid, dim3(256), 0, st, x, (const TT*)w, (const TT*)bias, z, W, E)
  if (dt == 0) {
    if (vec) LAUNCH(bf16_t, true);
    else LAUNCH(bf16_t, false);
  } else {
    if (vec) LAUNCH(float, true);
    else LAUNCH(float, false);
  }
#undef LAUNCH
  return (int)hipGetLastError();
}
