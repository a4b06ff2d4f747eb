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

int blocks_for(int64_t total) { return (int)((total + 255) / 256 < 65535 * 8 ? (total + 255) / 256 : 65535 * 8); }

}  // namespace

// x fp32 [T, W] (+= y1 + y2 in place when y1 is given; y2 needs y1); w null: no norm is produced.
extern "C" int areal_sum_norm(float* x, const void* y1, const void* y2, const void* w, float* o32, void* oc, int T, int W,
                              float eps, int dt, hipStream_t st) {
  if (T == 0) return 0;
  if (y2 && !y1) return -1;
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
  const int nb = blocks_for(n * F);
  if (dt == 0)
    hipLaunchKernelGGL(relu2_rows_kernel<bf16_t>, dim3(nb), dim3(256), 0, st, (const bf16_t*)z, row_stride, (bf16_t*)out,
                       n, F);
  else
    hipLaunchKernelGGL(relu2_rows_kernel<float>, dim3(nb), dim3(256), 0, st, (const float*)z, row_stride, (float*)out, n,
                       F);
  return (int)hipGetLastError();
}
