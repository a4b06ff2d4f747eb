// Sublayers between two RMS norms on an fp32 residual stream, with a learned average over the depth of the network:
//
//   x  <- x + mult * y / sqrt(mean(y^2) + eps) * (off + wb)          y: a sublayer's output, wb: the norm behind it
//   X_n = x;  x <- sum_{j <= n} a[j] X_j                             at the end of a layer: X_0 .. X_n are the stream
//                                                                    ahead of the first layer and behind every layer
//   h   = x / sqrt(mean(x^2) + eps) * (off + w)                      the norm the next sublayer (or the head) reads
//
// off = 1 for weights stored around zero, 0 for plain weights. `norm_add_avg_norm_kernel` does all three steps of a
// row in one launch (each is optional); rows up to 4096 wide that are multiples of 4 stay in registers and move as
// 8- / 16-byte vectors (`_vec`). `embed_pos_norm_kernel`: x = E[token] + P[position] as the fp32 stream, and the first
// norm of it.
#include "common.hpp"

namespace {

template <typename T> DEVINL float ldf(const T* p, size_t i);
template <> DEVINL float ldf<bf16_t>(const bf16_t* p, size_t i) { return bf2f(p[i]); }
template <> DEVINL float ldf<float>(const float* p, size_t i) { return p[i]; }
template <typename T> DEVINL void stf(T* p, size_t i, float v);
template <> DEVINL void stf<bf16_t>(bf16_t* p, size_t i, float v) { p[i] = f2bf(v); }
template <> DEVINL void stf<float>(float* p, size_t i, float v) { p[i] = v; }

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
// weights may sit anywhere in a flat parameter buffer: element loads
template <typename T> DEVINL f32x4 ldw4(const T* w, int i, float off) {
  return (f32x4){off + ldf<T>(w, i), off + ldf<T>(w, i + 1), off + ldf<T>(w, i + 2), off + ldf<T>(w, i + 3)};
}

struct RowArgs {
  const float* x_in;
  float* x_out;        // null: the new stream is not stored (it is only averaged and / or normed)
  const void* y;       // null: nothing is added
  const void* wb;
  float mult;
  const float* stack;  // X_0 ..: n_stack - 1 earlier streams, `stack_stride` floats apart (the newest is this row's x)
  int64_t stack_stride;
  int n_stack;         // 0: no average
  const void* avg;     // n_stack weights
  float* mix_out;
  const void* w_next;  // null: no norm
  float* o32;
  void* oc;
  int W;
  float eps, off;
};

template <typename T>
__global__ void __launch_bounds__(256) norm_add_avg_norm_kernel(RowArgs a) {
  __shared__ float red[16];
  const int W = a.W;
  const size_t base = (size_t)blockIdx.x * W;
  const T* y = reinterpret_cast<const T*>(a.y);
  float r = 0.f;
  if (y) {
    float ss = 0.f;
    for (int i = threadIdx.x; i < W; i += 256) {
      const float v = ldf<T>(y, base + i);
      ss += v * v;
    }
    r = 1.f / sqrtf(block_sum(ss, red) / (float)W + a.eps);
  }
  // where the row that the norm reads is kept between the two passes (every thread re-reads only what it wrote)
  float* keep = a.n_stack > 0 ? a.mix_out : a.x_out;
  float ss2 = 0.f;
  for (int i = threadIdx.x; i < W; i += 256) {
    float x = a.x_in[base + i];
    if (y) x += a.mult * (ldf<T>(y, base + i) * r * (a.off + ldf<T>(reinterpret_cast<const T*>(a.wb), i)));
    if (a.x_out) a.x_out[base + i] = x;
    if (a.n_stack > 0) {
      const T* av = reinterpret_cast<const T*>(a.avg);
      float m = ldf<T>(av, a.n_stack - 1) * x;
      for (int j = 0; j < a.n_stack - 1; ++j) m += ldf<T>(av, j) * a.stack[(size_t)j * a.stack_stride + base + i];
      x = m;
      a.mix_out[base + i] = x;
    }
    ss2 += x * x;
  }
  if (!a.w_next) return;
  const float r2 = 1.f / sqrtf(block_sum(ss2, red) / (float)W + a.eps);
  const float* src = keep ? keep : a.x_in;
  for (int i = threadIdx.x; i < W; i += 256) {
    const float h = src[base + i] * r2 * (a.off + ldf<T>(reinterpret_cast<const T*>(a.w_next), i));
    if (a.o32) a.o32[base + i] = h;
    if (a.oc) stf<T>(reinterpret_cast<T*>(a.oc), base + i, h);
  }
}

template <typename T, int NV>
__global__ void __launch_bounds__(256) norm_add_avg_norm_vec_kernel(RowArgs a) {
  __shared__ float red[16];
  const int W = a.W;
  const size_t base = (size_t)blockIdx.x * W;
  const T* y = reinterpret_cast<const T*>(a.y);
  f32x4 x[NV];
  if (y) {
    f32x4 yv[NV];
    float ss = 0.f;
#pragma unroll
    for (int v = 0; v < NV; ++v) {
      const int i = 4 * (threadIdx.x + 256 * v);
      if (i < W) {
        yv[v] = ld4<T>(y, base + i);
        x[v] = *reinterpret_cast<const f32x4*>(a.x_in + base + i);
        ss += yv[v][0] * yv[v][0] + yv[v][1] * yv[v][1] + yv[v][2] * yv[v][2] + yv[v][3] * yv[v][3];
      }
    }
    const float r = 1.f / sqrtf(block_sum(ss, red) / (float)W + a.eps);
#pragma unroll
    for (int v = 0; v < NV; ++v) {
      const int i = 4 * (threadIdx.x + 256 * v);
      if (i < W) x[v] += a.mult * (yv[v] * r * ldw4<T>(reinterpret_cast<const T*>(a.wb), i, a.off));
    }
  } else {
#pragma unroll
    for (int v = 0; v < NV; ++v) {
      const int i = 4 * (threadIdx.x + 256 * v);
      if (i < W) x[v] = *reinterpret_cast<const f32x4*>(a.x_in + base + i);
    }
  }
  float ss2 = 0.f;
#pragma unroll
  for (int v = 0; v < NV; ++v) {
    const int i = 4 * (threadIdx.x + 256 * v);
    if (i < W) {
      if (a.x_out) *reinterpret_cast<f32x4*>(a.x_out + base + i) = x[v];
      if (a.n_stack > 0) {
        const T* av = reinterpret_cast<const T*>(a.avg);
        f32x4 m = x[v] * ldf<T>(av, a.n_stack - 1);
        for (int j = 0; j < a.n_stack - 1; ++j)
          m += *reinterpret_cast<const f32x4*>(a.stack + (size_t)j * a.stack_stride + base + i) * ldf<T>(av, j);
        x[v] = m;
        *reinterpret_cast<f32x4*>(a.mix_out + base + i) = m;
      }
      ss2 += x[v][0] * x[v][0] + x[v][1] * x[v][1] + x[v][2] * x[v][2] + x[v][3] * x[v][3];
    }
  }
  if (!a.w_next) return;
  const float r2 = 1.f / sqrtf(block_sum(ss2, red) / (float)W + a.eps);
#pragma unroll
  for (int v = 0; v < NV; ++v) {
    const int i = 4 * (threadIdx.x + 256 * v);
    if (i < W) {
      const f32x4 h = x[v] * r2 * ldw4<T>(reinterpret_cast<const T*>(a.w_next), i, a.off);
      if (a.o32) *reinterpret_cast<f32x4*>(a.o32 + base + i) = h;
      if (a.oc) st4<T>(reinterpret_cast<T*>(a.oc), base + i, h);
    }
  }
}

template <typename T>
__global__ void __launch_bounds__(256) embed_pos_norm_kernel(
    const int64_t* __restrict__ tokens, const int* __restrict__ positions, const T* __restrict__ embed,
    const T* __restrict__ pos_table, int vocab, int n_pos, const T* __restrict__ w, float* __restrict__ x_out,
    float* __restrict__ o32, T* __restrict__ oc, int W, float eps, float off) {
  __shared__ float red[16];
  const size_t t = blockIdx.x, base = t * W;
  int64_t tok = tokens[t];
  tok = tok < 0 ? 0 : (tok >= vocab ? vocab - 1 : tok);
  const int p = min(max(positions[t], 0), n_pos - 1);
  float ss = 0.f;
  for (int i = threadIdx.x; i < W; i += 256) {
    const float x = ldf<T>(embed, (size_t)tok * W + i) + (pos_table ? ldf<T>(pos_table, (size_t)p * W + i) : 0.f);
    x_out[base + i] = x;
    ss += x * x;
  }
  if (!w) return;
  const float r = 1.f / sqrtf(block_sum(ss, red) / (float)W + eps);
  for (int i = threadIdx.x; i < W; i += 256) {
    const float h = x_out[base + i] * r * (off + ldf<T>(w, i));
    if (o32) o32[base + i] = h;
    if (oc) stf<T>(oc, base + i, h);
  }
}

}  // namespace

// All row tensors are [T, W] contiguous. x_in fp32; y / wb / avg / w_next / oc in the storage type `dt` (0: bf16,
// 1: fp32). stack: X_0 (first of n_stack - 1 earlier streams, stack_stride floats apart), or null with n_stack = 0.
extern "C" int areal_norm_add_avg_norm(const float* x_in, float* x_out, const void* y, const void* wb, float mult,
                                       const float* stack, int64_t stack_stride, int n_stack, const void* avg,
                                       float* mix_out, const void* w_next, float* o32, void* oc, int T, int W,
                                       float eps, int centered, int dt, hipStream_t st) {
  if (T == 0) return 0;
  if (W < 1 || n_stack < 0 || (y && !wb) || (n_stack > 0 && (!avg || !mix_out || (n_stack > 1 && !stack)))) return -1;
  if (w_next && n_stack == 0 && !x_out && y) return -1;  // the plain kernel keeps the row in one of its outputs
  const RowArgs a{x_in, x_out, y, wb, mult, stack, stack_stride, n_stack, avg, mix_out, w_next, o32, oc, W, eps,
                  centered ? 1.f : 0.f};
  const uintptr_t al = dt == 0 ? 8 : 16;
  const bool vec = W % 4 == 0 && W <= 4096 && stack_stride % 4 == 0 && ((uintptr_t)x_in % 16) == 0 &&
                   ((uintptr_t)x_out % 16) == 0 && ((uintptr_t)stack % 16) == 0 && ((uintptr_t)mix_out % 16) == 0 &&
                   ((uintptr_t)o32 % 16) == 0 && ((uintptr_t)y % al) == 0 && ((uintptr_t)oc % al) == 0;
#define GO(TT)                                                                                                  \
  do {                                                                                                          \
    if (vec && W <= 1024) hipLaunchKernelGGL((norm_add_avg_norm_vec_kernel<TT, 1>), dim3(T), dim3(256), 0, st, a); \
    else if (vec && W <= 2048) hipLaunchKernelGGL((norm_add_avg_norm_vec_kernel<TT, 2>), dim3(T), dim3(256), 0, st, a); \
    else if (vec) hipLaunchKernelGGL((norm_add_avg_norm_vec_kernel<TT, 4>), dim3(T), dim3(256), 0, st, a);       \
    else hipLaunchKernelGGL(norm_add_avg_norm_kernel<TT>, dim3(T), dim3(256), 0, st, a);                        \
  } while (0)
  if (dt == 0) GO(bf16_t);
  else GO(float);
#undef GO
  return (int)hipGetLastError();
}

// x_out fp32 [T, W] = embed[token] + pos_table[position] (pos_table null: the table row alone); with `w` also the
// norm of it, fp32 (o32) and / or storage type (oc).
extern "C" int areal_embed_pos_norm(const int64_t* tokens, const int* positions, const void* embed,
                                    const void* pos_table, int vocab, int n_pos, const void* w, float* x_out,
                                    float* o32, void* oc, int T, int W, float eps, int centered, int dt,
                                    hipStream_t st) {
  if (T == 0) return 0;
  if (W < 1 || vocab < 1 || (pos_table && n_pos < 1)) return -1;
  const float off = centered ? 1.f : 0.f;
  if (dt == 0)
    hipLaunchKernelGGL(embed_pos_norm_kernel<bf16_t>, dim3(T), dim3(256), 0, st, tokens, positions,
                       (const bf16_t*)embed, (const bf16_t*)pos_table, vocab, n_pos, (const bf16_t*)w, x_out, o32,
                       (bf16_t*)oc, W, eps, off);
  else
    hipLaunchKernelGGL(embed_pos_norm_kernel<float>, dim3(T), dim3(256), 0, st, tokens, positions, (const float*)embed,
                       (const float*)pos_table, vocab, n_pos, (const float*)w, x_out, o32, (float*)oc, W, eps, off);
  return (int)hipGetLastError();
}
