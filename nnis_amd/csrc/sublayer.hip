// What lies between the projections of sublayers that norm their outputs, gate their heads, pool their keys or
// route their tokens: row-wise kernels, all 32-bit inside whatever the storage type.
//
//   cast_rows          rows of one type as rows of another (the 32-bit stream as a sublayer's input)
//   rms_post_step      x += y / rms(y) * (offset + w), and the stream's rows in the activation type; y may stand for y + share * rows
//   poly_norm          a N(z) + b N(z^2) + c N(z^3) + e, N a division by the root mean square of a row
//   router_logits      a router's logits as 32-bit dot products
//   route_top          softmax of router logits, the `top` largest of score + correction, dense weights out
//   routed_act         weight[row, expert] * relu(z)^2 on the experts' fused up projection
//   rows_axpy          y[row] += c[row] * h[row]
//   sigmoid_gate       o *= sigmoid(g)
//   head_norm_write    per-head RMS norm of queries and keys, rotation (neighbouring channels or halves), queries out,
//                      keys and values into the pages
//   pool_blocks        the mean key and value of every block of `pool` tokens that a step completes
#include "common.h"

thread_local char g_nnis_error[512] = {0};
extern "C" const char* nnis_last_error() { return g_nnis_error; }

namespace {

constexpr float kLog2e = 1.4426950408889634f;
__device__ __forceinline__ float sigmoid_f(float z) { return 1.0f / (1.0f + expf(-z)); }

// -----------------------------------------------------------------------------
// The way out of a sublayer whose output alone is normed: x[row] += y[row] / sqrt(mean(y^2) + eps) * (offset + w),
// in place in the 32-bit stream, and h[row] = the new x in the activation type (what the next sublayer reads).
// A block a row; the row is read twice (the second time from the caches).
// -----------------------------------------------------------------------------
constexpr int kPostKeep = 16;  // values of a row that a thread keeps in registers between the two passes

__global__ __launch_bounds__(256) void rms_post_step_kernel(float* x, const void* __restrict__ y, int y_dtype,
                                                            const void* __restrict__ weight, int w_dtype, float offset, float eps,
                                                            void* h, int h_dtype, int width, const float* __restrict__ keep,
                                                            const void* h_in, int h_in_dtype) {
  __shared__ float scratch[16];
  const size_t base = (size_t)blockIdx.x * width;
  // everything the row needs is asked for before the sum is waited for: y, the stream and the weight, up to
  // kPostKeep values a thread; what lies beyond (rows wider than kPostKeep x the block) is read a second time
  // with `keep`: y stands for y + keep[row] * h_in[row] (h_in may be h itself: a row is read before it is written)
  const float share = keep ? keep[blockIdx.x] : 0.0f;
  float ys[kPostKeep], xs[kPostKeep], ws[kPostKeep];
  float ss = 0.0f;
#pragma unroll
  for (int i = 0; i < kPostKeep; ++i) {
    const int c = threadIdx.x + i * blockDim.x;
    if (c < width) {
      ys[i] = load_as_f32(y, y_dtype, base + c);
      if (keep) ys[i] = fmaf(share, load_as_f32(h_in, h_in_dtype, base + c), ys[i]);
      xs[i] = x[base + c];
      ws[i] = offset + load_as_f32(weight, w_dtype, c);
      ss = fmaf(ys[i], ys[i], ss);
    }
  }
  for (int c = threadIdx.x + kPostKeep * blockDim.x; c < width; c += blockDim.x) {
    float v = load_as_f32(y, y_dtype, base + c);
    if (keep) v = fmaf(share, load_as_f32(h_in, h_in_dtype, base + c), v);
    ss = fmaf(v, v, ss);
  }
  const float inv = 1.0f / sqrtf(block_sum(ss, scratch) / (float)width + eps);
#pragma unroll
  for (int i = 0; i < kPostKeep; ++i) {
    const int c = threadIdx.x + i * blockDim.x;
    if (c < width) {
      const float sum = xs[i] + ys[i] * inv * ws[i];
      x[base + c] = sum;
      if (h) store_from_f32(h, h_dtype, base + c, sum);
    }
  }
  for (int c = threadIdx.x + kPostKeep * blockDim.x; c < width; c += blockDim.x) {
    float v = load_as_f32(y, y_dtype, base + c);
    if (keep) v = fmaf(share, load_as_f32(h_in, h_in_dtype, base + c), v);
    const float sum = x[base + c] + v * inv * (offset + load_as_f32(weight, w_dtype, c));
    x[base + c] = sum;
    if (h) store_from_f32(h, h_dtype, base + c, sum);
  }
}

// The same, four channels a thread and access (rows of a multiple of four channels, a 32-bit weight): y and the
// rows out in one type T (bfloat16 with rows out, or 32-bit), the shared rows in T too.
__device__ __forceinline__ float4 load4(const float* p) { return *(const float4*)p; }
__device__ __forceinline__ float4 load4(const bf16_t* p) {
  typedef __attribute__((__vector_size__(4 * sizeof(__bf16)))) __bf16 bf16x4_t;
  const bf16x4_t v = *(const bf16x4_t*)p;
  return make_float4((float)v[0], (float)v[1], (float)v[2], (float)v[3]);
}
__device__ __forceinline__ void store4(float* p, float4 v) { *(float4*)p = v; }
__device__ __forceinline__ void store4(bf16_t* p, float4 v) {
  typedef __attribute__((__vector_size__(4 * sizeof(__bf16)))) __bf16 bf16x4_t;
  bf16x4_t o;
  o[0] = (__bf16)v.x; o[1] = (__bf16)v.y; o[2] = (__bf16)v.z; o[3] = (__bf16)v.w;
  *(bf16x4_t*)p = o;
}

constexpr int kPostKeep4 = 4;  // groups of four channels that a thread keeps: rows of up to 16 x the block's threads

template <typename T>
__global__ __launch_bounds__(256) void rms_post_step4_kernel(float* x, const T* __restrict__ y, const float* __restrict__ weight,
                                                             float offset, float eps, T* h, int width, const float* __restrict__ keep,
                                                             const T* h_in) {
  __shared__ float scratch[16];
  const size_t base = (size_t)blockIdx.x * width;
  const float share = keep ? keep[blockIdx.x] : 0.0f;
  float4 ys[kPostKeep4], xs[kPostKeep4], ws[kPostKeep4];
  float ss = 0.0f;
#pragma unroll
  for (int i = 0; i < kPostKeep4; ++i) {
    const int c = 4 * (threadIdx.x + i * blockDim.x);
    if (c < width) {
      ys[i] = load4(y + base + c);
      xs[i] = load4(x + base + c);
      ws[i] = load4(weight + c);
      if (keep) {
        const float4 r = load4(h_in + base + c);
        ys[i].x = fmaf(share, r.x, ys[i].x); ys[i].y = fmaf(share, r.y, ys[i].y);
        ys[i].z = fmaf(share, r.z, ys[i].z); ys[i].w = fmaf(share, r.w, ys[i].w);
      }
      ss = fmaf(ys[i].x, ys[i].x, fmaf(ys[i].y, ys[i].y, fmaf(ys[i].z, ys[i].z, fmaf(ys[i].w, ys[i].w, ss))));
    }
  }
  const float inv = 1.0f / sqrtf(block_sum(ss, scratch) / (float)width + eps);
#pragma unroll
  for (int i = 0; i < kPostKeep4; ++i) {
    const int c = 4 * (threadIdx.x + i * blockDim.x);
    if (c < width) {
      float4 sum;
      sum.x = xs[i].x + ys[i].x * inv * (offset + ws[i].x);
      sum.y = xs[i].y + ys[i].y * inv * (offset + ws[i].y);
      sum.z = xs[i].z + ys[i].z * inv * (offset + ws[i].z);
      sum.w = xs[i].w + ys[i].w * inv * (offset + ws[i].w);
      store4(x + base + c, sum);
      if (h) store4(h + base + c, sum);
    }
  }
}

// -----------------------------------------------------------------------------
// Between two sublayers of a layer that norms both ways with RMS norms: the way out of the one, the sum into the
// 32-bit stream and the way into the next in one kernel,
//   x[row] += y / sqrt(mean(y^2) + eps) * w_out;   h[row] = x / sqrt(mean(x^2) + eps) * w_in
// (y may stand for y + keep[row] * h_in[row], as in rms_post_step).  A block a row; a thread keeps up to kPostKeep
// values of the row in registers between the three passes and reads what lies beyond again.
// -----------------------------------------------------------------------------
__global__ __launch_bounds__(256) void rms_between_kernel(float* x, const void* __restrict__ y, int y_dtype, const void* __restrict__ w_out,
                                                          const void* __restrict__ w_in, int w_dtype, float eps, void* h, int h_dtype,
                                                          int width, const float* __restrict__ keep, const void* __restrict__ h_in,
                                                          int h_in_dtype) {
  __shared__ float scratch[16];
  __shared__ float scratch2[16];
  const size_t base = (size_t)blockIdx.x * width;
  const float share = keep ? keep[blockIdx.x] : 0.0f;
  float vs[kPostKeep];
  float ss = 0.0f;
  auto value = [&](int c) {
    float v = load_as_f32(y, y_dtype, base + c);
    if (keep) v = fmaf(share, load_as_f32(h_in, h_in_dtype, base + c), v);
    return v;
  };
#pragma unroll
  for (int i = 0; i < kPostKeep; ++i) {
    const int c = threadIdx.x + i * blockDim.x;
    vs[i] = c < width ? value(c) : 0.0f;
    ss = fmaf(vs[i], vs[i], ss);
  }
  for (int c = threadIdx.x + kPostKeep * blockDim.x; c < width; c += blockDim.x) {
    const float v = value(c);
    ss = fmaf(v, v, ss);
  }
  const float inv = 1.0f / sqrtf(block_sum(ss, scratch) / (float)width + eps);
  float ss2 = 0.0f;
#pragma unroll
  for (int i = 0; i < kPostKeep; ++i) {
    const int c = threadIdx.x + i * blockDim.x;
    if (c < width) {
      vs[i] = x[base + c] + vs[i] * inv * load_as_f32(w_out, w_dtype, c);
      x[base + c] = vs[i];
      ss2 = fmaf(vs[i], vs[i], ss2);
    }
  }
  for (int c = threadIdx.x + kPostKeep * blockDim.x; c < width; c += blockDim.x) {
    const float sum = x[base + c] + value(c) * inv * load_as_f32(w_out, w_dtype, c);
    x[base + c] = sum;
    ss2 = fmaf(sum, sum, ss2);
  }
  if (h == nullptr) return;
  const float inv2 = 1.0f / sqrtf(block_sum(ss2, scratch2) / (float)width + eps);
#pragma unroll
  for (int i = 0; i < kPostKeep; ++i) {
    const int c = threadIdx.x + i * blockDim.x;
    if (c < width) store_from_f32(h, h_dtype, base + c, vs[i] * inv2 * load_as_f32(w_in, w_dtype, c));
  }
  for (int c = threadIdx.x + kPostKeep * blockDim.x; c < width; c += blockDim.x)
    store_from_f32(h, h_dtype, base + c, x[base + c] * inv2 * load_as_f32(w_in, w_dtype, c));
}

// The same, four channels a thread and access (rows of a multiple of four channels, up to 16 x the block's threads):
// y, the shared rows and the rows out in one type T, the weights in W; the stream, y and both weights are asked for
// before the first sum is waited for.
template <typename T, typename W>
__global__ __launch_bounds__(256) void rms_between4_kernel(float* x, const T* __restrict__ y, const W* __restrict__ w_out,
                                                           const W* __restrict__ w_in, float eps, T* h, int width,
                                                           const float* __restrict__ keep, const T* __restrict__ h_in) {
  __shared__ float scratch[16];
  __shared__ float scratch2[16];
  const size_t base = (size_t)blockIdx.x * width;
  const float share = keep ? keep[blockIdx.x] : 0.0f;
  float4 ys[kPostKeep4], xs[kPostKeep4], wo[kPostKeep4], wi[kPostKeep4];
  float ss = 0.0f;
#pragma unroll
  for (int i = 0; i < kPostKeep4; ++i) {
    const int c = 4 * (threadIdx.x + i * blockDim.x);
    if (c < width) {
      ys[i] = load4(y + base + c);
      xs[i] = load4(x + base + c);
      wo[i] = load4(w_out + c);
      if (h) wi[i] = load4(w_in + c);
      if (keep) {
        const float4 r = load4(h_in + base + c);
        ys[i].x = fmaf(share, r.x, ys[i].x); ys[i].y = fmaf(share, r.y, ys[i].y);
        ys[i].z = fmaf(share, r.z, ys[i].z); ys[i].w = fmaf(share, r.w, ys[i].w);
      }
      ss = fmaf(ys[i].x, ys[i].x, fmaf(ys[i].y, ys[i].y, fmaf(ys[i].z, ys[i].z, fmaf(ys[i].w, ys[i].w, ss))));
    }
  }
  const float inv = 1.0f / sqrtf(block_sum(ss, scratch) / (float)width + eps);
  float ss2 = 0.0f;
#pragma unroll
  for (int i = 0; i < kPostKeep4; ++i) {
    const int c = 4 * (threadIdx.x + i * blockDim.x);
    if (c < width) {
      xs[i].x += ys[i].x * inv * wo[i].x; xs[i].y += ys[i].y * inv * wo[i].y;
      xs[i].z += ys[i].z * inv * wo[i].z; xs[i].w += ys[i].w * inv * wo[i].w;
      store4(x + base + c, xs[i]);
      ss2 = fmaf(xs[i].x, xs[i].x, fmaf(xs[i].y, xs[i].y, fmaf(xs[i].z, xs[i].z, fmaf(xs[i].w, xs[i].w, ss2))));
    }
  }
  if (h == nullptr) return;
  const float inv2 = 1.0f / sqrtf(block_sum(ss2, scratch2) / (float)width + eps);
#pragma unroll
  for (int i = 0; i < kPostKeep4; ++i) {
    const int c = 4 * (threadIdx.x + i * blockDim.x);
    if (c < width) store4(h + base + c, make_float4(xs[i].x * inv2 * wi[i].x, xs[i].y * inv2 * wi[i].y, xs[i].z * inv2 * wi[i].z, xs[i].w * inv2 * wi[i].w));
  }
}

// -----------------------------------------------------------------------------
// PolyNorm: out = a z / rms(z) + b z^2 / rms(z^2) + c z^3 / rms(z^3) + e, powers element by element, each root mean
// square over the row with eps inside the root; coef = (a, b, c, e) in device memory.
// -----------------------------------------------------------------------------
constexpr int kPolyKeep = 32;  // values of a row that a thread keeps in registers between the two passes

__global__ __launch_bounds__(256) void poly_norm_kernel(const void* __restrict__ z, int z_dtype, const float* __restrict__ coef,
                                                        float eps, void* __restrict__ out, int out_dtype, int width) {
  __shared__ float scratch[3][16];
  const size_t base = (size_t)blockIdx.x * width;
  float zs[kPolyKeep];
  float s2 = 0.0f, s4 = 0.0f, s6 = 0.0f;
  auto add = [&](float v) {
    const float v2 = v * v;
    s2 += v2;
    s4 = fmaf(v2, v2, s4);
    s6 = fmaf(v2 * v, v2 * v, s6);
  };
#pragma unroll
  for (int i = 0; i < kPolyKeep; ++i) {
    const int c = threadIdx.x + i * blockDim.x;
    if (c < width) {
      zs[i] = load_as_f32(z, z_dtype, base + c);
      add(zs[i]);
    }
  }
  for (int c = threadIdx.x + kPolyKeep * blockDim.x; c < width; c += blockDim.x) add(load_as_f32(z, z_dtype, base + c));
  const float n = (float)width;
  const float i1 = 1.0f / sqrtf(block_sum(s2, scratch[0]) / n + eps);
  const float i2 = 1.0f / sqrtf(block_sum(s4, scratch[1]) / n + eps);
  const float i3 = 1.0f / sqrtf(block_sum(s6, scratch[2]) / n + eps);
  const float a = coef[0] * i1, b = coef[1] * i2, cc = coef[2] * i3, e = coef[3];
#pragma unroll
  for (int i = 0; i < kPolyKeep; ++i) {
    const int c = threadIdx.x + i * blockDim.x;
    if (c < width) store_from_f32(out, out_dtype, base + c, fmaf(zs[i], fmaf(zs[i], fmaf(zs[i], cc, b), a), e));
  }
  for (int c = threadIdx.x + kPolyKeep * blockDim.x; c < width; c += blockDim.x) {
    const float v = load_as_f32(z, z_dtype, base + c);
    store_from_f32(out, out_dtype, base + c, fmaf(v, fmaf(v, fmaf(v, cc, b), a), e));
  }
}

// the same, four values a thread and access (rows of a multiple of four, in and out of one type)
constexpr int kPolyKeep4 = 8;  // groups of four that a thread keeps: rows of up to 32 x the block's threads

template <typename T>
__global__ __launch_bounds__(256) void poly_norm4_kernel(const T* __restrict__ z, const float* __restrict__ coef, float eps, T* __restrict__ out,
                                                         int width) {
  __shared__ float scratch[3][16];
  const size_t base = (size_t)blockIdx.x * width;
  float4 zs[kPolyKeep4];
  float s2 = 0.0f, s4 = 0.0f, s6 = 0.0f;
  auto add = [&](float v) {
    const float v2 = v * v;
    s2 += v2;
    s4 = fmaf(v2, v2, s4);
    s6 = fmaf(v2 * v, v2 * v, s6);
  };
#pragma unroll
  for (int i = 0; i < kPolyKeep4; ++i) {
    const int c = 4 * (threadIdx.x + i * blockDim.x);
    if (c < width) {
      zs[i] = load4(z + base + c);
      add(zs[i].x), add(zs[i].y), add(zs[i].z), add(zs[i].w);
    }
  }
  const float n = (float)width;
  const float i1 = 1.0f / sqrtf(block_sum(s2, scratch[0]) / n + eps);
  const float i2 = 1.0f / sqrtf(block_sum(s4, scratch[1]) / n + eps);
  const float i3 = 1.0f / sqrtf(block_sum(s6, scratch[2]) / n + eps);
  const float a = coef[0] * i1, b = coef[1] * i2, cc = coef[2] * i3, e = coef[3];
  auto act = [&](float v) { return fmaf(v, fmaf(v, fmaf(v, cc, b), a), e); };
#pragma unroll
  for (int i = 0; i < kPolyKeep4; ++i) {
    const int c = 4 * (threadIdx.x + i * blockDim.x);
    if (c < width) store4(out + base + c, make_float4(act(zs[i].x), act(zs[i].y), act(zs[i].z), act(zs[i].w)));
  }
}

// -----------------------------------------------------------------------------
// A router's logits are logits[row, e] = sum_c x[row, c] * w[e, c] in 32-bit, w float32 [n, width]: a block takes R
// rows, kept in LDS as floats; a wave takes an output at a time for all of them (lanes stride over the channels), so
// a row of the weight is read once a block.
// Routing: scores s = softmax(logits) over n outputs; the `top` outputs with the largest s + correction are chosen
// (the lower index on a tie); gates[row, e] = s_e for a chosen output below `experts`, 0 for the others; keep[row] =
// the sum of s over the chosen outputs from `experts` on (those hand the input through).  A wave a row.
// -----------------------------------------------------------------------------
constexpr int kRouteMost = 16;  // outputs a lane holds: n <= 64 * kRouteMost

// one row by one wave; `logits`: the row's n logits (global memory or LDS)
// group_count > 1: the outputs form that many equal groups of neighbours; a group's mark is its largest corrected
// score, and only outputs of the group_keep groups with the largest marks (the lower group on a tie) can be chosen.
__device__ __forceinline__ void route_row(const float* logits, const float* __restrict__ correction, int row, int n, int experts, int top,
                                          float* __restrict__ gates, float* __restrict__ keep, int lane, int group_count = 1,
                                          int group_keep = 1) {
  float s[kRouteMost], choice[kRouteMost];
  float top_logit = -INFINITY;
#pragma unroll
  for (int i = 0; i < kRouteMost; ++i) {
    const int e = i * kWave + lane;
    s[i] = e < n ? logits[e] : -INFINITY;
    top_logit = fmaxf(top_logit, s[i]);
  }
  top_logit = wave_max(top_logit);
  float sum = 0.0f;
#pragma unroll
  for (int i = 0; i < kRouteMost; ++i) {
    s[i] = (i * kWave + lane) < n ? expf(s[i] - top_logit) : 0.0f;
    sum += s[i];
  }
  const float inv = 1.0f / wave_sum(sum);
  unsigned chosen = 0;
#pragma unroll
  for (int i = 0; i < kRouteMost; ++i) {
    const int e = i * kWave + lane;
    s[i] *= inv;
    choice[i] = e < n ? s[i] + (correction ? correction[e] : 0.0f) : -INFINITY;
  }
  if (group_count > 1 && group_keep < group_count) {
    // lane g holds group g's mark (up to 64 groups); the kept groups are found one at a time
    const int size = n / group_count;
    float mark = -INFINITY;
    for (int g = 0; g < group_count; ++g) {
      float best = -INFINITY;
#pragma unroll
      for (int i = 0; i < kRouteMost; ++i) {
        const int e = i * kWave + lane;
        if (e < n && e / size == g) best = fmaxf(best, choice[i]);
      }
      best = wave_max(best);
      if (lane == g) mark = best;
    }
    unsigned long long allowed = 0ull;
    for (int round = 0; round < group_keep; ++round) {
      float best = lane < group_count && !(allowed >> lane & 1ull) ? mark : -INFINITY;
      int best_g = lane < group_count && !(allowed >> lane & 1ull) ? lane : 0x7fffffff;
#pragma unroll
      for (int offset = kWave / 2; offset > 0; offset >>= 1) {
        const float other = __shfl_xor(best, offset, kWave);
        const int other_g = __shfl_xor(best_g, offset, kWave);
        if (other_g != 0x7fffffff && (best_g == 0x7fffffff || other > best || (other == best && other_g < best_g))) {
          best = other;
          best_g = other_g;
        }
      }
      if (best_g == 0x7fffffff) break;
      allowed |= 1ull << best_g;
    }
#pragma unroll
    for (int i = 0; i < kRouteMost; ++i) {
      const int e = i * kWave + lane;
      if (e < n && !(allowed >> (e / size) & 1ull)) choice[i] = -INFINITY;
    }
  }
  float kept = 0.0f;
  for (int round = 0; round < top; ++round) {
    float best = -INFINITY;
    int best_e = 0x7fffffff;
#pragma unroll
    for (int i = 0; i < kRouteMost; ++i) {
      const int e = i * kWave + lane;
      if (!(chosen >> i & 1u) && e < n && choice[i] > -INFINITY && (choice[i] > best || (choice[i] == best && e < best_e))) {
        best = choice[i];
        best_e = e;
      }
    }
#pragma unroll
    for (int offset = kWave / 2; offset > 0; offset >>= 1) {
      const float other = __shfl_xor(best, offset, kWave);
      const int other_e = __shfl_xor(best_e, offset, kWave);
      if (other > best || (other == best && other_e < best_e)) {
        best = other;
        best_e = other_e;
      }
    }
    if (best_e == 0x7fffffff) break;  // fewer outputs than `top`
    if (best_e % kWave == lane) {
      const int i = best_e / kWave;
      chosen |= 1u << i;
#pragma unroll
      for (int k = 0; k < kRouteMost; ++k)
        if (k == i && best_e >= experts) kept += s[k];
    }
  }
#pragma unroll
  for (int i = 0; i < kRouteMost; ++i) {
    const int e = i * kWave + lane;
    if (e < experts) gates[(size_t)row * experts + e] = (chosen >> i & 1u) ? s[i] : 0.0f;
  }
  kept = wave_sum(kept);
  if (lane == 0) keep[row] = kept;
}

__global__ __launch_bounds__(256) void route_top_kernel(const float* __restrict__ logits, const float* __restrict__ correction, int rows,
                                                        int n, int experts, int top, float* __restrict__ gates,
                                                        float* __restrict__ keep, int group_count, int group_keep) {
  const int row = blockIdx.x * 4 + threadIdx.x / kWave;
  if (row >= rows) return;
  route_row(logits + (size_t)row * n, correction, row, n, experts, top, gates, keep, threadIdx.x % kWave, group_count, group_keep);
}

// the dot products of R rows with every output's weights, into `out` [R][n] (LDS or global memory with a row stride
// of n); `xs`: the rows as floats in LDS [R][width].  A wave an output at a time, four channels a lane and load.
template <int R>
__device__ __forceinline__ void router_dots(const float* xs, const float* __restrict__ w, float* out, int n, int width) {
  const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave, waves = blockDim.x / kWave;
  for (int e = wave; e < n; e += waves) {
    float acc[R];
#pragma unroll
    for (int r = 0; r < R; ++r) acc[r] = 0.0f;
    const float* row = w + (size_t)e * width;
    if (width % 4 == 0) {
#pragma unroll 4
      for (int c = 4 * lane; c < width; c += 4 * kWave) {
        const float4 wv = *(const float4*)(row + c);
#pragma unroll
        for (int r = 0; r < R; ++r) {
          const float4 xv = *(const float4*)(xs + r * width + c);
          acc[r] = fmaf(xv.x, wv.x, fmaf(xv.y, wv.y, fmaf(xv.z, wv.z, fmaf(xv.w, wv.w, acc[r]))));
        }
      }
    } else {
#pragma unroll 4
      for (int c = lane; c < width; c += kWave) {
        const float wv = row[c];
#pragma unroll
        for (int r = 0; r < R; ++r) acc[r] = fmaf(xs[r * width + c], wv, acc[r]);
      }
    }
#pragma unroll
    for (int r = 0; r < R; ++r) {
      const float total = wave_sum(acc[r]);
      if (lane == 0) out[r * n + e] = total;
    }
  }
}

// Logits and choice in one kernel: a block takes R rows (as floats in LDS), its waves the outputs' dot products into
// LDS, then wave r routes row r.
template <int R>
__global__ __launch_bounds__(R == 1 ? 1024 : 256) void route_kernel(const void* __restrict__ x, int x_dtype, const float* __restrict__ w,
                                                    const float* __restrict__ correction, int rows, int n, int width, int experts,
                                                    int top, float* __restrict__ gates, float* __restrict__ keep, int group_count,
                                                    int group_keep) {
  extern __shared__ __attribute__((aligned(16))) float lds[];  // [R][width] rows, then [R][n] logits
  float* xs = lds;
  float* lg = lds + (size_t)R * width;
  const int row0 = blockIdx.x * R;
  for (int i = threadIdx.x; i < R * width; i += blockDim.x) {
    const int r = i / width;
    xs[i] = row0 + r < rows ? load_as_f32(x, x_dtype, (size_t)(row0 + r) * width + i % width) : 0.0f;
  }
  __syncthreads();
  router_dots<R>(xs, w, lg, n, width);
  __syncthreads();
  const int wave = threadIdx.x / kWave;
  if (wave < R && row0 + wave < rows)
    route_row(lg + wave * n, correction, row0 + wave, n, experts, top, gates, keep, threadIdx.x % kWave, group_count, group_keep);
}

// the logits alone, to global memory [rows, n]
template <int R>
__global__ __launch_bounds__(256) void router_logits_kernel(const void* __restrict__ x, int x_dtype, const float* __restrict__ w,
                                                            float* __restrict__ logits, int rows, int n, int width) {
  extern __shared__ __attribute__((aligned(16))) float xs[];  // [R][width]
  const int row0 = blockIdx.x * R;
  for (int i = threadIdx.x; i < R * width; i += blockDim.x) {
    const int r = i / width;
    xs[i] = row0 + r < rows ? load_as_f32(x, x_dtype, (size_t)(row0 + r) * width + i % width) : 0.0f;
  }
  __syncthreads();
  const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave, waves = blockDim.x / kWave;
  for (int e = wave; e < n; e += waves) {
    const float* row = w + (size_t)e * width;
    float acc[R];
#pragma unroll
    for (int r = 0; r < R; ++r) acc[r] = 0.0f;
#pragma unroll 4
    for (int c = lane; c < width; c += kWave) {
      const float wv = row[c];
#pragma unroll
      for (int r = 0; r < R; ++r) acc[r] = fmaf(xs[r * width + c], wv, acc[r]);
    }
#pragma unroll
    for (int r = 0; r < R; ++r) {
      const float total = wave_sum(acc[r]);
      if (lane == 0 && row0 + r < rows) logits[(size_t)(row0 + r) * n + e] = total;
    }
  }
}

// out[row, e * ff + c] = gates[row, e] * relu(z[row, e * ff + c])^2
__global__ void routed_act_kernel(const void* __restrict__ z, int z_dtype, const float* __restrict__ gates, void* __restrict__ out,
                                  int out_dtype, int experts, int ff, size_t total) {
  const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= total) return;
  const size_t per_row = (size_t)experts * ff;
  const size_t row = i / per_row;
  const int e = (int)((i % per_row) / ff);
  const float g = gates[row * experts + e];
  const float v = fmaxf(load_as_f32(z, z_dtype, i), 0.0f);
  store_from_f32(out, out_dtype, i, g == 0.0f ? 0.0f : g * v * v);
}

// The gated form: z [rows, experts * 2 * ff], an expert's gate columns then its up columns;
// out[row, e * ff + c] = gates[row, e] * silu(z[row, e * 2 ff + c]) * z[row, e * 2 ff + ff + c]
__global__ void routed_gated_kernel(const void* __restrict__ z, int z_dtype, const float* __restrict__ gates, void* __restrict__ out,
                                    int out_dtype, int experts, int ff, size_t total) {
  const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= total) return;
  const size_t per_row = (size_t)experts * ff;
  const size_t row = i / per_row;
  const int e = (int)((i % per_row) / ff), c = (int)(i % ff);
  const float g = gates[row * experts + e];
  float v = 0.0f;
  if (g != 0.0f) {
    const size_t at = (row * experts + e) * 2 * (size_t)ff + c;
    const float a = load_as_f32(z, z_dtype, at), u = load_as_f32(z, z_dtype, at + ff);
    v = g * (a * sigmoid_f(a) * u);
  }
  store_from_f32(out, out_dtype, i, v);
}

// the gated form, eight bfloat16 values a thread (ff a multiple of 8); the gating itself rounds to bfloat16 before the score weighs it
__global__ void routed_gated_bf16x8_kernel(const bf16_t* __restrict__ z, const float* __restrict__ gates, bf16_t* __restrict__ out,
                                           int experts, int ff8, size_t total8) {
  const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= total8) return;
  const size_t per_row = (size_t)experts * ff8;
  const size_t row = i / per_row;
  const int e = (int)((i % per_row) / ff8), c8 = (int)(i % ff8);
  const float g = gates[row * experts + e];
  typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8_t;
  bf16x8_t o = {};
  if (g != 0.0f) {
    const bf16_t* at = z + ((row * experts + e) * 2 * (size_t)ff8 + c8) * 8;
    const bf16x8_t a = *(const bf16x8_t*)at, u = *(const bf16x8_t*)(at + (size_t)ff8 * 8);
#pragma unroll
    for (int k = 0; k < 8; ++k) {
      const float av = (float)a[k];
      o[k] = (__bf16)(g * (av * sigmoid_f(av) * (float)u[k]));
    }
  }
  *(bf16x8_t*)(out + i * 8) = o;
}

// the same, eight bfloat16 values a thread (ff a multiple of 8)
__global__ void routed_act_bf16x8_kernel(const bf16_t* __restrict__ z, const float* __restrict__ gates, bf16_t* __restrict__ out,
                                         int experts, int ff8, size_t total8) {
  const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= total8) return;
  const size_t per_row = (size_t)experts * ff8;
  const size_t row = i / per_row;
  const int e = (int)((i % per_row) / ff8);
  const float g = gates[row * experts + e];
  typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8_t;
  bf16x8_t v = g == 0.0f ? bf16x8_t{} : *(const bf16x8_t*)(z + i * 8);
  bf16x8_t o;
#pragma unroll
  for (int k = 0; k < 8; ++k) {
    const float a = fmaxf((float)v[k], 0.0f);
    o[k] = (__bf16)(g == 0.0f ? 0.0f : g * a * a);
  }
  *(bf16x8_t*)(out + i * 8) = o;
}

// y[row, c] += keep[row] * h[row, c]
__global__ void rows_axpy_kernel(void* __restrict__ y, int y_dtype, const void* __restrict__ h, int h_dtype,
                                 const float* __restrict__ keep, int width, size_t total) {
  const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= total) return;
  const float k = keep[i / width];
  if (k != 0.0f) store_from_f32(y, y_dtype, i, fmaf(k, load_as_f32(h, h_dtype, i), load_as_f32(y, y_dtype, i)));
}

// o[row, c] *= sigmoid(g[row * g_stride + c])
__global__ void sigmoid_gate_kernel(void* __restrict__ o, int o_dtype, const void* __restrict__ g, int g_dtype, int g_stride,
                                    int width, size_t total) {
  const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= total) return;
  const size_t row = i / width;
  const int c = (int)(i % width);
  store_from_f32(o, o_dtype, i, load_as_f32(o, o_dtype, i) * sigmoid_f(load_as_f32(g, g_dtype, row * g_stride + c)));
}

// -----------------------------------------------------------------------------
// Queries and keys of a fused projection's rows, head by head: an RMS norm over the head's channels with a weight
// shared by the heads (or none), then the rotation of the first rot_dim channels by the token's position -- channel
// 2i with 2i + 1 (`neighbours`) or channel i with i + rot_dim / 2 --, pair i by the angle whose cosine and sine are
// table[pos][i].  Queries go to q_out [tokens, heads * head_dim]; keys and the values beside them into the pages of
// the token's slot.  A wave a (token, head); a key head's wave also copies its value head.
// -----------------------------------------------------------------------------
constexpr int kHeadMost = 1024;

struct HeadWriteArgs {
  const void* rows;  // [tokens, stride]
  int dtype, stride;
  int q_col, k_col, v_col;  // first columns of the queries, keys and values in a row; k_col < 0: no keys or values
  void* q_out;
  int q_dtype;
  const void* q_weight;  // [head_dim] or null
  const void* k_weight;
  int w_dtype;
  float eps;
  const float* cos_table;  // [positions][rot_dim / 2] or null
  const float* sin_table;
  int table_positions, rot_dim, neighbours;
  const int* tok_slot;
  const int* tok_pos;
  void* k_pages;
  void* v_pages;
  int cache_dtype;
  const int* block_table;
  int max_pages;
  int heads, kv_heads, head_dim, value_dim;
};

__global__ __launch_bounds__(64) void head_norm_write_kernel(HeadWriteArgs a) {
  __shared__ float row[kHeadMost];
  const int token = blockIdx.x;
  const int head = blockIdx.y;
  const int lane = threadIdx.x;
  const int slot = a.tok_slot[token];
  if (slot < 0) return;
  const int pos = a.tok_pos[token];
  const bool is_key = head >= a.heads;
  const int hd = a.head_dim;
  const size_t in = (size_t)token * a.stride + (is_key ? a.k_col + (head - a.heads) * hd : a.q_col + head * hd);
  const void* weight = is_key ? a.k_weight : a.q_weight;
  float ss = 0.0f;
  for (int d = lane; d < hd; d += kWave) {
    const float v = load_as_f32(a.rows, a.dtype, in + d);
    row[d] = v;
    ss = fmaf(v, v, ss);
  }
  ss = wave_sum(ss);
  __syncthreads();
  if (weight) {
    const float inv = 1.0f / sqrtf(ss / (float)hd + a.eps);
    for (int d = lane; d < hd; d += kWave) row[d] = row[d] * inv * load_as_f32(weight, a.w_dtype, d);
    __syncthreads();
  }
  const bool rotate = a.cos_table != nullptr && pos < a.table_positions;
  const int half = a.rot_dim / 2;
  int page = -1;
  if (is_key) page = a.block_table[(size_t)slot * a.max_pages + pos / kPageTokens];
  const int in_page = pos % kPageTokens;
  for (int d = lane; d < hd; d += kWave) {
    float v = row[d];
    if (rotate && d < a.rot_dim) {
      int pair, partner;
      bool first;
      if (a.neighbours) {
        pair = d / 2, first = (d % 2) == 0, partner = first ? d + 1 : d - 1;
      } else {
        first = d < half, pair = first ? d : d - half, partner = first ? d + half : d - half;
      }
      const float c = a.cos_table[(size_t)pos * half + pair], s = a.sin_table[(size_t)pos * half + pair];
      v = first ? v * c - row[partner] * s : v * c + row[partner] * s;
    }
    if (!is_key) {
      store_from_f32(a.q_out, a.q_dtype, ((size_t)token * a.heads + head) * hd + d, v);
    } else {
      const size_t dst = ((size_t)page * a.kv_heads + (head - a.heads)) * nnis_k_page_elems(hd);
      store_from_f32(a.k_pages, a.cache_dtype, dst + nnis_k_offset(in_page, d), v);
    }
  }
  if (is_key) {
    const int kv_head = head - a.heads;
    const int vd = a.value_dim;
    const size_t src = (size_t)token * a.stride + a.v_col + (size_t)kv_head * vd;
    const size_t dst = ((size_t)page * a.kv_heads + kv_head) * nnis_v_page_elems(vd);
    for (int d = lane; d < vd; d += kWave)
      store_from_f32(a.v_pages, a.cache_dtype, dst + nnis_v_offset(d, in_page), load_as_f32(a.rows, a.dtype, src + d));
  }
}

// -----------------------------------------------------------------------------
// Pooled blocks: a token at position p with (p + 1) % pool == 0 completes block b = p / pool of its sequence; the
// block's key is the mean of its `pool` keys as the pages hold them, its value the mean of their values; both go to
// entry b of a second set of pages with a block table of its own.  Runs behind the step's cache write.  A sequence
// that brings n tokens from position p0 completes (p0 + n) / pool - p0 / pool blocks; the launch has a block for every
// one that the step's sequences can complete between them (tokens / pool + sequences), and each finds its
// (sequence, block) by counting through the sequences.
// -----------------------------------------------------------------------------
struct PoolArgs {
  const void* k_pages;
  const void* v_pages;
  int cache_dtype;
  const int* block_table;
  int max_pages;
  void* pool_k;
  void* pool_v;
  const int* pool_table;
  int pool_max_pages;
  const int* seq_slot;
  const int* seq_start;
  const int* seq_pos0;
  int batch;
  int kv_heads, head_dim, value_dim, pool;
};

// A block a (token that completes a block, key/value head).  Keys: a lane takes a token of the block, a wave a chunk of
// eight channels at a time (sixteen or thirty-two bytes of one token, next to each other in the page); the lanes'
// sums meet by shuffles.  Values: a page keeps eight tokens of a channel together, so a lane takes a channel and a
// wave runs over the block's tokens.
constexpr int kPoolMostValueChannels = 4096;  // (the waves' sums of a head's values meet in LDS)

template <typename CacheT>
__global__ __launch_bounds__(256) void pool_blocks_kernel(PoolArgs a) {
  const int kv_head = blockIdx.y;
  int left = blockIdx.x, slot = -1, b = 0;
  for (int i = 0; i < a.batch; ++i) {
    const int s = a.seq_slot[i];
    if (s < 0) continue;  // a padding row
    const int p0 = a.seq_pos0[i], n = a.seq_start[i + 1] - a.seq_start[i];
    const int count = (p0 + n) / a.pool - p0 / a.pool;
    if (left < count) {
      slot = s;
      b = p0 / a.pool + left;
      break;
    }
    left -= count;
  }
  if (slot < 0) return;  // fewer blocks were completed than the launch has room for
  const int first = b * a.pool;
  const int* pages = a.block_table + (size_t)slot * a.max_pages;
  const int out_page = a.pool_table[(size_t)slot * a.pool_max_pages + b / kPageTokens];
  const int out_at = b % kPageTokens;
  const float share = 1.0f / (float)a.pool;
  const int hd = a.head_dim, vd = a.value_dim;
  const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave, waves = blockDim.x / kWave;
  const CacheT* k_pages = (const CacheT*)a.k_pages;
  const CacheT* v_pages = (const CacheT*)a.v_pages;
  const size_t out = (size_t)out_page * a.kv_heads + kv_head;
  const int chunks = (hd + 7) / 8;
  for (int chunk = wave; chunk < chunks; chunk += waves) {
    float sum[8] = {0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f};
    for (int j = lane; j < a.pool; j += kWave) {
      const int p = first + j;
      const CacheT* at = k_pages + ((size_t)pages[p / kPageTokens] * a.kv_heads + kv_head) * nnis_k_page_elems(hd) + nnis_k_offset(p % kPageTokens, 8 * chunk);
#pragma unroll
      for (int e = 0; e < 8; ++e) sum[e] += to_f32(at[e]);
    }
#pragma unroll
    for (int e = 0; e < 8; ++e) sum[e] = wave_sum(sum[e]);
    if (lane < 8 && 8 * chunk + lane < hd) {
      float mine = sum[0];
#pragma unroll
      for (int e = 1; e < 8; ++e) mine = lane == e ? sum[e] : mine;
      ((CacheT*)a.pool_k)[out * nnis_k_page_elems(hd) + nnis_k_offset(out_at, 8 * chunk + lane)] = from_f32<CacheT>(mine * share);
    }
  }
  // values: lanes on channels, waves on the groups of eight tokens that a page keeps together for a channel (the
  // block's first and last group may reach beyond it: those tokens are left out); the waves' sums meet in LDS
  extern __shared__ float part_lds[];  // [waves][vd]
  const int group_first = first / 8, group_last = (first + a.pool - 1) / 8;
  for (int c0 = 0; c0 < vd; c0 += kWave) {
    const int c = c0 + lane;
    float sum = 0.0f;
    if (c < vd) {
      for (int group = group_first + wave; group <= group_last; group += waves) {
        const int p0 = 8 * group;
        const CacheT* at = v_pages + ((size_t)pages[p0 / kPageTokens] * a.kv_heads + kv_head) * nnis_v_page_elems(vd) + nnis_v_offset(c, p0 % kPageTokens);
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const float v = to_f32(at[e]);
          sum += (p0 + e >= first && p0 + e < first + a.pool) ? v : 0.0f;
        }
      }
      part_lds[wave * vd + c] = sum;
    }
  }
  __syncthreads();
  for (int c = threadIdx.x; c < vd; c += blockDim.x) {
    float sum = 0.0f;
    for (int w = 0; w < waves; ++w) sum += part_lds[w * vd + c];
    ((CacheT*)a.pool_v)[out * nnis_v_page_elems(vd) + nnis_v_offset(c, out_at)] = from_f32<CacheT>(sum * share);
  }
}

// out[r, :] = x[rows ? rows[r] : r, :] in the output's type
__global__ void cast_rows_kernel(const void* __restrict__ x, int x_dtype, void* __restrict__ out, int out_dtype,
                                 const int* __restrict__ rows, int width, size_t total) {
  const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= total) return;
  const size_t r = i / width;
  const size_t from = rows ? (size_t)rows[r] * width + i % width : i;
  store_from_f32(out, out_dtype, i, load_as_f32(x, x_dtype, from));
}

inline unsigned blocks_for(size_t total, int threads) { return (unsigned)((total + threads - 1) / threads); }

}  // namespace

extern "C" int nnis_cast_rows(const void* x, int x_dtype, void* out, int out_dtype, const int* rows, int out_rows, int width, void* stream) {
  NNIS_REQUIRE(x && out && width > 0, "cast_rows: missing operand");
  NNIS_REQUIRE(nnis_dtype_ok(x_dtype) && nnis_dtype_ok(out_dtype), "cast_rows: unknown dtype");
  if (out_rows <= 0) return 0;
  const size_t total = (size_t)out_rows * width;
  hipLaunchKernelGGL(cast_rows_kernel, dim3(blocks_for(total, 256)), dim3(256), 0, (hipStream_t)stream, x, x_dtype, out, out_dtype, rows,
                     width, total);
  NNIS_LAUNCH_CHECK("cast_rows");
  return 0;
}

extern "C" int nnis_rms_post_step(float* x, const void* y, int y_dtype, const void* weight, int w_dtype, float offset, float eps,
                                  void* h, int h_dtype, int rows, int width, const float* keep, const void* h_in, int h_in_dtype,
                                  void* stream) {
  NNIS_REQUIRE(x && y && weight && width > 0, "rms_post_step: missing operand");
  NNIS_REQUIRE((keep == nullptr) == (h_in == nullptr) && (h_in == nullptr || nnis_dtype_ok(h_in_dtype)), "rms_post_step: a share of rows needs both");
  NNIS_REQUIRE(nnis_dtype_ok(y_dtype) && nnis_dtype_ok(w_dtype) && (h == nullptr || nnis_dtype_ok(h_dtype)), "rms_post_step: unknown dtype");
  if (rows <= 0) return 0;
  // four channels a thread where the types and the row's length allow
  const int threads4 = width >= 2048 ? 256 : (width >= 512 ? 128 : 64);
  const bool fits4 = width % 4 == 0 && width <= 4 * kPostKeep4 * threads4 && w_dtype == NNIS_F32 && (uintptr_t)y % 16 == 0 &&
                     (uintptr_t)weight % 16 == 0 && (h == nullptr || (uintptr_t)h % 16 == 0) && (h_in == nullptr || (uintptr_t)h_in % 16 == 0) &&
                     (h_in == nullptr || h_in_dtype == y_dtype);
  if (fits4 && y_dtype == NNIS_BF16 && (h == nullptr || h_dtype == NNIS_BF16)) {
    hipLaunchKernelGGL(rms_post_step4_kernel<bf16_t>, dim3(rows), dim3(threads4), 0, (hipStream_t)stream, x, (const bf16_t*)y,
                       (const float*)weight, offset, eps, (bf16_t*)h, width, keep, (const bf16_t*)h_in);
    NNIS_LAUNCH_CHECK("rms_post_step");
    return 0;
  }
  if (fits4 && y_dtype == NNIS_F32 && (h == nullptr || h_dtype == NNIS_F32)) {
    hipLaunchKernelGGL(rms_post_step4_kernel<float>, dim3(rows), dim3(threads4), 0, (hipStream_t)stream, x, (const float*)y,
                       (const float*)weight, offset, eps, (float*)h, width, keep, (const float*)h_in);
    NNIS_LAUNCH_CHECK("rms_post_step");
    return 0;
  }
  hipLaunchKernelGGL(rms_post_step_kernel, dim3(rows), dim3(width >= 1024 ? 256 : (width >= 256 ? 128 : 64)), 0, (hipStream_t)stream, x, y,
                     y_dtype, weight, w_dtype, offset, eps, h, h_dtype, width, keep, h_in, h_in_dtype);
  NNIS_LAUNCH_CHECK("rms_post_step");
  return 0;
}

extern "C" int nnis_rms_between(float* x, const void* y, int y_dtype, const void* w_out, const void* w_in, int w_dtype, float eps, void* h,
                                int h_dtype, int rows, int width, const float* keep, const void* h_in, int h_in_dtype, void* stream) {
  NNIS_REQUIRE(x && y && w_out && width > 0 && eps > 0.0f, "rms_between: missing operand");
  NNIS_REQUIRE((h == nullptr) == (w_in == nullptr), "rms_between: the rows out come with the next norm's weight");
  NNIS_REQUIRE((keep == nullptr) == (h_in == nullptr) && (h_in == nullptr || nnis_dtype_ok(h_in_dtype)), "rms_between: a share of rows needs both");
  NNIS_REQUIRE(nnis_dtype_ok(y_dtype) && nnis_dtype_ok(w_dtype) && (h == nullptr || nnis_dtype_ok(h_dtype)), "rms_between: unknown dtype");
  if (rows <= 0) return 0;
  // four channels a thread where the types and the row's length allow
  const int threads4 = width >= 2048 ? 256 : (width >= 512 ? 128 : 64);
  const bool fits4 = width % 4 == 0 && width <= 4 * kPostKeep4 * threads4 && (uintptr_t)y % 16 == 0 && (uintptr_t)x % 16 == 0 &&
                     (uintptr_t)w_out % 16 == 0 && (uintptr_t)w_in % 16 == 0 && (uintptr_t)h % 16 == 0 && (uintptr_t)h_in % 16 == 0 &&
                     (h == nullptr || h_dtype == y_dtype) && (h_in == nullptr || h_in_dtype == y_dtype);
#define NNIS_BETWEEN4(T_, W_)                                                                                                     \
  hipLaunchKernelGGL((rms_between4_kernel<T_, W_>), dim3(rows), dim3(threads4), 0, (hipStream_t)stream, x, (const T_*)y, (const W_*)w_out, \
                     (const W_*)w_in, eps, (T_*)h, width, keep, (const T_*)h_in)
  if (fits4 && (y_dtype == NNIS_BF16 || w_dtype == NNIS_F32)) {
    if (y_dtype == NNIS_BF16 && w_dtype == NNIS_BF16) NNIS_BETWEEN4(bf16_t, bf16_t);
    else if (y_dtype == NNIS_BF16) NNIS_BETWEEN4(bf16_t, float);
    else NNIS_BETWEEN4(float, float);
    NNIS_LAUNCH_CHECK("rms_between");
    return 0;
  }
#undef NNIS_BETWEEN4
  hipLaunchKernelGGL(rms_between_kernel, dim3(rows), dim3(width >= 1024 ? 256 : (width >= 256 ? 128 : 64)), 0, (hipStream_t)stream, x, y,
                     y_dtype, w_out, w_in, w_dtype, eps, h, h_dtype, width, keep, h_in, h_in_dtype);
  NNIS_LAUNCH_CHECK("rms_between");
  return 0;
}

extern "C" int nnis_poly_norm(const void* z, int z_dtype, const float* coef, float eps, void* out, int out_dtype, int rows, int width,
                              void* stream) {
  NNIS_REQUIRE(z && coef && out && width > 0, "poly_norm: missing operand");
  NNIS_REQUIRE(nnis_dtype_ok(z_dtype) && nnis_dtype_ok(out_dtype), "poly_norm: unknown dtype");
  if (rows <= 0) return 0;
  const int threads4 = width >= 2048 ? 256 : (width >= 512 ? 128 : 64);
  if (width % 4 == 0 && width <= 4 * kPolyKeep4 * threads4 && z_dtype == out_dtype && (uintptr_t)z % 16 == 0 && (uintptr_t)out % 16 == 0) {
    if (z_dtype == NNIS_BF16) {
      hipLaunchKernelGGL(poly_norm4_kernel<bf16_t>, dim3(rows), dim3(threads4), 0, (hipStream_t)stream, (const bf16_t*)z, coef, eps, (bf16_t*)out, width);
    } else {
      hipLaunchKernelGGL(poly_norm4_kernel<float>, dim3(rows), dim3(threads4), 0, (hipStream_t)stream, (const float*)z, coef, eps, (float*)out, width);
    }
    NNIS_LAUNCH_CHECK("poly_norm");
    return 0;
  }
  hipLaunchKernelGGL(poly_norm_kernel, dim3(rows), dim3(width >= 1024 ? 256 : (width >= 256 ? 128 : 64)), 0, (hipStream_t)stream, z, z_dtype,
                     coef, eps, out, out_dtype, width);
  NNIS_LAUNCH_CHECK("poly_norm");
  return 0;
}

extern "C" int nnis_router_logits(const void* x, int x_dtype, const float* w, float* logits, int rows, int n, int width, void* stream) {
  NNIS_REQUIRE(x && w && logits && n > 0 && width > 0, "router_logits: missing operand");
  NNIS_REQUIRE(nnis_dtype_ok(x_dtype), "router_logits: unknown dtype");
  NNIS_REQUIRE(width <= 16384, "router_logits: rows of up to 16384 channels, got %d", width);
  if (rows <= 0) return 0;
  // several rows a block where they fit 48 KB of LDS and there are rows enough to fill the chip with such blocks
  const int together = rows <= 256 ? 1 : (width <= 3072 ? 4 : (width <= 6144 ? 2 : 1));
  const size_t lds = (size_t)together * width * sizeof(float);
  const dim3 grid((rows + together - 1) / together);
  if (together == 4) {
    hipLaunchKernelGGL((router_logits_kernel<4>), grid, dim3(256), lds, (hipStream_t)stream, x, x_dtype, w, logits, rows, n, width);
  } else if (together == 2) {
    hipLaunchKernelGGL((router_logits_kernel<2>), grid, dim3(256), lds, (hipStream_t)stream, x, x_dtype, w, logits, rows, n, width);
  } else {
    hipLaunchKernelGGL((router_logits_kernel<1>), grid, dim3(256), lds, (hipStream_t)stream, x, x_dtype, w, logits, rows, n, width);
  }
  NNIS_LAUNCH_CHECK("router_logits");
  return 0;
}

extern "C" int nnis_route(const void* x, int x_dtype, const float* w, const float* correction, int rows, int n, int width, int experts, int top,
                          float* gates, float* keep, int group_count, int group_keep, void* stream) {
  NNIS_REQUIRE(x && w && gates && keep && n > 0 && width > 0, "route: missing operand");
  NNIS_REQUIRE(group_count >= 1 && group_count <= kWave && n % group_count == 0 && group_keep >= 1 && group_keep <= group_count,
               "route: %d outputs in %d groups (up to %d, equal ones) of which %d are kept", n, group_count, kWave, group_keep);
  NNIS_REQUIRE(nnis_dtype_ok(x_dtype), "route: unknown dtype");
  NNIS_REQUIRE(n <= kWave * kRouteMost && width <= 8192, "route: up to %d outputs of rows of up to 8192 channels, got %d and %d", kWave * kRouteMost,
               n, width);
  NNIS_REQUIRE(experts >= 0 && experts <= n && top > 0 && top <= n, "route: %d experts and the %d largest of %d outputs", experts, top, n);
  if (rows <= 0) return 0;
  // several rows a block where they fit 48 KB of LDS and there are rows enough to fill the chip with such blocks
  const int together = rows <= 256 ? 1 : ((size_t)4 * (width + n) * 4 <= 49152 ? 4 : ((size_t)2 * (width + n) * 4 <= 49152 ? 2 : 1));
  const size_t lds = (size_t)together * (width + n) * sizeof(float);
  const dim3 grid((rows + together - 1) / together);
  hipStream_t s = (hipStream_t)stream;
  if (together == 4) {
    hipLaunchKernelGGL((route_kernel<4>), grid, dim3(256), lds, s, x, x_dtype, w, correction, rows, n, width, experts, top, gates, keep,
                       group_count, group_keep);
  } else if (together == 2) {
    hipLaunchKernelGGL((route_kernel<2>), grid, dim3(256), lds, s, x, x_dtype, w, correction, rows, n, width, experts, top, gates, keep,
                       group_count, group_keep);
  } else {
    // a row a block: a wave an output where the outputs are many, so that every weight row is asked for at once
    const int threads = n > 8 ? 1024 : (n > 4 ? 512 : 256);
    hipLaunchKernelGGL((route_kernel<1>), grid, dim3(threads), lds, s, x, x_dtype, w, correction, rows, n, width, experts, top, gates, keep,
                       group_count, group_keep);
  }
  NNIS_LAUNCH_CHECK("route");
  return 0;
}

extern "C" int nnis_route_top(const float* logits, const float* correction, int rows, int n, int experts, int top, float* gates,
                              float* keep, int group_count, int group_keep, void* stream) {
  NNIS_REQUIRE(logits && gates && keep, "route_top: missing operand");
  NNIS_REQUIRE(group_count >= 1 && group_count <= kWave && n % group_count == 0 && group_keep >= 1 && group_keep <= group_count,
               "route_top: %d outputs in %d groups (up to %d, equal ones) of which %d are kept", n, group_count, kWave, group_keep);
  NNIS_REQUIRE(n > 0 && n <= kWave * kRouteMost, "route_top: 1 to %d router outputs, got %d", kWave * kRouteMost, n);
  NNIS_REQUIRE(experts >= 0 && experts <= n && top > 0 && top <= n, "route_top: %d experts and the %d largest of %d outputs", experts, top, n);
  if (rows <= 0) return 0;
  hipLaunchKernelGGL(route_top_kernel, dim3((rows + 3) / 4), dim3(256), 0, (hipStream_t)stream, logits, correction, rows, n, experts, top,
                     gates, keep, group_count, group_keep);
  NNIS_LAUNCH_CHECK("route_top");
  return 0;
}

// form 0: z [rows, experts * ff], out = score * relu(z)^2; form 1: z [rows, experts * 2 * ff] (gate columns, then up
// columns, expert by expert), out = score * silu(gate) * up
extern "C" int nnis_routed_act(const void* z, int z_dtype, const float* gates, void* out, int out_dtype, int rows, int experts, int ff,
                               int form, void* stream) {
  NNIS_REQUIRE(z && gates && out && experts > 0 && ff > 0, "routed_act: missing operand");
  NNIS_REQUIRE(nnis_dtype_ok(z_dtype) && nnis_dtype_ok(out_dtype), "routed_act: unknown dtype");
  NNIS_REQUIRE(form == 0 || form == 1, "routed_act: unknown form %d", form);
  if (rows <= 0) return 0;
  const size_t total = (size_t)rows * experts * ff;
  if (form == 1) {
    if (z_dtype == NNIS_BF16 && out_dtype == NNIS_BF16 && ff % 8 == 0 && (uintptr_t)z % 16 == 0 && (uintptr_t)out % 16 == 0) {
      hipLaunchKernelGGL(routed_gated_bf16x8_kernel, dim3(blocks_for(total / 8, 256)), dim3(256), 0, (hipStream_t)stream, (const bf16_t*)z,
                         gates, (bf16_t*)out, experts, ff / 8, total / 8);
    } else {
      hipLaunchKernelGGL(routed_gated_kernel, dim3(blocks_for(total, 256)), dim3(256), 0, (hipStream_t)stream, z, z_dtype, gates, out,
                         out_dtype, experts, ff, total);
    }
    NNIS_LAUNCH_CHECK("routed_act");
    return 0;
  }
  if (z_dtype == NNIS_BF16 && out_dtype == NNIS_BF16 && ff % 8 == 0 && (uintptr_t)z % 16 == 0 && (uintptr_t)out % 16 == 0) {
    hipLaunchKernelGGL(routed_act_bf16x8_kernel, dim3(blocks_for(total / 8, 256)), dim3(256), 0, (hipStream_t)stream, (const bf16_t*)z, gates,
                       (bf16_t*)out, experts, ff / 8, total / 8);
    NNIS_LAUNCH_CHECK("routed_act");
    return 0;
  }
  hipLaunchKernelGGL(routed_act_kernel, dim3(blocks_for(total, 256)), dim3(256), 0, (hipStream_t)stream, z, z_dtype, gates, out, out_dtype,
                     experts, ff, total);
  NNIS_LAUNCH_CHECK("routed_act");
  return 0;
}

extern "C" int nnis_rows_axpy(void* y, int y_dtype, const void* h, int h_dtype, const float* keep, int rows, int width, void* stream) {
  NNIS_REQUIRE(y && h && keep && width > 0, "rows_axpy: missing operand");
  NNIS_REQUIRE(nnis_dtype_ok(y_dtype) && nnis_dtype_ok(h_dtype), "rows_axpy: unknown dtype");
  if (rows <= 0) return 0;
  const size_t total = (size_t)rows * width;
  hipLaunchKernelGGL(rows_axpy_kernel, dim3(blocks_for(total, 256)), dim3(256), 0, (hipStream_t)stream, y, y_dtype, h, h_dtype, keep, width,
                     total);
  NNIS_LAUNCH_CHECK("rows_axpy");
  return 0;
}

extern "C" int nnis_sigmoid_gate(void* o, int o_dtype, const void* g, int g_dtype, int g_stride, int rows, int width, void* stream) {
  NNIS_REQUIRE(o && g && width > 0 && g_stride >= width, "sigmoid_gate: missing operand");
  NNIS_REQUIRE(nnis_dtype_ok(o_dtype) && nnis_dtype_ok(g_dtype), "sigmoid_gate: unknown dtype");
  if (rows <= 0) return 0;
  const size_t total = (size_t)rows * width;
  hipLaunchKernelGGL(sigmoid_gate_kernel, dim3(blocks_for(total, 256)), dim3(256), 0, (hipStream_t)stream, o, o_dtype, g, g_dtype, g_stride,
                     width, total);
  NNIS_LAUNCH_CHECK("sigmoid_gate");
  return 0;
}

extern "C" int nnis_head_norm_write(const void* rows, int dtype, int stride, int q_col, int k_col, int v_col, void* q_out, int q_dtype,
                                    const void* q_weight, const void* k_weight, int w_dtype, float eps, const float* cos_table,
                                    const float* sin_table, int table_positions, int rot_dim, int neighbours, const int* tok_slot,
                                    const int* tok_pos, void* k_pages, void* v_pages, int cache_dtype, const int* block_table,
                                    int max_pages, int tokens, int heads, int kv_heads, int head_dim, int value_dim, void* stream) {
  NNIS_REQUIRE(rows && q_out && tok_slot && tok_pos, "head_norm_write: missing operand");
  NNIS_REQUIRE(nnis_dtype_ok(dtype) && nnis_dtype_ok(q_dtype), "head_norm_write: unknown dtype");
  NNIS_REQUIRE(heads > 0 && kv_heads >= 0 && head_dim > 0 && head_dim <= kHeadMost, "head_norm_write: heads of 1 to %d channels, got %d",
               kHeadMost, head_dim);
  NNIS_REQUIRE(rot_dim >= 0 && rot_dim <= head_dim && rot_dim % 2 == 0, "head_norm_write: rot_dim %d must be even and at most head_dim %d",
               rot_dim, head_dim);
  NNIS_REQUIRE((cos_table == nullptr) == (sin_table == nullptr), "head_norm_write: cos and sin tables must come together");
  NNIS_REQUIRE((q_weight == nullptr && k_weight == nullptr) || nnis_dtype_ok(w_dtype), "head_norm_write: unknown weight dtype");
  if (kv_heads > 0) {
    NNIS_REQUIRE(k_col >= 0 && v_col >= 0 && k_pages && v_pages && block_table && max_pages > 0 && nnis_dtype_ok(cache_dtype) && value_dim > 0,
                 "head_norm_write: keys without pages to go to");
  }
  if (tokens <= 0) return 0;
  HeadWriteArgs a;
  a.rows = rows; a.dtype = dtype; a.stride = stride; a.q_col = q_col; a.k_col = k_col; a.v_col = v_col;
  a.q_out = q_out; a.q_dtype = q_dtype; a.q_weight = q_weight; a.k_weight = k_weight; a.w_dtype = w_dtype; a.eps = eps;
  a.cos_table = cos_table; a.sin_table = sin_table; a.table_positions = table_positions; a.rot_dim = cos_table ? rot_dim : 0;
  a.neighbours = neighbours; a.tok_slot = tok_slot; a.tok_pos = tok_pos; a.k_pages = k_pages; a.v_pages = v_pages;
  a.cache_dtype = cache_dtype; a.block_table = block_table; a.max_pages = max_pages;
  a.heads = heads; a.kv_heads = kv_heads; a.head_dim = head_dim; a.value_dim = value_dim;
  hipLaunchKernelGGL(head_norm_write_kernel, dim3(tokens, heads + kv_heads), dim3(64), 0, (hipStream_t)stream, a);
  NNIS_LAUNCH_CHECK("head_norm_write");
  return 0;
}

extern "C" int nnis_pool_blocks(const void* k_pages, const void* v_pages, int cache_dtype, const int* block_table, int max_pages,
                                void* pool_k, void* pool_v, const int* pool_table, int pool_max_pages, const int* seq_slot,
                                const int* seq_start, const int* seq_pos0, int batch, int tokens, int kv_heads, int head_dim,
                                int value_dim, int pool, void* stream) {
  NNIS_REQUIRE(k_pages && v_pages && block_table && pool_k && pool_v && pool_table && seq_slot && seq_start && seq_pos0,
               "pool_blocks: missing operand");
  NNIS_REQUIRE(nnis_dtype_ok(cache_dtype) && max_pages > 0 && pool_max_pages > 0, "pool_blocks: bad pages");
  NNIS_REQUIRE(kv_heads > 0 && head_dim > 0 && value_dim > 0 && pool > 0, "pool_blocks: bad sizes");
  NNIS_REQUIRE(value_dim <= kPoolMostValueChannels, "pool_blocks: values of up to %d channels, got %d", kPoolMostValueChannels, value_dim);
  if (tokens <= 0 || batch <= 0) return 0;
  PoolArgs a;
  a.k_pages = k_pages; a.v_pages = v_pages; a.cache_dtype = cache_dtype; a.block_table = block_table; a.max_pages = max_pages;
  a.pool_k = pool_k; a.pool_v = pool_v; a.pool_table = pool_table; a.pool_max_pages = pool_max_pages;
  a.seq_slot = seq_slot; a.seq_start = seq_start; a.seq_pos0 = seq_pos0; a.batch = batch; a.kv_heads = kv_heads; a.head_dim = head_dim; a.value_dim = value_dim; a.pool = pool;
  if (cache_dtype == NNIS_F32) {
    hipLaunchKernelGGL(pool_blocks_kernel<float>, dim3(tokens / pool + batch, kv_heads), dim3(256), (size_t)4 * value_dim * sizeof(float), (hipStream_t)stream, a);
  } else {
    hipLaunchKernelGGL(pool_blocks_kernel<bf16_t>, dim3(tokens / pool + batch, kv_heads), dim3(256), (size_t)4 * value_dim * sizeof(float), (hipStream_t)stream, a);
  }
  NNIS_LAUNCH_CHECK("pool_blocks");
  return 0;
}
