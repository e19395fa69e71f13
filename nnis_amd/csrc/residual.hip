// Row-wise kernels around a residual that is kept as several streams, and the small fused steps of mixers
// that run side by side: an embedding with a hashed table of token pairs, the streams' update and weighted
// sum fused with the norm that follows, the mean of branches each normed by its root mean square, a gated
// activation with a choice of activation, and a bias added in place.
// Storage types are chosen at run time; every sum and statistic is 32-bit.
#include "common.h"

// -----------------------------------------------------------------------------
// Embedding with a table of token pairs: out[c][t, :] = table[id] + pairs[row], the same in every one of
// `copies` copies.  row = (previous * mul_prev + id * mul_cur) % buckets, or `buckets` (the table's last
// row) for a sequence's first token.  The token before the first one a step brings for a sequence is kept
// per slot in `last_token`; the block of a run's first row reads it and then stores the run's last id
// there (no other block reads that word).  Rows of one sequence follow one another and a slot appears in
// one run only.  A padding row (negative slot or id outside the table) is zero.
// -----------------------------------------------------------------------------
__global__ void embed_pair_kernel(const int* __restrict__ ids, const int* __restrict__ tok_slot, const int* __restrict__ tok_pos,
                                  int tokens, const void* __restrict__ table, int table_dtype, int vocab,
                                  const void* __restrict__ pairs, int pairs_dtype, int buckets, long long mul_prev,
                                  long long mul_cur, int* __restrict__ last_token, float* __restrict__ out, int copies, int width) {
  __shared__ int s_before;
  const int token = blockIdx.x;
  const int id = ids[token];
  const int slot = tok_slot[token];
  const size_t plane = (size_t)tokens * width;
  float* dst = out + (size_t)token * width;
  if (slot < 0 || id < 0 || id >= vocab) {
    for (int c = threadIdx.x; c < width; c += blockDim.x)
      for (int s = 0; s < copies; ++s) dst[s * plane + c] = 0.0f;
    return;
  }
  const int pos = tok_pos[token];
  const bool starts_run = token == 0 || tok_slot[token - 1] != slot;
  if (threadIdx.x == 0) s_before = starts_run ? last_token[slot] : ids[token - 1];
  __syncthreads();
  const int before = s_before;
  if (starts_run) {
    // the last row of this run leaves its id for the step that comes next
    for (int r = token + threadIdx.x; r < tokens && tok_slot[r] == slot; r += blockDim.x)
      if (r + 1 == tokens || tok_slot[r + 1] != slot) last_token[slot] = ids[r];
  }
  long long row = buckets;
  if (pos > 0 && before >= 0) row = ((long long)before * mul_prev + (long long)id * mul_cur) % buckets;
  const size_t base = (size_t)id * width, pair_base = (size_t)row * width;
  for (int c = threadIdx.x; c < width; c += blockDim.x) {
    const float v = load_as_f32(table, table_dtype, base + c) + load_as_f32(pairs, pairs_dtype, pair_base + c);
    for (int s = 0; s < copies; ++s) dst[s * plane + c] = v;
  }
}

extern "C" int nnis_embed_pair(const int* ids, const int* tok_slot, const int* tok_pos, int tokens, const void* table,
                               int table_dtype, int vocab, const void* pairs, int pairs_dtype, int buckets, long long mul_prev,
                               long long mul_cur, int* last_token, float* out, int copies, int width, void* stream) {
  NNIS_REQUIRE(nnis_dtype_ok(table_dtype) && nnis_dtype_ok(pairs_dtype), "embed_pair: unknown table dtype");
  NNIS_REQUIRE(tokens >= 0 && width > 0 && vocab > 0 && buckets > 0 && copies > 0, "embed_pair: bad sizes");
  NNIS_REQUIRE(mul_prev >= 0 && mul_cur >= 0, "embed_pair: the multipliers must not be negative");
  NNIS_REQUIRE(ids && tok_slot && tok_pos && last_token && out, "embed_pair: a pointer is missing");
  if (tokens == 0) return 0;
  hipLaunchKernelGGL(embed_pair_kernel, dim3(tokens), dim3(width >= 1024 ? 256 : 64), 0, (hipStream_t)stream, ids, tok_slot,
                     tok_pos, tokens, table, table_dtype, vocab, pairs, pairs_dtype, buckets, mul_prev, mul_cur, last_token, out,
                     copies, width);
  NNIS_LAUNCH_CHECK("embed_pair");
  return 0;
}

// -----------------------------------------------------------------------------
// Streams.  x [streams, tokens, width] in 32-bit.  One block a row, in up to three steps:
//   update (y given):  x_t <- sum_s mix[s, t] x_s + gain[t] * y      all streams at once, in place
//   read:              u = sum_t take[t] x_t                         (take null: every stream counts once)
//   norm (weight given): h = (u - mean) / sqrt(var + eps) * weight + bias, var the mean squared deviation
//                        (centred = 0: h = u / sqrt(mean(u^2) + eps) * weight [+ bias])
// Without a norm weight, h = u.  With `rows`, output row r reads input row rows[r] (then nothing is updated).
// u is held in LDS between the passes (width floats).
// -----------------------------------------------------------------------------
constexpr int kMostStreams = 8;

struct StreamArgs {
  float* x;
  int streams, tokens, width;
  const void* y;  // [tokens, width] or null
  int y_dtype;
  const float* mix;   // [streams, streams], [from, to]
  const float* gain;  // [streams]
  const float* take;  // [streams] or null
  const void* weight;  // [width] or null
  const void* bias;    // [width] or null
  int weight_dtype;
  int centred;
  float eps;
  void* h;  // [out_rows, width] or null
  int h_dtype;
  const int* rows;
};

__global__ void stream_kernel(StreamArgs a) {
  extern __shared__ float u_row[];
  __shared__ float scratch[16];
  const int out_row = blockIdx.x;
  const int row = a.rows ? a.rows[out_row] : out_row;
  const int S = a.streams;
  const size_t plane = (size_t)a.tokens * a.width;
  float* x = a.x + (size_t)row * a.width;
  float mix[kMostStreams][kMostStreams], gain[kMostStreams], take[kMostStreams];
#pragma unroll
  for (int s = 0; s < kMostStreams; ++s) {
    take[s] = s < S ? (a.take ? a.take[s] : 1.0f) : 0.0f;
    gain[s] = (a.y && s < S) ? a.gain[s] : 0.0f;
#pragma unroll
    for (int t = 0; t < kMostStreams; ++t) mix[s][t] = (a.y && s < S && t < S) ? a.mix[s * S + t] : 0.0f;
  }
  float sum = 0.0f;
  for (int c = threadIdx.x; c < a.width; c += blockDim.x) {
    float v[kMostStreams];
#pragma unroll
    for (int s = 0; s < kMostStreams; ++s) v[s] = s < S ? x[s * plane + c] : 0.0f;
    if (a.y) {
      const float y = load_as_f32(a.y, a.y_dtype, (size_t)row * a.width + c);
      float w[kMostStreams];
#pragma unroll
      for (int t = 0; t < kMostStreams; ++t) {
        float acc = 0.0f;
#pragma unroll
        for (int s = 0; s < kMostStreams; ++s) acc = fmaf(mix[s][t], v[s], acc);
        w[t] = fmaf(gain[t], y, acc);
      }
#pragma unroll
      for (int t = 0; t < kMostStreams; ++t) {
        v[t] = w[t];
        if (t < S) x[t * plane + c] = w[t];
      }
    }
    float u = 0.0f;
#pragma unroll
    for (int s = 0; s < kMostStreams; ++s) u = fmaf(take[s], v[s], u);
    u_row[c] = u;
    sum += u;
  }
  if (a.h == nullptr) return;
  const size_t out_base = (size_t)out_row * a.width;
  if (a.weight == nullptr) {
    __syncthreads();
    for (int c = threadIdx.x; c < a.width; c += blockDim.x) store_from_f32(a.h, a.h_dtype, out_base + c, u_row[c]);
    return;
  }
  const float inv_width = 1.0f / (float)a.width;
  const float mean = a.centred ? block_sum(sum, scratch) * inv_width : 0.0f;  // (block_sum's barriers order the LDS writes)
  float squares = 0.0f;
  if (!a.centred) __syncthreads();
  for (int c = threadIdx.x; c < a.width; c += blockDim.x) {
    const float d = u_row[c] - mean;
    squares = fmaf(d, d, squares);
  }
  const float scale = 1.0f / sqrtf(block_sum(squares, scratch) * inv_width + a.eps);
  for (int c = threadIdx.x; c < a.width; c += blockDim.x) {
    float v = ((u_row[c] - mean) * scale) * load_as_f32(a.weight, a.weight_dtype, c);
    if (a.bias) v += load_as_f32(a.bias, a.weight_dtype, c);
    store_from_f32(a.h, a.h_dtype, out_base + c, v);
  }
}

// The same with a row in registers: a thread takes CH pieces of 4 channels of every stream, asks for all of them at
// once (the loop above waits for memory once a piece), and keeps u in registers.  Widths in steps of 4 up to
// 4096 * CH... channels a block of up to 1024 threads covers.
typedef __attribute__((ext_vector_type(4))) float f32x4_r;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4_r;

__device__ __forceinline__ f32x4_r load4_r(const void* base, int dtype, size_t index) {
  if (dtype == NNIS_F32) return *(const f32x4_r*)((const float*)base + index);
  const bf16x4_r v = *(const bf16x4_r*)((const bf16_t*)base + index);
  return (f32x4_r){(float)v[0], (float)v[1], (float)v[2], (float)v[3]};
}

__device__ __forceinline__ void store4_r(void* base, int dtype, size_t index, f32x4_r v) {
  if (dtype == NNIS_F32) {
    *(f32x4_r*)((float*)base + index) = v;
  } else {
    bf16x4_r packed;
#pragma unroll
    for (int e = 0; e < 4; ++e) packed[e] = (__bf16)v[e];
    *(bf16x4_r*)((bf16_t*)base + index) = packed;
  }
}

template <int CH, int SMAX>
__global__ __launch_bounds__(1024) void stream_wide_kernel(StreamArgs a) {
  __shared__ float scratch[16];
  const int out_row = blockIdx.x;
  const int row = a.rows ? a.rows[out_row] : out_row;
  const int S = a.streams;
  const size_t plane = (size_t)a.tokens * a.width;
  float* x = a.x + (size_t)row * a.width;
  f32x4_r v[SMAX][CH], y[CH];
  bool inside[CH];
#pragma unroll
  for (int i = 0; i < CH; ++i) {
    const int col = 4 * (threadIdx.x + i * blockDim.x);
    inside[i] = col < a.width;
#pragma unroll
    for (int s = 0; s < SMAX; ++s) v[s][i] = (inside[i] && s < S) ? *(const f32x4_r*)(x + s * plane + col) : (f32x4_r){0.0f, 0.0f, 0.0f, 0.0f};
    y[i] = (a.y && inside[i]) ? load4_r(a.y, a.y_dtype, (size_t)row * a.width + col) : (f32x4_r){0.0f, 0.0f, 0.0f, 0.0f};
  }
  float take[SMAX];
#pragma unroll
  for (int s = 0; s < SMAX; ++s) take[s] = s < S ? (a.take ? a.take[s] : 1.0f) : 0.0f;
  if (a.y) {
    float mix[SMAX][SMAX], gain[SMAX];
#pragma unroll
    for (int s = 0; s < SMAX; ++s) {
      gain[s] = s < S ? a.gain[s] : 0.0f;
#pragma unroll
      for (int t = 0; t < SMAX; ++t) mix[s][t] = (s < S && t < S) ? a.mix[s * S + t] : 0.0f;
    }
#pragma unroll
    for (int i = 0; i < CH; ++i) {
      f32x4_r w[SMAX];
#pragma unroll
      for (int t = 0; t < SMAX; ++t) {
        w[t] = gain[t] * y[i];
#pragma unroll
        for (int s = 0; s < SMAX; ++s) w[t] += mix[s][t] * v[s][i];
      }
#pragma unroll
      for (int t = 0; t < SMAX; ++t) {
        v[t][i] = w[t];
        if (inside[i] && t < S) *(f32x4_r*)(x + t * plane + 4 * (threadIdx.x + i * blockDim.x)) = w[t];
      }
    }
  }
  if (a.h == nullptr) return;
  f32x4_r u[CH];
  float sum = 0.0f;
#pragma unroll
  for (int i = 0; i < CH; ++i) {
    u[i] = (f32x4_r){0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
    for (int s = 0; s < SMAX; ++s) u[i] += take[s] * v[s][i];
    sum += (u[i][0] + u[i][1]) + (u[i][2] + u[i][3]);
  }
  const size_t out_base = (size_t)out_row * a.width;
  float mean = 0.0f, scale = 1.0f;
  if (a.weight) {
    const float inv_width = 1.0f / (float)a.width;
    if (a.centred) mean = block_sum(sum, scratch) * inv_width;
    float squares = 0.0f;
#pragma unroll
    for (int i = 0; i < CH; ++i)
      if (inside[i]) {
#pragma unroll
        for (int e = 0; e < 4; ++e) squares = fmaf(u[i][e] - mean, u[i][e] - mean, squares);
      }
    scale = 1.0f / sqrtf(block_sum(squares, scratch) * inv_width + a.eps);
  }
#pragma unroll
  for (int i = 0; i < CH; ++i) {
    const int col = 4 * (threadIdx.x + i * blockDim.x);
    if (!inside[i]) continue;
    f32x4_r out = u[i];
    if (a.weight) {
      out = ((u[i] - mean) * scale) * load4_r(a.weight, a.weight_dtype, col);
      if (a.bias) out += load4_r(a.bias, a.weight_dtype, col);
    }
    store4_r(a.h, a.h_dtype, out_base + col, out);
  }
}

extern "C" int nnis_stream_step(float* x, int streams, int tokens, int width, const void* y, int y_dtype, const float* mix,
                                const float* gain, const float* take, const void* weight, const void* bias, int weight_dtype,
                                int centred, float eps, void* h, int h_dtype, const int* rows, int out_rows, void* stream) {
  NNIS_REQUIRE(streams >= 1 && streams <= kMostStreams, "streams: 1 to %d streams are taken, got %d", kMostStreams, streams);
  NNIS_REQUIRE(tokens >= 0 && width > 0 && width <= 16384, "streams: bad sizes tokens=%d width=%d", tokens, width);
  NNIS_REQUIRE(x != nullptr, "streams: x is missing");
  NNIS_REQUIRE(y == nullptr || (nnis_dtype_ok(y_dtype) && mix && gain && rows == nullptr),
               "streams: an update needs mix and gain and no row list");
  NNIS_REQUIRE(h == nullptr || nnis_dtype_ok(h_dtype), "streams: unknown output dtype %d", h_dtype);
  NNIS_REQUIRE(weight == nullptr || (nnis_dtype_ok(weight_dtype) && eps > 0.0f && h != nullptr), "streams: a norm needs a weight type, eps and an output");
  NNIS_REQUIRE(bias == nullptr || weight != nullptr, "streams: a bias comes with a weight");
  NNIS_REQUIRE(h != nullptr || y != nullptr, "streams: nothing to do");
  if (out_rows <= 0) return 0;
  StreamArgs a;
  a.x = x; a.streams = streams; a.tokens = tokens; a.width = width; a.y = y; a.y_dtype = y_dtype; a.mix = mix; a.gain = gain;
  a.take = take; a.weight = weight; a.bias = bias; a.weight_dtype = weight_dtype; a.centred = centred; a.eps = eps; a.h = h;
  a.h_dtype = h_dtype; a.rows = rows;
  const bool aligned = ((uintptr_t)x % 16 == 0) && ((uintptr_t)y % 16 == 0) && ((uintptr_t)h % 16 == 0) && ((uintptr_t)weight % 16 == 0) &&
                       ((uintptr_t)bias % 16 == 0);
  if (width % 4 == 0 && aligned && width / 4 <= 2048) {
    const int pieces = width / 4;
    const int per = pieces > 1024 ? 2 : 1;
    const int block = ((pieces + per - 1) / per + 63) / 64 * 64;
    hipStream_t s = (hipStream_t)stream;
    if (streams <= 4) {
      if (per == 1) hipLaunchKernelGGL((stream_wide_kernel<1, 4>), dim3(out_rows), dim3(block), 0, s, a);
      else hipLaunchKernelGGL((stream_wide_kernel<2, 4>), dim3(out_rows), dim3(block), 0, s, a);
    } else {
      if (per == 1) hipLaunchKernelGGL((stream_wide_kernel<1, kMostStreams>), dim3(out_rows), dim3(block), 0, s, a);
      else hipLaunchKernelGGL((stream_wide_kernel<2, kMostStreams>), dim3(out_rows), dim3(block), 0, s, a);
    }
    NNIS_LAUNCH_CHECK("stream_step");
    return 0;
  }
  const int threads = width >= 2048 ? 256 : (width >= 512 ? 128 : 64);
  hipLaunchKernelGGL(stream_kernel, dim3(out_rows), dim3(threads), (size_t)width * sizeof(float), (hipStream_t)stream, a);
  NNIS_LAUNCH_CHECK("stream_step");
  return 0;
}

// -----------------------------------------------------------------------------
// Branches side by side: out = (1 / n) sum_i  (y_i + b_i) / sqrt(mean((y_i + b_i)^2) + eps) * w_i,
// the mean over the row.  Up to kMostBranches inputs [tokens, width], each with a weight and, optionally, a
// bias that its producer has not added yet.  One block a row.
// -----------------------------------------------------------------------------
constexpr int kMostBranches = 4;

struct BranchArgs {
  const void* y[kMostBranches];
  const void* weight[kMostBranches];
  const void* bias[kMostBranches];
  int count;
  int y_dtype, weight_dtype;
  int width;
  float eps;
  void* out;
  int out_dtype;
};

__global__ void branch_mean_kernel(BranchArgs a) {
  __shared__ float scratch[16];
  const size_t base = (size_t)blockIdx.x * a.width;
  float scale[kMostBranches];
#pragma unroll
  for (int i = 0; i < kMostBranches; ++i) {
    scale[i] = 0.0f;
    if (i < a.count) {
      float squares = 0.0f;
      for (int c = threadIdx.x; c < a.width; c += blockDim.x) {
        float v = load_as_f32(a.y[i], a.y_dtype, base + c);
        if (a.bias[i]) v += load_as_f32(a.bias[i], a.weight_dtype, c);
        squares = fmaf(v, v, squares);
      }
      scale[i] = 1.0f / sqrtf(block_sum(squares, scratch) / (float)a.width + a.eps);
    }
  }
  const float share = 1.0f / (float)a.count;
  for (int c = threadIdx.x; c < a.width; c += blockDim.x) {
    float acc = 0.0f;
#pragma unroll
    for (int i = 0; i < kMostBranches; ++i)
      if (i < a.count) {
        float v = load_as_f32(a.y[i], a.y_dtype, base + c);
        if (a.bias[i]) v += load_as_f32(a.bias[i], a.weight_dtype, c);
        acc += (v * scale[i]) * load_as_f32(a.weight[i], a.weight_dtype, c);
      }
    store_from_f32(a.out, a.out_dtype, base + c, acc * share);
  }
}

// with a row in registers (as stream_wide_kernel): widths in steps of 4 up to 4096 channels
__global__ __launch_bounds__(1024) void branch_mean_wide_kernel(BranchArgs a) {
  __shared__ float scratch[16];
  const size_t base = (size_t)blockIdx.x * a.width;
  const int col = 4 * threadIdx.x;
  const bool inside = col < a.width;
  f32x4_r v[kMostBranches];
  float squares[kMostBranches];
#pragma unroll
  for (int i = 0; i < kMostBranches; ++i) {
    v[i] = (f32x4_r){0.0f, 0.0f, 0.0f, 0.0f};
    if (i < a.count && inside) {
      v[i] = load4_r(a.y[i], a.y_dtype, base + col);
      if (a.bias[i]) v[i] += load4_r(a.bias[i], a.weight_dtype, col);
    }
    squares[i] = (v[i][0] * v[i][0] + v[i][1] * v[i][1]) + (v[i][2] * v[i][2] + v[i][3] * v[i][3]);
  }
  f32x4_r acc = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
  for (int i = 0; i < kMostBranches; ++i)
    if (i < a.count) {
      const float scale = 1.0f / sqrtf(block_sum(squares[i], scratch) / (float)a.width + a.eps);
      if (inside) acc += (v[i] * scale) * load4_r(a.weight[i], a.weight_dtype, col);
    }
  if (inside) store4_r(a.out, a.out_dtype, base + col, acc * (1.0f / (float)a.count));
}

extern "C" int nnis_branch_mean(const void* const* y, const void* const* weight, const void* const* bias, int count, int y_dtype,
                                int weight_dtype, int tokens, int width, float eps, void* out, int out_dtype, void* stream) {
  NNIS_REQUIRE(count >= 1 && count <= kMostBranches, "branch_mean: 1 to %d branches are taken, got %d", kMostBranches, count);
  NNIS_REQUIRE(nnis_dtype_ok(y_dtype) && nnis_dtype_ok(weight_dtype) && nnis_dtype_ok(out_dtype), "branch_mean: unknown dtype");
  NNIS_REQUIRE(tokens >= 0 && width > 0 && eps > 0.0f, "branch_mean: bad sizes tokens=%d width=%d", tokens, width);
  if (tokens == 0) return 0;
  BranchArgs a;
  for (int i = 0; i < kMostBranches; ++i) {
    a.y[i] = i < count ? y[i] : nullptr;
    a.weight[i] = i < count ? weight[i] : nullptr;
    a.bias[i] = i < count ? bias[i] : nullptr;
    NNIS_REQUIRE(i >= count || (a.y[i] && a.weight[i]), "branch_mean: branch %d has no input or no weight", i);
  }
  a.count = count; a.y_dtype = y_dtype; a.weight_dtype = weight_dtype; a.width = width; a.eps = eps; a.out = out; a.out_dtype = out_dtype;
  bool aligned = (uintptr_t)out % 16 == 0;
  for (int i = 0; i < count; ++i)
    aligned = aligned && (uintptr_t)a.y[i] % 16 == 0 && (uintptr_t)a.weight[i] % 16 == 0 && (uintptr_t)a.bias[i] % 16 == 0;
  if (width % 4 == 0 && aligned && width / 4 <= 1024) {
    hipLaunchKernelGGL(branch_mean_wide_kernel, dim3(tokens), dim3((width / 4 + 63) / 64 * 64), 0, (hipStream_t)stream, a);
    NNIS_LAUNCH_CHECK("branch_mean");
    return 0;
  }
  const int threads = width >= 2048 ? 256 : (width >= 512 ? 128 : 64);
  hipLaunchKernelGGL(branch_mean_kernel, dim3(tokens), dim3(threads), 0, (hipStream_t)stream, a);
  NNIS_LAUNCH_CHECK("branch_mean");
  return 0;
}

// -----------------------------------------------------------------------------
// Gated activation on a fused [tokens, 2 * inner] projection (gate columns first): out = act(gate) * up.
//   act 0: SiLU, gate / (1 + exp(-gate))
//   act 1: the tanh form of GELU, 0.5 g (1 + tanh(sqrt(2 / pi) (g + 0.044715 g^3)))
//   act 2: ReLU, max(g, 0)
// -----------------------------------------------------------------------------
__device__ __forceinline__ float gate_activation(float g, int act) {
  if (act == 0) return g / (1.0f + expf(-g));
  if (act == 2) return fmaxf(g, 0.0f);
  const float inner = 0.7978845608028654f * (g + 0.044715f * g * g * g);
  return 0.5f * g * (1.0f + tanhf(inner));
}

__global__ void gated_act_kernel(const void* __restrict__ gate_up, int in_dtype, void* __restrict__ out, int out_dtype, int inner,
                                 size_t total, int act) {
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (size_t)gridDim.x * blockDim.x) {
    const size_t row = i / inner, col = i % inner;
    const float g = load_as_f32(gate_up, in_dtype, row * 2 * inner + col);
    const float u = load_as_f32(gate_up, in_dtype, row * 2 * inner + inner + col);
    store_from_f32(out, out_dtype, i, gate_activation(g, act) * u);
  }
}

// the same on bfloat16 rows whose width is a multiple of 8: 16-byte accesses, 8 channels a thread
typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8_r;

__global__ void gated_act_bf16_kernel(const bf16_t* __restrict__ gate_up, bf16_t* __restrict__ out, int inner, size_t groups, int act) {
  const int per_row = inner / 8;
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < groups; i += (size_t)gridDim.x * blockDim.x) {
    const size_t row = i / per_row;
    const int col = (int)(i % per_row) * 8;
    const bf16x8_r g = *(const bf16x8_r*)(gate_up + row * 2 * inner + col);
    const bf16x8_r u = *(const bf16x8_r*)(gate_up + row * 2 * inner + inner + col);
    bf16x8_r y;
#pragma unroll
    for (int e = 0; e < 8; ++e) y[e] = (__bf16)(gate_activation((float)g[e], act) * (float)u[e]);
    *(bf16x8_r*)(out + row * inner + col) = y;
  }
}

extern "C" int nnis_gated_act(const void* gate_up, int in_dtype, void* out, int out_dtype, int tokens, int inner, int act,
                              void* stream) {
  NNIS_REQUIRE(nnis_dtype_ok(in_dtype) && nnis_dtype_ok(out_dtype), "gated_act: unknown dtype");
  NNIS_REQUIRE(tokens >= 0 && inner > 0, "gated_act: bad sizes tokens=%d inner=%d", tokens, inner);
  NNIS_REQUIRE(act >= 0 && act <= 2, "gated_act: unknown activation %d", act);
  if (tokens == 0) return 0;
  if (in_dtype == NNIS_BF16 && out_dtype == NNIS_BF16 && inner % 8 == 0 && (uintptr_t)gate_up % 16 == 0 && (uintptr_t)out % 16 == 0) {
    const size_t groups = (size_t)tokens * (inner / 8);
    size_t wide_blocks = (groups + 255) / 256;
    if (wide_blocks > 65536) wide_blocks = 65536;
    hipLaunchKernelGGL(gated_act_bf16_kernel, dim3((unsigned)wide_blocks), dim3(256), 0, (hipStream_t)stream, (const bf16_t*)gate_up,
                       (bf16_t*)out, inner, groups, act);
    NNIS_LAUNCH_CHECK("gated_act_bf16");
    return 0;
  }
  const size_t total = (size_t)tokens * inner;
  size_t blocks = (total + 255) / 256;
  if (blocks > 65536) blocks = 65536;
  hipLaunchKernelGGL(gated_act_kernel, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream, gate_up, in_dtype, out,
                     out_dtype, inner, total, act);
  NNIS_LAUNCH_CHECK("gated_act");
  return 0;
}

// -----------------------------------------------------------------------------
// y[t, c] += bias[c], in place
// -----------------------------------------------------------------------------
__global__ void add_bias_kernel(void* __restrict__ y, int y_dtype, const void* __restrict__ bias, int bias_dtype, int width,
                                size_t total) {
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (size_t)gridDim.x * blockDim.x)
    store_from_f32(y, y_dtype, i, load_as_f32(y, y_dtype, i) + load_as_f32(bias, bias_dtype, i % width));
}

extern "C" int nnis_add_bias(void* y, int y_dtype, const void* bias, int bias_dtype, int tokens, int width, void* stream) {
  NNIS_REQUIRE(nnis_dtype_ok(y_dtype) && nnis_dtype_ok(bias_dtype), "add_bias: unknown dtype");
  NNIS_REQUIRE(tokens >= 0 && width > 0 && y && bias, "add_bias: bad arguments");
  if (tokens == 0) return 0;
  const size_t total = (size_t)tokens * width;
  size_t blocks = (total + 255) / 256;
  if (blocks > 65536) blocks = 65536;
  hipLaunchKernelGGL(add_bias_kernel, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream, y, y_dtype, bias, bias_dtype, width,
                     total);
  NNIS_LAUNCH_CHECK("add_bias");
  return 0;
}

// -----------------------------------------------------------------------------
// The residual stream's step around a norm without statistics, y -> tanh(alpha y) * w + b (alpha a scalar, w and
// b per channel; nothing of a row is summed, so any cut of a row into threads will do).  One kernel does what
// lies between two projections of a layer that norms its sublayers before and after:
//   v = x[src]                                       the stream, 32-bit (0 without one)
//   v += post ? tanh(post_alpha y) post_w + post_b : y     a sublayer's output, normed on its way in (if y)
//   v += rows_add[src]                                a second stream of rows (the embedding, on re-entry)
//   v += vec_add                                      a vector per channel
//   x_out[src] = v                                    (without a row list; x_out may be x itself)
//   h[r] = next ? tanh(next_alpha v) next_w + next_b : v   the input of what comes next (if h)
// src = rows ? rows[r] : r.  All arithmetic in 32-bit; y, the weights and h in the type their codes say.
// -----------------------------------------------------------------------------
struct TanhNormArgs {
  const float* x;
  float* x_out;
  const void* y;
  int y_dtype;
  const void* post_w;
  const void* post_b;
  float post_alpha;
  const float* rows_add;
  const void* vec_add;
  const void* next_w;
  const void* next_b;
  float next_alpha;
  int w_dtype;
  void* h;
  int h_dtype;
  const int* rows;
  int width;
  size_t total;  // output rows x width
};

__global__ void tanh_norm_step_kernel(TanhNormArgs a) {
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < a.total; i += (size_t)gridDim.x * blockDim.x) {
    const size_t r = i / a.width;
    const int c = (int)(i % a.width);
    const size_t src = (a.rows ? (size_t)a.rows[r] : r) * a.width + c;
    float v = a.x ? a.x[src] : 0.0f;
    if (a.y) {
      float y = load_as_f32(a.y, a.y_dtype, src);
      if (a.post_w) y = tanhf(a.post_alpha * y) * load_as_f32(a.post_w, a.w_dtype, c) + load_as_f32(a.post_b, a.w_dtype, c);
      v += y;
    }
    if (a.rows_add) v += a.rows_add[src];
    if (a.vec_add) v += load_as_f32(a.vec_add, a.w_dtype, c);
    if (a.x_out) a.x_out[src] = v;
    if (a.h) {
      const float h = a.next_w ? tanhf(a.next_alpha * v) * load_as_f32(a.next_w, a.w_dtype, c) + load_as_f32(a.next_b, a.w_dtype, c) : v;
      store_from_f32(a.h, a.h_dtype, i, h);
    }
  }
}

// The same, four channels a thread with 16-byte accesses of the 32-bit rows (8-byte ones of bfloat16): for widths in
// steps of 4 and operands on 16-byte boundaries.  Types as template arguments, so that no access hides behind a branch.
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4_r;
typedef __attribute__((ext_vector_type(4))) float f32x4_r;

template <typename T>
__device__ __forceinline__ f32x4_r load4(const void* base, size_t index);
template <>
__device__ __forceinline__ f32x4_r load4<float>(const void* base, size_t index) { return *(const f32x4_r*)((const float*)base + index); }
template <>
__device__ __forceinline__ f32x4_r load4<bf16_t>(const void* base, size_t index) {
  const bf16x4_r v = *(const bf16x4_r*)((const bf16_t*)base + index);
  return (f32x4_r){(float)v[0], (float)v[1], (float)v[2], (float)v[3]};
}
template <typename T>
__device__ __forceinline__ void store4(void* base, size_t index, f32x4_r v);
template <>
__device__ __forceinline__ void store4<float>(void* base, size_t index, f32x4_r v) { *(f32x4_r*)((float*)base + index) = v; }
template <>
__device__ __forceinline__ void store4<bf16_t>(void* base, size_t index, f32x4_r v) {
  *(bf16x4_r*)((bf16_t*)base + index) = (bf16x4_r){(__bf16)v[0], (__bf16)v[1], (__bf16)v[2], (__bf16)v[3]};
}

template <typename YT, typename WT, typename HT>
__global__ __launch_bounds__(256) void tanh_norm_step_wide_kernel(TanhNormArgs a) {
  const int quads = a.width / 4;
  const size_t total = a.total / 4;
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (size_t)gridDim.x * blockDim.x) {
    const size_t r = i / quads;
    const int c = (int)(i % quads) * 4;
    const size_t src = (a.rows ? (size_t)a.rows[r] : r) * a.width + c;
    // every operand asked for before the first is used
    f32x4_r v = {0.0f, 0.0f, 0.0f, 0.0f}, y = v, pw = v, pb = v, extra = v, vec = v, nw = v, nb = v;
    if (a.x) v = *(const f32x4_r*)(a.x + src);
    if (a.y) y = load4<YT>(a.y, src);
    if (a.post_w) {
      pw = load4<WT>(a.post_w, c);
      pb = load4<WT>(a.post_b, c);
    }
    if (a.rows_add) extra = *(const f32x4_r*)(a.rows_add + src);
    if (a.vec_add) vec = load4<WT>(a.vec_add, c);
    if (a.next_w) {
      nw = load4<WT>(a.next_w, c);
      nb = load4<WT>(a.next_b, c);
    }
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      if (a.y) v[e] += a.post_w ? tanhf(a.post_alpha * y[e]) * pw[e] + pb[e] : y[e];
      v[e] += extra[e] + vec[e];
    }
    if (a.x_out) *(f32x4_r*)(a.x_out + src) = v;
    if (a.h) {
      f32x4_r h = v;
      if (a.next_w) {
#pragma unroll
        for (int e = 0; e < 4; ++e) h[e] = tanhf(a.next_alpha * v[e]) * nw[e] + nb[e];
      }
      store4<HT>(a.h, i * 4, h);
    }
  }
}

template <typename YT, typename WT>
static void launch_tanh_wide(const TanhNormArgs& a, unsigned blocks, hipStream_t stream) {
  if (a.h_dtype == NNIS_F32) hipLaunchKernelGGL((tanh_norm_step_wide_kernel<YT, WT, float>), dim3(blocks), dim3(256), 0, stream, a);
  else hipLaunchKernelGGL((tanh_norm_step_wide_kernel<YT, WT, bf16_t>), dim3(blocks), dim3(256), 0, stream, a);
}

extern "C" int nnis_tanh_norm_step(const float* x, float* x_out, const void* y, int y_dtype, const void* post_w, const void* post_b,
                                   float post_alpha, const float* rows_add, const void* vec_add, const void* next_w,
                                   const void* next_b, float next_alpha, int w_dtype, void* h, int h_dtype, const int* rows,
                                   int out_rows, int width, void* stream) {
  NNIS_REQUIRE(nnis_dtype_ok(y_dtype) && nnis_dtype_ok(w_dtype) && nnis_dtype_ok(h_dtype), "tanh_norm_step: unknown dtype");
  NNIS_REQUIRE((x || y) && out_rows >= 0 && width > 0, "tanh_norm_step: bad arguments (rows %d, width %d)", out_rows, width);
  NNIS_REQUIRE((post_w == nullptr) == (post_b == nullptr) && (next_w == nullptr) == (next_b == nullptr),
               "tanh_norm_step: a norm comes with its weight and its bias");
  NNIS_REQUIRE(!(rows && x_out), "tanh_norm_step: a step over a list of rows leaves the stream as it is");
  NNIS_REQUIRE(x_out || h, "tanh_norm_step: nothing to write");
  if (out_rows == 0) return 0;
  TanhNormArgs a;
  a.x = x; a.x_out = x_out; a.y = y; a.y_dtype = y_dtype; a.post_w = post_w; a.post_b = post_b; a.post_alpha = post_alpha;
  a.rows_add = rows_add; a.vec_add = vec_add; a.next_w = next_w; a.next_b = next_b; a.next_alpha = next_alpha; a.w_dtype = w_dtype;
  a.h = h; a.h_dtype = h_dtype; a.rows = rows; a.width = width; a.total = (size_t)out_rows * width;
  bool wide = width % 4 == 0;
  for (const void* p : {(const void*)x, (const void*)x_out, y, post_w, post_b, (const void*)rows_add, vec_add, next_w, next_b, (const void*)h})
    wide = wide && (uintptr_t)p % 16 == 0;
  if (wide) {
    size_t quads = (a.total / 4 + 255) / 256;
    if (quads > 65536) quads = 65536;
    if (y_dtype == NNIS_F32) {
      if (w_dtype == NNIS_F32) launch_tanh_wide<float, float>(a, (unsigned)quads, (hipStream_t)stream);
      else launch_tanh_wide<float, bf16_t>(a, (unsigned)quads, (hipStream_t)stream);
    } else {
      if (w_dtype == NNIS_F32) launch_tanh_wide<bf16_t, float>(a, (unsigned)quads, (hipStream_t)stream);
      else launch_tanh_wide<bf16_t, bf16_t>(a, (unsigned)quads, (hipStream_t)stream);
    }
    NNIS_LAUNCH_CHECK("tanh_norm_step");
    return 0;
  }
  size_t blocks = (a.total + 255) / 256;
  if (blocks > 65536) blocks = 65536;
  hipLaunchKernelGGL(tanh_norm_step_kernel, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream, a);
  NNIS_LAUNCH_CHECK("tanh_norm_step");
  return 0;
}

// -----------------------------------------------------------------------------
// Logits bent by a cap, in place: x -> cap * tanh(x / cap)   (32-bit rows)
// -----------------------------------------------------------------------------
__global__ void tanh_cap_kernel(float* __restrict__ x, float cap, size_t total) {
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (size_t)gridDim.x * blockDim.x)
    x[i] = cap * tanhf(x[i] / cap);
}

extern "C" int nnis_tanh_cap(float* x, float cap, long long total, void* stream) {
  NNIS_REQUIRE(x && cap > 0.0f && total >= 0, "tanh_cap: bad arguments (cap %g)", (double)cap);
  if (total == 0) return 0;
  size_t blocks = ((size_t)total + 255) / 256;
  if (blocks > 65536) blocks = 65536;
  hipLaunchKernelGGL(tanh_cap_kernel, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream, x, cap, (size_t)total);
  NNIS_LAUNCH_CHECK("tanh_cap");
  return 0;
}

// -----------------------------------------------------------------------------
// Branches side by side, plainly: out = sum_i scale_i * y_i, the sum in 32-bit.  Up to kMostBranches inputs of one
// type and shape, each with a factor.
// -----------------------------------------------------------------------------
struct BranchSumArgs {
  const void* y[kMostBranches];
  float scale[kMostBranches];
  int count;
  int y_dtype;
  void* out;
  int out_dtype;
  size_t total;
};

__global__ void branch_sum_kernel(BranchSumArgs a) {
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < a.total; i += (size_t)gridDim.x * blockDim.x) {
    float sum = 0.0f;
#pragma unroll
    for (int b = 0; b < kMostBranches; ++b)
      if (b < a.count) sum = fmaf(a.scale[b], load_as_f32(a.y[b], a.y_dtype, i), sum);
    store_from_f32(a.out, a.out_dtype, i, sum);
  }
}

extern "C" int nnis_branch_sum(const void* const* y, const float* scale, int count, int y_dtype, long long total, void* out, int out_dtype,
                               void* stream) {
  NNIS_REQUIRE(count >= 1 && count <= kMostBranches, "branch_sum: 1 to %d branches are taken, got %d", kMostBranches, count);
  NNIS_REQUIRE(nnis_dtype_ok(y_dtype) && nnis_dtype_ok(out_dtype) && y && scale && out && total >= 0, "branch_sum: bad arguments");
  if (total == 0) return 0;
  BranchSumArgs a;
  for (int i = 0; i < kMostBranches; ++i) {
    a.y[i] = i < count ? y[i] : nullptr;
    a.scale[i] = i < count ? scale[i] : 0.0f;
    NNIS_REQUIRE(i >= count || a.y[i], "branch_sum: branch %d has no input", i);
  }
  a.count = count; a.y_dtype = y_dtype; a.out = out; a.out_dtype = out_dtype; a.total = (size_t)total;
  size_t blocks = ((size_t)total + 255) / 256;
  if (blocks > 65536) blocks = 65536;
  hipLaunchKernelGGL(branch_sum_kernel, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream, a);
  NNIS_LAUNCH_CHECK("branch_sum");
  return 0;
}

// -----------------------------------------------------------------------------
// Logits times a constant, in place (32-bit rows)
// -----------------------------------------------------------------------------
__global__ void scale_rows_kernel(float* __restrict__ x, float factor, size_t total) {
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (size_t)gridDim.x * blockDim.x) x[i] *= factor;
}

extern "C" int nnis_scale_rows(float* x, float factor, long long total, void* stream) {
  NNIS_REQUIRE(x && total >= 0, "scale_rows: bad arguments");
  if (total == 0) return 0;
  size_t blocks = ((size_t)total + 255) / 256;
  if (blocks > 65536) blocks = 65536;
  hipLaunchKernelGGL(scale_rows_kernel, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream, x, factor, (size_t)total);
  NNIS_LAUNCH_CHECK("scale_rows");
  return 0;
}
