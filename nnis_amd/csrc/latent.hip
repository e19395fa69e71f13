// Row-wise kernels of attention over a cached latent: every token keeps one normed vector c (and, where the
// mixer rotates, one rotated key part shared by all heads) instead of keys and values per head.  With the
// heads' key and value maps folded into the query and output projections, the latent is key and value of one
// shared key/value head: keys [c, rotated part], values c.  What is left between the projections is here:
//   latent_prepare   from one fused projection's row [query latent | c | rotated key part | gate logits]:
//                    the query latent divided by its root mean square and weighted; c likewise, written with
//                    the rotated key part into the token's page of keys and, alone, into its page of values;
//                    the gates as sigmoid(logit)
//   latent_rotate_q  the rotated channels of every head's query, in place
//   head_scale       a head's output multiplied by its gate, in place
// A rotation pairs channel 2i with channel 2i + 1: (u, v) -> (u cos a - v sin a, v cos a + u sin a), a =
// position * frequency i, cosines and sines from tables [positions, pairs] made on the host.  Norms, angles,
// rotations and gates are 32-bit; storage types are chosen at run time.
#include "common.h"

thread_local char g_nnis_error[512] = {0};
extern "C" const char* nnis_last_error() { return g_nnis_error; }

namespace {

struct PrepareArgs {
  const void* proj;  // [tokens, q_rank + kv_rank + rot_dim + gates]
  int proj_dtype;
  int q_rank, kv_rank, rot_dim, gates;
  const void* q_weight;  // [q_rank]
  const void* c_weight;  // [kv_rank]
  int w_dtype;
  float eps;
  const float* cos_table;  // [positions, rot_dim / 2]
  const float* sin_table;
  int positions;
  const int* tok_slot;
  const int* tok_pos;
  void* cq;  // [tokens, q_rank]
  int cq_dtype;
  void* k_pages;  // one key/value head: keys of kv_rank + rot_dim channels, values of kv_rank
  void* v_pages;
  int cache_dtype;
  const int* block_table;
  int max_pages;
  float* gate;  // [tokens, gates]
};

__global__ __launch_bounds__(256) void latent_prepare_kernel(PrepareArgs a) {
  __shared__ float scratch[16];
  const int token = blockIdx.x;
  const int row_width = a.q_rank + a.kv_rank + a.rot_dim + a.gates;
  const size_t row = (size_t)token * row_width;
  float ss_q = 0.0f, ss_c = 0.0f;
  for (int i = threadIdx.x; i < a.q_rank; i += blockDim.x) {
    const float v = load_as_f32(a.proj, a.proj_dtype, row + i);
    ss_q = fmaf(v, v, ss_q);
  }
  for (int i = threadIdx.x; i < a.kv_rank; i += blockDim.x) {
    const float v = load_as_f32(a.proj, a.proj_dtype, row + a.q_rank + i);
    ss_c = fmaf(v, v, ss_c);
  }
  const float inv_q = a.q_rank > 0 ? 1.0f / sqrtf(block_sum(ss_q, scratch) / (float)a.q_rank + a.eps) : 0.0f;
  const float inv_c = 1.0f / sqrtf(block_sum(ss_c, scratch) / (float)a.kv_rank + a.eps);
  for (int i = threadIdx.x; i < a.q_rank; i += blockDim.x)
    store_from_f32(a.cq, a.cq_dtype, (size_t)token * a.q_rank + i,
                   load_as_f32(a.proj, a.proj_dtype, row + i) * inv_q * load_as_f32(a.q_weight, a.w_dtype, i));
  for (int i = threadIdx.x; i < a.gates; i += blockDim.x) {
    const float g = load_as_f32(a.proj, a.proj_dtype, row + a.q_rank + a.kv_rank + a.rot_dim + i);
    a.gate[(size_t)token * a.gates + i] = 1.0f / (1.0f + expf(-g));
  }
  const int slot = a.tok_slot[token];
  if (slot < 0 || a.k_pages == nullptr) return;  // a padding row, or a run that keeps no cache of its own
  const int pos = a.tok_pos[token];
  const int page = a.block_table[(size_t)slot * a.max_pages + pos / kPageTokens];
  const int at = pos % kPageTokens;
  const size_t k_base = (size_t)page * nnis_k_page_elems(a.kv_rank + a.rot_dim);
  const size_t v_base = (size_t)page * nnis_v_page_elems(a.kv_rank);
  for (int i = threadIdx.x; i < a.kv_rank; i += blockDim.x) {
    const float c = load_as_f32(a.proj, a.proj_dtype, row + a.q_rank + i) * inv_c * load_as_f32(a.c_weight, a.w_dtype, i);
    store_from_f32(a.k_pages, a.cache_dtype, k_base + nnis_k_offset(at, i), c);
    store_from_f32(a.v_pages, a.cache_dtype, v_base + nnis_v_offset(i, at), c);
  }
  const int pairs = a.rot_dim / 2;
  const int table_row = pos < a.positions ? pos : a.positions - 1;  // (the engine refuses a step beyond the tables before it launches)
  for (int i = threadIdx.x; i < pairs; i += blockDim.x) {
    const float u = load_as_f32(a.proj, a.proj_dtype, row + a.q_rank + a.kv_rank + 2 * i);
    const float v = load_as_f32(a.proj, a.proj_dtype, row + a.q_rank + a.kv_rank + 2 * i + 1);
    const float c = a.cos_table[(size_t)table_row * pairs + i], s = a.sin_table[(size_t)table_row * pairs + i];
    store_from_f32(a.k_pages, a.cache_dtype, k_base + nnis_k_offset(at, a.kv_rank + 2 * i), u * c - v * s);
    store_from_f32(a.k_pages, a.cache_dtype, k_base + nnis_k_offset(at, a.kv_rank + 2 * i + 1), v * c + u * s);
  }
}

__global__ void latent_rotate_q_kernel(void* __restrict__ q, int q_dtype, int heads, int head_width, int first, int pairs,
                                       const float* __restrict__ cos_table, const float* __restrict__ sin_table, int positions,
                                       const int* __restrict__ tok_pos, size_t total) {
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (size_t)gridDim.x * blockDim.x) {
    const int pair = (int)(i % pairs);
    const size_t head_row = i / pairs;  // token * heads + head
    const int token = (int)(head_row / heads);
    int pos = tok_pos[token];
    pos = pos < 0 ? 0 : (pos < positions ? pos : positions - 1);
    const size_t at = head_row * head_width + first + 2 * pair;
    const float u = load_as_f32(q, q_dtype, at), v = load_as_f32(q, q_dtype, at + 1);
    const float c = cos_table[(size_t)pos * pairs + pair], s = sin_table[(size_t)pos * pairs + pair];
    store_from_f32(q, q_dtype, at, u * c - v * s);
    store_from_f32(q, q_dtype, at + 1, v * c + u * s);
  }
}

// logistic: the gates are logits still, and a head is multiplied by 1 / (1 + exp(-gate))
__device__ __forceinline__ float head_gate_of(float g, int logistic) { return logistic ? 1.0f / (1.0f + expf(-g)) : g; }

__global__ void head_scale_kernel(void* __restrict__ o, int o_dtype, const float* __restrict__ gate, int channels, size_t total,
                                  int logistic) {
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (size_t)gridDim.x * blockDim.x)
    store_from_f32(o, o_dtype, i, load_as_f32(o, o_dtype, i) * head_gate_of(gate[i / channels], logistic));
}

// the same on bfloat16 rows whose heads come in steps of 8 channels: 16-byte accesses
typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8_l;
__global__ void head_scale_bf16_kernel(bf16_t* __restrict__ o, const float* __restrict__ gate, int channels, size_t groups, int logistic) {
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < groups; i += (size_t)gridDim.x * blockDim.x) {
    const float g = head_gate_of(gate[(i * 8) / channels], logistic);
    bf16x8_l v = *(const bf16x8_l*)(o + i * 8);
#pragma unroll
    for (int e = 0; e < 8; ++e) v[e] = (__bf16)((float)v[e] * g);
    *(bf16x8_l*)(o + i * 8) = v;
  }
}

// -----------------------------------------------------------------------------
// A map of their own for every head: out[t, h, n] = (sum_k w[h, n, k] x[t, h, k]) * gate[t, h * N + n], x [tokens,
// heads * K], w [heads, N, K], gate (32-bit, optional) [tokens, heads * N].  The heads' value maps of attention over
// a latent where a gate element by element stands between them and the output projection, so that they cannot be
// folded into it.  A block takes R rows of one head, kept in LDS as floats; a wave takes an output at a time for all
// of them (lanes stride over k), so a row of the head's map is read once a block.  Sums are 32-bit.
// -----------------------------------------------------------------------------
template <int R>
__global__ __launch_bounds__(256) void heads_linear_kernel(const void* __restrict__ x, int x_dtype, const void* __restrict__ w, int w_dtype,
                                                           const float* __restrict__ gate, void* __restrict__ out, int out_dtype,
                                                           int tokens, int heads, int n, int k) {
  extern __shared__ __attribute__((aligned(16))) float xs[];  // [R][k]
  const int head = blockIdx.y, row0 = blockIdx.x * R;
  for (int i = threadIdx.x; i < R * k; i += blockDim.x) {
    const int r = i / k;
    xs[i] = row0 + r < tokens ? load_as_f32(x, x_dtype, ((size_t)(row0 + r) * heads + head) * k + i % k) : 0.0f;
  }
  __syncthreads();
  const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave, waves = blockDim.x / kWave;
  for (int o = wave; o < n; o += waves) {
    const size_t w_row = ((size_t)head * n + o) * k;
    float acc[R];
#pragma unroll
    for (int r = 0; r < R; ++r) acc[r] = 0.0f;
#pragma unroll 4
    for (int c = lane; c < k; c += kWave) {
      const float wv = load_as_f32(w, w_dtype, w_row + c);
#pragma unroll
      for (int r = 0; r < R; ++r) acc[r] = fmaf(xs[r * k + c], wv, acc[r]);
    }
#pragma unroll
    for (int r = 0; r < R; ++r) {
      const float total = wave_sum(acc[r]);
      if (lane == 0 && row0 + r < tokens) {
        const size_t at = ((size_t)(row0 + r) * heads + head) * n + o;
        store_from_f32(out, out_dtype, at, gate ? total * gate[at] : total);
      }
    }
  }
}

// The same on the matrix cores for bfloat16 rows and maps with K a multiple of 8, up to kHeadsLinearMostK: a block takes 16
// rows of one head; each of its 4 waves keeps the rows' K in operand registers and takes every fourth strip of 16
// outputs, whose weights come straight from memory (a head's map is small and read by every block of the head: it
// stays in the caches).  v_mfma_f32_16x16x32_bf16 with the map's rows as the first operand: lane l holds outputs
// 4 * (l / 16) .. + 3 of row l % 16, four consecutive outputs of one row, gated and stored together.
typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8_m;
typedef __attribute__((ext_vector_type(4))) float f32x4_m;
constexpr int kHeadsLinearMostK = 512;

template <int CHUNKS>
__global__ __launch_bounds__(256) void heads_linear_mfma_kernel(const bf16_t* __restrict__ x, const bf16_t* __restrict__ w,
                                                                const float* __restrict__ gate, bf16_t* __restrict__ out, int tokens,
                                                                int heads, int n, int k) {
  const int head = blockIdx.y, row0 = blockIdx.x * 16;
  const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
  const int r = lane % 16, group = lane / 16;
  const int token = min(row0 + r, tokens - 1);
  bf16x8_m rows[CHUNKS];
#pragma unroll
  for (int c = 0; c < CHUNKS; ++c) {
    const int at = c * 32 + group * 8;
    bf16x8_m v;
#pragma unroll
    for (int i = 0; i < 8; ++i) v[i] = (__bf16)0.0f;
    if (at < k) v = *(const bf16x8_m*)(x + ((size_t)token * heads + head) * k + at);
    rows[c] = v;
  }
  for (int strip = wave; strip * 16 < n; strip += 4) {
    const int o = min(strip * 16 + r, n - 1);
    const bf16_t* map = w + ((size_t)head * n + o) * k;
    f32x4_m acc = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
    for (int c = 0; c < CHUNKS; ++c) {
      const int at = c * 32 + group * 8;
      bf16x8_m v;
#pragma unroll
      for (int i = 0; i < 8; ++i) v[i] = (__bf16)0.0f;
      if (at < k) v = *(const bf16x8_m*)(map + at);
      acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(v, rows[c], acc, 0, 0, 0);
    }
    if (row0 + r >= tokens) continue;
    const int first = strip * 16 + group * 4;  // this lane's four outputs of row r
    const size_t at = ((size_t)(row0 + r) * heads + head) * n + first;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      if (first + e < n) out[at + e] = (__bf16)(gate ? acc[e] * gate[at + e] : acc[e]);
    }
  }
}

unsigned blocks_for(size_t total) {
  size_t blocks = (total + 255) / 256;
  return (unsigned)(blocks > 65536 ? 65536 : blocks);
}

}  // namespace

extern "C" int nnis_latent_prepare(const void* proj, int proj_dtype, int tokens, int q_rank, int kv_rank, int rot_dim, int gates,
                                   const void* q_weight, const void* c_weight, int w_dtype, float eps, const float* cos_table,
                                   const float* sin_table, int positions, const int* tok_slot, const int* tok_pos, void* cq,
                                   int cq_dtype, void* k_pages, void* v_pages, int cache_dtype, const int* block_table,
                                   int max_pages, float* gate, void* stream) {
  NNIS_REQUIRE(nnis_dtype_ok(proj_dtype) && nnis_dtype_ok(w_dtype) && nnis_dtype_ok(cq_dtype) && nnis_dtype_ok(cache_dtype),
               "latent_prepare: unknown dtype");
  NNIS_REQUIRE(tokens >= 0 && q_rank >= 0 && kv_rank > 0 && rot_dim >= 0 && rot_dim % 2 == 0 && gates >= 0,
               "latent_prepare: bad sizes (q_rank %d, kv_rank %d, rot_dim %d, gates %d)", q_rank, kv_rank, rot_dim, gates);
  NNIS_REQUIRE(proj && c_weight && tok_slot && tok_pos && eps > 0.0f, "latent_prepare: missing operands");
  NNIS_REQUIRE(q_rank == 0 || (q_weight && cq), "latent_prepare: a query latent needs its weight and its output");
  NNIS_REQUIRE(rot_dim == 0 || (cos_table && sin_table && positions > 0), "latent_prepare: a rotation needs its tables");
  NNIS_REQUIRE(gates == 0 || gate, "latent_prepare: gates need their output");
  NNIS_REQUIRE((k_pages == nullptr) == (v_pages == nullptr) && (k_pages == nullptr || (block_table && max_pages > 0)),
               "latent_prepare: pages come with values and a block table");
  if (tokens == 0) return 0;
  PrepareArgs a;
  a.proj = proj; a.proj_dtype = proj_dtype; a.q_rank = q_rank; a.kv_rank = kv_rank; a.rot_dim = rot_dim; a.gates = gates;
  a.q_weight = q_weight; a.c_weight = c_weight; a.w_dtype = w_dtype; a.eps = eps; a.cos_table = cos_table; a.sin_table = sin_table;
  a.positions = positions; a.tok_slot = tok_slot; a.tok_pos = tok_pos; a.cq = cq; a.cq_dtype = cq_dtype; a.k_pages = k_pages;
  a.v_pages = v_pages; a.cache_dtype = cache_dtype; a.block_table = block_table; a.max_pages = max_pages; a.gate = gate;
  const int widest = q_rank > kv_rank ? q_rank : kv_rank;
  const int threads = widest >= 256 ? 256 : (widest >= 128 ? 128 : 64);
  hipLaunchKernelGGL(latent_prepare_kernel, dim3(tokens), dim3(threads), 0, (hipStream_t)stream, a);
  NNIS_LAUNCH_CHECK("latent_prepare");
  return 0;
}

extern "C" int nnis_latent_rotate_q(void* q, int q_dtype, int tokens, int heads, int head_width, int first, int rot_dim,
                                    const float* cos_table, const float* sin_table, int positions, const int* tok_pos,
                                    void* stream) {
  NNIS_REQUIRE(nnis_dtype_ok(q_dtype), "latent_rotate_q: unknown dtype");
  NNIS_REQUIRE(q && cos_table && sin_table && tok_pos && positions > 0, "latent_rotate_q: missing operands");
  NNIS_REQUIRE(tokens >= 0 && heads > 0 && rot_dim > 0 && rot_dim % 2 == 0 && first >= 0 && first + rot_dim <= head_width,
               "latent_rotate_q: %d rotated channels from %d on do not fit heads of %d", rot_dim, first, head_width);
  if (tokens == 0) return 0;
  const size_t total = (size_t)tokens * heads * (rot_dim / 2);
  hipLaunchKernelGGL(latent_rotate_q_kernel, dim3(blocks_for(total)), dim3(256), 0, (hipStream_t)stream, q, q_dtype, heads,
                     head_width, first, rot_dim / 2, cos_table, sin_table, positions, tok_pos, total);
  NNIS_LAUNCH_CHECK("latent_rotate_q");
  return 0;
}

extern "C" int nnis_head_scale_of(void* o, int o_dtype, const float* gate, int tokens, int heads, int channels, int logistic, void* stream);

extern "C" int nnis_head_scale(void* o, int o_dtype, const float* gate, int tokens, int heads, int channels, void* stream) {
  return nnis_head_scale_of(o, o_dtype, gate, tokens, heads, channels, 0, stream);
}

// logistic: gate holds logits, and head h of token t is multiplied by sigmoid(gate[t, h])
extern "C" int nnis_head_scale_of(void* o, int o_dtype, const float* gate, int tokens, int heads, int channels, int logistic, void* stream) {
  NNIS_REQUIRE(nnis_dtype_ok(o_dtype), "head_scale: unknown dtype");
  NNIS_REQUIRE(o && gate && tokens >= 0 && heads > 0 && channels > 0, "head_scale: bad arguments");
  if (tokens == 0) return 0;
  const size_t total = (size_t)tokens * heads * channels;
  if (o_dtype == NNIS_BF16 && channels % 8 == 0 && (uintptr_t)o % 16 == 0) {
    hipLaunchKernelGGL(head_scale_bf16_kernel, dim3(blocks_for(total / 8)), dim3(256), 0, (hipStream_t)stream, (bf16_t*)o, gate, channels,
                       total / 8, logistic);
    NNIS_LAUNCH_CHECK("head_scale");
    return 0;
  }
  hipLaunchKernelGGL(head_scale_kernel, dim3(blocks_for(total)), dim3(256), 0, (hipStream_t)stream, o, o_dtype, gate, channels, total, logistic);
  NNIS_LAUNCH_CHECK("head_scale");
  return 0;
}

extern "C" int nnis_heads_linear(const void* x, int x_dtype, const void* w, int w_dtype, const float* gate, void* out, int out_dtype,
                                 int tokens, int heads, int n, int k, void* stream) {
  NNIS_REQUIRE(nnis_dtype_ok(x_dtype) && nnis_dtype_ok(w_dtype) && nnis_dtype_ok(out_dtype), "heads_linear: unknown dtype");
  NNIS_REQUIRE(x && w && out && tokens >= 0 && heads > 0 && heads <= 65535 && n > 0 && k > 0, "heads_linear: bad arguments");
  NNIS_REQUIRE((size_t)k * sizeof(float) <= 48 * 1024, "heads_linear: rows of up to 12288 channels a head, got %d", k);
  if (tokens == 0) return 0;
  hipStream_t s = (hipStream_t)stream;
  if (x_dtype == NNIS_BF16 && w_dtype == NNIS_BF16 && out_dtype == NNIS_BF16 && k % 8 == 0 && k <= kHeadsLinearMostK &&
      (uintptr_t)x % 16 == 0 && (uintptr_t)w % 16 == 0) {
    const dim3 tiles((tokens + 15) / 16, heads);
    const int chunks = (k + 31) / 32;
#define NNIS_HEADS_LINEAR(C_)   hipLaunchKernelGGL((heads_linear_mfma_kernel<C_>), tiles, dim3(256), 0, s, (const bf16_t*)x, (const bf16_t*)w, gate, (bf16_t*)out, tokens, heads, n, k)
    if (chunks <= 2) NNIS_HEADS_LINEAR(2);
    else if (chunks <= 4) NNIS_HEADS_LINEAR(4);
    else if (chunks <= 6) NNIS_HEADS_LINEAR(6);
    else if (chunks <= 8) NNIS_HEADS_LINEAR(8);
    else if (chunks <= 12) NNIS_HEADS_LINEAR(12);
    else NNIS_HEADS_LINEAR(16);
#undef NNIS_HEADS_LINEAR
    NNIS_LAUNCH_CHECK("heads_linear");
    return 0;
  }
  // several rows a block where they fit 48 KB of LDS and the step has rows enough
  const int rows = tokens >= 64 && (size_t)8 * k * 4 <= 49152 ? 8 : (tokens >= 4 && (size_t)4 * k * 4 <= 49152 ? 4 : 1);
  const dim3 grid((tokens + rows - 1) / rows, heads);
  const size_t lds = (size_t)rows * k * sizeof(float);
  if (rows == 8) hipLaunchKernelGGL((heads_linear_kernel<8>), grid, dim3(256), lds, s, x, x_dtype, w, w_dtype, gate, out, out_dtype, tokens, heads, n, k);
  else if (rows == 4) hipLaunchKernelGGL((heads_linear_kernel<4>), grid, dim3(256), lds, s, x, x_dtype, w, w_dtype, gate, out, out_dtype, tokens, heads, n, k);
  else hipLaunchKernelGGL((heads_linear_kernel<1>), grid, dim3(256), lds, s, x, x_dtype, w, w_dtype, gate, out, out_dtype, tokens, heads, n, k);
  NNIS_LAUNCH_CHECK("heads_linear");
  return 0;
}
