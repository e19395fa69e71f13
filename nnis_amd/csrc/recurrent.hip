// Mixers that carry a state of fixed size from token to token: a short causal convolution per channel, the
// selective scan (a diagonal recurrence per channel with input-dependent steps), gated linear attention (a
// matrix state per head with a decay per key channel; with one fixed decay a head and turned queries and keys it
// is retention), the per-head norm and gate behind it, the minGRU, and the gated delta rule (a matrix state per
// head whose every token first takes back what the state already holds under its key).
//
// A step's rows are packed: sequence b of the step owns rows seq_start[b] .. seq_start[b + 1] - 1, which
// continue the sequence in slot seq_slot[b] (negative: padding, nothing is read or written for it).  State
// lives per slot in 32-bit and is zero when a sequence starts; a kernel reads it at a run's first row and
// leaves it behind the run's last, so a prompt in one step, in portions, or token by token give the same.
// Decays, step sizes, exponentials and the recurrences themselves are 32-bit whatever the storage type.
#include "common.h"

thread_local char g_nnis_error[512] = {0};
extern "C" const char* nnis_last_error() { return g_nnis_error; }

namespace {

constexpr float kLog2e = 1.4426950408889634f;
// 2^x by the hardware's instruction (about one unit in the last place): the decays of a recurrence are powers of
// two of a product that is made once, exp(dt A) = 2^(dt (A log2 e))
__device__ __forceinline__ float exp2_fast(float x) { return __builtin_amdgcn_exp2f(x); }
__device__ __forceinline__ float sigmoid_f(float z) { return __builtin_amdgcn_rcpf(1.0f + exp2_fast(-z * kLog2e)); }
// log(1 + e^z) by the hardware's 2^x and log2: e^z itself where it is small (the sum 1 + e^z would round it away;
// three terms of the logarithm's series keep a relative error of e^3z / 4 < 2e-6 below e^z = 0.02), z where it is large
__device__ __forceinline__ float softplus_f(float z) {
  const float t = exp2_fast(z * kLog2e);
  const float small = t * (1.0f - t * (0.5f - t * (1.0f / 3.0f)));
  const float mid = __builtin_amdgcn_logf(1.0f + t) * 0.6931471805599453f;
  return z > 20.0f ? z : (t < 0.02f ? small : mid);
}
// log(sigmoid(z)) = min(z, 0) - log(1 + exp(-|z|))
__device__ __forceinline__ float log_sigmoid_f(float z) { return fminf(z, 0.0f) - log1pf(expf(-fabsf(z))); }

// -----------------------------------------------------------------------------
// Causal convolution per channel with SiLU: y[t, c] = silu(b[c] + sum_j w[c, j] x[t - (taps - 1) + j, c]),
// the last tap on the token itself, zeros before the sequence's start.  Inputs older than the step's first
// row come from `state` [slots, taps - 1, channels] (the sequence's last taps - 1 inputs, oldest first).
// -----------------------------------------------------------------------------
constexpr int kMostTaps = 16;

struct ConvArgs {
  const void* x;  // [tokens, x_stride]: the first `channels` columns
  int x_dtype;
  int x_stride;
  const void* weight;  // [channels, taps]
  const void* bias;    // [channels] or null
  int weight_dtype;
  float* state;
  const int* tok_slot;
  const int* tok_pos;
  const int* seq_slot;
  const int* seq_start;
  int tokens, batch, channels, taps;
  void* y;  // [tokens, channels]
  int y_dtype;
};

// the input `back` tokens before row `token` of the sequence in `slot` at position `pos` (back <= pos): a row of
// this step while the rows belong to the sequence, then the state's rows, newest last
__device__ __forceinline__ float conv_input(const ConvArgs& a, int token, int slot, int back, int c, bool& in_step, int& behind) {
  if (in_step && token - back >= 0 && a.tok_slot[token - back] == slot)
    return load_as_f32(a.x, a.x_dtype, (size_t)(token - back) * a.x_stride + c);
  in_step = false;
  ++behind;
  return a.state[((size_t)slot * (a.taps - 1) + (a.taps - 1 - behind)) * a.channels + c];
}

// A thread takes one channel over a strip of consecutive rows: its taps stay in registers and so do the last inputs
// while the rows go on in one sequence (one load a row); at a strip's or a sequence's first row they are looked up.
constexpr int kConvStrip = 16;

__global__ __launch_bounds__(256) void conv_silu_kernel(ConvArgs a) {
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  if (c >= a.channels) return;
  const int begin = blockIdx.y * kConvStrip, end = min(a.tokens, begin + kConvStrip);
  float w[kMostTaps], held[kMostTaps];  // held[j]: the input taps - 1 - j tokens back
#pragma unroll
  for (int j = 0; j < kMostTaps; ++j) {
    w[j] = j < a.taps ? load_as_f32(a.weight, a.weight_dtype, (size_t)c * a.taps + j) : 0.0f;
    held[j] = 0.0f;
  }
  const float bias = a.bias ? load_as_f32(a.bias, a.weight_dtype, c) : 0.0f;
  float fresh[kConvStrip];  // the strip's own inputs, all asked for at once
#pragma unroll
  for (int i = 0; i < kConvStrip; ++i) fresh[i] = begin + i < end ? load_as_f32(a.x, a.x_dtype, (size_t)(begin + i) * a.x_stride + c) : 0.0f;
  int before = -2;  // the slot of the row before, if its inputs are held
#pragma unroll
  for (int i = 0; i < kConvStrip; ++i) {
    const int token = begin + i;
    if (token >= end) break;
    const int slot = a.tok_slot[token];
    if (slot < 0) {
      store_from_f32(a.y, a.y_dtype, (size_t)token * a.channels + c, 0.0f);
      before = -2;
      continue;
    }
    if (slot == before) {
#pragma unroll
      for (int j = 0; j + 1 < kMostTaps; ++j)
        if (j + 1 < a.taps) held[j] = held[j + 1];
#pragma unroll
      for (int j = 0; j < kMostTaps; ++j)
        if (j == a.taps - 1) held[j] = fresh[i];
    } else {
      const int pos = a.tok_pos[token];
      bool in_step = true;
      int behind = 0;
#pragma unroll
      for (int back = 0; back < kMostTaps; ++back) {
        if (back < a.taps) {
          const float v = back <= pos ? conv_input(a, token, slot, back, c, in_step, behind) : 0.0f;  // zeros before the start
#pragma unroll
          for (int j = 0; j < kMostTaps; ++j)
            if (j == a.taps - 1 - back) held[j] = v;
        }
      }
      before = slot;
    }
    float acc = bias;
#pragma unroll
    for (int j = 0; j < kMostTaps; ++j) acc = fmaf(w[j], held[j], acc);  // (beyond the taps: zeros)
    store_from_f32(a.y, a.y_dtype, (size_t)token * a.channels + c, acc * sigmoid_f(acc));
  }
}

// A step of single tokens: output and state in one kernel, a thread a (sequence, channel).  The state's rows
// before a sequence's start are zeros (a slot starts so, and they are only ever moved down).
__global__ __launch_bounds__(256) void conv_single_kernel(ConvArgs a) {
  const int b = blockIdx.y;
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  if (c >= a.channels) return;
  const int token = a.seq_start[b];
  const int slot = a.seq_slot[b];
  if (slot < 0) {
    store_from_f32(a.y, a.y_dtype, (size_t)token * a.channels + c, 0.0f);
    return;
  }
  const int keep = a.taps - 1;
  float* state = a.state + (size_t)slot * keep * a.channels + c;
  const float now = load_as_f32(a.x, a.x_dtype, (size_t)token * a.x_stride + c);
  float acc = a.bias ? load_as_f32(a.bias, a.weight_dtype, c) : 0.0f;
  float older[kMostTaps];
#pragma unroll
  for (int j = 0; j < kMostTaps; ++j) {
    older[j] = j < keep ? state[(size_t)j * a.channels] : 0.0f;
    if (j < keep) acc = fmaf(load_as_f32(a.weight, a.weight_dtype, (size_t)c * a.taps + j), older[j], acc);
  }
  acc = fmaf(load_as_f32(a.weight, a.weight_dtype, (size_t)c * a.taps + keep), now, acc);
  store_from_f32(a.y, a.y_dtype, (size_t)token * a.channels + c, acc * sigmoid_f(acc));
#pragma unroll
  for (int j = 0; j < kMostTaps; ++j)
    if (j < keep) state[(size_t)j * a.channels] = j + 1 < keep ? older[j + 1] : now;
}

// after the outputs are taken: the state becomes the last taps - 1 inputs of each sequence (one thread a
// channel keeps the old ones it still needs in registers)
__global__ void conv_state_kernel(ConvArgs a) {
  const int b = blockIdx.y;
  const int slot = a.seq_slot[b];
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  if (slot < 0 || c >= a.channels) return;
  const int first = a.seq_start[b], count = a.seq_start[b + 1] - first;
  if (count <= 0) return;
  const int keep = a.taps - 1;
  float* state = a.state + (size_t)slot * keep * a.channels + c;
  float fresh[kMostTaps];
#pragma unroll
  for (int j = 0; j < kMostTaps; ++j) {
    if (j < keep) {
      const int back = keep - 1 - j;  // new row j holds the input `back` tokens before the run's last
      fresh[j] = back < count ? load_as_f32(a.x, a.x_dtype, (size_t)(first + count - 1 - back) * a.x_stride + c)
                              : state[(size_t)(j + count) * a.channels];
    }
  }
#pragma unroll
  for (int j = 0; j < kMostTaps; ++j)
    if (j < keep) state[(size_t)j * a.channels] = fresh[j];
}

// -----------------------------------------------------------------------------
// Selective scan.  Per channel c and state n, over a sequence's tokens:
//   dt = softplus(dt_pre[t, c] + dt_bias[c])
//   S[c, n] <- exp(dt * A[c, n]) S[c, n] + dt * x[t, c] * B[t, n]
//   y[t, c] = (sum_n S[c, n] C[t, n] + D[c] x[t, c]) * silu(z[t, c])
// A thread keeps 16 states of one channel (8 where there are no more); the lanes of a channel (a power of two, up to 8)
// sit side by side and add their parts of y by lane exchanges.  bc [tokens, 2 * states]: B then C.  A = -exp(A_log) comes
// ready-made.  state [slots, channels, states].
// -----------------------------------------------------------------------------
struct ScanArgs {
  const void* x;  // [tokens, channels]
  int x_dtype;
  const float* dt_pre;  // [tokens, channels]
  const float* bc;      // [tokens, 2 * states]
  const void* z;        // [tokens, z_stride]: the first `channels` columns from the pointer on
  int z_dtype, z_stride;
  const float* A;        // [channels, states]
  const float* D;        // [channels]
  const float* dt_bias;  // [channels]
  float* state;
  const int* seq_slot;
  const int* seq_start;
  int channels, states;
  void* y;  // [tokens, channels]
  int y_dtype;
  // a long run is cut into pieces of `piece` tokens that run side by side (see below)
  int piece, pieces;
  float* carried;   // [batch, pieces, channels, states]
  float* stepped;   // [batch, pieces, channels]: a piece's sum of step sizes
};

// A run of many tokens is a chain as long as the run.  The recurrence is linear in the state, so the run is cut
// into pieces that are taken side by side, in three passes: (1) every piece but the last runs from a zero state and
// leaves what it ends with, E_k, and the sum of its step sizes (the product of its decays is exp(A * that sum));
// (2) one thread a (channel, state) walks the pieces, I_0 = the sequence's state, I_(k+1) = exp(A sum_k) I_k + E_k,
// and leaves I_k in E_k's place; (3) every piece runs again, from I_k, and writes the outputs; the last one leaves
// the sequence's state.  PASS 0 is the plain run of a whole sequence by one block (single tokens, short runs).
// a lane's PER of a token's `n` values from `row`: 16-byte loads where the row allows them
template <int PER>
__device__ __forceinline__ void load_lane(float (&into)[PER], const float* row, int part, int n, bool wide) {
  if (wide && part * PER + PER <= n) {  // (a lane that reaches beyond the states takes them one by one, zeros beyond)
#pragma unroll
    for (int q = 0; q < PER / 4; ++q) {
      const float4 v = *(const float4*)(row + part * PER + 4 * q);
      into[4 * q] = v.x; into[4 * q + 1] = v.y; into[4 * q + 2] = v.z; into[4 * q + 3] = v.w;
    }
  } else {
#pragma unroll
    for (int j = 0; j < PER; ++j) into[j] = part * PER + j < n ? row[part * PER + j] : 0.0f;
  }
}

// PER: states a lane keeps (8, or 16: one lane a channel up to 16 states, half the lanes and none of the exchanges)
template <int LANES, int PASS, int PER>
__global__ __launch_bounds__(256) void selective_scan_kernel(ScanArgs a) {
  const int b = blockIdx.z, piece = blockIdx.y;
  const int slot = a.seq_slot[b];
  if (slot < 0) return;
  const int begin = a.seq_start[b], end = a.seq_start[b + 1];
  if (end <= begin) return;
  int first = begin, last = end, pieces_here = 1;
  if (PASS != 0) {
    pieces_here = (end - begin + a.piece - 1) / a.piece;
    if (piece >= pieces_here || (PASS == 1 && piece == pieces_here - 1)) return;
    first = begin + piece * a.piece;
    last = min(end, first + a.piece);
  }
  const int part = threadIdx.x % LANES;
  const int c = blockIdx.x * (256 / LANES) + threadIdx.x / LANES;
  const bool live = c < a.channels;
  const int cc = live ? c : 0;
  const int N = a.states;
  float S[PER], A[PER];
  float* state = a.state + ((size_t)slot * a.channels + cc) * N;
  float* carried = PASS == 0 ? nullptr : a.carried + (((size_t)b * a.pieces + piece) * a.channels + cc) * N;
#pragma unroll
  for (int j = 0; j < PER; ++j) {
    const int n = part * PER + j;
    const bool here = live && n < N;
    S[j] = !here || PASS == 1 ? 0.0f : (PASS == 0 ? state[n] : carried[n]);
    A[j] = here ? a.A[(size_t)cc * N + n] * kLog2e : 0.0f;  // (in powers of two)
  }
  const float D = a.D[cc], dt_bias = a.dt_bias[cc];
  float steps = 0.0f;
  // the token after this one is asked for before this one is worked on
  float x_next = load_as_f32(a.x, a.x_dtype, (size_t)first * a.channels + cc);
  float dt_next = a.dt_pre[(size_t)first * a.channels + cc];
  float z_next = PASS == 1 ? 0.0f : load_as_f32(a.z, a.z_dtype, (size_t)first * a.z_stride + cc);
  float B_next[PER], C_next[PER];
  const bool wide = N % 4 == 0 && ((uintptr_t)a.bc % 16 == 0);  // a lane's 8 values lie within the row, on 16-byte boundaries
  load_lane<PER>(B_next, a.bc + (size_t)first * 2 * N, part, N, wide);
#pragma unroll
  for (int j = 0; j < PER; ++j) C_next[j] = 0.0f;
  if (PASS != 1) load_lane<PER>(C_next, a.bc + (size_t)first * 2 * N + N, part, N, wide);
  for (int t = first; t < last; ++t) {
    const float x = x_next, z = z_next;
    // (the step size is the same in all lanes of a channel: one of them takes the logarithm)
    float dt = part == 0 ? softplus_f(dt_next + dt_bias) : 0.0f;
    if (LANES > 1) dt = __shfl(dt, (threadIdx.x % kWave) & ~(LANES - 1), kWave);
    float B[PER], C[PER];
#pragma unroll
    for (int j = 0; j < PER; ++j) {
      B[j] = B_next[j];
      C[j] = C_next[j];
    }
    const int ahead = t + 1 < last ? t + 1 : t;
    x_next = load_as_f32(a.x, a.x_dtype, (size_t)ahead * a.channels + cc);
    dt_next = a.dt_pre[(size_t)ahead * a.channels + cc];
    if (PASS != 1) z_next = load_as_f32(a.z, a.z_dtype, (size_t)ahead * a.z_stride + cc);
    load_lane<PER>(B_next, a.bc + (size_t)ahead * 2 * N, part, N, wide);
    if (PASS != 1) load_lane<PER>(C_next, a.bc + (size_t)ahead * 2 * N + N, part, N, wide);
    const float dx = dt * x;
    steps += dt;
    float acc = 0.0f;
#pragma unroll
    for (int j = 0; j < PER; ++j) {
      S[j] = fmaf(exp2_fast(dt * A[j]), S[j], dx * B[j]);  // (lanes beyond the states: A, B and S are zero)
      acc = fmaf(S[j], C[j], acc);
    }
    if (PASS != 1) {
#pragma unroll
      for (int offset = LANES / 2; offset > 0; offset >>= 1) acc += __shfl_xor(acc, offset, kWave);
      if (part == 0 && live) store_from_f32(a.y, a.y_dtype, (size_t)t * a.channels + c, (acc + D * x) * (z * sigmoid_f(z)));
    }
  }
  if (!live) return;
  if (PASS == 1) {
    if (part == 0) a.stepped[((size_t)b * a.pieces + piece) * a.channels + c] = steps;
  } else if (PASS == 3 && piece != pieces_here - 1) {
    return;
  }
  float* into = PASS == 1 ? carried : state;
#pragma unroll
  for (int j = 0; j < PER; ++j) {
    const int n = part * PER + j;
    if (n < N) into[n] = S[j];
  }
}

// pass (2): a thread a (sequence, channel, state)
__global__ void selective_scan_carry_kernel(ScanArgs a) {
  const int b = blockIdx.y;
  const int slot = a.seq_slot[b];
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (slot < 0 || i >= a.channels * a.states) return;
  const int count = a.seq_start[b + 1] - a.seq_start[b];
  if (count <= 0) return;
  const int pieces_here = (count + a.piece - 1) / a.piece;
  const int c = i / a.states;
  const float A = a.A[i];
  float I = a.state[(size_t)slot * a.channels * a.states + i];
  const size_t per = (size_t)a.channels * a.states;
  for (int k0 = 0; k0 < pieces_here; k0 += 8) {  // eight pieces' ends and steps asked for at once
    float E[8], steps[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const bool more = k0 + j + 1 < pieces_here;
      E[j] = more ? a.carried[((size_t)b * a.pieces + k0 + j) * per + i] : 0.0f;
      steps[j] = more ? a.stepped[((size_t)b * a.pieces + k0 + j) * a.channels + c] : 0.0f;
    }
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      if (k0 + j < pieces_here) {
        a.carried[((size_t)b * a.pieces + k0 + j) * per + i] = I;
        I = fmaf(expf(A * steps[j]), I, E[j]);
      }
    }
  }
}

// -----------------------------------------------------------------------------
// Gated linear attention.  Per head, over a sequence's tokens, with a state S [key channels, value channels]:
//   alpha = sigmoid(zd)^(1 / tau)            per key channel
//   S <- diag(alpha) S + k v^T
//   o = S^T (q * scale)
// A block takes one head of one sequence and a slab of value columns; a thread keeps 16 key rows of one
// column (of two where the head has columns enough), the threads of a column (a power of two, up to 16) sit 64 / GROUPS lanes apart in one wave and add
// their parts of o by lane exchanges.  Tokens come through LDS a chunk at a time (queries, keys, decays of
// the head and the slab's values), loaded by the whole block.  o is left raw, in 32-bit.
// -----------------------------------------------------------------------------
struct GlaArgs {
  const void* q;  // row t, head h: q + t * q_stride + h * key_dim  (k alike; v, with value_dim)
  const void* k;
  const void* v;
  int qkv_dtype;
  int q_stride, k_stride, v_stride;
  const float* zd;  // [tokens, heads * key_dim]: the logarithms of the decays (nnis_gla_decays)
  float scale;
  float* state;  // [slots, heads, key_dim, value_dim]
  const int* seq_slot;
  const int* seq_start;
  int heads, key_dim, value_dim;
  int chunk;   // tokens staged at a time
  float* out;  // [tokens, heads * value_dim]
  // a long run is cut into pieces of `piece` tokens that run side by side, as the selective scan's
  int piece, pieces;
  float* carried;  // [batch, pieces, heads, key_dim, value_dim]
  float* decayed;  // [batch, pieces, heads, key_dim]: a piece's sum of the decays' logarithms
  // Without `zd`: one fixed decay a head (retention), head_decay [2, heads]: the decays, then their logarithms.
  const float* head_decay;
  // With rot_dim > 0: the first rot_dim channels of every head of q and k are turned by the token's position while
  // they are staged, channel i with channel i + rot_dim / 2: (u, v) -> (u cos - v sin, v cos + u sin), tables
  // [rot_positions, rot_dim / 2], tok_pos one position a row of the step.
  const float* rot_cos;
  const float* rot_sin;
  const int* tok_pos;
  int rot_dim, rot_positions;
};

// channel `ch` of head `head` of row t, turned by the row's position where the head's first channels are
__device__ __forceinline__ float gla_turned(const GlaArgs& a, const void* base, int stride, int t, int head, int ch) {
  const size_t row = (size_t)t * stride + (size_t)head * a.key_dim;
  const float x = load_as_f32(base, a.qkv_dtype, row + ch);
  if (ch >= a.rot_dim) return x;
  const int half = a.rot_dim / 2;
  const bool low = ch < half;
  const int pair = low ? ch : ch - half;
  int pos = a.tok_pos[t];
  pos = pos < 0 ? 0 : (pos < a.rot_positions ? pos : a.rot_positions - 1);
  const float c = a.rot_cos[(size_t)pos * half + pair], s = a.rot_sin[(size_t)pos * half + pair];
  const float other = load_as_f32(base, a.qkv_dtype, row + (low ? ch + half : ch - half));
  return low ? x * c - other * s : x * c + other * s;
}

// PASS as in selective_scan_kernel: 0 a whole run; 1 a piece from a zero state, leaving its end and the sum of its
// decays' logarithms; 3 a piece from the state that the carry kernel left for it, writing the outputs.
// CPT: value columns a thread keeps (what it reads of queries, keys and decays serves them all)
template <int GROUPS, int PASS, int CPT>
__global__ __launch_bounds__(256) void gla_scan_kernel(GlaArgs a) {
  extern __shared__ __attribute__((aligned(16))) float lds[];
  constexpr int kSpan = 4 * (kWave / GROUPS);  // columns that the block's threads take side by side (4 waves)
  constexpr int kCols = CPT * kSpan;           // value columns of a block
  const int b = blockIdx.z / a.pieces, piece = blockIdx.z % a.pieces, head = blockIdx.y;
  const int slot = a.seq_slot[b];
  if (slot < 0) return;
  const int begin = a.seq_start[b], end = a.seq_start[b + 1];
  if (end <= begin) return;
  int first = begin, last = end, pieces_here = 1;
  if (PASS != 0) {
    pieces_here = (end - begin + a.piece - 1) / a.piece;
    if (piece >= pieces_here || (PASS == 1 && piece == pieces_here - 1)) return;
    first = begin + piece * a.piece;
    last = min(end, first + a.piece);
  }
  const int d = a.key_dim, e = a.value_dim;
  const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
  const int group = lane / (kWave / GROUPS);
  const int col_in_span = wave * (kWave / GROUPS) + lane % (kWave / GROUPS);
  float* qs = lds;                    // [chunk][d]
  float* ks = qs + a.chunk * d;       // [chunk][d]
  float* as = ks + a.chunk * d;       // [chunk][d]
  float* vs = as + a.chunk * d;       // [chunk][kCols]
  float S[CPT][16];
  int col[CPT];
  bool live[CPT];
  float* state[CPT];
  float* carried[CPT];
#pragma unroll
  for (int c = 0; c < CPT; ++c) {
    col[c] = blockIdx.x * kCols + c * kSpan + col_in_span;
    live[c] = col[c] < e;
    state[c] = a.state + (((size_t)slot * a.heads + head) * d) * e + (live[c] ? col[c] : 0);
    carried[c] = PASS == 0 ? nullptr : a.carried + ((((size_t)b * a.pieces + piece) * a.heads + head) * d) * e + (live[c] ? col[c] : 0);
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int row = group * 16 + r;
      const bool here = live[c] && row < d;
      S[c][r] = !here || PASS == 1 ? 0.0f : (PASS == 0 ? state[c][(size_t)row * e] : carried[c][(size_t)row * e]);
    }
  }
  float log_sum = 0.0f;  // PASS 1, threads below key_dim of the first slab: the sum of a key channel's log decays
  for (int t0 = first; t0 < last; t0 += a.chunk) {
    const int count = min(a.chunk, last - t0);
    __syncthreads();  // the chunk before has been read
    for (int i = threadIdx.x; i < count * d; i += blockDim.x) {
      const int t = t0 + i / d, ch = i % d;
      if (PASS != 1) qs[i] = gla_turned(a, a.q, a.q_stride, t, head, ch) * a.scale;
      ks[i] = gla_turned(a, a.k, a.k_stride, t, head, ch);
      as[i] = a.zd ? exp2_fast(a.zd[((size_t)t * a.heads + head) * d + ch] * kLog2e) : a.head_decay[head];
    }
    for (int i = threadIdx.x; i < count * kCols; i += blockDim.x) {
      const int t = t0 + i / kCols, cl = blockIdx.x * kCols + i % kCols;
      vs[i] = cl < e ? load_as_f32(a.v, a.qkv_dtype, (size_t)t * a.v_stride + head * e + cl) : 0.0f;
    }
    if (PASS == 1 && blockIdx.x == 0 && (int)threadIdx.x < d) {
      if (a.zd) {
        for (int j = 0; j < count; ++j) log_sum += a.zd[((size_t)(t0 + j) * a.heads + head) * d + threadIdx.x];
      } else {
        log_sum += (float)count * a.head_decay[a.heads + head];
      }
    }
    __syncthreads();
    for (int j = 0; j < count; ++j) {
      float v[CPT], acc[CPT];
#pragma unroll
      for (int c = 0; c < CPT; ++c) {
        v[c] = vs[j * kCols + c * kSpan + col_in_span];
        acc[c] = 0.0f;
      }
      const float* qj = qs + j * d + group * 16;
      const float* kj = ks + j * d + group * 16;
      const float* aj = as + j * d + group * 16;
      if (group * 16 + 16 <= d && d % 4 == 0) {  // whole rows of this group: 16 bytes a read
#pragma unroll
        for (int r4 = 0; r4 < 4; ++r4) {
          const float4 a4 = *(const float4*)(aj + 4 * r4), k4 = *(const float4*)(kj + 4 * r4);
          const float av[4] = {a4.x, a4.y, a4.z, a4.w}, kv[4] = {k4.x, k4.y, k4.z, k4.w};
#pragma unroll
          for (int c = 0; c < CPT; ++c)
#pragma unroll
            for (int i = 0; i < 4; ++i) S[c][4 * r4 + i] = fmaf(av[i], S[c][4 * r4 + i], kv[i] * v[c]);
          if (PASS != 1) {
            const float4 q4 = *(const float4*)(qj + 4 * r4);
            const float qv[4] = {q4.x, q4.y, q4.z, q4.w};
#pragma unroll
            for (int c = 0; c < CPT; ++c)
#pragma unroll
              for (int i = 0; i < 4; ++i) acc[c] = fmaf(S[c][4 * r4 + i], qv[i], acc[c]);
          }
        }
      } else {
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          if (group * 16 + r < d) {
#pragma unroll
            for (int c = 0; c < CPT; ++c) {
              S[c][r] = fmaf(aj[r], S[c][r], kj[r] * v[c]);
              if (PASS != 1) acc[c] = fmaf(S[c][r], qj[r], acc[c]);
            }
          }
        }
      }
      if (PASS != 1) {
#pragma unroll
        for (int c = 0; c < CPT; ++c) {
#pragma unroll
          for (int offset = kWave / 2; offset >= kWave / GROUPS; offset >>= 1) acc[c] += __shfl_xor(acc[c], offset, kWave);
          if (group == 0 && live[c]) a.out[((size_t)(t0 + j) * a.heads + head) * e + col[c]] = acc[c];
        }
      }
    }
  }
  if (PASS == 1 && blockIdx.x == 0 && (int)threadIdx.x < d)
    a.decayed[(((size_t)b * a.pieces + piece) * a.heads + head) * d + threadIdx.x] = log_sum;
  if (PASS == 3 && piece != pieces_here - 1) return;
#pragma unroll
  for (int c = 0; c < CPT; ++c) {
    if (!live[c]) continue;
    float* into = PASS == 1 ? carried[c] : state[c];
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int row = group * 16 + r;
      if (row < d) into[(size_t)row * e] = S[c][r];
    }
  }
}

// between the passes: a thread an element of a sequence's state walks the pieces, I_(k+1) = P_k I_k + E_k with P_k the
// product of piece k's decays of the element's key channel, and leaves I_k in E_k's place
__global__ void gla_carry_kernel(GlaArgs a) {
  const int b = blockIdx.y;
  const int slot = a.seq_slot[b];
  const size_t per = (size_t)a.heads * a.key_dim * a.value_dim;
  const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (slot < 0 || i >= per) return;
  const int count = a.seq_start[b + 1] - a.seq_start[b];
  if (count <= 0) return;
  const int pieces_here = (count + a.piece - 1) / a.piece;
  const size_t row = i / a.value_dim;  // (head, key channel)
  float I = a.state[(size_t)slot * per + i];
  for (int k0 = 0; k0 < pieces_here; k0 += 8) {  // eight pieces' ends and decays asked for at once
    float E[8], logs[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const bool more = k0 + j + 1 < pieces_here;
      E[j] = more ? a.carried[((size_t)b * a.pieces + k0 + j) * per + i] : 0.0f;
      logs[j] = more ? a.decayed[((size_t)b * a.pieces + k0 + j) * a.heads * a.key_dim + row] : 0.0f;
    }
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      if (k0 + j < pieces_here) {
        a.carried[((size_t)b * a.pieces + k0 + j) * per + i] = I;
        I = fmaf(expf(logs[j]), I, E[j]);
      }
    }
  }
}

// -----------------------------------------------------------------------------
// Behind the scan: each head's o normed by its root mean square over its channels, times a weight shared by
// the heads, times silu(gate):  y[t, h, :] = o / sqrt(mean(o^2) + eps) * w * silu(g[t, h, :]).  A wave a (token, head).
// -----------------------------------------------------------------------------
__global__ __launch_bounds__(256) void head_norm_gate_kernel(const float* __restrict__ o, const void* __restrict__ gate, int gate_dtype,
                                                             int gate_stride, const void* __restrict__ weight, int weight_dtype,
                                                             void* __restrict__ y, int y_dtype, int items, int heads, int dim, float eps) {
  const int item = blockIdx.x * 4 + threadIdx.x / kWave;
  const int lane = threadIdx.x % kWave;
  if (item >= items) return;
  const int token = item / heads, head = item % heads;
  const float* row = o + (size_t)item * dim;
  float squares = 0.0f;
  for (int c = lane; c < dim; c += kWave) squares = fmaf(row[c], row[c], squares);
  const float scale = 1.0f / sqrtf(wave_sum(squares) / (float)dim + eps);
  for (int c = lane; c < dim; c += kWave) {
    const float g = load_as_f32(gate, gate_dtype, (size_t)token * gate_stride + head * dim + c);
    const float v = (row[c] * scale) * (weight ? load_as_f32(weight, weight_dtype, c) : 1.0f);
    store_from_f32(y, y_dtype, (size_t)item * dim + c, v * (g * sigmoid_f(g)));
  }
}

}  // namespace

extern "C" int nnis_conv_silu(const void* x, int x_dtype, int x_stride, const void* weight, const void* bias, int weight_dtype,
                              float* state, const int* tok_slot, const int* tok_pos, const int* seq_slot, const int* seq_start,
                              int tokens, int batch, int channels, int taps, void* y, int y_dtype, int single, void* stream) {
  NNIS_REQUIRE(nnis_dtype_ok(x_dtype) && nnis_dtype_ok(weight_dtype) && nnis_dtype_ok(y_dtype), "conv: unknown dtype");
  NNIS_REQUIRE(taps >= 1 && taps <= kMostTaps, "conv: 1 to %d taps are taken, got %d", kMostTaps, taps);
  NNIS_REQUIRE(channels > 0 && x_stride >= channels && tokens >= 0 && batch >= 0, "conv: bad sizes");
  NNIS_REQUIRE(x && weight && tok_slot && tok_pos && seq_slot && seq_start && y && (state || taps == 1), "conv: a pointer is missing");
  if (tokens == 0 || batch == 0) return 0;
  ConvArgs a;
  a.x = x; a.x_dtype = x_dtype; a.x_stride = x_stride; a.weight = weight; a.bias = bias; a.weight_dtype = weight_dtype; a.state = state;
  a.tok_slot = tok_slot; a.tok_pos = tok_pos; a.seq_slot = seq_slot; a.seq_start = seq_start; a.tokens = tokens; a.batch = batch;
  a.channels = channels; a.taps = taps; a.y = y; a.y_dtype = y_dtype;
  NNIS_REQUIRE(batch <= 65535 && (tokens + kConvStrip - 1) / kConvStrip <= 65535, "conv: too many rows or sequences for the grid");
  const int width = channels >= 256 ? 256 : 64;
  if (single) {  // every sequence brings one token: row b is sequence b's
    NNIS_REQUIRE(tokens == batch, "conv: a step of single tokens has as many rows as sequences (%d and %d)", tokens, batch);
    hipLaunchKernelGGL(conv_single_kernel, dim3((channels + width - 1) / width, batch), dim3(width), 0, (hipStream_t)stream, a);
    NNIS_LAUNCH_CHECK("conv_single");
    return 0;
  }
  hipLaunchKernelGGL(conv_silu_kernel, dim3((channels + width - 1) / width, (tokens + kConvStrip - 1) / kConvStrip), dim3(width), 0,
                     (hipStream_t)stream, a);
  NNIS_LAUNCH_CHECK("conv_silu");
  if (taps > 1) {
    const int threads = channels >= 256 ? 256 : 64;
    hipLaunchKernelGGL(conv_state_kernel, dim3((channels + threads - 1) / threads, batch), dim3(threads), 0, (hipStream_t)stream, a);
    NNIS_LAUNCH_CHECK("conv_state");
  }
  return 0;
}

// piece, pieces: 0, or a run is cut into up to `pieces` pieces of `piece` tokens (then `carried`, float32 of batch * pieces *
// channels * states, and `stepped`, of batch * pieces * channels, are scratch of the call)
extern "C" int nnis_selective_scan(const void* x, int x_dtype, const float* dt_pre, const float* bc, const void* z, int z_dtype,
                                   int z_stride, const float* A, const float* D, const float* dt_bias, float* state,
                                   const int* seq_slot, const int* seq_start, int batch, int channels, int states, void* y,
                                   int y_dtype, int piece, int pieces, float* carried, float* stepped, void* stream) {
  NNIS_REQUIRE(nnis_dtype_ok(x_dtype) && nnis_dtype_ok(z_dtype) && nnis_dtype_ok(y_dtype), "selective_scan: unknown dtype");
  NNIS_REQUIRE(channels > 0 && states > 0 && states <= 128 && z_stride >= channels && batch >= 0,
               "selective_scan: bad sizes (channels %d, states %d: up to 128 are taken)", channels, states);
  NNIS_REQUIRE(x && dt_pre && bc && z && A && D && dt_bias && state && seq_slot && seq_start && y, "selective_scan: a pointer is missing");
  NNIS_REQUIRE(pieces <= 1 || (piece > 0 && carried && stepped && pieces <= 65535), "selective_scan: pieces need their length and scratch");
  NNIS_REQUIRE(batch <= 65535, "selective_scan: %d sequences exceed the grid limit", batch);
  if (batch == 0) return 0;
  ScanArgs a;
  a.x = x; a.x_dtype = x_dtype; a.dt_pre = dt_pre; a.bc = bc; a.z = z; a.z_dtype = z_dtype; a.z_stride = z_stride; a.A = A; a.D = D;
  a.dt_bias = dt_bias; a.state = state; a.seq_slot = seq_slot; a.seq_start = seq_start; a.channels = channels; a.states = states;
  a.y = y; a.y_dtype = y_dtype; a.piece = piece; a.pieces = pieces; a.carried = carried; a.stepped = stepped;
  const int need = (states + 15) / 16;  // lanes of 16 states (of 8 for up to 8 states)
  hipStream_t s = (hipStream_t)stream;
#define NNIS_SCAN(LANES_, PASS_, PIECES_, PER_)                                                                            \
  hipLaunchKernelGGL((selective_scan_kernel<LANES_, PASS_, PER_>), dim3((channels + 256 / LANES_ - 1) / (256 / LANES_), PIECES_, batch), \
                     dim3(256), 0, s, a)
#define NNIS_SCAN_PASS(PASS_, PIECES_)                     \
  do {                                                     \
    if (states <= 8) NNIS_SCAN(1, PASS_, PIECES_, 8);      \
    else if (need <= 1) NNIS_SCAN(1, PASS_, PIECES_, 16);  \
    else if (need <= 2) NNIS_SCAN(2, PASS_, PIECES_, 16);  \
    else if (need <= 4) NNIS_SCAN(4, PASS_, PIECES_, 16);  \
    else NNIS_SCAN(8, PASS_, PIECES_, 16);                 \
  } while (0)
  if (pieces <= 1) {
    NNIS_SCAN_PASS(0, 1);
  } else {
    NNIS_SCAN_PASS(1, pieces);
    hipLaunchKernelGGL(selective_scan_carry_kernel, dim3((channels * states + 255) / 256, batch), dim3(256), 0, s, a);
    NNIS_SCAN_PASS(3, pieces);
  }
#undef NNIS_SCAN_PASS
#undef NNIS_SCAN
  NNIS_LAUNCH_CHECK("selective_scan");
  return 0;
}

// piece, pieces: as nnis_selective_scan's (`carried`: batch * pieces * heads * key_dim * value_dim floats, `decayed`:
// batch * pieces * heads * key_dim)
// Without `zd`: `head_decay` [2, heads], one fixed decay a head and its logarithm.  rot_dim > 0: q's and k's first
// rot_dim channels of a head are turned by tok_pos[row] while staged (tables [rot_positions, rot_dim / 2]).
extern "C" int nnis_gla_scan_turned(const void* q, const void* k, const void* v, int qkv_dtype, int q_stride, int k_stride, int v_stride,
                                    const float* zd, const float* head_decay, const float* rot_cos, const float* rot_sin,
                                    int rot_dim, int rot_positions, const int* tok_pos, float scale, float* state,
                                    const int* seq_slot, const int* seq_start, int batch, int heads, int key_dim, int value_dim,
                                    float* out, int piece, int pieces, float* carried, float* decayed, void* stream);

extern "C" int nnis_gla_scan(const void* q, const void* k, const void* v, int qkv_dtype, int q_stride, int k_stride, int v_stride,
                             const float* zd, float scale, float* state, const int* seq_slot, const int* seq_start,
                             int batch, int heads, int key_dim, int value_dim, float* out, int piece, int pieces, float* carried,
                             float* decayed, void* stream) {
  NNIS_REQUIRE(zd, "gla_scan: the decays' logarithms are missing");
  return nnis_gla_scan_turned(q, k, v, qkv_dtype, q_stride, k_stride, v_stride, zd, nullptr, nullptr, nullptr, 0, 0, nullptr, scale,
                              state, seq_slot, seq_start, batch, heads, key_dim, value_dim, out, piece, pieces, carried, decayed, stream);
}

extern "C" int nnis_gla_scan_turned(const void* q, const void* k, const void* v, int qkv_dtype, int q_stride, int k_stride, int v_stride,
                                    const float* zd, const float* head_decay, const float* rot_cos, const float* rot_sin,
                                    int rot_dim, int rot_positions, const int* tok_pos, float scale, float* state,
                                    const int* seq_slot, const int* seq_start, int batch, int heads, int key_dim, int value_dim,
                                    float* out, int piece, int pieces, float* carried, float* decayed, void* stream) {
  NNIS_REQUIRE(nnis_dtype_ok(qkv_dtype), "gla_scan: unknown dtype %d", qkv_dtype);
  NNIS_REQUIRE((zd != nullptr) != (head_decay != nullptr), "gla_scan: decays a token and channel, or one a head");
  NNIS_REQUIRE(rot_dim >= 0 && rot_dim % 2 == 0 && rot_dim <= key_dim, "gla_scan: %d turned channels in heads of %d", rot_dim, key_dim);
  NNIS_REQUIRE(rot_dim == 0 || (rot_cos && rot_sin && tok_pos && rot_positions > 0), "gla_scan: a rotation needs tables and positions");
  NNIS_REQUIRE(heads > 0 && key_dim > 0 && key_dim <= 256 && value_dim > 0 && batch >= 0,
               "gla_scan: bad sizes (heads %d, key channels %d: up to 256 are taken, value channels %d)", heads, key_dim, value_dim);
  NNIS_REQUIRE(q && k && v && state && seq_slot && seq_start && out, "gla_scan: a pointer is missing");
  NNIS_REQUIRE(pieces <= 1 || (piece > 0 && carried && decayed), "gla_scan: pieces need their length and scratch");
  if (pieces < 1) pieces = 1;
  NNIS_REQUIRE((long long)batch * pieces <= 65535 && heads <= 65535, "gla_scan: %d sequences x %d pieces exceed the grid limit", batch, pieces);
  if (batch == 0) return 0;
  GlaArgs a;
  a.q = q; a.k = k; a.v = v; a.qkv_dtype = qkv_dtype; a.q_stride = q_stride; a.k_stride = k_stride; a.v_stride = v_stride; a.zd = zd;
  a.scale = scale; a.state = state; a.seq_slot = seq_slot; a.seq_start = seq_start; a.heads = heads;
  a.key_dim = key_dim; a.value_dim = value_dim; a.out = out; a.piece = piece; a.pieces = pieces; a.carried = carried; a.decayed = decayed;
  a.head_decay = head_decay; a.rot_cos = rot_cos; a.rot_sin = rot_sin; a.tok_pos = tok_pos; a.rot_dim = rot_dim; a.rot_positions = rot_positions;
  const int need = (key_dim + 15) / 16;
  const int groups = need <= 1 ? 1 : (need <= 2 ? 2 : (need <= 4 ? 4 : (need <= 8 ? 8 : 16)));
  const int span = 4 * (kWave / groups);
  hipStream_t s = (hipStream_t)stream;
  // Columns a thread keeps: two where the head has columns enough; four in the pass that writes no outputs (measured at 8
  // heads of 128 x 256 and 2,048 tokens, 1 / 2 / 4 columns: the first pass 107 / 76 / 62 us, the second 145 / 105 / 131).
  auto launch = [&](int pass) {
    const int most = pass == 1 ? 4 : 2;
    const int per_thread = (most >= 4 && value_dim >= 4 * span) ? 4 : (value_dim >= 2 * span ? 2 : 1);
    const int cols = per_thread * span;
    int chunk = (int)((40 * 1024) / ((3 * (size_t)key_dim + cols) * sizeof(float)));
    chunk = chunk > 32 ? 32 : (chunk < 1 ? 1 : chunk);
    a.chunk = chunk;
    const size_t lds = (size_t)chunk * (3 * key_dim + cols) * sizeof(float);
    const dim3 grid((value_dim + cols - 1) / cols, heads, batch * pieces);
#define NNIS_GLA_CASE(GROUPS_, PASS_)                                                                                  \
  if (per_thread == 4) hipLaunchKernelGGL((gla_scan_kernel<GROUPS_, PASS_, PASS_ == 1 ? 4 : 2>), grid, dim3(256), lds, s, a); \
  else if (per_thread == 2) hipLaunchKernelGGL((gla_scan_kernel<GROUPS_, PASS_, 2>), grid, dim3(256), lds, s, a);      \
  else hipLaunchKernelGGL((gla_scan_kernel<GROUPS_, PASS_, 1>), grid, dim3(256), lds, s, a)
#define NNIS_GLA_GROUPS(PASS_)                     \
  switch (groups) {                                \
    case 1: NNIS_GLA_CASE(1, PASS_); break;        \
    case 2: NNIS_GLA_CASE(2, PASS_); break;        \
    case 4: NNIS_GLA_CASE(4, PASS_); break;        \
    case 8: NNIS_GLA_CASE(8, PASS_); break;        \
    default: NNIS_GLA_CASE(16, PASS_); break;      \
  }
    if (pass == 0) { NNIS_GLA_GROUPS(0) } else if (pass == 1) { NNIS_GLA_GROUPS(1) } else { NNIS_GLA_GROUPS(3) }
#undef NNIS_GLA_GROUPS
#undef NNIS_GLA_CASE
  };
  if (pieces <= 1) {
    launch(0);
  } else {
    launch(1);
    const size_t per = (size_t)heads * key_dim * value_dim;
    hipLaunchKernelGGL(gla_carry_kernel, dim3((unsigned)((per + 255) / 256), batch), dim3(256), 0, s, a);
    launch(3);
  }
  NNIS_LAUNCH_CHECK("gla_scan");
  return 0;
}

// z[t, i] <- log(sigmoid(z[t, i] + bias[i])) / tau, in place: the logarithm of the decay sigmoid(.)^(1 / tau)
__global__ void gla_decays_kernel(float* __restrict__ z, const float* __restrict__ bias, int width, size_t total, float inv_tau) {
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (size_t)gridDim.x * blockDim.x)
    z[i] = log_sigmoid_f(z[i] + bias[i % width]) * inv_tau;
}

extern "C" int nnis_gla_decays(float* z, const float* bias, int tokens, int width, float tau, void* stream) {
  NNIS_REQUIRE(z && bias && tokens >= 0 && width > 0, "gla_decays: bad arguments");
  NNIS_REQUIRE(tau > 0.0f, "gla_decays: tau must be positive, got %g", (double)tau);
  if (tokens == 0) return 0;
  const size_t total = (size_t)tokens * width;
  size_t blocks = (total + 255) / 256;
  if (blocks > 65536) blocks = 65536;
  hipLaunchKernelGGL(gla_decays_kernel, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream, z, bias, width, total, 1.0f / tau);
  NNIS_LAUNCH_CHECK("gla_decays");
  return 0;
}

extern "C" int nnis_head_norm_gate(const float* o, const void* gate, int gate_dtype, int gate_stride, const void* weight,
                                   int weight_dtype, void* y, int y_dtype, int tokens, int heads, int dim, float eps, void* stream) {
  NNIS_REQUIRE(nnis_dtype_ok(gate_dtype) && (!weight || nnis_dtype_ok(weight_dtype)) && nnis_dtype_ok(y_dtype), "head_norm_gate: unknown dtype");
  NNIS_REQUIRE(tokens >= 0 && heads > 0 && dim > 0 && gate_stride >= heads * dim && eps > 0.0f, "head_norm_gate: bad sizes");
  NNIS_REQUIRE(o && gate && y, "head_norm_gate: a pointer is missing");
  const int items = tokens * heads;
  if (items == 0) return 0;
  hipLaunchKernelGGL(head_norm_gate_kernel, dim3((items + 3) / 4), dim3(256), 0, (hipStream_t)stream, o, gate, gate_dtype, gate_stride,
                     weight, weight_dtype, y, y_dtype, items, heads, dim, eps);
  NNIS_LAUNCH_CHECK("head_norm_gate");
  return 0;
}

// -----------------------------------------------------------------------------
// minGRU: a gated recurrence whose gates read the current token only.  Per channel
//     z = sigmoid(zp + bz),  u = up + bu,  c = u + 1/2 where u >= 0 and sigmoid(u) below,
//     S <- (1 - z) S + z c,  out = S * silu(g)
// over each sequence's rows, from and into state [slots, width] (32-bit).  `rows` is the fused projection's output
// [tokens, stride]: zp in columns 0 .. width - 1, up in the next `width`, g in the next.  A thread a channel.  The
// recurrence is linear in S, so a long run is cut into pieces (PASS 1: every piece but a sequence's last from a zero
// state, leaving the product of its 1 - z and its end state; PASS 2: every piece again from the state that the
// pieces before it hand on, which it adds up itself, writing the outputs, the last piece the sequence's state).
// -----------------------------------------------------------------------------
namespace {

struct MinGruArgs {
  const void* rows;
  int dtype, stride;
  const void* z_bias;
  const void* x_bias;
  int bias_dtype;
  float* state;
  const int* seq_slot;
  const int* seq_start;
  int batch, width;
  void* out;
  int out_dtype;
  int piece, pieces;  // tokens of a piece, most pieces of a sequence; pieces == 1: not cut
  float* decay;       // [batch, pieces, width]: a piece's product of 1 - z
  float* ends;        // [batch, pieces, width]: a piece's end state from zero
};

template <int PASS>
__global__ __launch_bounds__(256) void min_gru_kernel(MinGruArgs a) {
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  const int b = blockIdx.y / a.pieces;
  const int piece = blockIdx.y % a.pieces;
  const int slot = a.seq_slot[b];
  if (slot < 0 || c >= a.width) return;
  const int start = a.seq_start[b], stop = a.seq_start[b + 1];
  int first = start, last = stop;
  if (a.pieces > 1) {
    first = start + piece * a.piece;
    last = min(stop, first + a.piece);
    if (first >= stop) return;
    if (PASS == 1 && last == stop && piece > 0) return;  // a last piece's end state is the second pass's business (the first piece still keeps the state's copy)
  }
  const float bz = a.z_bias ? load_as_f32(a.z_bias, a.bias_dtype, c) : 0.0f;
  const float bu = a.x_bias ? load_as_f32(a.x_bias, a.bias_dtype, c) : 0.0f;
  float s = 0.0f, keep = 1.0f;
  const size_t mine = ((size_t)b * a.pieces + piece) * a.width + c;
  if (a.pieces == 1) {
    s = a.state[(size_t)slot * a.width + c];
  } else if (PASS == 1) {
    // the first piece runs from the sequence's state and keeps a copy of it where its product would go: the second
    // pass reads no state (its last piece writes it while others may not have started)
    if (piece == 0) a.decay[mine] = s = a.state[(size_t)slot * a.width + c];
  } else if (piece == 0) {
    s = a.decay[mine];
  } else {
    // what the pieces before this one hand on: the first piece's end, then I <- decay_k I + ends_k piece by piece
    s = a.ends[(size_t)b * a.pieces * a.width + c];
#pragma unroll 8
    for (int k = 1; k < piece; ++k) {  // (the loads do not wait for the sums: eight pieces' are asked for at a time)
      const size_t at = ((size_t)b * a.pieces + k) * a.width + c;
      s = fmaf(a.decay[at], s, a.ends[at]);
    }
  }
#pragma unroll 4
  for (int t = first; t < last; ++t) {
    const size_t at = (size_t)t * a.stride + c;
    const float z = sigmoid_f(load_as_f32(a.rows, a.dtype, at) + bz);
    const float u = load_as_f32(a.rows, a.dtype, at + a.width) + bu;
    const float cand = u >= 0.0f ? u + 0.5f : sigmoid_f(u);
    s = fmaf(z, cand - s, s);  // (1 - z) s + z cand
    if (PASS == 1) {
      keep *= 1.0f - z;
    } else {
      const float g = load_as_f32(a.rows, a.dtype, at + 2 * (size_t)a.width);
      store_from_f32(a.out, a.out_dtype, (size_t)t * a.width + c, s * g * sigmoid_f(g));
    }
  }
  if (PASS == 1) {
    if (piece > 0) a.decay[mine] = keep;
    a.ends[mine] = s;
  } else if (last == stop) {
    a.state[(size_t)slot * a.width + c] = s;
  }
}

}  // namespace

extern "C" int nnis_min_gru(const void* rows, int dtype, int stride, const void* z_bias, const void* x_bias, int bias_dtype, float* state,
                            const int* seq_slot, const int* seq_start, int batch, int width, void* out, int out_dtype, int piece,
                            int pieces, float* decay, float* ends, void* stream) {
  NNIS_REQUIRE(rows && state && seq_slot && seq_start && out, "min_gru: missing operand");
  NNIS_REQUIRE(nnis_dtype_ok(dtype) && nnis_dtype_ok(out_dtype) && ((z_bias == nullptr && x_bias == nullptr) || nnis_dtype_ok(bias_dtype)),
               "min_gru: unknown dtype");
  NNIS_REQUIRE(width > 0 && stride >= 3 * width, "min_gru: rows of %d columns do not hold three times %d channels", stride, width);
  NNIS_REQUIRE(pieces >= 1 && (pieces == 1 || (piece > 0 && decay && ends)), "min_gru: pieces without scratch");
  if (batch <= 0) return 0;
  MinGruArgs a;
  a.rows = rows; a.dtype = dtype; a.stride = stride; a.z_bias = z_bias; a.x_bias = x_bias; a.bias_dtype = bias_dtype;
  a.state = state; a.seq_slot = seq_slot; a.seq_start = seq_start; a.batch = batch; a.width = width; a.out = out;
  a.out_dtype = out_dtype; a.piece = piece; a.pieces = pieces; a.decay = decay; a.ends = ends;
  const int threads = width >= 256 ? 256 : 64;
  const dim3 grid((width + threads - 1) / threads, batch * pieces);
  if (pieces > 1) {
    hipLaunchKernelGGL(min_gru_kernel<1>, grid, dim3(threads), 0, (hipStream_t)stream, a);
    NNIS_LAUNCH_CHECK("min_gru (first pass)");
  }
  hipLaunchKernelGGL(min_gru_kernel<2>, grid, dim3(threads), 0, (hipStream_t)stream, a);
  NNIS_LAUNCH_CHECK("min_gru");
  return 0;
}

// -----------------------------------------------------------------------------
// Gated delta rule.  Per head, over a sequence's tokens, with a state S [key channels, value channels]:
//   S <- g S;   u = beta (v - S^T k);   S <- S + k u^T;   o = S^T q
// with q and k unit vectors over a head's channels (x / sqrt(sum x^2 + unit_eps); q also times q_scale), beta =
// sigmoid(b), g = exp(-rate_h * softplus(a + dt_bias_h)).  Query/key head of value head h: h / (heads / groups).
//
// Two kernels.  delta_prepare_kernel, a wave a (token, query/key head): the unit vectors in 32-bit, their product q . k,
// and, a thread a (token, value head), g and beta.  gated_delta_kernel, the recurrence: the columns of S do not meet, so
// a block takes one head of one sequence and a slab of value columns; a thread keeps 8 key rows of one column, and the
// threads of a column are neighbouring lanes, so that their parts of a sum meet by lane moves inside a row of 16
// lanes.  Written on the state before the token, a token needs ONE round of sums, of two numbers side by side:
//   a = S^T k,  b = S^T q  (before the token);   u = beta (v - g a);   o = g b + (q . k) u;   S <- g S + k u^T
// Tokens come through LDS a chunk at a time, copied by the whole block.  Everything but the rows' storage type is
// 32-bit; o is left raw, in 32-bit.
// -----------------------------------------------------------------------------
namespace {

struct DeltaArgs {
  const void* rows;  // row t: [q (groups * key_dim) | k (groups * key_dim) | v (heads * value_dim)]
  int dtype, stride;
  const float* ba;  // [tokens, 2 * heads]: b of every head, then a
  const float* rate;     // [heads]: exp(A_log)
  const float* dt_bias;  // [heads]
  float q_scale, unit_eps;
  float* unit;   // [tokens, groups, 2, key_dim]: q then k, unit vectors
  float* gates;  // [tokens, heads, 2]: g, beta;  behind them [tokens, groups]: q . k
  float* state;  // [slots, heads, value_dim, key_dim]: column by column
  const int* seq_slot;
  const int* seq_start;
  int tokens, heads, groups, key_dim, value_dim;
  int chunk;
  float* out;  // [tokens, heads * value_dim]
};

__global__ __launch_bounds__(256) void delta_prepare_kernel(DeltaArgs a) {
  const int d = a.key_dim;
  const int item = blockIdx.x * 4 + threadIdx.x / kWave;  // (token, query/key head)
  const int lane = threadIdx.x % kWave;
  const int items = a.tokens * a.groups;
  if (item < items) {
    const int t = item / a.groups, qk_head = item % a.groups;
    const size_t q_at = (size_t)t * a.stride + (size_t)qk_head * d;
    const size_t k_at = q_at + (size_t)a.groups * d;
    float sq = 0.0f, sk = 0.0f;
    for (int ch = lane; ch < d; ch += kWave) {
      const float q = load_as_f32(a.rows, a.dtype, q_at + ch), k = load_as_f32(a.rows, a.dtype, k_at + ch);
      sq = fmaf(q, q, sq);
      sk = fmaf(k, k, sk);
    }
    const float inv_q = (1.0f / sqrtf(wave_sum(sq) + a.unit_eps)) * a.q_scale;
    const float inv_k = 1.0f / sqrtf(wave_sum(sk) + a.unit_eps);
    float* into = a.unit + (size_t)item * 2 * d;
    float qk = 0.0f;
    for (int ch = lane; ch < d; ch += kWave) {
      const float q = load_as_f32(a.rows, a.dtype, q_at + ch) * inv_q, k = load_as_f32(a.rows, a.dtype, k_at + ch) * inv_k;
      into[ch] = q;
      into[d + ch] = k;
      qk = fmaf(q, k, qk);
    }
    qk = wave_sum(qk);
    if (lane == 0) a.gates[(size_t)a.tokens * a.heads * 2 + item] = qk;
  }
  // g and beta: a thread a (token, value head), dealt over the whole launch
  const int per_block = blockDim.x;
  for (int i = blockIdx.x * per_block + threadIdx.x; i < a.tokens * a.heads; i += gridDim.x * per_block) {
    const int t = i / a.heads, head = i % a.heads;
    const float* ba = a.ba + (size_t)t * 2 * a.heads;
    const float z = ba[a.heads + head] + a.dt_bias[head];
    const float soft = z > 20.0f ? z : log1pf(expf(z));
    a.gates[2 * (size_t)i] = expf(-a.rate[head] * soft);
    a.gates[2 * (size_t)i + 1] = 1.0f / (1.0f + expf(-ba[head]));
  }
}

// the sum of x over the GROUPS neighbouring lanes of a column (GROUPS a power of two up to 32): moves inside a row of
// 16 lanes, and one exchange between two rows for 32
template <int GROUPS>
__device__ __forceinline__ float column_sum(float x) {
  if (GROUPS >= 2) x += __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, x), 0xB1, 0xF, 0xF, true));   // lanes 1 0 3 2
  if (GROUPS >= 4) x += __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, x), 0x4E, 0xF, 0xF, true));   // lanes 2 3 0 1
  if (GROUPS >= 8) x += __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, x), 0x141, 0xF, 0xF, true));  // a half row mirrored
  if (GROUPS >= 16) x += __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, x), 0x140, 0xF, 0xF, true)); // a row mirrored
  if (GROUPS >= 32) x += __shfl_xor(x, 16, kWave);
  return x;
}

// what a thread needs of a token: its 8 key rows of q and k, the token's g, beta and q . k, its column's v
struct DeltaToken {
  float4 k[2], q[2], gate;
  float v;
};

template <int GROUPS>
__device__ __forceinline__ DeltaToken delta_token(const float* qk, const float* vs, const float* gs, int j, int group, int col_in_block,
                                                  int cols) {
  constexpr int kPad = GROUPS * 8;
  DeltaToken t;
  // (a thread's 8 key rows are two runs of 4, half the padded rows apart: a column's lanes then read 16 bytes each of
  // consecutive LDS, and no two of them meet in a bank)
  const float* qj = qk + j * 2 * kPad + group * 4;
  const float* kj = qj + kPad;
  t.k[0] = *(const float4*)kj;
  t.k[1] = *(const float4*)(kj + kPad / 2);
  t.q[0] = *(const float4*)qj;
  t.q[1] = *(const float4*)(qj + kPad / 2);
  t.gate = *(const float4*)(gs + 4 * j);
  t.v = vs[j * cols + col_in_block];
  return t;
}

// A thread keeps 8 key rows of one column; the GROUPS threads of a column are neighbouring lanes.  The state lies
// column by column, [slots, heads, value_dim, key_dim]: a column's threads read and write consecutive memory.
// A chunk's numbers are all asked for from memory before any of them is waited for.
template <int GROUPS>
__global__ __launch_bounds__(256) void gated_delta_kernel(DeltaArgs a) {
  extern __shared__ __attribute__((aligned(16))) float lds[];
  constexpr int kPad = GROUPS * 8;             // key rows as the threads see them (rows beyond key_dim are zero)
  constexpr int kPer = kWave / GROUPS;         // columns of a wave
  constexpr int kCols = 4 * kPer;              // columns of a block
  constexpr int kChunk = GROUPS >= 32 ? 16 : 32;  // tokens staged at a time
  constexpr int kQkLoads = (kChunk * 2 * kPad / 4 + 255) / 256;  // 16-byte loads a thread makes of a chunk's q and k
  constexpr int kVLoads = (kChunk * kCols + 255) / 256;
  const int b = blockIdx.z, head = blockIdx.y;
  const int slot = a.seq_slot[b];
  if (slot < 0) return;
  const int begin = a.seq_start[b], end = a.seq_start[b + 1];
  if (end <= begin) return;
  const int d = a.key_dim, e = a.value_dim;
  const int qk_head = head / (a.heads / a.groups);
  const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
  const int group = lane % GROUPS;             // which 8 key rows (two runs of 4)
  const int col_in_block = wave * kPer + lane / GROUPS;
  const int col = blockIdx.x * kCols + col_in_block;
  const bool live = col < e;
  float* qk = lds;                        // [chunk][2][kPad]: a token's q, then its k
  float* vs = qk + kChunk * 2 * kPad;     // [chunk][kCols]
  float* gs = vs + kChunk * kCols;        // [chunk][4]: g, beta, q . k
  float* state = a.state + (((size_t)slot * a.heads + head) * e + (live ? col : 0)) * d;
  int rows[8];  // the key rows this thread keeps
#pragma unroll
  for (int r = 0; r < 8; ++r) rows[r] = (r < 4 ? 0 : kPad / 2) + group * 4 + r % 4;
  float S[8];
#pragma unroll
  for (int r = 0; r < 8; ++r) S[r] = live && rows[r] < d ? state[rows[r]] : 0.0f;
  const size_t v_col0 = 2 * (size_t)a.groups * d;
  const float* qk_dots = a.gates + (size_t)a.tokens * a.heads * 2;
  const bool whole = d == kPad;  // a token's q and k are what LDS holds of it: copied 16 bytes at a time
  // A chunk's numbers wait in registers while the chunk before is worked on: they are asked for from memory before
  // that work begins, so a chunk's loads cost the recurrence nothing but the registers.
  float4 qk_in[kQkLoads];
  float v_in[kVLoads];
  float gate_in[3] = {0.0f, 0.0f, 0.0f};
  auto ask = [&](int t0) {
    const int count = min(kChunk, end - t0);
    if (whole) {
#pragma unroll
      for (int it = 0; it < kQkLoads; ++it) {
        const int f = threadIdx.x + it * 256, j = f / (kPad / 2), w = f % (kPad / 2);
        if (f < count * (kPad / 2)) qk_in[it] = *(const float4*)(a.unit + ((size_t)(t0 + j) * a.groups + qk_head) * 2 * d + 4 * w);
      }
    }
#pragma unroll
    for (int it = 0; it < kVLoads; ++it) {
      const int i = threadIdx.x + it * 256;
      const int t = t0 + i / kCols, cl = blockIdx.x * kCols + i % kCols;
      v_in[it] = i < count * kCols && cl < e ? load_as_f32(a.rows, a.dtype, (size_t)t * a.stride + v_col0 + (size_t)head * e + cl) : 0.0f;
    }
    if ((int)threadIdx.x < count) {
      const int t = t0 + threadIdx.x;
      gate_in[0] = a.gates[2 * ((size_t)t * a.heads + head)];
      gate_in[1] = a.gates[2 * ((size_t)t * a.heads + head) + 1];
      gate_in[2] = qk_dots[(size_t)t * a.groups + qk_head];
    }
  };
  ask(begin);
  for (int t0 = begin; t0 < end; t0 += kChunk) {
    const int count = min(kChunk, end - t0);
    __syncthreads();  // the chunk before has been read
    if (whole) {
#pragma unroll
      for (int it = 0; it < kQkLoads; ++it) {
        const int f = threadIdx.x + it * 256;
        if (f < count * (kPad / 2)) *(float4*)(qk + 4 * f) = qk_in[it];
      }
    } else {
      for (int i = threadIdx.x; i < count * 2 * kPad; i += blockDim.x) {
        const int j = i / (2 * kPad), ch = i % kPad, is_key = (i / kPad) & 1;
        qk[i] = ch < d ? a.unit[((size_t)(t0 + j) * a.groups + qk_head) * 2 * d + is_key * d + ch] : 0.0f;
      }
    }
#pragma unroll
    for (int it = 0; it < kVLoads; ++it) {
      const int i = threadIdx.x + it * 256;
      if (i < count * kCols) vs[i] = v_in[it];
    }
    if ((int)threadIdx.x < count) {
      gs[4 * threadIdx.x] = gate_in[0];
      gs[4 * threadIdx.x + 1] = gate_in[1];
      gs[4 * threadIdx.x + 2] = gate_in[2];
    }
    __syncthreads();
    if (t0 + kChunk < end) ask(t0 + kChunk);  // the next chunk's numbers, in flight from here on
    // a token's numbers are read from LDS while the token before is worked on
    DeltaToken next = delta_token<GROUPS>(qk, vs, gs, 0, group, col_in_block, kCols);
    for (int j = 0; j < count; ++j) {
      const DeltaToken now = next;
      if (j + 1 < count) next = delta_token<GROUPS>(qk, vs, gs, j + 1, group, col_in_block, kCols);
      __builtin_amdgcn_sched_barrier(0);  // (the reads stay up here, ahead of the work on the token before: left to itself the compiler moves them down to their use)
      const float kv[8] = {now.k[0].x, now.k[0].y, now.k[0].z, now.k[0].w, now.k[1].x, now.k[1].y, now.k[1].z, now.k[1].w};
      const float qv[8] = {now.q[0].x, now.q[0].y, now.q[0].z, now.q[0].w, now.q[1].x, now.q[1].y, now.q[1].z, now.q[1].w};
      float dot_k[2] = {0.0f, 0.0f}, dot_q[2] = {0.0f, 0.0f};
#pragma unroll
      for (int r = 0; r < 8; r += 2) {
        dot_k[0] = fmaf(S[r], kv[r], dot_k[0]);
        dot_k[1] = fmaf(S[r + 1], kv[r + 1], dot_k[1]);
        dot_q[0] = fmaf(S[r], qv[r], dot_q[0]);
        dot_q[1] = fmaf(S[r + 1], qv[r + 1], dot_q[1]);
      }
      const float with_k = column_sum<GROUPS>(dot_k[0] + dot_k[1]);
      const float with_q = column_sum<GROUPS>(dot_q[0] + dot_q[1]);
      const float g = now.gate.x;
      const float u = now.gate.y * (now.v - g * with_k);
#pragma unroll
      for (int r = 0; r < 8; ++r) S[r] = fmaf(kv[r], u, g * S[r]);
      if (group == 0 && live) a.out[((size_t)(t0 + j) * a.heads + head) * e + col] = fmaf(now.gate.z, u, g * with_q);
    }
  }
  if (!live) return;
#pragma unroll
  for (int r = 0; r < 8; ++r)
    if (rows[r] < d) state[rows[r]] = S[r];
}

}  // namespace

// Floats of scratch that nnis_gated_delta needs for `tokens` rows: the unit vectors, the gates and the products q . k.
extern "C" long long nnis_gated_delta_scratch(int tokens, int heads, int groups, int key_dim) {
  return (long long)tokens * ((long long)groups * 2 * key_dim + 2 * heads + groups);
}

// rows [tokens, stride] hold [q | k | v] behind the convolution; ba float32 [tokens, 2 * heads]; out float32 [tokens, heads *
// value_dim]; scratch: nnis_gated_delta_scratch floats
extern "C" int nnis_gated_delta(const void* rows, int dtype, int stride, const float* ba, const float* rate, const float* dt_bias,
                                float q_scale, float unit_eps, float* state, const int* seq_slot, const int* seq_start, int batch,
                                int tokens, int heads, int groups, int key_dim, int value_dim, float* out, float* scratch, void* stream) {
  NNIS_REQUIRE(nnis_dtype_ok(dtype), "gated_delta: unknown dtype %d", dtype);
  NNIS_REQUIRE(heads > 0 && groups > 0 && heads % groups == 0 && key_dim > 0 && key_dim <= 256 && value_dim > 0 && batch >= 0 && tokens >= 0,
               "gated_delta: bad sizes (heads %d on %d query/key heads, key channels %d: up to 256 are taken, value channels %d)", heads,
               groups, key_dim, value_dim);
  NNIS_REQUIRE(stride >= 2 * groups * key_dim + heads * value_dim, "gated_delta: rows of %d are too short", stride);
  NNIS_REQUIRE(rows && ba && rate && dt_bias && state && seq_slot && seq_start && out && scratch, "gated_delta: a pointer is missing");
  NNIS_REQUIRE(batch <= 65535 && heads <= 65535, "gated_delta: %d sequences exceed the grid limit", batch);
  if (batch == 0 || tokens == 0) return 0;
  DeltaArgs a;
  a.rows = rows; a.dtype = dtype; a.stride = stride; a.ba = ba; a.rate = rate; a.dt_bias = dt_bias; a.q_scale = q_scale;
  a.unit_eps = unit_eps; a.state = state; a.seq_slot = seq_slot; a.seq_start = seq_start; a.tokens = tokens; a.heads = heads;
  a.groups = groups; a.key_dim = key_dim; a.value_dim = value_dim; a.out = out;
  a.unit = scratch;
  a.gates = scratch + (size_t)tokens * groups * 2 * key_dim;
  hipStream_t s = (hipStream_t)stream;
  const int items = tokens * groups;
  hipLaunchKernelGGL(delta_prepare_kernel, dim3((items + 3) / 4), dim3(256), 0, s, a);
  const int need = (key_dim + 7) / 8;  // a thread keeps 8 key rows
  const int lane_groups = need <= 1 ? 1 : (need <= 2 ? 2 : (need <= 4 ? 4 : (need <= 8 ? 8 : (need <= 16 ? 16 : 32))));
  const int cols = 4 * (kWave / lane_groups);
  const int pad = lane_groups * 8;
  a.chunk = lane_groups >= 32 ? 16 : 32;  // (kChunk of the kernel)
  const size_t lds = (size_t)a.chunk * (2 * pad + cols + 4) * sizeof(float);
  const dim3 grid((value_dim + cols - 1) / cols, heads, batch);
  switch (lane_groups) {
    case 1: hipLaunchKernelGGL(gated_delta_kernel<1>, grid, dim3(256), lds, s, a); break;
    case 2: hipLaunchKernelGGL(gated_delta_kernel<2>, grid, dim3(256), lds, s, a); break;
    case 4: hipLaunchKernelGGL(gated_delta_kernel<4>, grid, dim3(256), lds, s, a); break;
    case 8: hipLaunchKernelGGL(gated_delta_kernel<8>, grid, dim3(256), lds, s, a); break;
    case 16: hipLaunchKernelGGL(gated_delta_kernel<16>, grid, dim3(256), lds, s, a); break;
    default: hipLaunchKernelGGL(gated_delta_kernel<32>, grid, dim3(256), lds, s, a); break;
  }
  NNIS_LAUNCH_CHECK("gated_delta");
  return 0;
}
