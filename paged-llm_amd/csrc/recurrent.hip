// Kernels for mixers that carry a state of fixed size per request instead of a growing cache:
//
//   causal_conv            a short causal convolution per channel over the tokens of each sequence, whose last
//                          taps - 1 inputs are carried from step to step in the request's state slot;
//   conv_state_update      leaves those inputs for the next step;
//   rotary_to_float        rotary encoding of heads into float rows (what enters a recurrence stays in float);
//   linear_recurrence      S_t = a_t S_(t-1) + k_t (g_t v_t)^T,  y_t = S_t^T q_t + skip * v_t  per head, S [N, P] in float
//                          in the state slot: the state-space scan (k = B, q = C, v = x, a = exp(-exp(A_log) dt), g = dt,
//                          skip = D) and retention (a = the head's decay, g = 1, no skip) are both this recurrence;
//   gated_group_norm       the gate and the root-mean-square norm over groups of channels behind a recurrence, in
//                          either order;
//   mlstm_gates            log-domain input and forget gates of a matrix memory under a running maximum: the decays and
//                          input factors that make it the linear recurrence above;
//   mlstm_output           behind that recurrence: the division by the normaliser, the norm per head, the gate.
//
// A batch is token-major without padding: sequence s owns rows cu_seqlens[s] .. cu_seqlens[s + 1] - 1, its state
// sits in slot state_slots[s], and seq_starts[s] == 0 says that it starts now, from a zero state, whatever the slot
// held.  Sequences may have no rows at all.  All arithmetic is float; T is the storage type of rows.
#include "common.h"

using namespace pllm;

__device__ __forceinline__ float load_as_f32(const void* p, int dtype, size_t i) {
  return dtype == PLLM_F32 ? reinterpret_cast<const float*>(p)[i] : __bfloat162float(reinterpret_cast<const bf16*>(p)[i]);
}
__device__ __forceinline__ float silu_f32(float z) { return z / (1.f + expf(-z)); }
// What a gate's raw value becomes behind a recurrence: z sigmoid(z), sigmoid(z), or 1 (no gate: nothing is read).
enum { kGateSilu = 0, kGateSigmoid = 1, kGateNone = 2 };
__device__ __forceinline__ float gate_f32(float z, int act) { return act == kGateSigmoid ? 1.f / (1.f + expf(-z)) : silu_f32(z); }

// ---------------------------------------------------------------------------------------------
constexpr int kMaxTaps = 16;      // most taps of a filter; filters of up to 8 taps take the smaller instance of the kernels
constexpr int kConvChunk = 64;     // tokens of one sequence that one workgroup walks

// out[t, c] = act(bias[c] + sum_j w[c, j] * in[t - (taps - 1) + j, c]); the last column of w meets the current token;
// inputs before the sequence's first token of this step come from the state (or are zero for a sequence that starts).
// state: [slots][channels][taps - 1] floats, oldest input first.
template <typename T, int MAXT>
__global__ __launch_bounds__(256) void causal_conv_kernel(
    const T* __restrict__ in, int in_stride, const float* __restrict__ w, const float* __restrict__ bias,
    float* state, size_t slot_stride, const int* __restrict__ state_slots,
    const int* __restrict__ seq_starts, const int* __restrict__ cu_seqlens, T* __restrict__ out, int out_stride,
    int channels, int taps, int act, int leave_state) {
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  const int seq = blockIdx.y;
  const int q_begin = cu_seqlens[seq], q_len = cu_seqlens[seq + 1] - q_begin;
  const int t0 = blockIdx.z * kConvChunk;
  if (c >= channels || t0 >= q_len) return;
  const int t1 = t0 + kConvChunk < q_len ? t0 + kConvChunk : q_len;
  const bool carried = seq_starts[seq] > 0;
  float* st = state + (size_t)state_slots[seq] * slot_stride + (size_t)c * (taps - 1);
  float wj[MAXT], win[MAXT];
#pragma unroll
  for (int j = 0; j < MAXT; ++j) {
    wj[j] = j < taps ? w[(size_t)c * taps + j] : 0.f;
    win[j] = 0.f;
    if (j < taps - 1) {
      const int rel = t0 - (taps - 1) + j;      // token of this step (>= 0) or an input of earlier steps (< 0)
      if (rel >= 0) win[j] = to_f32(in[(size_t)(q_begin + rel) * in_stride + c]);
      else if (carried) win[j] = st[(taps - 1) + rel];
    }
  }
  const float b = bias ? bias[c] : 0.f;
  // Eight tokens' inputs are asked for at once: one wait for memory per eight tokens, not per token.
  constexpr int kAhead = 8;
  for (int tb = t0; tb < t1; tb += kAhead) {
    T fetched[kAhead];
#pragma unroll
    for (int u = 0; u < kAhead; ++u)
      if (tb + u < t1) fetched[u] = in[(size_t)(q_begin + tb + u) * in_stride + c];
#pragma unroll
    for (int u = 0; u < kAhead; ++u) {
    const int t = tb + u;
    if (t >= t1) break;
    const float cur = to_f32(fetched[u]);
    float acc = b;
#pragma unroll
    for (int j = 0; j < MAXT - 1; ++j)
      if (j < taps - 1) acc = fmaf(wj[j], win[j], acc);
#pragma unroll
    for (int j = 0; j < MAXT; ++j)
      if (j == taps - 1) acc = fmaf(wj[j], cur, acc);
#pragma unroll
    for (int j = 0; j < MAXT - 1; ++j) {
      if (j < taps - 2) win[j] = win[j + 1];
      else if (j == taps - 2) win[j] = cur;
    }
    out[(size_t)(q_begin + t) * out_stride + c] = from_f32<T>(act ? silu_f32(acc) : acc);
    }
  }
  // With one chunk per sequence this thread alone has read the channel's state, and what it holds now are the last
  // taps - 1 inputs: it leaves them itself (with several chunks another kernel does, after all of them have read).
  if (leave_state) {
#pragma unroll
    for (int j = 0; j < MAXT - 1; ++j)
      if (j < taps - 1) st[j] = win[j];
  }
}

// state[k] <- the input at token q_len - (taps - 1) + k of this step, or what the state held for it.
template <typename T, int MAXT>
__global__ __launch_bounds__(256) void conv_state_update_kernel(
    const T* __restrict__ in, int in_stride, float* state, size_t slot_stride, const int* __restrict__ state_slots,
    const int* __restrict__ seq_starts, const int* __restrict__ cu_seqlens, int channels, int taps) {
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  const int seq = blockIdx.y;
  if (c >= channels) return;
  const int q_begin = cu_seqlens[seq], q_len = cu_seqlens[seq + 1] - q_begin;
  const bool carried = seq_starts[seq] > 0;
  float* st = state + (size_t)state_slots[seq] * slot_stride + (size_t)c * (taps - 1);
  float nv[MAXT];
#pragma unroll
  for (int k = 0; k < MAXT - 1; ++k) {
    nv[k] = 0.f;
    if (k < taps - 1) {
      const int rel = q_len - (taps - 1) + k;
      if (rel >= 0) nv[k] = to_f32(in[(size_t)(q_begin + rel) * in_stride + c]);
      else if (carried) nv[k] = st[q_len + k];
    }
  }
#pragma unroll
  for (int k = 0; k < MAXT - 1; ++k)
    if (k < taps - 1) st[k] = nv[k];
}

template <typename T, int MAXT>
static void launch_causal_conv(const void* in, int in_stride, const float* w, const float* bias, float* state, long slot_stride,
                               const int* state_slots, const int* seq_starts, const int* cu_seqlens, void* out, int out_stride,
                               int channels, int taps, int act, int num_seqs, int max_q_len, hipStream_t stream) {
  dim3 block(256), grid((channels + 255) / 256, num_seqs, (max_q_len + kConvChunk - 1) / kConvChunk);
  dim3 grid_state((channels + 255) / 256, num_seqs);
  const int fused = grid.z == 1 && taps > 1;
  hipLaunchKernelGGL((causal_conv_kernel<T, MAXT>), grid, block, 0, stream, (const T*)in, in_stride, w, bias, state,
                     (size_t)slot_stride, state_slots, seq_starts, cu_seqlens, (T*)out, out_stride, channels, taps, act, fused);
  if (taps > 1 && !fused)
    hipLaunchKernelGGL((conv_state_update_kernel<T, MAXT>), grid_state, block, 0, stream, (const T*)in, in_stride, state,
                       (size_t)slot_stride, state_slots, seq_starts, cu_seqlens, channels, taps);
}

PLLM_API int pllm_causal_conv(int dtype, const void* in, int in_stride, const float* w, const float* bias, float* state,
                              long slot_stride, const int* state_slots, const int* seq_starts, const int* cu_seqlens,
                              void* out, int out_stride, int channels, int taps, int act, int num_seqs, int max_q_len,
                              hipStream_t stream) {
  if (num_seqs <= 0 || max_q_len <= 0 || channels <= 0) return 0;
  if (taps < 1 || taps > kMaxTaps) return -2;
#define PLLM_CONV(T, MAXT) launch_causal_conv<T, MAXT>(in, in_stride, w, bias, state, slot_stride, state_slots, seq_starts, cu_seqlens, \
                                                       out, out_stride, channels, taps, act, num_seqs, max_q_len, stream)
  if (dtype == PLLM_F32) { if (taps <= 8) PLLM_CONV(float, 8); else PLLM_CONV(float, kMaxTaps); }
  else { if (taps <= 8) PLLM_CONV(bf16, 8); else PLLM_CONV(bf16, kMaxTaps); }
#undef PLLM_CONV
  PLLM_RETURN_LAST_ERROR();
}

// ---------------------------------------------------------------------------------------------
// out[t, h, i] = float(rotated in[t, h, i]) * scale: the first rot_dims elements of each head turn by the angle of the
// token's position (tables cos/sin [positions, rot_dims / 2]); partners are (i, i + rot_dims / 2) or, interleaved,
// (2i, 2i + 1).  The result stays in float.
// blockIdx.y == 1: a second set of heads `second_at` columns further in the rows, into out + second_out, times scale2
// (the keys behind the queries).
template <typename T>
__global__ void rotary_to_float_kernel(const T* __restrict__ in, int in_stride, const int* __restrict__ positions,
                                       const float* __restrict__ cos_t, const float* __restrict__ sin_t, float* __restrict__ out,
                                       int heads, int head_dim, int rot_dims, int interleaved, float scale, int second_at,
                                       size_t second_out, float scale2) {
  const int tok = blockIdx.x;
  if (blockIdx.y == 1) { in += second_at; out += second_out; scale = scale2; }
  const int half = rot_dims / 2;
  const T* row = in + (size_t)tok * in_stride;
  const size_t table = (size_t)positions[tok] * half;
  for (int idx = threadIdx.x; idx < heads * head_dim; idx += blockDim.x) {
    const int h = idx / head_dim, i = idx % head_dim;
    const T* head = row + (size_t)h * head_dim;
    float val = to_f32(head[i]);
    if (i < rot_dims) {
      int pair, partner;
      bool upper;
      if (interleaved) { pair = i >> 1; upper = i & 1; partner = i ^ 1; }
      else { upper = i >= half; pair = upper ? i - half : i; partner = upper ? i - half : i + half; }
      const float other = to_f32(head[partner]);
      float lo, hi;
      rotate_pair(upper ? other : val, upper ? val : other, cos_t[table + pair], sin_t[table + pair], lo, hi);
      val = upper ? hi : lo;
    }
    out[(size_t)tok * heads * head_dim + idx] = val * scale;
  }
}

PLLM_API int pllm_rotary_to_float(int dtype, const void* in, int in_stride, const int* positions, const float* cos_t,
                                  const float* sin_t, float* out, int num_tokens, int heads, int head_dim, int rot_dims,
                                  int interleaved, float scale, int sets, int second_at, long second_out, float scale2,
                                  hipStream_t stream) {
  if (num_tokens <= 0) return 0;
  if (rot_dims < 0 || rot_dims > head_dim || rot_dims % 2 || sets < 1 || sets > 2) return -2;
  dim3 grid(num_tokens, sets), block(256);
  if (dtype == PLLM_F32)
    hipLaunchKernelGGL(rotary_to_float_kernel<float>, grid, block, 0, stream, (const float*)in, in_stride, positions, cos_t, sin_t,
                       out, heads, head_dim, rot_dims, interleaved, scale, second_at, (size_t)second_out, scale2);
  else
    hipLaunchKernelGGL(rotary_to_float_kernel<bf16>, grid, block, 0, stream, (const bf16*)in, in_stride, positions, cos_t, sin_t,
                       out, heads, head_dim, rot_dims, interleaved, scale, second_at, (size_t)second_out, scale2);
  PLLM_RETURN_LAST_ERROR();
}

// ---------------------------------------------------------------------------------------------
struct RecurrenceArgs {
  const void* q; const void* k;        // [T, key_heads, N], element type qk_dtype, row stride qk_stride (elements)
  const void* v;                       // [T, heads, P], element type v_dtype, row stride v_stride
  const float* decay;                  // a_t per head: decay[t * decay_stride + h] (decay_stride 0: one number per head)
  const float* row_decay;              // or a decay per row of S: row_decay[t * row_decay_stride + h * N + n] (then `decay` is null and
                                       // S_t = diag(row_decay_t) S_(t-1) + k_t (g_t v_t)^T); not together with raw step sizes
  int row_decay_stride;
  const float* vscale;                 // g_t per head [T, heads], or null for 1
  // or both from raw step sizes [T, heads] (element type raw_dtype, row stride raw_stride):
  //   g_t = softplus(raw + raw_bias[h]) (no clamp),  a_t = exp(-exp(a_log[h]) * g_t)
  const void* raw; const float* raw_bias; const float* a_log;
  int raw_dtype, raw_stride;
  const float* skip;                   // [heads] or null
  float* state;                        // slot s, head h: state + s * slot_stride + h * N * P, as [N][P]
  const int* state_slots; const int* seq_starts; const int* cu_seqlens;
  float* out;                          // [T, heads * P]
  long slot_stride;
  int qk_dtype, qk_stride, v_dtype, v_stride, decay_stride;
  int heads, key_heads, N, P, pblocks;
  int ld;                              // elements of a row of S in the state and of a head in the output rows: P, or P + 1 when a
                                       // normaliser n_t = a_t n_(t-1) + g_t k_t stands behind the P columns (n as the last column of
                                       // S, n_t . q_t as the last element of the head's output)
};

// One workgroup per (sequence or chunk, head, block of 64 value channels); lane = value channel, so a token's update
// needs no exchange between lanes.  Wave w holds rows w * NR .. w * NR + NR - 1 of S in registers; with several waves
// their partial outputs are added through LDS in wave order.  A token's k and q are fetched by one lane each and read
// out lane by lane.
//
// Three forms (MODE):
//   kWhole       a sequence's tokens of this step one after the other, from the slot's state to the slot's state: steps
//                of single tokens and short portions;
//   kChunkState  long portions, first pass: the tokens of one chunk from a zero state, no outputs; leaves the chunk's
//                own contribution S_loc and the product of its decays in the workspace;
//   kChunkOut    third pass: a chunk's tokens from the state the sequence had when the chunk began (which the second
//                pass, recurrence_carry_kernel, has put where S_loc was), with outputs, no state written.
// With chunks, a long prompt's tokens are spread over the whole GPU instead of one workgroup per head; the additions
// into S associate differently than token by token, so results differ from the whole form by float rounding.
enum { kWhole = 0, kChunkState = 1, kChunkOut = 2 };

struct ChunkArgs {
  float* ws_state;      // [chunks][heads][N][P]
  float* ws_decay;      // [chunks][heads], or [chunks][heads][N] with a decay per row
  int chunk;            // tokens per chunk
  int num_seqs;
};

// Chunk j of the batch: sequences in order, each with ceil(q_len / chunk) chunks.  False when j is past the last one.
__device__ __forceinline__ bool find_chunk(const int* __restrict__ cu_seqlens, int num_seqs, int chunk, int j, int& seq, int& local) {
  int base = 0;
  for (int s = 0; s < num_seqs; ++s) {
    const int c = (cu_seqlens[s + 1] - cu_seqlens[s] + chunk - 1) / chunk;
    if (j < base + c) { seq = s; local = j - base; return true; }
    base += c;
  }
  return false;
}

template <int NR, int MAX_THREADS, int MODE>
__global__ __launch_bounds__(MAX_THREADS) void linear_recurrence_kernel(RecurrenceArgs a, ChunkArgs ca) {
  __shared__ float part[2][MAX_THREADS / 64][64];
  __shared__ float part_n[2][MAX_THREADS / 64];
  const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6, waves = blockDim.x >> 6;
  const int head = blockIdx.x / a.pblocks, pb = blockIdx.x % a.pblocks;
  const int p = pb * 64 + lane;
  const bool p_ok = p < a.P;
  int seq = blockIdx.y, local = 0;
  if (MODE != kWhole && !find_chunk(a.cu_seqlens, ca.num_seqs, ca.chunk, blockIdx.y, seq, local)) return;
  const int q_begin = a.cu_seqlens[seq], q_len = a.cu_seqlens[seq + 1] - q_begin;
  if (q_len <= 0) return;
  const int t_first = MODE == kWhole ? 0 : local * ca.chunk;
  const int t_last = MODE == kWhole ? q_len : (t_first + ca.chunk < q_len ? t_first + ca.chunk : q_len);
  const int kh = head / (a.heads / a.key_heads);
  const int n0 = wv * NR;
  const bool carried = a.seq_starts[seq] > 0;
  const int ld = a.ld;
  float* st = MODE == kWhole ? a.state + (size_t)a.state_slots[seq] * a.slot_stride + (size_t)head * a.N * ld
                             : ca.ws_state + ((size_t)blockIdx.y * a.heads + head) * a.N * ld;
  const bool from_state = MODE != kChunkState && (MODE == kChunkOut || carried);
  float S[NR];
#pragma unroll
  for (int i = 0; i < NR; ++i) S[i] = (from_state && p_ok && n0 + i < a.N) ? st[(size_t)(n0 + i) * ld + p] : 0.f;
  const float skip = a.skip ? a.skip[head] : 0.f;
  const float rate = a.raw ? expf(a.a_log[head]) : 0.f, raw_bias = a.raw ? a.raw_bias[head] : 0.f;
  const bool mine = lane < NR && n0 + lane < a.N;
  // The normaliser, where there is one: lane l of wave w holds n[w * NR + l], the row whose k and q it fetches anyway, so its
  // update is one multiply-add a token and n . q one sum over the wavefront; the head's first block of columns keeps it.
  const bool with_n = ld > a.P && pb == 0;
  float nl = (with_n && from_state && mine) ? st[(size_t)(n0 + lane) * ld + a.P] : 0.f;
  float decays = 1.f;
  // What a token needs from memory is asked for one token ahead, so that it travels while the token before is computed.
  struct Fetched { float k, q, x, a, g, d; };
  const bool by_row = a.row_decay != nullptr;
  float decays_l = 1.f;                                      // with a decay per row: the product for row n0 + lane
  auto fetch = [&](int t) {
    Fetched f;
    const size_t row = (size_t)(q_begin + t);
    const size_t qk_at = row * a.qk_stride + (size_t)kh * a.N + n0 + lane;
    f.k = mine ? load_as_f32(a.k, a.qk_dtype, qk_at) : 0.f;
    f.q = (MODE != kChunkState && mine) ? load_as_f32(a.q, a.qk_dtype, qk_at) : 0.f;
    f.x = p_ok ? load_as_f32(a.v, a.v_dtype, row * a.v_stride + (size_t)head * a.P + p) : 0.f;
    f.d = 1.f;
    if (by_row) {
      f.d = mine ? a.row_decay[row * a.row_decay_stride + (size_t)head * a.N + n0 + lane] : 1.f;
      f.a = 1.f;
      f.g = a.vscale ? a.vscale[row * a.heads + head] : 1.f;
    } else if (a.raw) {
      f.a = load_as_f32(a.raw, a.raw_dtype, row * a.raw_stride + head);
      f.g = 0.f;
    } else {
      f.a = a.decay[row * a.decay_stride + head];
      f.g = a.vscale ? a.vscale[row * a.heads + head] : 1.f;
    }
    return f;
  };
  // The state pass walks its chunk from the last token to the first: the chunk's own contribution is the sum over its
  // tokens of k_t (g_t v_t)^T times the decays of the tokens behind t, and that product is at hand when t is reached
  // from behind: one multiply-add per state row and token, no decay of the rows.
  Fetched next = fetch(MODE == kChunkState ? t_last - 1 : t_first);
  for (int n = t_first; n < t_last; ++n) {
    const int t = MODE == kChunkState ? t_last - 1 - (n - t_first) : n;
    const Fetched cur = next;
    if (n + 1 < t_last) next = fetch(MODE == kChunkState ? t - 1 : t + 1);
    const size_t row = (size_t)(q_begin + t);
    const float k_l = cur.k, q_l = cur.q, x = cur.x;
    float dec, xg, g;
    if (a.raw) {
      const float z = cur.a + raw_bias;
      const float step = z > 20.f ? z : log1pf(expf(z));
      dec = expf(-rate * step);
      g = step;
    } else {
      dec = cur.a;
      g = cur.g;
    }
    xg = x * g;
    if (by_row) {
      const float d_l = cur.d;
      if (MODE == kChunkState) {
        const float kw = k_l * decays_l;                  // decays_l: of the tokens behind t in the chunk, for this lane's row
#pragma unroll
        for (int i = 0; i < NR; ++i) S[i] = fmaf(row_lane(kw, i), xg, S[i]);
        if (with_n) nl = fmaf(kw, g, nl);
        decays_l *= d_l;
        continue;
      }
      float nq = 0.f;
      if (with_n) {
        nl = fmaf(k_l, g, d_l * nl);
        nq = wave_sum(nl * q_l);
      }
      float y[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int i = 0; i < NR; ++i) {
        const float kk = row_lane(k_l, i), qq = row_lane(q_l, i), dd = row_lane(d_l, i);
        S[i] = fmaf(kk, xg, dd * S[i]);
        y[i & 3] = fmaf(S[i], qq, y[i & 3]);
      }
      float total = (y[0] + y[1]) + (y[2] + y[3]);
      if (waves > 1) {
        part[t & 1][wv][lane] = total;
        if (with_n && lane == 0) part_n[t & 1][wv] = nq;
        __syncthreads();
        if (wv == 0) {
          total = part[t & 1][0][lane];
          for (int w = 1; w < waves; ++w) total += part[t & 1][w][lane];
          if (with_n) {
            nq = part_n[t & 1][0];
            for (int w = 1; w < waves; ++w) nq += part_n[t & 1][w];
          }
        }
      }
      if (wv == 0 && p_ok) a.out[row * (size_t)(a.heads * ld) + (size_t)head * ld + p] = fmaf(skip, x, total);
      if (wv == 0 && with_n && lane == 0) a.out[row * (size_t)(a.heads * ld) + (size_t)head * ld + a.P] = nq;
      continue;
    }
    if (MODE == kChunkState) {
      const float xw = xg * decays;                       // decays: of the tokens behind t in the chunk
#pragma unroll
      for (int i = 0; i < NR; ++i) S[i] = fmaf(row_lane(k_l, i), xw, S[i]);
      if (with_n) nl = fmaf(k_l, g * decays, nl);
      decays *= dec;
      continue;
    }
    float nq = 0.f;
    if (with_n) {
      nl = fmaf(k_l, g, dec * nl);
      nq = wave_sum(nl * q_l);
    }
    float y[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int i = 0; i < NR; ++i) {
      const float kk = row_lane(k_l, i), qq = row_lane(q_l, i);
      S[i] = fmaf(kk, xg, dec * S[i]);
      y[i & 3] = fmaf(S[i], qq, y[i & 3]);
    }
    float total = (y[0] + y[1]) + (y[2] + y[3]);
    if (waves > 1) {
      part[t & 1][wv][lane] = total;
      if (with_n && lane == 0) part_n[t & 1][wv] = nq;
      __syncthreads();
      if (wv == 0) {
        total = part[t & 1][0][lane];
        for (int w = 1; w < waves; ++w) total += part[t & 1][w][lane];
        if (with_n) {
          nq = part_n[t & 1][0];
          for (int w = 1; w < waves; ++w) nq += part_n[t & 1][w];
        }
      }
    }
    if (wv == 0 && p_ok) a.out[row * (size_t)(a.heads * ld) + (size_t)head * ld + p] = fmaf(skip, x, total);
    if (wv == 0 && with_n && lane == 0) a.out[row * (size_t)(a.heads * ld) + (size_t)head * ld + a.P] = nq;
  }
  if (MODE == kChunkOut) return;
  if (p_ok) {
#pragma unroll
    for (int i = 0; i < NR; ++i)
      if (n0 + i < a.N) st[(size_t)(n0 + i) * ld + p] = S[i];
  }
  if (with_n && mine) st[(size_t)(n0 + lane) * ld + a.P] = nl;
  if (MODE == kChunkState && by_row) {
    if (pb == 0 && mine) ca.ws_decay[((size_t)blockIdx.y * a.heads + head) * a.N + n0 + lane] = decays_l;
  } else if (MODE == kChunkState && threadIdx.x == 0 && pb == 0) ca.ws_decay[(size_t)blockIdx.y * a.heads + head] = decays;
}

// Second pass: per sequence and state element, chunk after chunk:  ws[c] <- the state before chunk c,
// S <- decays[c] * S + S_loc[c];  the state after the last chunk goes to the slot.
__global__ __launch_bounds__(256) void recurrence_carry_kernel(RecurrenceArgs a, ChunkArgs ca) {
  const size_t per_head = (size_t)a.N * a.ld, per_seq = per_head * a.heads;
  const size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int seq = blockIdx.y;
  if (idx >= per_seq) return;
  const int q_len = a.cu_seqlens[seq + 1] - a.cu_seqlens[seq];
  if (q_len <= 0) return;
  int base = 0;
  for (int s = 0; s < seq; ++s) base += (a.cu_seqlens[s + 1] - a.cu_seqlens[s] + ca.chunk - 1) / ca.chunk;
  const int chunks = (q_len + ca.chunk - 1) / ca.chunk;
  const int head = (int)(idx / per_head);
  const size_t decay_at = a.row_decay ? (size_t)head * a.N + (idx - (size_t)head * per_head) / a.ld : (size_t)head;
  const size_t decay_ld = a.row_decay ? (size_t)a.heads * a.N : (size_t)a.heads;
  float* slot = a.state + (size_t)a.state_slots[seq] * a.slot_stride + idx;
  float S = a.seq_starts[seq] > 0 ? *slot : 0.f;
  for (int c = 0; c < chunks; ++c) {
    float* w = ca.ws_state + (size_t)(base + c) * per_seq + idx;
    const float loc = *w;
    *w = S;
    S = fmaf(ca.ws_decay[(size_t)(base + c) * decay_ld + decay_at], S, loc);
  }
  *slot = S;
}

template <int MODE>
static void launch_recurrence(const RecurrenceArgs& a, const ChunkArgs& ca, dim3 grid, int waves, int need, hipStream_t stream) {
  dim3 block(64 * waves);
  if (waves > 4) hipLaunchKernelGGL((linear_recurrence_kernel<64, 1024, MODE>), grid, block, 0, stream, a, ca);
  else if (need <= 8) hipLaunchKernelGGL((linear_recurrence_kernel<8, 256, MODE>), grid, block, 0, stream, a, ca);
  else if (need <= 16) hipLaunchKernelGGL((linear_recurrence_kernel<16, 256, MODE>), grid, block, 0, stream, a, ca);
  else if (need <= 32) hipLaunchKernelGGL((linear_recurrence_kernel<32, 256, MODE>), grid, block, 0, stream, a, ca);
  else hipLaunchKernelGGL((linear_recurrence_kernel<64, 256, MODE>), grid, block, 0, stream, a, ca);
}

// v_cols: P, or P - 1 for a recurrence with a normaliser (v holds P - 1 columns per head; column P - 1 of S holds
// n_t = a_t n_(t-1) + g_t k_t, and the last element of a head's output n_t . q_t).
// chunk == 0: every sequence token by token in one workgroup per (head, block of channels).  chunk > 0: the three passes
// over chunks of that many tokens; ws_state holds max_chunks * heads * N * P floats and ws_decay max_chunks * heads, with
// max_chunks >= sum over the sequences of ceil(q_len / chunk) (total tokens / chunk + num_seqs is enough).
PLLM_API int pllm_linear_recurrence(const void* q, const void* k, int qk_dtype, int qk_stride, const void* v, int v_dtype,
                                    int v_stride, const float* decay, int decay_stride, const float* row_decay, int row_decay_stride,
                                    const float* vscale, const float* skip,
                                    const void* raw, int raw_dtype, int raw_stride, const float* raw_bias, const float* a_log,
                                    float* state, long slot_stride, const int* state_slots, const int* seq_starts,
                                    const int* cu_seqlens, float* out, int num_seqs, int heads, int key_heads, int N, int P,
                                    int v_cols, int chunk, int max_chunks, float* ws_state, float* ws_decay, hipStream_t stream) {
  if (num_seqs <= 0) return 0;
  if (heads <= 0 || key_heads <= 0 || heads % key_heads || N <= 0 || N > 1024 || P <= 0 || (v_cols != P && v_cols != P - 1)) return -2;
  if ((raw && (!raw_bias || !a_log)) || (!raw && !decay && !row_decay) || (row_decay && (raw || decay || heads != key_heads))) return -2;
  if (chunk < 0 || (chunk > 0 && (max_chunks <= 0 || max_chunks > 65535 || !ws_state || !ws_decay)) || num_seqs > 65535) return -2;
  RecurrenceArgs a;
  a.q = q; a.k = k; a.v = v; a.decay = decay; a.row_decay = row_decay; a.row_decay_stride = row_decay_stride; a.vscale = vscale; a.skip = skip; a.state = state;
  a.state_slots = state_slots; a.seq_starts = seq_starts; a.cu_seqlens = cu_seqlens; a.out = out;
  a.slot_stride = slot_stride; a.qk_dtype = qk_dtype; a.qk_stride = qk_stride; a.v_dtype = v_dtype; a.v_stride = v_stride;
  a.raw = raw; a.raw_dtype = raw_dtype; a.raw_stride = raw_stride; a.raw_bias = raw_bias; a.a_log = a_log;
  a.decay_stride = decay_stride; a.heads = heads; a.key_heads = key_heads; a.N = N; a.P = v_cols; a.ld = P; a.pblocks = (v_cols + 63) / 64;
  ChunkArgs ca{ws_state, ws_decay, chunk, num_seqs};
  const int waves = (N + 63) / 64, need = (N + waves - 1) / waves;   // rows of S per wave
  if (chunk == 0) {
    launch_recurrence<kWhole>(a, ca, dim3(heads * a.pblocks, num_seqs), waves, need, stream);
  } else {
    launch_recurrence<kChunkState>(a, ca, dim3(heads * a.pblocks, max_chunks), waves, need, stream);
    const size_t per_seq = (size_t)heads * N * P;     // (P: all columns of a row of S, the normaliser's among them)
    hipLaunchKernelGGL(recurrence_carry_kernel, dim3((unsigned)((per_seq + 255) / 256), num_seqs), dim3(256), 0, stream, a, ca);
    launch_recurrence<kChunkOut>(a, ca, dim3(heads * a.pblocks, max_chunks), waves, need, stream);
  }
  PLLM_RETURN_LAST_ERROR();
}

// ---------------------------------------------------------------------------------------------
// decay[t, h] = exp(-exp(A_log[h]) * dt),  dt[t, h] = softplus(raw[t, h] + bias[h])  (no clamp), both float.
template <typename T>
__global__ void step_sizes_kernel(const T* __restrict__ raw, int raw_stride, const float* __restrict__ bias,
                                  const float* __restrict__ a_log, float* __restrict__ dt, float* __restrict__ decay,
                                  int num_tokens, int heads) {
  const int idx = blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= num_tokens * heads) return;
  const int t = idx / heads, h = idx % heads;
  const float z = to_f32(raw[(size_t)t * raw_stride + h]) + bias[h];
  const float step = z > 20.f ? z : log1pf(expf(z));
  dt[idx] = step;
  decay[idx] = expf(-expf(a_log[h]) * step);
}

PLLM_API int pllm_step_sizes(int dtype, const void* raw, int raw_stride, const float* bias, const float* a_log, float* dt,
                             float* decay, int num_tokens, int heads, hipStream_t stream) {
  if (num_tokens <= 0 || heads <= 0) return 0;
  dim3 block(256), grid((num_tokens * heads + 255) / 256);
  if (dtype == PLLM_F32)
    hipLaunchKernelGGL(step_sizes_kernel<float>, grid, block, 0, stream, (const float*)raw, raw_stride, bias, a_log, dt, decay, num_tokens, heads);
  else
    hipLaunchKernelGGL(step_sizes_kernel<bf16>, grid, block, 0, stream, (const bf16*)raw, raw_stride, bias, a_log, dt, decay, num_tokens, heads);
  PLLM_RETURN_LAST_ERROR();
}

// ---------------------------------------------------------------------------------------------
// Behind a recurrence: y [T, inner] float, gate [T, inner] (row stride gate_stride), groups of `group` channels.
//   gate_first:   u = y * silu(gate);  out = u / sqrt(mean_group(u^2) + eps) * w
//   otherwise:    out = y / sqrt(mean_group(y^2) + eps) * silu(gate) [* w]
// One workgroup per token.  With at least as many groups as waves each wave takes whole groups; else the workgroup
// takes the groups one after the other.
template <typename T>
__global__ __launch_bounds__(256) void gated_group_norm_kernel(const float* __restrict__ y, const T* __restrict__ gate,
                                                               int gate_stride, const float* __restrict__ w, T* __restrict__ out,
                                                               int inner, int group, int gate_first, int gate_act, float eps) {
  __shared__ float scratch[16];
  const int row = blockIdx.x;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, waves = blockDim.x >> 6;
  const int groups = inner / group;
  const float* yr = y + (size_t)row * inner;
  const T* gr = gate + (size_t)row * gate_stride;
  T* orow = out + (size_t)row * inner;
  const bool by_wave = groups >= waves;
  const int first = by_wave ? wave : 0, step = by_wave ? waves : 1;
  const int i0 = by_wave ? lane : threadIdx.x, di = by_wave ? 64 : blockDim.x;
  for (int g = first; g < groups; g += step) {
    const int base = g * group;
    float ss = 0.f;
    for (int i = i0; i < group; i += di) {
      float u = yr[base + i];
      if (gate_first && gate_act != kGateNone) u *= gate_f32(to_f32(gr[base + i]), gate_act);
      ss = fmaf(u, u, ss);
    }
    ss = by_wave ? wave_sum(ss) : block_sum(ss, scratch);
    const float inv = 1.f / sqrtf(ss / (float)group + eps);
    for (int i = i0; i < group; i += di) {
      const float s = gate_act == kGateNone ? 1.f : gate_f32(to_f32(gr[base + i]), gate_act);
      float u = yr[base + i];
      u = gate_first ? (u * s) * inv : (u * inv) * s;
      if (w) u *= w[base + i];
      orow[base + i] = from_f32<T>(u);
    }
  }
}

// The same for groups whose channels a wave (or, with fewer groups than waves, a few waves side by side) holds in
// registers: every value is read once, four channels per lane and load.  Needs group % 4 == 0, rows that start on
// 16-byte (float) and 8-byte (bfloat16) boundaries, and at most kGroupRegs * 256 channels per wave.
constexpr int kGroupRegs = 8;

template <typename T> struct alignas(4 * sizeof(T)) Quad { T v[4]; };

template <typename T>
__global__ __launch_bounds__(256) void gated_group_norm_regs_kernel(const float* __restrict__ y, const T* __restrict__ gate,
                                                                    int gate_stride, const float* __restrict__ w, T* __restrict__ out,
                                                                    int inner, int group, int gate_first, int gate_act, float eps) {
  __shared__ float scratch[4];
  const int row = blockIdx.x;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int groups = inner / group;
  const int parts = groups >= 4 ? 1 : 4 / groups;          // waves side by side on one group (groups 1 or 2; 3 gives 1)
  const int slice = group / parts;                         // channels of a group that one wave takes
  const float* yr = y + (size_t)row * inner;
  const T* gr = gate + (size_t)row * gate_stride;
  T* orow = out + (size_t)row * inner;
  for (int g = wave / parts; g < groups; g += 4 / parts) {
    const int base = g * group + (wave % parts) * slice;
    float u[kGroupRegs][4], s[kGroupRegs][4];
    float ss = 0.f;
#pragma unroll
    for (int j = 0; j < kGroupRegs; ++j) {
      const int at = (j * 64 + lane) * 4;
      if (at < slice) {
        const float4 yv = *reinterpret_cast<const float4*>(yr + base + at);
        Quad<T> gv;
        if (gate_act != kGateNone) gv = *reinterpret_cast<const Quad<T>*>(gr + base + at);
        const float yy[4] = {yv.x, yv.y, yv.z, yv.w};
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          s[j][e] = gate_act == kGateNone ? 1.f : gate_f32(to_f32(gv.v[e]), gate_act);
          u[j][e] = gate_first ? yy[e] * s[j][e] : yy[e];
          ss = fmaf(u[j][e], u[j][e], ss);
        }
      }
    }
    ss = wave_sum(ss);
    if (parts > 1) {                                       // (then every wave runs this loop exactly once)
      scratch[wave] = ss;
      __syncthreads();
      ss = 0.f;
      for (int k = 0; k < parts; ++k) ss += scratch[(wave / parts) * parts + k];
    }
    const float inv = 1.f / sqrtf(ss / (float)group + eps);
#pragma unroll
    for (int j = 0; j < kGroupRegs; ++j) {
      const int at = (j * 64 + lane) * 4;
      if (at < slice) {
        Quad<T> o;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          float r = gate_first ? u[j][e] * inv : (u[j][e] * inv) * s[j][e];
          if (w) r *= w[base + at + e];
          o.v[e] = from_f32<T>(r);
        }
        *reinterpret_cast<Quad<T>*>(orow + base + at) = o;
      }
    }
  }
}

template <typename T>
static bool group_norm_in_registers(const float* y, const void* gate, int gate_stride, void* out, int inner, int group) {
  const int groups = inner / group, parts = groups >= 4 ? 1 : 4 / groups;
  return group % (4 * parts) == 0 && group / parts <= kGroupRegs * 256 && inner % 4 == 0 && gate_stride % 4 == 0 &&
         (uintptr_t)y % 16 == 0 && (uintptr_t)gate % (4 * sizeof(T)) == 0 && (uintptr_t)out % (4 * sizeof(T)) == 0;
}

PLLM_API int pllm_gated_group_norm(int dtype, const float* y, const void* gate, int gate_stride, const float* w, void* out,
                                   int num_tokens, int inner, int group, int gate_first, int gate_act, float eps, hipStream_t stream) {
  if (num_tokens <= 0) return 0;
  if (group <= 0 || inner % group || gate_act < 0 || gate_act > kGateNone || (!gate && gate_act != kGateNone)) return -2;
  dim3 grid(num_tokens), block(256);
  if (dtype == PLLM_F32) {
    if (group_norm_in_registers<float>(y, gate, gate_stride, out, inner, group))
      hipLaunchKernelGGL(gated_group_norm_regs_kernel<float>, grid, block, 0, stream, y, (const float*)gate, gate_stride, w, (float*)out,
                         inner, group, gate_first, gate_act, eps);
    else
      hipLaunchKernelGGL(gated_group_norm_kernel<float>, grid, block, 0, stream, y, (const float*)gate, gate_stride, w, (float*)out,
                         inner, group, gate_first, gate_act, eps);
  } else {
    if (group_norm_in_registers<bf16>(y, gate, gate_stride, out, inner, group))
      hipLaunchKernelGGL(gated_group_norm_regs_kernel<bf16>, grid, block, 0, stream, y, (const bf16*)gate, gate_stride, w, (bf16*)out,
                         inner, group, gate_first, gate_act, eps);
    else
      hipLaunchKernelGGL(gated_group_norm_kernel<bf16>, grid, block, 0, stream, y, (const bf16*)gate, gate_stride, w, (bf16*)out,
                         inner, group, gate_first, gate_act, eps);
  }
  PLLM_RETURN_LAST_ERROR();
}

// ---------------------------------------------------------------------------------------------
// Gates of a matrix memory with exponential input gates (mLSTM), per sequence and head, all in float:
//   i_t = cap tanh((raw_i + b_i) / cap),   f_t = log sigmoid(cap tanh((raw_f + b_f) / cap))         (log-domain gates)
//   m_t = max(f_t + m_(t-1), i_t)          a running maximum; m = 0 in front of a sequence's first token
//   decay[t, h] = exp(f_t + m_(t-1) - m_t),   take[t, h] = exp(i_t - m_t),   m_out[t, h] = m_t,
// so that S_t = decay_t S_(t-1) + take_t k_t v_t^T is the memory divided by exp(m_t).  m of a sequence's last token of
// this step stays in state[slot][m_at + h].
// One wavefront per (head, sequence) walks the sequence's tokens in blocks of 64: a lane makes its token's gates, and the
// maxima are a scan over the lanes of the maps m -> max(a + m, b) ((a, b) of later tokens after (a', b') of earlier
// ones is (a' + a, max(b' + a, b))); a lane past the sequence's end holds the identity (0, -inf).
__global__ __launch_bounds__(64) void mlstm_gates_kernel(const void* __restrict__ raw_i, const void* __restrict__ raw_f, int raw_dtype,
                                                         int raw_stride, const float* __restrict__ bias_i, const float* __restrict__ bias_f,
                                                         float cap, float* state, long slot_stride, int m_at,
                                                         const int* __restrict__ state_slots, const int* __restrict__ seq_starts,
                                                         const int* __restrict__ cu_seqlens, float* __restrict__ decay,
                                                         float* __restrict__ take, float* __restrict__ m_out, int heads) {
  const int lane = threadIdx.x, head = blockIdx.x, seq = blockIdx.y;
  const int q_begin = cu_seqlens[seq], q_len = cu_seqlens[seq + 1] - q_begin;
  if (q_len <= 0) return;
  float* st = state + (size_t)state_slots[seq] * slot_stride + m_at + head;
  float m_in = seq_starts[seq] > 0 ? *st : 0.f;
  const float bi = bias_i ? bias_i[head] : 0.f, bf = bias_f ? bias_f[head] : 0.f;
  for (int t0 = 0; t0 < q_len; t0 += 64) {
    const int t = t0 + lane;
    const bool ok = t < q_len;
    const size_t row = (size_t)(q_begin + (ok ? t : q_len - 1));
    float gi = load_as_f32(raw_i, raw_dtype, row * raw_stride + head) + bi;
    float gf = load_as_f32(raw_f, raw_dtype, row * raw_stride + head) + bf;
    if (cap > 0.f) {
      gi = cap * tanhf(gi / cap);
      gf = cap * tanhf(gf / cap);
    }
    gf = fminf(gf, 0.f) - log1pf(expf(-fabsf(gf)));
    float a = ok ? gf : 0.f, b = ok ? gi : -INFINITY;
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
      const float a_p = __shfl_up(a, off, 64), b_p = __shfl_up(b, off, 64);
      if (lane >= off) {
        b = fmaxf(b_p + a, b);
        a = a_p + a;
      }
    }
    const float m_t = fmaxf(a + m_in, b);
    float m_prev = __shfl_up(m_t, 1, 64);
    if (lane == 0) m_prev = m_in;
    if (ok) {
      const size_t at = row * heads + head;
      decay[at] = expf(gf + m_prev - m_t);
      take[at] = expf(gi - m_t);
      m_out[at] = m_t;
    }
    m_in = __shfl(m_t, 63, 64);
  }
  if (lane == 0) *st = m_in;
}

PLLM_API int pllm_mlstm_gates(const void* raw_i, const void* raw_f, int raw_dtype, int raw_stride, const float* bias_i,
                              const float* bias_f, float cap, float* state, long slot_stride, int m_at, const int* state_slots,
                              const int* seq_starts, const int* cu_seqlens, float* decay, float* take, float* m_out, int num_seqs,
                              int heads, hipStream_t stream) {
  if (num_seqs <= 0) return 0;
  if (heads <= 0 || num_seqs > 65535 || !raw_i || !raw_f || !state) return -2;
  hipLaunchKernelGGL(mlstm_gates_kernel, dim3(heads, num_seqs), dim3(64), 0, stream, raw_i, raw_f, raw_dtype, raw_stride, bias_i, bias_f,
                     cap, state, slot_stride, m_at, state_slots, seq_starts, cu_seqlens, decay, take, m_out, heads);
  PLLM_RETURN_LAST_ERROR();
}

// Behind the recurrence of a matrix memory with a normaliser: y [T, heads, P + 1] float holds S_t^T q_t in its first P
// columns and n_t . q_t in the last; m [T, heads] the running maxima.  Per token and head, in float:
//   o = y[:P] qscale / (max(|y[P] qscale|, exp(-m)) + 1e-6);   u = o / sqrt(mean(o^2) + eps) * w[head, :] * sigmoid(gate[head, :]);
// out [T, heads * P] in the type T.  One wavefront per (token, head).
template <typename T>
__global__ __launch_bounds__(64) void mlstm_output_kernel(const float* __restrict__ y, const float* __restrict__ m, const void* __restrict__ gate,
                                                          int gate_dtype, int gate_stride, const float* __restrict__ w, T* __restrict__ out,
                                                          int heads, int P, float qscale, float eps) {
  const int lane = threadIdx.x, tok = blockIdx.x, head = blockIdx.y;
  const float* row = y + ((size_t)tok * heads + head) * (P + 1);
  const float den = fmaxf(fabsf(row[P] * qscale), expf(-m[(size_t)tok * heads + head])) + 1e-6f;
  const float f = qscale / den;
  float sq = 0.f;
  for (int p = lane; p < P; p += 64) {
    const float o = row[p] * f;
    sq = fmaf(o, o, sq);
  }
  const float inv = 1.f / sqrtf(wave_sum(sq) / (float)P + eps);
  for (int p = lane; p < P; p += 64) {
    const size_t c = (size_t)head * P + p;
    const float g = load_as_f32(gate, gate_dtype, (size_t)tok * gate_stride + c);
    out[(size_t)tok * heads * P + c] = from_f32<T>(row[p] * f * inv * (w ? w[c] : 1.f) / (1.f + expf(-g)));
  }
}

PLLM_API int pllm_mlstm_output(int out_dtype, const float* y, const float* m, const void* gate, int gate_dtype, int gate_stride,
                               const float* w, void* out, int num_tokens, int heads, int P, float qscale, float eps, hipStream_t stream) {
  if (num_tokens <= 0) return 0;
  if (heads <= 0 || heads > 65535 || P <= 0) return -2;
  dim3 grid(num_tokens, heads), block(64);
  if (out_dtype == PLLM_F32)
    hipLaunchKernelGGL(mlstm_output_kernel<float>, grid, block, 0, stream, y, m, gate, gate_dtype, gate_stride, w, (float*)out, heads, P, qscale, eps);
  else
    hipLaunchKernelGGL(mlstm_output_kernel<bf16>, grid, block, 0, stream, y, m, gate, gate_dtype, gate_stride, w, (bf16*)out, heads, P, qscale, eps);
  PLLM_RETURN_LAST_ERROR();
}

// ---------------------------------------------------------------------------------------------
// out[t, c] = silu(rows[t, c]) as float for c < cols: the activated q, k and v of a recurrence whose operands stay in float
// from here on.  rows has a row stride of its own and either element type.
__global__ __launch_bounds__(256) void silu_to_float_kernel(const void* __restrict__ rows, int dtype, int stride, float* __restrict__ out,
                                                            int cols, size_t total) {
  const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= total) return;
  const size_t t = i / cols, c = i - t * cols;
  out[i] = silu_f32(load_as_f32(rows, dtype, t * stride + c));
}

PLLM_API int pllm_silu_to_float(const void* rows, int dtype, int stride, float* out, int num_tokens, int cols, hipStream_t stream) {
  if (num_tokens <= 0 || cols <= 0) return 0;
  const size_t total = (size_t)num_tokens * cols;
  hipLaunchKernelGGL(silu_to_float_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, stream, rows, dtype, stride, out, cols, total);
  PLLM_RETURN_LAST_ERROR();
}

// A forget gate with a lower bound per channel, whose complement is the key (a recurrence without a key product):
//   f = lower + (1 - lower) * sigmoid(raw_f + bias),   k = 1 - f,   q = silu(raw_q),
// from rows [T, >= 2 channels] laid out [raw_q | raw_f | ...]; out float [3][T][channels] = q, k, f.
__global__ __launch_bounds__(256) void bounded_forget_gates_kernel(const void* __restrict__ rows, int dtype, int stride,
                                                                   const float* __restrict__ bias, const float* __restrict__ lower,
                                                                   float* __restrict__ out, int channels, size_t total) {
  const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= total) return;
  const size_t t = i / channels, c = i - t * channels;
  const float zq = load_as_f32(rows, dtype, t * stride + c);
  const float zf = load_as_f32(rows, dtype, t * stride + channels + c) + (bias ? bias[c] : 0.f);
  const float lo = lower ? lower[c] : 0.f;
  const float sg = 1.f / (1.f + expf(-zf));
  const float f = lo + (1.f - lo) * sg;
  out[i] = silu_f32(zq);
  out[total + i] = 1.f - f;
  out[2 * total + i] = f;
}

PLLM_API int pllm_bounded_forget_gates(const void* rows, int dtype, int stride, const float* bias, const float* lower, float* out,
                                       int num_tokens, int channels, hipStream_t stream) {
  if (num_tokens <= 0 || channels <= 0) return 0;
  const size_t total = (size_t)num_tokens * channels;
  hipLaunchKernelGGL(bounded_forget_gates_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, stream, rows, dtype, stride, bias,
                     lower, out, channels, total);
  PLLM_RETURN_LAST_ERROR();
}
