// What an attention layer with normed queries and keys does between its input product and the paged attention
// kernels, and between those kernels and its output product:
//
//   attn_prepare      per token and head, from the float sums of the q/k/v product: + bias, a short causal convolution
//                     over time on every channel (inputs of earlier steps from the request's state slot), rotary
//                     encoding of the first rot elements of q and k heads (pairs (i, i + rot/2) or (2i, 2i + 1)),
//                     q and k divided by their root mean square over the head (unless qk_norm is 0), q written as rows of padded heads,
//                     k and v written into their cache pages; the values as projected (v_mode 0), divided by their root
//                     mean square over the head (1), or the keys as they were before their rotation, the product
//                     holding no value columns at all (2);
//   conv_inputs_keep  leaves the last taps - 1 projected rows of every sequence in its state slot;
//   gate_heads        out[t, h, :dv] = o[t, h, :dv] * sigmoid(gate[t, h]) from padded heads to packed ones.
//
// All arithmetic is float; T is the storage type of the query rows and of the pages.  Keys and values may differ in
// width (d and dv): the pages and the query rows hold heads of D >= max(d, dv) elements, the rest zero, so that the
// paged attention kernels, which know one head size, serve both.
#include "common.h"

using namespace pllm;

constexpr int kPrepMaxHead = 256;
constexpr int kPrepMaxTaps = 16;

// proj      [tokens, ld] float: columns [q heads * d | kv heads * d | kv heads * dv | ...]
// bias      [channels] float or null;  conv_w [channels, taps] float or null (null: no convolution)
// state     [slots][taps - 1][channels] float, oldest first: the projected values (with bias) of the tokens before
//           this step's; a sequence with seq_starts == 0 has zeros there whatever the slot holds.
// q_out     [tokens, heads * D];  k_pages [pages, kv heads, block, D];  v_pages [pages, kv heads, D, block]
template <typename T>
__global__ __launch_bounds__(64) void attn_prepare_kernel(
    const float* __restrict__ proj, int ld, const float* __restrict__ bias, const float* __restrict__ conv_w, int taps,
    const float* __restrict__ state, size_t slot_stride, const int* __restrict__ state_slots, const int* __restrict__ seq_starts,
    const int* __restrict__ cu_seqlens, int num_seqs, const int* __restrict__ positions, const float* __restrict__ cos_table,
    const float* __restrict__ sin_table, int rot, int interleaved, float eps, int qk_norm, int v_mode, int heads, int kv_heads, int d, int dv, int D,
    T* __restrict__ q_out, const int* __restrict__ slot_mapping, T* __restrict__ k_pages, T* __restrict__ v_pages, int block_size) {
  __shared__ float vals[kPrepMaxHead];
  const int lane = threadIdx.x;
  const int tok = blockIdx.x, hs = blockIdx.y;
  // which head this is: a query head, a key head or a value head
  int kind, head, base, width;
  if (hs < heads) { kind = 0; head = hs; base = hs * d; width = d; }
  else if (hs < heads + kv_heads) { kind = 1; head = hs - heads; base = heads * d + head * d; width = d; }
  else if (v_mode == 2) { kind = 2; head = hs - heads - kv_heads; base = heads * d + head * d; width = d; }
  else { kind = 2; head = hs - heads - kv_heads; base = (heads + kv_heads) * d + head * dv; width = dv; }
  const int channels = (heads + kv_heads) * d + (v_mode == 2 ? 0 : kv_heads * dv);

  int q_begin = 0, carried = 0;
  const float* st = nullptr;
  if (taps > 1) {
    int lo = 0, hi = num_seqs - 1;
    while (lo < hi) {
      const int mid = (lo + hi + 1) >> 1;
      if (cu_seqlens[mid] <= tok) lo = mid; else hi = mid - 1;
    }
    q_begin = cu_seqlens[lo];
    carried = seq_starts[lo] > 0;
    st = state + (size_t)state_slots[lo] * slot_stride;
  }
  const int local = tok - q_begin;

  float x[4];
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    const int e = lane + 64 * r;
    float v = 0.f;
    if (e < width) {
      const int c = base + e;
      const float b = bias ? bias[c] : 0.f;
      if (taps > 1) {
        for (int j = 0; j < taps; ++j) {
          const int rel = local - (taps - 1) + j;              // token of this step, or of earlier steps (< 0)
          float u = 0.f;
          if (rel >= 0) u = proj[(size_t)(q_begin + rel) * ld + c] + b;
          else if (carried) u = st[(size_t)(taps - 1 + rel) * channels + c];
          v = fmaf(conv_w[(size_t)c * taps + j], u, v);
        }
      } else {
        v = proj[(size_t)tok * ld + c] + b;
        if (conv_w) v *= conv_w[c];                              // one tap: a factor per channel
      }
    }
    x[r] = v;
    if (e < kPrepMaxHead) vals[e] = v;
  }
  __syncthreads();
  if (kind < 2) {
    const int pos = positions[tok];
    const int half = rot >> 1;
    float sq = 0.f;
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int e = lane + 64 * r;
      if (e < width && e < rot) {
        int pair, mate;
        bool low;
        if (interleaved) { pair = e >> 1; low = !(e & 1); mate = e ^ 1; }
        else { low = e < half; pair = low ? e : e - half; mate = low ? e + half : e - half; }
        const float c = cos_table[(size_t)pos * half + pair], s = sin_table[(size_t)pos * half + pair];
        const float other = vals[mate];
        float out_lo, out_hi;
        if (low) rotate_pair(x[r], other, c, s, out_lo, out_hi); else rotate_pair(other, x[r], c, s, out_lo, out_hi);
        x[r] = low ? out_lo : out_hi;
      }
      if (e < width) sq = fmaf(x[r], x[r], sq);
    }
    if (qk_norm) {
      const float inv = 1.f / sqrtf(wave_sum(sq) / (float)width + eps);
#pragma unroll
      for (int r = 0; r < 4; ++r) x[r] *= inv;
    }
  }
  if (kind == 2 && v_mode == 1) {
    float sq = 0.f;
#pragma unroll
    for (int r = 0; r < 4; ++r)
      if (lane + 64 * r < width) sq = fmaf(x[r], x[r], sq);
    const float inv = 1.f / sqrtf(wave_sum(sq) / (float)width + eps);
#pragma unroll
    for (int r = 0; r < 4; ++r) x[r] *= inv;
  }
  if (kind == 0) {
    T* out = q_out + ((size_t)tok * heads + head) * D;
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int e = lane + 64 * r;
      if (e < D) out[e] = from_f32<T>(e < width ? x[r] : 0.f);
    }
    return;
  }
  const int slot = slot_mapping ? slot_mapping[tok] : -1;
  if (slot < 0) return;
  const int page = slot / block_size, off = slot - page * block_size;
  if (kind == 1) {
    T* out = k_pages + (((size_t)page * kv_heads + head) * block_size + off) * D;
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int e = lane + 64 * r;
      if (e < D) out[e] = from_f32<T>(e < width ? x[r] : 0.f);
    }
  } else {
    T* out = v_pages + ((size_t)page * kv_heads + head) * D * block_size + off;
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int e = lane + 64 * r;
      if (e < D) out[(size_t)e * block_size] = from_f32<T>(e < width ? x[r] : 0.f);
    }
  }
}

// state[k] <- the projected row (with bias) of token q_len - (taps - 1) + k of this step, or what the state held for it.
__global__ __launch_bounds__(256) void conv_inputs_keep_kernel(
    const float* __restrict__ proj, int ld, const float* __restrict__ bias, float* state, size_t slot_stride,
    const int* __restrict__ state_slots, const int* __restrict__ seq_starts, const int* __restrict__ cu_seqlens, int channels, int taps) {
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  const int seq = blockIdx.y;
  if (c >= channels) return;
  const int q_begin = cu_seqlens[seq], q_len = cu_seqlens[seq + 1] - q_begin;
  if (q_len <= 0) return;
  const bool carried = seq_starts[seq] > 0;
  float* st = state + (size_t)state_slots[seq] * slot_stride;
  const float b = bias ? bias[c] : 0.f;
  float nv[kPrepMaxTaps];
#pragma unroll
  for (int k = 0; k < kPrepMaxTaps - 1; ++k) {
    nv[k] = 0.f;
    if (k < taps - 1) {
      const int rel = q_len - (taps - 1) + k;
      if (rel >= 0) nv[k] = proj[(size_t)(q_begin + rel) * ld + c] + b;
      else if (carried) nv[k] = st[(size_t)(q_len + k) * channels + c];
    }
  }
#pragma unroll
  for (int k = 0; k < kPrepMaxTaps - 1; ++k)
    if (k < taps - 1) st[(size_t)k * channels + c] = nv[k];
}

PLLM_API int pllm_attn_prepare(int dtype, const float* proj, int ld, const float* bias, const float* conv_w, int taps, float* state,
                               long slot_stride, const int* state_slots, const int* seq_starts, const int* cu_seqlens, int num_seqs,
                               const int* positions, const float* cos_table, const float* sin_table, int rot, int interleaved,
                               float eps, int qk_norm, int v_mode, int heads, int kv_heads, int d, int dv, int D, void* q_out, const int* slot_mapping,
                               void* k_pages, void* v_pages, int block_size, int num_tokens, hipStream_t stream) {
  if (num_tokens <= 0) return 0;
  if (d <= 0 || dv <= 0 || d > D || dv > D || D > kPrepMaxHead || rot < 0 || rot > d || (rot & 1) || taps > kPrepMaxTaps) return -2;
  if (v_mode < 0 || v_mode > 2 || (v_mode == 2 && dv != d)) return -2;
  if (rot > 0 && (!cos_table || !sin_table)) return -2;
  if (taps > 1 && (!conv_w || !state || !state_slots || !seq_starts || !cu_seqlens)) return -2;
  const bool write = slot_mapping && k_pages && v_pages;
  dim3 grid(num_tokens, heads + (write ? 2 * kv_heads : 0)), block(64);
#define PLLM_PREP(T)                                                                                                              \
  hipLaunchKernelGGL(attn_prepare_kernel<T>, grid, block, 0, stream, proj, ld, bias, conv_w, taps, state, (size_t)slot_stride,   \
                     state_slots, seq_starts, cu_seqlens, num_seqs, positions, cos_table, sin_table, rot, interleaved, eps, qk_norm, v_mode, heads, \
                     kv_heads, d, dv, D, (T*)q_out, slot_mapping, (T*)k_pages, (T*)v_pages, block_size)
  if (dtype == PLLM_F32) PLLM_PREP(float); else PLLM_PREP(bf16);
#undef PLLM_PREP
  if (taps > 1) {
    const int channels = (heads + kv_heads) * d + (v_mode == 2 ? 0 : kv_heads * dv);
    dim3 g2((channels + 255) / 256, num_seqs);
    hipLaunchKernelGGL(conv_inputs_keep_kernel, g2, dim3(256), 0, stream, proj, ld, bias, state, (size_t)slot_stride, state_slots,
                       seq_starts, cu_seqlens, channels, taps);
  }
  PLLM_RETURN_LAST_ERROR();
}

// ---------------------------------------------------------------------------------------------
// out[t, h * dv + e] = o[t, h * D + e] * sigmoid(gate[t * gate_ld + h])  for e < dv  (gate null: a plain repack).
template <typename T>
__global__ __launch_bounds__(256) void gate_heads_kernel(const T* __restrict__ o, int o_stride, const float* __restrict__ gate,
                                                         int gate_ld, T* __restrict__ out, int heads, int dv, int D) {
  const int t = blockIdx.x;
  for (int i = threadIdx.x; i < heads * dv; i += blockDim.x) {
    const int h = i / dv, e = i - h * dv;
    float v = to_f32(o[(size_t)t * o_stride + (size_t)h * D + e]);
    if (gate) v *= 1.f / (1.f + expf(-gate[(size_t)t * gate_ld + h]));
    out[(size_t)t * heads * dv + i] = from_f32<T>(v);
  }
}

PLLM_API int pllm_gate_heads(int dtype, const void* o, int o_stride, const float* gate, int gate_ld, void* out, int num_tokens,
                             int heads, int dv, int D, hipStream_t stream) {
  if (num_tokens <= 0) return 0;
  if (dv <= 0 || dv > D) return -2;
  dim3 grid(num_tokens), block(256);
  if (dtype == PLLM_F32)
    hipLaunchKernelGGL(gate_heads_kernel<float>, grid, block, 0, stream, (const float*)o, o_stride, gate, gate_ld, (float*)out, heads, dv, D);
  else
    hipLaunchKernelGGL(gate_heads_kernel<bf16>, grid, block, 0, stream, (const bf16*)o, o_stride, gate, gate_ld, (bf16*)out, heads, dv, D);
  PLLM_RETURN_LAST_ERROR();
}
