// Kernels for models whose residual stream is kept in float whatever the compute type: the embedding gather
// with a scale, a layer norm (weight and bias) of a branch's output that is added to the stream in the same
// kernel, and the conversion of stream rows to the compute type for the next product.  All arithmetic is
// float; T is only the storage type of the rows that go into or come out of matrix products.
#include "common.h"

using namespace pllm;

// ---------------------------------------------------------------------------------------------
// x[t, :] = float(table[ids[t], :]) * scale;  rows[t, :] = T(x[t, :]) when asked for.
template <typename T>
__global__ void embed_scaled_kernel(const int* __restrict__ ids, const T* __restrict__ table, float* __restrict__ x,
                                    T* __restrict__ rows, int hidden, int vocab, float scale) {
  const int t = blockIdx.x;
  int id = ids[t];
  id = id < 0 ? 0 : (id >= vocab ? vocab - 1 : id);  // the host has checked the range; never fault
  const T* src = table + (size_t)id * hidden;
  for (int i = threadIdx.x; i < hidden; i += blockDim.x) {
    const float v = to_f32(src[i]) * scale;
    x[(size_t)t * hidden + i] = v;
    if (rows) rows[(size_t)t * hidden + i] = from_f32<T>(v);
  }
}

PLLM_API int pllm_embed_scaled(int dtype, const int* ids, const void* table, float* x, void* rows, int num_tokens,
                               int hidden, int vocab, float scale, hipStream_t stream) {
  if (num_tokens <= 0) return 0;
  dim3 grid(num_tokens), block(256);
  if (dtype == PLLM_F32)
    hipLaunchKernelGGL(embed_scaled_kernel<float>, grid, block, 0, stream, ids, (const float*)table, x, (float*)rows, hidden, vocab, scale);
  else
    hipLaunchKernelGGL(embed_scaled_kernel<bf16>, grid, block, 0, stream, ids, (const bf16*)table, x, (bf16*)rows, hidden, vocab, scale);
  PLLM_RETURN_LAST_ERROR();
}

// ---------------------------------------------------------------------------------------------
// A token embedding with a hashed bigram row added:
//   x[t, :] = float(table[ids[t], :]) * scale + float(pairs[row(t), :]),
//   row(t) = (previous token * mul_prev + ids[t] * mul_cur) mod buckets, or `buckets` (the table's last row) for a
//   sequence's first token.
// The token before a step's first token of a sequence is what the sequence's slot of `last_token` holds (a sequence
// whose seq_starts is 0 has none); every sequence leaves its last token of this step there.  bigram_rows_kernel: one
// workgroup per sequence, which reads the slot before any of its threads writes it.
__global__ __launch_bounds__(256) void bigram_rows_kernel(const int* __restrict__ ids, const int* __restrict__ cu_seqlens,
                                                          const int* __restrict__ seq_starts, const int* __restrict__ state_slots,
                                                          int* last_token, long slot_stride, int* __restrict__ rows, int vocab,
                                                          int buckets, int mul_prev, int mul_cur) {
  const int seq = blockIdx.x;
  const int begin = cu_seqlens[seq], len = cu_seqlens[seq + 1] - begin;
  if (len <= 0) return;
  int* slot = last_token + (size_t)state_slots[seq] * slot_stride;
  const int carried = seq_starts[seq] > 0 ? *slot : -1;
  __syncthreads();
  for (int i = threadIdx.x; i < len; i += blockDim.x) {
    const int cur = ids[begin + i];
    const int prev = i > 0 ? ids[begin + i - 1] : carried;
    int row = buckets;
    if (prev >= 0) row = (int)(((long long)prev * mul_prev + (long long)cur * mul_cur) % buckets);
    rows[begin + i] = row < 0 ? row + buckets : row;
    if (i == len - 1) *slot = cur;
  }
}

template <typename T>
__global__ void embed_bigram_kernel(const int* __restrict__ ids, const int* __restrict__ pair_rows, const T* __restrict__ table,
                                    const T* __restrict__ pairs, float* __restrict__ x, int hidden, int vocab, int buckets, float scale) {
  const int t = blockIdx.x;
  int id = ids[t], pr = pair_rows[t];
  id = id < 0 ? 0 : (id >= vocab ? vocab - 1 : id);  // the host has checked the range; never fault
  pr = pr < 0 ? 0 : (pr > buckets ? buckets : pr);
  const T* src = table + (size_t)id * hidden;
  const T* add = pairs + (size_t)pr * hidden;
  for (int i = threadIdx.x; i < hidden; i += blockDim.x) x[(size_t)t * hidden + i] = to_f32(src[i]) * scale + to_f32(add[i]);
}

PLLM_API int pllm_embed_bigram(int dtype, const int* ids, const int* cu_seqlens, const int* seq_starts, const int* state_slots,
                               int* last_token, long slot_stride, int* pair_rows, const void* table, const void* pairs, float* x,
                               int num_tokens, int num_seqs, int hidden, int vocab, int buckets, int mul_prev, int mul_cur, float scale,
                               int move_state, hipStream_t stream) {
  if (num_tokens <= 0 || num_seqs <= 0) return 0;
  if (buckets <= 0 || hidden <= 0) return -2;
  if (move_state)
    hipLaunchKernelGGL(bigram_rows_kernel, dim3(num_seqs), dim3(256), 0, stream, ids, cu_seqlens, seq_starts, state_slots, last_token,
                       slot_stride, pair_rows, vocab, buckets, mul_prev, mul_cur);
  dim3 grid(num_tokens), block(256);
  if (dtype == PLLM_F32)
    hipLaunchKernelGGL(embed_bigram_kernel<float>, grid, block, 0, stream, ids, pair_rows, (const float*)table, (const float*)pairs, x,
                       hidden, vocab, buckets, scale);
  else
    hipLaunchKernelGGL(embed_bigram_kernel<bf16>, grid, block, 0, stream, ids, pair_rows, (const bf16*)table, (const bf16*)pairs, x,
                       hidden, vocab, buckets, scale);
  PLLM_RETURN_LAST_ERROR();
}

// ---------------------------------------------------------------------------------------------
// Layer norm of one row per workgroup:  y = (v - mean) / sqrt(var + eps) * w + b,  var = mean((v - mean)^2),
// with v = in[src] (src = row_index[r] or r).  Then
//   stream given:  stream[r] += y (float), and rows[r] = T(stream[r]) when rows is given;
//   no stream:     rows[r] = T(y).
// TI is the type of `in` (float, or the compute type), TO the type of `rows`.
template <typename TI, typename TO>
__global__ void layernorm_kernel(const TI* __restrict__ in, const int* __restrict__ row_index, const float* __restrict__ w,
                                 const float* __restrict__ b, float eps, float* stream_rows, TO* __restrict__ rows, int hidden) {
  extern __shared__ float lds[];
  float* row = lds;               // [hidden]
  float* scratch = lds + hidden;  // [16]
  const int r = blockIdx.x;
  const size_t src = row_index ? (size_t)row_index[r] : (size_t)r;
  const TI* v = in + src * hidden;
  float acc = 0.f;
  for (int i = threadIdx.x; i < hidden; i += blockDim.x) {
    const float f = to_f32(v[i]);
    row[i] = f;
    acc += f;
  }
  const float mean = block_sum(acc, scratch) / (float)hidden;
  float sq = 0.f;
  for (int i = threadIdx.x; i < hidden; i += blockDim.x) {
    const float d = row[i] - mean;
    sq = fmaf(d, d, sq);
  }
  const float var = block_sum(sq, scratch) / (float)hidden;
  const float inv = 1.f / sqrtf(var + eps);
  for (int i = threadIdx.x; i < hidden; i += blockDim.x) {
    float y = (row[i] - mean) * inv * w[i] + b[i];
    if (stream_rows) {
      y += stream_rows[(size_t)r * hidden + i];
      stream_rows[(size_t)r * hidden + i] = y;
    }
    if (rows) rows[(size_t)r * hidden + i] = from_f32<TO>(y);
  }
}

// The same with the row in registers, four elements per thread and load (hidden a multiple of 4 up to kRowRegs * 1024,
// rows on 16-byte boundaries in float and 8-byte ones in bfloat16): every value is read once.
constexpr int kRowRegs = 4;

template <typename T> struct alignas(4 * sizeof(T)) Quad { T v[4]; };

template <typename TI, typename TO>
__global__ __launch_bounds__(256) void layernorm_regs_kernel(const TI* __restrict__ in, const int* __restrict__ row_index,
                                                             const float* __restrict__ w, const float* __restrict__ b, float eps,
                                                             float* stream_rows, TO* __restrict__ rows, int hidden) {
  __shared__ float scratch[16];
  const int r = blockIdx.x;
  const size_t src = row_index ? (size_t)row_index[r] : (size_t)r;
  const TI* v = in + src * hidden;
  float x[kRowRegs][4], add[kRowRegs][4];
  float acc = 0.f;
#pragma unroll
  for (int j = 0; j < kRowRegs; ++j) {
    const int at = (j * 256 + threadIdx.x) * 4;
    if (at < hidden) {
      const Quad<TI> q = *reinterpret_cast<const Quad<TI>*>(v + at);
#pragma unroll
      for (int e = 0; e < 4; ++e) { x[j][e] = to_f32(q.v[e]); acc += x[j][e]; }
      if (stream_rows) {                                   // asked for early: it arrives while the sums are made
        const float4 sv = *reinterpret_cast<const float4*>(stream_rows + (size_t)r * hidden + at);
        add[j][0] = sv.x; add[j][1] = sv.y; add[j][2] = sv.z; add[j][3] = sv.w;
      }
    }
  }
  const float mean = block_sum(acc, scratch) / (float)hidden;
  float sq = 0.f;
#pragma unroll
  for (int j = 0; j < kRowRegs; ++j) {
    const int at = (j * 256 + threadIdx.x) * 4;
    if (at < hidden) {
#pragma unroll
      for (int e = 0; e < 4; ++e) { const float d = x[j][e] - mean; sq = fmaf(d, d, sq); }
    }
  }
  const float var = block_sum(sq, scratch) / (float)hidden;
  const float inv = 1.f / sqrtf(var + eps);
#pragma unroll
  for (int j = 0; j < kRowRegs; ++j) {
    const int at = (j * 256 + threadIdx.x) * 4;
    if (at < hidden) {
      const float4 wv = *reinterpret_cast<const float4*>(w + at), bv = *reinterpret_cast<const float4*>(b + at);
      const float ww[4] = {wv.x, wv.y, wv.z, wv.w}, bb[4] = {bv.x, bv.y, bv.z, bv.w};
      float y[4];
      Quad<TO> o;
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        y[e] = (x[j][e] - mean) * inv * ww[e] + bb[e];
        if (stream_rows) y[e] += add[j][e];
        o.v[e] = from_f32<TO>(y[e]);
      }
      if (stream_rows) *reinterpret_cast<float4*>(stream_rows + (size_t)r * hidden + at) = make_float4(y[0], y[1], y[2], y[3]);
      if (rows) *reinterpret_cast<Quad<TO>*>(rows + (size_t)r * hidden + at) = o;
    }
  }
}

// in_dtype / out_dtype: PLLM_F32 or PLLM_BF16.
PLLM_API int pllm_layernorm(int in_dtype, int out_dtype, const void* in, const int* row_index, const float* w, const float* b,
                            float eps, float* stream_rows, void* rows, int num_rows, int hidden, hipStream_t stream) {
  if (num_rows <= 0) return 0;
  if (hidden <= 0) return -2;
  dim3 grid(num_rows), block(256);
  const size_t lds = (size_t)(hidden + 16) * sizeof(float);
  const bool in_regs = hidden % 4 == 0 && hidden <= kRowRegs * 1024 && (uintptr_t)in % 16 == 0 && (uintptr_t)w % 16 == 0 &&
                       (uintptr_t)b % 16 == 0 && (uintptr_t)stream_rows % 16 == 0 && (uintptr_t)rows % 16 == 0;
#define PLLM_LN(TI, TO)                                                                                                          \
  do {                                                                                                                          \
    if (in_regs) {                                                                                                              \
      hipLaunchKernelGGL((layernorm_regs_kernel<TI, TO>), grid, block, 0, stream, (const TI*)in, row_index, w, b, eps,          \
                         stream_rows, (TO*)rows, hidden);                                                                       \
      break;                                                                                                                    \
    }                                                                                                                           \
    if (lds > 48 * 1024) {                                                                                                      \
      hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(layernorm_kernel<TI, TO>),                               \
                                         hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);                                \
      if (e != hipSuccess) return (int)e;                                                                                       \
    }                                                                                                                           \
    hipLaunchKernelGGL((layernorm_kernel<TI, TO>), grid, block, lds, stream, (const TI*)in, row_index, w, b, eps, stream_rows, \
                       (TO*)rows, hidden);                                                                                      \
  } while (0)
  if (in_dtype == PLLM_F32 && out_dtype == PLLM_F32) PLLM_LN(float, float);
  else if (in_dtype == PLLM_F32 && out_dtype == PLLM_BF16) PLLM_LN(float, bf16);
  else if (in_dtype == PLLM_BF16 && out_dtype == PLLM_BF16) PLLM_LN(bf16, bf16);
  else if (in_dtype == PLLM_BF16 && out_dtype == PLLM_F32) PLLM_LN(bf16, float);
  else return -3;
#undef PLLM_LN
  PLLM_RETURN_LAST_ERROR();
}

// ---------------------------------------------------------------------------------------------
// rows = bf16(x), element by element.
__global__ void round_rows_kernel(const float* __restrict__ x, bf16* __restrict__ rows, size_t n) {
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x)
    rows[i] = __float2bfloat16(x[i]);
}

PLLM_API int pllm_round_rows(const float* x, void* rows, long n, hipStream_t stream) {
  if (n <= 0) return 0;
  const int blocks = (int)((n + 255) / 256 < 4096 ? (n + 255) / 256 : 4096);
  hipLaunchKernelGGL(round_rows_kernel, dim3(blocks), dim3(256), 0, stream, x, (bf16*)rows, (size_t)n);
  PLLM_RETURN_LAST_ERROR();
}

// ---------------------------------------------------------------------------------------------
// RMS norms on both sides of a branch over a float stream, one row per workgroup:
//   branch given:  y = branch[r] (+ bias);  stream[r] += mult * y / sqrt(mean(y^2) + eps) * w_branch      (in place)
//                  (w_branch null: the branch is not normed, stream[r] += mult * y: a pre-norm block's sum)
//   then, rows given:  rows[r] = T(s / sqrt(mean(s^2) + eps) * w_next)  with s the row of the stream as it is now
//                      (w_next null: rows[r] = T(s), the stream in the compute type).
// Without a branch the stream's row is src = row_index[r] (or r) and nothing is written to the stream.  The weights
// are the factors themselves (an architecture that stores them around zero adds the one when it loads them).
// `rows` has a row stride of its own, so that it may be a part of wider rows.
// A branch that is the weighted sum of two (two mixers side by side): branch[r][i] = first_scale * branch[r][i] +
// second_scale * second[r][i], formed where the branch is read.  second null: the branch as it is.
struct BranchPair {
  const float* second; float first_scale, second_scale;
};

template <typename TO>
__global__ __launch_bounds__(256) void rms_sandwich_kernel(const float* __restrict__ branch, const BranchPair pair, const float* __restrict__ bias,
                                                           const float* __restrict__ w_branch, float mult, float* stream,
                                                           const int* __restrict__ row_index, const float* __restrict__ w_next, float eps,
                                                           TO* __restrict__ rows, long rows_stride, int hidden) {
  extern __shared__ float lds[];
  float* row = lds;               // [hidden]
  float* scratch = lds + hidden;  // [16]
  const int r = blockIdx.x;
  const size_t src = (!branch && row_index) ? (size_t)row_index[r] : (size_t)r;
  float* s = stream + src * hidden;
  float sq = 0.f;
  if (branch) {
    const float* v = branch + (size_t)r * hidden;
    const float* v2 = pair.second ? pair.second + (size_t)r * hidden : nullptr;
    float bsq = 0.f;
    for (int i = threadIdx.x; i < hidden; i += blockDim.x) {
      const float f = (v2 ? pair.first_scale * v[i] + pair.second_scale * v2[i] : v[i]) + (bias ? bias[i] : 0.f);
      row[i] = f;
      bsq = fmaf(f, f, bsq);
    }
    const float inv = w_branch ? 1.f / sqrtf(block_sum(bsq, scratch) / (float)hidden + eps) : 1.f;
    for (int i = threadIdx.x; i < hidden; i += blockDim.x) {
      const float y = s[i] + mult * (w_branch ? row[i] * inv * w_branch[i] : row[i]);
      s[i] = y;
      row[i] = y;
      sq = fmaf(y, y, sq);
    }
  } else {
    for (int i = threadIdx.x; i < hidden; i += blockDim.x) {
      const float y = s[i];
      row[i] = y;
      sq = fmaf(y, y, sq);
    }
  }
  if (!rows) return;
  TO* out = rows + (size_t)r * rows_stride;
  if (w_next) {
    const float inv = 1.f / sqrtf(block_sum(sq, scratch) / (float)hidden + eps);
    for (int i = threadIdx.x; i < hidden; i += blockDim.x) out[i] = from_f32<TO>(row[i] * inv * w_next[i]);
  } else {
    for (int i = threadIdx.x; i < hidden; i += blockDim.x) out[i] = from_f32<TO>(row[i]);
  }
}

// The same with a branch, for rows of up to 4,096 elements that 256 threads hold in registers (16 each): everything a
// row needs (branch and bias, the stream's row, both weights) is asked for before the first sum, so the kernel waits
// for memory once where the one above waits three times (decode steps: the weights have left the caches since the last
// layer).  Elements, partial sums and their order are the ones of the kernel above.  The branch may still be a sum of
// experts' rows (`sum.expert_out` set): branch[r][i] = sum over k < top, in order, of weights[r, k] * (row_of_pair[r, k]
// >= 0 ? expert_out[row_of_pair[r, k]][i] : h[r][i]), formed here instead of by a kernel of its own.
struct ChoiceSum {
  const float* expert_out; const void* h; long ld_h; const int* row_of_pair; const float* weights; int top;
};
constexpr int kHeldPerThread = 16, kHeldThreads = 256;

template <typename TO, typename TH>
__global__ __launch_bounds__(kHeldThreads) void rms_sandwich_held_kernel(const float* __restrict__ branch, const BranchPair pair, const ChoiceSum sum,
                                                                         const float* __restrict__ bias, const float* __restrict__ w_branch,
                                                                         float mult, float* stream, const float* __restrict__ w_next, float eps,
                                                                         TO* __restrict__ rows, long rows_stride, int hidden) {
  __shared__ float scratch[16];
  const int r = blockIdx.x, tid = threadIdx.x;
  float* s = stream + (size_t)r * hidden;
  float f[kHeldPerThread], sv[kHeldPerThread], wb[kHeldPerThread], wn[kHeldPerThread];
#pragma unroll
  for (int j = 0; j < kHeldPerThread; ++j) {
    const int i = tid + kHeldThreads * j;
    const bool in = i < hidden;
    sv[j] = in ? s[i] : 0.f;
    wb[j] = (in && w_branch) ? w_branch[i] : 1.f;
    wn[j] = (in && w_next) ? w_next[i] : 1.f;
    f[j] = (in && !sum.expert_out) ? branch[(size_t)r * hidden + i] : 0.f;
    if (in && pair.second) f[j] = pair.first_scale * f[j] + pair.second_scale * pair.second[(size_t)r * hidden + i];
  }
  if (sum.expert_out) {
    const TH* own = reinterpret_cast<const TH*>(sum.h) + (size_t)r * sum.ld_h;
    for (int k = 0; k < sum.top; ++k) {
      const int row = sum.row_of_pair[(size_t)r * sum.top + k];
      const float wk = sum.weights[(size_t)r * sum.top + k];
      const float* e = sum.expert_out + (size_t)(row >= 0 ? row : 0) * hidden;
#pragma unroll
      for (int j = 0; j < kHeldPerThread; ++j) {
        const int i = tid + kHeldThreads * j;
        if (i < hidden) f[j] = fmaf(wk, row >= 0 ? e[i] : to_f32(own[i]), f[j]);
      }
    }
  }
  float bsq = 0.f;
#pragma unroll
  for (int j = 0; j < kHeldPerThread; ++j) {
    const int i = tid + kHeldThreads * j;
    if (i < hidden) {
      if (bias) f[j] += bias[i];
      bsq = fmaf(f[j], f[j], bsq);
    }
  }
  const float inv = w_branch ? 1.f / sqrtf(block_sum(bsq, scratch) / (float)hidden + eps) : 1.f;
  float sq = 0.f;
#pragma unroll
  for (int j = 0; j < kHeldPerThread; ++j) {
    const int i = tid + kHeldThreads * j;
    if (i < hidden) {
      const float y = sv[j] + mult * (w_branch ? f[j] * inv * wb[j] : f[j]);
      s[i] = y;
      sv[j] = y;
      sq = fmaf(y, y, sq);
    }
  }
  if (!rows) return;
  TO* out = rows + (size_t)r * rows_stride;
  const float inv_next = w_next ? 1.f / sqrtf(block_sum(sq, scratch) / (float)hidden + eps) : 1.f;
#pragma unroll
  for (int j = 0; j < kHeldPerThread; ++j) {
    const int i = tid + kHeldThreads * j;
    if (i < hidden) out[i] = from_f32<TO>(w_next ? sv[j] * inv_next * wn[j] : sv[j]);
  }
}

template <typename TO>
static void launch_sandwich_held(int h_dtype, const float* branch, const BranchPair& pair, const ChoiceSum& sum, const float* bias, const float* w_branch, float mult,
                                 float* stream, const float* w_next, float eps, void* rows, long rows_stride, int num_rows, int hidden,
                                 hipStream_t stream_) {
  if (h_dtype == PLLM_F32)
    hipLaunchKernelGGL((rms_sandwich_held_kernel<TO, float>), dim3(num_rows), dim3(kHeldThreads), 0, stream_, branch, pair, sum, bias, w_branch, mult,
                       stream, w_next, eps, (TO*)rows, rows_stride, hidden);
  else
    hipLaunchKernelGGL((rms_sandwich_held_kernel<TO, bf16>), dim3(num_rows), dim3(kHeldThreads), 0, stream_, branch, pair, sum, bias, w_branch, mult,
                       stream, w_next, eps, (TO*)rows, rows_stride, hidden);
}

// A branch that is a sum of experts' rows (see above); rows of up to 4,096 elements.
PLLM_API int pllm_rms_sandwich_sum(int out_dtype, int h_dtype, const float* expert_out, const void* h, long ld_h, const int* row_of_pair,
                                   const float* weights, int top, const float* bias, const float* w_branch, float mult, float* stream,
                                   const float* w_next, float eps, void* rows, long rows_stride, int num_rows, int hidden, hipStream_t stream_) {
  if (num_rows <= 0) return 0;
  if (hidden <= 0 || hidden > kHeldPerThread * kHeldThreads || !stream || !w_branch || !expert_out || !h || !row_of_pair || !weights || top <= 0) return -2;
  const ChoiceSum sum{expert_out, h, ld_h, row_of_pair, weights, top};
  if (out_dtype == PLLM_F32) launch_sandwich_held<float>(h_dtype, nullptr, BranchPair{nullptr, 1.f, 1.f}, sum, bias, w_branch, mult, stream, w_next, eps, rows, rows_stride, num_rows, hidden, stream_);
  else launch_sandwich_held<bf16>(h_dtype, nullptr, BranchPair{nullptr, 1.f, 1.f}, sum, bias, w_branch, mult, stream, w_next, eps, rows, rows_stride, num_rows, hidden, stream_);
  PLLM_RETURN_LAST_ERROR();
}

static int rms_sandwich_launch(int out_dtype, const float* branch, const BranchPair pair, const float* bias, const float* w_branch, float mult,
                               float* stream, const int* row_index, const float* w_next, float eps, void* rows, long rows_stride,
                               int num_rows, int hidden, hipStream_t stream_) {
  if (num_rows <= 0) return 0;
  if (hidden <= 0 || !stream) return -2;
  if (branch && hidden <= kHeldPerThread * kHeldThreads) {
    const ChoiceSum none{nullptr, nullptr, 0, nullptr, nullptr, 0};
    if (out_dtype == PLLM_F32) launch_sandwich_held<float>(PLLM_F32, branch, pair, none, bias, w_branch, mult, stream, w_next, eps, rows, rows_stride, num_rows, hidden, stream_);
    else launch_sandwich_held<bf16>(PLLM_F32, branch, pair, none, bias, w_branch, mult, stream, w_next, eps, rows, rows_stride, num_rows, hidden, stream_);
    PLLM_RETURN_LAST_ERROR();
  }
  const size_t lds = (size_t)(hidden + 16) * sizeof(float);
  dim3 grid(num_rows), block(256);
#define PLLM_SW(TO)                                                                                                        \
  do {                                                                                                                    \
    if (lds > 48 * 1024) {                                                                                                \
      hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(rms_sandwich_kernel<TO>),                          \
                                         hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);                          \
      if (e != hipSuccess) return (int)e;                                                                                 \
    }                                                                                                                     \
    hipLaunchKernelGGL(rms_sandwich_kernel<TO>, grid, block, lds, stream_, branch, pair, bias, w_branch, mult, stream, row_index, \
                       w_next, eps, (TO*)rows, rows_stride, hidden);                                                      \
  } while (0)
  if (out_dtype == PLLM_F32) PLLM_SW(float); else PLLM_SW(bf16);
#undef PLLM_SW
  PLLM_RETURN_LAST_ERROR();
}

PLLM_API int pllm_rms_sandwich(int out_dtype, const float* branch, const float* bias, const float* w_branch, float mult, float* stream,
                               const int* row_index, const float* w_next, float eps, void* rows, long rows_stride, int num_rows,
                               int hidden, hipStream_t stream_) {
  return rms_sandwich_launch(out_dtype, branch, BranchPair{nullptr, 1.f, 1.f}, bias, w_branch, mult, stream, row_index, w_next, eps, rows,
                             rows_stride, num_rows, hidden, stream_);
}

// The same with a branch that is first_scale * branch + second_scale * second (both float rows like the stream).
PLLM_API int pllm_rms_sandwich_pair(int out_dtype, const float* branch, float first_scale, const float* second, float second_scale,
                                    const float* bias, const float* w_branch, float mult, float* stream, const float* w_next, float eps,
                                    void* rows, long rows_stride, int num_rows, int hidden, hipStream_t stream_) {
  if (!branch || !second) return -2;
  return rms_sandwich_launch(out_dtype, branch, BranchPair{second, first_scale, second_scale}, bias, w_branch, mult, stream, nullptr, w_next,
                             eps, rows, rows_stride, num_rows, hidden, stream_);
}

// ---------------------------------------------------------------------------------------------
// out[t, at : at + hidden] = T(x[t, :]): float rows into a part of wider rows of the compute type.
template <typename TO>
__global__ void place_rows_kernel(const float* __restrict__ x, TO* __restrict__ out, long out_stride, int hidden) {
  const int t = blockIdx.x;
  for (int i = threadIdx.x; i < hidden; i += blockDim.x) out[(size_t)t * out_stride + i] = from_f32<TO>(x[(size_t)t * hidden + i]);
}

PLLM_API int pllm_place_rows(int out_dtype, const float* x, void* out, long out_stride, int num_rows, int hidden, hipStream_t stream) {
  if (num_rows <= 0) return 0;
  dim3 grid(num_rows), block(256);
  if (out_dtype == PLLM_F32) hipLaunchKernelGGL(place_rows_kernel<float>, grid, block, 0, stream, x, (float*)out, out_stride, hidden);
  else hipLaunchKernelGGL(place_rows_kernel<bf16>, grid, block, 0, stream, x, (bf16*)out, out_stride, hidden);
  PLLM_RETURN_LAST_ERROR();
}

// ---------------------------------------------------------------------------------------------
// Dynamic tanh, a norm that computes no statistics, y = tanh(alpha x) * w + b element by element, around a float stream:
//   branch given:  stream[r] += branch[r] in place (no row_index then);
//   rows given:    rows[r] = T(tanh(alpha * stream[src]) * w + b), src = row_index[r] or r, with the stream as it is
//                  after the sum.
// One workgroup per row; four elements per thread and load where `vec` says the rows allow it (hidden a multiple of 4,
// rows on 16-byte boundaries in float and 8-byte ones in T).
template <typename TO>
__global__ __launch_bounds__(256) void dyt_kernel(const float* __restrict__ branch, float* stream, const int* __restrict__ row_index,
                                                  float alpha, const float* __restrict__ w, const float* __restrict__ b,
                                                  TO* __restrict__ rows, long rows_stride, int hidden, int vec) {
  const int r = blockIdx.x;
  const size_t src = row_index ? (size_t)row_index[r] : (size_t)r;
  float* x = stream + src * hidden;
  const float* d = branch ? branch + (size_t)r * hidden : nullptr;
  TO* out = rows ? rows + (size_t)r * rows_stride : nullptr;
  if (vec) {
    for (int i = 4 * threadIdx.x; i < hidden; i += 4 * blockDim.x) {
      float4 v = *reinterpret_cast<const float4*>(x + i);
      if (d) {
        const float4 e = *reinterpret_cast<const float4*>(d + i);
        v.x += e.x; v.y += e.y; v.z += e.z; v.w += e.w;
        *reinterpret_cast<float4*>(x + i) = v;
      }
      if (out) {
        const float4 ww = *reinterpret_cast<const float4*>(w + i), bb = *reinterpret_cast<const float4*>(b + i);
        Quad<TO> o;
        o.v[0] = from_f32<TO>(fmaf(tanhf(alpha * v.x), ww.x, bb.x));
        o.v[1] = from_f32<TO>(fmaf(tanhf(alpha * v.y), ww.y, bb.y));
        o.v[2] = from_f32<TO>(fmaf(tanhf(alpha * v.z), ww.z, bb.z));
        o.v[3] = from_f32<TO>(fmaf(tanhf(alpha * v.w), ww.w, bb.w));
        *reinterpret_cast<Quad<TO>*>(out + i) = o;
      }
    }
    return;
  }
  for (int i = threadIdx.x; i < hidden; i += blockDim.x) {
    float v = x[i];
    if (d) {
      v += d[i];
      x[i] = v;
    }
    if (out) out[i] = from_f32<TO>(fmaf(tanhf(alpha * v), w[i], b[i]));
  }
}

PLLM_API int pllm_dyt(int out_dtype, const float* branch, float* stream, const int* row_index, float alpha, const float* w,
                      const float* b, void* rows, long rows_stride, int num_rows, int hidden, hipStream_t stream_) {
  if (num_rows <= 0) return 0;
  if (branch && row_index) return -2;
  if (rows && (!w || !b)) return -2;
  const size_t out_bytes = out_dtype == PLLM_F32 ? 4 : 2;
  const int vec = hidden % 4 == 0 && ((uintptr_t)stream & 15) == 0 && (!branch || ((uintptr_t)branch & 15) == 0) &&
                  (!rows || (((uintptr_t)rows % (4 * out_bytes)) == 0 && rows_stride % 4 == 0 && ((uintptr_t)w & 15) == 0 && ((uintptr_t)b & 15) == 0));
  dim3 grid(num_rows), block(hidden >= 1024 ? 256 : (hidden >= 256 ? 64 * ((hidden / 4 + 63) / 64) : 64));
  if (out_dtype == PLLM_F32)
    hipLaunchKernelGGL(dyt_kernel<float>, grid, block, 0, stream_, branch, stream, row_index, alpha, w, b, (float*)rows, rows_stride, hidden, vec);
  else
    hipLaunchKernelGGL(dyt_kernel<bf16>, grid, block, 0, stream_, branch, stream, row_index, alpha, w, b, (bf16*)rows, rows_stride, hidden, vec);
  PLLM_RETURN_LAST_ERROR();
}

// The same behind routed experts, whose weighted sum this kernel forms where it would have read the branch:
//   branch[r] = sum_k (weights_inside && row >= 0 ? 1 : weights[r, k]) * (row >= 0 ? expert_out[row] : h[r]),  row = row_of_pair[r, k],
//               in the order of k, + shared[r] * (shared_gate ? sigmoid(shared_gate[r * gate_ld]) : 1) when shared is given;
//   stream[r] += branch[r];   rows[r] = T(tanh(alpha * stream[r]) * w + b) when rows is given.
template <typename TO, typename TH>
__global__ __launch_bounds__(256) void dyt_sum_kernel(const float* __restrict__ expert_out, const TH* __restrict__ h, long ld_h,
                                                      const int* __restrict__ row_of_pair, const float* __restrict__ weights, int top,
                                                      int weights_inside, const float* __restrict__ shared,
                                                      const float* __restrict__ shared_gate, int gate_ld, float* stream, float alpha,
                                                      const float* __restrict__ w, const float* __restrict__ b, TO* __restrict__ rows,
                                                      long rows_stride, int hidden) {
  const int r = blockIdx.x;
  float* x = stream + (size_t)r * hidden;
  TO* out = rows ? rows + (size_t)r * rows_stride : nullptr;
  const float sg = shared ? (shared_gate ? 1.f / (1.f + expf(-shared_gate[(size_t)r * gate_ld])) : 1.f) : 0.f;
  for (int i = threadIdx.x; i < hidden; i += blockDim.x) {
    float acc = 0.f;
    for (int k = 0; k < top; ++k) {
      const int row = row_of_pair[(size_t)r * top + k];
      const float v = row >= 0 ? expert_out[(size_t)row * hidden + i] : to_f32(h[(size_t)r * ld_h + i]);
      if (weights_inside && row >= 0) acc += v;
      else acc = fmaf(weights[(size_t)r * top + k], v, acc);
    }
    if (shared) acc = fmaf(sg, shared[(size_t)r * hidden + i], acc);
    const float v = x[i] + acc;
    x[i] = v;
    if (out) out[i] = from_f32<TO>(fmaf(tanhf(alpha * v), w[i], b[i]));
  }
}

// The same with four elements per thread and load, the choices' rows and weights read once per workgroup into LDS and
// the rows of four choices asked for before the first of them is added (hidden a multiple of 4, at most kSumTop choices,
// rows on 16-byte boundaries): the loads of a step no longer wait for one another.
constexpr int kSumTop = 64, kSumAhead = 4;

template <typename TO, typename TH>
__global__ __launch_bounds__(256) void dyt_sum_vec_kernel(const float* __restrict__ expert_out, const TH* __restrict__ h, long ld_h,
                                                          const int* __restrict__ row_of_pair, const float* __restrict__ weights, int top,
                                                          int weights_inside, const float* __restrict__ shared,
                                                          const float* __restrict__ shared_gate, int gate_ld, float* stream, float alpha,
                                                          const float* __restrict__ w, const float* __restrict__ b, TO* __restrict__ rows,
                                                          long rows_stride, int hidden) {
  __shared__ int row_s[kSumTop];
  __shared__ float weight_s[kSumTop];
  const int r = blockIdx.x;
  if ((int)threadIdx.x < top) {
    const int row = row_of_pair[(size_t)r * top + threadIdx.x];
    row_s[threadIdx.x] = row;
    weight_s[threadIdx.x] = (weights_inside && row >= 0) ? 1.f : weights[(size_t)r * top + threadIdx.x];
  }
  float* x = stream + (size_t)r * hidden;
  TO* out = rows ? rows + (size_t)r * rows_stride : nullptr;
  const float sg = shared ? (shared_gate ? 1.f / (1.f + expf(-shared_gate[(size_t)r * gate_ld])) : 1.f) : 0.f;
  __syncthreads();
  for (int i = 4 * threadIdx.x; i < hidden; i += 4 * blockDim.x) {
    const float4 x4 = *reinterpret_cast<const float4*>(x + i);
    float4 s4 = make_float4(0.f, 0.f, 0.f, 0.f);
    if (shared) s4 = *reinterpret_cast<const float4*>(shared + (size_t)r * hidden + i);
    float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
    for (int k0 = 0; k0 < top; k0 += kSumAhead) {
      float4 v[kSumAhead];
#pragma unroll
      for (int j = 0; j < kSumAhead; ++j) {
        const int k = k0 + j < top ? k0 + j : top - 1;
        const int row = row_s[k];
        if (row >= 0) v[j] = *reinterpret_cast<const float4*>(expert_out + (size_t)row * hidden + i);
        else v[j] = make_float4(to_f32(h[(size_t)r * ld_h + i]), to_f32(h[(size_t)r * ld_h + i + 1]), to_f32(h[(size_t)r * ld_h + i + 2]),
                                to_f32(h[(size_t)r * ld_h + i + 3]));
      }
#pragma unroll
      for (int j = 0; j < kSumAhead; ++j)
        if (k0 + j < top) {
          const float wt = weight_s[k0 + j];
          if (weights_inside && row_s[k0 + j] >= 0) { acc.x += v[j].x; acc.y += v[j].y; acc.z += v[j].z; acc.w += v[j].w; }
          else { acc.x = fmaf(wt, v[j].x, acc.x); acc.y = fmaf(wt, v[j].y, acc.y); acc.z = fmaf(wt, v[j].z, acc.z); acc.w = fmaf(wt, v[j].w, acc.w); }
        }
    }
    if (shared) { acc.x = fmaf(sg, s4.x, acc.x); acc.y = fmaf(sg, s4.y, acc.y); acc.z = fmaf(sg, s4.z, acc.z); acc.w = fmaf(sg, s4.w, acc.w); }
    const float4 v = make_float4(x4.x + acc.x, x4.y + acc.y, x4.z + acc.z, x4.w + acc.w);
    *reinterpret_cast<float4*>(x + i) = v;
    if (out) {
      const float4 ww = *reinterpret_cast<const float4*>(w + i), bb = *reinterpret_cast<const float4*>(b + i);
      Quad<TO> o;
      o.v[0] = from_f32<TO>(fmaf(tanhf(alpha * v.x), ww.x, bb.x));
      o.v[1] = from_f32<TO>(fmaf(tanhf(alpha * v.y), ww.y, bb.y));
      o.v[2] = from_f32<TO>(fmaf(tanhf(alpha * v.z), ww.z, bb.z));
      o.v[3] = from_f32<TO>(fmaf(tanhf(alpha * v.w), ww.w, bb.w));
      *reinterpret_cast<Quad<TO>*>(out + i) = o;
    }
  }
}

PLLM_API int pllm_dyt_sum(int out_dtype, int h_dtype, const float* expert_out, const void* h, long ld_h, const int* row_of_pair,
                          const float* weights, int top, int weights_inside, const float* shared, const float* shared_gate, int gate_ld,
                          float* stream, float alpha, const float* w, const float* b, void* rows, long rows_stride, int num_rows,
                          int hidden, hipStream_t stream_) {
  if (num_rows <= 0) return 0;
  if (top <= 0 || (rows && (!w || !b))) return -2;
  const size_t out_bytes = out_dtype == PLLM_F32 ? 4 : 2;
  const bool vec = hidden % 4 == 0 && top <= kSumTop && ((uintptr_t)stream & 15) == 0 && ((uintptr_t)expert_out & 15) == 0 &&
                   (!shared || ((uintptr_t)shared & 15) == 0) &&
                   (!rows || (((uintptr_t)rows % (4 * out_bytes)) == 0 && rows_stride % 4 == 0 && ((uintptr_t)w & 15) == 0 && ((uintptr_t)b & 15) == 0));
  if (vec) {
    const int threads = hidden >= 1024 ? 256 : (hidden / 4 + 63) / 64 * 64;
    dim3 vgrid(num_rows), vblock(threads < 64 ? 64 : threads);
#define PLLM_DSV(TO, TH)                                                                                                              \
  hipLaunchKernelGGL((dyt_sum_vec_kernel<TO, TH>), vgrid, vblock, 0, stream_, expert_out, (const TH*)h, ld_h, row_of_pair, weights, top, \
                     weights_inside, shared, shared_gate, gate_ld, stream, alpha, w, b, (TO*)rows, rows_stride, hidden)
    if (out_dtype == PLLM_F32) { if (h_dtype == PLLM_F32) PLLM_DSV(float, float); else PLLM_DSV(float, bf16); }
    else { if (h_dtype == PLLM_F32) PLLM_DSV(bf16, float); else PLLM_DSV(bf16, bf16); }
#undef PLLM_DSV
    PLLM_RETURN_LAST_ERROR();
  }
  dim3 grid(num_rows), block(hidden >= 1024 ? 256 : (hidden >= 128 ? 128 : 64));
#define PLLM_DS(TO, TH)                                                                                                              \
  hipLaunchKernelGGL((dyt_sum_kernel<TO, TH>), grid, block, 0, stream_, expert_out, (const TH*)h, ld_h, row_of_pair, weights, top,    \
                     weights_inside, shared, shared_gate, gate_ld, stream, alpha, w, b, (TO*)rows, rows_stride, hidden)
  if (out_dtype == PLLM_F32) { if (h_dtype == PLLM_F32) PLLM_DS(float, float); else PLLM_DS(float, bf16); }
  else { if (h_dtype == PLLM_F32) PLLM_DS(bf16, float); else PLLM_DS(bf16, bf16); }
#undef PLLM_DS
  PLLM_RETURN_LAST_ERROR();
}

// ---------------------------------------------------------------------------------------------
// out = sa * a + sb * b, element by element in float: two mixers' outputs that enter the stream as one branch.
template <typename T>
__global__ __launch_bounds__(256) void scaled_sum_kernel(const T* __restrict__ a, float sa, const T* __restrict__ b, float sb,
                                                         T* __restrict__ out, size_t n) {
  const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) out[i] = from_f32<T>(sa * to_f32(a[i]) + sb * to_f32(b[i]));
}

PLLM_API int pllm_scaled_sum(int dtype, const void* a, float sa, const void* b, float sb, void* out, long n, hipStream_t stream) {
  if (n <= 0) return 0;
  dim3 grid((unsigned)((n + 255) / 256)), block(256);
  if (dtype == PLLM_F32)
    hipLaunchKernelGGL(scaled_sum_kernel<float>, grid, block, 0, stream, (const float*)a, sa, (const float*)b, sb, (float*)out, (size_t)n);
  else
    hipLaunchKernelGGL(scaled_sum_kernel<bf16>, grid, block, 0, stream, (const bf16*)a, sa, (const bf16*)b, sb, (bf16*)out, (size_t)n);
  PLLM_RETURN_LAST_ERROR();
}
