// Attention over a compressed key/value latent kept in pages.
//
// Per token the cache holds one latent vector c [rank] (RMS-normed with a weight) and one rotated key part
// kr [rot] that all heads share.  A head's key is [W_uk c ; kr] and its value W_uv c, so with
// qa = W_uk^T q_plain (the query carried into the latent space) the score is (qa . c + q_rot . kr) * scale and the
// output is W_uv (sum_n p_n c_n): the kernels here work on c and kr alone.
//
// That is attention with one key/value head that all query heads share: key row [c | kr] (padded with zeros to
// `width` elements), value c.  The pages hold exactly that, in the layouts of the framework's paged attention kernels,
// which then serve this mixer as they are:
//   k_pages [pages, 1, block_size, width]   rows [c | kr | 0]
//   v_pages [pages, 1, width, block_size]   c transposed inside the page (optional: only for those kernels)
// a slot is page * block_size + offset, -1 for a token that writes nothing.
//
//   latent_prepare    per token: the RMS norm of the latent, the rotation of kr and of every head's q_rot, the write
//                     of [c | kr] (and of c transposed) into the token's slot, and the heads' rotated query parts put
//                     behind where their latent-space parts go in the query rows [T, heads, width];
//   latent_attention  for latents wider than those kernels take: one wavefront per (token, head), softmax over the
//                     visible keys (causal, inside the window when there is one), keys walked in tiles of 64 aligned
//                     to absolute positions, so that the order of every sum is the same however the tokens were cut.
// All arithmetic is float; T is the storage type.
#include "common.h"

using namespace pllm;

// rows [T, row_stride] (type TI: the pages' type T, or float sums of the product that made them): heads x [plain | rot] of
// the queries at column 0, then the down-projection [rank | rot] at column `down_at`.  q_out [T, heads, width]: columns
// rank .. rank + rot of every head receive its rotated part and the columns behind them zeros (columns 0 .. rank are
// another kernel's).  rot may be 0: a latent without a rotated part (the queries' columns are not read then).
// With q_rank > 0 the rows also hold a latent of the queries at column q_at: cq_out [T, q_rank] receives its RMS norm
// times q_norm_w (the operand of the product that expands it into the heads' queries).
template <typename TI, typename T>
__global__ __launch_bounds__(256) void latent_prepare_kernel(
    const TI* __restrict__ rows, int row_stride, int down_at, const int* __restrict__ positions, const float* __restrict__ cos_t,
    const float* __restrict__ sin_t, const float* __restrict__ norm_w, float eps, const int* __restrict__ slots,
    T* __restrict__ k_pages, T* __restrict__ v_pages, T* __restrict__ q_out, int heads, int plain, int rot, int rank,
    int width, int block_size, int interleaved, int q_at, int q_rank, const float* __restrict__ q_norm_w, T* __restrict__ cq_out) {
  __shared__ float scratch[16];
  const int tok = blockIdx.x;
  const TI* row = rows + (size_t)tok * row_stride;
  const int half = rot / 2;
  const size_t table = half ? (size_t)positions[tok] * half : 0;
  const int slot = slots ? slots[tok] : -1;
  T* k_row = k_pages + (size_t)(slot < 0 ? 0 : slot) * width;
  T* v_col = v_pages ? v_pages + ((size_t)(slot < 0 ? 0 : slot / block_size) * width) * block_size + (slot < 0 ? 0 : slot % block_size) : nullptr;
  // the latent: c = down[:rank] / sqrt(mean(down[:rank]^2) + eps) * w
  float ss = 0.f;
  for (int i = threadIdx.x; i < rank; i += blockDim.x) {
    const float v = to_f32(row[down_at + i]);
    ss = fmaf(v, v, ss);
  }
  const float inv = 1.f / sqrtf(block_sum(ss, scratch) / (float)rank + eps);
  if (slot >= 0) {
    for (int i = threadIdx.x; i < rank; i += blockDim.x) {
      const T c = from_f32<T>(to_f32(row[down_at + i]) * inv * norm_w[i]);
      k_row[i] = c;
      if (v_col) v_col[(size_t)i * block_size] = c;
    }
  }
  if (q_rank > 0) {
    float sq = 0.f;
    for (int i = threadIdx.x; i < q_rank; i += blockDim.x) {
      const float v = to_f32(row[q_at + i]);
      sq = fmaf(v, v, sq);
    }
    const float inv_q = 1.f / sqrtf(block_sum(sq, scratch) / (float)q_rank + eps);
    for (int i = threadIdx.x; i < q_rank; i += blockDim.x)
      cq_out[(size_t)tok * q_rank + i] = from_f32<T>(to_f32(row[q_at + i]) * inv_q * q_norm_w[i]);
  }
  // rotated parts: pair j of the shared key part (unit == heads) and of every head's query part
  for (int idx = threadIdx.x; idx < (heads + 1) * half; idx += blockDim.x) {
    const int unit = idx / half, j = idx % half;
    const TI* part = unit == heads ? row + down_at + rank : row + (size_t)unit * (plain + rot) + plain;
    const int lo_at = interleaved ? 2 * j : j, hi_at = interleaved ? 2 * j + 1 : j + half;
    float lo, hi;
    rotate_pair(to_f32(part[lo_at]), to_f32(part[hi_at]), cos_t[table + j], sin_t[table + j], lo, hi);
    T* dst = unit == heads ? (slot >= 0 ? k_row + rank : nullptr) : q_out + ((size_t)tok * heads + unit) * width + rank;
    if (dst) {
      dst[lo_at] = from_f32<T>(lo);
      dst[hi_at] = from_f32<T>(hi);
    }
  }
  const int pad = width - rank - rot;
  for (int idx = threadIdx.x; idx < heads * pad; idx += blockDim.x)
    q_out[((size_t)tok * heads + idx / pad) * width + rank + rot + idx % pad] = from_f32<T>(0.f);
}

// rows_dtype: the type of `rows` (the pages' type `dtype`, or float).
PLLM_API int pllm_latent_prepare(int dtype, int rows_dtype, const void* rows, int row_stride, int down_at, const int* positions,
                                 const float* cos_t, const float* sin_t, const float* norm_w, float eps, const int* slots, void* k_pages,
                                 void* v_pages, void* q_out, int num_tokens, int heads, int plain, int rot, int rank, int width,
                                 int block_size, int interleaved, int q_at, int q_rank, const float* q_norm_w, void* cq_out,
                                 hipStream_t stream) {
  if (num_tokens <= 0) return 0;
  if (rot < 0 || rot % 2 || rank <= 0 || heads <= 0 || plain < 0 || width < rank + rot || block_size <= 0) return -2;
  if (rot > 0 && (!cos_t || !sin_t)) return -2;
  if (q_rank < 0 || (q_rank > 0 && (!q_norm_w || !cq_out))) return -2;
  if (rows_dtype != dtype && rows_dtype != PLLM_F32) return -2;
  dim3 grid(num_tokens), block(256);
#define PLLM_LP(TI, T)                                                                                                             \
  hipLaunchKernelGGL((latent_prepare_kernel<TI, T>), grid, block, 0, stream, (const TI*)rows, row_stride, down_at, positions, cos_t, \
                     sin_t, norm_w, eps, slots, (T*)k_pages, (T*)v_pages, (T*)q_out, heads, plain, rot, rank, width, block_size,    \
                     interleaved, q_at, q_rank, q_norm_w, (T*)cq_out)
  if (dtype == PLLM_F32) PLLM_LP(float, float);
  else if (rows_dtype == PLLM_F32) PLLM_LP(float, bf16);
  else PLLM_LP(bf16, bf16);
#undef PLLM_LP
  PLLM_RETURN_LAST_ERROR();
}

constexpr int kMaxRank = 1024;      // latent sizes the attention kernel takes (16 output channels per lane)
constexpr int kMaxRot = 256;

// q [T, heads, width] rows [qa | q_rot | 0] (contiguous); out [T, heads, rank]: sum_n p_n c_n.
template <typename T>
__global__ __launch_bounds__(64) void latent_attention_kernel(
    const T* __restrict__ q, const T* __restrict__ k_pages, T* __restrict__ out, const int* __restrict__ block_tables,
    int bt_stride, const int* __restrict__ cu_seqlens_q, const int* __restrict__ seq_lens_k, int num_seqs, int heads,
    int rank, int rot, int width, int block_size, float scale, int window) {
  __shared__ float q_s[kMaxRank + kMaxRot];
  __shared__ float p_s[64];
  __shared__ int slot_s[64];
  const int lane = threadIdx.x;
  const int tok = blockIdx.x, head = blockIdx.y;

  int lo = 0, hi = num_seqs - 1;                       // sequence of this token: the last s with cu[s] <= tok
  while (lo < hi) {
    const int mid = (lo + hi + 1) >> 1;
    if (cu_seqlens_q[mid] <= tok) lo = mid; else hi = mid - 1;
  }
  const int seq = lo;
  const int q_begin = cu_seqlens_q[seq], num_q = cu_seqlens_q[seq + 1] - q_begin;
  const int len_k = seq_lens_k[seq];
  const int q_pos = len_k - num_q + (tok - q_begin);
  const int* bt = block_tables + (size_t)seq * bt_stride;

  for (int i = lane; i < rank + rot; i += 64) q_s[i] = to_f32(q[((size_t)tok * heads + head) * width + i]);
  __syncthreads();

  const int first_key = (window > 0 && q_pos - window + 1 > 0) ? q_pos - window + 1 : 0;
  constexpr int kPerLane = kMaxRank / 64;
  float acc[kPerLane];
#pragma unroll
  for (int r = 0; r < kPerLane; ++r) acc[r] = 0.f;
  float m = -INFINITY, l = 0.f;

  for (int n0 = (first_key / 64) * 64; n0 <= q_pos; n0 += 64) {
    const int n = n0 + lane;
    const bool visible = n >= first_key && n <= q_pos;
    float s = -INFINITY;
    int slot = 0;
    if (visible) {
      slot = bt[n / block_size] * block_size + n % block_size;
      const T* key = k_pages + (size_t)slot * width;
      float dot = 0.f;
      for (int i = 0; i < rank + rot; ++i) dot = fmaf(q_s[i], to_f32(key[i]), dot);
      s = dot * scale;
    }
    const float m_new = fmaxf(m, wave_max(s));   // finite: the tile holds at least one visible key
    const float alpha = expf(m - m_new);          // 0 on the first tile
    const float p = visible ? expf(s - m_new) : 0.f;
    l = l * alpha + wave_sum(p);
    m = m_new;
    __syncthreads();
    p_s[lane] = p;
    slot_s[lane] = slot;
    __syncthreads();
    const int count = (q_pos - n0 + 1 < 64) ? q_pos - n0 + 1 : 64;
#pragma unroll
    for (int r = 0; r < kPerLane; ++r) {
      const int i = lane + r * 64;
      if (i >= rank) break;
      float a = acc[r] * alpha;
      for (int j = 0; j < count; ++j) {
        const float pj = p_s[j];
        if (pj != 0.f) a = fmaf(pj, to_f32(k_pages[(size_t)slot_s[j] * width + i]), a);
      }
      acc[r] = a;
    }
  }
  const float inv_l = 1.f / l;
#pragma unroll
  for (int r = 0; r < kPerLane; ++r) {
    const int i = lane + r * 64;
    if (i < rank) out[((size_t)tok * heads + head) * rank + i] = from_f32<T>(acc[r] * inv_l);
  }
}

PLLM_API int pllm_latent_attention(int dtype, const void* q, const void* k_pages, void* out, const int* block_tables,
                                   int bt_stride, const int* cu_seqlens_q, const int* seq_lens_k, int num_seqs, int total_q,
                                   int heads, int rank, int rot, int width, int block_size, float scale, int window,
                                   hipStream_t stream) {
  if (total_q <= 0 || num_seqs <= 0) return 0;
  if (rank <= 0 || rank > kMaxRank || rot < 0 || rot > kMaxRot || heads <= 0 || block_size <= 0 || width < rank + rot) return -2;
  dim3 grid(total_q, heads), block(64);
  if (dtype == PLLM_F32)
    hipLaunchKernelGGL(latent_attention_kernel<float>, grid, block, 0, stream, (const float*)q, (const float*)k_pages, (float*)out,
                       block_tables, bt_stride, cu_seqlens_q, seq_lens_k, num_seqs, heads, rank, rot, width, block_size, scale, window);
  else
    hipLaunchKernelGGL(latent_attention_kernel<bf16>, grid, block, 0, stream, (const bf16*)q, (const bf16*)k_pages, (bf16*)out,
                       block_tables, bt_stride, cu_seqlens_q, seq_lens_k, num_seqs, heads, rank, rot, width, block_size, scale, window);
  PLLM_RETURN_LAST_ERROR();
}
