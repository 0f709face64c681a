// Paged causal attention without a softmax, in bfloat16 on the matrix cores, for prompt portions and for decoding:
//
//   out[query] = sum over visible keys n of  sigmoid(cap(scale * q . k_n) + head_bias[head]) * v_n,
//
// the weights not normalised over the keys.  A query at position i sees key n when n <= i and (i - n < window or
// n < keep_first): a sliding window beside the sequence's first keep_first positions (window 0: every key).
// cap(x) = c tanh(x / c) for c > 0.  Compiled once per head size (-DHEAD_DIM=16..256 in steps of 16).
//
// The layouts are those of the softmax kernels: q [tokens, heads, D] rows, k_pages [pages, kv_heads, block, D],
// v_pages [pages, kv_heads, D, block] (transposed inside a page), block a power of two of at least 16 positions.
// Work item = (sequence, kv head, tile of 16 * NCB columns); a column is a (query token, head of the kv head's group)
// pair, c = token * G + head_in_group, so the G heads that share a kv head sit side by side and every loaded key tile
// serves all of them.  Scores are computed transposed, S^T = K Q^T, with v_mfma_f32_16x16x32_bf16: the A operand is a
// tile of 16 keys straight from the page, the B operand Q^T held in registers; the result leaves every lane with four
// keys of one column, already in the B-operand layout of O^T = V^T P^T.  With no running maximum and no sum to carry,
// a block of 64 keys adds to the output and nothing else; the WAVES wavefronts of a workgroup deal the blocks of the
// visible keys among themselves (the kept first positions' blocks, then the window's) and add their outputs through
// LDS in wave order.  Weights are float and rounded to bfloat16 for the second product, as the softmax kernels round
// their probabilities.  Values of keys that no column of the tile may see are zeroed (0 * stale data stays 0).
#include "common.h"
#include <type_traits>

using namespace pllm;

#ifndef HEAD_DIM
#error "compile with -DHEAD_DIM=<16..256, multiple of 16>"
#endif
static_assert(HEAD_DIM % 16 == 0 && HEAD_DIM >= 16 && HEAD_DIM <= 256, "head size must be 16..256 in steps of 16");

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
typedef __attribute__((ext_vector_type(4))) float floatx4;
typedef const int __attribute__((address_space(4))) * ConstantInts;
__device__ __forceinline__ ConstantInts as_constant(const int* p) { return (ConstantInts)p; }

constexpr int D = HEAD_DIM;
constexpr int KSTEPS = (D + 31) / 32;    // MFMA steps over the head dimension for K Q^T
constexpr int DBLOCKS = D / 16;          // 16-channel blocks of the output
constexpr float kLog2e = 1.4426950408889634f;

__device__ __forceinline__ bf16x8 zero8() {
  bf16x8 z;
#pragma unroll
  for (int i = 0; i < 8; ++i) z[i] = (__bf16)0.0f;
  return z;
}

template <int NCB, int WAVES, bool TWO>
__global__ __launch_bounds__(WAVES * 64) void sigmoid_attention_kernel(
    const bf16* __restrict__ q, int q_stride, const bf16* __restrict__ k_pages, const bf16* __restrict__ v_pages,
    bf16* __restrict__ out, int out_stride, const int* __restrict__ block_tables, int bt_stride,
    const int* __restrict__ cu_seqlens_q, const int* __restrict__ seq_lens_k, int num_heads, int num_kv_heads,
    int block_size, float scale, int window, int keep_first, float cap, const float* __restrict__ head_bias) {
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), r = lane & 15, g = lane >> 4;
  const int bs_shift = __builtin_ctz(block_size);
  const int seq = blockIdx.z, kvh = blockIdx.y;
  const int G = num_heads / num_kv_heads;
  const int q_begin = as_constant(cu_seqlens_q)[seq], num_q = as_constant(cu_seqlens_q)[seq + 1] - q_begin;
  const int len_k = as_constant(seq_lens_k)[seq];
  const int num_cols = num_q * G;
  const int col0 = blockIdx.x * 16 * NCB;
  if (col0 >= num_cols) return;
  const int last_col = min(col0 + 16 * NCB, num_cols) - 1;
  const int pos0 = len_k - num_q;                               // position of the sequence's first query
  const int qpos_min = pos0 + col0 / G, qpos_max = pos0 + last_col / G;
  // Keys any column of this tile may see: [0, kept) and [vis_lo, vis_hi)
  const int vis_hi = qpos_max + 1;
  const int vis_lo = first_visible_key(qpos_min, window);
  int k_lo = vis_lo & ~63;
  int kept = min(keep_first, vis_hi);
  if (kept >= k_lo) { k_lo = 0; kept = 0; }                     // the two ranges meet: one range from the sequence's start
  const int blocks_kept = (kept + 63) >> 6, blocks = blocks_kept + ((vis_hi - k_lo + 63) >> 6);

  // ---- this lane's column in each column block, and Q^T in B-operand layout
  int my_qpos[NCB], my_first[NCB];
  bool my_valid[NCB];
  size_t my_out[NCB];
  bf16x8 qreg[NCB][KSTEPS];
  float my_bias[NCB];                                           // log2(e) * head_bias
#pragma unroll
  for (int cb = 0; cb < NCB; ++cb) {
    const int c = col0 + cb * 16 + r;
    my_valid[cb] = c < num_cols;
    const int tok = my_valid[cb] ? c / G : 0, hg = my_valid[cb] ? c - tok * G : 0;
    my_qpos[cb] = my_valid[cb] ? pos0 + tok : -1;               // -1: sees nothing
    my_first[cb] = first_visible_key(my_qpos[cb], window);
    const size_t row = (size_t)(q_begin + tok) * q_stride + (size_t)(kvh * G + hg) * D;
    my_out[cb] = (size_t)(q_begin + tok) * out_stride + (size_t)(kvh * G + hg) * D;
    my_bias[cb] = (head_bias && my_valid[cb]) ? head_bias[kvh * G + hg] * kLog2e : 0.f;
#pragma unroll
    for (int s = 0; s < KSTEPS; ++s) {
      const int dd = s * 32 + g * 8;
      qreg[cb][s] = (my_valid[cb] && dd < D) ? *reinterpret_cast<const bf16x8*>(q + row + dd) : zero8();
    }
  }
  floatx4 acc[NCB][DBLOCKS];
#pragma unroll
  for (int cb = 0; cb < NCB; ++cb)
#pragma unroll
    for (int db = 0; db < DBLOCKS; ++db) acc[cb][db] = floatx4{0.f, 0.f, 0.f, 0.f};

  // the score in log2 units: log2(e) * cap(scale * s), with c tanh(x / c) = c (1 - 2 / (2^(2 log2(e) x / c) + 1))
  const bool capped = cap > 0.f;
  const float sl2 = scale * kLog2e, cap_l2 = cap * kLog2e, cap_in = capped ? 2.f * kLog2e * scale / cap : 0.f;

  ConstantInts bt = as_constant(block_tables) + (size_t)seq * bt_stride;
  const size_t page_elems = (size_t)block_size * D;             // one kv head's part of a page
  const size_t page_stride = page_elems * num_kv_heads;

  // One block = 64 keys = four tiles of 16.  All of a block's keys and values are asked for together, and where the
  // registers hold two blocks the next one travels while this one is used: a prompt of a few thousand tokens leaves
  // a SIMD with two wavefronts or fewer, which cannot hide each other's waits for memory.
  struct KVBlock {
    bf16x8 k[4][KSTEPS];
    bf16x4 v[4][DBLOCKS];
    bool on[4];
    int n0;
  };
  auto load_block = [&](KVBlock& blk, int b) {
    const bool in_kept = b < blocks_kept;
    blk.n0 = in_kept ? b * 64 : k_lo + (b - blocks_kept) * 64;
    const int limit = in_kept ? kept : vis_hi;                  // keys of this block at or beyond it are nobody's
#pragma unroll
    for (int kt = 0; kt < 4; ++kt) {
      const int nk = blk.n0 + kt * 16;
      blk.on[kt] = nk < limit;                                  // uniform
      if (!blk.on[kt]) continue;
      const int page = bt[nk >> bs_shift];
      const int off = nk & (block_size - 1);
      const size_t base = (size_t)page * page_stride + (size_t)kvh * page_elems;
      const bf16* krow = k_pages + base + (size_t)(off + r) * D;
#pragma unroll
      for (int s = 0; s < KSTEPS; ++s) {
        const int dd = s * 32 + g * 8;
        blk.k[kt][s] = (dd < D) ? *reinterpret_cast<const bf16x8*>(krow + dd) : zero8();
      }
      const bf16* vrow = v_pages + base + off + g * 4;          // + channel * block_size
#pragma unroll
      for (int db = 0; db < DBLOCKS; ++db) blk.v[kt][db] = *reinterpret_cast<const bf16x4*>(vrow + (size_t)(db * 16 + r) * block_size);
    }
  };
  // (seen_by_all: every key of the block is visible to every column of a full tile, so nothing is masked)
  auto compute_block_as = [&](KVBlock& blk, auto seen_by_all) {
    constexpr bool kAll = decltype(seen_by_all)::value;
    const int n0 = blk.n0;
    // ---- S^T = K Q^T for four tiles of 16 keys, then the weights; lane holds keys n0 + kt*16 + g*4 + i of its column
    bf16x8 p_op[2][NCB];                                        // B operands of the second product
#pragma unroll
    for (int kt = 0; kt < 4; ++kt) {
#pragma unroll
      for (int cb = 0; cb < NCB; ++cb) {
        floatx4 s_t = floatx4{0.f, 0.f, 0.f, 0.f};
        if (blk.on[kt]) {
#pragma unroll
          for (int s = 0; s < KSTEPS; ++s) s_t = __builtin_amdgcn_mfma_f32_16x16x32_bf16(blk.k[kt][s], qreg[cb][s], s_t, 0, 0, 0);
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int n = n0 + kt * 16 + g * 4 + i;
          const bool vis = kAll || (blk.on[kt] && n <= my_qpos[cb] && (n >= my_first[cb] || n < keep_first));
          float z = capped ? fmaf(-2.f * cap_l2, __builtin_amdgcn_rcpf(__builtin_amdgcn_exp2f(s_t[i] * cap_in) + 1.f), cap_l2) : s_t[i] * sl2;
          z += my_bias[cb];
          const float p = __builtin_amdgcn_rcpf(1.f + __builtin_amdgcn_exp2f(-z));
          p_op[kt >> 1][cb][(kt & 1) * 4 + i] = (__bf16)(vis ? p : 0.f);
        }
      }
    }
    // ---- O^T += V^T P^T : A operand = 16 channels x 32 keys (k slots 0-3: tile 2a, 4-7: tile 2a+1)
#pragma unroll
    for (int a = 0; a < 2; ++a) {
      if (!blk.on[2 * a]) continue;
#pragma unroll
      for (int db = 0; db < DBLOCKS; ++db) {
        bf16x8 vreg;
#pragma unroll
        for (int h = 0; h < 2; ++h) {
          const int kt = 2 * a + h;
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            const int n = n0 + kt * 16 + g * 4 + i;
            const bool anybody = kAll || (blk.on[kt] && n < vis_hi && (n >= vis_lo || n < keep_first));
            vreg[h * 4 + i] = anybody ? blk.v[kt][db][i] : (__bf16)0.0f;
          }
        }
#pragma unroll
        for (int cb = 0; cb < NCB; ++cb)
          acc[cb][db] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vreg, p_op[a][cb], acc[cb][db], 0, 0, 0);
      }
    }
  };
  const int first_of_last = first_visible_key(qpos_max, window);
  const bool full_tile = col0 + 16 * NCB <= num_cols;
  auto compute_block = [&](KVBlock& blk) {
    const int n0 = blk.n0;
    const bool all = full_tile && blk.on[3] && n0 + 63 <= qpos_min && (n0 >= first_of_last || n0 + 64 <= keep_first);
    if (all) compute_block_as(blk, std::true_type{}); else compute_block_as(blk, std::false_type{});
  };
  constexpr bool kTwoBlocks = TWO && 4 * KSTEPS * 4 + 4 * DBLOCKS * 2 <= 64;
  if constexpr (kTwoBlocks) {
    KVBlock blk_a, blk_b;
    int b = wave;
    if (b < blocks) {
      load_block(blk_a, b);
      while (true) {
        const int b1 = b + WAVES;
        const bool has1 = b1 < blocks;
        if (has1) load_block(blk_b, b1);
        compute_block(blk_a);
        if (!has1) break;
        const int b2 = b1 + WAVES;
        const bool has2 = b2 < blocks;
        if (has2) load_block(blk_a, b2);
        compute_block(blk_b);
        if (!has2) break;
        b = b2;
      }
    }
  } else {
    KVBlock blk;
    for (int b = wave; b < blocks; b += WAVES) {
      load_block(blk, b);
      compute_block(blk);
    }
  }

  if constexpr (WAVES > 1) {
    // ---- the wavefronts' outputs added in wave order
    extern __shared__ float lds[];                               // [WAVES][NCB * DBLOCKS * 4][64]
#pragma unroll
    for (int cb = 0; cb < NCB; ++cb)
#pragma unroll
      for (int db = 0; db < DBLOCKS; ++db)
#pragma unroll
        for (int i = 0; i < 4; ++i) lds[((size_t)(wave * NCB + cb) * DBLOCKS * 4 + db * 4 + i) * 64 + lane] = acc[cb][db][i];
    __syncthreads();
    // entry e = (cb, db, i); thread (e, lane) owns column cb*16 + r, channel db*16 + g*4 + i
    for (int e = wave; e < NCB * DBLOCKS * 4; e += WAVES) {
      const int cb = e / (DBLOCKS * 4), rest = e - cb * DBLOCKS * 4, db = rest >> 2, i = rest & 3;
      const int c = col0 + cb * 16 + r;
      if (c >= num_cols) continue;
      float o = 0.f;
      for (int w = 0; w < WAVES; ++w) o += lds[((size_t)(w * NCB + cb) * DBLOCKS * 4 + rest) * 64 + lane];
      const int tok = c / G, hg = c - tok * G;
      out[(size_t)(q_begin + tok) * out_stride + (size_t)(kvh * G + hg) * D + db * 16 + g * 4 + i] = __float2bfloat16(o);
    }
    return;
  }
#pragma unroll
  for (int cb = 0; cb < NCB; ++cb) {
    if (!my_valid[cb]) continue;
#pragma unroll
    for (int db = 0; db < DBLOCKS; ++db) {
      bf16x4 o;
#pragma unroll
      for (int i = 0; i < 4; ++i) o[i] = (__bf16)acc[cb][db][i];
      *reinterpret_cast<bf16x4*>(out + my_out[cb] + db * 16 + g * 4) = o;
    }
  }
}

// max_q_len: a bound on the queries of one sequence of this launch (the grid covers that many columns per sequence
// and kv head; tiles past a sequence's own columns leave at once).  ncb: tiles of 16 columns per workgroup (1 or 2);
// waves: wavefronts per workgroup that share its columns and deal its key blocks (1, 2, 4 or 8); two_blocks: the next
// block's loads are asked for before this block is used (head sizes up to 64).  q, out: rows of heads * D bfloat16
// elements with 16-byte aligned strides.
PLLM_API int pllm_sigmoid_attention(const void* q, int q_stride, const void* k_pages, const void* v_pages, void* out, int out_stride,
                                    const int* block_tables, int bt_stride, const int* cu_seqlens_q, const int* seq_lens_k,
                                    int num_seqs, int max_q_len, int num_heads, int num_kv_heads, int block_size, float scale,
                                    int window, int keep_first, float cap, const float* head_bias, int ncb, int waves, int two_blocks,
                                    hipStream_t stream) {
  if (num_seqs <= 0 || max_q_len <= 0) return 0;
  if (num_kv_heads <= 0 || num_heads % num_kv_heads || block_size < 16 || (block_size & (block_size - 1)) || window < 0 || keep_first < 0 ||
      !(cap >= 0.f) || (q_stride & 7) || (out_stride & 3) || num_seqs > 65535 || num_kv_heads > 65535)
    return -2;
  const int G = num_heads / num_kv_heads;
  const long cols = (long)max_q_len * G;
#define PLLM_SIGMOID(NCB, WAVES, TWO)                                                                                                   \
  hipLaunchKernelGGL((sigmoid_attention_kernel<NCB, WAVES, TWO>), dim3((unsigned)((cols + 16 * NCB - 1) / (16 * NCB)), num_kv_heads, num_seqs), \
                     dim3(WAVES * 64), WAVES > 1 ? (size_t)WAVES * NCB * DBLOCKS * 4 * 64 * sizeof(float) : 0, stream, (const bf16*)q, q_stride,  \
                     (const bf16*)k_pages, (const bf16*)v_pages, (bf16*)out, out_stride, block_tables, bt_stride, cu_seqlens_q, seq_lens_k,     \
                     num_heads, num_kv_heads, block_size, scale, window, keep_first, cap, head_bias)
#define PLLM_SIGMOID_WAVES(NCB, TWO)                                       \
  switch (waves) {                                                          \
    case 1: PLLM_SIGMOID(NCB, 1, TWO); break;                               \
    case 2: PLLM_SIGMOID(NCB, 2, TWO); break;                               \
    case 4: PLLM_SIGMOID(NCB, 4, TWO); break;                               \
    case 8: PLLM_SIGMOID(NCB, 8, TWO); break;                               \
    default: return -2;                                                     \
  }
  if ((size_t)waves * ncb * DBLOCKS * 4 * 64 * sizeof(float) > 64 * 1024 && waves > 1) return -2;
  if (ncb == 1 && two_blocks) { PLLM_SIGMOID_WAVES(1, true) }
  else if (ncb == 1) { PLLM_SIGMOID_WAVES(1, false) }
  else if (ncb == 2 && !two_blocks) { PLLM_SIGMOID_WAVES(2, false) }
  else return -2;
#undef PLLM_SIGMOID_WAVES
#undef PLLM_SIGMOID
  PLLM_RETURN_LAST_ERROR();
}
