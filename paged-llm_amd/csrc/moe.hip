// A feed-forward of routed experts: every token goes through `top` of `experts` small gated feed-forwards (and, where
// the router says so, through pass-through experts that hand the token back), weighted by router scores.
//
//   moe_route      per token: router outputs in float, softmax over all of them, the choice among the best groups of
//                  neighbouring experts by score + correction, the weights = the chosen experts' plain scores;
//   moe_align      the (token, choice) pairs sorted by expert: per expert a run of rows, cut into tiles of rows;
//   moe_expert_gemm the experts' products over those runs: act(gate h) * (up h) from the tokens' rows, and the down
//                  product from the activations; one tile of rows per workgroup, every row's sums in ascending k,
//                  so a pair's result does not depend on which other pairs share its tile or in which order
//                  (bfloat16: on the matrix cores; float32, and sizes that fit no 16-byte load: plain multiply-adds);
//   moe_combine    out[t] = sum over the token's choices, in their order, of weight * (expert output | the token's row).
//
// Router, softmax, weights and the final sum are float; T is the storage type of rows, activations and matrices.
#include "common.h"

using namespace pllm;

constexpr int kMoeTileRows = 16;      // rows (pairs) of the smallest tile of the experts' products
constexpr int kMoeMaxTileRows = 128;  // ... and of the largest (steps with many pairs per expert); 64 in between

// ---------------------------------------------------------------------------------------------
// n = experts + pass-through experts router outputs; groups of n / groups neighbours; a group's mark is its largest
// corrected score; only experts of the `keep` best groups can be chosen (ties: the lower index wins).
constexpr int kRouteThreads = 1024, kRoutePieces = 16;   // threads of a workgroup in steps of few tokens; pieces the products are cut into

template <typename T, int TOK>
__global__ __launch_bounds__(kRouteThreads) void moe_route_kernel(const T* __restrict__ h, int ld, const float* __restrict__ router_w,
                                                                  const float* __restrict__ correction, int num_tokens, int width, int n_all,
                                                                  int extra, int scoring, int groups, int keep, int top, int segments,
                                                                  int* __restrict__ ids, float* __restrict__ weights, float* __restrict__ extras) {
  extern __shared__ float lds[];
  // n_all rows of the router matrix: the first n = n_all - extra are the experts' (scores, the choice), the last `extra`
  // are further outputs of the same product that go to `extras` [tokens, extra] as they are
  const int n = n_all - extra;
  const int per_token = 2 * n_all + groups + segments * n_all;       // floats of LDS that one token has
  const int t0 = blockIdx.x * TOK;                           // this workgroup's tokens: t0 .. t0 + TOK - 1
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const T* row[TOK];
#pragma unroll
  for (int k = 0; k < TOK; ++k) row[k] = h + (size_t)min(t0 + k, num_tokens - 1) * ld;     // (tokens past the last repeat it: not stored)
  // The router's products.  A piece of work is eight router rows times one of `segments` equal parts of the tokens'
  // rows, and the wavefronts (16 for one token; 4 or 8 where a workgroup has as many tokens) take the pieces in turn: one pass over the part
  // with eight independent loads and sums per element and token, several elements under way (few tokens, a router matrix
  // that the experts' weights have pushed out of the caches since the last layer: what counts is how few loads wait for
  // one another; many tokens: a router element is fetched once for TOK of them).  A router output is the sum of its
  // parts in ascending order, each part summed lane by lane and then over the wavefront, whatever TOK is.
  const int batches = (n_all + 7) / 8;
  const int seg = ((width + segments - 1) / segments + 63) & ~63;
  for (int piece = wave; piece < batches * segments; piece += (int)(blockDim.x >> 6)) {
    const int e0 = (piece / segments) * 8, sg = piece % segments;
    const int from = sg * seg, to = min(width, from + seg);
    float acc[8][TOK];
#pragma unroll
    for (int j = 0; j < 8; ++j)
#pragma unroll
      for (int k = 0; k < TOK; ++k) acc[j][k] = 0.f;
    const float* w = router_w + (size_t)e0 * width;
    if (TOK == 1 && e0 + 8 <= n_all) {
      // every load of eight elements' worth asked for before the first sum: 72 loads under way, one trip to memory
      for (int i0 = from + lane; i0 < to; i0 += 8 * 64) {
        float x[8], wv[8][8];
#pragma unroll
        for (int u = 0; u < 8; ++u) {
          const int i = min(i0 + u * 64, to - 1);
          x[u] = i0 + u * 64 < to ? to_f32(row[0][i]) : 0.f;      // (an element past the part counts as zero times a valid weight)
#pragma unroll
          for (int j = 0; j < 8; ++j) wv[u][j] = w[(size_t)j * width + i];
        }
#pragma unroll
        for (int u = 0; u < 8; ++u)
#pragma unroll
          for (int j = 0; j < 8; ++j) acc[j][0] = fmaf(x[u], wv[u][j], acc[j][0]);
      }
    } else if (e0 + 8 <= n_all) {
#pragma unroll(TOK >= 8 ? 1 : 2)
      for (int i = from + lane; i < to; i += 64) {
        float x[TOK];
#pragma unroll
        for (int k = 0; k < TOK; ++k) x[k] = to_f32(row[k][i]);
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          const float wj = w[(size_t)j * width + i];
#pragma unroll
          for (int k = 0; k < TOK; ++k) acc[j][k] = fmaf(x[k], wj, acc[j][k]);
        }
      }
    } else {
      for (int i = from + lane; i < to; i += 64) {
        float x[TOK];
#pragma unroll
        for (int k = 0; k < TOK; ++k) x[k] = to_f32(row[k][i]);
#pragma unroll
        for (int j = 0; j < 8; ++j)
          if (e0 + j < n_all) {
            const float wj = w[(size_t)j * width + i];
#pragma unroll
            for (int k = 0; k < TOK; ++k) acc[j][k] = fmaf(x[k], wj, acc[j][k]);
          }
      }
    }
#pragma unroll
    for (int j = 0; j < 8; ++j)
#pragma unroll
      for (int k = 0; k < TOK; ++k) {
        const float total = wave_sum(acc[j][k]);
        if (lane == 0 && e0 + j < n_all) lds[k * per_token + 2 * n_all + groups + sg * n_all + e0 + j] = total;
      }
  }
  __syncthreads();
  for (int i = threadIdx.x; i < TOK * n_all; i += blockDim.x) {
    const int k = i / n_all, e = i - k * n_all;
    const float* part = lds + k * per_token + 2 * n_all + groups;
    float total = part[e];
    for (int sg = 1; sg < segments; ++sg) total += part[sg * n_all + e];
    if (e < n) lds[k * per_token + e] = total;
    else if (t0 + k < num_tokens) extras[(size_t)(t0 + k) * extra + (e - n)] = total;
  }
  __syncthreads();
  // The choice: wavefront k makes token t0 + k's (the others keep them company at the barriers).
  const int t = t0 + wave;
  const bool chooser = wave < TOK && t < num_tokens;
  float* score = lds + (wave < TOK ? wave : 0) * per_token;   // [n]  router outputs, then scores
  float* choice = score + n_all;                              // [n]  score + correction, -inf once taken or shut out
  float* mark = score + 2 * n_all;                            // [groups]
  // Lane l looks after router outputs l, l + 64, ...; a largest element is found by a maximum over the wavefront and
  // then the lowest index that holds it (ties: the lower index wins).
  auto lowest_at = [&](const float* values, int count) {
    float mine = -INFINITY;
    for (int e = lane; e < count; e += 64) mine = fmaxf(mine, values[e]);
    const float best = wave_max(mine);
    float at = 3.0e9f;
    for (int e = lane; e < count; e += 64)
      if (values[e] == best) { at = (float)e; break; }
    return (int)(-wave_max(-at));
  };
  if (chooser && scoring == 1) {
    // scores by a sigmoid of every router output on its own
    for (int e = lane; e < n; e += 64) {
      const float sc = 1.f / (1.f + expf(-score[e]));
      score[e] = sc;
      choice[e] = sc + (correction ? correction[e] : 0.f);
    }
  } else if (chooser) {
    float m = -INFINITY;
    for (int e = lane; e < n; e += 64) m = fmaxf(m, score[e]);
    m = wave_max(m);
    float sum = 0.f;
    for (int e = lane; e < n; e += 64) { const float x = expf(score[e] - m); score[e] = x; sum += x; }
    sum = wave_sum(sum);
    const float inv = 1.f / sum;
    for (int e = lane; e < n; e += 64) {
      const float sc = score[e] * inv;
      score[e] = sc;
      choice[e] = sc + (correction ? correction[e] : 0.f);
    }
  }
  __syncthreads();
  const int per = n / groups;
  if (keep < groups) {
    if (chooser)
      for (int g = lane; g < groups; g += 64) {
        float best = -INFINITY;
        for (int e = g * per; e < (g + 1) * per; ++e) best = fmaxf(best, choice[e]);
        mark[g] = best;
      }
    __syncthreads();
    // the `keep` best groups are taken one by one (a taken group's mark becomes -inf); the others' experts are shut out
    for (int k = 0; k < keep; ++k) {
      if (chooser) {
        const int at = lowest_at(mark, groups);
        if (lane == 0) mark[at] = -INFINITY;
      }
      __syncthreads();
    }
    if (chooser)
      for (int e = lane; e < n; e += 64)
        if (mark[e / per] != -INFINITY) choice[e] = -INFINITY;
    __syncthreads();
  }
  for (int k = 0; k < top; ++k) {
    if (chooser) {
      const int at = lowest_at(choice, n);
      if (lane == 0) {
        ids[(size_t)t * top + k] = at;
        weights[(size_t)t * top + k] = score[at];
        choice[at] = -INFINITY;
      }
    }
    __syncthreads();
  }
}

// n_all = n + extra rows of the router matrix; scoring 0: softmax over the n router outputs, 1: a sigmoid of each.
PLLM_API int pllm_moe_route(int dtype, const void* h, int ld, const float* router_w, const float* correction, int num_tokens, int width,
                            int n_all, int extra, int scoring, int groups, int keep, int top, int* ids, float* weights, float* extras,
                            hipStream_t stream) {
  if (num_tokens <= 0) return 0;
  const int n = n_all - extra;
  if (extra < 0 || (extra > 0 && !extras) || scoring < 0 || scoring > 1) return -2;
  if (n <= 0 || groups <= 0 || n % groups || keep <= 0 || keep > groups || top <= 0 || top > (n / groups) * keep) return -2;
  // as many parts of the row as make 16 pieces (1, 2, 4, 8 or 16 parts), none shorter than 64 elements: by the router's
  // shape alone, so that a token's scores do not depend on the step it is in
  int segments = 1;
  while (segments < kRoutePieces && ((n_all + 7) / 8) * segments < kRoutePieces && width / (2 * segments) >= 64) segments *= 2;
  const size_t lds_one = (size_t)(2 * n_all + groups + segments * n_all) * sizeof(float);
  // tokens to a workgroup (one wavefront each for the choice): 8 in steps of 512 tokens and more, 4 from 128 on, else one
  // token to sixteen wavefronts
  const int tok = (num_tokens >= 512 && 8 * lds_one <= 48 * 1024) ? 8 : (num_tokens >= 128 && 4 * lds_one <= 48 * 1024) ? 4 : 1;
  const size_t lds = lds_one * tok;
#define PLLM_ROUTE(T, TOK, THREADS)                                                                                              \
  hipLaunchKernelGGL((moe_route_kernel<T, TOK>), dim3((num_tokens + TOK - 1) / TOK), dim3(THREADS), lds, stream, (const T*)h, ld, \
                     router_w, correction, num_tokens, width, n_all, extra, scoring, groups, keep, top, segments, ids, weights, extras)
  if (dtype == PLLM_F32) { if (tok == 8) PLLM_ROUTE(float, 8, 512); else if (tok == 4) PLLM_ROUTE(float, 4, 256); else PLLM_ROUTE(float, 1, kRouteThreads); }
  else { if (tok == 8) PLLM_ROUTE(bf16, 8, 512); else if (tok == 4) PLLM_ROUTE(bf16, 4, 256); else PLLM_ROUTE(bf16, 1, kRouteThreads); }
#undef PLLM_ROUTE
  PLLM_RETURN_LAST_ERROR();
}

// ---------------------------------------------------------------------------------------------
// ids [pairs] -> the pairs of experts < `experts` sorted by expert.
//   sorted_pair [pairs]   the pair at each sorted row (rows past the last one: untouched)
//   row_of_pair [pairs]   the sorted row of each pair, -1 for a pass-through expert
//   tiles [max_tiles][3]  (expert, first row, rows) of every tile of at most tile_rows rows; tiles[.][2] = 0 past the last
// One workgroup; the order of the pairs of one expert is whatever the atomics give (the products do not depend on it).
constexpr int kMoeMaxExperts = 1024;

__global__ __launch_bounds__(1024) void moe_align_kernel(const int* __restrict__ ids, int pairs, int experts, int* __restrict__ sorted_pair,
                                                         int* __restrict__ row_of_pair, int* __restrict__ tiles, int max_tiles, int tile_rows) {
  __shared__ int count[kMoeMaxExperts], first[kMoeMaxExperts], cursor[kMoeMaxExperts];
  for (int e = threadIdx.x; e < experts; e += blockDim.x) { count[e] = 0; cursor[e] = 0; }
  __syncthreads();
  for (int p = threadIdx.x; p < pairs; p += blockDim.x) {
    const int e = ids[p];
    if (e >= 0 && e < experts) atomicAdd(&count[e], 1);
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    int at = 0, nt = 0;
    for (int e = 0; e < experts; ++e) {
      first[e] = at;
      for (int r = 0; r < count[e] && nt < max_tiles; r += tile_rows, ++nt) {
        tiles[3 * nt] = e;
        tiles[3 * nt + 1] = at + r;
        tiles[3 * nt + 2] = min(tile_rows, count[e] - r);
      }
      at += count[e];
    }
    for (; nt < max_tiles; ++nt) { tiles[3 * nt] = 0; tiles[3 * nt + 1] = 0; tiles[3 * nt + 2] = 0; }
  }
  __syncthreads();
  for (int p = threadIdx.x; p < pairs; p += blockDim.x) {
    const int e = ids[p];
    if (e >= 0 && e < experts) {
      const int row = first[e] + atomicAdd(&cursor[e], 1);
      sorted_pair[row] = p;
      row_of_pair[p] = row;
    } else {
      row_of_pair[p] = -1;
    }
  }
}

PLLM_API int pllm_moe_align(const int* ids, int pairs, int experts, int* sorted_pair, int* row_of_pair, int* tiles, int max_tiles,
                            int tile_rows, hipStream_t stream) {
  if (pairs <= 0) return 0;
  if (tile_rows < kMoeTileRows || tile_rows % kMoeTileRows || tile_rows > kMoeMaxTileRows) return -2;
  if (experts <= 0 || experts > kMoeMaxExperts || max_tiles < (pairs + tile_rows - 1) / tile_rows + experts) return -2;
  hipLaunchKernelGGL(moe_align_kernel, dim3(1), dim3(1024), 0, stream, ids, pairs, experts, sorted_pair, row_of_pair, tiles, max_tiles, tile_rows);
  PLLM_RETURN_LAST_ERROR();
}

// ---------------------------------------------------------------------------------------------
// One tile of rows of one expert times 64 of the expert's weight rows, plain multiply-adds with float sums in ascending k.
//   GATED: a[row] = rows_in[sorted_pair[row] / top] (the token's row), w = [gate; up] [experts, 2 n_out, K],
//          out[row, n] = T(act(gate . a) * (up . a));
//   else:  a[row] = rows_in[row] (the activations, already sorted), w [experts, n_out, K], out[row, n] = float sum.
constexpr int kMoeCols = 64, kMoeK = 32;

template <typename T, bool GATED>
__global__ __launch_bounds__(256) void moe_expert_gemm_kernel(const T* __restrict__ rows_in, int ld_in, const T* __restrict__ w,
                                                              const int* __restrict__ tiles, const int* __restrict__ sorted_pair, int top,
                                                              int n_out, int K, void* __restrict__ out_, int ld_out, int act,
                                                              const float* __restrict__ pair_scale) {
  __shared__ float a_s[kMoeTileRows][kMoeK + 1];
  __shared__ float w_s[(GATED ? 2 : 1) * kMoeCols][kMoeK + 1];
  __shared__ int src[kMoeTileRows];
  const int tile = blockIdx.x;
  const int expert = tiles[3 * tile], row0 = tiles[3 * tile + 1], nrows = tiles[3 * tile + 2];
  if (nrows <= 0) return;
  const int n0 = blockIdx.y * kMoeCols;
  const int tid = threadIdx.x;
  if (tid < kMoeTileRows) src[tid] = tid < nrows ? (GATED ? sorted_pair[row0 + tid] / top : row0 + tid) : -1;
  __syncthreads();
  const T* we = w + (size_t)expert * (GATED ? 2 : 1) * n_out * K;
  const int r = tid >> 4, cg = tid & 15;           // this thread: row r, columns cg, cg + 16, cg + 32, cg + 48
  float acc[4] = {0.f, 0.f, 0.f, 0.f}, acc2[4] = {0.f, 0.f, 0.f, 0.f};
  for (int k0 = 0; k0 < K; k0 += kMoeK) {
    for (int i = tid; i < kMoeTileRows * kMoeK; i += 256) {
      const int rr = i / kMoeK, kk = i - rr * kMoeK;
      a_s[rr][kk] = (src[rr] >= 0 && k0 + kk < K) ? to_f32(rows_in[(size_t)src[rr] * ld_in + k0 + kk]) : 0.f;
    }
    for (int i = tid; i < (GATED ? 2 : 1) * kMoeCols * kMoeK; i += 256) {
      const int cc = i / kMoeK, kk = i - cc * kMoeK;
      const int half = cc / kMoeCols, col = n0 + (cc - half * kMoeCols);
      w_s[cc][kk] = (col < n_out && k0 + kk < K) ? to_f32(we[((size_t)half * n_out + col) * K + k0 + kk]) : 0.f;
    }
    __syncthreads();
#pragma unroll 8
    for (int kk = 0; kk < kMoeK; ++kk) {
      const float a = a_s[r][kk];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        acc[j] = fmaf(a, w_s[cg + 16 * j][kk], acc[j]);
        if (GATED) acc2[j] = fmaf(a, w_s[kMoeCols + cg + 16 * j][kk], acc2[j]);
      }
    }
    __syncthreads();
  }
  if (r >= nrows) return;
  const float ps = (GATED && pair_scale) ? pair_scale[sorted_pair[row0 + r]] : 1.f;
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int col = n0 + cg + 16 * j;
    if (col >= n_out) continue;
    if (GATED) reinterpret_cast<T*>(out_)[(size_t)(row0 + r) * ld_out + col] = from_f32<T>(gate_activation(acc[j] * ps, act) * (acc2[j] * ps));
    else reinterpret_cast<float*>(out_)[(size_t)(row0 + r) * ld_out + col] = acc[j];
  }
}

// ---------------------------------------------------------------------------------------------
// The same products in bfloat16 on the matrix cores (v_mfma_f32_16x16x32_bf16), operands straight from memory into the
// registers the instruction reads: lane (r, g) = (lane & 15, lane >> 4) holds elements 8 g .. 8 g + 7 of row r of a
// k-step of 32, for the tile's rows (gathered through sorted_pair for the gated product) and for 16 weight rows alike.
// A workgroup is one tile of MT * 16 rows of one expert times 4 wavefronts * U blocks of 16 outputs (gated: the
// gate's and the up product's 16 rows each); a wavefront keeps U * MT (gated: 2 U MT) accumulators.  In steps of few
// tokens (MT = 1) every wavefront streams weight rows that no other one reads, which is all there is to do: such a step
// is bound by the chosen experts' bytes.  In prompt steps (tiles of 64 rows) the four wavefronts read the same rows
// (the first one's misses are the others' cache hits) and each of its own weight rows once per 64 rows.
// An output element is one accumulator over ascending k-steps whatever MT and U are, so its value does not depend on
// the tile it is in, the kernel's shape or the other rows.  K % 8 == 0, ld_in % 8 == 0; a last k-step beyond K reads zeros.
typedef __attribute__((ext_vector_type(8))) __bf16 moe_bf16x8;
typedef __attribute__((ext_vector_type(4))) float moe_floatx4;

template <bool GATED, int MT, int U>
__global__ __launch_bounds__(256) void moe_expert_mfma_kernel(const bf16* __restrict__ rows_in, int ld_in, const bf16* __restrict__ w,
                                                              const int* __restrict__ tiles, const int* __restrict__ sorted_pair, int top,
                                                              int n_out, int K, void* __restrict__ out_, int ld_out, int act,
                                                              const float* __restrict__ pair_scale) {
  constexpr int W = GATED ? 2 : 1;
  const int tile = blockIdx.x;
  const int expert = tiles[3 * tile], row0 = tiles[3 * tile + 1], nrows = tiles[3 * tile + 2];
  if (nrows <= 0) return;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int r = lane & 15, g = lane >> 4;
  const int block0 = (blockIdx.y * 4 + wave) * U;           // this wavefront's first block of 16 outputs
  if (block0 * 16 >= n_out) return;
  const bf16* a_ptr[MT];
#pragma unroll
  for (int t = 0; t < MT; ++t) {
    const int row = row0 + min(t * 16 + r, nrows - 1);       // rows past the tile's last repeat it: never stored
    const int src = GATED ? sorted_pair[row] / top : row;
    a_ptr[t] = rows_in + (size_t)src * ld_in + 8 * g;
  }
  const bf16* we = w + (size_t)expert * W * n_out * K;
  const bf16* w_ptr[U][W];
#pragma unroll
  for (int u = 0; u < U; ++u) {
    const int col = min((block0 + u) * 16 + r, n_out - 1);   // outputs past the last repeat it: never stored
#pragma unroll
    for (int h = 0; h < W; ++h) w_ptr[u][h] = we + ((size_t)h * n_out + col) * K + 8 * g;
  }
  moe_floatx4 acc[U][W][MT];
#pragma unroll
  for (int u = 0; u < U; ++u)
#pragma unroll
    for (int h = 0; h < W; ++h)
#pragma unroll
      for (int t = 0; t < MT; ++t) acc[u][h][t] = moe_floatx4{0.f, 0.f, 0.f, 0.f};
  const int k_whole = K & ~31;
  int k_done = 0;
  if (MT == 1) {
    // A tile of 16 rows streams weights and does little else.  Two k-steps at a time, with a lane holding 16
    // neighbouring elements of its row (32 bytes; four lanes read a whole line of 128) of which the first eight feed one
    // matrix instruction and the last eight the next: rows and weights are cut the same way, so the 64 products of an
    // output are the same ones, summed in two other halves than with 8 + 8 elements 32 apart.  Four such pairs of
    // steps are under way per wavefront.
    const int k_pairs = K & ~63;
#pragma unroll 4
    for (int k0 = 0; k0 < k_pairs; k0 += 64) {
      moe_bf16x8 a[2], b[U][W][2];
#pragma unroll
      for (int half = 0; half < 2; ++half) {
        a[half] = *reinterpret_cast<const moe_bf16x8*>(a_ptr[0] + k0 + 8 * g + 8 * half);
#pragma unroll
        for (int u = 0; u < U; ++u)
#pragma unroll
          for (int h = 0; h < W; ++h) b[u][h][half] = *reinterpret_cast<const moe_bf16x8*>(w_ptr[u][h] + k0 + 8 * g + 8 * half);
      }
#pragma unroll
      for (int half = 0; half < 2; ++half)
#pragma unroll
        for (int u = 0; u < U; ++u)
#pragma unroll
          for (int h = 0; h < W; ++h) acc[u][h][0] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(b[u][h][half], a[half], acc[u][h][0], 0, 0, 0);
    }
    k_done = k_pairs;
  }
  // (the large tiles hold 4 + 2 operands and 8 accumulators a k-step, and two steps at a time fill the registers)
#pragma unroll 2
  for (int k0 = k_done; k0 < k_whole; k0 += 32) {
    moe_bf16x8 a[MT], b[U][W];
#pragma unroll
    for (int t = 0; t < MT; ++t) a[t] = *reinterpret_cast<const moe_bf16x8*>(a_ptr[t] + k0);
#pragma unroll
    for (int u = 0; u < U; ++u)
#pragma unroll
      for (int h = 0; h < W; ++h) b[u][h] = *reinterpret_cast<const moe_bf16x8*>(w_ptr[u][h] + k0);
#pragma unroll
    for (int u = 0; u < U; ++u)
#pragma unroll
      for (int h = 0; h < W; ++h)
#pragma unroll
        for (int t = 0; t < MT; ++t) acc[u][h][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(b[u][h], a[t], acc[u][h][t], 0, 0, 0);
  }
  if (k_whole < K) {                                         // the last, partial k-step: lanes whose eight elements lie beyond K hold zeros
    const bool in = k_whole + 8 * g < K;
    const moe_bf16x8 zero = {0, 0, 0, 0, 0, 0, 0, 0};
    moe_bf16x8 a[MT], b[U][W];
#pragma unroll
    for (int t = 0; t < MT; ++t) a[t] = in ? *reinterpret_cast<const moe_bf16x8*>(a_ptr[t] + k_whole) : zero;
#pragma unroll
    for (int u = 0; u < U; ++u)
#pragma unroll
      for (int h = 0; h < W; ++h) b[u][h] = in ? *reinterpret_cast<const moe_bf16x8*>(w_ptr[u][h] + k_whole) : zero;
#pragma unroll
    for (int u = 0; u < U; ++u)
#pragma unroll
      for (int h = 0; h < W; ++h)
#pragma unroll
        for (int t = 0; t < MT; ++t) acc[u][h][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(b[u][h], a[t], acc[u][h][t], 0, 0, 0);
  }
  // a lane's four sums: outputs 4 g .. 4 g + 3 of its block, for row r of every row tile
#pragma unroll
  for (int t = 0; t < MT; ++t) {
    const int row = t * 16 + r;
    if (row >= nrows) continue;
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int col = (block0 + u) * 16 + 4 * g;
      if (col >= n_out) continue;
      if (GATED) {
        bf16* o = reinterpret_cast<bf16*>(out_) + (size_t)(row0 + row) * ld_out + col;
        const float ps = pair_scale ? pair_scale[sorted_pair[row0 + row]] : 1.f;      // a factor on the pair's input row
#pragma unroll
        for (int i = 0; i < 4; ++i)
          if (col + i < n_out) o[i] = from_f32<bf16>(gate_activation(acc[u][0][t][i] * ps, act) * (acc[u][W - 1][t][i] * ps));
      } else {
        float* o = reinterpret_cast<float*>(out_) + (size_t)(row0 + row) * ld_out + col;
        if (col + 3 < n_out && (ld_out & 3) == 0) {
          *reinterpret_cast<float4*>(o) = make_float4(acc[u][0][t][0], acc[u][0][t][1], acc[u][0][t][2], acc[u][0][t][3]);
        } else {
#pragma unroll
          for (int i = 0; i < 4; ++i)
            if (col + i < n_out) o[i] = acc[u][0][t][i];
        }
      }
    }
  }
}

// Steps of so few pairs that the kernel above would leave most compute units without a workgroup (one request: `top`
// tiles of one row each): a workgroup is one tile of 16 rows times ONE block of 16 outputs, and its four wavefronts cut
// K between them in quarters that are multiples of 64; each streams its part of the 16 (gated: 32) weight rows as the
// kernel above does, two k-steps at a time, and the quarters' sums meet in LDS, where the first wavefront adds them in
// the quarters' order and stores.  Four times the wavefronts for the same bytes.  An output is the sum of four
// accumulators instead of one, so it may differ from the other kernels' in the last place; which kernel runs depends
// on the step's number of pairs alone.
template <bool GATED>
__global__ __launch_bounds__(256) void moe_expert_splitk_kernel(const bf16* __restrict__ rows_in, int ld_in, const bf16* __restrict__ w,
                                                                const int* __restrict__ tiles, const int* __restrict__ sorted_pair, int top,
                                                                int n_out, int K, void* __restrict__ out_, int ld_out, int act,
                                                                const float* __restrict__ pair_scale) {
  constexpr int W = GATED ? 2 : 1;
  __shared__ float part[3][W][4][64];
  const int tile = blockIdx.x;
  const int expert = tiles[3 * tile], row0 = tiles[3 * tile + 1], nrows = tiles[3 * tile + 2];
  if (nrows <= 0) return;                                    // the whole workgroup: no barrier is left behind
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int r = lane & 15, g = lane >> 4;
  const int block0 = blockIdx.y;
  const int row = row0 + min(r, nrows - 1);                  // rows past the tile's last repeat it: never stored
  const bf16* a_ptr = rows_in + (size_t)(GATED ? sorted_pair[row] / top : row) * ld_in + 8 * g;
  const bf16* we = w + (size_t)expert * W * n_out * K;
  const int col_r = min(block0 * 16 + r, n_out - 1);         // outputs past the last repeat it: never stored
  const bf16* w_ptr[W];
#pragma unroll
  for (int h = 0; h < W; ++h) w_ptr[h] = we + ((size_t)h * n_out + col_r) * K + 8 * g;
  const int quarter = ((K + 3) / 4 + 63) & ~63;
  const int k_begin = min(K, wave * quarter), k_end = min(K, k_begin + quarter);
  moe_floatx4 acc[W];
#pragma unroll
  for (int h = 0; h < W; ++h) acc[h] = moe_floatx4{0.f, 0.f, 0.f, 0.f};
  const int k_pairs = k_begin + ((k_end - k_begin) & ~63);
#pragma unroll 4
  for (int k0 = k_begin; k0 < k_pairs; k0 += 64) {
    moe_bf16x8 a[2], b[W][2];
#pragma unroll
    for (int half = 0; half < 2; ++half) {
      a[half] = *reinterpret_cast<const moe_bf16x8*>(a_ptr + k0 + 8 * g + 8 * half);
#pragma unroll
      for (int h = 0; h < W; ++h) b[h][half] = *reinterpret_cast<const moe_bf16x8*>(w_ptr[h] + k0 + 8 * g + 8 * half);
    }
#pragma unroll
    for (int half = 0; half < 2; ++half)
#pragma unroll
      for (int h = 0; h < W; ++h) acc[h] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(b[h][half], a[half], acc[h], 0, 0, 0);
  }
  // what is left of the last quarter: at most one whole k-step of 32 and a partial one (lanes beyond K hold zeros)
  for (int k0 = k_pairs; k0 < k_end; k0 += 32) {
    const bool in = k0 + 8 * g < k_end;
    const moe_bf16x8 zero = {0, 0, 0, 0, 0, 0, 0, 0};
    const moe_bf16x8 a = in ? *reinterpret_cast<const moe_bf16x8*>(a_ptr + k0) : zero;
#pragma unroll
    for (int h = 0; h < W; ++h) {
      const moe_bf16x8 b = in ? *reinterpret_cast<const moe_bf16x8*>(w_ptr[h] + k0) : zero;
      acc[h] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(b, a, acc[h], 0, 0, 0);
    }
  }
  if (wave > 0) {
#pragma unroll
    for (int h = 0; h < W; ++h)
#pragma unroll
      for (int i = 0; i < 4; ++i) part[wave - 1][h][i][lane] = acc[h][i];
  }
  __syncthreads();
  if (wave > 0) return;
#pragma unroll
  for (int q = 0; q < 3; ++q)
#pragma unroll
    for (int h = 0; h < W; ++h)
#pragma unroll
      for (int i = 0; i < 4; ++i) acc[h][i] += part[q][h][i][lane];
  // a lane's four sums: outputs 4 g .. 4 g + 3 of the block, for row r
  if (r >= nrows) return;
  const int col = block0 * 16 + 4 * g;
  if (col >= n_out) return;
  if (GATED) {
    bf16* o = reinterpret_cast<bf16*>(out_) + (size_t)(row0 + r) * ld_out + col;
    const float ps = pair_scale ? pair_scale[sorted_pair[row0 + r]] : 1.f;
#pragma unroll
    for (int i = 0; i < 4; ++i)
      if (col + i < n_out) o[i] = from_f32<bf16>(gate_activation(acc[0][i] * ps, act) * (acc[W - 1][i] * ps));
  } else {
    float* o = reinterpret_cast<float*>(out_) + (size_t)(row0 + r) * ld_out + col;
#pragma unroll
    for (int i = 0; i < 4; ++i)
      if (col + i < n_out) o[i] = acc[0][i];
  }
}

// Prompt steps with 128 pairs or more per expert: a workgroup is a tile of 128 rows of one expert times 128 weight rows
// (gated: 64 of the gate's and the 64 of the up product that belong to them), staged through LDS in k-steps of 64, two
// buffers deep: every thread fetches eight pieces of 16 bytes of the steps ahead into registers while the matrix cores
// work on this one, and stores a step's pieces behind the products of the step before; one barrier a step, which waits
// for LDS stores only.  LDS holds blocks of 16 rows x 32 elements (1 KB) in
// the operand's order with a row's four pieces XOR-ed by the row's quarter, so that a wavefront's fetch of an operand
// meets no bank twice.  A wavefront owns 64 x 64 of the tile: 4 + 4 operands and 16 matrix instructions per 32
// elements of k.  The sums run over ascending k in one accumulator per output, as in the kernel above.
constexpr int kBigRows = 128;

// A workgroup barrier that waits for this wavefront's LDS stores and nothing else: loads from memory that are under way
// stay under way across it (a barrier with a fence in front waits for them all, and with them for the steps asked for ahead).
__device__ __forceinline__ void tile_barrier() {
  __builtin_amdgcn_s_waitcnt(0xC07F);                         // lgkmcnt(0); vmcnt and expcnt as they are
  asm volatile("s_barrier" ::: "memory");
}

template <bool GATED>
__global__ __launch_bounds__(256) void moe_expert_tile_kernel(const bf16* __restrict__ rows_in, int ld_in, const bf16* __restrict__ w,
                                                              const int* __restrict__ tiles, const int* __restrict__ sorted_pair, int top,
                                                              int n_out, int K, void* __restrict__ out_, int ld_out, int act,
                                                              const float* __restrict__ pair_scale) {
  __shared__ __attribute__((aligned(16))) unsigned char lds[2][2][2][8 * 1024];   // [buffer][rows | weights][half of the k-step][8 blocks]
  const int tile = blockIdx.x;
  const int expert = tiles[3 * tile], row0 = tiles[3 * tile + 1], nrows = tiles[3 * tile + 2];
  if (nrows <= 0) return;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int n0 = blockIdx.y * (GATED ? 64 : 128);            // this workgroup's first output
  const bf16* we = w + (size_t)expert * (GATED ? 2 : 1) * n_out * K;
  // as a loader: pieces tid and tid + 256 of each 8 KB (block p / 64; row (p % 64) / 4 and piece p % 4 of the block)
  const bf16* a_src[2];
  const bf16* b_src[2];
  int put[2], piece_k;
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const int p = tid + 256 * i, b = p >> 6, lr = (p & 63) >> 2, lg = p & 3;
    const int rr = row0 + min(b * 16 + lr, nrows - 1);       // rows past the tile's last repeat it: never stored
    a_src[i] = rows_in + (size_t)(GATED ? sorted_pair[rr] / top : rr) * ld_in + lg * 8;
    const int col = GATED ? min(n0 + (b & 3) * 16 + lr, n_out - 1) + (b >> 2) * n_out : min(n0 + b * 16 + lr, n_out - 1);
    b_src[i] = we + (size_t)col * K + lg * 8;
    put[i] = b * 1024 + (lr * 4 + (lg ^ ((lr >> 2) & 3))) * 16;
  }
  piece_k = (tid & 3) * 8;
  typedef moe_bf16x8 piece_t;
  // Three sets of registers: the pieces of step s + 1 were asked for two steps ago and go into LDS behind the products
  // of step s, those of steps s + 2 and s + 3 are under way.  (Measured the same as one step under way: what bounds the
  // kernel is the 32 KB that a workgroup draws from the L2 per step, 1.7 GB a call at width 2,048 and 2,048 tokens.)
  piece_t fetched[3][2][2][2];                               // [set][rows | weights][half][i]
  const piece_t zero = {0, 0, 0, 0, 0, 0, 0, 0};
  auto fetch = [&](piece_t (&set)[2][2][2], int k0) {
#pragma unroll
    for (int kh = 0; kh < 2; ++kh) {
      const int k = k0 + kh * 32;
      const bool in = k + piece_k < K;                        // K % 8 == 0: a piece lies inside or outside
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        set[0][kh][i] = in ? *reinterpret_cast<const piece_t*>(a_src[i] + k) : zero;
        set[1][kh][i] = in ? *reinterpret_cast<const piece_t*>(b_src[i] + k) : zero;
      }
    }
  };
  auto store = [&](const piece_t (&set)[2][2][2], int buf) {
#pragma unroll
    for (int o = 0; o < 2; ++o)
#pragma unroll
      for (int kh = 0; kh < 2; ++kh)
#pragma unroll
        for (int i = 0; i < 2; ++i) *reinterpret_cast<piece_t*>(&lds[buf][o][kh][put[i]]) = set[o][kh][i];
  };
  const int r = lane & 15, g = lane >> 4, wm = wave >> 1, wn = wave & 1;
  const int take = (r * 4 + (g ^ ((r >> 2) & 3))) * 16;     // where this lane's operand lies in a block
  int a_blk[4], b_blk[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    a_blk[j] = (wm * 4 + j) * 1024 + take;
    b_blk[j] = (GATED ? ((j >> 1) * 4 + wn * 2 + (j & 1)) : (wn * 4 + j)) * 1024 + take;
  }
  moe_floatx4 acc[4][4];                                     // [weights' block][rows' block]
#pragma unroll
  for (int j = 0; j < 4; ++j)
#pragma unroll
    for (int t = 0; t < 4; ++t) acc[j][t] = moe_floatx4{0.f, 0.f, 0.f, 0.f};
  auto products = [&](int buf) {
#pragma unroll
    for (int kh = 0; kh < 2; ++kh) {
      piece_t a[4], b[4];
#pragma unroll
      for (int t = 0; t < 4; ++t) a[t] = *reinterpret_cast<const piece_t*>(&lds[buf][0][kh][a_blk[t]]);
#pragma unroll
      for (int j = 0; j < 4; ++j) b[j] = *reinterpret_cast<const piece_t*>(&lds[buf][1][kh][b_blk[j]]);
#pragma unroll
      for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int t = 0; t < 4; ++t) acc[j][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(b[j], a[t], acc[j][t], 0, 0, 0);
    }
  };
  const int steps = (K + 63) / 64;
  fetch(fetched[0], 0);
  if (steps > 1) fetch(fetched[1], 64);
  if (steps > 2) fetch(fetched[2], 128);
  store(fetched[0], 0);
  tile_barrier();
  // step s: ask for step s + 3 into the set that step s came from, multiply step s, put step s + 1 into the other buffer
#define PLLM_TILE_STEP(S, FREE_SET, NEXT_SET)                         \
  {                                                                   \
    if ((S) + 3 < steps) fetch(fetched[FREE_SET], ((S) + 3) * 64);    \
    products((S) & 1);                                                \
    if ((S) + 1 < steps) store(fetched[NEXT_SET], ((S) + 1) & 1);     \
    tile_barrier();                                                  \
  }
  for (int s3 = 0; s3 < steps; s3 += 3) {
    PLLM_TILE_STEP(s3, 0, 1)
    if (s3 + 1 < steps) PLLM_TILE_STEP(s3 + 1, 1, 2)
    if (s3 + 2 < steps) PLLM_TILE_STEP(s3 + 2, 2, 0)
  }
#undef PLLM_TILE_STEP
  // a lane's four sums: outputs 4 g .. 4 g + 3 of a weights' block, for row r of a rows' block
#pragma unroll
  for (int t = 0; t < 4; ++t) {
    const int row = wm * 64 + t * 16 + r;
    if (row >= nrows) continue;
    if (GATED) {
      const float ps = pair_scale ? pair_scale[sorted_pair[row0 + row]] : 1.f;        // a factor on the pair's input row
#pragma unroll
      for (int j = 0; j < 2; ++j) {
        const int col = n0 + wn * 32 + j * 16 + 4 * g;
        bf16* o = reinterpret_cast<bf16*>(out_) + (size_t)(row0 + row) * ld_out + col;
#pragma unroll
        for (int i = 0; i < 4; ++i)
          if (col + i < n_out) o[i] = from_f32<bf16>(gate_activation(acc[j][t][i] * ps, act) * (acc[j + 2][t][i] * ps));
      }
    } else {
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int col = n0 + wn * 64 + j * 16 + 4 * g;
        if (col >= n_out) continue;
        float* o = reinterpret_cast<float*>(out_) + (size_t)(row0 + row) * ld_out + col;
        if (col + 3 < n_out && (ld_out & 3) == 0) {
          *reinterpret_cast<float4*>(o) = make_float4(acc[j][t][0], acc[j][t][1], acc[j][t][2], acc[j][t][3]);
        } else {
#pragma unroll
          for (int i = 0; i < 4; ++i)
            if (col + i < n_out) o[i] = acc[j][t][i];
        }
      }
    }
  }
}

constexpr int kSplitBelowWorkgroups = 256;                   // the compute units of the GPU this is written for

template <bool GATED>
static void launch_moe_mfma(int tile_rows, int max_tiles, int pairs, const bf16* rows_in, int ld_in, const bf16* w, const int* tiles,
                            const int* sorted_pair, int top, int n_out, int K, void* out, int ld_out, int act, const float* pair_scale,
                            hipStream_t stream) {
  const int blocks = (n_out + 15) / 16;
  if (tile_rows >= kBigRows) {
    dim3 grid(max_tiles, GATED ? (n_out + 63) / 64 : (n_out + 127) / 128);
    hipLaunchKernelGGL((moe_expert_tile_kernel<GATED>), grid, dim3(256), 0, stream, rows_in, ld_in, w, tiles, sorted_pair, top, n_out, K, out, ld_out, act, pair_scale);
  } else if (tile_rows >= 64) {
    constexpr int U = GATED ? 1 : 2;
    dim3 grid(max_tiles, (blocks + 4 * U - 1) / (4 * U));
    hipLaunchKernelGGL((moe_expert_mfma_kernel<GATED, 4, U>), grid, dim3(256), 0, stream, rows_in, ld_in, w, tiles, sorted_pair, top, n_out, K, out, ld_out, act, pair_scale);
  } else if ((long)min(pairs, max_tiles) * ((blocks + 3) / 4) < kSplitBelowWorkgroups && K >= 256) {
    // at most `pairs` tiles hold a row: too few workgroups of the kernel below to reach every compute unit
    dim3 grid(max_tiles, blocks);
    hipLaunchKernelGGL((moe_expert_splitk_kernel<GATED>), grid, dim3(256), 0, stream, rows_in, ld_in, w, tiles, sorted_pair, top, n_out, K, out, ld_out, act, pair_scale);
  } else {
    dim3 grid(max_tiles, (blocks + 3) / 4);
    hipLaunchKernelGGL((moe_expert_mfma_kernel<GATED, 1, 1>), grid, dim3(256), 0, stream, rows_in, ld_in, w, tiles, sorted_pair, top, n_out, K, out, ld_out, act, pair_scale);
  }
}

// pair_scale (gated product only, or null): a factor per pair, indexed like the ids, by which the pair's input row counts
// as multiplied (it is applied to the gate's and the up product's float sums).
// tile_rows: what moe_align was given.  Tiles of more than 16 rows are for the matrix-core kernel alone (bfloat16,
// K and ld_in multiples of 8, 16-byte aligned operands); the plain kernel takes tiles of 16.
// pairs: how many (token, choice) pairs the tiles hold between them (no more than that many tiles hold a row).
PLLM_API int pllm_moe_expert_gemm(int dtype, int gated, const void* rows_in, int ld_in, const void* w, const int* tiles, int max_tiles,
                                  int tile_rows, const int* sorted_pair, int pairs, int top, int n_out, int K, void* out, int ld_out, int act,
                                  const float* pair_scale, hipStream_t stream) {
  if (max_tiles <= 0) return 0;
  if (n_out <= 0 || K <= 0 || top <= 0 || pairs < 0 || act < 0 || act >= PLLM_ACT_COUNT) return -2;
  const bool matrix_cores = dtype == PLLM_BF16 && K % 8 == 0 && ld_in % 8 == 0 && ((uintptr_t)rows_in & 15) == 0 && ((uintptr_t)w & 15) == 0;
  if (tile_rows != kMoeTileRows && !(matrix_cores && (tile_rows == 64 || tile_rows == kMoeMaxTileRows))) return -2;
  if (matrix_cores) {
    if (gated) launch_moe_mfma<true>(tile_rows, max_tiles, pairs, (const bf16*)rows_in, ld_in, (const bf16*)w, tiles, sorted_pair, top, n_out, K, out, ld_out, act, pair_scale, stream);
    else launch_moe_mfma<false>(tile_rows, max_tiles, pairs, (const bf16*)rows_in, ld_in, (const bf16*)w, tiles, sorted_pair, top, n_out, K, out, ld_out, act, pair_scale, stream);
    PLLM_RETURN_LAST_ERROR();
  }
  dim3 grid(max_tiles, (n_out + kMoeCols - 1) / kMoeCols), block(256);
#define PLLM_MOE(T, G)                                                                                                         \
  hipLaunchKernelGGL((moe_expert_gemm_kernel<T, G>), grid, block, 0, stream, (const T*)rows_in, ld_in, (const T*)w, tiles,    \
                     sorted_pair, top, n_out, K, out, ld_out, act, pair_scale)
  if (dtype == PLLM_F32) { if (gated) PLLM_MOE(float, true); else PLLM_MOE(float, false); }
  else { if (gated) PLLM_MOE(bf16, true); else PLLM_MOE(bf16, false); }
#undef PLLM_MOE
  PLLM_RETURN_LAST_ERROR();
}

// ---------------------------------------------------------------------------------------------
// out[t, :] = sum_k weights[t, k] * (row_of_pair[t, k] >= 0 ? expert_out[row_of_pair[t, k], :] : h[t, :]), in the order of k;
// weights_inside: the experts' rows count once (their weight went into their input), only a pass-through row takes its weight.
// shared (float [tokens, width], or null): + shared[t, :] * (shared_gate ? sigmoid(shared_gate[t * gate_ld]) : 1), a feed-forward
// that every token passes, with one gate per token.
template <typename T>
__global__ __launch_bounds__(256) void moe_combine_kernel(const float* __restrict__ expert_out, const T* __restrict__ h, int ld_h,
                                                          const int* __restrict__ row_of_pair, const float* __restrict__ weights,
                                                          int weights_inside, const float* __restrict__ shared,
                                                          const float* __restrict__ shared_gate, int gate_ld,
                                                          int top, int width, float* __restrict__ out) {
  const int t = blockIdx.x;
  const float sg = shared ? (shared_gate ? 1.f / (1.f + expf(-shared_gate[(size_t)t * gate_ld])) : 1.f) : 0.f;
  for (int i = threadIdx.x; i < width; i += blockDim.x) {
    float acc = 0.f;
    for (int k = 0; k < top; ++k) {
      const int row = row_of_pair[(size_t)t * top + k];
      const float v = row >= 0 ? expert_out[(size_t)row * width + i] : to_f32(h[(size_t)t * ld_h + i]);
      if (weights_inside && row >= 0) acc += v;
      else acc = fmaf(weights[(size_t)t * top + k], v, acc);
    }
    if (shared) acc = fmaf(sg, shared[(size_t)t * width + i], acc);
    out[(size_t)t * width + i] = acc;
  }
}

PLLM_API int pllm_moe_combine(int dtype, const float* expert_out, const void* h, int ld_h, const int* row_of_pair, const float* weights,
                              int weights_inside, const float* shared, const float* shared_gate, int gate_ld,
                              int num_tokens, int top, int width, float* out, hipStream_t stream) {
  if (num_tokens <= 0) return 0;
  dim3 grid(num_tokens), block(256);
  if (dtype == PLLM_F32)
    hipLaunchKernelGGL(moe_combine_kernel<float>, grid, block, 0, stream, expert_out, (const float*)h, ld_h, row_of_pair, weights,
                       weights_inside, shared, shared_gate, gate_ld, top, width, out);
  else
    hipLaunchKernelGGL(moe_combine_kernel<bf16>, grid, block, 0, stream, expert_out, (const bf16*)h, ld_h, row_of_pair, weights,
                       weights_inside, shared, shared_gate, gate_ld, top, width, out);
  PLLM_RETURN_LAST_ERROR();
}
