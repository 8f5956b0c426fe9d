// A mixture of experts: every token goes through `top` of `experts` small gated feed-forward layers.
//   * `ts_moe_route`: router logits z = W_r h in 32-bit (h as it is stored), scores s = sigmoid(z); the `top`
//     experts with the largest s + correction are chosen (ties: the lower index); their weights are their s,
//     divided by the chosen ones' sum (+ 1e-20) if `normalize`, times `scale`. With `softmax_chosen` the logits
//     themselves are the scores, and the weights are the softmax over the chosen experts' logits alone. With
//     `scoring` 2 the scores are the softmax over all the router's outputs. The router may have `extras` more rows
//     than experts: their logits' sigmoids are left beside the choice (a gate on a shared expert, say).
//   * `ts_moe_group`: the step's (token, choice) pairs grouped by expert, and the groups cut into tiles of rows
//     that one workgroup of the product takes: [expert, first index, rows] per tile, rows 0 for the tiles of the
//     launch that the step does not fill (the launch is sized for the worst case, so nothing comes back to the host).
//   * `ts_moe_gemm`: for every tile, rows of the operand (a token's row, or a pair's) times the tile's expert's
//     matrix; with `glu` the matrix holds gate rows, then up rows, and the capped gated unit
//     g = min(gate, L), u = clamp(up, -L, L), y = g sigmoid(slope g) (u + shift) leaves instead of the sums.
//     Without `glu`, `act` 1 squares the sums' positive parts on their way out (experts of the form W_down relu(W_up h)^2).
//     Every row's sums run over k in ascending order whatever the tile it lands in.
//   * `ts_moe_combine`: out[token] = sum over its choices, in order, of weight * the pair's row (+ a shared
//     expert's row, times a gate per token if there is one). A choice at or beyond `real` is an identity expert: it
//     has no matrices, `ts_moe_group` leaves its pairs out of every tile, and its row is the token's input itself.
// float32 runs 32-bit multiply-adds; bfloat16 operands go through the matrix cores with 32-bit sums.
#include "common.h"

#define MOE_THREADS 256
#define MOE_ROUTE_TOKENS 4
#define MOE_MAX_EXPERTS 1024
#define MOE_MAX_TOP 32

#define MOE_ROUTE_CHUNK 2048      // elements of a token's row that lie in LDS at a time
#define MOE_ROUTE_THREADS 1024    // sixteen waves: an expert each at a time, so that a step of few tokens has all its loads in flight at once

template <typename TX>
__global__ void __launch_bounds__(MOE_ROUTE_THREADS)
moe_route_kernel(int32_t* __restrict__ ids_out, float* __restrict__ w_out, const TX* __restrict__ x,
                 const float* __restrict__ router, const float* __restrict__ correction, int num_tokens, int K, int E, int top,
                 float scale, int normalize, int scoring, int extras, float* __restrict__ extra_out) {
  const bool softmax_chosen = scoring == 1;
  const int rows = E + extras;                            // rows of the router: the experts, then the extras
  extern __shared__ float lds[];
  float* s_s = lds;                                       // [MOE_ROUTE_TOKENS][rows] logits, then scores
  float* c_s = lds + MOE_ROUTE_TOKENS * rows;             // [MOE_ROUTE_TOKENS][rows] choice scores
  float* x_s = c_s + MOE_ROUTE_TOKENS * rows;                // [MOE_ROUTE_TOKENS][MOE_ROUTE_CHUNK] the tokens' rows, 32-bit
  const int wave = threadIdx.x / TS_WAVE, lane = threadIdx.x & (TS_WAVE - 1);
  const int t0 = blockIdx.x * MOE_ROUTE_TOKENS;
  const int nt = min(MOE_ROUTE_TOKENS, num_tokens - t0);
  for (int i = threadIdx.x; i < MOE_ROUTE_TOKENS * rows; i += MOE_ROUTE_THREADS) s_s[i] = 0.f;
  const bool by4 = K % 4 == 0 && ((uintptr_t)router & 15) == 0;     // (rows of the router in 16-byte pieces)
  // a stretch of the rows into LDS, then every wave takes experts in turn: a lane reads the router's row side by
  // side with its neighbours, all of a stretch's pieces asked for before the first is used
  for (int k0 = 0; k0 < K; k0 += MOE_ROUTE_CHUNK) {
    const int kn = min(MOE_ROUTE_CHUNK, K - k0);
    __syncthreads();
#pragma unroll 8
    for (int i = threadIdx.x; i < MOE_ROUTE_TOKENS * kn; i += MOE_ROUTE_THREADS) {
      const int r = i / kn, k = i - r * kn;
      x_s[r * MOE_ROUTE_CHUNK + k] = r < nt ? Num<TX>::ld(x + (int64_t)(t0 + r) * K + k0 + k) : 0.f;
    }
    __syncthreads();
    for (int e = wave; e < rows; e += MOE_ROUTE_THREADS / TS_WAVE) {
      float acc[MOE_ROUTE_TOKENS];
#pragma unroll
      for (int r = 0; r < MOE_ROUTE_TOKENS; ++r) acc[r] = 0.f;
      const float* wr = router + (int64_t)e * K + k0;
      if (by4) {
        constexpr int PIECES = MOE_ROUTE_CHUNK / (4 * TS_WAVE);
        float4 w[PIECES];
#pragma unroll
        for (int i = 0; i < PIECES; ++i) {
          const int k = 4 * (lane + TS_WAVE * i);
          w[i] = k < kn ? *(const float4*)(wr + k) : make_float4(0.f, 0.f, 0.f, 0.f);
        }
#pragma unroll
        for (int i = 0; i < PIECES; ++i) {
          const int k = 4 * (lane + TS_WAVE * i);
          if (k >= kn) continue;
#pragma unroll
          for (int r = 0; r < MOE_ROUTE_TOKENS; ++r) {
            const float4 xv = *(const float4*)(x_s + r * MOE_ROUTE_CHUNK + k);
            acc[r] = fmaf(w[i].x, xv.x, fmaf(w[i].y, xv.y, fmaf(w[i].z, xv.z, fmaf(w[i].w, xv.w, acc[r]))));
          }
        }
      } else {
#pragma unroll 8
        for (int k = lane; k < kn; k += TS_WAVE) {
          const float w = wr[k];
#pragma unroll
          for (int r = 0; r < MOE_ROUTE_TOKENS; ++r) acc[r] = fmaf(w, x_s[r * MOE_ROUTE_CHUNK + k], acc[r]);
        }
      }
#pragma unroll
      for (int r = 0; r < MOE_ROUTE_TOKENS; ++r) {
        const float z = wave_sum(acc[r]);
        if (lane == 0) s_s[r * rows + e] += z;                // (an expert is one wave's: no other adds to it)
      }
    }
  }
  __syncthreads();
  for (int i = threadIdx.x; i < MOE_ROUTE_TOKENS * rows; i += MOE_ROUTE_THREADS) {
    const int e = i % rows;
    const float sc = (softmax_chosen || (scoring == 2 && e < E)) ? s_s[i] : 1.0f / (1.0f + expf(-s_s[i]));
    s_s[i] = sc;
    c_s[i] = sc + ((correction && e < E) ? correction[e] : 0.f);
  }
  __syncthreads();
  if (wave >= nt) return;                                 // a wave per token from here on
  const int r = wave, t = t0 + wave;
  s_s += r * rows;
  c_s += r * rows;
  if (extras && lane < extras) extra_out[(int64_t)t * extras + lane] = s_s[E + lane];
  if (scoring == 2) {                                     // the softmax over all the experts' logits
    float top_logit = -INFINITY;
    for (int e = lane; e < E; e += TS_WAVE) top_logit = fmaxf(top_logit, s_s[e]);
    top_logit = wave_max(top_logit);
    float total = 0.f;
    for (int e = lane; e < E; e += TS_WAVE) total += expf(s_s[e] - top_logit);
    total = wave_sum(total);
    wave_sync();
    for (int e = lane; e < E; e += TS_WAVE) {
      const float sc = expf(s_s[e] - top_logit) / total;
      s_s[e] = sc;
      c_s[e] = sc + (correction ? correction[e] : 0.f);
    }
    wave_sync();
  }
  // lane j keeps the j-th choice (top <= 32 lanes of the 64)
  float my_pick = 0.f;
  int my_choice = 0;
  for (int j = 0; j < top; ++j) {
    float best = -INFINITY;
    int at = 0x7fffffff;
    for (int e = lane; e < E; e += TS_WAVE) {
      const float c = c_s[e];
      if (c > best) { best = c; at = e; }                 // (ascending e: the lower index wins a tie)
    }
#pragma unroll
    for (int off = TS_WAVE / 2; off > 0; off >>= 1) {
      const float ob = __shfl_xor(best, off, TS_WAVE);
      const int oa = __shfl_xor(at, off, TS_WAVE);
      if (ob > best || (ob == best && oa < at)) { best = ob; at = oa; }
    }
    if (at >= E) at = j;                                  // (scores that are no numbers: still valid indices)
    if (lane == j) { my_choice = at; my_pick = s_s[at]; }
    wave_sync();
    if (lane == 0) c_s[at] = -INFINITY;
    wave_sync();
  }
  if (softmax_chosen) {                                   // the chosen logits' softmax: the first choice is the largest
    const float top_logit = __shfl(my_pick, 0, TS_WAVE);
    my_pick = lane < top ? expf(my_pick - top_logit) : 0.f;
  }
  const float total = wave_sum(my_pick);                  // (the lanes beyond `top` hold 0)
  const float mult = (softmax_chosen ? 1.0f / total : normalize ? 1.0f / (total + 1e-20f) : 1.0f) * scale;
  if (lane < top) {
    ids_out[(int64_t)t * top + lane] = my_choice;
    w_out[(int64_t)t * top + lane] = my_pick * mult;
  }
}

extern "C" int ts_moe_route(int32_t* ids_out, float* w_out, const void* x, int x_dtype, const float* router,
                            const float* correction, int num_tokens, int K, int E, int top, float scale, int normalize,
                            int scoring, int extras, float* extra_out, hipStream_t stream) {
  if (num_tokens <= 0) return TS_OK;
  if (K <= 0 || E <= 0 || E > MOE_MAX_EXPERTS || top <= 0 || top > MOE_MAX_TOP || top > E || scoring < 0 || scoring > 2 ||
      extras < 0 || extras > TS_WAVE || (extras && !extra_out))
    return TS_BAD_SHAPE;
  const unsigned blocks = (num_tokens + MOE_ROUTE_TOKENS - 1) / MOE_ROUTE_TOKENS;
  const size_t lds = (size_t)MOE_ROUTE_TOKENS * (2 * (E + extras) + MOE_ROUTE_CHUNK) * sizeof(float);
  if (x_dtype == 0)
    moe_route_kernel<float><<<blocks, MOE_ROUTE_THREADS, lds, stream>>>(ids_out, w_out, (const float*)x, router, correction,
                                                                        num_tokens, K, E, top, scale, normalize, scoring, extras, extra_out);
  else if (x_dtype == 1)
    moe_route_kernel<bf16_t><<<blocks, MOE_ROUTE_THREADS, lds, stream>>>(ids_out, w_out, (const bf16_t*)x, router, correction,
                                                                         num_tokens, K, E, top, scale, normalize, scoring, extras, extra_out);
  else return TS_BAD_DTYPE;
  return ts_check_launch();
}

// One workgroup: counts per expert, their running sums, the tiles, then every pair into its expert's stretch.
#define MOE_GROUP_THREADS 1024
__global__ void __launch_bounds__(MOE_GROUP_THREADS)
moe_group_kernel(const int32_t* __restrict__ ids, int32_t* __restrict__ sorted, int32_t* __restrict__ tiles, int P, int E,
                 int tile_rows, int max_tiles) {
  __shared__ int count_s[MOE_MAX_EXPERTS];
  __shared__ int first_s[MOE_MAX_EXPERTS + 1];
  __shared__ int tile_s[MOE_MAX_EXPERTS + 1];
  for (int e = threadIdx.x; e < E; e += MOE_GROUP_THREADS) count_s[e] = 0;
  __syncthreads();
  for (int p = threadIdx.x; p < P; p += MOE_GROUP_THREADS)
    if (ids[p] < E) atomicAdd(&count_s[ids[p]], 1);          // (a choice beyond the experts with matrices: an identity expert, in no tile)
  __syncthreads();
  if (threadIdx.x == 0) {
    int first = 0, tile = 0;
    for (int e = 0; e < E; ++e) {
      first_s[e] = first;
      tile_s[e] = tile;
      first += count_s[e];
      tile += (count_s[e] + tile_rows - 1) / tile_rows;
    }
    first_s[E] = first;
    tile_s[E] = tile;
  }
  __syncthreads();
  for (int e = threadIdx.x; e < E; e += MOE_GROUP_THREADS) {
    const int n = count_s[e];
    for (int i = 0, tile = tile_s[e]; i < n && tile < max_tiles; i += tile_rows, ++tile) {
      tiles[3 * tile] = e;
      tiles[3 * tile + 1] = first_s[e] + i;
      tiles[3 * tile + 2] = min(tile_rows, n - i);
    }
  }
  for (int tile = tile_s[E] + threadIdx.x; tile < max_tiles; tile += MOE_GROUP_THREADS) {
    tiles[3 * tile] = 0;
    tiles[3 * tile + 1] = 0;
    tiles[3 * tile + 2] = 0;
  }
  // every pair into its expert's stretch, in the order the threads come by (a row's sums do not depend on its
  // place in a tile, so the order inside an expert changes no result)
  __syncthreads();
  for (int e = threadIdx.x; e < E; e += MOE_GROUP_THREADS) count_s[e] = 0;
  __syncthreads();
  for (int p = threadIdx.x; p < P; p += MOE_GROUP_THREADS) {
    const int e = ids[p];
    if (e < E) sorted[first_s[e] + atomicAdd(&count_s[e], 1)] = p;
  }
}

extern "C" int ts_moe_group(const int32_t* ids, int32_t* sorted, int32_t* tiles, int P, int E, int tile_rows, int max_tiles,
                            hipStream_t stream) {
  if (P <= 0) return TS_OK;
  // (tiles of a step: at most P / tile_rows full ones and one partly filled per expert that has pairs)
  if (E <= 0 || E > MOE_MAX_EXPERTS || tile_rows <= 0 || max_tiles < P / tile_rows + (E < P ? E : P)) return TS_BAD_SHAPE;
  moe_group_kernel<<<1, MOE_GROUP_THREADS, 0, stream>>>(ids, sorted, tiles, P, E, tile_rows, max_tiles);
  return ts_check_launch();
}

#define MOE_BM 16
#define MOE_DIES 8
#define MOE_BN 64
#define MOE_KC 32

// What an ungated expert's sums pass on their way out: 0 nothing, 1 the square of relu.
static __device__ __forceinline__ float moe_act(float s, int act) {
  if (act == 1) { const float r = fmaxf(s, 0.f); return r * r; }
  return s;
}

static __device__ __forceinline__ float moe_unit(float g, float u, float limit, float slope, float shift) {
  if (limit > 0.f) {
    g = fminf(g, limit);
    u = fminf(fmaxf(u, -limit), limit);
  }
  return g / (1.0f + expf(-slope * g)) * (u + shift);
}

// Plain 32-bit multiply-adds: a tile of up to 16 rows by 64 columns a workgroup; thread (column, row quarter).
template <typename TX, typename TO>
__global__ void __launch_bounds__(MOE_THREADS)
moe_gemm_kernel(TO* __restrict__ out, const TX* __restrict__ x, const TX* __restrict__ w, const int32_t* __restrict__ sorted,
                const int32_t* __restrict__ tiles, int src_div, int N, int K, int glu, float limit, float slope, float shift, int act) {
  __shared__ float x_s[MOE_BM][MOE_KC + 1];
  __shared__ float w_s[2][MOE_BN][MOE_KC + 1];
  __shared__ int row_s[MOE_BM];
  const int tile = blockIdx.x;
  const int rows = tiles[3 * tile + 2];
  if (rows == 0) return;
  const int e = tiles[3 * tile], first = tiles[3 * tile + 1];
  const int n0 = blockIdx.y * MOE_BN;
  const int tx = threadIdx.x & (MOE_BN - 1), ty = threadIdx.x / MOE_BN;
  if (threadIdx.x < MOE_BM) row_s[threadIdx.x] = threadIdx.x < rows ? sorted[first + threadIdx.x] : -1;
  __syncthreads();
  const int64_t expert_rows = glu ? 2 * (int64_t)N : N;
  const TX* we = w + (int64_t)e * expert_rows * K;
  float acc[4] = {0.f, 0.f, 0.f, 0.f}, acc2[4] = {0.f, 0.f, 0.f, 0.f};
  for (int k0 = 0; k0 < K; k0 += MOE_KC) {
    for (int i = threadIdx.x; i < MOE_BM * MOE_KC; i += MOE_THREADS) {
      const int r = i / MOE_KC, kk = i - r * MOE_KC;
      const int p = row_s[r];
      x_s[r][kk] = (p >= 0 && k0 + kk < K) ? Num<TX>::ld(x + (int64_t)(p / src_div) * K + k0 + kk) : 0.f;
    }
    for (int i = threadIdx.x; i < MOE_BN * MOE_KC; i += MOE_THREADS) {
      const int c = i / MOE_KC, kk = i - c * MOE_KC;
      const bool in = n0 + c < N && k0 + kk < K;
      w_s[0][c][kk] = in ? Num<TX>::ld(we + (int64_t)(n0 + c) * K + k0 + kk) : 0.f;
      if (glu) w_s[1][c][kk] = in ? Num<TX>::ld(we + (int64_t)(N + n0 + c) * K + k0 + kk) : 0.f;
    }
    __syncthreads();
#pragma unroll 8
    for (int kk = 0; kk < MOE_KC; ++kk) {
      const float wv = w_s[0][tx][kk];
      const float wu = glu ? w_s[1][tx][kk] : 0.f;
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const float xv = x_s[ty * 4 + r][kk];
        acc[r] = fmaf(xv, wv, acc[r]);
        acc2[r] = fmaf(xv, wu, acc2[r]);
      }
    }
    __syncthreads();
  }
  if (n0 + tx >= N) return;
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    const int p = row_s[ty * 4 + r];
    if (p < 0) continue;
    const float y = glu ? moe_unit(acc[r], acc2[r], limit, slope, shift) : moe_act(acc[r], act);
    Num<TO>::st(out + (int64_t)p * N + n0 + tx, y);
  }
}

// bfloat16 on the matrix cores: a workgroup of four waves takes a tile's rows (TM blocks of 16) by 4 x TN x 16
// columns, each wave TN column blocks of all the rows. Operands go from memory straight into the instruction's
// registers: lane (r, g) holds eight consecutive k of row r of a block, 16 bytes, for the rows of x (gathered by
// pair) as for the rows of the expert's matrix. The product is formed as y^T = W x^T, which leaves a lane four
// consecutive columns of one row of y. With GLU a lane holds a gate sum and its up sum side by side and stores
// the unit. K is a multiple of 32; a tile's missing rows and a matrix's missing columns are computed on
// repeated rows and not stored.
typedef uint32_t moe_u32x4 __attribute__((ext_vector_type(4)));
typedef __bf16 moe_bf16x8 __attribute__((ext_vector_type(8)));
typedef float moe_f32x4 __attribute__((ext_vector_type(4)));

static __device__ __forceinline__ moe_f32x4 moe_mfma(moe_u32x4 a, moe_u32x4 b, moe_f32x4 acc) {
  return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(moe_bf16x8, a), __builtin_bit_cast(moe_bf16x8, b), acc, 0, 0, 0);
}

// Four adjacent columns of a row, `left` of which exist: one store where all do and the place is whole pieces.
static __device__ __forceinline__ void moe_store4(float* p, const float (&y)[4], int left) {
  if (left >= 4 && ((uintptr_t)p & 15) == 0) { *(float4*)p = make_float4(y[0], y[1], y[2], y[3]); return; }
  for (int c = 0; c < 4 && c < left; ++c) p[c] = y[c];
}
static __device__ __forceinline__ void moe_store4(bf16_t* p, const float (&y)[4], int left) {
  if (left >= 4 && ((uintptr_t)p & 7) == 0) {
    uint2 v;
    v.x = (uint32_t)f2bf(y[0]) | ((uint32_t)f2bf(y[1]) << 16);
    v.y = (uint32_t)f2bf(y[2]) | ((uint32_t)f2bf(y[3]) << 16);
    *(uint2*)p = v;
    return;
  }
  for (int c = 0; c < 4 && c < left; ++c) p[c] = f2bf(y[c]);
}

template <int TM, int TN, bool GLU, typename TO>
__global__ void __launch_bounds__(MOE_THREADS)
moe_gemm_mfma_kernel(TO* __restrict__ out, const bf16_t* __restrict__ x, const bf16_t* __restrict__ w,
                     const int32_t* __restrict__ sorted, const int32_t* __restrict__ tiles, int src_div, int N, int K,
                     float limit, float slope, float shift, int act) {
  constexpr int SETS = GLU ? 2 : 1;
  const int tile = blockIdx.x;
  const int rows = tiles[3 * tile + 2];
  if (rows == 0) return;
  const int e = tiles[3 * tile], first = tiles[3 * tile + 1];
  const int wave = threadIdx.x / TS_WAVE, lane = threadIdx.x & (TS_WAVE - 1);
  const int r = lane & 15, g = lane >> 4;
  const int n0 = (blockIdx.y * 4 + wave) * TN * 16;
  if (n0 >= N) return;
  const int64_t expert_rows = GLU ? 2 * (int64_t)N : N;
  const bf16_t* we = w + (int64_t)e * expert_rows * K;
  int pair[TM];
  const bf16_t* xp[TM];
  const bf16_t* wp[SETS][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i) {
    pair[i] = sorted[first + min(16 * i + r, rows - 1)];
    xp[i] = x + (int64_t)(pair[i] / src_div) * K + 8 * g;
  }
#pragma unroll
  for (int j = 0; j < TN; ++j) {
    const int col = min(n0 + 16 * j + r, N - 1);
    wp[0][j] = we + (int64_t)col * K + 8 * g;
    if constexpr (GLU) wp[1][j] = we + (int64_t)(N + col) * K + 8 * g;
  }
  moe_f32x4 acc[SETS][TN][TM];
#pragma unroll
  for (int s = 0; s < SETS; ++s)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int i = 0; i < TM; ++i) acc[s][j][i] = (moe_f32x4){0.f, 0.f, 0.f, 0.f};
  for (int k0 = 0; k0 < K; k0 += 32) {
    moe_u32x4 fx[TM], fw[SETS][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i) fx[i] = *(const moe_u32x4*)(xp[i] + k0);
#pragma unroll
    for (int s = 0; s < SETS; ++s)
#pragma unroll
      for (int j = 0; j < TN; ++j) fw[s][j] = *(const moe_u32x4*)(wp[s][j] + k0);
#pragma unroll
    for (int s = 0; s < SETS; ++s)
#pragma unroll
      for (int j = 0; j < TN; ++j)
#pragma unroll
        for (int i = 0; i < TM; ++i) acc[s][j][i] = moe_mfma(fw[s][j], fx[i], acc[s][j][i]);
  }
  // lane (r, g) of block (j, i): row 16 i + r of the tile, columns n0 + 16 j + 4 g .. + 3
#pragma unroll
  for (int i = 0; i < TM; ++i) {
    if (16 * i + r >= rows) continue;
    TO* orow = out + (int64_t)pair[i] * N;
#pragma unroll
    for (int j = 0; j < TN; ++j) {
      const int col = n0 + 16 * j + 4 * g;
      float y[4];
#pragma unroll
      for (int c = 0; c < 4; ++c) {
        if constexpr (GLU) y[c] = moe_unit(acc[0][j][i][c], acc[1][j][i][c], limit, slope, shift);
        else y[c] = moe_act(acc[0][j][i][c], act);
      }
      moe_store4(orow + col, y, N - col);
    }
  }
}

// Tiles of 16 rows, for steps of few tokens, where the experts' matrices are streamed once and nothing else counts:
// a workgroup takes a tile's rows by 16 columns (with GLU: 16 gate and 16 up columns), and its four waves take a
// quarter of K each, four k-steps' loads in flight at a time, so that a step with one token still has a thousand
// waves asking for memory. The quarters' sums meet through LDS and are added in the waves' order: a row's result
// depends on K alone, not on the tile or the batch it lands in.
template <bool GLU, typename TO>
__global__ void __launch_bounds__(MOE_THREADS)
moe_gemm_stream_kernel(TO* __restrict__ out, const bf16_t* __restrict__ x, const bf16_t* __restrict__ w,
                       const int32_t* __restrict__ sorted, const int32_t* __restrict__ tiles, int src_div, int N, int K,
                       float limit, float slope, float shift, int act) {
  constexpr int SETS = GLU ? 2 : 1;
  constexpr int WAVES = MOE_THREADS / TS_WAVE, DEPTH = 4;
  __shared__ moe_f32x4 part_s[WAVES - 1][SETS][TS_WAVE];
  const int tile = blockIdx.x;
  const int rows = tiles[3 * tile + 2];
  if (rows == 0) return;
  const int e = tiles[3 * tile], first = tiles[3 * tile + 1];
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / TS_WAVE), lane = threadIdx.x & (TS_WAVE - 1);
  const int r = lane & 15, g = lane >> 4;
  const int n0 = blockIdx.y * 16;
  const int64_t expert_rows = GLU ? 2 * (int64_t)N : N;
  const bf16_t* we = w + (int64_t)e * expert_rows * K;
  const int pair = sorted[first + min(r, rows - 1)];
  const int col = min(n0 + r, N - 1);
  const int steps = K / 32, s0 = wave * steps / WAVES, s1 = (wave + 1) * steps / WAVES;
  const bf16_t* xp = x + (int64_t)(pair / src_div) * K + 8 * g;
  const bf16_t* wp[SETS];
  wp[0] = we + (int64_t)col * K + 8 * g;
  if constexpr (GLU) wp[1] = we + (int64_t)(N + col) * K + 8 * g;
  moe_f32x4 acc[SETS];
#pragma unroll
  for (int s = 0; s < SETS; ++s) acc[s] = (moe_f32x4){0.f, 0.f, 0.f, 0.f};
  int s = s0;
  for (; s + DEPTH <= s1; s += DEPTH) {
    moe_u32x4 fx[DEPTH], fw[SETS][DEPTH];
#pragma unroll
    for (int d = 0; d < DEPTH; ++d) {
      fx[d] = *(const moe_u32x4*)(xp + 32 * (s + d));
#pragma unroll
      for (int t = 0; t < SETS; ++t) fw[t][d] = *(const moe_u32x4*)(wp[t] + 32 * (s + d));
    }
#pragma unroll
    for (int d = 0; d < DEPTH; ++d)
#pragma unroll
      for (int t = 0; t < SETS; ++t) acc[t] = moe_mfma(fw[t][d], fx[d], acc[t]);
  }
  for (; s < s1; ++s) {
    const moe_u32x4 fx = *(const moe_u32x4*)(xp + 32 * s);
#pragma unroll
    for (int t = 0; t < SETS; ++t) acc[t] = moe_mfma(*(const moe_u32x4*)(wp[t] + 32 * s), fx, acc[t]);
  }
  if (wave > 0) {
#pragma unroll
    for (int t = 0; t < SETS; ++t) part_s[wave - 1][t][lane] = acc[t];
  }
  __syncthreads();
  if (wave > 0) return;
#pragma unroll
  for (int v = 0; v < WAVES - 1; ++v)
#pragma unroll
    for (int t = 0; t < SETS; ++t) acc[t] += part_s[v][t][lane];
  // lane (r, g): row r of the tile, columns n0 + 4 g .. + 3
  if (r >= rows) return;
  TO* orow = out + (int64_t)pair * N;
  const int c0 = n0 + 4 * g;
  float y[4];
#pragma unroll
  for (int c = 0; c < 4; ++c) {
    if constexpr (GLU) y[c] = moe_unit(acc[0][c], acc[1][c], limit, slope, shift);
    else y[c] = moe_act(acc[0][c], act);
  }
  moe_store4(orow + c0, y, N - c0);
}

// Tiles of 128 rows, for steps that give an expert hundreds of rows: both operands go through LDS, fetched a whole
// 128-byte line of a row by eight threads side by side and read from LDS as the matrix instruction wants them (lane
// (r, g) of block b and half h: row 16 b + r, elements 32 h + 8 g .. + 7),
// 64 of K at a time, two k-steps in flight (one in an LDS buffer being multiplied, the next in registers on its way
// into the other buffer), as in the engine's tiled product for plain matrices; here the rows of x are gathered by
// pair, the matrix is the tile's expert's, and the rows of y go to their pairs' places. A workgroup of WM x WN
// waves takes 128 rows by 128 columns (with GLU: 64 gate and 64 up columns, whose sums meet in one lane). K is a
// multiple of 64.
template <int WM, int WN, bool GLU, typename TO>
__global__ void __launch_bounds__(WM * WN * TS_WAVE)
moe_gemm_lds_kernel(TO* __restrict__ out, const bf16_t* __restrict__ x, const bf16_t* __restrict__ w,
                    const int32_t* __restrict__ sorted, const int32_t* __restrict__ tiles, int num_tiles, int col_blocks,
                    int src_div, int N, int K, float limit, float slope, float shift, int act) {
  constexpr int BM = 128, BN = 128;
  constexpr int THREADS = WM * WN * TS_WAVE;
  constexpr int FX = BM / 16 * 2, FW = BN / 16 * 2;       // fragments (a kilobyte each) of a k-step of 64
  constexpr int TM = BM / WM / 16, TN = BN / WN / 16;     // 16 x 16 blocks of a wave
  constexpr int LX = FX * 64 / THREADS, LW = FW * 64 / THREADS;
  static_assert(!GLU || WN == 1, "a gate sum and its up sum must meet in one wave");
  __shared__ moe_u32x4 lds[2][(FX + FW) * 64];
  // Workgroups go to the chip's eight dies in turn, each die with a cache of its own: die d takes the d-th eighth
  // of the (tile, column block) list, column blocks innermost and tiles in the experts' order, so that the
  // workgroups a die runs at one time share a few tiles' rows and one expert's columns in its cache.
  const int per_die = gridDim.x / MOE_DIES;
  const int item = (blockIdx.x % MOE_DIES) * per_die + blockIdx.x / MOE_DIES;
  if (item >= num_tiles * col_blocks) return;
  const int tile = item / col_blocks;
  const int rows = tiles[3 * tile + 2];
  if (rows == 0) return;
  const int e = tiles[3 * tile], first = tiles[3 * tile + 1];
  // (with GLU a workgroup's 128 columns of the product are 64 columns of y)
  const int n0 = (item - tile * col_blocks) * (GLU ? BN / 2 : BN);
  const int t = threadIdx.x, lane = t % TS_WAVE, r = lane % 16, g = lane / 16;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / TS_WAVE), wm = wave % WM, wn = wave / WM;
  const bf16_t* we = w + (int64_t)e * (GLU ? 2 : 1) * N * K;
  const bf16_t* xp[LX];
  const bf16_t* wp[LW];
  // (fetching: eight threads side by side take the eight 16-byte pieces of one row's 64 k, a whole line of memory)
  int place[LX > LW ? LX : LW];
#pragma unroll
  for (int i = 0; i < LX; ++i) {
    const int row = (t + THREADS * i) / 8, piece = (t + THREADS * i) % 8;
    const int pair = sorted[first + min(row, rows - 1)];
    xp[i] = x + (int64_t)(pair / src_div) * K + 8 * piece;
  }
#pragma unroll
  for (int i = 0; i < LW; ++i) {
    const int row = (t + THREADS * i) / 8, piece = (t + THREADS * i) % 8;
    int col = row;
    if (GLU) col = min(n0 + col % (BN / 2), N - 1) + (col >= BN / 2 ? N : 0);
    else col = min(n0 + col, N - 1);
    wp[i] = we + (int64_t)col * K + 8 * piece;
  }
  // (in LDS row R keeps its piece c at place c ^ (R % 8): the eight threads that store a row fill its 128 bytes, and the
  // lanes that read one piece of eight rows in a row for the matrix instruction find them in eight different places)
  static_assert(LX == LW, "as many pieces of x as of the matrix a thread");
#pragma unroll
  for (int i = 0; i < LX; ++i) {
    const int row = (t + THREADS * i) / 8, piece = (t + THREADS * i) % 8;
    place[i] = row * 8 + (piece ^ (row & 7));
  }
  moe_u32x4 sx0[LX], sw0[LW], sx1[LX], sw1[LW];
  moe_f32x4 acc[TN][TM];
#pragma unroll
  for (int j = 0; j < TN; ++j)
#pragma unroll
    for (int i = 0; i < TM; ++i) acc[j][i] = (moe_f32x4){0.f, 0.f, 0.f, 0.f};
#define MOE_FETCH(S, k0)                                                                                  \
  do {                                                                                                    \
    _Pragma("unroll") for (int i = 0; i < LX; ++i) sx##S[i] = *(const moe_u32x4*)(xp[i] + (k0));          \
    _Pragma("unroll") for (int i = 0; i < LW; ++i) sw##S[i] = *(const moe_u32x4*)(wp[i] + (k0));          \
  } while (0)
#define MOE_STASH(S)                                                                                      \
  do {                                                                                                    \
    _Pragma("unroll") for (int i = 0; i < LX; ++i) lds[S][place[i]] = sx##S[i];                           \
    _Pragma("unroll") for (int i = 0; i < LW; ++i) lds[S][FX * 64 + place[i]] = sw##S[i];                 \
  } while (0)
#define MOE_MULTIPLY(S)                                                                                   \
  _Pragma("unroll") for (int h = 0; h < 2; ++h) {                                                         \
    moe_u32x4 fx[TM], fw[TN];                                                                             \
    _Pragma("unroll") for (int i = 0; i < TM; ++i)                                                        \
      fx[i] = lds[S][((wm * TM + i) * 16 + r) * 8 + ((4 * h + g) ^ (r & 7))];                             \
    _Pragma("unroll") for (int j = 0; j < TN; ++j)                                                        \
      fw[j] = lds[S][FX * 64 + ((wn * TN + j) * 16 + r) * 8 + ((4 * h + g) ^ (r & 7))];                   \
    _Pragma("unroll") for (int j = 0; j < TN; ++j)                                                        \
      _Pragma("unroll") for (int i = 0; i < TM; ++i) acc[j][i] = moe_mfma(fw[j], fx[i], acc[j][i]);       \
  }
  const int steps = K / 64;
  MOE_FETCH(0, 0);
  if (steps == 1) {
    MOE_STASH(0);
    __syncthreads();
    MOE_MULTIPLY(0)
  } else {
    MOE_FETCH(1, 64);
    MOE_STASH(0);
    __syncthreads();
    int s = 0;
    for (; s + 3 < steps; s += 2) {
      MOE_FETCH(0, 64 * (s + 2));
      MOE_MULTIPLY(0)
      MOE_STASH(1);
      __syncthreads();
      MOE_FETCH(1, 64 * (s + 3));
      MOE_MULTIPLY(1)
      MOE_STASH(0);
      __syncthreads();
    }
    // two or three steps are left: step s in buffer 0, step s + 1 in register set 1
    if (steps - s == 3) {
      MOE_FETCH(0, 64 * (s + 2));
      MOE_MULTIPLY(0)
      MOE_STASH(1);
      __syncthreads();
      MOE_MULTIPLY(1)
      MOE_STASH(0);
      __syncthreads();
      MOE_MULTIPLY(0)
    } else {
      MOE_MULTIPLY(0)
      MOE_STASH(1);
      __syncthreads();
      MOE_MULTIPLY(1)
    }
  }
#undef MOE_FETCH
#undef MOE_STASH
#undef MOE_MULTIPLY
  // lane (r, g) of block (j, i): row 16 (wm TM + i) + r of the tile, columns .. + 4 g .. + 3
#pragma unroll
  for (int i = 0; i < TM; ++i) {
    const int m = (wm * TM + i) * 16 + r;
    if (m >= rows) continue;
    TO* orow = out + (int64_t)sorted[first + m] * N;
    if constexpr (GLU) {
#pragma unroll
      for (int j = 0; j < TN / 2; ++j) {
        const int n = n0 + j * 16 + 4 * g;
        float y[4];
#pragma unroll
        for (int c = 0; c < 4; ++c) y[c] = moe_unit(acc[j][i][c], acc[j + TN / 2][i][c], limit, slope, shift);
        moe_store4(orow + n, y, N - n);
      }
    } else {
#pragma unroll
      for (int j = 0; j < TN; ++j) {
        const int n = n0 + (wn * TN + j) * 16 + 4 * g;
        const float y[4] = {moe_act(acc[j][i][0], act), moe_act(acc[j][i][1], act), moe_act(acc[j][i][2], act), moe_act(acc[j][i][3], act)};
        moe_store4(orow + n, y, N - n);
      }
    }
  }
}

extern "C" int ts_moe_gemm(void* out, int out_dtype, const void* x, int x_dtype, const void* w, const int32_t* sorted,
                           const int32_t* tiles, int max_tiles, int tile_rows, int src_div, int N, int K, int glu, float limit,
                           float slope, float shift, int act, hipStream_t stream) {
  if (max_tiles <= 0) return TS_OK;
  if (act < 0 || act > 1 || (glu && act)) return TS_BAD_SHAPE;
  if (N <= 0 || K <= 0 || src_div <= 0 || (tile_rows != 16 && tile_rows != 64 && tile_rows != 128)) return TS_BAD_SHAPE;
  const bool mfma = x_dtype == 1 && K % 32 == 0 && (((uintptr_t)x | (uintptr_t)w) & 15) == 0;
  if (tile_rows == 128) {
    if (!mfma || K % 64) return TS_BAD_SHAPE;
    const int col_blocks = glu ? (N + 63) / 64 : (N + 127) / 128;
    const int64_t items = (int64_t)max_tiles * col_blocks;
    if (items > 0x3fffffff) return TS_BAD_SHAPE;
    const unsigned grid = (unsigned)((items + MOE_DIES - 1) / MOE_DIES * MOE_DIES);
#define MOE_LDS(WM, WN, GLU, TO) \
    moe_gemm_lds_kernel<WM, WN, GLU, TO><<<grid, WM * WN * TS_WAVE, 0, stream>>>((TO*)out, (const bf16_t*)x, (const bf16_t*)w, sorted, \
                                                                                  tiles, max_tiles, col_blocks, src_div, N, K, limit, slope, shift, act)
    if (glu && out_dtype == 1) MOE_LDS(4, 1, true, bf16_t);
    else if (!glu && out_dtype == 0) MOE_LDS(2, 2, false, float);
    else if (!glu && out_dtype == 1) MOE_LDS(2, 2, false, bf16_t);
    else return TS_BAD_DTYPE;
#undef MOE_LDS
    return ts_check_launch();
  }
  if (mfma) {
    if (tile_rows == 16) {
      dim3 grid(max_tiles, (N + 15) / 16);
      if (grid.y > 65535) return TS_BAD_SHAPE;
#define MOE_STREAM(GLU, TO) \
      moe_gemm_stream_kernel<GLU, TO><<<grid, MOE_THREADS, 0, stream>>>((TO*)out, (const bf16_t*)x, (const bf16_t*)w, sorted, tiles, \
                                                                        src_div, N, K, limit, slope, shift, act)
      if (glu && out_dtype == 1) MOE_STREAM(true, bf16_t);
      else if (!glu && out_dtype == 0) MOE_STREAM(false, float);
      else if (!glu && out_dtype == 1) MOE_STREAM(false, bf16_t);
      else return TS_BAD_DTYPE;
#undef MOE_STREAM
      return ts_check_launch();
    }
    // (a wave takes 32 columns of all the tile's rows; with the gate, 32 gate and 32 up columns)
    dim3 grid(max_tiles, (N + 127) / 128);
    if (grid.y > 65535) return TS_BAD_SHAPE;
#define MOE_MFMA(TM, GLU, TO) \
    moe_gemm_mfma_kernel<TM, 2, GLU, TO><<<grid, MOE_THREADS, 0, stream>>>((TO*)out, (const bf16_t*)x, (const bf16_t*)w, sorted, \
                                                                           tiles, src_div, N, K, limit, slope, shift, act)
    if (glu && out_dtype == 1) MOE_MFMA(4, true, bf16_t);
    else if (!glu && out_dtype == 0) MOE_MFMA(4, false, float);
    else if (!glu && out_dtype == 1) MOE_MFMA(4, false, bf16_t);
    else return TS_BAD_DTYPE;
#undef MOE_MFMA
    return ts_check_launch();
  }
  if (tile_rows != MOE_BM) return TS_BAD_SHAPE;
  dim3 grid(max_tiles, (N + MOE_BN - 1) / MOE_BN);
  if (grid.y > 65535) return TS_BAD_SHAPE;
#define MOE_LAUNCH(TX, TO) \
  moe_gemm_kernel<TX, TO><<<grid, MOE_THREADS, 0, stream>>>((TO*)out, (const TX*)x, (const TX*)w, sorted, tiles, src_div, N, K, \
                                                            glu, limit, slope, shift, act)
  if (x_dtype == 0 && out_dtype == 0) MOE_LAUNCH(float, float);
  else if (x_dtype == 1 && out_dtype == 1) MOE_LAUNCH(bf16_t, bf16_t);
  else if (x_dtype == 1 && out_dtype == 0) MOE_LAUNCH(bf16_t, float);
  else return TS_BAD_DTYPE;
#undef MOE_LAUNCH
  return ts_check_launch();
}

// A thread per four columns of a token (or per column, where rows are no whole 16-byte pieces): a step of one token
// spreads over the row's width and waits for memory once.
template <int VEC, typename TX>
__global__ void __launch_bounds__(MOE_THREADS)
moe_combine_kernel(float* __restrict__ out, const float* __restrict__ rows, const float* __restrict__ weights,
                   const float* __restrict__ shared, int width, int top, const int32_t* __restrict__ ids, int real,
                   const TX* __restrict__ x, const float* __restrict__ shared_gate) {
  const int64_t t = blockIdx.x;
  const int i = (blockIdx.y * MOE_THREADS + threadIdx.x) * VEC;
  if (i >= width) return;
  float acc[VEC];
#pragma unroll
  for (int c = 0; c < VEC; ++c) acc[c] = 0.f;
  for (int j = 0; j < top; ++j) {
    const float w = weights[t * top + j];
    if (ids && ids[t * top + j] >= real) {                // an identity expert: the token's input itself
#pragma unroll
      for (int c = 0; c < VEC; ++c) acc[c] = fmaf(w, Num<TX>::ld(x + t * width + i + c), acc[c]);
      continue;
    }
    const float* row = rows + (t * top + j) * width + i;
    if constexpr (VEC == 4) {
      const float4 v = *(const float4*)row;
      acc[0] = fmaf(w, v.x, acc[0]); acc[1] = fmaf(w, v.y, acc[1]); acc[2] = fmaf(w, v.z, acc[2]); acc[3] = fmaf(w, v.w, acc[3]);
    } else {
      acc[0] = fmaf(w, row[0], acc[0]);
    }
  }
  const float g = shared_gate ? shared_gate[t] : 1.0f;
  if constexpr (VEC == 4) {
    if (shared) {
      const float4 v = *(const float4*)(shared + t * width + i);
      acc[0] = fmaf(g, v.x, acc[0]); acc[1] = fmaf(g, v.y, acc[1]); acc[2] = fmaf(g, v.z, acc[2]); acc[3] = fmaf(g, v.w, acc[3]);
    }
    *(float4*)(out + t * width + i) = make_float4(acc[0], acc[1], acc[2], acc[3]);
  } else {
    if (shared) acc[0] = fmaf(g, shared[t * width + i], acc[0]);
    out[t * width + i] = acc[0];
  }
}

extern "C" int ts_moe_combine(float* out, const float* rows, const float* weights, const float* shared, int num_tokens,
                              int width, int top, const int32_t* ids, int real, const void* x, int x_dtype,
                              const float* shared_gate, hipStream_t stream) {
  if (num_tokens <= 0) return TS_OK;
  if (width <= 0 || top <= 0 || (ids && !x) || (shared_gate && !shared)) return TS_BAD_SHAPE;
  if (x_dtype != 0 && x_dtype != 1) return TS_BAD_DTYPE;
  const bool by4 = width % 4 == 0 && (((uintptr_t)out | (uintptr_t)rows | (uintptr_t)shared) & 15) == 0;
  const int per_block = MOE_THREADS * (by4 ? 4 : 1);
  dim3 grid(num_tokens, (width + per_block - 1) / per_block);
  if (grid.y > 65535) return TS_BAD_SHAPE;
#define MOE_COMBINE(VEC, TX) \
  moe_combine_kernel<VEC, TX><<<grid, MOE_THREADS, 0, stream>>>(out, rows, weights, shared, width, top, ids, real, (const TX*)x, shared_gate)
  if (by4 && x_dtype == 0) MOE_COMBINE(4, float);
  else if (by4) MOE_COMBINE(4, bf16_t);
  else if (x_dtype == 0) MOE_COMBINE(1, float);
  else MOE_COMBINE(1, bf16_t);
#undef MOE_COMBINE
  return ts_check_launch();
}
