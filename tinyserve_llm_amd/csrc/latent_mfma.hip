// Multi-query attention over cached latent rows on the matrix cores (bfloat16 caches). A token's cached row is
// [c | r] (`rank` + `rot` numbers); the values are the rows' first `rank` numbers, which the cache also keeps once
// more, transposed inside its pages ([rank, page_size]), because the product P.V wants, for one dimension,
// consecutive keys side by side. All heads of a token share the keys, so the heads are the rows of the matrix
// products: a workgroup owns a tile of 16 rows (16 heads of one token, or all heads of several tokens of one
// request where a token has fewer than 16), its four waves (eight where the step has few tiles) walk the tile's keys in
// 32-key steps, each wave every fourth (eighth) step, with a running maximum and sum of their own, and add their parts up through shared memory, one wave
// after the other (the order of every sum is fixed).
//     S^T[key, row] = K[key, :] . Q[row, :]       v_mfma_f32_16x16x32_bf16, keys as rows, Q from shared memory
//     P = 2^(S scale log2 e - m), 32-bit, carried into the second product as two bfloat16 terms
//     O^T[dim, row] += V^T[dim, key] . P[row, key]
// Queries arrive 32-bit and are rounded to bfloat16 once, as the keys were. Scores, maxima, weights and sums are
// 32-bit. Causal, with a sliding window or chunks (`ts_first_key`).
#include "attention_mfma.h"

#define LM_ROWS 16
#define LM_FEW_TILES 512       // fewer workgroups than this: eight waves a tile instead of four

// NKS: 32-wide steps over a cached row that the kernel is built for (row <= 32 NKS); NVB: 16-wide blocks of the
// values (rank <= 16 NVB). Steps and blocks beyond the actual sizes are skipped by uniform branches.
template <int NKS, int NVB, int LM_WAVES, typename TO>
__global__ void __launch_bounds__(LM_WAVES * TS_WAVE)
latent_attention_mfma_kernel(TO* __restrict__ out, const float* __restrict__ q, const bf16_t* __restrict__ k_cache,
                             const bf16_t* __restrict__ v_cache, const int32_t* __restrict__ block_tables,
                             const int32_t* __restrict__ seq_of_token, const int32_t* __restrict__ positions,
                             const int32_t* __restrict__ tiles, int num_tiles, int tile_tokens, int nh, int rank, int row,
                             int64_t kp, int64_t ks, int64_t vp, int64_t vd, int max_blocks, float scale_log2, int window,
                             int page_run, int num_tokens) {
  constexpr int LM_THREADS = LM_WAVES * TS_WAVE;
  constexpr int QS = NKS * 32 + 8;                          // a row of the queries in shared memory, skewed
  __shared__ __attribute__((aligned(16))) bf16_t q_s[LM_ROWS][QS];
  __shared__ __attribute__((aligned(16))) float o_s[LM_ROWS][NVB * 16 + 4];
  __shared__ float m_s[LM_WAVES][LM_ROWS], l_s[LM_WAVES][LM_ROWS];
  // tiles that lie side by side in the step go to one die's second-level cache: they read the same keys
  const int per_die = (num_tiles + 7) / 8;
  const int tile = (blockIdx.x & 7) * per_die + (blockIdx.x >> 3);
  if (tile >= num_tiles) return;
  const int t0 = tiles ? tiles[2 * tile] : tile;
  const int count = tiles ? tiles[2 * tile + 1] : 1;
  const int hb = blockIdx.y;
  const int heads_here = min(nh - 16 * hb, 16);            // heads of a token in this tile
  const int wave = wave_index(), lane = threadIdx.x & (TS_WAVE - 1);
  const int r = lane & 15, g = lane >> 4;
  const int nks = (row + 31) / 32, nvb = rank / 16;
  // row i of the tile: token t0 + i / heads_here, head 16 hb + i % heads_here
  const int my_tok = r / heads_here, my_head = 16 * hb + r % heads_here;
  const bool my_valid = my_tok < count && my_tok < tile_tokens;
  const int pos0 = positions[t0];
  const int my_pos = my_valid ? pos0 + my_tok : -1;        // (a tile's tokens are consecutive positions of one request)
  const int my_lo = my_valid ? ts_first_key(my_pos, window) : 0;
  const int lo_min = ts_first_key(pos0, window), pos_max = pos0 + count - 1;
  const int32_t* table = block_tables + (int64_t)seq_of_token[t0] * max_blocks;

  // the tile's queries, rounded once, zeros where there is no row or no dimension
  for (int i = threadIdx.x; i < LM_ROWS * NKS * 32; i += LM_THREADS) {
    const int rr = i / (NKS * 32), d = i - rr * (NKS * 32);
    const int tok = rr / heads_here, head = 16 * hb + rr % heads_here;
    float v = 0.f;
    if (tok < count && tok < tile_tokens && d < row) v = q[((int64_t)(t0 + tok) * nh + head) * row + d];
    q_s[rr][d] = f2bf(v);
  }
  __syncthreads();

  float4_t acc[NVB];
#pragma unroll
  for (int db = 0; db < NVB; ++db) acc[db] = (float4_t){0.f, 0.f, 0.f, 0.f};
  float m = -INFINITY, l = 0.f;
  const int kb0 = lo_min & ~31;
  for (int kb = kb0 + 32 * wave; kb <= pos_max; kb += 32 * LM_WAVES) {
    // the step lies inside one page of the pool (pages of 32 keys)
    const int pg = kb >> 5;
    const int64_t page = ((int64_t)table[pg >> page_run] << page_run) + (pg & ((1 << page_run) - 1));
    const bf16_t* kbase = k_cache + page * kp;
    const bf16_t* vbase = v_cache + page * vp;
    // every lane loads, whatever its step and block, from an address inside the page (the row's last piece, the last
    // dimension's keys): loads under branches would be waited for one by one. What is read past the row's end meets
    // zeros of the queries; blocks past the values' end are not multiplied.
    uint4 kf[2][NKS], vf[NVB];
#pragma unroll
    for (int tau = 0; tau < 2; ++tau) {
      const bf16_t* krow = kbase + (int64_t)(8 * (r >> 2) + 4 * tau + (r & 3)) * ks;
#pragma unroll
      for (int c = 0; c < NKS; ++c) kf[tau][c] = *(const uint4*)(krow + min(32 * c + 8 * g, row - 8));
    }
#pragma unroll
    for (int db = 0; db < NVB; ++db) vf[db] = *(const uint4*)(vbase + (int64_t)min(16 * db + r, rank - 1) * vd + 8 * g);
    float s[8];
#pragma unroll
    for (int tau = 0; tau < 2; ++tau) {
      float4_t st = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int c = 0; c < NKS; ++c)
        if (c < nks) st = mfma32(kf[tau][c], *(const uint4*)&q_s[r][32 * c + 8 * g], st);
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int key = kb + 8 * g + 4 * tau + j;
        s[4 * tau + j] = (key >= my_lo && key <= my_pos) ? st[j] * scale_log2 : -INFINITY;
      }
    }
    float top = s[0];
#pragma unroll
    for (int j = 1; j < 8; ++j) top = fmaxf(top, s[j]);
    const float m_new = fmaxf(m, row_max(top));
    const float m_safe = m_new == -INFINITY ? 0.f : m_new;
    const float alpha = fast_exp2(m - m_safe);              // (m = -inf: nothing summed yet, and 2^-inf = 0)
    float p[8], sum = 0.f;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      p[j] = fast_exp2(s[j] - m_safe);
      sum += p[j];
    }
    l = l * alpha + sum;
    m = m_new;
    uint4 hi, lo;
    uint32_t* hw = (uint32_t*)&hi;
    uint32_t* lw = (uint32_t*)&lo;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      hw[j] = pack_bf16(p[2 * j], p[2 * j + 1]);
      const float r0 = p[2 * j] - __uint_as_float(hw[j] << 16), r1 = p[2 * j + 1] - __uint_as_float(hw[j] & 0xffff0000u);
      lw[j] = pack_bf16(r0, r1);
    }
#pragma unroll
    for (int db = 0; db < NVB; ++db)
      if (db < nvb) {
        float4_t a = acc[db];
#pragma unroll
        for (int j = 0; j < 4; ++j) a[j] *= alpha;
        a = mfma32(vf[db], hi, a);
        acc[db] = mfma32(vf[db], lo, a);
      }
  }
  // the four waves' parts: a common maximum, then the sums and the rows one wave after the other
  l = row_sum(l);
  if (g == 0) m_s[wave][r] = m;
  __syncthreads();
  float top = m_s[0][r];
#pragma unroll
  for (int w = 1; w < LM_WAVES; ++w) top = fmaxf(top, m_s[w][r]);
  const float top_safe = top == -INFINITY ? 0.f : top;
  const float mine = fast_exp2(m - top_safe);
  if (g == 0) l_s[wave][r] = l * mine;
  for (int w = 0; w < LM_WAVES; ++w) {
    if (wave == w) {
#pragma unroll
      for (int db = 0; db < NVB; ++db)
        if (db < nvb) {
          float* dst = &o_s[r][16 * db + 4 * g];
#pragma unroll
          for (int j = 0; j < 4; ++j) dst[j] = (w == 0 ? 0.f : dst[j]) + acc[db][j] * mine;
        }
    }
    __syncthreads();
  }
  for (int i = threadIdx.x; i < LM_ROWS * rank; i += LM_THREADS) {
    const int rr = i / rank, d = i - rr * rank;
    const int tok = rr / heads_here, head = 16 * hb + rr % heads_here;
    if (tok >= count || tok >= tile_tokens) continue;
    float total = 0.f;
#pragma unroll
    for (int w = 0; w < LM_WAVES; ++w) total += l_s[w][rr];
    Num<TO>::st(out + ((int64_t)(t0 + tok) * nh + head) * rank + d, o_s[rr][d] / total);
  }
}

// Whether the kernel is built for a cached row of `row` numbers of which `rank` are the values.
extern "C" int ts_latent_mfma_takes(int rank, int row) {
  return rank > 0 && rank % 16 == 0 && row % 8 == 0 && rank <= row && row <= 320 && rank <= 256;
}

// tiles: int32 [num_tiles, 2] (first token, token count <= tile_tokens), every tile inside one request, or null:
// every token a tile of its own. tile_tokens = max(1, 16 / heads) where a token has fewer than 16 heads.
extern "C" int ts_paged_attention_latent_mfma(void* out, int out_dtype, const float* q, const void* k_cache, const void* v_cache,
                                              const int32_t* block_tables, const int32_t* seq_of_token, const int32_t* positions,
                                              const int32_t* tiles, int num_tiles, int tile_tokens, int num_tokens, int nh, int rank,
                                              int rot, int page_size, int64_t kp, int64_t ks, int64_t vp, int64_t vd,
                                              int64_t v_slot, int max_blocks, float scale, int window, int page_run,
                                              hipStream_t stream) {
  if (num_tiles <= 0 || num_tokens <= 0) return TS_OK;
  const int row = rank + rot;
  if (!ts_latent_mfma_takes(rank, row) || nh <= 0 || page_size != 32 || v_slot != 1 || kp % 8 || ks % 8 || vp % 8 || vd % 8 ||
      ((uintptr_t)k_cache & 15) || ((uintptr_t)v_cache & 15) || max_blocks <= 0 || page_run < 0 || page_run > 16 ||
      tile_tokens < 1 || tile_tokens * min(nh, 16) > LM_ROWS || (nh > 16 && tile_tokens != 1) || (!tiles && num_tiles != num_tokens))
    return TS_BAD_SHAPE;
  dim3 grid(((num_tiles + 7) / 8) * 8, (nh + 15) / 16);
  const float scale_log2 = scale * 1.4426950408889634f;
  const bool few = (int64_t)grid.x * grid.y < LM_FEW_TILES;
#define LM_LAUNCH(NKS, NVB, TO) \
  if (few) LM_LAUNCH_W(NKS, NVB, 8, TO); else LM_LAUNCH_W(NKS, NVB, 4, TO)
#define LM_LAUNCH_W(NKS, NVB, W, TO) \
  latent_attention_mfma_kernel<NKS, NVB, W, TO><<<grid, W * TS_WAVE, 0, stream>>>((TO*)out, q, (const bf16_t*)k_cache, \
      (const bf16_t*)v_cache, block_tables, seq_of_token, positions, tiles, num_tiles, tile_tokens, nh, rank, row, kp, ks, vp, vd, \
      max_blocks, scale_log2, window, page_run, num_tokens)
#define LM_PICK(TO) \
  do { \
    if (row <= 160 && rank <= 128) { LM_LAUNCH(5, 8, TO); } \
    else { LM_LAUNCH(10, 16, TO); } \
  } while (0)
  if (out_dtype == 0) LM_PICK(float);
  else if (out_dtype == 1) LM_PICK(bf16_t);
  else return TS_BAD_DTYPE;
#undef LM_PICK
#undef LM_LAUNCH
#undef LM_LAUNCH_W
  return ts_check_launch();
}
