// Multi-query attention over cached latent rows on the matrix cores (bfloat16 caches). A token's cached row is
// [c | r] (`rank` + `rot` numbers); the values are the rows' first `rank` numbers, which the cache also keeps once
// more, transposed inside its pages ([rank, page_size]), because the product P.V wants, for one dimension,
// consecutive keys side by side. All heads of a token share the keys, so the heads are the rows of the matrix
// products: a workgroup owns a tile of 32 rows (32 heads of one token, or all heads of several tokens of one request
// where a token has fewer) and walks the tile's keys in 32-key steps. Its four waves split the dimensions, not the
// keys: a cached row is long, and a wave that held whole rows and whole value columns would have registers for
// nothing else. Of every step
//     S^T[key, row] = K[key, :] . Q[row, :]       v_mfma_f32_16x16x32_bf16, keys as rows, Q from shared memory:
//                                                 each wave sums over its quarter of the row's 32-wide pieces, the
//                                                 quarters meet in shared memory and every wave adds them in one order
//     P = 2^(S scale log2 e - m), 32-bit, the same in every wave; into the second product as two bfloat16 terms
//     O^T[dim, row] += V^T[dim, key] . P[row, key]  each wave its quarter of the value columns
// while the next step's keys and values are on their way. Where a step has few tiles (decoded tokens) the keys of a
// tile are cut into stretches, a workgroup each, whose parts (maximum, sum, unnormalised rows) a second kernel adds up.
// Queries arrive 32-bit and are rounded to bfloat16 once, as the keys were. Scores, maxima, weights and sums are
// 32-bit. Causal, with a sliding window or chunks (`ts_first_key`).
#include "attention_mfma.h"

#define LM_WAVES 4
#define LM_THREADS (LM_WAVES * TS_WAVE)
#define LM_RT 2                 // 16-row tiles of a workgroup
#define LM_ROWS (16 * LM_RT)
#define LM_MAX_SPLITS 16

// CPW: 32-wide pieces of a cached row per wave (row <= 128 CPW); VPW: 16-wide blocks of value columns per wave
// (rank <= 64 VPW). Wave w takes pieces w, w + 4, ... and blocks w, w + 4, ...; those past the actual sizes are loaded
// from a valid address (the row's last piece, the last column) and not multiplied.
template <int CPW, int VPW, typename TO>
__global__ void __launch_bounds__(LM_THREADS)
latent_attention_mfma_kernel(TO* __restrict__ out, float* __restrict__ part_o, float* __restrict__ part_ml,
                             const float* __restrict__ q, const bf16_t* __restrict__ k_cache, const bf16_t* __restrict__ v_cache,
                             const int32_t* __restrict__ block_tables, const int32_t* __restrict__ seq_of_token,
                             const int32_t* __restrict__ positions, const int32_t* __restrict__ tiles, int num_tiles,
                             int tile_tokens, int heads_block, int nh, int rank, int row, int64_t kp, int64_t ks, int64_t vp,
                             int64_t vd, int max_blocks, float scale_log2, int window, int page_run, int splits) {
  constexpr int QS = CPW * 128 + 8;                         // a row of the queries in shared memory, skewed
  __shared__ __attribute__((aligned(16))) bf16_t q_s[LM_ROWS][QS];
  __shared__ __attribute__((aligned(16))) float4_t s_part[2][LM_WAVES][LM_RT][2][TS_WAVE];
  // tiles that lie side by side in the step go to one die's second-level cache: they read the same keys
  const int per_die = (num_tiles + 7) / 8;
  const int tile = (blockIdx.x & 7) * per_die + (blockIdx.x >> 3);
  if (tile >= num_tiles) return;
  const int t0 = tiles ? tiles[2 * tile] : tile;
  const int count = tiles ? tiles[2 * tile + 1] : 1;
  const int hb = blockIdx.y, split = blockIdx.z;
  const int heads_here = min(nh - heads_block * hb, heads_block);      // heads of a token in this tile
  const int wave = wave_index(), lane = threadIdx.x & (TS_WAVE - 1);
  const int r = lane & 15, g = lane >> 4;
  const int nks = (row + 31) / 32, nvb = rank / 16;
  // row i of the tile: token t0 + i / heads_here, head heads_block hb + i % heads_here
  const int pos0 = positions[t0];
  int my_pos[LM_RT], my_lo[LM_RT];
#pragma unroll
  for (int rt = 0; rt < LM_RT; ++rt) {
    const int tok = (16 * rt + r) / heads_here;
    const bool valid = tok < count && tok < tile_tokens;
    my_pos[rt] = valid ? pos0 + tok : -1;                   // (a tile's tokens are consecutive positions of one request)
    my_lo[rt] = valid ? ts_first_key(my_pos[rt], window) : 0;
  }
  const int lo_min = ts_first_key(pos0, window), pos_max = pos0 + count - 1;
  const int32_t* table = block_tables + (int64_t)seq_of_token[t0] * max_blocks;

  // the tile's queries, rounded once, zeros where there is no row or no dimension. Every thread's loads go out
  // together, each from an address inside the step's queries (a row without a token reads the tile's first).
  __shared__ int64_t src_s[LM_ROWS];
  if (threadIdx.x < LM_ROWS) {
    const int tok = threadIdx.x / heads_here, head = heads_block * hb + threadIdx.x % heads_here;
    src_s[threadIdx.x] = (tok < count && tok < tile_tokens) ? ((int64_t)(t0 + tok) * nh + head) * row : -1;
  }
  __syncthreads();
  {
    constexpr int F4 = CPW * 32, PER = LM_ROWS * F4 / LM_THREADS;       // 16-byte pieces of a row; of a thread
    const int64_t fallback = ((int64_t)t0 * nh + heads_block * hb) * row;
    float4 got[PER];
#pragma unroll
    for (int it = 0; it < PER; ++it) {
      const int i = threadIdx.x + it * LM_THREADS, rr = i / F4, d = 4 * (i - rr * F4);
      const int64_t src = src_s[rr];
      got[it] = *(const float4*)(q + (src < 0 ? fallback : src) + min(d, row - 4));
    }
#pragma unroll
    for (int it = 0; it < PER; ++it) {
      const int i = threadIdx.x + it * LM_THREADS, rr = i / F4, d = 4 * (i - rr * F4);
      const bool in = src_s[rr] >= 0 && d < row;
      uint2 packed;
      packed.x = in ? pack_bf16(got[it].x, got[it].y) : 0u;
      packed.y = in ? pack_bf16(got[it].z, got[it].w) : 0u;
      *(uint2*)&q_s[rr][d] = packed;
    }
  }
  __syncthreads();

  float4_t acc[LM_RT][VPW];
#pragma unroll
  for (int rt = 0; rt < LM_RT; ++rt)
#pragma unroll
    for (int i = 0; i < VPW; ++i) acc[rt][i] = (float4_t){0.f, 0.f, 0.f, 0.f};
  float m[LM_RT], l[LM_RT];
#pragma unroll
  for (int rt = 0; rt < LM_RT; ++rt) m[rt] = -INFINITY, l[rt] = 0.f;
  // this workgroup's stretch of the tile's 32-key steps
  const int kb0 = lo_min & ~31;
  const int steps = ((pos_max - kb0) >> 5) + 1, per = (steps + splits - 1) / splits;
  const int first = split * per, last = min(steps, first + per) - 1;       // (an empty stretch: last < first)
  auto page_of = [&](int step) -> int64_t {                  // a step lies inside one page of the pool (pages of 32 keys)
    const int pg = (kb0 >> 5) + step;
    return ((int64_t)table[pg >> page_run] << page_run) + (pg & ((1 << page_run) - 1));
  };
  // every lane loads, whatever its piece and block, from an address inside the page: loads under branches would be
  // waited for one by one. What is read past the row's end meets zeros of the queries.
  auto load_keys = [&](uint4 (&kf)[2][CPW], int64_t page) {
#pragma unroll
    for (int tau = 0; tau < 2; ++tau) {
      const bf16_t* krow = k_cache + page * kp + (int64_t)(8 * (r >> 2) + 4 * tau + (r & 3)) * ks;
#pragma unroll
      for (int i = 0; i < CPW; ++i) kf[tau][i] = *(const uint4*)(krow + min(32 * (wave + LM_WAVES * i) + 8 * g, row - 8));
    }
  };
  auto load_values = [&](uint4 (&vf)[VPW], int64_t page) {
#pragma unroll
    for (int i = 0; i < VPW; ++i)
      vf[i] = *(const uint4*)(v_cache + page * vp + (int64_t)min(16 * (wave + LM_WAVES * i) + r, rank - 1) * vd + 8 * g);
  };
  uint4 kf[2][CPW], vf[VPW], kn[2][CPW], vn[VPW];
  if (first <= last) {
    const int64_t page = page_of(first);
    load_keys(kf, page);
    load_values(vf, page);
  }
  for (int step = first; step <= last; ++step) {
    const int64_t page_next = page_of(min(step + 1, last));  // (the last step asks for itself again)
    load_keys(kn, page_next);
    load_values(vn, page_next);
    const int kb = kb0 + 32 * step, par = (step - first) & 1;
#pragma unroll
    for (int rt = 0; rt < LM_RT; ++rt)
#pragma unroll
      for (int tau = 0; tau < 2; ++tau) {
        float4_t st = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int i = 0; i < CPW; ++i) {
          const int c = wave + LM_WAVES * i;
          if (c < nks) st = mfma32(kf[tau][i], *(const uint4*)&q_s[16 * rt + r][32 * c + 8 * g], st);
        }
        s_part[par][wave][rt][tau][lane] = st;
      }
    __syncthreads();                                         // (one a step: the next step writes the other half)
    uint4 hi[LM_RT], lo[LM_RT];
    float alpha[LM_RT];
#pragma unroll
    for (int rt = 0; rt < LM_RT; ++rt) {
      float s[8];
#pragma unroll
      for (int tau = 0; tau < 2; ++tau) {
        float4_t st = s_part[par][0][rt][tau][lane];
#pragma unroll
        for (int w = 1; w < LM_WAVES; ++w) {
          const float4_t o = s_part[par][w][rt][tau][lane];
#pragma unroll
          for (int j = 0; j < 4; ++j) st[j] += o[j];
        }
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const int key = kb + 8 * g + 4 * tau + j;
          s[4 * tau + j] = (key >= my_lo[rt] && key <= my_pos[rt]) ? st[j] * scale_log2 : -INFINITY;
        }
      }
      float top = s[0];
#pragma unroll
      for (int j = 1; j < 8; ++j) top = fmaxf(top, s[j]);
      const float m_new = fmaxf(m[rt], row_max(top));
      const float m_safe = m_new == -INFINITY ? 0.f : m_new;
      alpha[rt] = fast_exp2(m[rt] - m_safe);                 // (m = -inf: nothing summed yet, and 2^-inf = 0)
      float p[8], sum = 0.f;
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        p[j] = fast_exp2(s[j] - m_safe);
        sum += p[j];
      }
      l[rt] = l[rt] * alpha[rt] + sum;
      m[rt] = m_new;
      uint32_t* hw = (uint32_t*)&hi[rt];
      uint32_t* lw = (uint32_t*)&lo[rt];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        hw[j] = pack_bf16(p[2 * j], p[2 * j + 1]);
        const float r0 = p[2 * j] - __uint_as_float(hw[j] << 16), r1 = p[2 * j + 1] - __uint_as_float(hw[j] & 0xffff0000u);
        lw[j] = pack_bf16(r0, r1);
      }
    }
#pragma unroll
    for (int i = 0; i < VPW; ++i)
      if (wave + LM_WAVES * i < nvb) {
#pragma unroll
        for (int rt = 0; rt < LM_RT; ++rt) {
          float4_t a = acc[rt][i];
#pragma unroll
          for (int j = 0; j < 4; ++j) a[j] *= alpha[rt];
          a = mfma32(vf[i], hi[rt], a);
          acc[rt][i] = mfma32(vf[i], lo[rt], a);
        }
      }
#pragma unroll
    for (int tau = 0; tau < 2; ++tau)
#pragma unroll
      for (int i = 0; i < CPW; ++i) kf[tau][i] = kn[tau][i];
#pragma unroll
    for (int i = 0; i < VPW; ++i) vf[i] = vn[i];
  }
  // lane (r, g) holds, of row 16 rt + r, the columns 16 db + 4 g .. + 3 of its wave's blocks
#pragma unroll
  for (int rt = 0; rt < LM_RT; ++rt) {
    const int rr = 16 * rt + r;
    const int tok = rr / heads_here, head = heads_block * hb + rr % heads_here;
    const float total = row_sum(l[rt]);                      // (every lane takes part, whatever its row)
    if (tok >= count || tok >= tile_tokens) continue;
    const int64_t item = (int64_t)(t0 + tok) * nh + head;
    if (splits == 1) {
      const float inv = 1.0f / total;
#pragma unroll
      for (int i = 0; i < VPW; ++i) {
        const int db = wave + LM_WAVES * i;
        if (db >= nvb) continue;
        TO* dst = out + item * rank + 16 * db + 4 * g;
#pragma unroll
        for (int j = 0; j < 4; ++j) Num<TO>::st(dst + j, acc[rt][i][j] * inv);
      }
    } else {
      float* dst = part_o + (item * splits + split) * rank;
#pragma unroll
      for (int i = 0; i < VPW; ++i) {
        const int db = wave + LM_WAVES * i;
        if (db >= nvb) continue;
        *(float4_t*)(dst + 16 * db + 4 * g) = acc[rt][i];
      }
      if (wave == 0 && g == 0) {
        part_ml[(item * splits + split) * 2] = m[rt];
        part_ml[(item * splits + split) * 2 + 1] = total;
      }
    }
  }
}

// One workgroup per (token, head), a thread per value column: the stretches' parts to one row. m is in units of log2.
template <typename TO>
__global__ void __launch_bounds__(LM_THREADS)
latent_attention_combine_kernel(TO* __restrict__ out, const float* __restrict__ part_o, const float* __restrict__ part_ml,
                                int rank, int splits) {
  const int64_t item = blockIdx.x;
  const float* ml = part_ml + item * splits * 2;
  float ms[LM_MAX_SPLITS], ls[LM_MAX_SPLITS], top = -INFINITY;
#pragma unroll
  for (int z = 0; z < LM_MAX_SPLITS; ++z) {
    ms[z] = ml[2 * min(z, splits - 1)];
    ls[z] = ml[2 * min(z, splits - 1) + 1];
    top = fmaxf(top, ms[z]);
  }
  float weight[LM_MAX_SPLITS], total = 0.f;
#pragma unroll
  for (int z = 0; z < LM_MAX_SPLITS; ++z) {
    weight[z] = z < splits ? fast_exp2(ms[z] - top) : 0.f;   // (a stretch without keys: 2^-inf = 0)
    total += weight[z] * ls[z];
  }
  const float inv = 1.0f / total;
  for (int d = threadIdx.x; d < rank; d += LM_THREADS) {
    float part[LM_MAX_SPLITS];
#pragma unroll
    for (int z = 0; z < LM_MAX_SPLITS; ++z) part[z] = part_o[(item * splits + min(z, splits - 1)) * rank + d];
    float sum = 0.f;
#pragma unroll
    for (int z = 0; z < LM_MAX_SPLITS; ++z) sum = fmaf(weight[z], part[z], sum);
    Num<TO>::st(out + item * rank + d, sum * inv);
  }
}

// Whether the kernel is built for a cached row of `row` numbers of which `rank` are the values.
extern "C" int ts_latent_mfma_takes(int rank, int row) {
  return rank > 0 && rank % 16 == 0 && row % 8 == 0 && rank <= row && row <= 640 && rank <= 512;
}

// tiles: int32 [num_tiles, 2] (first token, token count <= tile_tokens), every tile inside one request, or null:
// every token a tile of its own. A tile's rows are tile_tokens tokens by heads_block heads (at most 32 together);
// heads beyond heads_block take further workgroups. splits > 1: part_o float32 [tokens, heads, splits, rank] and
// part_ml float32 [tokens, heads, splits, 2] receive the stretches' parts.
extern "C" int ts_paged_attention_latent_mfma(void* out, int out_dtype, const float* q, const void* k_cache, const void* v_cache,
                                              const int32_t* block_tables, const int32_t* seq_of_token, const int32_t* positions,
                                              const int32_t* tiles, int num_tiles, int tile_tokens, int num_tokens, int nh, int rank,
                                              int rot, int page_size, int64_t kp, int64_t ks, int64_t vp, int64_t vd,
                                              int64_t v_slot, int max_blocks, float scale, int window, int page_run, int splits,
                                              float* part_o, float* part_ml, hipStream_t stream) {
  if (num_tiles <= 0 || num_tokens <= 0) return TS_OK;
  const int row = rank + rot;
  const int heads_block = min(nh, LM_ROWS);
  if (!ts_latent_mfma_takes(rank, row) || nh <= 0 || page_size != 32 || v_slot != 1 || kp % 8 || ks % 8 || vp % 8 || vd % 8 ||
      ((uintptr_t)k_cache & 15) || ((uintptr_t)v_cache & 15) || max_blocks <= 0 || page_run < 0 || page_run > 16 ||
      tile_tokens < 1 || tile_tokens * heads_block > LM_ROWS || (!tiles && (num_tiles != num_tokens || tile_tokens != 1)) ||
      splits < 1 || splits > LM_MAX_SPLITS || (splits > 1 && (!part_o || !part_ml)))
    return TS_BAD_SHAPE;
  dim3 grid(((num_tiles + 7) / 8) * 8, (nh + heads_block - 1) / heads_block, splits);
  const float scale_log2 = scale * 1.4426950408889634f;
#define LM_LAUNCH(CPW, VPW, TO) \
  latent_attention_mfma_kernel<CPW, VPW, TO><<<grid, LM_THREADS, 0, stream>>>((TO*)out, part_o, part_ml, q, (const bf16_t*)k_cache, \
      (const bf16_t*)v_cache, block_tables, seq_of_token, positions, tiles, num_tiles, tile_tokens, heads_block, nh, rank, row, kp, ks, \
      vp, vd, max_blocks, scale_log2, window, page_run, splits)
#define LM_PICK(TO) \
  do { \
    if (row <= 256 && rank <= 128) LM_LAUNCH(2, 2, TO); \
    else if (row <= 384 && rank <= 256) LM_LAUNCH(3, 4, TO); \
    else LM_LAUNCH(5, 8, TO); \
    if (splits > 1) { \
      const int64_t items = (int64_t)num_tokens * nh; \
      latent_attention_combine_kernel<TO><<<(unsigned)items, LM_THREADS, 0, stream>>>((TO*)out, part_o, part_ml, rank, splits); \
    } \
  } while (0)
  if (out_dtype == 0) LM_PICK(float);
  else if (out_dtype == 1) LM_PICK(bf16_t);
  else return TS_BAD_DTYPE;
#undef LM_PICK
#undef LM_LAUNCH
  return ts_check_launch();
}

// ---- products per head on the matrix cores ---------------------------------------------------------------------
// y[t, h, n] = sum_k x[t, h, k] w[h][n][k] for bfloat16 matrices whose k runs along memory (a matrix stored [k, n]
// comes as a transposed copy), x 32-bit (rounded to bfloat16 once, as a projection's operand is) or bfloat16, 32-bit
// sums, times sigmoid(gate) on the way out if there is one. A workgroup makes 64 tokens by 64 columns of one head, a
// wave 16 tokens: the matrix's rows are the instruction's rows, so that a lane ends with four adjacent columns of
// one token. Operands come straight from memory in 16-byte pieces; pieces past K are zeros of x against the
// matrix's last piece.
#define HM_TOKENS 64
#define HM_COLS 64

template <typename TX, typename TO>
__global__ void __launch_bounds__(LM_THREADS)
heads_gemm_mfma_kernel(TO* __restrict__ y, int64_t y_token, int64_t y_head, const TX* __restrict__ x, int64_t x_token,
                       int64_t x_head, const bf16_t* __restrict__ w, int64_t w_head, int64_t w_n, int num_tokens, int N, int K,
                       const float* __restrict__ gate, int64_t gate_token) {
  const int wave = wave_index(), lane = threadIdx.x & (TS_WAVE - 1);
  const int r = lane & 15, g = lane >> 4;
  const int h = blockIdx.y, n0 = blockIdx.z * HM_COLS;
  const int t = blockIdx.x * HM_TOKENS + 16 * wave + r;
  const TX* xrow = x + (int64_t)min(t, num_tokens - 1) * x_token + (int64_t)h * x_head;
  const bf16_t* wh = w + (int64_t)h * w_head;
  float4_t acc[HM_COLS / 16];
#pragma unroll
  for (int nb = 0; nb < HM_COLS / 16; ++nb) acc[nb] = (float4_t){0.f, 0.f, 0.f, 0.f};
#pragma unroll 4
  for (int k0 = 0; k0 < K; k0 += 32) {
    const int k = k0 + 8 * g, kc = min(k, K - 8);
    uint4 b;
    if constexpr (sizeof(TX) == 4) {
      const float4 lo = *(const float4*)(xrow + kc), hi = *(const float4*)(xrow + kc + 4);
      b = make_uint4(pack_bf16(lo.x, lo.y), pack_bf16(lo.z, lo.w), pack_bf16(hi.x, hi.y), pack_bf16(hi.z, hi.w));
    } else {
      b = *(const uint4*)(xrow + kc);
    }
    if (k >= K) b = make_uint4(0, 0, 0, 0);
#pragma unroll
    for (int nb = 0; nb < HM_COLS / 16; ++nb) {
      const int n = min(n0 + 16 * nb + r, N - 1);
      acc[nb] = mfma32(*(const uint4*)(wh + (int64_t)n * w_n + kc), b, acc[nb]);
    }
  }
  if (t >= num_tokens) return;
#pragma unroll
  for (int nb = 0; nb < HM_COLS / 16; ++nb)
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int n = n0 + 16 * nb + 4 * g + j;
      if (n >= N) continue;
      float v = acc[nb][j];
      if (gate) v = v / (1.0f + expf(-gate[(int64_t)t * gate_token + (int64_t)h * N + n]));
      Num<TO>::st(y + (int64_t)t * y_token + (int64_t)h * y_head + n, v);
    }
}

// w: bfloat16 [heads][N][K] with K along memory (stride w_n between rows, a multiple of 8; K a multiple of 8);
// x rows 16-byte aligned.
extern "C" int ts_heads_gemm_mfma(void* y, int y_dtype, int64_t y_token, int64_t y_head, const void* x, int x_dtype,
                                  int64_t x_token, int64_t x_head, const void* w, int64_t w_head, int64_t w_n, int num_tokens,
                                  int heads, int N, int K, const float* gate, int64_t gate_token, hipStream_t stream) {
  if (num_tokens <= 0) return TS_OK;
  const int x_size = x_dtype == 0 ? 4 : 2;
  if (heads <= 0 || heads > 65535 || N <= 0 || K < 8 || K % 8 || w_n % 8 || w_head % 8 || ((uintptr_t)w & 15) ||
      ((uintptr_t)x & 15) || (x_token * x_size) % 16 || (x_head * x_size) % 16 || (N + HM_COLS - 1) / HM_COLS > 65535)
    return TS_BAD_SHAPE;
  dim3 grid((num_tokens + HM_TOKENS - 1) / HM_TOKENS, heads, (N + HM_COLS - 1) / HM_COLS);
#define HM_LAUNCH(TX, TO) \
  heads_gemm_mfma_kernel<TX, TO><<<grid, LM_THREADS, 0, stream>>>((TO*)y, y_token, y_head, (const TX*)x, x_token, x_head, \
      (const bf16_t*)w, w_head, w_n, num_tokens, N, K, gate, gate_token)
  if (x_dtype == 0 && y_dtype == 0) HM_LAUNCH(float, float);
  else if (x_dtype == 0 && y_dtype == 1) HM_LAUNCH(float, bf16_t);
  else if (x_dtype == 1 && y_dtype == 0) HM_LAUNCH(bf16_t, float);
  else if (x_dtype == 1 && y_dtype == 1) HM_LAUNCH(bf16_t, bf16_t);
  else return TS_BAD_DTYPE;
#undef HM_LAUNCH
  return ts_check_launch();
}
