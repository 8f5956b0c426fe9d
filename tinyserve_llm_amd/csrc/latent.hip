// Attention through a low-rank latent. A token caches one row [c | r]: its latent c (`rank` numbers, normalised)
// and one rotated key part r (`rot` numbers) that all heads share. With the keys' and values' up-projections
// taken to the query's and the output's side (score_h = (W_uk,h^T q_h) . c + q_rot,h . r, out_h = W_uv,h sum_j p_j c_j),
// attention is multi-query attention over those rows, whose first `rank` numbers are also the values.
//   * `ts_segment_rmsnorm`: a stretch of every row divided by its root mean square (eps inside the root) times a
//     weight, 32-bit, to a place and storage type of its own (norms over whole projections or parts of them).
//   * `ts_latent_finish`: what lies between the fused down-projection and the cache: the query latent's norm, the
//     key/value latent's norm, the rotation of the shared key part (pairs (2i, 2i+1), angle in 64-bit, cosine and
//     sine times an amplitude), and the write of [c | r] to the token's cache slot (and of c once more into the
//     pages that hold the values transposed, for the matrix-core kernel of latent_mfma.hip).
//   * `ts_rotate_heads`: a stretch of every head turned by the token's position, to a place of its own.
//   * `ts_heads_gemm`: y[t, h, :] = x[t, h, :] . W[h] for per-head matrices with free strides (so W may be used as
//     stored or transposed), 32-bit multiply-adds in ascending k; optionally times sigmoid(gate) on the way out.
//   * `ts_paged_attention_latent`: multi-query attention over the cached rows: causal, windowed or chunked
//     (`ts_first_key`), softmax in 32-bit; keys are visited in chunks of 64 counted from position 0, so the order of
//     every sum depends on the token's position alone. One workgroup per token; its waves take the heads in turn.
#include "common.h"

#define LT_WAVES 4
#define LT_THREADS (LT_WAVES * TS_WAVE)
#define LT_MAX_ROW 640          // rank + rot of a cached row
#define LT_MAX_RANK 512

static __device__ __forceinline__ float lt_block_sum(float v, float* red) {
  const int wave = threadIdx.x / TS_WAVE, lane = threadIdx.x & (TS_WAVE - 1);
  v = wave_sum(v);
  __syncthreads();                                         // (the buffer's last readers are done)
  if (lane == 0) red[wave] = v;
  __syncthreads();
  float s = 0.f;
#pragma unroll
  for (int w = 0; w < LT_WAVES; ++w) s += red[w];
  return s;
}

template <typename TO>
__global__ void __launch_bounds__(LT_THREADS)
segment_rmsnorm_kernel(TO* __restrict__ out, int64_t out_stride, const float* __restrict__ x, int64_t x_stride, int size,
                       const float* __restrict__ weight, float eps) {
  __shared__ float red[LT_WAVES];
  const float* row = x + (int64_t)blockIdx.x * x_stride;
  float squares = 0.f;
  for (int d = threadIdx.x; d < size; d += LT_THREADS) squares = fmaf(row[d], row[d], squares);
  const float inv = 1.0f / sqrtf(lt_block_sum(squares, red) / (float)size + eps);
  TO* dst = out + (int64_t)blockIdx.x * out_stride;
  for (int d = threadIdx.x; d < size; d += LT_THREADS) Num<TO>::st(dst + d, row[d] * inv * (weight ? weight[d] : 1.0f));
}

extern "C" int ts_segment_rmsnorm(void* out, int out_dtype, int64_t out_stride, const float* x, int64_t x_stride, int size,
                                  const float* weight, float eps, int num_rows, hipStream_t stream) {
  if (num_rows <= 0) return TS_OK;
  if (size <= 0 || x_stride < size || out_stride < size) return TS_BAD_SHAPE;
  if (out_dtype == 0)
    segment_rmsnorm_kernel<float><<<num_rows, LT_THREADS, 0, stream>>>((float*)out, out_stride, x, x_stride, size, weight, eps);
  else if (out_dtype == 1)
    segment_rmsnorm_kernel<bf16_t><<<num_rows, LT_THREADS, 0, stream>>>((bf16_t*)out, out_stride, x, x_stride, size, weight, eps);
  else return TS_BAD_DTYPE;
  return ts_check_launch();
}

// Two stretches of every row in one launch, in place (the norms over a token's whole q and whole k projection):
// workgroup (row, 0) takes the first, (row, 1) the second.
__global__ void __launch_bounds__(LT_THREADS)
segment_rmsnorm_pair_kernel(float* __restrict__ x, int64_t x_stride, int off0, int size0, const float* __restrict__ w0, int off1,
                            int size1, const float* __restrict__ w1, float eps) {
  __shared__ float red[LT_WAVES];
  const int off = blockIdx.y ? off1 : off0, size = blockIdx.y ? size1 : size0;
  const float* weight = blockIdx.y ? w1 : w0;
  float* row = x + (int64_t)blockIdx.x * x_stride + off;
  float squares = 0.f;
  for (int d = threadIdx.x; d < size; d += LT_THREADS) squares = fmaf(row[d], row[d], squares);
  const float inv = 1.0f / sqrtf(lt_block_sum(squares, red) / (float)size + eps);
  for (int d = threadIdx.x; d < size; d += LT_THREADS) row[d] = row[d] * inv * weight[d];
}

extern "C" int ts_segment_rmsnorm_pair(float* x, int64_t x_stride, int off0, int size0, const float* w0, int off1, int size1,
                                       const float* w1, float eps, int num_rows, hipStream_t stream) {
  if (num_rows <= 0) return TS_OK;
  if (size0 <= 0 || size1 <= 0 || off0 < 0 || off1 < off0 + size0 || off1 + size1 > x_stride || !w0 || !w1) return TS_BAD_SHAPE;
  segment_rmsnorm_pair_kernel<<<dim3(num_rows, 2), LT_THREADS, 0, stream>>>(x, x_stride, off0, size0, w0, off1, size1, w1, eps);
  return ts_check_launch();
}

// The angle position * f in 64-bit, brought to [-pi, pi] before the 32-bit sine and cosine.
static __device__ __forceinline__ void lt_angle(int pos, double f, float amplitude, float* cs, float* sn) {
  const double angle = (double)pos * f;
  const double turns = rint(angle * 0.15915494309189535);
  sincosf((float)fma(-turns, 6.283185307179586, angle), sn, cs);
  *cs *= amplitude;
  *sn *= amplitude;
}

template <typename TO>
__global__ void __launch_bounds__(LT_THREADS)
latent_finish_kernel(TO* __restrict__ cq_out, TO* __restrict__ cache, const float* __restrict__ down, int64_t stride,
                     int q_off, int q_rank, int kv_off, int rank, int rot, const float* __restrict__ q_weight,
                     const float* __restrict__ kv_weight, float eps, const double* __restrict__ freqs, float amplitude,
                     const int32_t* __restrict__ positions, const int32_t* __restrict__ slots, int page_size, int64_t kp,
                     int64_t ks, TO* __restrict__ vcache, int64_t vp, int64_t vd) {
  __shared__ float red[LT_WAVES];
  const int t = blockIdx.x;
  const float* row = down + (int64_t)t * stride;
  if (q_rank > 0) {
    const float* q = row + q_off;
    float squares = 0.f;
    for (int d = threadIdx.x; d < q_rank; d += LT_THREADS) squares = fmaf(q[d], q[d], squares);
    const float inv = 1.0f / sqrtf(lt_block_sum(squares, red) / (float)q_rank + eps);
    for (int d = threadIdx.x; d < q_rank; d += LT_THREADS) Num<TO>::st(cq_out + (int64_t)t * q_rank + d, q[d] * inv * q_weight[d]);
  }
  const int slot = slots ? slots[t] : -1;
  if (slot < 0 || !cache) return;                          // (uniform over the workgroup)
  const int page = slot / page_size, off = slot - page * page_size;
  TO* dst = cache + page * kp + off * ks;
  const float* c = row + kv_off;
  float squares = 0.f;
  for (int d = threadIdx.x; d < rank; d += LT_THREADS) squares = fmaf(c[d], c[d], squares);
  const float inv = 1.0f / sqrtf(lt_block_sum(squares, red) / (float)rank + eps);
  TO* vdst = vcache ? vcache + page * vp + off : nullptr;  // the latent once more, transposed inside the page
  for (int d = threadIdx.x; d < rank; d += LT_THREADS) {
    const float v = c[d] * inv * kv_weight[d];
    Num<TO>::st(dst + d, v);
    if (vdst) Num<TO>::st(vdst + (int64_t)d * vd, v);
  }
  const int pos = positions[t];
  for (int pair = threadIdx.x; pair < rot / 2; pair += LT_THREADS) {
    float cs, sn;
    lt_angle(pos, freqs[pair], amplitude, &cs, &sn);
    const float u = c[rank + 2 * pair], v = c[rank + 2 * pair + 1];
    Num<TO>::st(dst + rank + 2 * pair, u * cs - v * sn);
    Num<TO>::st(dst + rank + 2 * pair + 1, v * cs + u * sn);
  }
}

extern "C" int ts_latent_finish(void* cq_out, void* cache, int out_dtype, const float* down, int64_t stride, int q_off,
                                int q_rank, int kv_off, int rank, int rot, const float* q_weight, const float* kv_weight,
                                float eps, const double* freqs, float amplitude, const int32_t* positions,
                                const int32_t* slots, int page_size, int64_t kp, int64_t ks, void* vcache, int64_t vp,
                                int64_t vd, int num_tokens, hipStream_t stream) {
  if (num_tokens <= 0) return TS_OK;
  if (rank <= 0 || rot < 0 || rot % 2 || q_rank < 0 || q_off < 0 || kv_off < 0 || page_size <= 0 ||
      q_off + q_rank > stride || kv_off + rank + rot > stride || (rot > 0 && !freqs))
    return TS_BAD_SHAPE;
#define LT_FINISH(TO) \
  latent_finish_kernel<TO><<<num_tokens, LT_THREADS, 0, stream>>>((TO*)cq_out, (TO*)cache, down, stride, q_off, q_rank, kv_off, \
      rank, rot, q_weight, kv_weight, eps, freqs, amplitude, positions, slots, page_size, kp, ks, (TO*)vcache, vp, vd)
  if (out_dtype == 0) LT_FINISH(float);
  else if (out_dtype == 1) LT_FINISH(bf16_t);
  else return TS_BAD_DTYPE;
#undef LT_FINISH
  return ts_check_launch();
}

// One thread per (token, head, pair). `back`: by minus the angle. `gate` (32-bit, a number per token and head,
// `gate_token` apart from token to token): the turned pair is multiplied by sigmoid(gate[t, h]).
template <typename TI, typename TO>
__global__ void __launch_bounds__(LT_THREADS)
rotate_heads_kernel(TO* __restrict__ dst, int64_t dst_token, int64_t dst_head, const TI* __restrict__ src, int64_t src_token,
                    int64_t src_head, int heads, int rot, int interleaved, const double* __restrict__ freqs, float amplitude,
                    const int32_t* __restrict__ positions, int64_t items, int back, const float* __restrict__ gate,
                    int64_t gate_token) {
  const int64_t item = (int64_t)blockIdx.x * LT_THREADS + threadIdx.x;
  if (item >= items) return;
  const int half = rot / 2;
  const int pair = (int)(item % half);
  const int h = (int)((item / half) % heads);
  const int64_t t = item / ((int64_t)half * heads);
  float cs, sn;
  lt_angle(positions[t], freqs[pair], amplitude, &cs, &sn);
  if (back) sn = -sn;
  const float g = gate ? 1.0f / (1.0f + expf(-gate[t * gate_token + h])) : 1.0f;
  const int a = interleaved ? 2 * pair : pair, b = interleaved ? 2 * pair + 1 : pair + half;
  const TI* s = src + t * src_token + h * src_head;
  TO* d = dst + t * dst_token + h * dst_head;
  const float u = Num<TI>::ld(s + a), v = Num<TI>::ld(s + b);
  Num<TO>::st(d + a, (u * cs - v * sn) * g);
  Num<TO>::st(d + b, (v * cs + u * sn) * g);
}

extern "C" int ts_rotate_heads(void* dst, int out_dtype, int64_t dst_token, int64_t dst_head, const void* src, int in_dtype,
                               int64_t src_token, int64_t src_head, int heads, int rot, int interleaved, const double* freqs,
                               float amplitude, const int32_t* positions, int num_tokens, int back, const float* gate,
                               int64_t gate_token, hipStream_t stream) {
  if (num_tokens <= 0 || rot == 0) return TS_OK;
  if (heads <= 0 || rot < 0 || rot % 2 || !freqs) return TS_BAD_SHAPE;
  const int64_t items = (int64_t)num_tokens * heads * (rot / 2);
  const int64_t blocks = (items + LT_THREADS - 1) / LT_THREADS;
  if (blocks > 0x7fffffff) return TS_BAD_SHAPE;
#define LT_ROTATE(TI, TO) \
  rotate_heads_kernel<TI, TO><<<(unsigned)blocks, LT_THREADS, 0, stream>>>((TO*)dst, dst_token, dst_head, (const TI*)src, src_token, \
      src_head, heads, rot, interleaved, freqs, amplitude, positions, items, back, gate, gate_token)
  if (in_dtype == 0 && out_dtype == 0) LT_ROTATE(float, float);
  else if (in_dtype == 0 && out_dtype == 1) LT_ROTATE(float, bf16_t);
  else if (in_dtype == 1 && out_dtype == 1) LT_ROTATE(bf16_t, bf16_t);
  else return TS_BAD_DTYPE;
#undef LT_ROTATE
  return ts_check_launch();
}

// A tile of 16 tokens by 64 columns of one head a workgroup; thread (column, token quarter).
#define HG_BM 16
#define HG_BN 64
#define HG_KC 32
template <typename TX, typename TW, typename TO>
__global__ void __launch_bounds__(LT_THREADS)
heads_gemm_kernel(TO* __restrict__ y, int64_t y_token, int64_t y_head, const TX* __restrict__ x, int64_t x_token, int64_t x_head,
                  const TW* __restrict__ w, int64_t w_head, int64_t w_k, int64_t w_n, int num_tokens, int N, int K,
                  const float* __restrict__ gate, int64_t gate_token) {
  __shared__ float x_s[HG_BM][HG_KC + 1];
  __shared__ float w_s[HG_KC][HG_BN + 1];
  const int t0 = blockIdx.x * HG_BM, h = blockIdx.y, n0 = blockIdx.z * HG_BN;
  const int tx = threadIdx.x & (HG_BN - 1), ty = threadIdx.x / HG_BN;
  const TW* wh = w + (int64_t)h * w_head;
  float acc[4] = {0.f, 0.f, 0.f, 0.f};
  for (int k0 = 0; k0 < K; k0 += HG_KC) {
    for (int i = threadIdx.x; i < HG_BM * HG_KC; i += LT_THREADS) {
      const int r = i / HG_KC, kk = i - r * HG_KC;
      x_s[r][kk] = (t0 + r < num_tokens && k0 + kk < K) ? Num<TX>::ld(x + (int64_t)(t0 + r) * x_token + h * x_head + k0 + kk) : 0.f;
    }
    for (int i = threadIdx.x; i < HG_KC * HG_BN; i += LT_THREADS) {
      // (neighbouring threads along whichever way the matrix is contiguous)
      const int kk = w_n == 1 ? i / HG_BN : i % HG_KC, c = w_n == 1 ? i % HG_BN : i / HG_KC;
      w_s[kk][c] = (n0 + c < N && k0 + kk < K) ? Num<TW>::ld(wh + (int64_t)(k0 + kk) * w_k + (int64_t)(n0 + c) * w_n) : 0.f;
    }
    __syncthreads();
#pragma unroll 8
    for (int kk = 0; kk < HG_KC; ++kk) {
      const float wv = w_s[kk][tx];
#pragma unroll
      for (int r = 0; r < 4; ++r) acc[r] = fmaf(x_s[ty * 4 + r][kk], wv, acc[r]);
    }
    __syncthreads();
  }
  if (n0 + tx >= N) return;
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    const int t = t0 + ty * 4 + r;
    if (t >= num_tokens) continue;
    float v = acc[r];
    if (gate) v = v / (1.0f + expf(-gate[(int64_t)t * gate_token + (int64_t)h * N + n0 + tx]));
    Num<TO>::st(y + (int64_t)t * y_token + h * y_head + n0 + tx, v);
  }
}

extern "C" int ts_heads_gemm(void* y, int y_dtype, int64_t y_token, int64_t y_head, const void* x, int x_dtype, int64_t x_token,
                             int64_t x_head, const void* w, int w_dtype, int64_t w_head, int64_t w_k, int64_t w_n, int num_tokens,
                             int heads, int N, int K, const float* gate, int64_t gate_token, hipStream_t stream) {
  if (num_tokens <= 0) return TS_OK;
  if (heads <= 0 || heads > 65535 || N <= 0 || K <= 0 || (N + HG_BN - 1) / HG_BN > 65535) return TS_BAD_SHAPE;
  dim3 grid((num_tokens + HG_BM - 1) / HG_BM, heads, (N + HG_BN - 1) / HG_BN);
#define HG_LAUNCH(TX, TW, TO) \
  heads_gemm_kernel<TX, TW, TO><<<grid, LT_THREADS, 0, stream>>>((TO*)y, y_token, y_head, (const TX*)x, x_token, x_head, (const TW*)w, \
      w_head, w_k, w_n, num_tokens, N, K, gate, gate_token)
  if (x_dtype == 0 && w_dtype == 0 && y_dtype == 0) HG_LAUNCH(float, float, float);
  else if (x_dtype == 0 && w_dtype == 1 && y_dtype == 0) HG_LAUNCH(float, bf16_t, float);
  else if (x_dtype == 0 && w_dtype == 1 && y_dtype == 1) HG_LAUNCH(float, bf16_t, bf16_t);
  else if (x_dtype == 1 && w_dtype == 1 && y_dtype == 1) HG_LAUNCH(bf16_t, bf16_t, bf16_t);
  else if (x_dtype == 1 && w_dtype == 1 && y_dtype == 0) HG_LAUNCH(bf16_t, bf16_t, float);
  else return TS_BAD_DTYPE;
#undef HG_LAUNCH
  return ts_check_launch();
}

// One workgroup per token. The token's queries lie in LDS as they are needed, a head a wave at a time; a wave
// walks the keys in chunks of 64 (a key a lane for the scores, a dimension a lane for the weighted sum).
template <typename TC, typename TQ, typename TO>
__global__ void __launch_bounds__(LT_THREADS)
paged_attention_latent_kernel(TO* __restrict__ out, const TQ* __restrict__ q, const TC* __restrict__ cache,
                              const int32_t* __restrict__ block_tables, const int32_t* __restrict__ seq_of_token,
                              const int32_t* __restrict__ positions, int nh, int rank, int row, int page_size, int64_t kp,
                              int64_t ks, int max_blocks, float scale, int window, int page_run) {
  __shared__ float q_s[LT_WAVES][LT_MAX_ROW];
  __shared__ float p_s[LT_WAVES][TS_WAVE];
  __shared__ int64_t row_s[LT_WAVES][TS_WAVE];             // element offset of each key's cached row
  const int wave = threadIdx.x / TS_WAVE, lane = threadIdx.x & (TS_WAVE - 1);
  const int t = blockIdx.x;
  const int pos = positions[t];
  const int32_t* table = block_tables + (int64_t)seq_of_token[t] * max_blocks;
  const int lo = ts_first_key(pos, window);
  for (int h = wave; h < nh; h += LT_WAVES) {              // (wave-uniform: no block barrier below)
    const TQ* qrow = q + ((int64_t)t * nh + h) * row;
    wave_sync();
    for (int d = lane; d < row; d += TS_WAVE) q_s[wave][d] = Num<TQ>::ld(qrow + d);
    wave_sync();
    float m = -INFINITY, l = 0.f;
    float acc[LT_MAX_RANK / TS_WAVE];
#pragma unroll
    for (int i = 0; i < LT_MAX_RANK / TS_WAVE; ++i) acc[i] = 0.f;
    for (int c0 = (lo / TS_WAVE) * TS_WAVE; c0 <= pos; c0 += TS_WAVE) {
      const int key = c0 + lane;
      const bool valid = key >= lo && key <= pos;
      float s = -INFINITY;
      int64_t rowoff = 0;
      if (valid) {
        const int pg = key / page_size, slot = key % page_size;
        const int64_t page = ((int64_t)table[pg >> page_run] << page_run) + (pg & ((1 << page_run) - 1));
        rowoff = page * kp + (int64_t)slot * ks;
        const TC* kr = cache + rowoff;
        float dot = 0.f;
        for (int d = 0; d < row; ++d) dot = fmaf(q_s[wave][d], Num<TC>::ld(kr + d), dot);
        s = dot * scale;
      }
      const float m_new = fmaxf(m, wave_max(s));           // finite: the chunk holds at least one visible key
      const float p = valid ? expf(s - m_new) : 0.f;
      const float alpha = expf(m - m_new);
      l = l * alpha + wave_sum(p);
      m = m_new;
      p_s[wave][lane] = p;
      row_s[wave][lane] = rowoff;
      wave_sync();
      const int first = lo > c0 ? lo - c0 : 0;
      const int last = pos - c0 < TS_WAVE - 1 ? pos - c0 : TS_WAVE - 1;
#pragma unroll
      for (int i = 0; i < LT_MAX_RANK / TS_WAVE; ++i) {
        const int d = lane + i * TS_WAVE;
        if (d < rank) {
          float a = acc[i] * alpha;
          for (int j = first; j <= last; ++j) a = fmaf(p_s[wave][j], Num<TC>::ld(cache + row_s[wave][j] + d), a);
          acc[i] = a;
        }
      }
      wave_sync();
    }
    TO* orow = out + ((int64_t)t * nh + h) * rank;
    const float inv = 1.0f / l;
#pragma unroll
    for (int i = 0; i < LT_MAX_RANK / TS_WAVE; ++i) {
      const int d = lane + i * TS_WAVE;
      if (d < rank) Num<TO>::st(orow + d, acc[i] * inv);
    }
  }
}

extern "C" int ts_paged_attention_latent(void* out, int out_dtype, const void* q, int q_dtype, const void* cache, int cache_dtype,
                                         const int32_t* block_tables, const int32_t* seq_of_token, const int32_t* positions,
                                         int num_tokens, int nh, int rank, int rot, int page_size, int64_t kp, int64_t ks,
                                         int max_blocks, float scale, int window, int page_run, hipStream_t stream) {
  if (num_tokens <= 0) return TS_OK;
  if (nh <= 0 || rank <= 0 || rank > LT_MAX_RANK || rot < 0 || rank + rot > LT_MAX_ROW || page_size <= 0 || max_blocks <= 0 ||
      page_run < 0 || page_run > 16)
    return TS_BAD_SHAPE;
#define LT_ATTEND(TC, TQ, TO) \
  paged_attention_latent_kernel<TC, TQ, TO><<<num_tokens, LT_THREADS, 0, stream>>>((TO*)out, (const TQ*)q, (const TC*)cache, \
      block_tables, seq_of_token, positions, nh, rank, rank + rot, page_size, kp, ks, max_blocks, scale, window, page_run)
  if (cache_dtype == 0 && q_dtype == 0 && out_dtype == 0) LT_ATTEND(float, float, float);
  else if (cache_dtype == 1 && q_dtype == 0 && out_dtype == 1) LT_ATTEND(bf16_t, float, bf16_t);
  else if (cache_dtype == 1 && q_dtype == 0 && out_dtype == 0) LT_ATTEND(bf16_t, float, float);
  else if (cache_dtype == 1 && q_dtype == 1 && out_dtype == 1) LT_ATTEND(bf16_t, bf16_t, bf16_t);
  else return TS_BAD_DTYPE;
#undef LT_ATTEND
  return ts_check_launch();
}
