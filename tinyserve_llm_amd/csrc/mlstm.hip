// The matrix memory of an mLSTM as a recurrent mixer. Per head a state S [dim, vdim], a normaliser n [dim] and a
// running maximum m of the log gates, all 32-bit, all zero at a request's start. For a token with q (already
// times dim^(-1/2)), k, v and the gates' raw sums a_i, a_f:
//     i = cap tanh((a_i + b_i) / cap),  f = logsigmoid(cap tanh((a_f + b_f) / cap)),
//     m' = max(f + m, i),  S' = exp(f + m - m') S + exp(i - m') k v^T,  n' = exp(f + m - m') n + exp(i - m') k,
//     o = S'^T q / (max(|n' . q|, exp(-m')) + 1e-6).
//   * `ts_mlstm_scan`: one workgroup per (request, head, slice of the value columns) walks the request's tokens of
//     the step in order, the state's slice in registers (columns of S are independent of each other; n and m are
//     kept by every slice, the first one stores them), and leaves o, 32-bit. The state is read from the request's
//     slot at the start and written back at the end.
//   * `ts_mlstm_finish`: each head's o divided by its root mean square, times a weight, times sigmoid(gate), to
//     the storage type of the output projection's operand.
// A token's row of the fused projection is [q | k | v | a_i | a_f | gate], 32-bit.
#include "common.h"

#define ML_THREADS 256
#define ML_WAVES (ML_THREADS / TS_WAVE)
#define ML_MAX_DIM 1024         // of a query / key head
#define ML_MAX_COLS 256         // value columns of a slice

// RPT: rows of S (dimensions of k) that a thread keeps of its column.
template <int RPT>
__global__ void __launch_bounds__(ML_THREADS)
mlstm_scan_kernel(float* __restrict__ out, const float* __restrict__ proj, int64_t stride, const float* __restrict__ i_bias,
                  const float* __restrict__ f_bias, float* __restrict__ state, const int32_t* __restrict__ cu_seqlens,
                  const int32_t* __restrict__ state_slots, int heads, int dim, int vdim, int cols, float cap, float q_scale) {
  extern __shared__ float lds[];
  // [2][2 dim + cols + 2]: q, k, the slice's v, the gates' raw sums of the token at hand and of the next one
  const int in_size = 2 * dim + cols + 2;
  float* in_s = lds;
  float* part_s = lds + 2 * in_size;                       // [2][groups][cols] partial sums of o
  __shared__ float nq_s[2][ML_WAVES];
  const int seq = blockIdx.x, h = blockIdx.y, v0 = blockIdx.z * cols;
  const int nc = min(cols, vdim - v0);                     // this slice's columns
  const int groups = ML_THREADS / cols;                    // threads side by side along the rows of a column
  const int col = threadIdx.x % cols, grp = threadIdx.x / cols;
  const bool holds = grp < groups && col < nc;
  const int wave = threadIdx.x / TS_WAVE, lane = threadIdx.x & (TS_WAVE - 1);
  const int t_begin = cu_seqlens[seq], t_end = cu_seqlens[seq + 1];
  const int64_t per_head = (int64_t)dim * vdim + dim + 1;
  float* st = state + ((int64_t)state_slots[seq] * heads + h) * per_head;
  float S[RPT];
#pragma unroll
  for (int r = 0; r < RPT; ++r) {
    const int d = grp + r * groups;
    S[r] = (holds && d < dim) ? st[(int64_t)d * vdim + v0 + col] : 0.f;
  }
  float n[ML_MAX_DIM / ML_THREADS];
#pragma unroll
  for (int r = 0; r < ML_MAX_DIM / ML_THREADS; ++r) {
    const int d = threadIdx.x + r * ML_THREADS;
    n[r] = d < dim ? st[(int64_t)dim * vdim + d] : 0.f;
  }
  float m = st[(int64_t)dim * vdim + dim];
  const float bi = i_bias[h], bf = f_bias[h];
  const int q_at = h * dim, k_at = heads * dim + h * dim, v_at = 2 * heads * dim + h * vdim + v0;
  const int i_at = 2 * heads * dim + heads * vdim + h, f_at = i_at + heads;
  auto fetch = [&](int t, int buf) {
    const float* row = proj + (int64_t)t * stride;
    float* dst = in_s + buf * in_size;
    for (int e = threadIdx.x; e < in_size; e += ML_THREADS) {
      float v;
      if (e < dim) v = row[q_at + e] * q_scale;
      else if (e < 2 * dim) v = row[k_at + e - dim];
      else if (e < 2 * dim + cols) v = e - 2 * dim < nc ? row[v_at + e - 2 * dim] : 0.f;
      else v = row[e == 2 * dim + cols ? i_at : f_at];
      dst[e] = v;
    }
  };
  if (t_begin < t_end) fetch(t_begin, 0);
  __syncthreads();
  for (int t = t_begin; t < t_end; ++t) {
    const int buf = (t - t_begin) & 1;
    if (t + 1 < t_end) fetch(t + 1, buf ^ 1);              // (that buffer's readers passed the barrier a token ago)
    const float* q_s = in_s + buf * in_size;
    const float* k_s = q_s + dim;
    const float* v_s = k_s + dim;
    const float gi = cap * tanhf((v_s[cols] + bi) / cap);
    const float zf = cap * tanhf((v_s[cols + 1] + bf) / cap);
    const float gf = fminf(zf, 0.f) - log1pf(expf(-fabsf(zf)));      // logsigmoid
    const float m_new = fmaxf(gf + m, gi);
    const float keep = expf(gf + m - m_new), take = expf(gi - m_new);
    m = m_new;
    float nq = 0.f;
#pragma unroll
    for (int r = 0; r < ML_MAX_DIM / ML_THREADS; ++r) {
      const int d = threadIdx.x + r * ML_THREADS;
      if (d < dim) {
        n[r] = fmaf(keep, n[r], take * k_s[d]);
        nq = fmaf(n[r], q_s[d], nq);
      }
    }
    nq = wave_sum(nq);
    if (lane == 0) nq_s[buf][wave] = nq;
    float o = 0.f;
    const float tv = holds ? take * v_s[col] : 0.f;
#pragma unroll
    for (int r = 0; r < RPT; ++r) {
      const int d = grp + r * groups;
      if (d < dim) {
        S[r] = fmaf(keep, S[r], k_s[d] * tv);
        o = fmaf(S[r], q_s[d], o);
      }
    }
    if (grp < groups) part_s[(buf * groups + grp) * cols + col] = o;
    __syncthreads();
    if (threadIdx.x < nc) {
      float sum = 0.f;
      for (int g = 0; g < groups; ++g) sum += part_s[(buf * groups + g) * cols + threadIdx.x];
      float dot = 0.f;
#pragma unroll
      for (int w = 0; w < ML_WAVES; ++w) dot += nq_s[buf][w];
      out[(int64_t)t * heads * vdim + h * vdim + v0 + threadIdx.x] = sum / (fmaxf(fabsf(dot), expf(-m_new)) + 1e-6f);
    }
  }
#pragma unroll
  for (int r = 0; r < RPT; ++r) {
    const int d = grp + r * groups;
    if (holds && d < dim) st[(int64_t)d * vdim + v0 + col] = S[r];
  }
  if (blockIdx.z == 0) {
#pragma unroll
    for (int r = 0; r < ML_MAX_DIM / ML_THREADS; ++r) {
      const int d = threadIdx.x + r * ML_THREADS;
      if (d < dim) st[(int64_t)dim * vdim + d] = n[r];
    }
    if (threadIdx.x == 0) st[(int64_t)dim * vdim + dim] = m;
  }
}

extern "C" int ts_mlstm_scan(float* out, const float* proj, int64_t stride, const float* i_bias, const float* f_bias,
                             float* state, const int32_t* cu_seqlens, const int32_t* state_slots, int num_seqs, int heads,
                             int dim, int vdim, int cols, float cap, float q_scale, hipStream_t stream) {
  if (num_seqs <= 0) return TS_OK;
  if (heads <= 0 || heads > 65535 || dim <= 0 || dim > ML_MAX_DIM || vdim <= 0 || cols <= 0 || cols > ML_MAX_COLS ||
      cols > ML_THREADS || !(cap > 0.f))
    return TS_BAD_SHAPE;
  const int slices = (vdim + cols - 1) / cols;
  if (slices > 65535) return TS_BAD_SHAPE;
  const int groups = ML_THREADS / cols;
  const int rpt = (dim + groups - 1) / groups;
  dim3 grid(num_seqs, heads, slices);
  const size_t lds = (size_t)(2 * (2 * dim + cols + 2) + 2 * groups * cols) * sizeof(float);
#define ML_LAUNCH(RPT) \
  mlstm_scan_kernel<RPT><<<grid, ML_THREADS, lds, stream>>>(out, proj, stride, i_bias, f_bias, state, cu_seqlens, state_slots, \
                                                            heads, dim, vdim, cols, cap, q_scale)
  if (rpt <= 8) ML_LAUNCH(8);
  else if (rpt <= 16) ML_LAUNCH(16);
  else if (rpt <= 32) ML_LAUNCH(32);
  else if (rpt <= 64) ML_LAUNCH(64);
  else return TS_BAD_SHAPE;
#undef ML_LAUNCH
  return ts_check_launch();
}

// One wave per (token, head). `weight_head`: elements between two heads' weights (0: one weight of a head's size that all
// heads share; null weight: none). `silu_gate`: the gate is g sigmoid(g) instead of sigmoid(g).
template <typename TO>
__global__ void __launch_bounds__(ML_THREADS)
mlstm_finish_kernel(TO* __restrict__ out, const float* __restrict__ o, const float* __restrict__ weight,
                    const float* __restrict__ gate, int64_t gate_stride, int heads, int vdim, float eps, int64_t items,
                    int weight_head, int silu_gate) {
  const int wave = threadIdx.x / TS_WAVE, lane = threadIdx.x & (TS_WAVE - 1);
  const int64_t item = (int64_t)blockIdx.x * ML_WAVES + wave;
  if (item >= items) return;
  const int64_t t = item / heads;
  const int h = (int)(item - t * heads);
  const float* row = o + item * vdim;
  float squares = 0.f;
  for (int d = lane; d < vdim; d += TS_WAVE) squares = fmaf(row[d], row[d], squares);
  const float inv = 1.0f / sqrtf(wave_sum(squares) / (float)vdim + eps);
  for (int d = lane; d < vdim; d += TS_WAVE) {
    const float g = gate[t * gate_stride + h * vdim + d];
    const float w = weight ? weight[h * weight_head + d] : 1.0f;
    const float s = 1.0f / (1.0f + expf(-g));
    Num<TO>::st(out + item * vdim + d, row[d] * inv * w * (silu_gate ? g * s : s));
  }
}

extern "C" int ts_mlstm_finish(void* out, int out_dtype, const float* o, const float* weight, const float* gate,
                               int64_t gate_stride, int num_tokens, int heads, int vdim, float eps, int weight_head,
                               int silu_gate, hipStream_t stream) {
  if (num_tokens <= 0) return TS_OK;
  if (heads <= 0 || vdim <= 0 || (weight_head != 0 && weight_head != vdim)) return TS_BAD_SHAPE;
  const int64_t items = (int64_t)num_tokens * heads;
  const int64_t blocks = (items + ML_WAVES - 1) / ML_WAVES;
  if (blocks > 0x7fffffff) return TS_BAD_SHAPE;
  if (out_dtype == 0)
    mlstm_finish_kernel<float><<<(unsigned)blocks, ML_THREADS, 0, stream>>>((float*)out, o, weight, gate, gate_stride, heads, vdim, eps, items, weight_head, silu_gate);
  else if (out_dtype == 1)
    mlstm_finish_kernel<bf16_t><<<(unsigned)blocks, ML_THREADS, 0, stream>>>((bf16_t*)out, o, weight, gate, gate_stride, heads, vdim, eps, items, weight_head, silu_gate);
  else return TS_BAD_DTYPE;
  return ts_check_launch();
}

// ---- long portions: the recurrence in chunks of 64 tokens ------------------------------------------------------
// With b_t the sum of the log forget gates from the chunk's first token to t, c_j = i_j - b_j, and (S0, n0, m0) the
// state before the chunk, the recurrence unrolls to
//     m_t = b_t + max(m0, max_{j<=t} c_j),   S_t = exp(b_t + m0 - m_t) S0 + sum_{j<=t} exp(b_t + c_j - m_t) k_j v_j^T,
// so a chunk's read-outs are products over the chunk's tokens once S0 is known, and S0 follows from the chunks before
// by a short scan. Three kernels, each a workgroup per (chunk, head[, slice of 64 value columns]), all 32-bit:
//   * `mlstm_chunk_sums`: what a chunk adds to the state, sum_j exp(b_L + c_j - m_loc) k_j [v_j^T | 1] with
//     m_loc = b_L + max_j c_j, beside b_L and m_loc;
//   * `mlstm_chunk_scan`: element by element over a request's chunks in order, S <- exp(b_L + m - m') S + exp(m_loc - m') dS
//     with m' = max(b_L + m, m_loc); leaves every chunk's S0 where its sums were, m0 beside, and the last state in the slot;
//   * `mlstm_chunk_out`: o_t = (g_t S0^T q_t + sum_j P_tj v_j) / (max(|g_t n0.q_t + sum_j P_tj|, exp(-m_t)) + 1e-6) with
//     g_t = exp(b_t + m0 - m_t), P_tj = exp(b_t + c_j - m_t) q_t.k_j for j <= t.
#define MC_L 64
#define MC_THREADS 256
#define MC_PAD 68            // a transposed tile's row in shared memory: 16-byte pieces, rows four banks apart

struct ChunkGates { float b, c, gi; bool valid; };

// In the first wave, lane t: the gates of token t of the chunk, the running sum of the log forget gates and c.
static __device__ __forceinline__ ChunkGates mc_gates(const float* __restrict__ proj, int64_t stride, int tok0, int len, int i_at,
                                                      int f_at, float bi, float bf, float cap) {
  const int t = threadIdx.x;
  ChunkGates g;
  g.valid = t < len;
  float gf = 0.f;
  g.gi = 0.f;
  if (g.valid) {
    const float* row = proj + (int64_t)(tok0 + t) * stride;
    g.gi = cap * tanhf((row[i_at] + bi) / cap);
    const float zf = cap * tanhf((row[f_at] + bf) / cap);
    gf = fminf(zf, 0.f) - log1pf(expf(-fabsf(zf)));
  }
  float b = gf;
#pragma unroll
  for (int off = 1; off < TS_WAVE; off <<= 1) {
    const float up = __shfl_up(b, off, TS_WAVE);
    if (t >= off) b += up;
  }
  g.b = b;
  g.c = g.valid ? g.gi - b : -INFINITY;
  return g;
}

__global__ void __launch_bounds__(MC_THREADS)
mlstm_chunk_sums_kernel(float* __restrict__ buf, float* __restrict__ scalars, const float* __restrict__ proj, int64_t stride,
                        const float* __restrict__ i_bias, const float* __restrict__ f_bias, const int32_t* __restrict__ chunks,
                        int heads, int dim, int vdim, float cap) {
  __shared__ __attribute__((aligned(16))) float k_s[MC_L][MC_L];     // [token][dimension], times the token's weight
  __shared__ __attribute__((aligned(16))) float v_s[MC_L][MC_L];     // [token][value column]
  __shared__ float e_s[MC_L];
  const int chunk = blockIdx.x, h = blockIdx.y, v0 = blockIdx.z * MC_L;
  const int tok0 = chunks[4 * chunk], len = chunks[4 * chunk + 1];
  const int k_at = heads * dim + h * dim, v_at = 2 * heads * dim + h * vdim + v0;
  const int i_at = 2 * heads * dim + heads * vdim + h, f_at = i_at + heads;
  const int64_t per_head = (int64_t)dim * vdim + dim;
  float* dst = buf + ((int64_t)chunk * heads + h) * per_head;
  if (threadIdx.x < TS_WAVE) {
    const ChunkGates g = mc_gates(proj, stride, tok0, len, i_at, f_at, i_bias[h], f_bias[h], cap);
    const float bL = __shfl(g.b, len - 1, TS_WAVE);
    const float u = g.valid ? bL + g.c : -INFINITY;
    const float m_loc = wave_max(u);
    e_s[threadIdx.x] = g.valid ? expf(u - m_loc) : 0.f;
    if (threadIdx.x == 0 && blockIdx.z == 0) {
      scalars[((int64_t)chunk * heads + h) * 2] = bL;
      scalars[((int64_t)chunk * heads + h) * 2 + 1] = m_loc;
    }
  }
  for (int i = threadIdx.x; i < MC_L * MC_L; i += MC_THREADS) {
    const int j = i / MC_L, vv = i - j * MC_L;
    v_s[j][vv] = (j < len && v0 + vv < vdim) ? proj[(int64_t)(tok0 + j) * stride + v_at + vv] : 0.f;
  }
  const int ty = threadIdx.x / 16, tx = threadIdx.x & 15;
  for (int d0 = 0; d0 < dim; d0 += MC_L) {
    __syncthreads();                                         // (e_s is there; the tile's last readers are done)
    for (int i = threadIdx.x; i < MC_L * MC_L; i += MC_THREADS) {
      const int j = i / MC_L, dd = i - j * MC_L;
      k_s[j][dd] = (j < len && d0 + dd < dim) ? proj[(int64_t)(tok0 + j) * stride + k_at + d0 + dd] * e_s[j] : 0.f;
    }
    __syncthreads();
    float acc[4][4] = {};
    for (int j = 0; j < MC_L; ++j) {
      const float4 kk = *(const float4*)&k_s[j][4 * ty];
      const float4 vv = *(const float4*)&v_s[j][4 * tx];
      const float ka[4] = {kk.x, kk.y, kk.z, kk.w}, va[4] = {vv.x, vv.y, vv.z, vv.w};
#pragma unroll
      for (int a = 0; a < 4; ++a)
#pragma unroll
        for (int b = 0; b < 4; ++b) acc[a][b] = fmaf(ka[a], va[b], acc[a][b]);
    }
#pragma unroll
    for (int a = 0; a < 4; ++a)
#pragma unroll
      for (int b = 0; b < 4; ++b) {
        const int d = d0 + 4 * ty + a, v = v0 + 4 * tx + b;
        if (d < dim && v < vdim) dst[(int64_t)d * vdim + v] = acc[a][b];
      }
    if (blockIdx.z == 0 && threadIdx.x < MC_L && d0 + threadIdx.x < dim) {
      float sum = 0.f;
      for (int j = 0; j < MC_L; ++j) sum += k_s[j][threadIdx.x];
      dst[(int64_t)dim * vdim + d0 + threadIdx.x] = sum;
    }
  }
}

// chunk_cu: int32 [requests + 1], the requests' chunks lie in order from chunk_cu[s] to chunk_cu[s + 1]
__global__ void __launch_bounds__(MC_THREADS)
mlstm_chunk_scan_kernel(float* __restrict__ buf, float* __restrict__ m_start, const float* __restrict__ scalars,
                        float* __restrict__ state, const int32_t* __restrict__ chunk_cu, const int32_t* __restrict__ state_slots,
                        int heads, int dim, int vdim) {
  const int seq = blockIdx.x, h = blockIdx.y;
  const int64_t per_head = (int64_t)dim * vdim + dim;
  const int64_t e = (int64_t)blockIdx.z * MC_THREADS + threadIdx.x;
  float* st = state + ((int64_t)state_slots[seq] * heads + h) * (per_head + 1);
  const bool mine = e < per_head;
  float S = mine ? st[e] : 0.f;
  float m = st[per_head];
  const int c_end = chunk_cu[seq + 1];
  for (int c = chunk_cu[seq]; c < c_end; ++c) {
    const int64_t at = (int64_t)c * heads + h;
    const float bL = scalars[2 * at], m_loc = scalars[2 * at + 1];
    const float m_new = fmaxf(bL + m, m_loc);
    if (mine) {
      float* p = buf + at * per_head + e;
      const float add = *p;
      *p = S;
      S = expf(bL + m - m_new) * S + expf(m_loc - m_new) * add;
    }
    if (e == 0) m_start[at] = m;
    m = m_new;
  }
  if (mine) st[e] = S;
  // (the slot's m is read by every workgroup of this request and head, whenever each starts: it stays as it is here,
  // and the read-out kernel, which runs after all of them, writes the new one)
}

// One workgroup per (chunk, head, slice of 64 value columns); thread (ty, tx) owns tokens 4 ty .. + 3 and columns
// (of keys, then of values) 4 tx .. + 3.
__global__ void __launch_bounds__(MC_THREADS)
mlstm_chunk_out_kernel(float* __restrict__ out, const float* __restrict__ buf, const float* __restrict__ m_start,
                       const float* __restrict__ proj, int64_t stride, const float* __restrict__ i_bias,
                       const float* __restrict__ f_bias, float* __restrict__ state, const int32_t* __restrict__ chunks,
                       const int32_t* __restrict__ state_slots, int heads, int dim, int vdim, float cap, float q_scale) {
  __shared__ __attribute__((aligned(16))) float qT_s[MC_L][MC_PAD];  // [dimension][token]; later the weights [key token][token]
  __shared__ __attribute__((aligned(16))) float kT_s[MC_L][MC_PAD];  // [dimension][key token]
  __shared__ __attribute__((aligned(16))) float s0_s[MC_L][MC_L];    // [dimension][value column] of the state before the chunk
  __shared__ __attribute__((aligned(16))) float v_s[MC_L][MC_L];     // [key token][value column]
  __shared__ float n0_s[MC_L], b_s[MC_L], c_s[MC_L], m_s[MC_L], g_s[MC_L], nq_s[MC_L], den_s[MC_L];
  const int chunk = blockIdx.x, h = blockIdx.y, v0 = blockIdx.z * MC_L;
  const int tok0 = chunks[4 * chunk], len = chunks[4 * chunk + 1];
  const int q_at = h * dim, k_at = heads * dim + h * dim, v_at = 2 * heads * dim + h * vdim + v0;
  const int i_at = 2 * heads * dim + heads * vdim + h, f_at = i_at + heads;
  const int64_t per_head = (int64_t)dim * vdim + dim;
  const float* src = buf + ((int64_t)chunk * heads + h) * per_head;
  const float m0 = m_start[(int64_t)chunk * heads + h];
  if (threadIdx.x < TS_WAVE) {
    const ChunkGates g = mc_gates(proj, stride, tok0, len, i_at, f_at, i_bias[h], f_bias[h], cap);
    float top = g.c;                                         // the largest c up to this token
#pragma unroll
    for (int off = 1; off < TS_WAVE; off <<= 1) {
      const float up = __shfl_up(top, off, TS_WAVE);
      if ((int)threadIdx.x >= off) top = fmaxf(top, up);
    }
    const float m = g.b + fmaxf(m0, top);
    b_s[threadIdx.x] = g.b;
    c_s[threadIdx.x] = g.c;
    m_s[threadIdx.x] = m;
    g_s[threadIdx.x] = expf(g.b + m0 - m);
    nq_s[threadIdx.x] = 0.f;
    // the request's last chunk leaves the running maximum in the slot
    if (chunks[4 * chunk + 3] && blockIdx.z == 0 && (int)threadIdx.x == len - 1)
      state[((int64_t)state_slots[chunks[4 * chunk + 2]] * heads + h) * (per_head + 1) + per_head] = m;
  }
  for (int i = threadIdx.x; i < MC_L * MC_L; i += MC_THREADS) {
    const int j = i / MC_L, vv = i - j * MC_L;
    v_s[j][vv] = (j < len && v0 + vv < vdim) ? proj[(int64_t)(tok0 + j) * stride + v_at + vv] : 0.f;
  }
  const int ty = threadIdx.x / 16, tx = threadIdx.x & 15;
  float A[4][4] = {}, QS[4][4] = {};
  float nq = 0.f;
  for (int d0 = 0; d0 < dim; d0 += MC_L) {
    __syncthreads();
    for (int i = threadIdx.x; i < MC_L * MC_L; i += MC_THREADS) {
      const int t = i / MC_L, dd = i - t * MC_L;
      const bool in = t < len && d0 + dd < dim;
      const float* row = proj + (int64_t)(tok0 + t) * stride;
      qT_s[dd][t] = in ? row[q_at + d0 + dd] * q_scale : 0.f;
      kT_s[dd][t] = in ? row[k_at + d0 + dd] : 0.f;
      const int d = i / MC_L, vv = i - d * MC_L;             // (the same index read as [dimension][value column])
      s0_s[d][vv] = (d0 + d < dim && v0 + vv < vdim) ? src[(int64_t)(d0 + d) * vdim + v0 + vv] : 0.f;
    }
    if (threadIdx.x < MC_L) n0_s[threadIdx.x] = d0 + threadIdx.x < dim ? src[(int64_t)dim * vdim + d0 + threadIdx.x] : 0.f;
    __syncthreads();
    for (int dd = 0; dd < MC_L; ++dd) {
      const float4 q4 = *(const float4*)&qT_s[dd][4 * ty];
      const float4 k4 = *(const float4*)&kT_s[dd][4 * tx];
      const float4 s4 = *(const float4*)&s0_s[dd][4 * tx];
      const float qa[4] = {q4.x, q4.y, q4.z, q4.w}, ka[4] = {k4.x, k4.y, k4.z, k4.w}, sa[4] = {s4.x, s4.y, s4.z, s4.w};
#pragma unroll
      for (int a = 0; a < 4; ++a)
#pragma unroll
        for (int b = 0; b < 4; ++b) {
          A[a][b] = fmaf(qa[a], ka[b], A[a][b]);
          QS[a][b] = fmaf(qa[a], sa[b], QS[a][b]);
        }
    }
    if (threadIdx.x < MC_L)
      for (int dd = 0; dd < MC_L; ++dd) nq = fmaf(qT_s[dd][threadIdx.x], n0_s[dd], nq);
  }
  __syncthreads();                                           // (the last tile's readers are done: qT_s becomes the weights)
#pragma unroll
  for (int a = 0; a < 4; ++a)
#pragma unroll
    for (int b = 0; b < 4; ++b) {
      const int t = 4 * ty + a, j = 4 * tx + b;
      const bool seen = j <= t && t < len;
      qT_s[j][t] = seen ? A[a][b] * expf(b_s[t] + c_s[j] - m_s[t]) : 0.f;
    }
  __syncthreads();
  if (threadIdx.x < MC_L) {
    float sum = g_s[threadIdx.x] * nq;
    for (int j = 0; j < MC_L; ++j) sum += qT_s[j][threadIdx.x];
    den_s[threadIdx.x] = fmaxf(fabsf(sum), expf(-m_s[threadIdx.x])) + 1e-6f;
  }
  float num[4][4];
#pragma unroll
  for (int a = 0; a < 4; ++a)
#pragma unroll
    for (int b = 0; b < 4; ++b) num[a][b] = g_s[4 * ty + a] * QS[a][b];
  for (int j = 0; j < MC_L; ++j) {
    const float4 p4 = *(const float4*)&qT_s[j][4 * ty];
    const float4 v4 = *(const float4*)&v_s[j][4 * tx];
    const float pa[4] = {p4.x, p4.y, p4.z, p4.w}, va[4] = {v4.x, v4.y, v4.z, v4.w};
#pragma unroll
    for (int a = 0; a < 4; ++a)
#pragma unroll
      for (int b = 0; b < 4; ++b) num[a][b] = fmaf(pa[a], va[b], num[a][b]);
  }
  __syncthreads();                                           // (den_s is there)
#pragma unroll
  for (int a = 0; a < 4; ++a)
#pragma unroll
    for (int b = 0; b < 4; ++b) {
      const int t = 4 * ty + a, v = v0 + 4 * tx + b;
      if (t < len && v < vdim) out[(int64_t)(tok0 + t) * heads * vdim + h * vdim + v] = num[a][b] / den_s[t];
    }
}

// chunks: int32 [num_chunks, 4] = (first token of the step, tokens 1 .. 64, request of the step, 1 if the request's last
// chunk), a request's chunks in order and side by side; chunk_cu: int32 [requests + 1]; buf: float32
// [num_chunks, heads, dim vdim + dim]; scalars: float32 [num_chunks, heads, 2]; m_start: float32 [num_chunks, heads].
extern "C" int ts_mlstm_scan_chunks(float* out, const float* proj, int64_t stride, const float* i_bias, const float* f_bias,
                                    float* state, const int32_t* chunks, const int32_t* chunk_cu, const int32_t* state_slots,
                                    float* buf, float* scalars, float* m_start, int num_chunks, int num_seqs, int heads, int dim,
                                    int vdim, float cap, float q_scale, hipStream_t stream) {
  if (num_chunks <= 0 || num_seqs <= 0) return TS_OK;
  if (heads <= 0 || heads > 65535 || dim <= 0 || vdim <= 0 || !(cap > 0.f)) return TS_BAD_SHAPE;
  const int slices = (vdim + MC_L - 1) / MC_L;
  const int64_t per_head = (int64_t)dim * vdim + dim;
  const int64_t scan_blocks = (per_head + MC_THREADS - 1) / MC_THREADS;
  if (slices > 65535 || scan_blocks > 65535) return TS_BAD_SHAPE;
  mlstm_chunk_sums_kernel<<<dim3(num_chunks, heads, slices), MC_THREADS, 0, stream>>>(buf, scalars, proj, stride, i_bias, f_bias,
                                                                                       chunks, heads, dim, vdim, cap);
  mlstm_chunk_scan_kernel<<<dim3(num_seqs, heads, (unsigned)scan_blocks), MC_THREADS, 0, stream>>>(buf, m_start, scalars, state, chunk_cu,
                                                                                                   state_slots, heads, dim, vdim);
  mlstm_chunk_out_kernel<<<dim3(num_chunks, heads, slices), MC_THREADS, 0, stream>>>(out, buf, m_start, proj, stride, i_bias, f_bias,
                                                                                      state, chunks, state_slots, heads, dim, vdim, cap,
                                                                                      q_scale);
  return ts_check_launch();
}
