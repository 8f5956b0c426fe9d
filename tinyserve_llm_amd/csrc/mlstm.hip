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

// One wave per (token, head).
template <typename TO>
__global__ void __launch_bounds__(ML_THREADS)
mlstm_finish_kernel(TO* __restrict__ out, const float* __restrict__ o, const float* __restrict__ weight,
                    const float* __restrict__ gate, int64_t gate_stride, int heads, int vdim, float eps, int64_t items) {
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
    Num<TO>::st(out + item * vdim + d, row[d] * inv * weight[h * vdim + d] / (1.0f + expf(-g)));
  }
}

extern "C" int ts_mlstm_finish(void* out, int out_dtype, const float* o, const float* weight, const float* gate,
                               int64_t gate_stride, int num_tokens, int heads, int vdim, float eps, hipStream_t stream) {
  if (num_tokens <= 0) return TS_OK;
  if (heads <= 0 || vdim <= 0) return TS_BAD_SHAPE;
  const int64_t items = (int64_t)num_tokens * heads;
  const int64_t blocks = (items + ML_WAVES - 1) / ML_WAVES;
  if (blocks > 0x7fffffff) return TS_BAD_SHAPE;
  if (out_dtype == 0)
    mlstm_finish_kernel<float><<<(unsigned)blocks, ML_THREADS, 0, stream>>>((float*)out, o, weight, gate, gate_stride, heads, vdim, eps, items);
  else if (out_dtype == 1)
    mlstm_finish_kernel<bf16_t><<<(unsigned)blocks, ML_THREADS, 0, stream>>>((bf16_t*)out, o, weight, gate, gate_stride, heads, vdim, eps, items);
  else return TS_BAD_DTYPE;
  return ts_check_launch();
}
