// A residual stream kept in 32-bit floats whatever the storage type of the activations around it:
//   * token rows of the embedding table into the stream,
//   * the stream's update x += mult * (a + b + bias) by what two parallel branches (or one) have made,
//     with up to two weighted RMS norms of the updated row on the way out (both share the row's mean
//     square, which is taken once), or the norms alone, or the norms of a few picked rows,
//   * a bias and an activation between two projections of a dense feed-forward.
// Sums, mean squares, roots and scalings are 32-bit; what leaves for a projection is rounded to the
// activations' storage type only at the store. Every row is worked on by one workgroup and by itself:
// a row's result does not depend on the rows beside it.
#include "common.h"

#define RS_THREADS 256

// value of element i of a row stored as float (code 0) or bfloat16 (code 1)
static __device__ __forceinline__ float rs_load(const void* p, int code, int64_t i) {
  return code == 0 ? ((const float*)p)[i] : bf2f(((const bf16_t*)p)[i]);
}
static __device__ __forceinline__ void rs_store(void* p, int code, int64_t i, float v) {
  if (code == 0) ((float*)p)[i] = v;
  else ((bf16_t*)p)[i] = f2bf(v);
}

static __device__ __forceinline__ float block_sum(float v, float* scratch) {
  v = wave_sum(v);
  const int wave = threadIdx.x / TS_WAVE, lane = threadIdx.x & (TS_WAVE - 1);
  __syncthreads();                 // (scratch may still be read from a sum before)
  if (lane == 0) scratch[wave] = v;
  __syncthreads();
  float total = 0.f;
  for (int w = 0; w < RS_THREADS / TS_WAVE; ++w) total += scratch[w];
  return total;
}

__global__ void __launch_bounds__(RS_THREADS)
embedding_stream_kernel(float* __restrict__ out, const void* __restrict__ table, const int32_t* __restrict__ ids,
                        int hidden, int code) {
  const int64_t t = blockIdx.x;
  const int64_t src = (int64_t)ids[t] * hidden;
  for (int i = threadIdx.x; i < hidden; i += RS_THREADS) out[t * hidden + i] = rs_load(table, code, src + i);
}

extern "C" int ts_embedding_stream(float* out, const void* table, const int32_t* ids, int num_tokens, int hidden,
                                   int dtype, hipStream_t stream) {
  if (num_tokens <= 0) return TS_OK;
  if (hidden <= 0) return TS_BAD_SHAPE;
  if (dtype != 0 && dtype != 1) return TS_BAD_DTYPE;
  embedding_stream_kernel<<<num_tokens, RS_THREADS, 0, stream>>>(out, table, ids, hidden, dtype);
  return ts_check_launch();
}

// Row r of the grid: stream row t = rows ? rows[r] : r.
//   update (a or b given; rows must be null): x[t] += mult * (a[t] + b[t] + bias), written back
//   norms (h1 / h2 given): h[r] = x[t] / sqrt(mean(x[t]^2) + eps) * w, of the updated row
__global__ void __launch_bounds__(RS_THREADS)
stream_update_norm_kernel(float* __restrict__ x, const void* __restrict__ a, int a_code, const void* __restrict__ b,
                          int b_code, const void* __restrict__ bias, int bias_code, float mult,
                          void* __restrict__ h1, void* __restrict__ h2, int h_code, const void* __restrict__ w1,
                          const void* __restrict__ w2, int w_code, float eps, const int32_t* __restrict__ rows,
                          int width) {
  __shared__ float scratch[RS_THREADS / TS_WAVE];
  const int64_t r = blockIdx.x;
  const int64_t t = rows ? rows[r] : r;
  float* xr = x + t * width;
  const bool update = a || b;
  float squares = 0.f;
  for (int i = threadIdx.x; i < width; i += RS_THREADS) {
    float v = xr[i];
    if (update) {
      float add = 0.f;
      if (a) add += rs_load(a, a_code, t * width + i);
      if (b) add += rs_load(b, b_code, t * width + i);
      if (bias) add += rs_load(bias, bias_code, i);
      v = fmaf(mult, add, v);
      xr[i] = v;
    }
    squares = fmaf(v, v, squares);
  }
  if (!h1 && !h2) return;
  const float total = block_sum(squares, scratch);
  const float inv = 1.0f / sqrtf(total / (float)width + eps);
  for (int i = threadIdx.x; i < width; i += RS_THREADS) {
    const float v = xr[i] * inv;       // (this thread's own elements, as it has just written them)
    if (h1) rs_store(h1, h_code, r * width + i, v * rs_load(w1, w_code, i));
    if (h2) rs_store(h2, h_code, r * width + i, v * rs_load(w2, w_code, i));
  }
}

// The same for rows of up to RS_THREADS * HELD elements whose branches are 32-bit and whose norms' weights, bias and
// outputs share the type H: every load of the row goes out before the first is used (no branch on a storage type
// or on whether an operand is there stands between two loads: an operand that is not there is read from another of
// its shape and counts times 0), and the updated row stays in registers between the sum of squares and the scaling.
#define RS_HELD 16
template <typename H, typename W, int HELD, bool NORMS>
__global__ void __launch_bounds__(RS_THREADS)
stream_update_norm_held_kernel(float* __restrict__ x, const float* __restrict__ a, const float* __restrict__ b,
                               const H* __restrict__ bias, float mult, H* __restrict__ h1, H* __restrict__ h2,
                               const W* __restrict__ w1, const W* __restrict__ w2, float eps,
                               const int32_t* __restrict__ rows, int width) {
  __shared__ float scratch[RS_THREADS / TS_WAVE];
  const int64_t r = blockIdx.x;
  const int64_t t = rows ? rows[r] : r;
  float* xr = x + t * width;
  const bool update = a || b, bias_on = bias && update;
  // an operand that is not there is read from another of its size (the row itself; a norm's weight) and not used
  const float* ar = (a ? a : x) + t * width;
  const float* br = (b ? b : x) + t * width;
  const W* wa = w1 ? w1 : w2;
  const W* wb = w2 ? w2 : w1;
  const H* bs = bias ? bias : (NORMS ? (const H*)wa : (const H*)xr);
  float v[HELD], va[HELD], vb[HELD], vbias[HELD], wva[HELD], wvb[HELD];
#pragma unroll
  for (int j = 0; j < HELD; ++j) {
    const int i = min(threadIdx.x + j * RS_THREADS, width - 1);     // (a lane beyond the row reads its last element, and stores nothing)
    v[j] = xr[i];
    va[j] = ar[i];
    vb[j] = br[i];
    vbias[j] = Num<H>::ld(bs + i);
    if constexpr (NORMS) {
      wva[j] = Num<W>::ld(wa + i);
      wvb[j] = Num<W>::ld(wb + i);
    }
  }
  float squares = 0.f;
#pragma unroll
  for (int j = 0; j < HELD; ++j) {
    const int i = threadIdx.x + j * RS_THREADS;
    // x + mult * (a + b + bias), the sum of the branches first
    const float add = (a ? va[j] : 0.f) + (b ? vb[j] : 0.f) + (bias_on ? vbias[j] : 0.f);
    v[j] = update ? fmaf(mult, add, v[j]) : v[j];
    if (update && i < width) xr[i] = v[j];
    squares = i < width ? fmaf(v[j], v[j], squares) : squares;
  }
  if constexpr (NORMS) {
    const float total = block_sum(squares, scratch);
    const float inv = 1.0f / sqrtf(total / (float)width + eps);
#pragma unroll
    for (int j = 0; j < HELD; ++j) {
      const int i = threadIdx.x + j * RS_THREADS;
      if (i < width) {
        const float n = v[j] * inv;
        if (h1) Num<H>::st(h1 + r * width + i, n * wva[j]);
        if (h2) Num<H>::st(h2 + r * width + i, n * wvb[j]);
      }
    }
  }
}

extern "C" int ts_stream_update_norm(float* x, const void* a, int a_dtype, const void* b, int b_dtype, const void* bias,
                                     int bias_dtype, float mult, void* h1, void* h2, int h_dtype, const void* w1,
                                     const void* w2, int w_dtype, float eps, const int32_t* rows, int num_rows, int width,
                                     hipStream_t stream) {
  if (num_rows <= 0) return TS_OK;
  if (width <= 0 || !x || (rows && (a || b)) || (h1 && !w1) || (h2 && !w2)) return TS_BAD_SHAPE;
  for (int code : {a_dtype, b_dtype, bias_dtype, h_dtype, w_dtype})
    if (code != 0 && code != 1) return TS_BAD_DTYPE;
  const bool typed = (!a || a_dtype == 0) && (!b || b_dtype == 0) && width <= RS_THREADS * RS_HELD &&
                     (!bias || bias_dtype == h_dtype || !(h1 || h2)) && (!(h1 || h2) || w_dtype == h_dtype || w_dtype == 0);
  if (typed) {
    const int code = (h1 || h2) ? h_dtype : bias_dtype;
#define RS_TYPED_W(H, W, HELD, NN) \
  stream_update_norm_held_kernel<H, W, HELD, NN><<<num_rows, RS_THREADS, 0, stream>>>(x, (const float*)a, (const float*)b, \
      (const H*)bias, mult, (H*)h1, (H*)h2, (const W*)w1, (const W*)w2, eps, rows, width)
  // (norm weights kept in 32-bit beside outputs in bfloat16: norms whose weights are sums made in 32-bit)
#define RS_TYPED_N(H, HELD, NN) \
  if (sizeof(H) == 2 && w_dtype == 0 && (h1 || h2)) { RS_TYPED_W(H, float, HELD, NN); } else { RS_TYPED_W(H, H, HELD, NN); }
#define RS_TYPED(H, HELD) if (h1 || h2) { RS_TYPED_N(H, HELD, true); } else { RS_TYPED_N(H, HELD, false); }
#define RS_TYPED_H(H) \
  if (width <= RS_THREADS * 4) { RS_TYPED(H, 4); } else if (width <= RS_THREADS * 8) { RS_TYPED(H, 8); } else { RS_TYPED(H, RS_HELD); }
    if (code == 0) { RS_TYPED_H(float) } else { RS_TYPED_H(bf16_t) }
#undef RS_TYPED_H
#undef RS_TYPED
#undef RS_TYPED_N
#undef RS_TYPED_W
    return ts_check_launch();
  }
  stream_update_norm_kernel<<<num_rows, RS_THREADS, 0, stream>>>(x, a, a_dtype, b, b_dtype, bias, bias_dtype, mult, h1, h2,
                                                                 h_dtype, w1, w2, w_dtype, eps, rows, width);
  return ts_check_launch();
}

// out[t, i] = act(in[t, i] + bias[i]); act 0: none, 1: relu squared, 2: gelu (tanh form), 3: silu, 4: tanh
static __device__ __forceinline__ float rs_activate(float z, int act) {
  switch (act) {
    case 1: { const float r = fmaxf(z, 0.f); return r * r; }
    case 2: return 0.5f * z * (1.0f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z)));
    case 3: return z / (1.0f + expf(-z));
    case 4: return tanhf(z);
    default: return z;
  }
}

__global__ void __launch_bounds__(RS_THREADS)
bias_activation_kernel(void* __restrict__ out, int out_code, const void* __restrict__ in, int in_code,
                       const void* __restrict__ bias, int bias_code, int64_t total, int width, int act) {
  for (int64_t idx = (int64_t)blockIdx.x * RS_THREADS + threadIdx.x; idx < total; idx += (int64_t)gridDim.x * RS_THREADS) {
    const int i = (int)(idx % width);
    float z = rs_load(in, in_code, idx);
    if (bias) z += rs_load(bias, bias_code, i);
    rs_store(out, out_code, idx, rs_activate(z, act));
  }
}

// Four elements a thread (rows of a multiple of four elements, 16-byte aligned 32-bit input, bfloat16 or 32-bit output).
template <typename TO>
__global__ void __launch_bounds__(RS_THREADS)
bias_activation_by4_kernel(TO* __restrict__ out, const float* __restrict__ in, const void* __restrict__ bias, int bias_code,
                           int64_t fours, int width, int act) {
  for (int64_t idx = (int64_t)blockIdx.x * RS_THREADS + threadIdx.x; idx < fours; idx += (int64_t)gridDim.x * RS_THREADS) {
    const int i = (int)((idx * 4) % width);
    const float4 z4 = *(const float4*)(in + idx * 4);
    float z[4] = {z4.x, z4.y, z4.z, z4.w};
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      if (bias) z[k] += rs_load(bias, bias_code, i + k);
      z[k] = rs_activate(z[k], act);
    }
    if constexpr (sizeof(TO) == 4) {
      *(float4*)((float*)out + idx * 4) = make_float4(z[0], z[1], z[2], z[3]);
    } else {
      uint2 packed;
      packed.x = (uint32_t)f2bf(z[0]) | ((uint32_t)f2bf(z[1]) << 16);
      packed.y = (uint32_t)f2bf(z[2]) | ((uint32_t)f2bf(z[3]) << 16);
      *(uint2*)((bf16_t*)out + idx * 4) = packed;
    }
  }
}

extern "C" int ts_bias_activation(void* out, int out_dtype, const void* in, int in_dtype, const void* bias, int bias_dtype,
                                  int num_rows, int width, int act, hipStream_t stream) {
  if (num_rows <= 0) return TS_OK;
  if (width <= 0 || act < 0 || act > 4) return TS_BAD_SHAPE;
  for (int code : {out_dtype, in_dtype, bias_dtype})
    if (code != 0 && code != 1) return TS_BAD_DTYPE;
  const int64_t total = (int64_t)num_rows * width;
  if (in_dtype == 0 && width % 4 == 0 && (((uintptr_t)in | (uintptr_t)out) & 15) == 0) {
    const int64_t fours = total / 4;
    int64_t groups = (fours + RS_THREADS - 1) / RS_THREADS;
    if (groups > 16384) groups = 16384;
    if (out_dtype == 0)
      bias_activation_by4_kernel<float><<<(unsigned)groups, RS_THREADS, 0, stream>>>((float*)out, (const float*)in, bias, bias_dtype,
                                                                                    fours, width, act);
    else
      bias_activation_by4_kernel<bf16_t><<<(unsigned)groups, RS_THREADS, 0, stream>>>((bf16_t*)out, (const float*)in, bias, bias_dtype,
                                                                                     fours, width, act);
    return ts_check_launch();
  }
  int64_t blocks = (total + RS_THREADS - 1) / RS_THREADS;
  if (blocks > 16384) blocks = 16384;
  bias_activation_kernel<<<(unsigned)blocks, RS_THREADS, 0, stream>>>(out, out_dtype, in, in_dtype, bias, bias_dtype, total,
                                                                     width, act);
  return ts_check_launch();
}

// ---- a branch that passes an RMS norm of its own (and a learned scale per channel) before it is added ----
// Row r: x[r] += a[r] / sqrt(mean(a[r]^2) + post_eps) * post_w * scale   (scale may be absent),
// then, if asked for, h[r] = x[r] / sqrt(mean(x[r]^2) + eps) * w (the next norm), or h[r] = x[r] itself (w absent),
// rounded to h's storage type at the store. A workgroup a row; every sum is taken by the same tree whatever the batch.
__global__ void __launch_bounds__(RS_THREADS)
stream_post_norm_kernel(float* __restrict__ x, const float* __restrict__ a, const float* __restrict__ post_w,
                        const float* __restrict__ scale, float post_eps, void* __restrict__ h, int h_code,
                        const float* __restrict__ w, float eps, int width) {
  __shared__ float scratch[RS_THREADS / TS_WAVE];
  const int64_t r = blockIdx.x;
  float* xr = x + r * width;
  const float* ar = a + r * width;
  float squares = 0.f;
  for (int i = threadIdx.x; i < width; i += RS_THREADS) squares = fmaf(ar[i], ar[i], squares);
  const float inv_a = 1.0f / sqrtf(block_sum(squares, scratch) / (float)width + post_eps);
  squares = 0.f;
  for (int i = threadIdx.x; i < width; i += RS_THREADS) {
    float add = ar[i] * inv_a * post_w[i];
    if (scale) add *= scale[i];
    const float v = xr[i] + add;
    xr[i] = v;
    squares = fmaf(v, v, squares);
  }
  if (!h) return;
  float inv = 1.0f;
  if (w) inv = 1.0f / sqrtf(block_sum(squares, scratch) / (float)width + eps);
  for (int i = threadIdx.x; i < width; i += RS_THREADS)      // (this thread's own elements, as it has just written them)
    rs_store(h, h_code, r * width + i, w ? xr[i] * inv * w[i] : xr[i]);
}

// The same for rows of up to RS_THREADS * HELD elements: every load of the row, the branch and the weights goes out before
// the first is used, and the row stays in registers between the sums of squares and the scalings (a lane beyond the row
// reads the row's last element and stores nothing). The sums are taken by the same tree over the same lanes' parts.
template <typename H, int HELD>
__global__ void __launch_bounds__(RS_THREADS)
stream_post_norm_held_kernel(float* __restrict__ x, const float* __restrict__ a, const float* __restrict__ post_w,
                             const float* __restrict__ scale, float post_eps, H* __restrict__ h, const float* __restrict__ w,
                             float eps, int width) {
  __shared__ float scratch[RS_THREADS / TS_WAVE];
  const int64_t r = blockIdx.x;
  float* xr = x + r * width;
  const float* ar = a + r * width;
  const float* sc = scale ? scale : post_w;
  const float* wn = w ? w : post_w;
  float v[HELD], va[HELD], pw[HELD], ps[HELD], nw[HELD];
#pragma unroll
  for (int j = 0; j < HELD; ++j) {
    const int i = min(threadIdx.x + j * RS_THREADS, width - 1);
    v[j] = xr[i];
    va[j] = ar[i];
    pw[j] = post_w[i];
    ps[j] = sc[i];
    nw[j] = wn[i];
  }
  float squares = 0.f;
#pragma unroll
  for (int j = 0; j < HELD; ++j) squares = threadIdx.x + j * RS_THREADS < width ? fmaf(va[j], va[j], squares) : squares;
  const float inv_a = 1.0f / sqrtf(block_sum(squares, scratch) / (float)width + post_eps);
  squares = 0.f;
#pragma unroll
  for (int j = 0; j < HELD; ++j) {
    const int i = threadIdx.x + j * RS_THREADS;
    float add = va[j] * inv_a * pw[j];
    if (scale) add *= ps[j];
    v[j] += add;
    if (i < width) {
      xr[i] = v[j];
      squares = fmaf(v[j], v[j], squares);
    }
  }
  if (!h) return;
  float inv = 1.0f;
  if (w) inv = 1.0f / sqrtf(block_sum(squares, scratch) / (float)width + eps);
#pragma unroll
  for (int j = 0; j < HELD; ++j) {
    const int i = threadIdx.x + j * RS_THREADS;
    if (i < width) Num<H>::st(h + r * width + i, w ? v[j] * inv * nw[j] : v[j]);
  }
}

extern "C" int ts_stream_post_norm(float* x, const float* a, const float* post_w, const float* scale, float post_eps, void* h,
                                   int h_dtype, const float* w, float eps, int num_rows, int width, hipStream_t stream) {
  if (num_rows <= 0) return TS_OK;
  if (width <= 0 || !x || !a || !post_w) return TS_BAD_SHAPE;
  if (h_dtype != 0 && h_dtype != 1) return TS_BAD_DTYPE;
  if (width <= RS_THREADS * RS_HELD) {
#define RS_POST(H, HELD) \
    stream_post_norm_held_kernel<H, HELD><<<num_rows, RS_THREADS, 0, stream>>>(x, a, post_w, scale, post_eps, (H*)h, w, eps, width)
#define RS_POST_H(H) \
    if (width <= RS_THREADS * 4) { RS_POST(H, 4); } else if (width <= RS_THREADS * 8) { RS_POST(H, 8); } else { RS_POST(H, RS_HELD); }
    if (h_dtype == 0) { RS_POST_H(float) } else { RS_POST_H(bf16_t) }
#undef RS_POST_H
#undef RS_POST
    return ts_check_launch();
  }
  stream_post_norm_kernel<<<num_rows, RS_THREADS, 0, stream>>>(x, a, post_w, scale, post_eps, h, h_dtype, w, eps, width);
  return ts_check_launch();
}

// out = sa * a + sb * b, element by element (what two mixers side by side have made, each with its own factor)
__global__ void __launch_bounds__(RS_THREADS)
scaled_sum_kernel(float* __restrict__ out, const float* __restrict__ a, float sa, const float* __restrict__ b, float sb, int64_t total) {
  for (int64_t i = (int64_t)blockIdx.x * RS_THREADS + threadIdx.x; i < total; i += (int64_t)gridDim.x * RS_THREADS)
    out[i] = fmaf(sb, b[i], sa * a[i]);
}

extern "C" int ts_scaled_sum(float* out, const float* a, float sa, const float* b, float sb, int64_t total, hipStream_t stream) {
  if (total <= 0) return TS_OK;
  int64_t blocks = (total + RS_THREADS - 1) / RS_THREADS;
  if (blocks > 16384) blocks = 16384;
  scaled_sum_kernel<<<(unsigned)blocks, RS_THREADS, 0, stream>>>(out, a, sa, b, sb, total);
  return ts_check_launch();
}

// out[t, j] = act(sums[t, j]) * table[ids[t], offset + j]: a gate's sums times a stretch of a token's row of a table
__global__ void __launch_bounds__(RS_THREADS)
gather_gate_kernel(void* __restrict__ out, int out_code, const float* __restrict__ sums, const void* __restrict__ table,
                   int table_code, int64_t table_stride, int offset, const int32_t* __restrict__ ids, int64_t total, int width, int act) {
  for (int64_t idx = (int64_t)blockIdx.x * RS_THREADS + threadIdx.x; idx < total; idx += (int64_t)gridDim.x * RS_THREADS) {
    const int64_t t = idx / width;
    const int j = (int)(idx - t * width);
    rs_store(out, out_code, idx, rs_activate(sums[idx], act) * rs_load(table, table_code, (int64_t)ids[t] * table_stride + offset + j));
  }
}

extern "C" int ts_gather_gate(void* out, int out_dtype, const float* sums, const void* table, int table_dtype, int64_t table_stride,
                              int offset, const int32_t* ids, int num_rows, int width, int act, hipStream_t stream) {
  if (num_rows <= 0) return TS_OK;
  if (width <= 0 || offset < 0 || table_stride < offset + width || act < 0 || act > 4) return TS_BAD_SHAPE;
  if ((out_dtype | table_dtype) & ~1) return TS_BAD_DTYPE;
  const int64_t total = (int64_t)num_rows * width;
  int64_t blocks = (total + RS_THREADS - 1) / RS_THREADS;
  if (blocks > 16384) blocks = 16384;
  gather_gate_kernel<<<(unsigned)blocks, RS_THREADS, 0, stream>>>(out, out_dtype, sums, table, table_dtype, table_stride, offset, ids,
                                                                 total, width, act);
  return ts_check_launch();
}
