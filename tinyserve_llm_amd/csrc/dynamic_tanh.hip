// The dynamic-tanh norm n(x) = tanh(alpha x) w + b (alpha one scalar, w and b vectors; no mean, no
// variance: every element by itself) on a residual stream that is kept in 32-bit floats:
//   * `ts_dyt`: the norm of given rows (optionally of x + residual, with the sum written out, and
//     optionally of a few picked rows),
//   * `ts_dyt_stream`: the stream's update x += n_post(a) by what a branch has made, passed through the
//     norm that follows the branch, and on the way out the norm that precedes the next branch, n_pre(x),
//     rounded to the projections' storage type only at the store,
//   * `ts_embedding_dyt_stream`: token rows of the table times a scale, through a norm, into the stream.
// alpha, w and b are 32-bit; alpha is read from device memory, so a recorded step needs no host value.
// The hyperbolic tangent is taken as 1 - 2 / (exp(2 z) + 1) with the 32-bit library exponential.
#include "common.h"

#define DT_THREADS 256

static __device__ __forceinline__ float dt_load(const void* p, int code, int64_t i) {
  return code == 0 ? ((const float*)p)[i] : bf2f(((const bf16_t*)p)[i]);
}
static __device__ __forceinline__ void dt_store(void* p, int code, int64_t i, float v) {
  if (code == 0) ((float*)p)[i] = v;
  else ((bf16_t*)p)[i] = f2bf(v);
}
static __device__ __forceinline__ float dt_tanh(float z) { return tanhf(z); }

__global__ void __launch_bounds__(DT_THREADS)
dyt_kernel(void* __restrict__ out, int out_code, const void* __restrict__ x, int x_code, const void* __restrict__ residual,
           int r_code, void* __restrict__ sum_out, int s_code, const float* __restrict__ alpha, const float* __restrict__ w,
           const float* __restrict__ b, const int32_t* __restrict__ rows, int width) {
  const int64_t r = blockIdx.x;
  const int64_t t = rows ? rows[r] : r;
  const float a = alpha[0];
  for (int i = threadIdx.x; i < width; i += DT_THREADS) {
    float v = dt_load(x, x_code, t * width + i);
    if (residual) {
      v += dt_load(residual, r_code, t * width + i);
      if (sum_out) {
        dt_store(sum_out, s_code, t * width + i, v);
        if (s_code == 1) v = bf2f(f2bf(v));      // (the norm reads the stream as it is kept)
      }
    }
    dt_store(out, out_code, r * width + i, fmaf(dt_tanh(a * v), w[i], b[i]));
  }
}

extern "C" int ts_dyt(void* out, int out_dtype, const void* x, int x_dtype, const void* residual, int r_dtype, void* sum_out,
                      int s_dtype, const float* alpha, const float* w, const float* b, const int32_t* rows, int n, int width,
                      hipStream_t stream) {
  if (n <= 0) return TS_OK;
  if (width <= 0 || (rows && residual)) return TS_BAD_SHAPE;
  if ((out_dtype | x_dtype | r_dtype | s_dtype) & ~1) return TS_BAD_DTYPE;
  dyt_kernel<<<n, DT_THREADS, 0, stream>>>(out, out_dtype, x, x_dtype, residual, r_dtype, sum_out, s_dtype, alpha, w, b, rows,
                                          width);
  return ts_check_launch();
}

// Four consecutive elements a thread, all loads of a thread before its first use.
__global__ void __launch_bounds__(DT_THREADS)
dyt_stream_kernel(float* __restrict__ x, const void* __restrict__ a, int a_code, const float* __restrict__ post_alpha,
                  const float* __restrict__ post_w, const float* __restrict__ post_b, void* __restrict__ out, int out_code,
                  const float* __restrict__ pre_alpha, const float* __restrict__ pre_w, const float* __restrict__ pre_b,
                  int width, int64_t total) {
  const int64_t at = ((int64_t)blockIdx.x * DT_THREADS + threadIdx.x) * 4;
  if (at >= total) return;
  const int col = (int)(at % width);            // (width a multiple of 4: the four share a row)
  float4 xv = *(const float4*)(x + at);
  float v[4] = {xv.x, xv.y, xv.z, xv.w};
  if (a) {
    float av[4];
    if (a_code == 0) {
      const float4 t = *(const float4*)((const float*)a + at);
      av[0] = t.x; av[1] = t.y; av[2] = t.z; av[3] = t.w;
    } else {
      const uint2 t = *(const uint2*)((const bf16_t*)a + at);
      av[0] = __uint_as_float(t.x << 16); av[1] = __uint_as_float(t.x & 0xffff0000u);
      av[2] = __uint_as_float(t.y << 16); av[3] = __uint_as_float(t.y & 0xffff0000u);
    }
    if (post_alpha) {
      const float pa = post_alpha[0];
      const float4 pw = *(const float4*)(post_w + col), pb = *(const float4*)(post_b + col);
      av[0] = fmaf(dt_tanh(pa * av[0]), pw.x, pb.x);
      av[1] = fmaf(dt_tanh(pa * av[1]), pw.y, pb.y);
      av[2] = fmaf(dt_tanh(pa * av[2]), pw.z, pb.z);
      av[3] = fmaf(dt_tanh(pa * av[3]), pw.w, pb.w);
    }
#pragma unroll
    for (int e = 0; e < 4; ++e) v[e] += av[e];
    *(float4*)(x + at) = make_float4(v[0], v[1], v[2], v[3]);
  }
  if (out) {
    const float na = pre_alpha[0];
    const float4 nw = *(const float4*)(pre_w + col), nb = *(const float4*)(pre_b + col);
    const float y0 = fmaf(dt_tanh(na * v[0]), nw.x, nb.x), y1 = fmaf(dt_tanh(na * v[1]), nw.y, nb.y);
    const float y2 = fmaf(dt_tanh(na * v[2]), nw.z, nb.z), y3 = fmaf(dt_tanh(na * v[3]), nw.w, nb.w);
    if (out_code == 0) *(float4*)((float*)out + at) = make_float4(y0, y1, y2, y3);
    else {
      uint2 r;
      r.x = (uint32_t)f2bf(y0) | ((uint32_t)f2bf(y1) << 16);
      r.y = (uint32_t)f2bf(y2) | ((uint32_t)f2bf(y3) << 16);
      *(uint2*)((bf16_t*)out + at) = r;
    }
  }
}

// Any width: an element a thread.
__global__ void __launch_bounds__(DT_THREADS)
dyt_stream_plain_kernel(float* __restrict__ x, const void* __restrict__ a, int a_code, const float* __restrict__ post_alpha,
                        const float* __restrict__ post_w, const float* __restrict__ post_b, void* __restrict__ out, int out_code,
                        const float* __restrict__ pre_alpha, const float* __restrict__ pre_w, const float* __restrict__ pre_b,
                        int width, int64_t total) {
  const int64_t at = (int64_t)blockIdx.x * DT_THREADS + threadIdx.x;
  if (at >= total) return;
  const int col = (int)(at % width);
  float v = x[at];
  if (a) {
    float av = dt_load(a, a_code, at);
    if (post_alpha) av = fmaf(dt_tanh(post_alpha[0] * av), post_w[col], post_b[col]);
    v += av;
    x[at] = v;
  }
  if (out) dt_store(out, out_code, at, fmaf(dt_tanh(pre_alpha[0] * v), pre_w[col], pre_b[col]));
}

extern "C" int ts_dyt_stream(float* x, const void* a, int a_dtype, const float* post_alpha, const float* post_w,
                             const float* post_b, void* out, int out_dtype, const float* pre_alpha, const float* pre_w,
                             const float* pre_b, int n, int width, hipStream_t stream) {
  if (n <= 0) return TS_OK;
  if (width <= 0 || (out && !pre_alpha) || (post_alpha && !a)) return TS_BAD_SHAPE;
  if ((a_dtype | out_dtype) & ~1) return TS_BAD_DTYPE;
  const int64_t total = (int64_t)n * width;
  if (width % 4 == 0) {
    const int64_t blocks = (total / 4 + DT_THREADS - 1) / DT_THREADS;
    if (blocks > 0x7fffffff) return TS_BAD_SHAPE;
    dyt_stream_kernel<<<(unsigned)blocks, DT_THREADS, 0, stream>>>(x, a, a_dtype, post_alpha, post_w, post_b, out, out_dtype,
                                                                   pre_alpha, pre_w, pre_b, width, total);
  } else {
    const int64_t blocks = (total + DT_THREADS - 1) / DT_THREADS;
    if (blocks > 0x7fffffff) return TS_BAD_SHAPE;
    dyt_stream_plain_kernel<<<(unsigned)blocks, DT_THREADS, 0, stream>>>(x, a, a_dtype, post_alpha, post_w, post_b, out,
                                                                         out_dtype, pre_alpha, pre_w, pre_b, width, total);
  }
  return ts_check_launch();
}

__global__ void __launch_bounds__(DT_THREADS)
embedding_dyt_stream_kernel(float* __restrict__ out, const void* __restrict__ table, int code, const int32_t* __restrict__ ids,
                            float scale, const float* __restrict__ alpha, const float* __restrict__ w,
                            const float* __restrict__ b, int hidden) {
  const int64_t t = blockIdx.x;
  const int64_t src = (int64_t)ids[t] * hidden;
  const float a = alpha ? alpha[0] : 0.f;
  for (int i = threadIdx.x; i < hidden; i += DT_THREADS) {
    float v = dt_load(table, code, src + i) * scale;
    if (alpha) v = fmaf(dt_tanh(a * v), w[i], b[i]);
    out[t * hidden + i] = v;
  }
}

extern "C" int ts_embedding_dyt_stream(float* out, const void* table, int dtype, const int32_t* ids, float scale,
                                       const float* alpha, const float* w, const float* b, int num_tokens, int hidden,
                                       hipStream_t stream) {
  if (num_tokens <= 0) return TS_OK;
  if (hidden <= 0) return TS_BAD_SHAPE;
  if (dtype & ~1) return TS_BAD_DTYPE;
  embedding_dyt_stream_kernel<<<num_tokens, DT_THREADS, 0, stream>>>(out, table, dtype, ids, scale, alpha, w, b, hidden);
  return ts_check_launch();
}

// The capped gated unit between the two projections of a feed-forward: from a row [gate | up] of 32-bit (or
// stored) sums, g = min(gate, limit), u = clamp(up, -limit, limit), y = g sigmoid(slope g) (u + 1).
// limit <= 0: no cap. Rows may be picked through `row_stride` (a row of the operand may be wider than 2 ff).
__global__ void __launch_bounds__(DT_THREADS)
capped_glu_kernel(void* __restrict__ out, int out_code, const void* __restrict__ gate_up, int in_code, int64_t row_stride,
                  int ff, float limit, float slope, float up_shift, int64_t total, int relu) {
  const int64_t at = (int64_t)blockIdx.x * DT_THREADS + threadIdx.x;
  if (at >= total) return;
  const int64_t t = at / ff;
  const int i = (int)(at - t * ff);
  float g = dt_load(gate_up, in_code, t * row_stride + i);
  float u = dt_load(gate_up, in_code, t * row_stride + ff + i);
  if (limit > 0.f) {
    g = fminf(g, limit);
    u = fminf(fmaxf(u, -limit), limit);
  }
  // (`relu`: the gate passes where it is positive, max(g, 0) (u + up_shift), instead of through a sigmoid)
  const float y = (relu ? fmaxf(g, 0.f) : g / (1.0f + expf(-slope * g))) * (u + up_shift);
  dt_store(out, out_code, at, y);
}

extern "C" int ts_capped_glu(void* out, int out_dtype, const void* gate_up, int in_dtype, int64_t row_stride, int n, int ff,
                             float limit, float slope, float up_shift, int relu, hipStream_t stream) {
  if (n <= 0) return TS_OK;
  if (ff <= 0 || row_stride < 2 * (int64_t)ff) return TS_BAD_SHAPE;
  if ((out_dtype | in_dtype) & ~1) return TS_BAD_DTYPE;
  const int64_t total = (int64_t)n * ff;
  const int64_t blocks = (total + DT_THREADS - 1) / DT_THREADS;
  if (blocks > 0x7fffffff) return TS_BAD_SHAPE;
  capped_glu_kernel<<<(unsigned)blocks, DT_THREADS, 0, stream>>>(out, out_dtype, gate_up, in_dtype, row_stride, ff, limit, slope,
                                                                 up_shift, total, relu);
  return ts_check_launch();
}
