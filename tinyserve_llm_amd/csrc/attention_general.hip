// Attention with the options that the matrix-core kernels of the plain rotate-half, softmax kind do not have,
// for every storage type and every size:
//   * `ts_qkv_finish`: what lies between the q|k|v projection and the cache. Rotary positions on the first
//     `rot` dimensions of each q and k head, pairing (2i, 2i+1) (interleaved) or (i, i + rot/2) (halves), the
//     angle p * f_i taken in 64-bit from a table of frequencies (no table over positions: a request may be of
//     any length), cosine and sine times `amplitude` (1 for plain rotary positions); then, optionally, each q and k head divided by its root mean square, and each value head
//     likewise; q goes to [tokens, heads, dim], k and v to their cache slots. Key and value heads may
//     differ in size.
//   * `ts_paged_attention_general`: one wavefront per (token, query head) over the request's pages, causal,
//     optionally windowed; score = q.k * scale, optionally capped as cap * tanh(score / cap); softmax,
//     optionally with a sink: a key of score 0 that has no value, i.e. one more in the denominator; or with
//     learned sinks, exp(sinks[head]) in the denominator instead of 1. Optionally a penalty on distance,
//     slopes[head] * (position - key's position), is taken off every score, and the output row is multiplied
//     element by element by sigmoid(gate) on its way out (gate: 32-bit rows of the step, one element per output).
//     Scores, weights and the weighted sum are 32-bit. Keys are visited in chunks of 64 counted from position
//     0, so the order of every sum depends on the token's position alone.
#include "common.h"

#define AG_WAVES 4
#define AG_MAX_HD 256

// One workgroup per token: the token's angles are taken once (sine and cosine of position * f_i for every pair,
// left in LDS), then the workgroup's waves take the token's heads in turn, one head a wave at a time.
template <typename TI, typename TO>
__global__ void __launch_bounds__(AG_WAVES * TS_WAVE)
qkv_finish_kernel(TO* __restrict__ q_out, TO* __restrict__ k_cache, TO* __restrict__ v_cache, const TI* __restrict__ qkv,
                  const double* __restrict__ freqs, const int32_t* __restrict__ positions,
                  const int32_t* __restrict__ slots, int num_tokens, int nh, int nkv, int hd, int vd_size, int rot,
                  int interleaved, int qk_norm, float qk_eps, int v_norm, float v_eps, int page_size, int64_t kp,
                  int64_t ks, int64_t kh, int64_t vp, int64_t vs, int64_t vh, int64_t vd, int with_values, float amplitude) {
  __shared__ float head_s[AG_WAVES][AG_MAX_HD];
  __shared__ float cos_s[AG_MAX_HD / 2], sin_s[AG_MAX_HD / 2];
  const int wave = threadIdx.x / TS_WAVE, lane = threadIdx.x & (TS_WAVE - 1);
  const int heads = nh + (with_values ? 2 : 1) * nkv;       // (without: the values go through `v_finish_kernel`)
  const int t = blockIdx.x;
  const int half = rot / 2;
  const int pos = positions[t];
  for (int pair = threadIdx.x; pair < half; pair += AG_WAVES * TS_WAVE) {
    // the angle in 64-bit, brought to [-pi, pi] before the 32-bit sine and cosine
    const double angle = (double)pos * freqs[pair];
    const double turns = rint(angle * 0.15915494309189535);
    const float a = (float)fma(-turns, 6.283185307179586, angle);
    float sn, cs;
    sincosf(a, &sn, &cs);
    cos_s[pair] = cs * amplitude;
    sin_s[pair] = sn * amplitude;
  }
  __syncthreads();
  const int64_t row = (int64_t)(nh + nkv) * hd + (int64_t)nkv * vd_size;
  const int slot = slots ? slots[t] : -1;
  const bool stores = slot >= 0 && k_cache;
  const int page = stores ? slot / page_size : 0, off = stores ? slot - page * page_size : 0;
  for (int h = wave; h < heads; h += AG_WAVES) {             // (wave-uniform: no block barrier below)
    const bool is_q = h < nh, is_v = h >= nh + nkv;
    if (!is_q && !stores) continue;                          // nothing to write for this token
    const int size = is_v ? vd_size : hd;
    const TI* src = qkv + t * row + (is_v ? (int64_t)(nh + nkv) * hd + (int64_t)(h - nh - nkv) * vd_size : (int64_t)h * hd);
    wave_sync();                                             // (the head before has been read out of head_s)
    for (int d = lane; d < size; d += TS_WAVE) head_s[wave][d] = Num<TI>::ld(src + d);
    wave_sync();
    float y[AG_MAX_HD / TS_WAVE];
    float squares = 0.f;
#pragma unroll
    for (int i = 0; i < AG_MAX_HD / TS_WAVE; ++i) {
      const int d = lane + i * TS_WAVE;
      float v = 0.f;
      if (d < size) {
        v = head_s[wave][d];
        if (!is_v && d < rot) {
          // the pair's index, this element's partner, and whether this element is the pair's first
          const int pair = interleaved ? d >> 1 : (d < half ? d : d - half);
          const bool first = interleaved ? !(d & 1) : d < half;
          const int partner = interleaved ? d ^ 1 : (first ? d + half : d - half);
          const float cs = cos_s[pair], sn = sin_s[pair], w = head_s[wave][partner];
          v = first ? v * cs - w * sn : v * cs + w * sn;
        }
      }
      y[i] = v;
      squares = fmaf(v, v, squares);
    }
    float scale = 1.0f;
    if (is_v ? v_norm : qk_norm) scale = 1.0f / sqrtf(wave_sum(squares) / (float)size + (is_v ? v_eps : qk_eps));
    TO* dst = is_q ? q_out + ((int64_t)t * nh + h) * hd
              : !is_v ? k_cache + page * kp + off * ks + (int64_t)(h - nh) * kh
                      : v_cache + page * vp + off * vs + (int64_t)(h - nh - nkv) * vh;
    const int64_t step = is_v ? vd : 1;
#pragma unroll
    for (int i = 0; i < AG_MAX_HD / TS_WAVE; ++i) {
      const int d = lane + i * TS_WAVE;
      if (d < size) Num<TO>::st(dst + (int64_t)d * step, y[i] * scale);
    }
  }
}

// The same for heads whose sizes are multiples of eight: a thread holds a piece of eight consecutive elements
// of a head (whole pairs of the interleaved layout; for the halves layout the partner piece is fetched as well), GS threads side by side hold a head (GS the power of two that covers the larger head size),
// and a thread takes every `slices`-th head of its token: 16 slices for steps of many tokens, so that a token's
// angles are taken 16 times and not once per head; a slice per head for steps of few, which have threads to spare
// and no time for one head after the other. All of a thread's loads for a head go out together.
#define AG_SLICES 16
template <typename T> struct Piece8;
template <> struct Piece8<float> {
  static __device__ __forceinline__ void ld(const float* p, float* o) {
    const float4 lo = *(const float4*)p, hi = *(const float4*)(p + 4);
    o[0] = lo.x; o[1] = lo.y; o[2] = lo.z; o[3] = lo.w; o[4] = hi.x; o[5] = hi.y; o[6] = hi.z; o[7] = hi.w;
  }
  static __device__ __forceinline__ void st(float* p, const float* v) {
    *(float4*)p = make_float4(v[0], v[1], v[2], v[3]);
    *(float4*)(p + 4) = make_float4(v[4], v[5], v[6], v[7]);
  }
};
template <> struct Piece8<bf16_t> {
  static __device__ __forceinline__ void ld(const bf16_t* p, float* o) {
    const uint4 r = *(const uint4*)p;
    const uint32_t w[4] = {r.x, r.y, r.z, r.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) { o[2 * i] = __uint_as_float(w[i] << 16); o[2 * i + 1] = __uint_as_float(w[i] & 0xffff0000u); }
  }
  static __device__ __forceinline__ void st(bf16_t* p, const float* v) {
    uint4 r;
    r.x = (uint32_t)f2bf(v[0]) | ((uint32_t)f2bf(v[1]) << 16);
    r.y = (uint32_t)f2bf(v[2]) | ((uint32_t)f2bf(v[3]) << 16);
    r.z = (uint32_t)f2bf(v[4]) | ((uint32_t)f2bf(v[5]) << 16);
    r.w = (uint32_t)f2bf(v[6]) | ((uint32_t)f2bf(v[7]) << 16);
    *(uint4*)p = r;
  }
};

template <typename TI, typename TO, int GS>
__global__ void __launch_bounds__(AG_WAVES * TS_WAVE)
qkv_finish_pieces_kernel(TO* __restrict__ q_out, TO* __restrict__ k_cache, TO* __restrict__ v_cache, const TI* __restrict__ qkv,
                         const double* __restrict__ freqs, const int32_t* __restrict__ positions,
                         const int32_t* __restrict__ slots, int num_tokens, int nh, int nkv, int hd, int vd_size, int rot,
                         int interleaved, int qk_norm, float qk_eps, int v_norm, float v_eps, int page_size, int64_t kp,
                         int64_t ks, int64_t kh, int64_t vp, int64_t vs, int64_t vh, int64_t vd, int with_values, float amplitude, int slices) {
  const int64_t gid = (int64_t)blockIdx.x * (AG_WAVES * TS_WAVE) + threadIdx.x;
  const int piece = (int)(gid % GS);
  const int slice = (int)((gid / GS) % slices);
  const int64_t t64 = gid / ((int64_t)GS * slices);
  const bool live = t64 < num_tokens;                      // (lanes beyond the step go along for the shuffles and store nothing)
  const int t = live ? (int)t64 : num_tokens - 1;
  const int heads = nh + (with_values ? 2 : 1) * nkv;
  const int d0 = 8 * piece, half = rot / 2;
  const int pos = positions[t];
  const int slot = slots ? slots[t] : -1;
  const bool stores = live && slot >= 0 && k_cache;
  const int page = stores ? slot / page_size : 0, off = stores ? slot - page * page_size : 0;
  // this piece's angles: element e turns with pair (d0 + e) / 2 (interleaved) or (d0 + e) mod half (halves)
  float cs[8], sn[8];
  auto angles = [&]() {
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      cs[e] = 1.f; sn[e] = 0.f;
      const int d = d0 + e;
      if (d < rot && (!interleaved || !(e & 1))) {
        const int pair = interleaved ? d >> 1 : (d < half ? d : d - half);
        // the angle in 64-bit, brought to [-pi, pi] before the 32-bit sine and cosine
        const double angle = (double)pos * freqs[pair];
        const double turns = rint(angle * 0.15915494309189535);
        sincosf((float)fma(-turns, 6.283185307179586, angle), &sn[e], &cs[e]);
        cs[e] *= amplitude; sn[e] *= amplitude;
      }
      if (interleaved && (e & 1)) { cs[e] = cs[e - 1]; sn[e] = sn[e - 1]; }
    }
  };
  const int64_t row = (int64_t)(nh + nkv) * hd + (int64_t)nkv * vd_size;
  const TI* trow = qkv + (int64_t)t * row;
  // where a head's piece lies in the token's row, and how many of its elements there are for this thread (8 or 0)
  auto piece_of = [&](int h) {
    const bool is_v = h >= nh + nkv;
    return trow + (is_v ? (int64_t)(nh + nkv) * hd + (int64_t)(h - nh - nkv) * vd_size : (int64_t)h * hd) + d0;
  };
  auto has_piece = [&](int h) { return h < heads && d0 < (h >= nh + nkv ? vd_size : hd); };
  // everything after a head's piece has arrived
  auto finish = [&](int h, const float (&x)[8]) {
    const bool is_q = h < nh, is_v = h >= nh + nkv;
    const int size = is_v ? vd_size : hd;
    const bool mine = d0 < size;
    float w[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    const bool turns_here = !is_v && mine && d0 < rot;
    if (turns_here && !interleaved) Piece8<TI>::ld(piece_of(h) + (d0 < half ? half : -half), w);   // (rot a multiple of 16: whole pieces)
    float y[8], squares = 0.f;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      float v = x[e];
      if (turns_here && d0 + e < rot) {
        const float partner = interleaved ? x[e ^ 1] : w[e];
        const bool first = interleaved ? !(e & 1) : d0 < half;
        v = first ? v * cs[e] - partner * sn[e] : v * cs[e] + partner * sn[e];
      }
      y[e] = v;
      squares = fmaf(v, v, squares);
    }
    float scale = 1.0f;
    if (is_v ? v_norm : qk_norm) {                           // (the same for all threads of a head: they shuffle together)
#pragma unroll
      for (int o = GS / 2; o > 0; o >>= 1) squares += __shfl_xor(squares, o, TS_WAVE);
      scale = 1.0f / sqrtf(squares / (float)size + (is_v ? v_eps : qk_eps));
    }
#pragma unroll
    for (int e = 0; e < 8; ++e) y[e] *= scale;
    if (!mine || !live) return;
    if (is_q) Piece8<TO>::st(q_out + ((int64_t)t * nh + h) * hd + d0, y);
    else if (!stores) return;
    else if (!is_v) Piece8<TO>::st(k_cache + page * kp + off * ks + (int64_t)(h - nh) * kh + d0, y);
    else {
      TO* dst = v_cache + page * vp + off * vs + (int64_t)(h - nh - nkv) * vh + (int64_t)d0 * vd;
#pragma unroll
      for (int e = 0; e < 8; ++e) Num<TO>::st(dst + (int64_t)e * vd, y[e]);
    }
  };
  constexpr int AHEAD = 8;                                   // heads whose pieces a thread asks for before it works on the first
  if ((heads + slices - 1) / slices <= AHEAD) {
    float xs[AHEAD][8];
#pragma unroll
    for (int k = 0; k < AHEAD; ++k) {
      const int h = slice + k * slices;
#pragma unroll
      for (int e = 0; e < 8; ++e) xs[k][e] = 0.f;
      if (has_piece(h)) Piece8<TI>::ld(piece_of(h), xs[k]);
    }
    angles();                                                // (while the pieces are on their way)
#pragma unroll
    for (int k = 0; k < AHEAD; ++k) {
      const int h = slice + k * slices;
      if (h < heads) finish(h, xs[k]);
    }
    return;
  }
  angles();
  for (int h = slice; h < heads; h += slices) {
    float x[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    if (has_piece(h)) Piece8<TI>::ld(piece_of(h), x);
    finish(h, x);
  }
}

// The values of AG_VTOK consecutive tokens of one key/value head, through LDS: rows are read along their
// dimensions, normalised, and written with the lanes along the tokens, so that tokens in consecutive slots
// of a page (whose values lie side by side there, pages holding values transposed) leave in whole segments.
#define AG_VTOK 32
template <typename TI, typename TO>
__global__ void __launch_bounds__(AG_WAVES * TS_WAVE)
v_finish_kernel(TO* __restrict__ v_cache, const TI* __restrict__ qkv, const int32_t* __restrict__ slots, int num_tokens,
                int64_t row, int64_t v_first, int vd_size, int v_norm, float v_eps, int page_size, int64_t vp, int64_t vs,
                int64_t vh, int64_t vd) {
  __shared__ float rows_s[AG_VTOK][AG_MAX_HD + 1];
  __shared__ float scale_s[AG_VTOK];
  __shared__ int slot_s[AG_VTOK];
  const int wave = threadIdx.x / TS_WAVE, lane = threadIdx.x & (TS_WAVE - 1);
  const int t0 = blockIdx.x * AG_VTOK, g = blockIdx.y;
  const int nt = min(AG_VTOK, num_tokens - t0);
  // the tile's rows into LDS, every thread's loads independent of each other
  const TI* tile = qkv + (int64_t)t0 * row + v_first + (int64_t)g * vd_size;
#pragma unroll 8
  for (int i = threadIdx.x; i < nt * vd_size; i += AG_WAVES * TS_WAVE) {
    const int tl = i / vd_size, d = i - tl * vd_size;
    rows_s[tl][d] = Num<TI>::ld(tile + (int64_t)tl * row + d);
  }
  if (threadIdx.x < nt) slot_s[threadIdx.x] = slots[t0 + threadIdx.x];
  __syncthreads();
  for (int tl = wave; tl < nt; tl += AG_WAVES) {
    float squares = 0.f;
    for (int d = lane; d < vd_size; d += TS_WAVE) squares = fmaf(rows_s[tl][d], rows_s[tl][d], squares);
    squares = wave_sum(squares);
    if (lane == 0) scale_s[tl] = v_norm ? 1.0f / sqrtf(squares / (float)vd_size + v_eps) : 1.0f;
  }
  __syncthreads();
  for (int i = threadIdx.x; i < vd_size * AG_VTOK; i += AG_WAVES * TS_WAVE) {
    const int d = i / AG_VTOK, tl = i - d * AG_VTOK;
    if (tl >= nt) continue;
    const int slot = slot_s[tl];
    if (slot < 0) continue;
    const int page = slot / page_size, off = slot - page * page_size;
    Num<TO>::st(v_cache + page * vp + off * vs + (int64_t)g * vh + (int64_t)d * vd, rows_s[tl][d] * scale_s[tl]);
  }
}

extern "C" int ts_qkv_finish(void* q_out, void* k_cache, void* v_cache, const void* qkv, const double* freqs,
                             const int32_t* positions, const int32_t* slots, int num_tokens, int nh, int nkv, int hd,
                             int vd_size, int rot, int interleaved, int qk_norm, float qk_eps, int v_norm, float v_eps,
                             int page_size, int64_t kp, int64_t ks, int64_t kh, int64_t vp, int64_t vs, int64_t vh,
                             int64_t vd, int in_dtype, int out_dtype, float amplitude, hipStream_t stream) {
  if (num_tokens <= 0) return TS_OK;
  if (hd <= 0 || hd > AG_MAX_HD || vd_size <= 0 || vd_size > AG_MAX_HD || nh <= 0 || nkv <= 0 || rot < 0 || rot > hd || rot % 2 ||
      page_size <= 0 || (rot > 0 && !freqs))
    return TS_BAD_SHAPE;
  // several tokens of a step: their values leave through the tile kernel (a single token's, with its head)
  const int v_tiles = k_cache && num_tokens >= 256 && nkv <= 65535;
  const int64_t blocks = num_tokens;
  const int64_t row = (int64_t)(nh + nkv) * hd + (int64_t)nkv * vd_size;
  dim3 v_grid((num_tokens + AG_VTOK - 1) / AG_VTOK, nkv);
  // heads in pieces of eight elements: sizes that are multiples of 8 (of 16 where halves are paired), 16-byte aligned rows
  const int in_piece = in_dtype == 0 ? 32 : 16, out_piece = out_dtype == 0 ? 32 : 16;
  const bool pieces = hd % 8 == 0 && vd_size % 8 == 0 && (interleaved ? rot % 2 == 0 : rot % 16 == 0) &&
                      ((uintptr_t)qkv % in_piece) == 0 && ((uintptr_t)q_out % out_piece) == 0 &&
                      (!k_cache || (((uintptr_t)k_cache % out_piece) == 0 && kp % 8 == 0 && ks % 8 == 0 && kh % 8 == 0));
  int gs = 4;
  while (gs * 8 < (hd > vd_size ? hd : vd_size)) gs *= 2;
  const int all_heads = nh + (v_tiles ? 1 : 2) * nkv;
  const int slices = (int64_t)num_tokens * AG_SLICES * gs >= 65536 ? AG_SLICES : all_heads;
  const int64_t piece_threads = (int64_t)num_tokens * slices * gs;
  const unsigned piece_blocks = (unsigned)((piece_threads + AG_WAVES * TS_WAVE - 1) / (AG_WAVES * TS_WAVE));
#define QF_ARGS(TI, TO) \
      (TO*)q_out, (TO*)k_cache, (TO*)v_cache, (const TI*)qkv, freqs, positions, slots, num_tokens, nh, nkv, hd, vd_size, rot, \
      interleaved, qk_norm, qk_eps, v_norm, v_eps, page_size, kp, ks, kh, vp, vs, vh, vd, !v_tiles, amplitude
#define QF_LAUNCH(TI, TO) \
  if (!pieces) qkv_finish_kernel<TI, TO><<<(unsigned)blocks, AG_WAVES * TS_WAVE, 0, stream>>>(QF_ARGS(TI, TO)); \
  else if (gs == 4) qkv_finish_pieces_kernel<TI, TO, 4><<<piece_blocks, AG_WAVES * TS_WAVE, 0, stream>>>(QF_ARGS(TI, TO), slices); \
  else if (gs == 8) qkv_finish_pieces_kernel<TI, TO, 8><<<piece_blocks, AG_WAVES * TS_WAVE, 0, stream>>>(QF_ARGS(TI, TO), slices); \
  else if (gs == 16) qkv_finish_pieces_kernel<TI, TO, 16><<<piece_blocks, AG_WAVES * TS_WAVE, 0, stream>>>(QF_ARGS(TI, TO), slices); \
  else qkv_finish_pieces_kernel<TI, TO, 32><<<piece_blocks, AG_WAVES * TS_WAVE, 0, stream>>>(QF_ARGS(TI, TO), slices); \
  if (v_tiles) v_finish_kernel<TI, TO><<<v_grid, AG_WAVES * TS_WAVE, 0, stream>>>( \
      (TO*)v_cache, (const TI*)qkv, slots, num_tokens, row, (int64_t)(nh + nkv) * hd, vd_size, v_norm, v_eps, page_size, vp, vs, vh, vd)
  if (in_dtype == 0 && out_dtype == 0) { QF_LAUNCH(float, float); }
  else if (in_dtype == 0 && out_dtype == 1) { QF_LAUNCH(float, bf16_t); }
  else if (in_dtype == 1 && out_dtype == 1) { QF_LAUNCH(bf16_t, bf16_t); }
  else return TS_BAD_DTYPE;
#undef QF_LAUNCH
#undef QF_ARGS
  return ts_check_launch();
}

template <typename T>
__global__ void __launch_bounds__(AG_WAVES * TS_WAVE)
paged_attention_general_kernel(T* __restrict__ out, const T* __restrict__ q, const T* __restrict__ k_cache,
                               const T* __restrict__ v_cache, const int32_t* __restrict__ block_tables,
                               const int32_t* __restrict__ seq_of_token, const int32_t* __restrict__ positions,
                               int num_tokens, int nh, int nkv, int hd, int vd_size, int page_size, int64_t kp, int64_t ks,
                               int64_t kh, int64_t vp, int64_t vs, int64_t vh, int64_t vd, int max_blocks, float scale,
                               float softcap, int sink, int window, int page_run, const float* __restrict__ sinks,
                               const float* __restrict__ slopes, const float* __restrict__ gate, int64_t gate_stride) {
  __shared__ float q_s[AG_WAVES][AG_MAX_HD];
  __shared__ float p_s[AG_WAVES][TS_WAVE];
  __shared__ int64_t row_s[AG_WAVES][TS_WAVE];   // element offset of each key's value row
  const int wave = threadIdx.x / TS_WAVE, lane = threadIdx.x & (TS_WAVE - 1);
  const int64_t item = (int64_t)blockIdx.x * AG_WAVES + wave;
  if (item >= (int64_t)num_tokens * nh) return;
  const int t = (int)(item / nh), h = (int)(item - (int64_t)t * nh);
  const int kvh = h / (nh / nkv);
  const int pos = positions[t];
  const int32_t* table = block_tables + (int64_t)seq_of_token[t] * max_blocks;
  const T* qrow = q + ((int64_t)t * nh + h) * hd;
  for (int d = lane; d < hd; d += TS_WAVE) q_s[wave][d] = Num<T>::ld(qrow + d);
  wave_sync();

  const int lo = ts_first_key(pos, window);
  // the sink is a key of score 0 without a value: it starts the running maximum and the sum
  // (a learned sink is the same key with a score of its own)
  float m = sinks ? sinks[h] : sink ? 0.f : -INFINITY, l = (sinks || sink) ? 1.f : 0.f;
  const float slope = slopes ? slopes[h] : 0.f;
  float acc[AG_MAX_HD / TS_WAVE] = {0.f, 0.f, 0.f, 0.f};
  const float inv_cap = softcap > 0.f ? 1.0f / softcap : 0.f;

  for (int c0 = (lo / TS_WAVE) * TS_WAVE; c0 <= pos; c0 += TS_WAVE) {
    const int key = c0 + lane;
    const bool valid = key >= lo && key <= pos;
    float s = -INFINITY;
    int64_t rowoff = 0;
    if (valid) {
      const int pg = key / page_size, slot = key % page_size;
      const int64_t page = ((int64_t)table[pg >> page_run] << page_run) + (pg & ((1 << page_run) - 1));
      rowoff = page * vp + (int64_t)slot * vs + (int64_t)kvh * vh;
      const T* kr = k_cache + page * kp + (int64_t)slot * ks + (int64_t)kvh * kh;
      float dot = 0.f;
      for (int d = 0; d < hd; ++d) dot = fmaf(q_s[wave][d], Num<T>::ld(kr + d), dot);
      s = dot * scale;
      if (softcap > 0.f) s = softcap * tanhf(s * inv_cap);
      s -= slope * (float)(pos - key);
    }
    const float m_new = fmaxf(m, wave_max(s));  // finite: the chunk holds at least one visible key
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
    for (int i = 0; i < AG_MAX_HD / TS_WAVE; ++i) {
      const int d = lane + i * TS_WAVE;
      if (d < vd_size) {
        float a = acc[i] * alpha;
        for (int j = first; j <= last; ++j) a = fmaf(p_s[wave][j], Num<T>::ld(v_cache + row_s[wave][j] + (int64_t)d * vd), a);
        acc[i] = a;
      }
    }
    wave_sync();
  }
  T* orow = out + ((int64_t)t * nh + h) * vd_size;
  const float inv = 1.0f / l;
#pragma unroll
  for (int i = 0; i < AG_MAX_HD / TS_WAVE; ++i) {
    const int d = lane + i * TS_WAVE;
    if (d < vd_size) {
      float o = acc[i] * inv;
      if (gate) o = o / (1.0f + expf(-gate[(int64_t)t * gate_stride + (int64_t)h * vd_size + d]));
      Num<T>::st(orow + d, o);
    }
  }
}

extern "C" int ts_paged_attention_general(void* out, const void* q, const void* k_cache, const void* v_cache,
                                          const int32_t* block_tables, const int32_t* seq_of_token,
                                          const int32_t* positions, int num_tokens, int nh, int nkv, int hd, int vd_size,
                                          int page_size, int64_t kp, int64_t ks, int64_t kh, int64_t vp, int64_t vs,
                                          int64_t vh, int64_t vd, int max_blocks, float scale, float softcap, int sink,
                                          int window, int dtype, int page_run, const float* sinks, const float* slopes,
                                          const float* gate, int64_t gate_stride, hipStream_t stream) {
  if (num_tokens <= 0) return TS_OK;
  if (hd <= 0 || hd > AG_MAX_HD || vd_size <= 0 || vd_size > AG_MAX_HD || nkv <= 0 || nh % nkv || page_size <= 0 ||
      max_blocks <= 0 || page_run < 0 || page_run > 16 || softcap < 0.f)
    return TS_BAD_SHAPE;
  const int64_t items = (int64_t)num_tokens * nh;
  const int64_t blocks = (items + AG_WAVES - 1) / AG_WAVES;
  if (blocks > 0x7fffffff) return TS_BAD_SHAPE;
  dim3 grid((unsigned)blocks), block(AG_WAVES * TS_WAVE);
  if (dtype == 0)
    paged_attention_general_kernel<float><<<grid, block, 0, stream>>>(
        (float*)out, (const float*)q, (const float*)k_cache, (const float*)v_cache, block_tables, seq_of_token, positions,
        num_tokens, nh, nkv, hd, vd_size, page_size, kp, ks, kh, vp, vs, vh, vd, max_blocks, scale, softcap, sink, window,
        page_run, sinks, slopes, gate, gate_stride);
  else if (dtype == 1)
    paged_attention_general_kernel<bf16_t><<<grid, block, 0, stream>>>(
        (bf16_t*)out, (const bf16_t*)q, (const bf16_t*)k_cache, (const bf16_t*)v_cache, block_tables, seq_of_token, positions,
        num_tokens, nh, nkv, hd, vd_size, page_size, kp, ks, kh, vp, vs, vh, vd, max_blocks, scale, softcap, sink, window,
        page_run, sinks, slopes, gate, gate_stride);
  else
    return TS_BAD_DTYPE;
  return ts_check_launch();
}

// ---- what some designs do to the projected rows before q and k turn ----
// In place on the 32-bit rows q | k | v of a step, one wave per (token, head):
//   * each q head and each k head divided by its root mean square (eps inside the root) and multiplied by a weight
//     of the head's size that all heads share (q_weight / k_weight; absent: that kind of head is left alone);
//   * each value head turned by the token's position over all its dimensions (v_freqs [vd / 2], 64-bit; pair m is
//     dimensions (m, m + vd/2), or (2m, 2m + 1) if `v_interleaved`), so that the cache holds rotated values.
__global__ void __launch_bounds__(AG_WAVES * TS_WAVE)
qkv_prepare_kernel(float* __restrict__ qkv, const int32_t* __restrict__ positions, int nh, int nkv, int hd, int vd_size,
                   const float* __restrict__ q_weight, const float* __restrict__ k_weight, float eps,
                   const double* __restrict__ v_freqs, int v_interleaved, int64_t items) {
  const int wave = threadIdx.x / TS_WAVE, lane = threadIdx.x & (TS_WAVE - 1);
  const int64_t item = (int64_t)blockIdx.x * AG_WAVES + wave;
  if (item >= items) return;
  const int heads = nh + 2 * nkv;
  const int64_t t = item / heads;
  const int h = (int)(item - t * heads);
  const int64_t row = (int64_t)(nh + nkv) * hd + (int64_t)nkv * vd_size;
  if (h < nh + nkv) {
    const float* weight = h < nh ? q_weight : k_weight;
    if (!weight) return;
    float* head = qkv + t * row + (int64_t)h * hd;
    float squares = 0.f;
    for (int d = lane; d < hd; d += TS_WAVE) squares = fmaf(head[d], head[d], squares);
    const float inv = 1.0f / sqrtf(wave_sum(squares) / (float)hd + eps);
    for (int d = lane; d < hd; d += TS_WAVE) head[d] = head[d] * inv * weight[d];
    return;
  }
  if (!v_freqs) return;
  float* head = qkv + t * row + (int64_t)(nh + nkv) * hd + (int64_t)(h - nh - nkv) * vd_size;
  const int half = vd_size / 2;
  const int pos = positions[t];
  for (int pair = lane; pair < half; pair += TS_WAVE) {
    const double angle = (double)pos * v_freqs[pair];
    const double turns = rint(angle * 0.15915494309189535);
    float sn, cs;
    sincosf((float)fma(-turns, 6.283185307179586, angle), &sn, &cs);
    const int a = v_interleaved ? 2 * pair : pair, b = v_interleaved ? 2 * pair + 1 : pair + half;
    const float u = head[a], v = head[b];
    head[a] = u * cs - v * sn;
    head[b] = v * cs + u * sn;
  }
}

extern "C" int ts_qkv_prepare(float* qkv, const int32_t* positions, int num_tokens, int nh, int nkv, int hd, int vd_size,
                              const float* q_weight, const float* k_weight, float eps, const double* v_freqs,
                              int v_interleaved, hipStream_t stream) {
  if (num_tokens <= 0 || (!q_weight && !k_weight && !v_freqs)) return TS_OK;
  if (nh <= 0 || nkv <= 0 || hd <= 0 || vd_size <= 0 || (v_freqs && vd_size % 2)) return TS_BAD_SHAPE;
  const int64_t items = (int64_t)num_tokens * (nh + 2 * nkv);
  const int64_t blocks = (items + AG_WAVES - 1) / AG_WAVES;
  if (blocks > 0x7fffffff) return TS_BAD_SHAPE;
  qkv_prepare_kernel<<<(unsigned)blocks, AG_WAVES * TS_WAVE, 0, stream>>>(qkv, positions, nh, nkv, hd, vd_size, q_weight, k_weight,
                                                                         eps, v_freqs, v_interleaved, items);
  return ts_check_launch();
}
