// Linear attention with a decay per key channel, as a recurrent mixer. Per head a state S [dim, vdim], 32-bit, zero
// at a request's start. For a token with q, k [dim], v [vdim] and decays w [dim] in (0, 1) there are two orders:
//     decay first  (gated linear attention):   S' = diag(w) S + k v^T,  o = S'^T q;
//     read first   (RWKV-style, with a bonus): o = (S + diag(u) k v^T)^T q,  S' = diag(w) S + k v^T,
// u [heads, dim] a learned bonus that only the current token's k v^T gets.
//   * `ts_decay_factors`: the decays from raw sums z and a bias b per head and channel, in 32-bit:
//     sigmoid form w = sigmoid(z + b)^(1 / tau) = exp(logsigmoid(z + b) / tau); double exponent w = exp(-exp(z + b)).
//   * `ts_decay_scan`: one workgroup per (request, head, slice of the value columns) walks the request's tokens of
//     the step in order. A wave owns 16 value columns (four lanes share a column's rows and add their parts up
//     through the wave's own exchanges) or 64 (a lane keeps a whole column, in four partial sums that it adds in the
//     exchanges' order: the same result bit for bit), so a token needs no barrier: only a block of tokens does, whose
//     q, k, w and v go through LDS together, in 16-byte pieces whose places a thread works out once; the next block's
//     loads are in flight while this one is worked on. The state is read from the request's slot at the start and
//     written back at the end. A column's sum runs over the rows in an order that the sizes alone fix. Heads of more
//     than 256 dimensions, and sizes or places that are no whole 16-byte pieces, take a kernel that fetches element
//     by element, with 4 columns a wave.
//   * `ts_token_shift`: x_s[t] = h[t] + (h[t-1] - h[t]) mu_s for several mixes s at once, h[t-1] of a request's first
//     token of the step being the row its state slot keeps (zeros for a new request); `ts_token_shift_keep` then
//     leaves each request's last row of the step in its slot.
#include "common.h"

#define DS_MAX_STAGED 32        // elements of a block of tokens that a thread carries from memory to LDS
#define DS_MAX_BLOCK 16         // tokens of a block

static __device__ __forceinline__ float ds_decay(float z, int form, float inv_tau) {
  if (form == 0) return expf((fminf(z, 0.f) - log1pf(expf(-fabsf(z)))) * inv_tau);
  return expf(-expf(z));
}

// WC: value columns of a wave (64 / WC lanes share a column); R4: groups of four rows that a lane keeps of it.
template <int WC, int R4, bool READ_FIRST>
__global__ void __launch_bounds__(256)
decay_scan_kernel(float* __restrict__ out, const float* __restrict__ q, int64_t q_stride, const float* __restrict__ k,
                  int64_t k_stride, const float* __restrict__ v, int64_t v_stride, const float* __restrict__ w,
                  int64_t w_stride, const float* __restrict__ bonus,
                  float* __restrict__ state, int64_t state_stride, const int32_t* __restrict__ cu_seqlens,
                  const int32_t* __restrict__ state_slots, int heads, int dim, int vdim,
                  float q_scale, int block_tokens) {
  extern __shared__ float lds[];
  constexpr int GROUPS = TS_WAVE / WC;
  const int threads = blockDim.x, waves = threads / TS_WAVE;
  const int cols = waves * WC;                              // value columns of the workgroup
  const int dim4 = (dim + 3) & ~3;                          // q, k and w rows in LDS, padded to whole fours
  const int in_size = 3 * dim4 + cols;                      // per token: q | k | w | the slice's v
  const int seq = blockIdx.x, h = blockIdx.y, v0 = blockIdx.z * cols;
  const int wave = threadIdx.x / TS_WAVE, lane = threadIdx.x & (TS_WAVE - 1);
  const int col = wave * WC + (lane % WC), grp = lane / WC;
  const bool live = v0 + col < vdim;
  const int t_begin = cu_seqlens[seq], t_end = cu_seqlens[seq + 1];
  if (t_begin >= t_end) return;
  float* st = state + (int64_t)state_slots[seq] * state_stride + (int64_t)h * dim * vdim;
  float S[R4 * 4], U[READ_FIRST ? R4 * 4 : 1];
#pragma unroll
  for (int r = 0; r < R4; ++r)
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int d = (r * GROUPS + grp) * 4 + j;
      S[r * 4 + j] = (live && d < dim) ? st[(int64_t)d * vdim + v0 + col] : 0.f;
      if constexpr (READ_FIRST) U[r * 4 + j] = d < dim ? bonus[h * dim + d] : 0.f;
    }
  // one element of a block of tokens: (token of the block, place in its row of LDS) -> its value, ready for use
  auto fetch = [&](int t0, int nt, int e) -> float {
    const int tl = e / in_size, p = e - tl * in_size;
    if (tl >= nt) return 0.f;
    const int64_t t = t0 + tl;
    if (p < dim4) return p < dim ? q[t * q_stride + h * dim + p] * q_scale : 0.f;
    if (p < 2 * dim4) return p - dim4 < dim ? k[t * k_stride + h * dim + p - dim4] : 0.f;
    if (p < 3 * dim4) {
      const int d = p - 2 * dim4;
      return d < dim ? w[t * w_stride + h * dim + d] : 1.f;
    }
    const int c = p - 3 * dim4;
    return v0 + c < vdim ? v[t * v_stride + h * vdim + v0 + c] : 0.f;
  };
  const int block_size = block_tokens * in_size;
  for (int e = threadIdx.x; e < block_size; e += threads) lds[e] = fetch(t_begin, min(block_tokens, t_end - t_begin), e);
  __syncthreads();
  int buf = 0;
  for (int t0 = t_begin; t0 < t_end; t0 += block_tokens, buf ^= 1) {
    const int nt = min(block_tokens, t_end - t0);
    const int next0 = t0 + block_tokens, next_n = min(block_tokens, t_end - next0);
    float staged[DS_MAX_STAGED];
    if (next_n > 0) {
#pragma unroll
      for (int i = 0; i < DS_MAX_STAGED; ++i) {
        const int e = threadIdx.x + i * threads;
        staged[i] = e < block_size ? fetch(next0, next_n, e) : 0.f;
      }
    }
    const float* base = lds + buf * block_size;
    for (int tl = 0; tl < nt; ++tl) {
      const float* q_s = base + tl * in_size;
      const float* k_s = q_s + dim4;
      const float* w_s = k_s + dim4;
      const float vc = w_s[dim4 + col];
      float o = 0.f;
#pragma unroll
      for (int r = 0; r < R4; ++r) {
        const int d0 = (r * GROUPS + grp) * 4;
        if (d0 < dim4) {
          const float4 q4 = *(const float4*)(q_s + d0), k4 = *(const float4*)(k_s + d0), w4 = *(const float4*)(w_s + d0);
          const float qq[4] = {q4.x, q4.y, q4.z, q4.w}, kk[4] = {k4.x, k4.y, k4.z, k4.w}, ww[4] = {w4.x, w4.y, w4.z, w4.w};
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            const float kv = kk[j] * vc;
            float& s = S[r * 4 + j];
            if constexpr (READ_FIRST) {
              o = fmaf(fmaf(U[r * 4 + j], kv, s), qq[j], o);
              s = fmaf(ww[j], s, kv);
            } else {
              s = fmaf(ww[j], s, kv);
              o = fmaf(s, qq[j], o);
            }
          }
        }
      }
#pragma unroll
      for (int off = WC; off < TS_WAVE; off <<= 1) o += __shfl_xor(o, off, TS_WAVE);
      if (grp == 0 && live) out[(int64_t)(t0 + tl) * heads * vdim + h * vdim + v0 + col] = o;
    }
    if (next_n > 0) {
      float* dst = lds + (buf ^ 1) * block_size;
#pragma unroll
      for (int i = 0; i < DS_MAX_STAGED; ++i) {
        const int e = threadIdx.x + i * threads;
        if (e < block_size) dst[e] = staged[i];
      }
    }
    __syncthreads();
  }
#pragma unroll
  for (int r = 0; r < R4; ++r)
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int d = (r * GROUPS + grp) * 4 + j;
      if (live && d < dim) st[(int64_t)d * vdim + v0 + col] = S[r * 4 + j];
    }
}

// The same walk where everything comes in whole 16-byte pieces (dim and vdim multiples of four up to 256 dimensions,
// rows and places 16-byte aligned). A column's rows are dealt out in fours to GROUPS shares (4 for heads of less than 64
// dimensions, 16 up to 127, else 32): share g takes the fours g, g + GROUPS, ... in ascending order, and the shares' sums meet in a
// tree (neighbours first). Narrow form: a share is a lane, 64 / GROUPS columns a wave, the tree is the wave's exchanges.
// Wide form (steps of few tokens a request): a lane keeps a whole column and all its shares' sums, 64 columns a wave, so
// that the state's rows are read and written whole cache lines at a time; the tree is the same, so is every bit of the
// result. RG: fours of rows a share takes. A thread carries up to NP pieces of every token of a block of TB tokens: which
// ones, from where and to where it works out once.
template <int GROUPS, bool WIDE, int RG, bool READ_FIRST, int NP, int TB>
__global__ void __launch_bounds__(256)
decay_scan_pieces_kernel(float* __restrict__ out, const float* __restrict__ q, int64_t q_stride, const float* __restrict__ k,
                         int64_t k_stride, const float* __restrict__ v, int64_t v_stride, const float* __restrict__ w,
                         int64_t w_stride, const float* __restrict__ bonus, float* __restrict__ state, int64_t state_stride,
                         const int32_t* __restrict__ cu_seqlens, const int32_t* __restrict__ state_slots, int heads, int dim,
                         int vdim, float q_scale) {
  extern __shared__ float lds[];
  constexpr int WC = WIDE ? TS_WAVE : TS_WAVE / GROUPS;     // columns of a wave
  constexpr int VG = WIDE ? GROUPS : 1;                     // shares of a column that a lane keeps
  // per token in LDS: q | k | w, each padded with zeros to the rows that the shares walk (so that no read of a row has to
  // ask whether the row exists: a branch there would keep a token's reads from going out together), then the slice's v;
  // behind the two blocks of tokens, the bonus (padded likewise) where there is one
  constexpr int DIMP = RG * GROUPS * 4;
  const int threads = blockDim.x, waves = threads / TS_WAVE;
  const int cols = waves * WC;
  const int in_size = 3 * DIMP + cols;
  const int seq = blockIdx.x, h = blockIdx.y, v0 = blockIdx.z * cols;
  const int wave = threadIdx.x / TS_WAVE, lane = threadIdx.x & (TS_WAVE - 1);
  const int col = wave * WC + (lane % WC), grp = WIDE ? 0 : lane / WC;
  const bool live = v0 + col < vdim;
  const int t_begin = cu_seqlens[seq], t_end = cu_seqlens[seq + 1];
  if (t_begin >= t_end) return;
  float* st = state + (int64_t)state_slots[seq] * state_stride + (int64_t)h * dim * vdim;
  float S[RG * VG * 4];
#pragma unroll
  for (int r = 0; r < RG; ++r)
#pragma unroll
    for (int g = 0; g < VG; ++g)
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int d = (r * GROUPS + grp + g) * 4 + j;
        S[(r * VG + g) * 4 + j] = (live && d < dim) ? st[(int64_t)d * vdim + v0 + col] : 0.f;
      }
  // this thread's pieces of a token: source (at token 0), stride from token to token, place in the token's row of LDS
  const int d4 = dim / 4, pieces = 3 * d4 + cols / 4;
  const float* src[NP];
  int64_t stride[NP];
  float mult[NP];
  bool has[NP];
  int place[NP];
#pragma unroll
  for (int i = 0; i < NP; ++i) {
    const int p = threadIdx.x + i * threads;
    has[i] = p < pieces;
    mult[i] = 1.f;
    src[i] = q;
    stride[i] = 0;
    place[i] = 0;
    if (p < d4) { src[i] = q + h * dim + 4 * p; stride[i] = q_stride; mult[i] = q_scale; place[i] = 4 * p; }
    else if (p < 2 * d4) { src[i] = k + h * dim + 4 * (p - d4); stride[i] = k_stride; place[i] = DIMP + 4 * (p - d4); }
    else if (p < 3 * d4) { src[i] = w + h * dim + 4 * (p - 2 * d4); stride[i] = w_stride; place[i] = 2 * DIMP + 4 * (p - 2 * d4); }
    else if (p < pieces) {
      const int c = 4 * (p - 3 * d4);
      has[i] = v0 + c < vdim;                               // (a slice's last columns may lie beyond the head: zeros)
      src[i] = v + h * vdim + v0 + c;
      stride[i] = v_stride;
      place[i] = 3 * DIMP + c;
    }
  }
  float4 staged[NP][TB];
  auto load = [&](int t0, int nt) {
#pragma unroll
    for (int i = 0; i < NP; ++i)
#pragma unroll
      for (int tl = 0; tl < TB; ++tl) {
        float4 x = make_float4(0.f, 0.f, 0.f, 0.f);
        if (has[i] && tl < nt) x = *(const float4*)(src[i] + (int64_t)(t0 + tl) * stride[i]);
        staged[i][tl] = make_float4(x.x * mult[i], x.y * mult[i], x.z * mult[i], x.w * mult[i]);
      }
  };
  auto store = [&](float* dst) {
#pragma unroll
    for (int i = 0; i < NP; ++i) {
      const int p = threadIdx.x + i * threads;
      if (p < pieces) {
#pragma unroll
        for (int tl = 0; tl < TB; ++tl) *(float4*)(dst + tl * in_size + place[i]) = staged[i][tl];
      }
    }
  };
  const int block_size = TB * in_size;
  float* u_s = lds + 2 * block_size;
  if (DIMP != dim)
    for (int e = threadIdx.x; e < 2 * block_size; e += threads) lds[e] = 0.f;      // (the pads, once: no store goes there again)
  if constexpr (READ_FIRST)
    for (int e = threadIdx.x; e < DIMP; e += threads) u_s[e] = e < dim ? bonus[h * dim + e] : 0.f;
  load(t_begin, min(TB, t_end - t_begin));
  if (DIMP != dim) __syncthreads();
  store(lds);
  __syncthreads();
  int buf = 0;
  for (int t0 = t_begin; t0 < t_end; t0 += TB, buf ^= 1) {
    const int nt = min(TB, t_end - t0);
    const int next_n = min(TB, t_end - t0 - TB);
    if (next_n > 0) load(t0 + TB, next_n);
    const float* base = lds + buf * block_size;
    auto token = [&](int tl) -> float {
      const float* q_s = base + tl * in_size;
      const float* k_s = q_s + DIMP;
      const float* w_s = k_s + DIMP;
      const float vc = w_s[DIMP + col];
      float o[VG];
#pragma unroll
      for (int g = 0; g < VG; ++g) o[g] = 0.f;
#pragma unroll
      for (int r = 0; r < RG; ++r)
#pragma unroll
        for (int g = 0; g < VG; ++g) {
          const int d0 = (r * GROUPS + grp + g) * 4;         // (a row beyond the head: k = 0 keeps its S at 0, q = 0 adds nothing)
          const float4 q4 = *(const float4*)(q_s + d0), k4 = *(const float4*)(k_s + d0), w4 = *(const float4*)(w_s + d0);
          const float qq[4] = {q4.x, q4.y, q4.z, q4.w}, kk[4] = {k4.x, k4.y, k4.z, k4.w}, ww[4] = {w4.x, w4.y, w4.z, w4.w};
          float uu[4] = {0.f, 0.f, 0.f, 0.f};
          if constexpr (READ_FIRST) {
            const float4 u4 = *(const float4*)(u_s + d0);
            uu[0] = u4.x; uu[1] = u4.y; uu[2] = u4.z; uu[3] = u4.w;
          }
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            const float kv = kk[j] * vc;
            float& s = S[(r * VG + g) * 4 + j];
            if constexpr (READ_FIRST) {
              o[g] = fmaf(fmaf(uu[j], kv, s), qq[j], o[g]);
              s = fmaf(ww[j], s, kv);
            } else {
              s = fmaf(ww[j], s, kv);
              o[g] = fmaf(s, qq[j], o[g]);
            }
          }
        }
      if constexpr (WIDE) {                                  // the shares' sums, neighbours first
#pragma unroll
        for (int span = 1; span < VG; span <<= 1)
#pragma unroll
          for (int g = 0; g < VG; g += 2 * span) o[g] += o[g + span];
      }
      return o[0];
    };
    auto put = [&](int tl, float sum) {
      if (grp == 0 && live) out[(int64_t)(t0 + tl) * heads * vdim + h * vdim + v0 + col] = sum;
    };
    if (!WIDE && nt == TB) {
      // a whole block: its tokens side by side in the code (the state is the only thing one token hands the next), and the
      // lanes' shares of all its tokens meet afterwards, stage by stage for the eight tokens at once: an exchange waits a
      // hundred cycles for its answer, and a token's four in a row were most of what a token cost
      float part[TB];
#pragma unroll
      for (int tl = 0; tl < TB; ++tl) part[tl] = token(tl);
#pragma unroll
      for (int off = WC; off < TS_WAVE; off <<= 1)
#pragma unroll
        for (int tl = 0; tl < TB; ++tl) part[tl] += __shfl_xor(part[tl], off, TS_WAVE);
#pragma unroll
      for (int tl = 0; tl < TB; ++tl) put(tl, part[tl]);
    } else {
      for (int tl = 0; tl < nt; ++tl) {
        float sum = token(tl);
        if constexpr (!WIDE) {
#pragma unroll
          for (int off = WC; off < TS_WAVE; off <<= 1) sum += __shfl_xor(sum, off, TS_WAVE);
        }
        put(tl, sum);
      }
    }
    if (next_n > 0) store(lds + (buf ^ 1) * block_size);
    __syncthreads();
  }
#pragma unroll
  for (int r = 0; r < RG; ++r)
#pragma unroll
    for (int g = 0; g < VG; ++g)
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int d = (r * GROUPS + grp + g) * 4 + j;
        if (live && d < dim) st[(int64_t)d * vdim + v0 + col] = S[(r * VG + g) * 4 + j];
      }
}

// Tokens of a block for a workgroup of `threads`: as many as a thread can carry and 64 KB of LDS hold twice.
static int ds_block_tokens(int threads, int in_size) {
  int n = (DS_MAX_STAGED * threads) / in_size;
  const int lds = (64 * 1024) / (2 * in_size * (int)sizeof(float));
  if (n > lds) n = lds;
  if (n > DS_MAX_BLOCK) n = DS_MAX_BLOCK;
  return n;
}

// `wide`: a wave owns 64 columns instead of 16 (steps of few tokens a request: the state's rows are read and written
// whole cache lines at a time, and nothing is exchanged between lanes); the result is the same bit for bit.
extern "C" int ts_decay_scan(float* out, const float* q, int64_t q_stride, const float* k, int64_t k_stride, const float* v,
                             int64_t v_stride, const float* w, int64_t w_stride, const float* bonus, float* state,
                             int64_t state_stride, const int32_t* cu_seqlens, const int32_t* state_slots, int num_seqs, int heads,
                             int dim, int vdim, float q_scale, int read_first, int waves, int wide, hipStream_t stream) {
  if (num_seqs <= 0) return TS_OK;
  if (heads <= 0 || heads > 65535 || dim <= 0 || dim > 1024 || vdim <= 0 || waves < 1 || waves > 4 || (read_first && !bonus) ||
      state_stride < (int64_t)heads * dim * vdim)
    return TS_BAD_SHAPE;
  const bool pieces = dim <= 256 && dim % 4 == 0 && vdim % 4 == 0 && ((q_stride | k_stride | v_stride | w_stride | state_stride) & 3) == 0 &&
                      (((uintptr_t)q | (uintptr_t)k | (uintptr_t)v | (uintptr_t)w) & 15) == 0;
  if (pieces) {
    const int groups = dim < 64 ? 4 : dim < 128 ? 16 : 32;  // (by the head's size alone: both forms then sum in one order)
    if (!wide && groups >= 16) waves = 4;                   // (4 or 2 columns a wave: a workgroup's waves share what is staged)
    const int wc = wide ? 64 : TS_WAVE / groups;
    const int cols = waves * wc;
    const int slices = (vdim + cols - 1) / cols;
    if (slices > 65535) return TS_BAD_SHAPE;
    const int threads = waves * TS_WAVE;
    const int np = ((3 * dim + cols) / 4 + threads - 1) / threads;
    const int fours = (dim / 4 + groups - 1) / groups;      // fours of rows a share takes,
    const int rg = fours <= 1 ? 1 : fours <= 2 ? 2 : fours <= 4 ? 4 : 8;      // as the instances have them
    const int in_size = 3 * rg * groups * 4 + cols;
    dim3 grid(num_seqs, heads, slices);
#define DS_FARGS out, q, q_stride, k, k_stride, v, v_stride, w, w_stride, bonus, state, state_stride, cu_seqlens, state_slots, heads, dim, \
                 vdim, q_scale
#define DS_FAST3(G, WD, RG, RF, NP, TB) \
    decay_scan_pieces_kernel<G, WD, RG, RF, NP, TB><<<grid, threads, (size_t)(2 * TB * in_size + rg * groups * 4) * sizeof(float), stream>>>(DS_FARGS)
#define DS_FAST2(G, WD, RG, NP, TB) \
    { if (np > NP) return TS_BAD_SHAPE; if (read_first) { DS_FAST3(G, WD, RG, true, NP, TB); } else { DS_FAST3(G, WD, RG, false, NP, TB); } }
    // (pieces of a token that a thread carries, by the head's size whatever the workgroup's waves; at most 16 pieces in
    // flight. The narrow form takes blocks of 16 tokens where LDS holds two of them: a block's loads have the time the
    // block before takes to be worked on, and that has to cover a trip to memory)
    if (groups == 4) {
      if (wide) {
        if (rg == 1) DS_FAST2(4, true, 1, 1, 8) else if (rg == 2) DS_FAST2(4, true, 2, 1, 8) else DS_FAST2(4, true, 4, 1, 8)
      } else {
        if (rg == 1) DS_FAST2(4, false, 1, 1, 16) else if (rg == 2) DS_FAST2(4, false, 2, 1, 16) else DS_FAST2(4, false, 4, 1, 16)
      }
    } else if (groups == 16) {
      if (wide) {
        if (rg <= 1) DS_FAST2(16, true, 1, 1, 8) else DS_FAST2(16, true, 2, 2, 8)
      } else {
        if (rg <= 1) DS_FAST2(16, false, 1, 1, 16) else DS_FAST2(16, false, 2, 1, 16)
      }
    } else if (wide) {
      if (rg <= 1) DS_FAST2(32, true, 1, 2, 8) else DS_FAST2(32, true, 2, 4, 4)
    } else {
      if (rg <= 1) DS_FAST2(32, false, 1, 1, 16) else DS_FAST2(32, false, 2, 1, 8)
    }
#undef DS_FAST2
#undef DS_FAST3
#undef DS_FARGS
    return ts_check_launch();
  }
  const int wc = dim <= 256 ? 16 : 4;                       // longer heads: more lanes share a column
  const int groups = TS_WAVE / wc;
  if (wc == 4) waves = 4;                                   // (their rows of q, k and w need a whole workgroup's hands)
  const int cols = waves * wc;
  const int slices = (vdim + cols - 1) / cols;
  if (slices > 65535) return TS_BAD_SHAPE;
  const int dim4 = (dim + 3) & ~3;
  const int in_size = 3 * dim4 + cols;
  const int block_tokens = ds_block_tokens(waves * TS_WAVE, in_size);
  if (block_tokens < 1) return TS_BAD_SHAPE;
  const int r4 = (dim4 / 4 + groups - 1) / groups;          // fours of rows a lane keeps
  dim3 grid(num_seqs, heads, slices);
  const size_t lds = (size_t)2 * block_tokens * in_size * sizeof(float);
#define DS_ARGS out, q, q_stride, k, k_stride, v, v_stride, w, w_stride, bonus, state, state_stride, cu_seqlens, state_slots, \
                heads, dim, vdim, q_scale, block_tokens
#define DS_LAUNCH(WC, R4) \
  if (read_first) decay_scan_kernel<WC, R4, true><<<grid, waves * TS_WAVE, lds, stream>>>(DS_ARGS); \
  else decay_scan_kernel<WC, R4, false><<<grid, waves * TS_WAVE, lds, stream>>>(DS_ARGS)
  if (wc == 16) {
    if (r4 <= 1) { DS_LAUNCH(16, 1); }
    else if (r4 <= 2) { DS_LAUNCH(16, 2); }
    else if (r4 <= 4) { DS_LAUNCH(16, 4); }
    else if (r4 <= 8) { DS_LAUNCH(16, 8); }
    else if (r4 <= 16) { DS_LAUNCH(16, 16); }
    else return TS_BAD_SHAPE;
  } else {
    if (r4 <= 8) { DS_LAUNCH(4, 8); }
    else if (r4 <= 16) { DS_LAUNCH(4, 16); }
    else return TS_BAD_SHAPE;
  }
#undef DS_LAUNCH
#undef DS_ARGS
  return ts_check_launch();
}

// w = sigmoid(z + b)^(1 / tau) (form 0) or exp(-exp(z + b)) (form 1), element by element; b repeats every `width`.
__global__ void __launch_bounds__(256)
decay_factors_kernel(float* __restrict__ w, const float* __restrict__ z, int64_t z_stride, const float* __restrict__ bias, int width,
                     int64_t total, int form, float inv_tau) {
  for (int64_t at = (int64_t)blockIdx.x * 256 + threadIdx.x; at < total; at += (int64_t)gridDim.x * 256) {
    const int64_t t = at / width;
    const int i = (int)(at - t * width);
    w[at] = ds_decay(z[t * z_stride + i] + bias[i], form, inv_tau);
  }
}

extern "C" int ts_decay_factors(float* w, const float* z, int64_t z_stride, const float* bias, int num_tokens, int width, int form,
                                float tau, hipStream_t stream) {
  if (num_tokens <= 0) return TS_OK;
  if (width <= 0 || z_stride < width || (form != 0 && form != 1) || !(tau > 0.f)) return TS_BAD_SHAPE;
  const int64_t total = (int64_t)num_tokens * width;
  int64_t blocks = (total + 255) / 256;
  if (blocks > 16384) blocks = 16384;
  decay_factors_kernel<<<(unsigned)blocks, 256, 0, stream>>>(w, z, z_stride, bias, width, total, form, 1.0f / tau);
  return ts_check_launch();
}

// A thread per (token, element): every mix of the element at once.
template <typename T>
__global__ void __launch_bounds__(256)
token_shift_kernel(T* __restrict__ out, const T* __restrict__ h, const float* __restrict__ mu, const float* __restrict__ kept,
                   int64_t kept_stride, const int32_t* __restrict__ cu_seqlens, const int32_t* __restrict__ seq_of_token,
                   const int32_t* __restrict__ state_slots, int num_tokens, int width, int mixes) {
  const int64_t at = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (at >= (int64_t)num_tokens * width) return;
  const int64_t t = at / width;
  const int i = (int)(at - t * width);
  const int seq = seq_of_token[t];
  const float x = Num<T>::ld(h + at);
  const float before = t == cu_seqlens[seq] ? kept[(int64_t)state_slots[seq] * kept_stride + i] : Num<T>::ld(h + at - width);
  for (int s = 0; s < mixes; ++s)
    Num<T>::st(out + ((int64_t)s * num_tokens + t) * width + i, fmaf(before - x, mu[s * width + i], x));
}

template <typename T>
__global__ void __launch_bounds__(256)
token_shift_keep_kernel(float* __restrict__ kept, int64_t kept_stride, const T* __restrict__ h,
                        const int32_t* __restrict__ cu_seqlens, const int32_t* __restrict__ state_slots, int width) {
  const int seq = blockIdx.x;
  const int first = cu_seqlens[seq], last = cu_seqlens[seq + 1] - 1;
  if (last < first) return;
  for (int i = blockIdx.y * 256 + threadIdx.x; i < width; i += gridDim.y * 256)
    kept[(int64_t)state_slots[seq] * kept_stride + i] = Num<T>::ld(h + (int64_t)last * width + i);
}

extern "C" int ts_token_shift(void* out, const void* h, int dtype, const float* mu, const float* kept, int64_t kept_stride,
                              const int32_t* cu_seqlens, const int32_t* seq_of_token, const int32_t* state_slots,
                              int num_tokens, int width, int mixes, hipStream_t stream) {
  if (num_tokens <= 0) return TS_OK;
  if (width <= 0 || mixes <= 0 || kept_stride < width) return TS_BAD_SHAPE;
  const int64_t blocks = ((int64_t)num_tokens * width + 255) / 256;
  if (blocks > 0x7fffffff) return TS_BAD_SHAPE;
  if (dtype == 0)
    token_shift_kernel<float><<<(unsigned)blocks, 256, 0, stream>>>((float*)out, (const float*)h, mu, kept, kept_stride, cu_seqlens,
                                                                   seq_of_token, state_slots, num_tokens, width, mixes);
  else if (dtype == 1)
    token_shift_kernel<bf16_t><<<(unsigned)blocks, 256, 0, stream>>>((bf16_t*)out, (const bf16_t*)h, mu, kept, kept_stride, cu_seqlens,
                                                                    seq_of_token, state_slots, num_tokens, width, mixes);
  else return TS_BAD_DTYPE;
  return ts_check_launch();
}

extern "C" int ts_token_shift_keep(float* kept, int64_t kept_stride, const void* h, int dtype, const int32_t* cu_seqlens,
                                   const int32_t* state_slots, int num_seqs, int width, hipStream_t stream) {
  if (num_seqs <= 0) return TS_OK;
  if (width <= 0 || kept_stride < width) return TS_BAD_SHAPE;
  dim3 grid(num_seqs, (width + 1023) / 1024 > 64 ? 64 : (width + 1023) / 1024);
  if (dtype == 0)
    token_shift_keep_kernel<float><<<grid, 256, 0, stream>>>(kept, kept_stride, (const float*)h, cu_seqlens, state_slots, width);
  else if (dtype == 1)
    token_shift_keep_kernel<bf16_t><<<grid, 256, 0, stream>>>(kept, kept_stride, (const bf16_t*)h, cu_seqlens, state_slots, width);
  else return TS_BAD_DTYPE;
  return ts_check_launch();
}
