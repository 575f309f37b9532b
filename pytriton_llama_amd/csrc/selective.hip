// The selective scan of Mamba: per channel c a state vector S[c, :] of N floats that decays and
// takes input at rates that depend on the token,
//
//   dt_c = softplus(w_dt[c, :] . r + b_c)            r [R]: the token's low-rank step input
//   S[c, n] <- exp(dt_c A[c, n]) S[c, n] + dt_c x_c B_n,      A = -exp(A_log)
//   y_c = sum_n S[c, n] C_n + D_c x_c,    out_c = y_c * silu(z_c)
//
// with x behind a short causal convolution over time (bias, SiLU). Everything is float32; the
// state [C, N] and the convolution's last taps - 1 inputs [taps - 1, C] live in the request's
// state slot. Every channel goes its own way given r, B and C, so the channels are spread over the
// chip: a workgroup takes 16 channels of one sequence, a channel is held by 16 lanes (one row of a
// wave for the data-parallel lane moves), each lane with NPL of its N states in registers (state n
// in lane n % 16). The tokens of a sequence are walked in order, 16 at a time through LDS; the
// step sizes of the 16 tokens are computed side by side before the walk, so that the chain from
// token to token is one multiply-add a state. The result does not depend on how the sequence was
// cut into steps.
//
// ptl_selective_conv: xc[t, c] = silu(sum_j w[c, j] x[t - taps + 1 + j, c] + b[c]); inputs before the
//   step's first token come from the slot's tail (zeros for a new request); float32, and a copy in
//   the engine's dtype for the product that follows.
// ptl_selective_scan: the recurrence and the gate.
// ptl_selective_scan_segments: the same for a step with long portions, whose rows are cut into
//   segments that are walked side by side (described where it stands, below).
#include "common.h"
#include <math.h>

#define SCHUNK 16

__device__ __forceinline__ float row16_sum(float v) {
  // the sum over the 16 lanes of a row, in every lane: rotations by 8, 4, 2 and 1 inside the row
  v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x128, 0xf, 0xf, false));
  v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x124, 0xf, 0xf, false));
  v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x122, 0xf, 0xf, false));
  v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x121, 0xf, 0xf, false));
  return v;
}

__device__ __forceinline__ float softplus_f(float x) { return x > 20.f ? x : log1pf(expf(x)); }
__device__ __forceinline__ float silu_f(float z) { return z / (1.0f + expf(-z)); }

// grid (channel blocks of 256, blocks of SCHUNK rows of the longest sequence, sequences)
template <typename TO>
__global__ void __launch_bounds__(256)
selective_conv_kernel(float* __restrict__ xc, TO* __restrict__ xc_lp, const float* __restrict__ p, long ldp,
                      int x_off, const float* __restrict__ cw, const float* __restrict__ cb,
                      const float* __restrict__ state, long slot_stride, long tail_off,
                      const int32_t* __restrict__ q_start, const int32_t* __restrict__ state_slots, int C,
                      int taps) {
  const int seq = blockIdx.z;
  const int row0 = q_start[seq];
  const int qlen = q_start[seq + 1] - row0;
  const int i0 = blockIdx.y * SCHUNK;
  if (i0 >= qlen) return;
  const int c = blockIdx.x * 256 + threadIdx.x;
  if (c >= C) return;
  const float* tail = state + (size_t)state_slots[seq] * slot_stride + tail_off;
  const float bias = cb ? cb[c] : 0.f;
  const int i1 = min(i0 + SCHUNK, qlen);
  if (taps <= 8) {
    // the last inputs stay in registers, the newest in the last place and the taps aligned to it, so
    // that every input is read once (and taps - 1 before the block's first row)
    float wv[8], win[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const int k = j - (8 - taps);        // the tap in place j
      wv[j] = k >= 0 ? cw[(size_t)c * taps + k] : 0.f;
      win[j] = 0.f;
      if (k >= 0 && j < 7) {
        const int r = i0 - (taps - 1) + k;
        win[j] = r >= 0 ? p[(size_t)(row0 + r) * ldp + x_off + c] : tail[(size_t)(taps - 1 + r) * C + c];
      }
    }
    for (int i = i0; i < i1; ++i) {
      win[7] = p[(size_t)(row0 + i) * ldp + x_off + c];
      float s = bias;
#pragma unroll
      for (int j = 0; j < 8; ++j) s = fmaf(wv[j], win[j], s);
#pragma unroll
      for (int j = 0; j < 7; ++j) win[j] = win[j + 1];
      const float v = silu_f(s);
      xc[(size_t)(row0 + i) * C + c] = v;
      if (xc_lp) xc_lp[(size_t)(row0 + i) * C + c] = from_float<TO>(v);
    }
    return;
  }
  for (int i = i0; i < i1; ++i) {
    float s = bias;
    for (int j = 0; j < taps; ++j) {
      const int r = i - (taps - 1) + j;
      const float x = r >= 0 ? p[(size_t)(row0 + r) * ldp + x_off + c] : tail[(size_t)(taps - 1 + r) * C + c];
      s = fmaf(cw[(size_t)c * taps + j], x, s);
    }
    const float v = silu_f(s);
    xc[(size_t)(row0 + i) * C + c] = v;
    if (xc_lp) xc_lp[(size_t)(row0 + i) * C + c] = from_float<TO>(v);
  }
}

extern "C" int ptl_selective_conv(float* xc, void* xc_lp, int lp_dtype, const float* p, long ldp, int x_off,
                                  const float* cw, const float* cb, int taps, const float* state,
                                  long slot_stride, long tail_off, const int32_t* q_start,
                                  const int32_t* state_slots, int n_seqs, int max_q_len, int C,
                                  hipStream_t st) {
  if (n_seqs <= 0 || max_q_len <= 0) return PTL_OK;
  if (C <= 0 || taps < 1 || n_seqs > 65535) return PTL_ERR_ARG;
  const int yb = (max_q_len + SCHUNK - 1) / SCHUNK;
  if (yb > 65535) return PTL_ERR_ARG;
  dim3 grid((C + 255) / 256, yb, n_seqs);
  if (xc_lp && lp_dtype == PTL_DTYPE_BF16)
    selective_conv_kernel<bf16_t><<<grid, 256, 0, st>>>(xc, (bf16_t*)xc_lp, p, ldp, x_off, cw, cb, state,
                                                        slot_stride, tail_off, q_start, state_slots, C, taps);
  else if (!xc_lp || lp_dtype == PTL_DTYPE_F32)
    selective_conv_kernel<float><<<grid, 256, 0, st>>>(xc, (float*)xc_lp, p, ldp, x_off, cw, cb, state,
                                                       slot_stride, tail_off, q_start, state_slots, C, taps);
  else
    return PTL_ERR_ARG;
  return ptl_launch_status();
}

struct SelArgs {
  void* out;                     // [T, C] in the engine's dtype
  const float* xc;               // [T, C]
  const float* z; long ldz;      // z[t * ldz + c]
  const float* r; long ldr;      // r[t * ldr + i], i < R; B at b_off, C at c_off of the same row
  int b_off, c_off;
  const float* w_dt;             // [C, R]
  const float* dt_b;             // [C]
  const float* A_log;            // [C, N]
  const float* D;                // [C]
  float* state; long slot_stride;
  const int32_t* q_start; const int32_t* state_slots;
  int C, N, R;
  int chunk;                     // tokens that go through LDS at a time: 1 to SCHUNK
};

// LDS of a workgroup, in floats: rows [chunk][R + 2 N] | w_dt [16][R] | x, z, dt, y [SCHUNK][16] each
static inline size_t scan_lds_floats(int N, int R, int chunk) {
  return (size_t)chunk * (R + 2 * N) + 16 * R + 4 * SCHUNK * 16;
}

template <int NPL, typename TO>
__global__ void __launch_bounds__(256) selective_scan_kernel(SelArgs a) {
  extern __shared__ float lds[];
  const int N = a.N, R = a.R, C = a.C;
  const int RW = R + 2 * N;
  const int CH = a.chunk;
  float* rows = lds;                       // [CH][RW]: r | B | C of the chunk's tokens
  float* wdt = rows + CH * RW;             // [16][R]
  float* xs = wdt + 16 * R;                // [SCHUNK][16]
  float* zs = xs + SCHUNK * 16;
  float* dts = zs + SCHUNK * 16;
  float* ys = dts + SCHUNK * 16;
  const int tid = threadIdx.x;
  const int seq = blockIdx.y;
  const int row0 = a.q_start[seq];
  const int qlen = a.q_start[seq + 1] - row0;
  if (qlen <= 0) return;
  const int c0 = blockIdx.x * 16;
  const int cg = tid >> 4, l = tid & 15;
  const int c = min(c0 + cg, C - 1);       // (a channel past the end repeats the last one; never stored)
  const bool live = c0 + cg < C;
  float* st = a.state + (size_t)a.state_slots[seq] * a.slot_stride + (size_t)c * N;
  float S[NPL], A[NPL];
#pragma unroll
  for (int i = 0; i < NPL; ++i) {
    const int n = l + 16 * i;
    S[i] = n < N ? st[n] : 0.f;
    A[i] = n < N ? -expf(a.A_log[(size_t)c * N + n]) : 0.f;
  }
  const float Dc = a.D[c];
  for (int i = tid; i < 16 * R; i += 256) {
    const int ch = min(c0 + i / R, C - 1);
    wdt[i] = a.w_dt[(size_t)ch * R + i % R];
  }
  // the thread that computes the step size of (token tid >> 4, channel tid & 15)
  const int dch = min(c0 + (tid & 15), C - 1);
  const float dtb = a.dt_b[dch];
  const float dtb_own = a.dt_b[c];         // of the channel this thread walks
  for (int t0 = 0; t0 < qlen; t0 += CH) {
    const int nt = min(CH, qlen - t0);
    __syncthreads();                       // the chunk before is done with
    for (int i = tid; i < nt * RW; i += 256) {
      const int t = i / RW, k = i - t * RW;
      const size_t row = (size_t)(row0 + t0 + t) * a.ldr;
      rows[i] = k < R ? a.r[row + k] : (k < R + N ? a.r[row + a.b_off + (k - R)] : a.r[row + a.c_off + (k - R - N)]);
    }
    {
      const int t = tid >> 4, ch = min(c0 + (tid & 15), C - 1);
      if (t < nt) {
        xs[tid] = a.xc[(size_t)(row0 + t0 + t) * C + ch];
        zs[tid] = a.z[(size_t)(row0 + t0 + t) * a.ldz + ch];
      }
    }
    __syncthreads();
    if (nt <= 4) {
      // few tokens: the 16 lanes of a channel share a token's sum
      for (int t = 0; t < nt; ++t) {
        const float* rr = rows + t * RW;
        const float* ww = wdt + cg * R;
        float s = 0.f;
        for (int k = l; k < R; k += 16) s = fmaf(ww[k], rr[k], s);
        s = row16_sum(s);
        if (l == 0) dts[t * 16 + cg] = softplus_f(s + dtb_own);
      }
    } else {
      const int t = tid >> 4, ch = tid & 15;
      if (t < nt) {
        float s = dtb;
        const float* rr = rows + t * RW;
        const float* ww = wdt + ch * R;
        for (int k = 0; k < R; ++k) s = fmaf(ww[k], rr[k], s);
        dts[tid] = softplus_f(s);
      }
    }
    __syncthreads();
    for (int t = 0; t < nt; ++t) {
      const float dt = dts[t * 16 + cg];
      const float xv = xs[t * 16 + cg];
      const float dx = dt * xv;
      const float* Bs = rows + t * RW + R;
      const float* Cs = Bs + N;
      float acc = 0.f;
#pragma unroll
      for (int i = 0; i < NPL; ++i) {
        const int n = min(l + 16 * i, N - 1);
        S[i] = fmaf(expf(dt * A[i]), S[i], dx * Bs[n]);
        acc = fmaf(l + 16 * i < N ? S[i] : 0.f, Cs[n], acc);
      }
      acc = row16_sum(acc);
      if (l == 0) ys[t * 16 + cg] = fmaf(Dc, xv, acc);
    }
    __syncthreads();
    {
      const int t = tid >> 4, ch = tid & 15;
      if (t < nt && c0 + ch < C)
        reinterpret_cast<TO*>(a.out)[(size_t)(row0 + t0 + t) * C + c0 + ch] =
            from_float<TO>(ys[tid] * silu_f(zs[tid]));
    }
  }
  if (live) {
#pragma unroll
    for (int i = 0; i < NPL; ++i) {
      const int n = l + 16 * i;
      if (n < N) st[n] = S[i];
    }
  }
}

template <typename TO>
static int launch_scan(const SelArgs& a, int n_seqs, hipStream_t st) {
  const int N = a.N;
  const size_t lds = scan_lds_floats(N, a.R, a.chunk) * sizeof(float);
  dim3 grid((a.C + 15) / 16, n_seqs);
#define GO(NPL)                                                                                      \
  {                                                                                                  \
    if (lds > 48 * 1024 &&                                                                           \
        hipFuncSetAttribute((const void*)selective_scan_kernel<NPL, TO>,                             \
                            hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess)     \
      return PTL_ERR_LAUNCH;                                                                         \
    selective_scan_kernel<NPL, TO><<<grid, 256, lds, st>>>(a);                                       \
    return ptl_launch_status();                                                                      \
  }
  if (N <= 16) GO(1)
  if (N <= 32) GO(2)
  if (N <= 64) GO(4)
  if (N <= 128) GO(8)
  GO(16)
#undef GO
}

// out [T, C] (engine dtype) from xc [T, C], z (float32, row stride ldz), the float32 rows r | B | C
// (row stride ldr; r from column 0, B from b_off, C from c_off), w_dt [C, R], dt_b [C], A_log [C, N],
// D [C] (all float32) and the slots' states [C, N] at the start of a slot. max_q_len: the rows of the
// step's longest sequence, or 0 when not known.
extern "C" int ptl_selective_scan(void* out, int out_dtype, const float* xc, const float* z, long ldz,
                                  const float* r, long ldr, int b_off, int c_off, const float* w_dt,
                                  const float* dt_b, const float* A_log, const float* D, float* state,
                                  long slot_stride, const int32_t* q_start, const int32_t* state_slots,
                                  int n_seqs, int max_q_len, int C, int N, int R, hipStream_t st) {
  if (n_seqs <= 0) return PTL_OK;
  // a step of short sequences (decoded tokens) keeps fewer rows in LDS, so that more workgroups fit
  const int chunk = max_q_len > 0 && max_q_len < SCHUNK ? max_q_len : SCHUNK;
  if (C <= 0 || N <= 0 || N > 256 || R <= 0 || n_seqs > 65535 ||
      scan_lds_floats(N, R, chunk) * sizeof(float) > 150 * 1024)
    return PTL_ERR_ARG;
  SelArgs a{out, xc, z, ldz, r, ldr, b_off, c_off, w_dt, dt_b, A_log, D, state, slot_stride, q_start,
            state_slots, C, N, R, chunk};
  if (out_dtype == PTL_DTYPE_F32) return launch_scan<float>(a, n_seqs, st);
  if (out_dtype == PTL_DTYPE_BF16) return launch_scan<bf16_t>(a, n_seqs, st);
  return PTL_ERR_ARG;
}

// ---------------------------------------------------------------------------
// Long portions: segments walked side by side.
//
// The transition of a state is a scalar, S <- e S + b with e = exp(dt A), so over a segment of
// tokens S_end = exp(A sum(dt)) S_start + E, where E is what the segment makes of a zero state.
// Four kernels:
//   dt:       the step sizes of all rows, dt[t, c] = softplus(w_dt[c, :] . r_t + b_c), as a float32
//             product on the matrix cores (64 rows x 128 channels a workgroup);
//   local:    every segment from a zero state: E [N][C] and sum(dt) [C] into the workspace;
//   combine:  the sequences' segments one after the other: the start state of each, and the
//             slot's state behind the last;
//   final:    every segment again from its start state, with the read-out and the gate.
// In local and final a lane holds one channel and all its N states in registers (N up to 32),
// so a token's dt, x and z are read once a channel, rows of B and C are the same for the whole
// wave, and no sum goes across lanes. Per token the arithmetic is that of the chain; the sums
// over the states and over the tokens before a segment are taken in another order.
// FAST: exp(dt A) as one hardware exponential of dt (A log2 e), and the softplus from the
// hardware's exponential and logarithm; used where the engine's dtype is not float32.

#define SEG_LOG2E 1.4426950408889634f

typedef float seg_f32x16 __attribute__((ext_vector_type(16)));

// softplus from the hardware's exponential and logarithm (a step size below 1e-7 comes out as 0)
__device__ __forceinline__ float softplus_fast(float x) { return x > 20.f ? x : __logf(1.0f + __expf(x)); }

// dt[t, c] = softplus(b[c] + sum_k w[c, k] r[t, k]) on the matrix cores in float32
// (v_mfma_f32_32x32x2_f32: float32 operands and sums). A wave takes 32 rows x 64 channels, a
// workgroup of four waves 64 x 128. Of a block of 8 k, lane l holds r[t0 + l % 32][4 (l / 32) ..+3]
// and the same entries of two rows of w; product m of the four takes entry m of every lane, so both
// operands see the same k in the same place. VEC: rows of r and w allow 16-byte loads.
template <bool VEC, bool FAST>
__global__ void __launch_bounds__(256)
selective_dt_kernel(float* __restrict__ dt, const float* __restrict__ r, long ldr,
                    const float* __restrict__ w, const float* __restrict__ b, int T, int C, int R) {
  const int wave = threadIdx.x >> 6, l = threadIdx.x & 63;
  const int t0 = blockIdx.y * 64 + (wave >> 1) * 32, c0 = blockIdx.x * 128 + (wave & 1) * 64;
  if (t0 >= T || c0 >= C) return;
  const int j = l & 31, h = l >> 5;
  const float* rp = r + (size_t)min(t0 + j, T - 1) * ldr;
  const float* w0 = w + (size_t)min(c0 + j, C - 1) * R;
  const float* w1 = w + (size_t)min(c0 + 32 + j, C - 1) * R;
  seg_f32x16 acc0, acc1;
#pragma unroll
  for (int v = 0; v < 16; ++v) acc0[v] = acc1[v] = 0.f;
#pragma unroll 4
  for (int k0 = 0; k0 < R; k0 += 8) {
    const int k = k0 + 4 * h;
    float av[4], b0[4], b1[4];
    if (VEC && k0 + 8 <= R) {
      const float4 x = *reinterpret_cast<const float4*>(rp + k);
      const float4 y0 = *reinterpret_cast<const float4*>(w0 + k);
      const float4 y1 = *reinterpret_cast<const float4*>(w1 + k);
      av[0] = x.x; av[1] = x.y; av[2] = x.z; av[3] = x.w;
      b0[0] = y0.x; b0[1] = y0.y; b0[2] = y0.z; b0[3] = y0.w;
      b1[0] = y1.x; b1[1] = y1.y; b1[2] = y1.z; b1[3] = y1.w;
    } else {
#pragma unroll
      for (int m = 0; m < 4; ++m) {
        const bool in = k + m < R;
        av[m] = in ? rp[k + m] : 0.f;
        b0[m] = in ? w0[k + m] : 0.f;
        b1[m] = in ? w1[k + m] : 0.f;
      }
    }
#pragma unroll
    for (int m = 0; m < 4; ++m) {
      acc0 = __builtin_amdgcn_mfma_f32_32x32x2f32(av[m], b0[m], acc0, 0, 0, 0);
      acc1 = __builtin_amdgcn_mfma_f32_32x32x2f32(av[m], b1[m], acc1, 0, 0, 0);
    }
  }
  // entry v of a lane: row 8 (v / 4) + 4 (l / 32) + v % 4 of the tile, column l % 32
  const int ca = c0 + j, cb = c0 + 32 + j;
  const float ba = ca < C ? b[ca] : 0.f, bb = cb < C ? b[cb] : 0.f;
#pragma unroll
  for (int v = 0; v < 16; ++v) {
    const int t = t0 + 8 * (v >> 2) + 4 * h + (v & 3);
    if (t >= T) continue;
    if (ca < C) dt[(size_t)t * C + ca] = FAST ? softplus_fast(acc0[v] + ba) : softplus_f(acc0[v] + ba);
    if (cb < C) dt[(size_t)t * C + cb] = FAST ? softplus_fast(acc1[v] + bb) : softplus_f(acc1[v] + bb);
  }
}

// The workspace of segment g of sequence s: [N][C] states and [C] sums of dt.
__device__ __forceinline__ size_t seg_work(int seq, int segments, int g, int C, int N) {
  return (size_t)(seq * segments + g) * (size_t)(N + 1) * C;
}

// grid (blocks of 64 channels, segments, sequences), one wave a workgroup
template <int NS, bool EXACT, bool FAST, bool FINAL, typename TO>
__global__ void __launch_bounds__(64)
selective_segment_kernel(TO* __restrict__ out, const float* __restrict__ dt, const float* __restrict__ xc,
                         const float* __restrict__ z, long ldz, const float* __restrict__ r, long ldr,
                         int b_off, int c_off, const float* __restrict__ A_log, const float* __restrict__ D,
                         float* __restrict__ ends, const float* __restrict__ starts, int segments, int seg_len,
                         const int32_t* __restrict__ q_start, int C, int N) {
  const int seq = blockIdx.z, g = blockIdx.y;
  const int row0 = q_start[seq];
  const int qlen = q_start[seq + 1] - row0;
  const int i0 = g * seg_len;
  if (i0 >= qlen) return;
  const int i1 = min(i0 + seg_len, qlen);
  const int c = blockIdx.x * 64 + threadIdx.x;
  const bool live = c < C;
  const int cc = min(c, C - 1);            // (a lane past the end repeats the last channel; never stored)
  const size_t wk = seg_work(seq, segments, g, C, N);
  float A[NS], S[NS];
#pragma unroll
  for (int n = 0; n < NS; ++n) {
    const bool in = EXACT || n < N;
    A[n] = in ? -expf(A_log[(size_t)cc * N + n]) * (FAST ? SEG_LOG2E : 1.f) : 0.f;
    S[n] = (FINAL && in) ? starts[wk + (size_t)n * C + cc] : 0.f;
  }
  const float Dc = D[cc];
  float sum = 0.f;
  size_t row = (size_t)(row0 + i0);
  float d = dt[row * C + cc], x = xc[row * C + cc], zz = FINAL ? z[row * ldz + cc] : 0.f;
  for (int i = i0; i < i1; ++i, ++row) {
    const float dc = d, xv = x, zc = zz;
    if (i + 1 < i1) {                      // the next token's, while this one is worked on
      d = dt[(row + 1) * C + cc];
      x = xc[(row + 1) * C + cc];
      if (FINAL) zz = z[(row + 1) * ldz + cc];
    }
    const float* __restrict__ Bt = r + row * ldr + b_off;
    const float* __restrict__ Ct = r + row * ldr + c_off;
    const float dx = dc * xv;
    float acc = 0.f;
#pragma unroll
    for (int n = 0; n < NS; ++n) {
      if (EXACT || n < N) {
        const float e = FAST ? __builtin_amdgcn_exp2f(dc * A[n]) : expf(dc * A[n]);
        S[n] = fmaf(e, S[n], dx * Bt[n]);
        if (FINAL) acc = fmaf(S[n], Ct[n], acc);
      }
    }
    if (FINAL) {
      if (live) out[row * C + c] = from_float<TO>(fmaf(Dc, xv, acc) * silu_f(zc));
    } else {
      sum += dc;
    }
  }
  if (!FINAL && live) {
#pragma unroll
    for (int n = 0; n < NS; ++n)
      if (EXACT || n < N) ends[wk + (size_t)n * C + c] = S[n];
    ends[wk + (size_t)N * C + c] = sum;
  }
}

// grid (blocks of 256 (state, channel) pairs, sequences): a thread takes one state of one channel
// through the sequence's segments
__global__ void __launch_bounds__(256)
selective_combine_kernel(float* __restrict__ starts, const float* __restrict__ ends, float* __restrict__ state,
                         long slot_stride, const float* __restrict__ A_log, int segments, int seg_len,
                         const int32_t* __restrict__ q_start, const int32_t* __restrict__ state_slots, int C,
                         int N) {
  const int seq = blockIdx.y;
  const int qlen = q_start[seq + 1] - q_start[seq];
  if (qlen <= 0) return;
  const int G = (qlen + seg_len - 1) / seg_len;
  const size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (idx >= (size_t)C * N) return;
  const int n = (int)(idx / C), c = (int)(idx - (size_t)n * C);
  float* st = state + (size_t)state_slots[seq] * slot_stride + (size_t)c * N + n;
  const float A = -expf(A_log[(size_t)c * N + n]);
  float S = *st;
#pragma unroll 4
  for (int g = 0; g < G; ++g) {
    const size_t wk = seg_work(seq, segments, g, C, N);
    const float E = ends[wk + (size_t)n * C + c];
    const float sd = ends[wk + (size_t)N * C + c];
    starts[wk + (size_t)n * C + c] = S;
    S = fmaf(expf(A * sd), S, E);
  }
  *st = S;
}

struct SegLaunch {
  void* out; const float* dt; const float* xc; const float* z; long ldz; const float* r; long ldr;
  int b_off, c_off; const float* A_log; const float* D; float* ends; float* starts; int segments, seg_len;
  const int32_t* q_start; int C, N, n_seqs;
};

template <int NS, bool EXACT, bool FAST, typename TO>
static int launch_segments(const SegLaunch& a, bool final, hipStream_t st) {
  dim3 grid((a.C + 63) / 64, a.segments, a.n_seqs);
  if (final)
    selective_segment_kernel<NS, EXACT, FAST, true, TO><<<grid, 64, 0, st>>>(
        (TO*)a.out, a.dt, a.xc, a.z, a.ldz, a.r, a.ldr, a.b_off, a.c_off, a.A_log, a.D, a.ends, a.starts,
        a.segments, a.seg_len, a.q_start, a.C, a.N);
  else
    selective_segment_kernel<NS, EXACT, FAST, false, TO><<<grid, 64, 0, st>>>(
        (TO*)a.out, a.dt, a.xc, a.z, a.ldz, a.r, a.ldr, a.b_off, a.c_off, a.A_log, a.D, a.ends, a.starts,
        a.segments, a.seg_len, a.q_start, a.C, a.N);
  return ptl_launch_status();
}

template <bool FAST, typename TO>
static int launch_segments_n(const SegLaunch& a, bool final, hipStream_t st) {
  const int N = a.N;
  if (N == 8) return launch_segments<8, true, FAST, TO>(a, final, st);
  if (N == 16) return launch_segments<16, true, FAST, TO>(a, final, st);
  if (N == 32) return launch_segments<32, true, FAST, TO>(a, final, st);
  if (N < 8) return launch_segments<8, false, FAST, TO>(a, final, st);
  if (N < 16) return launch_segments<16, false, FAST, TO>(a, final, st);
  return launch_segments<32, false, FAST, TO>(a, final, st);
}

// The selective scan of a step with long portions. T rows in all; every sequence's rows are cut
// into segments of seg_len tokens, at most ``segments`` a sequence. dt_work: T * C floats;
// work: 2 * n_seqs * segments * (N + 1) * C floats. N up to 32.
extern "C" int ptl_selective_scan_segments(void* out, int out_dtype, const float* xc, const float* z, long ldz,
                                           const float* r, long ldr, int b_off, int c_off, const float* w_dt,
                                           const float* dt_b, const float* A_log, const float* D, float* state,
                                           long slot_stride, float* dt_work, float* work, int segments,
                                           int seg_len, const int32_t* q_start, const int32_t* state_slots,
                                           int n_seqs, int T, int C, int N, int R, int fast, hipStream_t st) {
  if (n_seqs <= 0 || T <= 0) return PTL_OK;
  if (C <= 0 || N <= 0 || N > 32 || R <= 0 || n_seqs > 65535 || segments <= 0 || segments > 65535 ||
      seg_len <= 0 || (T + 63) / 64 > 65535)
    return PTL_ERR_ARG;
  {
    dim3 grid((C + 127) / 128, (T + 63) / 64);
    const bool vec = R % 4 == 0 && ldr % 4 == 0 && ((uintptr_t)r & 15) == 0 && ((uintptr_t)w_dt & 15) == 0;
    if (vec && fast)
      selective_dt_kernel<true, true><<<grid, 256, 0, st>>>(dt_work, r, ldr, w_dt, dt_b, T, C, R);
    else if (vec)
      selective_dt_kernel<true, false><<<grid, 256, 0, st>>>(dt_work, r, ldr, w_dt, dt_b, T, C, R);
    else if (fast)
      selective_dt_kernel<false, true><<<grid, 256, 0, st>>>(dt_work, r, ldr, w_dt, dt_b, T, C, R);
    else
      selective_dt_kernel<false, false><<<grid, 256, 0, st>>>(dt_work, r, ldr, w_dt, dt_b, T, C, R);
    if (int e = ptl_launch_status()) return e;
  }
  float* ends = work;
  float* starts = work + (size_t)n_seqs * segments * (size_t)(N + 1) * C;
  SegLaunch a{out, dt_work, xc, z, ldz, r, ldr, b_off, c_off, A_log, D, ends, starts, segments, seg_len,
              q_start, C, N, n_seqs};
  for (int pass = 0; pass < 2; ++pass) {
    int e;
    if (out_dtype == PTL_DTYPE_F32)
      e = fast ? launch_segments_n<true, float>(a, pass == 1, st) : launch_segments_n<false, float>(a, pass == 1, st);
    else if (out_dtype == PTL_DTYPE_BF16)
      e = fast ? launch_segments_n<true, bf16_t>(a, pass == 1, st)
               : launch_segments_n<false, bf16_t>(a, pass == 1, st);
    else
      return PTL_ERR_ARG;
    if (e) return e;
    if (pass == 0) {
      dim3 grid((unsigned)(((size_t)C * N + 255) / 256), n_seqs);
      selective_combine_kernel<<<grid, 256, 0, st>>>(starts, ends, state, slot_stride, A_log, segments, seg_len,
                                                     q_start, state_slots, C, N);
      if (int e2 = ptl_launch_status()) return e2;
    }
  }
  return PTL_OK;
}
