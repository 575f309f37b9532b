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
};

// LDS of a workgroup, in floats: rows [SCHUNK][R + 2 N] | w_dt [16][R] | x, z, dt, y [SCHUNK][16] each
static inline size_t scan_lds_floats(int N, int R) { return (size_t)SCHUNK * (R + 2 * N) + 16 * R + 4 * SCHUNK * 16; }

template <int NPL, typename TO>
__global__ void __launch_bounds__(256) selective_scan_kernel(SelArgs a) {
  extern __shared__ float lds[];
  const int N = a.N, R = a.R, C = a.C;
  const int RW = R + 2 * N;
  float* rows = lds;                       // [SCHUNK][RW]: r | B | C of the chunk's tokens
  float* wdt = rows + SCHUNK * RW;         // [16][R]
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
  for (int t0 = 0; t0 < qlen; t0 += SCHUNK) {
    const int nt = min(SCHUNK, qlen - t0);
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
    {
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
  const size_t lds = scan_lds_floats(N, a.R) * sizeof(float);
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
// D [C] (all float32) and the slots' states [C, N] at the start of a slot.
extern "C" int ptl_selective_scan(void* out, int out_dtype, const float* xc, const float* z, long ldz,
                                  const float* r, long ldr, int b_off, int c_off, const float* w_dt,
                                  const float* dt_b, const float* A_log, const float* D, float* state,
                                  long slot_stride, const int32_t* q_start, const int32_t* state_slots,
                                  int n_seqs, int C, int N, int R, hipStream_t st) {
  if (n_seqs <= 0) return PTL_OK;
  if (C <= 0 || N <= 0 || N > 256 || R <= 0 || n_seqs > 65535 ||
      scan_lds_floats(N, R) * sizeof(float) > 150 * 1024)
    return PTL_ERR_ARG;
  SelArgs a{out, xc, z, ldz, r, ldr, b_off, c_off, w_dt, dt_b, A_log, D, state, slot_stride, q_start,
            state_slots, C, N, R};
  if (out_dtype == PTL_DTYPE_F32) return launch_scan<float>(a, n_seqs, st);
  if (out_dtype == PTL_DTYPE_BF16) return launch_scan<bf16_t>(a, n_seqs, st);
  return PTL_ERR_ARG;
}
