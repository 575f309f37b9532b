// Latent attention: every token keeps one compressed vector c [R] and one rotated key part
// kr [dr] that all heads share; the keys and values of a head are linear maps of c. So the
// per-head maps move to the query side and the attention itself runs over the cache as it
// lies, with one "kv head" of size R + dr whose keys are [c | kr] and whose values are c:
//
//   score_h(i, j) = qn_h(i) . (Uk_h c_j) + qr_h(i) . kr_j = (Uk_h^T qn_h(i)) . c_j + qr_h(i) . kr_j
//   out_h(i)      = Uv_h sum_j p_h(i, j) c_j
//
// ptl_latent_prepare: per token, from the rows of projections (queries and down-projection, in
//   one matrix or in two): the RMS norm of the first R entries of the down-projection (float32,
//   weight w), the rotation of its last dr entries, both written to the cache slot [c | kr]; and
//   the rotation of the dr rotated entries of every query head, written behind the R entries
//   that ptl_gemm_heads_nt fills (query rows [H, R + dr]). Rotation of the first 2 * n_pairs
//   entries, angle = position * inv_freq[i], float32, sine and cosine times ``mag``: neighbouring
//   pairs (2i, 2i+1), or, with ``half_layout``, entry i with entry i + n_pairs; the rest of the
//   dr entries pass unchanged.
// ptl_gemm_heads_nt: out[t, h, :] = x[t, h, :] W_h^T for per-head matrices W [H, N, K], with an
//   optional factor sigmoid(gate[t, h]) on the result (an output gate per head).
#include "common.h"
#include "mfma.h"
#include <math.h>

template <typename T>
__global__ void __launch_bounds__(256)
latent_prepare_kernel(T* __restrict__ q_out, long ldq, const T* __restrict__ q_src, long ldqs, int q_off,
                      const T* __restrict__ kv_src, long ldkv, int kv_off,
                      const int32_t* __restrict__ positions, const float* __restrict__ inv_freq,
                      int n_pairs, int half_layout, float mag, const float* __restrict__ c_w, float eps,
                      const int32_t* __restrict__ slots, T* __restrict__ cache, int H, int dn, int dr, int R) {
  extern __shared__ float cs[];          // cos [dr/2], sin [dr/2], scratch [16]
  const int half = dr >> 1;
  float* cosv = cs;
  float* sinv = cs + half;
  float* scratch = cs + 2 * half;
  const int t = blockIdx.x;
  const float pos = (float)positions[t];
  for (int j = threadIdx.x; j < half; j += 256) {
    float s = 0.f, c = 1.f;
    if (j < n_pairs) {
      sincosf(pos * inv_freq[j], &s, &c);
      s *= mag;
      c *= mag;
    }
    cosv[j] = c;
    sinv[j] = s;
  }
  __syncthreads();
  // the two entries pair j turns: (2j, 2j+1), or (j, j + n_pairs) among the rotating ones of the
  // half layout (the pairs behind them are the entries that pass)
  const bool halves = half_layout != 0;
  T* qrow = q_out + (size_t)t * ldq;
  for (int i = threadIdx.x; i < H * half; i += 256) {
    const int h = i / half, j = i - h * half;
    const int a = (halves && j < n_pairs) ? j : 2 * j;
    const int b = (halves && j < n_pairs) ? j + n_pairs : 2 * j + 1;
    const T* src = q_src + (size_t)t * ldqs + q_off + (size_t)h * (dn + dr) + dn;
    const float u = to_float<T>(src[a]), v = to_float<T>(src[b]);
    T* dst = qrow + (size_t)h * (R + dr) + R;
    dst[a] = from_float<T>(u * cosv[j] - v * sinv[j]);
    dst[b] = from_float<T>(v * cosv[j] + u * sinv[j]);
  }
  if (kv_off < 0 || !slots) return;
  const int64_t slot = slots[t];
  if (slot < 0) return;                   // (uniform over the workgroup)
  const T* d = kv_src + (size_t)t * ldkv + kv_off;
  float ss = 0.f;
  for (int i = threadIdx.x; i < R; i += 256) {
    const float v = to_float<T>(d[i]);
    ss = fmaf(v, v, ss);
  }
  ss = block_sum(ss, scratch);
  const float r = 1.0f / sqrtf(ss / (float)R + eps);
  T* dst = cache + (size_t)slot * (R + dr);
  for (int i = threadIdx.x; i < R; i += 256) dst[i] = from_float<T>(to_float<T>(d[i]) * r * c_w[i]);
  for (int j = threadIdx.x; j < half; j += 256) {
    const int a = (halves && j < n_pairs) ? j : 2 * j;
    const int b = (halves && j < n_pairs) ? j + n_pairs : 2 * j + 1;
    const float u = to_float<T>(d[R + a]), v = to_float<T>(d[R + b]);
    dst[R + a] = from_float<T>(u * cosv[j] - v * sinv[j]);
    dst[R + b] = from_float<T>(v * cosv[j] + u * sinv[j]);
  }
}

// q_out [T, H, R + dr] (row stride ldq); q_src [T, ldqs] with the queries [H, dn + dr] from column
// q_off; kv_src [T, ldkv] (it may be q_src) with the down-projection [R + dr] from column kv_off
// (kv_off < 0: the layer has none and writes no cache); cache: [slots, R + dr] (pages of one kv
// head, so slot * (R + dr) is the row); slots null: nothing is written.
extern "C" int ptl_latent_prepare(void* q_out, long ldq, const void* q_src, long ldqs, int q_off,
                                  const void* kv_src, long ldkv, int kv_off,
                                  const int32_t* positions, const float* inv_freq, int n_pairs,
                                  int half_layout, float mag,
                                  const float* c_w, float eps, const int32_t* slots, void* cache,
                                  int T_, int H, int dn, int dr, int R, int dtype, hipStream_t st) {
  if (T_ <= 0) return PTL_OK;
  if (H <= 0 || dn < 0 || dr < 0 || (dr & 1) || R <= 0 || n_pairs < 0 || 2 * n_pairs > dr) return PTL_ERR_ARG;
  if (n_pairs > 0 && !inv_freq) return PTL_ERR_ARG;
  if (!q_src || (kv_off >= 0 && !kv_src)) return PTL_ERR_ARG;
  if (kv_off >= 0 && slots && (!cache || !c_w)) return PTL_ERR_ARG;
  const size_t lds = (size_t)(dr + 16) * sizeof(float);
  if (dtype == PTL_DTYPE_F32)
    latent_prepare_kernel<float><<<T_, 256, lds, st>>>((float*)q_out, ldq, (const float*)q_src, ldqs, q_off,
                                                       (const float*)kv_src, ldkv, kv_off, positions, inv_freq,
                                                       n_pairs, half_layout, mag, c_w, eps, slots,
                                                       (float*)cache, H, dn, dr, R);
  else if (dtype == PTL_DTYPE_BF16)
    latent_prepare_kernel<bf16_t><<<T_, 256, lds, st>>>((bf16_t*)q_out, ldq, (const bf16_t*)q_src, ldqs, q_off,
                                                        (const bf16_t*)kv_src, ldkv, kv_off, positions,
                                                        inv_freq, n_pairs, half_layout, mag, c_w, eps, slots,
                                                        (bf16_t*)cache, H, dn, dr, R);
  else
    return PTL_ERR_ARG;
  return ptl_launch_status();
}

// ---------------------------------------------------------------------------------------------
// Per-head products, vector-FMA form for any sizes and both dtypes (float32 accumulation): the
// tile scheme of ptl_gemm_nt with the head as blockIdx.z.
#define HT 64
#define HK 16

template <typename T>
__global__ void __launch_bounds__(256)
gemm_heads_nt_kernel(T* __restrict__ out, long ldo, long ohs, const T* __restrict__ x, long ldx, long xhs,
                     const T* __restrict__ w, int M, int N, int K, const T* __restrict__ gate, long ldg) {
  __shared__ float As[HK][HT + 4];
  __shared__ float Bs[HK][HT + 4];
  const int tid = threadIdx.x;
  const int h = blockIdx.z;
  const int m0 = blockIdx.y * HT, n0 = blockIdx.x * HT;
  x += (size_t)h * xhs;
  w += (size_t)h * N * K;
  out += (size_t)h * ohs;
  const int lr = tid >> 2, lk = (tid & 3) << 2;
  const int ty = tid >> 4, tx = tid & 15;
  float acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = 0.f;
  for (int k0 = 0; k0 < K; k0 += HK) {
    const int m = m0 + lr, n = n0 + lr;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int k = k0 + lk + i;
      As[lk + i][lr] = (m < M && k < K) ? to_float<T>(x[(size_t)m * ldx + k]) : 0.f;
      Bs[lk + i][lr] = (n < N && k < K) ? to_float<T>(w[(size_t)n * K + k]) : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int k = 0; k < HK; ++k) {
      float a[4], b[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) a[i] = As[k][ty * 4 + i];
#pragma unroll
      for (int j = 0; j < 4; ++j) b[j] = Bs[k][tx * 4 + j];
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(a[i], b[j], acc[i][j]);
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int m = m0 + ty * 4 + i;
    if (m >= M) continue;
    float f = 1.f;
    if (gate) f = 1.0f / (1.0f + expf(-to_float<T>(gate[(size_t)m * ldg + h])));
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int n = n0 + tx * 4 + j;
      if (n < N) out[(size_t)m * ldo + n] = from_float<T>(acc[i][j] * f);
    }
  }
}

// Matrix-core form for bfloat16: a wave owns 16 rows x 64 columns of one head's result and takes
// its fragments straight from memory (both operands are contiguous along K: eight consecutive
// values a lane, one 16-byte load), four waves a workgroup share the columns' weights through
// the caches. Needs K % 8 == 0 and 16-byte aligned rows of x and W.
__global__ void __launch_bounds__(256)
gemm_heads_nt_mfma_kernel(bf16_t* __restrict__ out, long ldo, long ohs, const bf16_t* __restrict__ x, long ldx,
                          long xhs, const bf16_t* __restrict__ w, int M, int N, int K,
                          const bf16_t* __restrict__ gate, long ldg) {
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int ln = lane & 15, lg = lane >> 4;
  const int h = blockIdx.z;
  const int m0 = blockIdx.y * 64 + wave * 16, n0 = blockIdx.x * 64;
  if (m0 >= M) return;
  x += (size_t)h * xhs;
  w += (size_t)h * N * K;
  out += (size_t)h * ohs;
  const int am = m0 + ln;
  const bf16_t* arow = x + (size_t)min(am, M - 1) * ldx;
  const bf16_t* brow[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) brow[j] = w + (size_t)min(n0 + 16 * j + ln, N - 1) * K;
  f32x4_t acc[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) acc[j] = f32x4_t{0.f, 0.f, 0.f, 0.f};
  const uint4 zero = make_uint4(0, 0, 0, 0);
  for (int k0 = 0; k0 < K; k0 += 32) {
    const int k = k0 + 8 * lg;
    Frag8 a, b[4];
    a.u = k < K ? *reinterpret_cast<const uint4*>(arow + k) : zero;
#pragma unroll
    for (int j = 0; j < 4; ++j) b[j].u = k < K ? *reinterpret_cast<const uint4*>(brow[j] + k) : zero;
    // result tile [n, m]: the weights as A (rows n), x as B (columns m)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(b[j].v, a.v, acc[j], 0, 0, 0);
  }
  // lane holds, of tile j, column m = m0 + ln and rows n = n0 + 16 j + 4 lg + i
  if (am < M) {
    float f = 1.f;
    if (gate) f = 1.0f / (1.0f + expf(-bf16_to_float(gate[(size_t)am * ldg + h])));
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int n = n0 + 16 * j + 4 * lg + i;
        if (n < N) out[(size_t)am * ldo + n] = float_to_bf16(acc[j][i] * f);
      }
  }
}

// out[t, h, n] at out[t * ldo + h * ohs + n]; x[t, h, k] at x[t * ldx + h * xhs + k]; w [H, N, K]
// dense; gate (or null): gate[t * ldg + h], the logit whose sigmoid multiplies head h of row t.
extern "C" int ptl_gemm_heads_nt(void* out, long ldo, long ohs, const void* x, long ldx, long xhs,
                                 const void* w, int M, int H, int N, int K, const void* gate, long ldg,
                                 int dtype, hipStream_t st) {
  if (M <= 0 || H <= 0 || N <= 0) return PTL_OK;
  if (K <= 0) return PTL_ERR_ARG;
  dim3 grid((N + HT - 1) / HT, (M + HT - 1) / HT, H);
  if (grid.y > 65535 || grid.z > 65535) return PTL_ERR_ARG;
  if (dtype == PTL_DTYPE_F32) {
    gemm_heads_nt_kernel<float><<<grid, 256, 0, st>>>((float*)out, ldo, ohs, (const float*)x, ldx, xhs,
                                                      (const float*)w, M, N, K, (const float*)gate, ldg);
  } else if (dtype == PTL_DTYPE_BF16) {
    const bool fast = K % 8 == 0 && ldx % 8 == 0 && xhs % 8 == 0 &&
                      ((uintptr_t)x | (uintptr_t)w) % 16 == 0;
    if (fast)
      gemm_heads_nt_mfma_kernel<<<grid, 256, 0, st>>>((bf16_t*)out, ldo, ohs, (const bf16_t*)x, ldx, xhs,
                                                      (const bf16_t*)w, M, N, K, (const bf16_t*)gate, ldg);
    else
      gemm_heads_nt_kernel<bf16_t><<<grid, 256, 0, st>>>((bf16_t*)out, ldo, ohs, (const bf16_t*)x, ldx, xhs,
                                                         (const bf16_t*)w, M, N, K, (const bf16_t*)gate, ldg);
  } else {
    return PTL_ERR_ARG;
  }
  return ptl_launch_status();
}
