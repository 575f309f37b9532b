// A residual stream that is kept in float32 whatever the engine's dtype, and the norms that read
// and feed it:
//
//   Dynamic Tanh          y = tanh(alpha * x) * w + b            (elementwise, nothing of the row)
//   RMS norm              y = x * rsqrt(mean(x^2) + eps) * w
//
// ptl_stream_add_dyt: stream += post(y) and out = pre(stream) in one pass over the rows: the norm
//   behind a sublayer, the residual sum and the norm in front of the next sublayer. Every piece
//   is optional: no y (only the norm in front), no post norm (a plain sum), no out, and a copy
//   of the new stream in the engine's dtype for a product that reads the stream itself.
// ptl_stream_add_rmsnorm: stream += rmsnorm(y) * w, the same with a norm that needs the row.
// ptl_stream_add_rmsnorm_sum: the same for a result that is a weighted sum of two and a bias.
// ptl_stream_rmsnorm: the RMS norm of rows of the stream, in the engine's type.
// ptl_dyt: the norm alone, for rows that are no stream (the rows picked for the head).
// ptl_embedding_scaled: stream[t] = table[ids[t]] * scale, in float32 (``copies`` times side by side in
//   a row, for a model that keeps several streams).
// ptl_hyper_mix: several residual streams a token (hyper-connections): the streams' update behind a
//   sublayer and the read-out with its RMS norm in front of the next one (where it stands, below).
// ptl_gelu_gather_mul: out[t, j] = gelu_tanh(z[t, j]) * table[ids[t], col0 + j]: a gate on a
//   per-token vector looked up in a table that several layers share.
//
// All arithmetic is float32; tanhf / expf are the accurate ones.
#include "common.h"
#include <math.h>

struct DytArgs {
  const float* w;     // [H]; null: the norm is absent
  const float* b;     // [H] or null
  float alpha;
};

__device__ __forceinline__ float dyt_apply(const DytArgs& n, float x, int c) {
  const float y = tanhf(n.alpha * x) * n.w[c];
  return n.b ? y + n.b[c] : y;
}

template <typename TY, typename TO>
__global__ void __launch_bounds__(256)
stream_add_dyt_kernel(float* __restrict__ stream, const TY* __restrict__ y, DytArgs post,
                      TO* __restrict__ out, DytArgs pre, TO* __restrict__ copy, size_t total, int H) {
  size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
  const size_t step = (size_t)gridDim.x * 256;
  for (; i < total; i += step) {
    const int c = (int)(i % H);
    float s = stream[i];
    if (y) {
      const float v = to_float<TY>(y[i]);
      s += post.w ? dyt_apply(post, v, c) : v;
      stream[i] = s;
    }
    if (out) out[i] = from_float<TO>(dyt_apply(pre, s, c));
    if (copy) copy[i] = from_float<TO>(s);
  }
}

template <typename TY, typename TO>
static int launch_add_dyt(float* stream, const void* y, DytArgs post, void* out, DytArgs pre, void* copy,
                          size_t total, int H, hipStream_t st) {
  size_t blocks = (total + 255) / 256;
  if (blocks > 65536) blocks = 65536;
  stream_add_dyt_kernel<TY, TO><<<(int)blocks, 256, 0, st>>>(stream, (const TY*)y, post, (TO*)out, pre,
                                                            (TO*)copy, total, H);
  return ptl_launch_status();
}

// y_dtype: of y; out_dtype: of out and copy. Null pointers switch the pieces off (see above).
extern "C" int ptl_stream_add_dyt(float* stream, const void* y, int y_dtype, const float* post_w,
                                  const float* post_b, float post_alpha, void* out, int out_dtype,
                                  const float* pre_w, const float* pre_b, float pre_alpha, void* copy,
                                  int T_, int H, hipStream_t st) {
  if (T_ <= 0) return PTL_OK;
  if (H <= 0 || !stream || (out && !pre_w)) return PTL_ERR_ARG;
  const DytArgs post{post_w, post_b, post_alpha}, pre{pre_w, pre_b, pre_alpha};
  const size_t total = (size_t)T_ * H;
#define GO(TY, TO) return launch_add_dyt<TY, TO>(stream, y, post, out, pre, copy, total, H, st)
  if (y_dtype == PTL_DTYPE_F32 && out_dtype == PTL_DTYPE_F32) GO(float, float);
  if (y_dtype == PTL_DTYPE_F32 && out_dtype == PTL_DTYPE_BF16) GO(float, bf16_t);
  if (y_dtype == PTL_DTYPE_BF16 && out_dtype == PTL_DTYPE_BF16) GO(bf16_t, bf16_t);
  if (y_dtype == PTL_DTYPE_BF16 && out_dtype == PTL_DTYPE_F32) GO(bf16_t, float);
#undef GO
  return PTL_ERR_ARG;
}

template <typename TX, typename TO>
__global__ void __launch_bounds__(256)
dyt_kernel(TO* __restrict__ out, const TX* __restrict__ x, DytArgs n, size_t total, int H) {
  size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
  const size_t step = (size_t)gridDim.x * 256;
  for (; i < total; i += step) out[i] = from_float<TO>(dyt_apply(n, to_float<TX>(x[i]), (int)(i % H)));
}

extern "C" int ptl_dyt(void* out, int out_dtype, const void* x, int x_dtype, const float* w,
                       const float* b, float alpha, int T_, int H, hipStream_t st) {
  if (T_ <= 0) return PTL_OK;
  if (H <= 0 || !w) return PTL_ERR_ARG;
  const DytArgs n{w, b, alpha};
  const size_t total = (size_t)T_ * H;
  size_t blocks = (total + 255) / 256;
  if (blocks > 65536) blocks = 65536;
#define GO(TX, TO)                                                                                   \
  {                                                                                                  \
    dyt_kernel<TX, TO><<<(int)blocks, 256, 0, st>>>((TO*)out, (const TX*)x, n, total, H);            \
    return ptl_launch_status();                                                                      \
  }
  if (x_dtype == PTL_DTYPE_F32 && out_dtype == PTL_DTYPE_F32) GO(float, float);
  if (x_dtype == PTL_DTYPE_F32 && out_dtype == PTL_DTYPE_BF16) GO(float, bf16_t);
  if (x_dtype == PTL_DTYPE_BF16 && out_dtype == PTL_DTYPE_BF16) GO(bf16_t, bf16_t);
  if (x_dtype == PTL_DTYPE_BF16 && out_dtype == PTL_DTYPE_F32) GO(bf16_t, float);
#undef GO
  return PTL_ERR_ARG;
}

// One workgroup a row: the sum of squares of y, then stream += y * rsqrt(mean + eps) * w and, when
// asked for, out = pre(stream) and the copy of the new stream.
template <typename TY, typename TO>
__global__ void __launch_bounds__(256)
stream_add_rmsnorm_kernel(float* __restrict__ stream, const TY* __restrict__ y, const float* __restrict__ w,
                          float eps, TO* __restrict__ out, DytArgs pre, TO* __restrict__ copy, int H) {
  __shared__ float scratch[16];
  const size_t row = (size_t)blockIdx.x * H;
  float ss = 0.f;
  for (int c = threadIdx.x; c < H; c += 256) {
    const float v = to_float<TY>(y[row + c]);
    ss = fmaf(v, v, ss);
  }
  ss = block_sum(ss, scratch);
  const float r = 1.0f / sqrtf(ss / (float)H + eps);
  for (int c = threadIdx.x; c < H; c += 256) {
    const float s = stream[row + c] + to_float<TY>(y[row + c]) * r * w[c];
    stream[row + c] = s;
    if (out) out[row + c] = from_float<TO>(dyt_apply(pre, s, c));
    if (copy) copy[row + c] = from_float<TO>(s);
  }
}

extern "C" int ptl_stream_add_rmsnorm(float* stream, const void* y, int y_dtype, const float* w, float eps,
                                      void* out, int out_dtype, const float* pre_w, const float* pre_b,
                                      float pre_alpha, void* copy, int T_, int H, hipStream_t st) {
  if (T_ <= 0) return PTL_OK;
  if (H <= 0 || !stream || !y || !w || (out && !pre_w)) return PTL_ERR_ARG;
  const DytArgs pre{pre_w, pre_b, pre_alpha};
#define GO(TY, TO)                                                                                   \
  {                                                                                                  \
    stream_add_rmsnorm_kernel<TY, TO><<<T_, 256, 0, st>>>(stream, (const TY*)y, w, eps, (TO*)out, pre, \
                                                          (TO*)copy, H);                             \
    return ptl_launch_status();                                                                      \
  }
  if (y_dtype == PTL_DTYPE_F32 && out_dtype == PTL_DTYPE_F32) GO(float, float);
  if (y_dtype == PTL_DTYPE_F32 && out_dtype == PTL_DTYPE_BF16) GO(float, bf16_t);
  if (y_dtype == PTL_DTYPE_BF16 && out_dtype == PTL_DTYPE_BF16) GO(bf16_t, bf16_t);
  if (y_dtype == PTL_DTYPE_BF16 && out_dtype == PTL_DTYPE_F32) GO(bf16_t, float);
#undef GO
  return PTL_ERR_ARG;
}

// The same for a sublayer whose result is a weighted sum that has not been added up yet:
// y = a y1 + b y2 + c bias (y2 and bias optional), stream += rmsnorm(y) * w. The sum is float32.
template <typename TY, typename TO>
__global__ void __launch_bounds__(256)
stream_add_rmsnorm_sum_kernel(float* __restrict__ stream, const TY* __restrict__ y1, float a,
                              const TY* __restrict__ y2, float b, const float* __restrict__ bias, float c,
                              const float* __restrict__ w, float eps, TO* __restrict__ copy, int H) {
  __shared__ float scratch[16];
  const size_t row = (size_t)blockIdx.x * H;
  float ss = 0.f;
  for (int j = threadIdx.x; j < H; j += 256) {
    float v = a * to_float<TY>(y1[row + j]);
    if (y2) v = fmaf(b, to_float<TY>(y2[row + j]), v);
    if (bias) v = fmaf(c, bias[j], v);
    ss = fmaf(v, v, ss);
  }
  ss = block_sum(ss, scratch);
  const float r = 1.0f / sqrtf(ss / (float)H + eps);
  for (int j = threadIdx.x; j < H; j += 256) {
    float v = a * to_float<TY>(y1[row + j]);
    if (y2) v = fmaf(b, to_float<TY>(y2[row + j]), v);
    if (bias) v = fmaf(c, bias[j], v);
    const float s = stream[row + j] + v * r * w[j];
    stream[row + j] = s;
    if (copy) copy[row + j] = from_float<TO>(s);
  }
}

extern "C" int ptl_stream_add_rmsnorm_sum(float* stream, const void* y1, float a, const void* y2, float b,
                                          int y_dtype, const float* bias, float c, const float* w, float eps,
                                          void* copy, int out_dtype, int T_, int H, hipStream_t st) {
  if (T_ <= 0) return PTL_OK;
  if (H <= 0 || !stream || !y1 || !w) return PTL_ERR_ARG;
#define GO(TY, TO)                                                                                    \
  {                                                                                                   \
    stream_add_rmsnorm_sum_kernel<TY, TO><<<T_, 256, 0, st>>>(stream, (const TY*)y1, a, (const TY*)y2, b, \
                                                              bias, c, w, eps, (TO*)copy, H);         \
    return ptl_launch_status();                                                                       \
  }
  if (y_dtype == PTL_DTYPE_F32 && out_dtype == PTL_DTYPE_F32) GO(float, float);
  if (y_dtype == PTL_DTYPE_F32 && out_dtype == PTL_DTYPE_BF16) GO(float, bf16_t);
  if (y_dtype == PTL_DTYPE_BF16 && out_dtype == PTL_DTYPE_BF16) GO(bf16_t, bf16_t);
  if (y_dtype == PTL_DTYPE_BF16 && out_dtype == PTL_DTYPE_F32) GO(bf16_t, float);
#undef GO
  return PTL_ERR_ARG;
}

// out = x * rsqrt(mean(x^2) + eps) * w for rows of a float32 stream, in the engine's type (the rows
// picked for the head).
template <typename TO>
__global__ void __launch_bounds__(256)
stream_rmsnorm_kernel(TO* __restrict__ out, const float* __restrict__ x, const float* __restrict__ w,
                      float eps, int H) {
  __shared__ float scratch[16];
  const size_t row = (size_t)blockIdx.x * H;
  float ss = 0.f;
  for (int j = threadIdx.x; j < H; j += 256) ss = fmaf(x[row + j], x[row + j], ss);
  ss = block_sum(ss, scratch);
  const float r = 1.0f / sqrtf(ss / (float)H + eps);
  for (int j = threadIdx.x; j < H; j += 256) out[row + j] = from_float<TO>(x[row + j] * r * w[j]);
}

extern "C" int ptl_stream_rmsnorm(void* out, int out_dtype, const float* x, const float* w, float eps,
                                  int T_, int H, hipStream_t st) {
  if (T_ <= 0) return PTL_OK;
  if (H <= 0 || !x || !w) return PTL_ERR_ARG;
  if (out_dtype == PTL_DTYPE_F32)
    stream_rmsnorm_kernel<float><<<T_, 256, 0, st>>>((float*)out, x, w, eps, H);
  else if (out_dtype == PTL_DTYPE_BF16)
    stream_rmsnorm_kernel<bf16_t><<<T_, 256, 0, st>>>((bf16_t*)out, x, w, eps, H);
  else
    return PTL_ERR_ARG;
  return ptl_launch_status();
}

template <typename T>
__global__ void embedding_scaled_kernel(float* __restrict__ out, const T* __restrict__ table,
                                        const int32_t* __restrict__ ids, int H, int V, float scale,
                                        int copies) {
  const int t = blockIdx.x;
  int id = ids[t];
  if (id < 0 || id >= V) id = 0;          // checked on the host; never read out of bounds
  const T* src = table + (size_t)id * H;
  float* dst = out + (size_t)t * H * copies;
  for (int i = threadIdx.x; i < H; i += blockDim.x) {
    const float v = to_float<T>(src[i]) * scale;
    for (int s = 0; s < copies; ++s) dst[(size_t)s * H + i] = v;
  }
}

extern "C" int ptl_embedding_scaled(float* out, const void* table, const int32_t* ids, int T_, int H,
                                    int V, float scale, int copies, int dtype, hipStream_t st) {
  if (T_ <= 0) return PTL_OK;
  if (H <= 0 || V <= 0 || copies < 1) return PTL_ERR_ARG;
  const int threads = H >= 1024 ? 256 : (H >= 256 ? 128 : 64);
  if (dtype == PTL_DTYPE_F32)
    embedding_scaled_kernel<float><<<T_, threads, 0, st>>>(out, (const float*)table, ids, H, V, scale, copies);
  else if (dtype == PTL_DTYPE_BF16)
    embedding_scaled_kernel<bf16_t><<<T_, threads, 0, st>>>(out, (const bf16_t*)table, ids, H, V, scale, copies);
  else
    return PTL_ERR_ARG;
  return ptl_launch_status();
}

// out[t] = e * rsqrt(mean(e^2) + eps) * w with e = table[ids[t]] * scale, as float32: a residual
// stream that starts from the normed embedding, in one pass over the row.
template <typename T>
__global__ void __launch_bounds__(256)
embedding_rmsnorm_kernel(float* __restrict__ out, const T* __restrict__ table, const int32_t* __restrict__ ids,
                         const float* __restrict__ w, float eps, int H, int V, float scale) {
  __shared__ float scratch[16];
  const int t = blockIdx.x;
  int id = ids[t];
  if (id < 0 || id >= V) id = 0;          // checked on the host; never read out of bounds
  const T* src = table + (size_t)id * H;
  float* dst = out + (size_t)t * H;
  float ss = 0.f;
  for (int j = threadIdx.x; j < H; j += 256) {
    const float v = to_float<T>(src[j]) * scale;
    ss = fmaf(v, v, ss);
  }
  ss = block_sum(ss, scratch);
  const float r = 1.0f / sqrtf(ss / (float)H + eps);
  for (int j = threadIdx.x; j < H; j += 256) dst[j] = to_float<T>(src[j]) * scale * r * w[j];
}

extern "C" int ptl_embedding_rmsnorm(float* out, const void* table, const int32_t* ids, const float* w,
                                     float eps, int T_, int H, int V, float scale, int dtype, hipStream_t st) {
  if (T_ <= 0) return PTL_OK;
  if (H <= 0 || V <= 0 || !w) return PTL_ERR_ARG;
  if (dtype == PTL_DTYPE_F32)
    embedding_rmsnorm_kernel<float><<<T_, 256, 0, st>>>(out, (const float*)table, ids, w, eps, H, V, scale);
  else if (dtype == PTL_DTYPE_BF16)
    embedding_rmsnorm_kernel<bf16_t><<<T_, 256, 0, st>>>(out, (const bf16_t*)table, ids, w, eps, H, V, scale);
  else
    return PTL_ERR_ARG;
  return ptl_launch_status();
}

__device__ __forceinline__ float gelu_tanh(float z) {
  return 0.5f * z * (1.0f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z)));
}

template <typename T>
__global__ void __launch_bounds__(256)
gelu_gather_mul_kernel(T* __restrict__ out, const T* __restrict__ z, const T* __restrict__ table,
                       const int32_t* __restrict__ ids, int n, int ld, int col0, int V, size_t total) {
  const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= total) return;
  const size_t t = i / n;
  const int j = (int)(i - t * n);
  int id = ids[t];
  if (id < 0 || id >= V) id = 0;
  const float e = to_float<T>(table[(size_t)id * ld + col0 + j]);
  out[i] = from_float<T>(gelu_tanh(to_float<T>(z[i])) * e);
}

// z, out [T, n] dense; table [V, ld]; the token's vector is table[id, col0 : col0 + n]
extern "C" int ptl_gelu_gather_mul(void* out, const void* z, const void* table, const int32_t* ids,
                                   int T_, int n, int ld, int col0, int V, int dtype, hipStream_t st) {
  if (T_ <= 0) return PTL_OK;
  if (n <= 0 || V <= 0 || col0 < 0 || col0 + n > ld) return PTL_ERR_ARG;
  const size_t total = (size_t)T_ * n;
  const size_t blocks = (total + 255) / 256;
  if (blocks > 0x7fffffff) return PTL_ERR_ARG;
  if (dtype == PTL_DTYPE_F32)
    gelu_gather_mul_kernel<float><<<(int)blocks, 256, 0, st>>>((float*)out, (const float*)z,
                                                               (const float*)table, ids, n, ld, col0, V, total);
  else if (dtype == PTL_DTYPE_BF16)
    gelu_gather_mul_kernel<bf16_t><<<(int)blocks, 256, 0, st>>>((bf16_t*)out, (const bf16_t*)z,
                                                                (const bf16_t*)table, ids, n, ld, col0, V, total);
  else
    return PTL_ERR_ARG;
  return ptl_launch_status();
}

// Hyper-connections: a token has S residual streams x_1 .. x_S, [T, S, H] float32. Around a sublayer
//
//   u = sum_s in[s] x_s;   y = sublayer(rmsnorm(u) w);   x_t <- sum_s mix[s, t] x_s + out[t] y
//
// (all streams at once from the old ones). One kernel makes the update behind a sublayer and the
// read-out in front of the next one: with y, the streams are updated in place; with nw, u is read
// from the (new) streams and normed into ``out``. Either half may be absent. Null coefficients
// stand for a single plain stream: in = ones, mix = the identity, out = ones (then S = 1 is the
// residual sum in front of a norm, and in = ones alone is the sum of the streams). One workgroup
// a token (of 1,024 threads when the rows are few, else 256); u waits in LDS between the pass that makes it and the one that scales it.
#define HYPER_MAX_S 16

template <int SM, int NT, typename TY, typename TO>
__global__ void __launch_bounds__(NT)
hyper_mix_kernel(float* __restrict__ streams, const TY* __restrict__ y, const float* __restrict__ mix,
                 const float* __restrict__ outc, const float* __restrict__ inc, const float* __restrict__ nw,
                 float eps, TO* __restrict__ out, int S, int H) {
  extern __shared__ float us[];            // [H]
  __shared__ float scratch[16];
  __shared__ float cm[HYPER_MAX_S * HYPER_MAX_S], co[HYPER_MAX_S], ci[HYPER_MAX_S];
  const int tid = threadIdx.x;
  if (tid < S * S) cm[tid] = mix ? mix[tid] : (tid / S == tid % S ? 1.f : 0.f);
  if (tid < S) {
    co[tid] = outc ? outc[tid] : 1.f;
    ci[tid] = inc ? inc[tid] : 1.f;
  }
  __syncthreads();
  float* row = streams + (size_t)blockIdx.x * S * H;
  float ss = 0.f;
  for (int c = tid; c < H; c += NT) {
    float x[SM];
#pragma unroll
    for (int s = 0; s < SM; ++s) x[s] = s < S ? row[(size_t)s * H + c] : 0.f;
    if (y) {
      const float v = to_float<TY>(y[(size_t)blockIdx.x * H + c]);
      float nx[SM];
#pragma unroll
      for (int t = 0; t < SM; ++t) {
        float a = t < S ? co[t] * v : 0.f;         // (entries from S on are not there: never read)
#pragma unroll
        for (int s = 0; s < SM; ++s) a = fmaf(s < S && t < S ? cm[s * S + t] : 0.f, x[s], a);
        nx[t] = t < S ? a : 0.f;
      }
#pragma unroll
      for (int t = 0; t < SM; ++t) {
        x[t] = nx[t];
        if (t < S) row[(size_t)t * H + c] = nx[t];
      }
    }
    if (nw) {
      float u = 0.f;
#pragma unroll
      for (int s = 0; s < SM; ++s) u = fmaf(s < S ? ci[s] : 0.f, x[s], u);
      us[c] = u;
      ss = fmaf(u, u, ss);
    }
  }
  if (!nw) return;
  ss = block_sum(ss, scratch);
  const float r = 1.0f / sqrtf(ss / (float)H + eps);
  for (int c = tid; c < H; c += NT) out[(size_t)blockIdx.x * H + c] = from_float<TO>(us[c] * r * nw[c]);
}

template <typename TY, typename TO>
static int launch_hyper(float* streams, const void* y, const float* mix, const float* outc, const float* inc,
                        const float* nw, float eps, void* out, int T_, int S, int H, hipStream_t st) {
  const size_t lds = nw ? (size_t)H * sizeof(float) : 0;
  // few rows: a row's entries over 1,024 threads, so that a thread's loads are one or two deep
  const bool few = T_ <= 512 && H > 256;
#define GO(SM)                                                                                       \
  {                                                                                                  \
    if (lds > 48 * 1024 &&                                                                           \
        (hipFuncSetAttribute((const void*)hyper_mix_kernel<SM, 256, TY, TO>,                         \
                             hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess ||  \
         hipFuncSetAttribute((const void*)hyper_mix_kernel<SM, 1024, TY, TO>,                        \
                             hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess))   \
      return PTL_ERR_LAUNCH;                                                                         \
    if (few)                                                                                         \
      hyper_mix_kernel<SM, 1024, TY, TO><<<T_, 1024, lds, st>>>(streams, (const TY*)y, mix, outc, inc, nw, \
                                                                eps, (TO*)out, S, H);                \
    else                                                                                             \
      hyper_mix_kernel<SM, 256, TY, TO><<<T_, 256, lds, st>>>(streams, (const TY*)y, mix, outc, inc, nw,   \
                                                              eps, (TO*)out, S, H);                  \
    return ptl_launch_status();                                                                      \
  }
  if (S <= 1) GO(1)
  if (S <= 2) GO(2)
  if (S <= 4) GO(4)
  if (S <= 8) GO(8)
  GO(16)
#undef GO
}

// streams [T, S, H] float32 (updated in place when y is given); y [T, H] of y_dtype or null; mix
// [S, S] (from, to), outc [S], inc [S] float32 or null; nw [H] float32 or null: no read-out; out
// [T, H] of out_dtype.
extern "C" int ptl_hyper_mix(float* streams, const void* y, int y_dtype, const float* mix, const float* outc,
                             const float* inc, const float* nw, float eps, void* out, int out_dtype, int T_,
                             int S, int H, hipStream_t st) {
  if (T_ <= 0) return PTL_OK;
  if (H <= 0 || S < 1 || S > HYPER_MAX_S || !streams || (nw && !out) || (!y && !nw) ||
      (size_t)H * sizeof(float) > 150 * 1024)
    return PTL_ERR_ARG;
#define GO(TY, TO) return launch_hyper<TY, TO>(streams, y, mix, outc, inc, nw, eps, out, T_, S, H, st)
  if (y_dtype == PTL_DTYPE_F32 && out_dtype == PTL_DTYPE_F32) GO(float, float);
  if (y_dtype == PTL_DTYPE_F32 && out_dtype == PTL_DTYPE_BF16) GO(float, bf16_t);
  if (y_dtype == PTL_DTYPE_BF16 && out_dtype == PTL_DTYPE_BF16) GO(bf16_t, bf16_t);
  if (y_dtype == PTL_DTYPE_BF16 && out_dtype == PTL_DTYPE_F32) GO(bf16_t, float);
#undef GO
  return PTL_ERR_ARG;
}
