// A routed feed-forward (mixture of experts) that never leaves the device, so that a step with
// one can be recorded as a graph:
//
//   ptl_moe_topk      per token: scores = sigmoid(logits) or softmax(logits) in float32, the ``top``
//                     largest (by score plus a per-expert correction, when one is given), their
//                     experts and scores (the score without the correction is the weight, with or
//                     without a renormalisation over the chosen ones, times a constant); with
//                     groups, the experts form equal groups of neighbours, a group's score is the
//                     sum of its two largest choice scores, and only experts of the best ``keep``
//                     groups can be chosen; experts
//                     from ``real`` on have no matrices and return their input: their pairs get
//                     expert -1 and their weights are added up per token; and the sigmoid of extra
//                     logit columns behind the experts' (a gate of a shared expert)
//   ptl_moe_sort      the (token, choice) pairs ordered by expert: positions, the tiles of
//                     MOE_TM rows that the products walk, all by one workgroup
//   ptl_moe_gate_up   per tile: rows gathered from x, the expert's gate and up matrices, and
//                     the gated activation, written in sorted order. The routing weight scales
//                     the expert's input (it is applied to both products, which are linear) or
//                     is left for the output
//   ptl_moe_up        the same for experts without a gate: act(up(x)), one matrix
//   ptl_moe_down      per tile: the expert's down matrix on the sorted rows
//   ptl_moe_combine   per token: the sum of its choices' rows (times the weight when it scales
//                     the output), plus gate * a shared expert's row, plus the token's input times
//                     the weights of its experts that return their input
//   ptl_unary_act     an ungated expert's activation on a dense product
//   ptl_gated_act     the experts' activation on a dense [T, 2I] gate|up product
//
// Activation kinds: 0: silu(g) * u;  1: g' = min(g, limit), u' = clamp(u, -limit, limit),
// g' * sigmoid(1.702 g') * (u' + 1). Without a gate: 2: relu(u)^2.
#include "common.h"
#include "mfma.h"
#include <math.h>

#define MOE_TM 64

__device__ __forceinline__ float sigmoidf_(float z) { return 1.0f / (1.0f + expf(-z)); }

__device__ __forceinline__ float gated_act(int kind, float g, float u, float limit) {
  if (kind == 1) {
    g = fminf(g, limit);
    u = fminf(fmaxf(u, -limit), limit);
    return g * sigmoidf_(1.702f * g) * (u + 1.0f);
  }
  return g * sigmoidf_(g) * u;
}

__device__ __forceinline__ float unary_act(int kind, float u) {
  (void)kind;                            // (2: the square of relu, the only one so far)
  const float r = fmaxf(u, 0.f);
  return r * r;
}

// One wave a token. Lane l holds the logits of experts l, l + 64, ...: TOPK_PER_LANE of them
// (1, 4 or 16, the least that covers the router's outputs).
#define TOPK_MAX_PER_LANE 16
#define SCORE_SIGMOID 0
#define SCORE_SOFTMAX 1
template <int TOPK_PER_LANE>
__global__ void __launch_bounds__(256)
moe_topk_kernel(const float* __restrict__ logits, int ld, int T_, int E, int top, int extra,
                int renormalize, int score_fn, const float* __restrict__ bias, int real, float renorm_eps,
                float wscale, int n_groups, int keep_groups, int32_t* __restrict__ idx,
                float* __restrict__ wgt, float* __restrict__ extra_out, float* __restrict__ ident_out) {
  __shared__ float choice[4][64 * TOPK_PER_LANE];      // a token's choice scores (groups only)
  const int t = blockIdx.x * 4 + (threadIdx.x >> 6);
  const int lane = threadIdx.x & 63;
  if (t >= T_) return;
  const float* z = logits + (size_t)t * ld;
  // v: what the choice goes by; sc: the score that becomes the weight. Sigmoid scores without a
  // correction are chosen by their logits (the same order, and no ties where the sigmoid saturates).
  float v[TOPK_PER_LANE], sc[TOPK_PER_LANE];
  float zmax = -INFINITY;
#pragma unroll
  for (int i = 0; i < TOPK_PER_LANE; ++i) {
    const int e = lane + 64 * i;
    v[i] = e < E ? z[e] : -INFINITY;
    zmax = fmaxf(zmax, v[i]);
  }
  if (score_fn == SCORE_SOFTMAX) {
    zmax = wave_max(zmax);
    float den = 0.f;
#pragma unroll
    for (int i = 0; i < TOPK_PER_LANE; ++i) {
      sc[i] = lane + 64 * i < E ? expf(v[i] - zmax) : 0.f;
      den += sc[i];
    }
    den = wave_sum(den);
#pragma unroll
    for (int i = 0; i < TOPK_PER_LANE; ++i) sc[i] /= den;
  } else {
#pragma unroll
    for (int i = 0; i < TOPK_PER_LANE; ++i) sc[i] = sigmoidf_(v[i]);
  }
  if (score_fn == SCORE_SOFTMAX || bias || n_groups > 1) {      // (a group's score sums scores)
#pragma unroll
    for (int i = 0; i < TOPK_PER_LANE; ++i) {
      const int e = lane + 64 * i;
      if (e < E) v[i] = bias ? sc[i] + bias[e] : sc[i];
    }
  }
  if (n_groups > 1 && keep_groups < n_groups) {
    // Groups of E / n_groups neighbours; lane g scores group g by its two largest choice scores
    // (a group of one: by its only one); the best keep_groups groups stay (ties: the lower
    // group), the choice scores of all others become minus infinity.
    float* cs = choice[threadIdx.x >> 6];
#pragma unroll
    for (int i = 0; i < TOPK_PER_LANE; ++i)
      if (lane + 64 * i < E) cs[lane + 64 * i] = v[i];
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    const int per = E / n_groups;
    float gs = -INFINITY;
    if (lane < n_groups) {
      float b1 = -INFINITY, b2 = -INFINITY;
      for (int j = 0; j < per; ++j) {
        const float x = cs[lane * per + j];
        if (x > b1) { b2 = b1; b1 = x; }
        else if (x > b2) b2 = x;
      }
      gs = per > 1 ? b1 + b2 : b1;
    }
    int kept = 0;
    for (int k = 0; k < keep_groups; ++k) {
      float best = gs;
      int at = gs == -INFINITY ? 0x7fffffff : lane;
#pragma unroll
      for (int o = 32; o > 0; o >>= 1) {
        const float ob = __shfl_xor(best, o, 64);
        const int oa = __shfl_xor(at, o, 64);
        if (ob > best || (ob == best && oa < at)) {
          best = ob;
          at = oa;
        }
      }
      if (lane == at) {
        kept = 1;
        gs = -INFINITY;
      }
    }
#pragma unroll
    for (int i = 0; i < TOPK_PER_LANE; ++i) {
      const int e = lane + 64 * i;
      const int k = __shfl(kept, (e < E ? e / per : 0) & 63, 64);
      if (e < E && !k) v[i] = -INFINITY;
    }
  }
  float sum = 0.f, ident = 0.f;
  for (int k = 0; k < top; ++k) {
    float best = -INFINITY;
    int at = 0x7fffffff;
#pragma unroll
    for (int i = 0; i < TOPK_PER_LANE; ++i) {
      const int e = lane + 64 * i;
      if (e < E && (v[i] > best || (v[i] == best && e < at)) && v[i] != -INFINITY) {
        best = v[i];
        at = e;
      }
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
      const float ob = __shfl_xor(best, o, 64);
      const int oa = __shfl_xor(at, o, 64);
      if (ob > best || (ob == best && oa < at)) {
        best = ob;
        at = oa;
      }
    }
    if (at >= E) at = k;                 // (only when a logit is NaN: the NaN then shows in the output)
    float mine = 0.f;
#pragma unroll
    for (int i = 0; i < TOPK_PER_LANE; ++i)
      if (lane + 64 * i == at) {
        v[i] = -INFINITY;
        mine = sc[i];
      }
    const float s = __shfl(mine, at & 63, 64);
    sum += s;
    if (lane == 0) {
      idx[(size_t)t * top + k] = at < real ? at : -1;
      wgt[(size_t)t * top + k] = s;
    }
  }
  if (lane == 0) {
    for (int k = 0; k < top; ++k) {
      float w = wgt[(size_t)t * top + k];
      if (renormalize || wscale != 1.f) {
        if (renormalize) w /= sum + renorm_eps;
        w *= wscale;
        wgt[(size_t)t * top + k] = w;
      }
      if (idx[(size_t)t * top + k] < 0) ident += w;
    }
    if (ident_out) ident_out[t] = ident;
  }
  if (lane < extra) extra_out[(size_t)t * extra + lane] = sigmoidf_(z[E + lane]);
}

// logits [T, ld]: E router outputs a row, then ``extra`` columns. score_fn: 0 sigmoid, 1 softmax over
// the E outputs. bias [E] or null: added to the scores for the choice only. real: the first ``real``
// outputs are experts with matrices, the others return their input (idx -1; ident_out [T], which
// must be given when real < E, receives the sum of their weights). Weights: the scores, divided by
// their sum + renorm_eps when ``renormalize``, times wscale. n_groups > 1: the E outputs form that
// many equal groups of neighbours (at most 64) of which the best keep_groups can be chosen from.
extern "C" int ptl_moe_topk(const float* logits, int ld, int T_, int E, int top, int extra, int renormalize,
                            int score_fn, const float* bias, int real, float renorm_eps, float wscale,
                            int n_groups, int keep_groups, int32_t* idx, float* wgt, float* extra_out,
                            float* ident_out, hipStream_t st) {
  if (T_ <= 0) return PTL_OK;
  if (n_groups > 1 && (n_groups > 64 || E % n_groups || keep_groups < 1 || keep_groups > n_groups ||
                       (long)keep_groups * (E / n_groups) < top))
    return PTL_ERR_ARG;
  if (E <= 0 || top <= 0 || top > E || E > 64 * TOPK_MAX_PER_LANE || extra < 0 || extra > 64 || ld < E + extra ||
      (extra && !extra_out) || real < 0 || real > E || (real < E && !ident_out) ||
      (score_fn != SCORE_SIGMOID && score_fn != SCORE_SOFTMAX))
    return PTL_ERR_ARG;
#define GO(PER)                                                                                              \
  moe_topk_kernel<PER><<<(T_ + 3) / 4, 256, 0, st>>>(logits, ld, T_, E, top, extra, renormalize, score_fn, bias, \
                                                     real, renorm_eps, wscale, n_groups, keep_groups, idx, wgt,  \
                                                     extra_out, ident_out)
  if (E <= 64) GO(1);
  else if (E <= 256) GO(4);
  else GO(16);
#undef GO
  return ptl_launch_status();
}

// One workgroup. A = pairs (token, choice). Writes: pos_of[a] (the sorted position of pair a; -1
// for a pair whose expert is outside 0..E-1 and takes no part in the products),
// sorted[p] (the pair at position p), expert_end[e] (one past the last position of expert e),
// and the tile list: tile_expert[i] (-1: no tile), tile_row0[i] for i < max_tiles.
__global__ void __launch_bounds__(1024)
moe_sort_kernel(const int32_t* __restrict__ idx, int A, int E, int32_t* __restrict__ pos_of,
                int32_t* __restrict__ sorted, int32_t* __restrict__ expert_end,
                int32_t* __restrict__ tile_expert, int32_t* __restrict__ tile_row0, int max_tiles) {
  extern __shared__ int32_t sh[];        // count [E], start [E], n_tiles [1]
  int32_t* count = sh;
  int32_t* start = sh + E;
  int32_t* n_tiles = sh + 2 * E;
  for (int e = threadIdx.x; e < E; e += 1024) count[e] = 0;
  __syncthreads();
  for (int a = threadIdx.x; a < A; a += 1024) {
    const int e = idx[a];
    if (e >= 0 && e < E) atomicAdd(&count[e], 1);
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    int at = 0, tile = 0;
    for (int e = 0; e < E; ++e) {
      const int c = count[e];
      start[e] = at;
      for (int r = 0; r < c && tile < max_tiles; r += MOE_TM, ++tile) {
        tile_expert[tile] = e;
        tile_row0[tile] = at + r;
      }
      at += c;
      expert_end[e] = at;
      count[e] = 0;                      // from here on: the places of the expert handed out
    }
    *n_tiles = tile;
  }
  __syncthreads();
  for (int i = *n_tiles + threadIdx.x; i < max_tiles; i += 1024) {
    tile_expert[i] = -1;
    tile_row0[i] = 0;
  }
  // places inside an expert by a counter in LDS: which pair gets which place varies from run
  // to run, the results do not (a row's result does not depend on its place in a tile)
  for (int a = threadIdx.x; a < A; a += 1024) {
    const int e = idx[a];
    if (e < 0 || e >= E) {                 // a pair without an expert's matrices
      pos_of[a] = -1;
      continue;
    }
    const int p = start[e] + atomicAdd(&count[e], 1);
    sorted[p] = a;
    pos_of[a] = p;
  }
}

extern "C" int ptl_moe_max_tiles(int A, int E) { return (A + MOE_TM - 1) / MOE_TM + (A < E ? A : E); }

extern "C" int ptl_moe_sort(const int32_t* idx, int A, int E, int32_t* pos_of, int32_t* sorted,
                            int32_t* expert_end, int32_t* tile_expert, int32_t* tile_row0, int max_tiles,
                            hipStream_t st) {
  if (A <= 0) return PTL_OK;
  if (E <= 0 || E > 8192 || max_tiles < ptl_moe_max_tiles(A, E)) return PTL_ERR_ARG;
  moe_sort_kernel<<<1, 1024, (2 * E + 1) * sizeof(int32_t), st>>>(idx, A, E, pos_of, sorted, expert_end,
                                                                  tile_expert, tile_row0, max_tiles);
  return ptl_launch_status();
}

// ---------------------------------------------------------------------------------------------
// The experts' products over the tile list. Vector-FMA form (any sizes, both dtypes): a tile of
// MOE_TM sorted rows x 64 result columns a workgroup; the gate|up product keeps two sums an
// output (gate row n and up row I + n of the expert's [2 I, K] matrix).
#define MK 16
// what a product is: the down matrix on the sorted rows; gate|up on rows gathered from x, with
// the gated activation; up alone on gathered rows, with an activation of one value
#define MODE_DOWN 0
#define MODE_GATE_UP 1
#define MODE_UP 2

template <typename T, int MODE>
__global__ void __launch_bounds__(256)
moe_gemm_kernel(T* __restrict__ out, long ldo, const T* __restrict__ x, long ldx, const T* __restrict__ w,
                const int32_t* __restrict__ tile_expert, const int32_t* __restrict__ tile_row0,
                const int32_t* __restrict__ expert_end, const int32_t* __restrict__ sorted,
                const float* __restrict__ wgt, int top, int N, int K, int act, float limit) {
  constexpr bool GATE_UP = MODE == MODE_GATE_UP;
  constexpr bool GATHER = MODE != MODE_DOWN;
  const int e = tile_expert[blockIdx.y];
  if (e < 0) return;
  const int row0 = tile_row0[blockIdx.y];
  const int rows = min(MOE_TM, expert_end[e] - row0);
  __shared__ float As[MK][MOE_TM + 4];
  __shared__ float Bs[GATE_UP ? 2 : 1][MK][64 + 4];
  __shared__ int32_t src_row[MOE_TM];
  __shared__ float row_w[MOE_TM];
  const int tid = threadIdx.x;
  if (tid < MOE_TM) {
    int r = -1;
    float f = 1.f;
    if (tid < rows) {
      if (GATHER) {
        const int a = sorted[row0 + tid];
        r = a / top;
        if (wgt) f = wgt[a];
      } else {
        r = row0 + tid;
      }
    }
    src_row[tid] = r;
    row_w[tid] = f;
  }
  __syncthreads();
  const int n0 = blockIdx.x * 64;
  const size_t wrows = GATE_UP ? 2 * (size_t)N : (size_t)N;
  w += (size_t)e * wrows * K;
  const int lr = tid >> 2, lk = (tid & 3) << 2;
  const int ty = tid >> 4, tx = tid & 15;
  float acc[GATE_UP ? 2 : 1][4][4];
#pragma unroll
  for (int g = 0; g < (GATE_UP ? 2 : 1); ++g)
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j) acc[g][i][j] = 0.f;
  const int my_src = src_row[lr];
  for (int k0 = 0; k0 < K; k0 += MK) {
    const int n = n0 + lr;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int k = k0 + lk + i;
      As[lk + i][lr] = (my_src >= 0 && k < K) ? to_float<T>(x[(size_t)my_src * ldx + k]) : 0.f;
      Bs[0][lk + i][lr] = (n < N && k < K) ? to_float<T>(w[(size_t)n * K + k]) : 0.f;
      if (GATE_UP) Bs[1][lk + i][lr] = (n < N && k < K) ? to_float<T>(w[((size_t)N + n) * K + k]) : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int k = 0; k < MK; ++k) {
      float a[4], b[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) a[i] = As[k][ty * 4 + i];
#pragma unroll
      for (int g = 0; g < (GATE_UP ? 2 : 1); ++g) {
#pragma unroll
        for (int j = 0; j < 4; ++j) b[j] = Bs[g][k][tx * 4 + j];
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
          for (int j = 0; j < 4; ++j) acc[g][i][j] = fmaf(a[i], b[j], acc[g][i][j]);
      }
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int m = ty * 4 + i;
    if (m >= rows) continue;
    const float f = row_w[m];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int n = n0 + tx * 4 + j;
      if (n >= N) continue;
      float v;
      if (GATE_UP)
        v = gated_act(act, acc[0][i][j] * f, acc[GATE_UP ? 1 : 0][i][j] * f, limit);
      else if (MODE == MODE_UP)
        v = unary_act(act, acc[0][i][j] * f);
      else
        v = acc[0][i][j];
      out[(size_t)(row0 + m) * ldo + n] = from_float<T>(v);
    }
  }
}

// Matrix-core forms for bfloat16 (K % 8 == 0, aligned rows).
//
// Few pairs (a decode step): fragments straight from memory, 64 result columns a workgroup. A
// tile of at most 16 rows (nearly every tile of a decode step) is shared by the four waves
// along K, 32 values in turn, so that four times as many loads of the expert's weights are under
// way; their partial sums meet in LDS. Taller tiles: a wave owns 16 of the rows.
template <int MODE>
__global__ void __launch_bounds__(256)
moe_gemm_mfma_kernel(bf16_t* __restrict__ out, long ldo, const bf16_t* __restrict__ x, long ldx,
                     const bf16_t* __restrict__ w, const int32_t* __restrict__ tile_expert,
                     const int32_t* __restrict__ tile_row0, const int32_t* __restrict__ expert_end,
                     const int32_t* __restrict__ sorted, const float* __restrict__ wgt, int top, int N, int K,
                     int act, float limit) {
  constexpr bool GATE_UP = MODE == MODE_GATE_UP;
  constexpr bool GATHER = MODE != MODE_DOWN;
  constexpr int G = GATE_UP ? 2 : 1;
  __shared__ float red[3][G * 4][4][64];
  const int e = tile_expert[blockIdx.y];
  if (e < 0) return;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int ln = lane & 15, lg = lane >> 4;
  const int tile_rows = min(MOE_TM, expert_end[e] - tile_row0[blockIdx.y]);
  const bool split = tile_rows <= 16;
  const int row0 = tile_row0[blockIdx.y] + (split ? 0 : 16 * wave);
  const int rows = min(16, expert_end[e] - row0);
  if (rows <= 0) return;                 // (never in a split tile: its waves all stay)
  const int n0 = blockIdx.x * 64;
  const size_t wrows = GATE_UP ? 2 * (size_t)N : (size_t)N;
  w += (size_t)e * wrows * K;
  const int mr = min(ln, rows - 1);
  int src = row0 + mr;
  float f = 1.f;
  if (GATHER) {
    const int a = sorted[src];
    src = a / top;
    if (wgt) f = wgt[a];
  }
  const bf16_t* arow = x + (size_t)src * ldx;
  const bf16_t* brow[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) brow[j] = w + (size_t)min(n0 + 16 * j + ln, N - 1) * K;
  f32x4_t acc[G][4];
#pragma unroll
  for (int g = 0; g < G; ++g)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[g][j] = f32x4_t{0.f, 0.f, 0.f, 0.f};
  const uint4 zero = make_uint4(0, 0, 0, 0);
  const size_t up = (size_t)N * K;
  const int kstep = split ? 128 : 32;
  for (int k0 = split ? 32 * wave : 0; k0 < K; k0 += kstep) {
    const int k = k0 + 8 * lg;
    Frag8 a, b[G][4];
    a.u = k < K ? *reinterpret_cast<const uint4*>(arow + k) : zero;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      b[0][j].u = k < K ? load_once(brow[j] + k) : zero;
      if (GATE_UP) b[G - 1][j].u = k < K ? load_once(brow[j] + up + k) : zero;
    }
#pragma unroll
    for (int g = 0; g < G; ++g)
#pragma unroll
      for (int j = 0; j < 4; ++j)
        acc[g][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(b[g][j].v, a.v, acc[g][j], 0, 0, 0);
  }
  if (split) {
    if (wave > 0) {
#pragma unroll
      for (int g = 0; g < G; ++g)
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
          for (int i = 0; i < 4; ++i) red[wave - 1][g * 4 + j][i][lane] = acc[g][j][i];
    }
    __syncthreads();
    if (wave > 0) return;
#pragma unroll
    for (int v = 0; v < 3; ++v)
#pragma unroll
      for (int g = 0; g < G; ++g)
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
          for (int i = 0; i < 4; ++i) acc[g][j][i] += red[v][g * 4 + j][i][lane];
  }
  if (ln < rows) {
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int n = n0 + 16 * j + 4 * lg + i;
        if (n >= N) continue;
        float v;
        if (GATE_UP)
          v = gated_act(act, acc[0][j][i] * f, acc[G - 1][j][i] * f, limit);
        else if (MODE == MODE_UP)
          v = unary_act(act, acc[0][j][i] * f);
        else
          v = acc[0][j][i];
        out[(size_t)(row0 + ln) * ldo + n] = float_to_bf16(v);
      }
  }
}

// Many pairs (a prompt portion): tiles through LDS. A workgroup owns 64 sorted rows x 128 rows
// of the expert's matrix (gate|up: 64 gate rows and the 64 up rows that belong to them, so that
// the activation meets in one lane; down: 128 result columns); a wave owns 32 rows x 64 of the
// 128. Chunks of 64 along K go from global memory straight into LDS (global_load_lds_dwordx4:
// every lane names its own 16 bytes, a wave's 64 pieces land side by side, no register carries
// them), two buffers, the next chunk in flight while this one is multiplied. Rows lie unpadded
// (128 bytes); the 16-byte pieces of a row are permuted by the row number (piece c of row r lies
// at c ^ ((r >> 1) & 7)), which keeps the fragment reads free of bank conflicts. Rows past the
// tile's end read some valid row (their results are never stored). Needs K % 64 == 0.
#define TB_K 64
#define TB_BROWS 128

template <int MODE>
__global__ void __launch_bounds__(256)
moe_gemm_tiled_kernel(bf16_t* __restrict__ out, long ldo, const bf16_t* __restrict__ x, long ldx,
                      const bf16_t* __restrict__ w, const int32_t* __restrict__ tile_expert,
                      const int32_t* __restrict__ tile_row0, const int32_t* __restrict__ expert_end,
                      const int32_t* __restrict__ sorted, const float* __restrict__ wgt, int top, int N, int K,
                      int act, float limit) {
  constexpr bool GATE_UP = MODE == MODE_GATE_UP;
  constexpr bool GATHER = MODE != MODE_DOWN;
  const int e = tile_expert[blockIdx.y];
  if (e < 0) return;
  __shared__ __attribute__((aligned(1024))) bf16_t As0[64 * TB_K];
  __shared__ __attribute__((aligned(1024))) bf16_t As1[64 * TB_K];
  __shared__ __attribute__((aligned(1024))) bf16_t Bs0[TB_BROWS * TB_K];
  __shared__ __attribute__((aligned(1024))) bf16_t Bs1[TB_BROWS * TB_K];
  __shared__ int32_t src_row[64];
  __shared__ float row_w[64];
  const int tid = threadIdx.x;
  const int row0 = tile_row0[blockIdx.y];
  const int rows = min(MOE_TM, expert_end[e] - row0);
  if (tid < 64) {
    const int t = min(tid, rows - 1);
    int r;
    float f = 1.f;
    if (GATHER) {
      const int a = sorted[row0 + t];
      r = a / top;
      if (wgt) f = wgt[a];
    } else {
      r = row0 + t;
    }
    src_row[tid] = r;
    row_w[tid] = f;
  }
  __syncthreads();
  const int n0 = blockIdx.x * (GATE_UP ? TB_BROWS / 2 : TB_BROWS);
  const size_t wrows = GATE_UP ? 2 * (size_t)N : (size_t)N;
  w += (size_t)e * wrows * K;
  const int wave = tid >> 6, lane = tid & 63;
  // the pieces this lane names: slot s = 64 (instruction) + lane holds row s / 8, piece (s % 8) ^ swz
  const bf16_t* a_src[2];
  const bf16_t* b_src[4];
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const int slot = 64 * (wave * 2 + i) + lane;
    const int r = slot >> 3, c = (slot & 7) ^ ((r >> 1) & 7);
    a_src[i] = x + (size_t)src_row[r] * ldx + 8 * c;
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int slot = 64 * (wave * 4 + i) + lane;
    const int r = slot >> 3, c = (slot & 7) ^ ((r >> 1) & 7);
    size_t grow;
    if (GATE_UP) {
      const int col = min(n0 + (r & 63), N - 1);
      grow = r < 64 ? (size_t)col : (size_t)N + col;
    } else {
      grow = (size_t)min(n0 + r, N - 1);
    }
    b_src[i] = w + grow * K + 8 * c;
  }
  auto fetch = [&](int k0, bf16_t* Ab, bf16_t* Bb) {
#pragma unroll
    for (int i = 0; i < 2; ++i)
      __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(a_src[i] + k0),
                                       (__attribute__((address_space(3))) void*)(Ab + 512 * (wave * 2 + i)), 16, 0, 0);
#pragma unroll
    for (int i = 0; i < 4; ++i)
      __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(b_src[i] + k0),
                                       (__attribute__((address_space(3))) void*)(Bb + 512 * (wave * 4 + i)), 16, 0, 0);
  };
  const int ln = lane & 15, lg = lane >> 4;
  const int rh = wave & 1, cg = wave >> 1;
  // where this lane reads its fragments: row * 64 elements, piece (4 ks + lg) ^ swz(row)
  int a_row[2], b_row[4];
#pragma unroll
  for (int i = 0; i < 2; ++i) a_row[i] = rh * 32 + 16 * i + ln;
#pragma unroll
  for (int j = 0; j < 4; ++j)
    b_row[j] = (GATE_UP ? (j >> 1) * 64 + cg * 32 + (j & 1) * 16 : cg * 64 + 16 * j) + ln;
  f32x4_t acc[2][4];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = f32x4_t{0.f, 0.f, 0.f, 0.f};
  auto mult = [&](const bf16_t* Ab, const bf16_t* Bb) {
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) {
      Frag8 a[2], b[4];
#pragma unroll
      for (int i = 0; i < 2; ++i)
        a[i].u = *reinterpret_cast<const uint4*>(Ab + a_row[i] * TB_K + 8 * ((4 * ks + lg) ^ ((a_row[i] >> 1) & 7)));
#pragma unroll
      for (int j = 0; j < 4; ++j)
        b[j].u = *reinterpret_cast<const uint4*>(Bb + b_row[j] * TB_K + 8 * ((4 * ks + lg) ^ ((b_row[j] >> 1) & 7)));
      __builtin_amdgcn_sched_barrier(0);       // all reads of the stage first, then its products
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(b[j].v, a[i].v, acc[i][j], 0, 0, 0);
    }
  };
  const int chunks = K / TB_K;
  fetch(0, As0, Bs0);
  __builtin_amdgcn_s_waitcnt(0x0F70);        // vmcnt(0): this wave's loads into LDS have landed
  __syncthreads();
  for (int c = 0; c < chunks; c += 2) {
    if (c + 1 < chunks) fetch((c + 1) * TB_K, As1, Bs1);
    mult(As0, Bs0);
    __builtin_amdgcn_s_waitcnt(0x0F70);
    __syncthreads();
    if (c + 1 >= chunks) break;
    if (c + 2 < chunks) fetch((c + 2) * TB_K, As0, Bs0);
    mult(As1, Bs1);
    __builtin_amdgcn_s_waitcnt(0x0F70);
    __syncthreads();
  }
  // lane holds, of tile (i, j): row m = rh * 32 + 16 i + ln, weight rows (b_row[j] - ln) + 4 lg + q
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const int m = rh * 32 + 16 * i + ln;
    if (m >= rows) continue;
    const float f = row_w[m];
    bf16_t* orow = out + (size_t)(row0 + m) * ldo;
#pragma unroll
    for (int j = 0; j < (GATE_UP ? 2 : 4); ++j)
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int n = GATE_UP ? n0 + cg * 32 + 16 * j + 4 * lg + q : n0 + cg * 64 + 16 * j + 4 * lg + q;
        if (n >= N) continue;
        const float v = GATE_UP ? gated_act(act, acc[i][j][q] * f, acc[i][GATE_UP ? j + 2 : j][q] * f, limit)
                                : (MODE == MODE_UP ? unary_act(act, acc[i][j][q] * f) : acc[i][j][q]);
        orow[n] = float_to_bf16(v);
      }
  }
}

// pairs from which on the tiles go through LDS (below: a decode step, tiles of a few rows)
#define MOE_TILED_FROM 128

static bool mfma_ok(const void* x, long ldx, const void* w, int K) {
  return K % 8 == 0 && ldx % 8 == 0 && ((uintptr_t)x | (uintptr_t)w) % 16 == 0;
}

// out [A, I] (sorted order) = act(w_a * x[token] Wg_e^T, w_a * x[token] Wu_e^T); w [E, 2 I, K];
// wgt null: the routing weight is not applied here.
extern "C" int ptl_moe_gate_up(void* out, long ldo, const void* x, long ldx, const void* w,
                               const int32_t* tile_expert, const int32_t* tile_row0,
                               const int32_t* expert_end, const int32_t* sorted, const float* wgt,
                               int max_tiles, int pairs, int top, int I, int K, int act, float limit, int dtype,
                               hipStream_t st) {
  if (max_tiles <= 0) return PTL_OK;
  if (I <= 0 || K <= 0 || top <= 0 || max_tiles > 65535) return PTL_ERR_ARG;
  dim3 grid((I + 63) / 64, max_tiles);
  if (dtype == PTL_DTYPE_F32)
    moe_gemm_kernel<float, MODE_GATE_UP><<<grid, 256, 0, st>>>((float*)out, ldo, (const float*)x, ldx, (const float*)w,
                                                       tile_expert, tile_row0, expert_end, sorted, wgt, top, I,
                                                       K, act, limit);
  else if (dtype == PTL_DTYPE_BF16 && mfma_ok(x, ldx, w, K) && pairs >= MOE_TILED_FROM && K % TB_K == 0) {
    dim3 wide((I + TB_BROWS / 2 - 1) / (TB_BROWS / 2), max_tiles);
    moe_gemm_tiled_kernel<MODE_GATE_UP><<<wide, 256, 0, st>>>((bf16_t*)out, ldo, (const bf16_t*)x, ldx,
                                                      (const bf16_t*)w, tile_expert, tile_row0, expert_end,
                                                      sorted, wgt, top, I, K, act, limit);
  }
  else if (dtype == PTL_DTYPE_BF16 && mfma_ok(x, ldx, w, K))
    moe_gemm_mfma_kernel<MODE_GATE_UP><<<grid, 256, 0, st>>>((bf16_t*)out, ldo, (const bf16_t*)x, ldx,
                                                     (const bf16_t*)w, tile_expert, tile_row0, expert_end,
                                                     sorted, wgt, top, I, K, act, limit);
  else if (dtype == PTL_DTYPE_BF16)
    moe_gemm_kernel<bf16_t, MODE_GATE_UP><<<grid, 256, 0, st>>>((bf16_t*)out, ldo, (const bf16_t*)x, ldx,
                                                        (const bf16_t*)w, tile_expert, tile_row0, expert_end,
                                                        sorted, wgt, top, I, K, act, limit);
  else
    return PTL_ERR_ARG;
  return ptl_launch_status();
}

// out [A, I] (sorted order) = act(w_a * x[token] Wu_e^T) for experts without a gate; w [E, I, K];
// wgt null: the routing weight is not applied here.
extern "C" int ptl_moe_up(void* out, long ldo, const void* x, long ldx, const void* w,
                          const int32_t* tile_expert, const int32_t* tile_row0, const int32_t* expert_end,
                          const int32_t* sorted, const float* wgt, int max_tiles, int pairs, int top, int I,
                          int K, int act, int dtype, hipStream_t st) {
  if (max_tiles <= 0) return PTL_OK;
  if (I <= 0 || K <= 0 || top <= 0 || max_tiles > 65535 || act != 2) return PTL_ERR_ARG;
  dim3 grid((I + 63) / 64, max_tiles);
  if (dtype == PTL_DTYPE_F32)
    moe_gemm_kernel<float, MODE_UP><<<grid, 256, 0, st>>>((float*)out, ldo, (const float*)x, ldx,
                                                          (const float*)w, tile_expert, tile_row0, expert_end,
                                                          sorted, wgt, top, I, K, act, 0.f);
  else if (dtype == PTL_DTYPE_BF16 && mfma_ok(x, ldx, w, K) && pairs >= MOE_TILED_FROM && K % TB_K == 0) {
    dim3 wide((I + TB_BROWS - 1) / TB_BROWS, max_tiles);
    moe_gemm_tiled_kernel<MODE_UP><<<wide, 256, 0, st>>>((bf16_t*)out, ldo, (const bf16_t*)x, ldx,
                                                         (const bf16_t*)w, tile_expert, tile_row0, expert_end,
                                                         sorted, wgt, top, I, K, act, 0.f);
  } else if (dtype == PTL_DTYPE_BF16 && mfma_ok(x, ldx, w, K))
    moe_gemm_mfma_kernel<MODE_UP><<<grid, 256, 0, st>>>((bf16_t*)out, ldo, (const bf16_t*)x, ldx,
                                                        (const bf16_t*)w, tile_expert, tile_row0, expert_end,
                                                        sorted, wgt, top, I, K, act, 0.f);
  else if (dtype == PTL_DTYPE_BF16)
    moe_gemm_kernel<bf16_t, MODE_UP><<<grid, 256, 0, st>>>((bf16_t*)out, ldo, (const bf16_t*)x, ldx,
                                                           (const bf16_t*)w, tile_expert, tile_row0,
                                                           expert_end, sorted, wgt, top, I, K, act, 0.f);
  else
    return PTL_ERR_ARG;
  return ptl_launch_status();
}

// out [A, N] (sorted order) = x [A, K] (sorted order) Wd_e^T; w [E, N, K]
extern "C" int ptl_moe_down(void* out, long ldo, const void* x, long ldx, const void* w,
                            const int32_t* tile_expert, const int32_t* tile_row0, const int32_t* expert_end,
                            int max_tiles, int pairs, int N, int K, int dtype, hipStream_t st) {
  if (max_tiles <= 0) return PTL_OK;
  if (N <= 0 || K <= 0 || max_tiles > 65535) return PTL_ERR_ARG;
  dim3 grid((N + 63) / 64, max_tiles);
  if (dtype == PTL_DTYPE_F32)
    moe_gemm_kernel<float, MODE_DOWN><<<grid, 256, 0, st>>>((float*)out, ldo, (const float*)x, ldx, (const float*)w,
                                                        tile_expert, tile_row0, expert_end, nullptr, nullptr, 1,
                                                        N, K, 0, 0.f);
  else if (dtype == PTL_DTYPE_BF16 && mfma_ok(x, ldx, w, K) && pairs >= MOE_TILED_FROM && K % TB_K == 0) {
    dim3 wide((N + TB_BROWS - 1) / TB_BROWS, max_tiles);
    moe_gemm_tiled_kernel<MODE_DOWN><<<wide, 256, 0, st>>>((bf16_t*)out, ldo, (const bf16_t*)x, ldx,
                                                       (const bf16_t*)w, tile_expert, tile_row0, expert_end,
                                                       nullptr, nullptr, 1, N, K, 0, 0.f);
  } else if (dtype == PTL_DTYPE_BF16 && mfma_ok(x, ldx, w, K))
    moe_gemm_mfma_kernel<MODE_DOWN><<<grid, 256, 0, st>>>((bf16_t*)out, ldo, (const bf16_t*)x, ldx,
                                                      (const bf16_t*)w, tile_expert, tile_row0, expert_end,
                                                      nullptr, nullptr, 1, N, K, 0, 0.f);
  else if (dtype == PTL_DTYPE_BF16)
    moe_gemm_kernel<bf16_t, MODE_DOWN><<<grid, 256, 0, st>>>((bf16_t*)out, ldo, (const bf16_t*)x, ldx,
                                                         (const bf16_t*)w, tile_expert, tile_row0, expert_end,
                                                         nullptr, nullptr, 1, N, K, 0, 0.f);
  else
    return PTL_ERR_ARG;
  return ptl_launch_status();
}

// y[t, :] = sum_k f_k * rows[pos_of[t * top + k], :] + gate[t * ldg] * shared[t, :]
//           + ident[t] * xin[t, :], float32.
// f_k = wgt[t * top + k] when wgt is given (the weight scales the expert's output), else 1. A pair
// with pos_of < 0 has no row (its expert returns its input: that is the last term).
template <typename T>
__global__ void __launch_bounds__(256)
moe_combine_kernel(float* __restrict__ y, const T* __restrict__ rows, long ldr, const int32_t* __restrict__ pos_of,
                   const float* __restrict__ wgt, int top, const T* __restrict__ shared,
                   const float* __restrict__ gate, int ldg, const T* __restrict__ xin, long ldx,
                   const float* __restrict__ ident, int N) {
  const size_t t = blockIdx.y;
  const int n = blockIdx.x * 256 + threadIdx.x;
  if (n >= N) return;
  float s = 0.f;
  for (int k = 0; k < top; ++k) {
    const int p = pos_of[t * top + k];
    if (p < 0) continue;
    const float v = to_float<T>(rows[(size_t)p * ldr + n]);
    s += wgt ? v * wgt[t * top + k] : v;
  }
  if (shared) {
    const float v = to_float<T>(shared[t * N + n]);
    s += gate ? v * gate[t * ldg] : v;
  }
  if (ident) s = fmaf(ident[t], to_float<T>(xin[t * ldx + n]), s);
  y[t * N + n] = s;
}

// bfloat16 rows with N a multiple of 8 and aligned row starts: 8 columns a thread
__global__ void __launch_bounds__(256)
moe_combine_bf16_vec_kernel(float* __restrict__ y, const bf16_t* __restrict__ rows, long ldr,
                            const int32_t* __restrict__ pos_of, const float* __restrict__ wgt, int top,
                            const bf16_t* __restrict__ shared, const float* __restrict__ gate, int ldg,
                            const bf16_t* __restrict__ xin, long ldx, const float* __restrict__ ident, int N8) {
  const size_t t = blockIdx.y;
  const int c = blockIdx.x * 256 + threadIdx.x;
  if (c >= N8) return;
  float s[8];
#pragma unroll
  for (int j = 0; j < 8; ++j) s[j] = 0.f;
  union V { uint4 u; bf16_t e[8]; };
  for (int k = 0; k < top; ++k) {
    const int p = pos_of[t * top + k];
    if (p < 0) continue;
    V v;
    v.u = load_once(rows + (size_t)p * ldr + 8 * c);
    const float f = wgt ? wgt[t * top + k] : 1.f;
#pragma unroll
    for (int j = 0; j < 8; ++j) s[j] += bf16_to_float(v.e[j]) * f;
  }
  if (shared) {
    V v;
    v.u = load_once(shared + (t * N8 + c) * 8);
    const float f = gate ? gate[t * ldg] : 1.f;
#pragma unroll
    for (int j = 0; j < 8; ++j) s[j] += bf16_to_float(v.e[j]) * f;
  }
  if (ident) {
    V v;
    v.u = *reinterpret_cast<const uint4*>(xin + t * ldx + 8 * c);
    const float f = ident[t];
#pragma unroll
    for (int j = 0; j < 8; ++j) s[j] = fmaf(f, bf16_to_float(v.e[j]), s[j]);
  }
  float4* dst = reinterpret_cast<float4*>(y + (t * N8 + c) * 8);
  dst[0] = make_float4(s[0], s[1], s[2], s[3]);
  dst[1] = make_float4(s[4], s[5], s[6], s[7]);
}

// ident [T] with xin [T, N] (row stride ldx, the rows' dtype) or both null
extern "C" int ptl_moe_combine(float* y, const void* rows, long ldr, const int32_t* pos_of, const float* wgt,
                               int top, const void* shared, const float* gate, int ldg, const void* xin,
                               long ldx, const float* ident, int T_, int N, int dtype, hipStream_t st) {
  if (T_ <= 0) return PTL_OK;
  if (N <= 0 || top <= 0 || T_ > 65535 * 64 || (ident && !xin)) return PTL_ERR_ARG;
  for (int t0 = 0; t0 < T_; t0 += 65535) {
    const int nt = T_ - t0 < 65535 ? T_ - t0 : 65535;
    dim3 grid((N + 255) / 256, nt);
    const size_t o = (size_t)t0;
    if (dtype == PTL_DTYPE_BF16 && N % 8 == 0 && ldr % 8 == 0 && (!ident || ldx % 8 == 0) &&
        ((uintptr_t)rows | (uintptr_t)shared | (uintptr_t)(ident ? xin : nullptr)) % 16 == 0 &&
        (uintptr_t)y % 16 == 0) {
      dim3 vgrid((N / 8 + 255) / 256, nt);
      moe_combine_bf16_vec_kernel<<<vgrid, 256, 0, st>>>(
          y + o * N, (const bf16_t*)rows, ldr, pos_of + o * top, wgt ? wgt + o * top : nullptr, top,
          shared ? (const bf16_t*)shared + o * N : nullptr, gate ? gate + o * ldg : nullptr, ldg,
          ident ? (const bf16_t*)xin + o * ldx : nullptr, ldx, ident ? ident + o : nullptr, N / 8);
      continue;
    }
    if (dtype == PTL_DTYPE_F32)
      moe_combine_kernel<float><<<grid, 256, 0, st>>>(
          y + o * N, (const float*)rows, ldr, pos_of + o * top, wgt ? wgt + o * top : nullptr, top,
          shared ? (const float*)shared + o * N : nullptr, gate ? gate + o * ldg : nullptr, ldg,
          ident ? (const float*)xin + o * ldx : nullptr, ldx, ident ? ident + o : nullptr, N);
    else if (dtype == PTL_DTYPE_BF16)
      moe_combine_kernel<bf16_t><<<grid, 256, 0, st>>>(
          y + o * N, (const bf16_t*)rows, ldr, pos_of + o * top, wgt ? wgt + o * top : nullptr, top,
          shared ? (const bf16_t*)shared + o * N : nullptr, gate ? gate + o * ldg : nullptr, ldg,
          ident ? (const bf16_t*)xin + o * ldx : nullptr, ldx, ident ? ident + o : nullptr, N);
    else
      return PTL_ERR_ARG;
  }
  return ptl_launch_status();
}

template <typename T>
__global__ void __launch_bounds__(256)
gated_act_kernel(T* __restrict__ out, const T* __restrict__ gu, int I, size_t total, int act, float limit) {
  size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
  const size_t step = (size_t)gridDim.x * 256;
  for (; i < total; i += step) {
    const size_t t = i / I;
    const int c = (int)(i - t * I);
    out[i] = from_float<T>(gated_act(act, to_float<T>(gu[t * 2 * I + c]), to_float<T>(gu[t * 2 * I + I + c]), limit));
  }
}

// bfloat16 rows with I a multiple of 8: 16-byte loads (marked as read once) and stores
__global__ void __launch_bounds__(256)
gated_act_bf16_vec_kernel(bf16_t* __restrict__ out, const bf16_t* __restrict__ gu, int I8, int act, float limit) {
  const int c = blockIdx.x * 256 + threadIdx.x;
  if (c >= I8) return;
  const size_t t = blockIdx.y;
  const bf16_t* row = gu + (t * 2 * I8 + c) * 8;
  union { uint4 u; bf16_t e[8]; } g, u, o;
  g.u = load_once(row);
  u.u = load_once(row + (size_t)I8 * 8);
#pragma unroll
  for (int j = 0; j < 8; ++j)
    o.e[j] = float_to_bf16(gated_act(act, bf16_to_float(g.e[j]), bf16_to_float(u.e[j]), limit));
  *reinterpret_cast<uint4*>(out + (t * I8 + c) * 8) = o.u;
}

// out [T, I] = act(gu[:, :I], gu[:, I:]) for a dense gate|up product [T, 2 I]
extern "C" int ptl_gated_act(void* out, const void* gate_up, int T_, int I, int act, float limit, int dtype,
                             hipStream_t st) {
  if (T_ <= 0) return PTL_OK;
  if (I <= 0) return PTL_ERR_ARG;
  if (dtype == PTL_DTYPE_BF16 && I % 8 == 0 && T_ <= 65535 && ((uintptr_t)out | (uintptr_t)gate_up) % 16 == 0) {
    dim3 grid((I / 8 + 255) / 256, T_);
    gated_act_bf16_vec_kernel<<<grid, 256, 0, st>>>((bf16_t*)out, (const bf16_t*)gate_up, I / 8, act, limit);
    return ptl_launch_status();
  }
  const size_t total = (size_t)T_ * I;
  size_t blocks = (total + 255) / 256;
  if (blocks > 65536) blocks = 65536;
  if (dtype == PTL_DTYPE_F32)
    gated_act_kernel<float><<<(int)blocks, 256, 0, st>>>((float*)out, (const float*)gate_up, I, total, act, limit);
  else if (dtype == PTL_DTYPE_BF16)
    gated_act_kernel<bf16_t><<<(int)blocks, 256, 0, st>>>((bf16_t*)out, (const bf16_t*)gate_up, I, total, act, limit);
  else
    return PTL_ERR_ARG;
  return ptl_launch_status();
}

template <typename T>
__global__ void __launch_bounds__(256)
unary_act_kernel(T* __restrict__ out, const T* __restrict__ in, size_t total, int act) {
  size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
  const size_t step = (size_t)gridDim.x * 256;
  for (; i < total; i += step) out[i] = from_float<T>(unary_act(act, to_float<T>(in[i])));
}

// bfloat16 with a total that is a multiple of 8: 16-byte loads (marked as read once) and stores
__global__ void __launch_bounds__(256)
unary_act_bf16_vec_kernel(bf16_t* __restrict__ out, const bf16_t* __restrict__ in, size_t total8, int act) {
  size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
  const size_t step = (size_t)gridDim.x * 256;
  for (; i < total8; i += step) {
    union { uint4 u; bf16_t e[8]; } v, o;
    v.u = load_once(in + i * 8);
#pragma unroll
    for (int j = 0; j < 8; ++j) o.e[j] = float_to_bf16(unary_act(act, bf16_to_float(v.e[j])));
    *reinterpret_cast<uint4*>(out + i * 8) = o.u;
  }
}

// out [T, I] = act(in) for a dense up product of an expert without a gate (act 2: relu(u)^2)
extern "C" int ptl_unary_act(void* out, const void* in, int T_, int I, int act, int dtype, hipStream_t st) {
  if (T_ <= 0) return PTL_OK;
  if (I <= 0 || act != 2) return PTL_ERR_ARG;
  const size_t total = (size_t)T_ * I;
  if (dtype == PTL_DTYPE_BF16 && total % 8 == 0 && ((uintptr_t)out | (uintptr_t)in) % 16 == 0) {
    size_t blocks = (total / 8 + 255) / 256;
    if (blocks > 65536) blocks = 65536;
    unary_act_bf16_vec_kernel<<<(int)blocks, 256, 0, st>>>((bf16_t*)out, (const bf16_t*)in, total / 8, act);
    return ptl_launch_status();
  }
  size_t blocks = (total + 255) / 256;
  if (blocks > 65536) blocks = 65536;
  if (dtype == PTL_DTYPE_F32)
    unary_act_kernel<float><<<(int)blocks, 256, 0, st>>>((float*)out, (const float*)in, total, act);
  else if (dtype == PTL_DTYPE_BF16)
    unary_act_kernel<bf16_t><<<(int)blocks, 256, 0, st>>>((bf16_t*)out, (const bf16_t*)in, total, act);
  else
    return PTL_ERR_ARG;
  return ptl_launch_status();
}
