// A mixture of experts for any sizes, float32 or bfloat16 storage: the router (logits and scores in
// 32-bit, the `top` largest scores chosen, ties to the lower index) and the experts row by row:
//   y[m] = sum over the chosen experts e, in the order they were chosen, of  W_down[e] act(W_up[e] (s_e h[m]))
// with the score scaling the expert's input (scale_input) or its output, and act = relu(z)^2.
// Products accumulate in 32-bit with fused multiply-adds in a fixed order; what a product reads is rounded
// to the storage type first (the scaled input, the activated rows), as a matrix-core kernel's operands are.
#include "common.h"
#include "tinyinfer_kernels.h"

TI_ERROR_API

#define MOE_MAX_EXPERTS 1024
#define MOE_MAX_TOP 64

// score kinds
#define MOE_SIGMOID 0
#define MOE_SOFTMAX 1
#define MOE_SOFTMAX_CHOSEN 2      // the largest logits are chosen; the weights are the softmax over the chosen logits alone

template <typename T> struct Piece;
template <> struct Piece<float> {
  static constexpr int N = 4;
  static __device__ __forceinline__ void load(const float* p, float* v) {
    const float4 a = *reinterpret_cast<const float4*>(p);
    v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w;
  }
};
template <> struct Piece<bf16_t> {
  static constexpr int N = 8;
  static __device__ __forceinline__ void load(const bf16_t* p, float* v) {
    const uint4 a = *reinterpret_cast<const uint4*>(p);
    const unsigned w[4] = {a.x, a.y, a.z, a.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      v[2 * i] = __uint_as_float(w[i] << 16);
      v[2 * i + 1] = __uint_as_float(w[i] & 0xffff0000u);
    }
  }
};

// the wavefront's share of a . b over n elements: a in LDS or memory as floats through `fa`, b a row of the weight
template <typename T, bool VEC, class FA>
__device__ __forceinline__ float wave_dot(FA fa, const T* __restrict__ b, int n, int lane) {
  float z = 0.f;
  if (VEC) {
    constexpr int N = Piece<T>::N;
    for (int c = lane * N; c < n; c += 64 * N) {
      float v[N];
      Piece<T>::load(b + c, v);
#pragma unroll
      for (int i = 0; i < N; ++i) z = fmaf(fa(c + i), v[i], z);
    }
  } else {
    for (int c = lane; c < n; c += 64) z = fmaf(fa(c), ld<T>(b + c), z);
  }
  return group_sum<64>(z);
}

// ------------------------------------------------------------ router
// A workgroup per token.  Logits: wavefront w takes experts w, w + 4, ...; lanes share the token's row in pieces of
// 16 bytes (lane l the pieces l, l + 64, ... in ascending order, then a butterfly).  Choice: the first wavefront
// holds the scores (lane l the experts l, l + 64, ...) and takes the largest `top` times.
template <typename T, bool VEC>
__global__ void __launch_bounds__(256)
moe_route_kernel(const T* __restrict__ h, const float* __restrict__ router, int* __restrict__ ids, float* __restrict__ wts,
                 int W, int E, int top, int score_kind, int renormalize, const float* __restrict__ correction = nullptr,
                 int n_groups = 0, int keep = 0, float weight_scale = 1.f, float sum_floor = 0.f) {
  __shared__ float s_score[MOE_MAX_EXPERTS];
  __shared__ float s_plain[MOE_MAX_EXPERTS];      // the scores the weights are taken from, where the choice reads corrected ones
  __shared__ float s_group[MOE_MAX_EXPERTS];
  __shared__ float red[4];
  const bool corrected = correction != nullptr || n_groups > 1;
  const int m = blockIdx.x;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const T* row = h + (size_t)m * W;
  for (int e = wave; e < E; e += 4) {
    const float z = wave_dot<T, VEC>([&](int c) { return router[(size_t)e * W + c]; }, row, W, lane);
    if (lane == 0) s_score[e] = z;
  }
  __syncthreads();
  if (score_kind == MOE_SOFTMAX) {
    float mx = -INFINITY;
    for (int e = threadIdx.x; e < E; e += 256) mx = fmaxf(mx, s_score[e]);
    mx = block_max<256>(mx, red);
    float sum = 0.f;
    for (int e = threadIdx.x; e < E; e += 256) sum += expf(s_score[e] - mx);
    sum = block_sum<256>(sum, red);
    for (int e = threadIdx.x; e < E; e += 256) s_score[e] = expf(s_score[e] - mx) / sum;
  } else if (score_kind == MOE_SIGMOID) {
    for (int e = threadIdx.x; e < E; e += 256) s_score[e] = 1.0f / (1.0f + expf(-s_score[e]));
  }
  __syncthreads();
  if (corrected) {
    // the choice reads score + correction; the weights keep the score itself
    for (int e = threadIdx.x; e < E; e += 256) {
      s_plain[e] = s_score[e];
      if (correction) s_score[e] += correction[e];
    }
    __syncthreads();
    if (n_groups > 1) {
      // groups of E / n_groups neighbours: a group's score is the sum of its two largest choice scores; experts outside
      // the `keep` best groups (ties to the lower group) cannot be chosen
      const int per = E / n_groups;
      for (int g = threadIdx.x; g < n_groups; g += 256) {
        float a = -INFINITY, b = -INFINITY;
        for (int e = g * per; e < (g + 1) * per; ++e) {
          const float s = s_score[e];
          if (s > a) {
            b = a;
            a = s;
          } else if (s > b) {
            b = s;
          }
        }
        s_group[g] = per > 1 ? a + b : a;
      }
      __syncthreads();
      for (int g = threadIdx.x; g < n_groups; g += 256) {
        int better = 0;
        for (int o = 0; o < n_groups; ++o) better += (s_group[o] > s_group[g] || (s_group[o] == s_group[g] && o < g)) ? 1 : 0;
        if (better >= keep)
          for (int e = g * per; e < (g + 1) * per; ++e) s_score[e] = -INFINITY;
      }
      __syncthreads();
    }
  }
  if (wave != 0) return;
  float total = 0.f, first = 0.f;
  for (int k = 0; k < top; ++k) {
    float best = -INFINITY;
    int at = 0x7fffffff;
    for (int e = lane; e < E; e += 64) {
      const float s = s_score[e];
      if (s > best) {      // ascending e: the first of equals stays
        best = s;
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
    if (corrected) best = s_plain[at];
    if (lane == 0) {
      ids[(size_t)m * top + k] = at;
      wts[(size_t)m * top + k] = best;
      s_score[at] = -INFINITY;
    }
    if (score_kind == MOE_SOFTMAX_CHOSEN) {
      // the first choice is the largest logit: every weight is exp(z - z_first) over the sum of those, in the order of choice
      if (k == 0) first = best;
      const float w = expf(best - first);
      if (lane == 0) wts[(size_t)m * top + k] = w;
      total += w;
    } else {
      total += best;
    }
    __builtin_amdgcn_wave_barrier();
    __threadfence_block();
  }
  if ((renormalize || score_kind == MOE_SOFTMAX_CHOSEN) && lane < top) wts[(size_t)m * top + lane] /= total + sum_floor;
  if (weight_scale != 1.f && lane < top) wts[(size_t)m * top + lane] *= weight_scale;
}

extern "C" int ti_moe_route(int dtype, const void* h, const float* router, int* ids, float* wts, int M, int W, int E, int top,
                            int score_kind, int renormalize, hipStream_t stream) {
  return ti_moe_route_grouped(dtype, h, router, nullptr, ids, wts, M, W, E, top, score_kind, renormalize, 0, 0, 1.f, 0.f, stream);
}

// the same with what a grouped router adds: `correction` f32 [E] (null: none) joins the scores for the choice only; the experts
// form n_groups groups of neighbours of which the `keep` best may be chosen from (n_groups <= 1: no groups); the weights are
// the chosen experts' uncorrected scores, divided by their sum + sum_floor where `renormalize`, times weight_scale
extern "C" int ti_moe_route_grouped(int dtype, const void* h, const float* router, const float* correction, int* ids, float* wts,
                                    int M, int W, int E, int top, int score_kind, int renormalize, int n_groups, int keep,
                                    float weight_scale, float sum_floor, hipStream_t stream) {
  TI_REQUIRE(n_groups <= 1 || (E % n_groups == 0 && keep >= 1 && keep <= n_groups && (long)keep * (E / n_groups) >= top),
             "moe_route: %d groups of which %d are kept do not fit %d experts and top %d", n_groups, keep, E, top);
  TI_REQUIRE((!correction && n_groups <= 1) || score_kind != MOE_SOFTMAX_CHOSEN, "moe_route: a correction or groups do not go with weights from the chosen logits");
  TI_REQUIRE(M >= 0 && W > 0 && E > 0 && E <= MOE_MAX_EXPERTS && top > 0 && top <= E && top <= MOE_MAX_TOP,
             "moe_route: bad sizes M=%d W=%d experts=%d top=%d (up to %d experts, top up to %d)", M, W, E, top, MOE_MAX_EXPERTS,
             MOE_MAX_TOP);
  TI_REQUIRE(score_kind == MOE_SIGMOID || score_kind == MOE_SOFTMAX || score_kind == MOE_SOFTMAX_CHOSEN, "moe_route: unknown score kind %d", score_kind);
  if (M == 0) return 0;
  const int piece = dtype == TI_F32 ? 4 : 8;
  const bool vec = W % piece == 0 && ((uintptr_t)h & 15) == 0;
#define MOE_ROUTE(T, V) moe_route_kernel<T, V><<<M, 256, 0, stream>>>((const T*)h, router, ids, wts, W, E, top, score_kind, renormalize, correction, n_groups, keep, weight_scale, sum_floor)
  if (dtype == TI_F32) {
    if (vec) MOE_ROUTE(float, true);
    else MOE_ROUTE(float, false);
  } else if (dtype == TI_BF16) {
    if (vec) MOE_ROUTE(bf16_t, true);
    else MOE_ROUTE(bf16_t, false);
  } else {
    TI_REQUIRE(false, "moe_route: unknown dtype %d", dtype);
  }
#undef MOE_ROUTE
  TI_LAUNCH_CHECK();
  return 0;
}

// ------------------------------------------------------------ the experts, an output a wavefront
// up [E][F][W], down [E][W][F] in T.  Two kernels, both with a workgroup per (expert, 16 outputs): the workgroup finds the
// pairs (token, choice) of its expert, NP at a time, keeps their input rows in LDS and walks its rows of the weight once for
// all of them: an expert's weights are read once a step however many tokens chose it.
//   act[pair][f] = relu(up[e][f] . (s h[token]))^2 rounded to T;   part[pair][c] = down[e][c] . act[pair]
// and a token's rows of `part` are added in the order its experts were chosen by whoever reads them (moe_sum_pairs, or the
// norm that follows).  A wavefront owns four outputs; its lanes share a row of the weight in pieces of 16 bytes (lane l the
// pieces l, l + 64, ... in ascending order, then a butterfly): the order of every sum is fixed, whatever else the step holds.
#define MOE_ROWS 4      // outputs a wavefront

// the next pairs of expert e from pair `next` on, at most NP: their indices to s_pairs, (count, where to go on) to s_found.
// Called by the first wavefront.
template <int NP>
__device__ __forceinline__ void next_pairs(const int* __restrict__ ids, int n_pairs, int e, int next, int* s_pairs, int* s_found) {
  const int lane = threadIdx.x & 63;
  int n = 0, i = next;
  while (i < n_pairs && n < NP) {
    const bool hit = i + lane < n_pairs && ids[i + lane] == e;
    unsigned long long mask = __ballot(hit);
    int consumed = 64;
    while (mask) {
      const int b = __ffsll((long long)mask) - 1;
      if (n == NP) {       // this one waits for the next round
        consumed = b;
        break;
      }
      if (lane == 0) s_pairs[n] = i + b;
      ++n;
      mask &= mask - 1;
    }
    i += consumed;
  }
  if (lane == 0) {
    s_found[0] = n;
    s_found[1] = i;
  }
}

// z[r][p] = rows[p] . b[r] for the NP rows in LDS (T) and MOE_ROWS rows of the weight in memory, K apart (rows of the weight
// beyond the last one are read as the last one): the loads of all the weight's rows are in flight together.  Every sum runs
// over a lane's pieces in ascending order, then a butterfly.
template <typename T, bool VEC, int NP>
__device__ __forceinline__ void wave_dots(const T* rows, int n_live, const T* __restrict__ b, int n_rows_w, int K, int lane,
                                          float (*z)[NP]) {
#pragma unroll
  for (int r = 0; r < MOE_ROWS; ++r)
#pragma unroll
    for (int p = 0; p < NP; ++p) z[r][p] = 0.f;
  const T* br[MOE_ROWS];
#pragma unroll
  for (int r = 0; r < MOE_ROWS; ++r) br[r] = b + (size_t)(r < n_rows_w ? r : n_rows_w - 1) * K;
  if (VEC) {
    constexpr int N = Piece<T>::N;
    for (int c = lane * N; c < K; c += 64 * N) {
      float v[MOE_ROWS][N];
#pragma unroll
      for (int r = 0; r < MOE_ROWS; ++r) Piece<T>::load(br[r] + c, v[r]);
#pragma unroll
      for (int p = 0; p < NP; ++p)
        if (p < n_live) {
          float a[N];
          Piece<T>::load(rows + (size_t)p * K + c, a);
#pragma unroll
          for (int r = 0; r < MOE_ROWS; ++r)
#pragma unroll
            for (int i = 0; i < N; ++i) z[r][p] = fmaf(a[i], v[r][i], z[r][p]);
        }
    }
  } else {
    for (int c = lane; c < K; c += 64) {
      float v[MOE_ROWS];
#pragma unroll
      for (int r = 0; r < MOE_ROWS; ++r) v[r] = ld<T>(br[r] + c);
#pragma unroll
      for (int p = 0; p < NP; ++p)
        if (p < n_live) {
          const float a = ld<T>(rows + (size_t)p * K + c);
#pragma unroll
          for (int r = 0; r < MOE_ROWS; ++r) z[r][p] = fmaf(a, v[r], z[r][p]);
        }
    }
  }
#pragma unroll
  for (int r = 0; r < MOE_ROWS; ++r)
#pragma unroll
    for (int p = 0; p < NP; ++p) z[r][p] = group_sum<64>(z[r][p]);
}

// DOWN false: rows are the tokens' inputs h (scaled by the score where it scales the input), K = W, outputs F, relu^2 to act.
// DOWN true: rows are act, K = F, outputs W, 32-bit to part (times the score where it scales the output).
// plain (DOWN false): the sums are stored as they are, in 32-bit (a gated activation over [gate | up] follows in a kernel of its own).
template <typename T, bool VEC, int NP, bool DOWN>
__global__ void __launch_bounds__(256)
moe_expert_rows_kernel(const T* __restrict__ in, const int* __restrict__ ids, const float* __restrict__ wts, const T* __restrict__ w,
                       void* __restrict__ out, int n_pairs, int K, int N, int top, int scale_input, int plain) {
  extern __shared__ __attribute__((aligned(16))) unsigned char raw[];
  T* rows = reinterpret_cast<T*>(raw);      // [NP][K]
  __shared__ int s_pairs[NP], s_found[2];
  const int e = blockIdx.x;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int n0 = (blockIdx.y * 4 + wave) * MOE_ROWS;
  const T* we = w + (size_t)e * N * K;
  int next = 0;
  while (next < n_pairs) {
    if (wave == 0) next_pairs<NP>(ids, n_pairs, e, next, s_pairs, s_found);
    __syncthreads();
    const int n_live = s_found[0];
    next = s_found[1];
    if (n_live == 0) break;
    for (int p = 0; p < n_live; ++p) {
      const int pair = s_pairs[p];
      const T* src = DOWN ? in + (size_t)pair * K : in + (size_t)(pair / top) * K;
      const float s = (!DOWN && scale_input) ? wts[pair] : 1.f;
      for (int c = threadIdx.x; c < K; c += 256) st<T>(rows + (size_t)p * K + c, DOWN ? ld<T>(src + c) : ld<T>(src + c) * s);
    }
    __syncthreads();
    if (n0 < N) {
      float z[MOE_ROWS][NP];
      const int n_rows_w = min(MOE_ROWS, N - n0);
      wave_dots<T, VEC, NP>(rows, n_live, we + (size_t)n0 * K, n_rows_w, K, lane, z);
      if (lane == 0) {
#pragma unroll
        for (int r = 0; r < MOE_ROWS; ++r)
#pragma unroll
          for (int p = 0; p < NP; ++p)
            if (r < n_rows_w && p < n_live) {
              const int pair = s_pairs[p], n = n0 + r;
              if (DOWN) {
                ((float*)out)[(size_t)pair * N + n] = scale_input ? z[r][p] : z[r][p] * wts[pair];
              } else if (plain) {      // the sums themselves, 32-bit: an activation over several of them follows
                ((float*)out)[(size_t)pair * N + n] = z[r][p];
              } else {
                const float a = fmaxf(z[r][p], 0.f);
                st<T>((T*)out + (size_t)pair * N + n, a * a);
              }
            }
      }
    }
    __syncthreads();      // the rows and the list are read to the end before the next round writes them
  }
}

// y[m] = sum_k part[m top + k], k ascending
__global__ void moe_sum_pairs_kernel(const float* __restrict__ part, float* __restrict__ y, int W, int top) {
  const int m = blockIdx.x;
  for (int c = threadIdx.x; c < W; c += blockDim.x) {
    float v = part[(size_t)m * top * W + c];
    for (int k = 1; k < top; ++k) v += part[((size_t)m * top + k) * W + c];
    y[(size_t)m * W + c] = v;
  }
}

template <typename T, bool VEC, int NP, bool DOWN>
static void launch_expert_rows(const void* in, const int* ids, const float* wts, const void* w, void* out, int n_pairs, int K, int N,
                               int top, int scale_input, int E, hipStream_t stream, int plain) {
  const dim3 grid(E, (N + 4 * MOE_ROWS - 1) / (4 * MOE_ROWS));
  moe_expert_rows_kernel<T, VEC, NP, DOWN><<<grid, 256, (size_t)NP * K * sizeof(T), stream>>>((const T*)in, ids, wts, (const T*)w, out,
                                                                                               n_pairs, K, N, top, scale_input, plain);
}
template <typename T, bool VEC, bool DOWN>
static int expert_rows(const void* in, const int* ids, const float* wts, const void* w, void* out, int n_pairs, int K, int N, int top,
                       int scale_input, int E, hipStream_t stream, int plain = 0) {
  const size_t row = (size_t)K * sizeof(T), room = 48 * 1024;      // rows of the pairs a round holds in LDS
  if (4 * row <= room) launch_expert_rows<T, VEC, 4, DOWN>(in, ids, wts, w, out, n_pairs, K, N, top, scale_input, E, stream, plain);
  else if (2 * row <= room) launch_expert_rows<T, VEC, 2, DOWN>(in, ids, wts, w, out, n_pairs, K, N, top, scale_input, E, stream, plain);
  else if (row <= 64 * 1024) launch_expert_rows<T, VEC, 1, DOWN>(in, ids, wts, w, out, n_pairs, K, N, top, scale_input, E, stream, plain);
  else return 1;
  return 0;
}

// act: scratch in the dtype of h, [M top][F]; part: f32 [M top][W], a token's rows to be added in ascending order: into y where
// y is given, else by the caller
extern "C" int ti_moe_experts_rows(int dtype, const void* h, const int* ids, const float* wts, const void* up, const void* down,
                                   void* act, float* part, float* y, int M, int W, int F, int E, int top, int scale_input,
                                   hipStream_t stream) {
  TI_REQUIRE(M >= 0 && W > 0 && F > 0 && top > 0 && E > 0, "moe_experts: bad sizes M=%d W=%d F=%d top=%d", M, W, F, top);
  if (M == 0) return 0;
  TI_REQUIRE((F + 4 * MOE_ROWS - 1) / (4 * MOE_ROWS) <= 65535 && (W + 4 * MOE_ROWS - 1) / (4 * MOE_ROWS) <= 65535,
             "moe_experts: sizes W=%d F=%d are too large", W, F);
  const int es = dtype == TI_F32 ? 4 : 2;
  const int piece = 16 / es;
  const bool vec = W % piece == 0 && F % piece == 0 && (((uintptr_t)up | (uintptr_t)down | (uintptr_t)act | (uintptr_t)h) & 15) == 0;
  const int n_pairs = M * top;
  int rc;
#define MOE_BOTH(T, V)                                                                                              \
  do {                                                                                                              \
    rc = expert_rows<T, V, false>(h, ids, wts, up, act, n_pairs, W, F, top, scale_input, E, stream);                \
    if (rc == 0) rc = expert_rows<T, V, true>(act, ids, wts, down, part, n_pairs, F, W, top, scale_input, E, stream); \
  } while (0)
  if (dtype == TI_F32) {
    if (vec) MOE_BOTH(float, true);
    else MOE_BOTH(float, false);
  } else if (dtype == TI_BF16) {
    if (vec) MOE_BOTH(bf16_t, true);
    else MOE_BOTH(bf16_t, false);
  } else {
    TI_REQUIRE(false, "moe_experts: unknown dtype %d", dtype);
  }
#undef MOE_BOTH
  TI_REQUIRE(rc == 0, "moe_experts: a row of %d or %d entries does not fit the workgroup's 64 KB", W, F);
  if (y) moe_sum_pairs_kernel<<<M, 256, 0, stream>>>(part, y, W, top);
  TI_LAUNCH_CHECK();
  return 0;
}

// ------------------------------------------------------------ gated experts
// y[m] = sum_k s_k W_down[e_k] act(W_gate[e_k] h, W_up[e_k] h): gate_up [E][2F][W] holds an expert's gate rows above its up rows.
//   act_kind 1: g = min(g, limit), u = clamp(u, -limit, limit); g * sigmoid(alpha g) * (u + 1)        0: silu(g) * u
// z: f32 scratch [M top][2F] (the two products' sums), act: scratch of the dtype of h [M top][F], part: f32 [M top][W].
template <typename T>
__global__ void moe_gate_kernel(const float* __restrict__ z, T* __restrict__ act, long n_pairs, int F, int kind, float limit, float alpha) {
  const long n = n_pairs * F;
  for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (long)gridDim.x * blockDim.x) {
    const long pair = i / F;
    const int f = (int)(i % F);
    float g = z[pair * 2 * F + f], u = z[pair * 2 * F + F + f];
    float y;
    if (kind == 0) {
      y = g / (1.0f + expf(-g)) * u;
    } else {
      g = fminf(g, limit);
      u = fminf(fmaxf(u, -limit), limit);
      y = g / (1.0f + expf(-alpha * g)) * (u + 1.0f);
    }
    st<T>(act + i, y);
  }
}

extern "C" int ti_moe_experts_rows_gated(int dtype, const void* h, const int* ids, const float* wts, const void* gate_up, const void* down,
                                         float* z, void* act, float* part, float* y, int M, int W, int F, int E, int top, int act_kind,
                                         float limit, float alpha, hipStream_t stream) {
  TI_REQUIRE(M >= 0 && W > 0 && F > 0 && top > 0 && E > 0, "moe_experts: bad sizes M=%d W=%d F=%d top=%d", M, W, F, top);
  TI_REQUIRE(act_kind == 0 || act_kind == 1, "moe_experts: unknown gated activation %d", act_kind);
  if (M == 0) return 0;
  TI_REQUIRE((2 * F + 4 * MOE_ROWS - 1) / (4 * MOE_ROWS) <= 65535 && (W + 4 * MOE_ROWS - 1) / (4 * MOE_ROWS) <= 65535,
             "moe_experts: sizes W=%d F=%d are too large", W, F);
  const int es = dtype == TI_F32 ? 4 : 2;
  const int piece = 16 / es;
  const bool vec = W % piece == 0 && F % piece == 0 && (((uintptr_t)gate_up | (uintptr_t)down | (uintptr_t)act | (uintptr_t)h) & 15) == 0;
  const int n_pairs = M * top;
  const long n_act = (long)n_pairs * F;
  const unsigned blocks = (unsigned)((n_act + 255) / 256 < 16384 ? (n_act + 255) / 256 : 16384);
  int rc;
#define MOE_GATED(T, V)                                                                                                 \
  do {                                                                                                                  \
    rc = expert_rows<T, V, false>(h, ids, wts, gate_up, z, n_pairs, W, 2 * F, top, 0, E, stream, 1);                    \
    if (rc == 0) {                                                                                                      \
      moe_gate_kernel<T><<<blocks, 256, 0, stream>>>(z, (T*)act, n_pairs, F, act_kind, limit, alpha);                   \
      rc = expert_rows<T, V, true>(act, ids, wts, down, part, n_pairs, F, W, top, 0, E, stream);                        \
    }                                                                                                                   \
  } while (0)
  if (dtype == TI_F32) {
    if (vec) MOE_GATED(float, true);
    else MOE_GATED(float, false);
  } else if (dtype == TI_BF16) {
    if (vec) MOE_GATED(bf16_t, true);
    else MOE_GATED(bf16_t, false);
  } else {
    TI_REQUIRE(false, "moe_experts: unknown dtype %d", dtype);
  }
#undef MOE_GATED
  TI_REQUIRE(rc == 0, "moe_experts: a row of %d or %d entries does not fit the workgroup's 64 KB", W, F);
  if (y) moe_sum_pairs_kernel<<<M, 256, 0, stream>>>(part, y, W, top);
  TI_LAUNCH_CHECK();
  return 0;
}
