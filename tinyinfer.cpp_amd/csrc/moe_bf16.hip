// The experts of a mixture of experts for steps of many tokens, bfloat16 on the matrix cores of gfx950.
//
//   1. moe_group: counts the (token, expert) pairs of every expert, lays the experts' runs of rows one after
//      the other and cuts them into tiles of 128 rows: offsets, the list of tiles, cursors at zero.
//   2. moe_place: every pair takes a free row of its expert's run (which row does not matter: a row of a
//      product depends on no other row) and writes its scaled input there, rounded to bfloat16.
//   3. two grouped products over the tiles: act = relu(A up_e^T)^2 (bfloat16), out = act down_e^T (32-bit).
//      Weights are the A operand of v_mfma_f32_16x16x32_bf16 and tokens the 16 columns, both in their own
//      layouts through LDS; a lane ends with four consecutive outputs of one token.
//   4. a token's rows are added in the order its experts were chosen: by the norm that reads them next
//      (it is handed the list `where`), or by moe_combine.
#include "common.h"
#include "tinyinfer_kernels.h"

TI_ERROR_API

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float floatx4;
union Frag8 {
  uint4 u;
  bf16x8 v;
};

#define MOE_TILE 128         // rows (pairs) of a tile
#define MOE_MAX_E 1024

// meta int32: [0] number of tiles, [1 .. E + 1] offsets of the experts' runs, then E cursors, then tiles [max][3] =
// (expert, first row, rows).  One workgroup.
__global__ void __launch_bounds__(1024)
moe_group_kernel(const int* __restrict__ ids, int n_pairs, int E, int* __restrict__ meta) {
  __shared__ int count[MOE_MAX_E];
  __shared__ int first_tile[MOE_MAX_E + 1];
  for (int e = threadIdx.x; e < E; e += 1024) count[e] = 0;
  __syncthreads();
  for (int i = threadIdx.x; i < n_pairs; i += 1024) atomicAdd(&count[ids[i]], 1);
  __syncthreads();
  int* offsets = meta + 1;
  int* cursors = meta + 1 + E + 1;
  int* tiles = cursors + E;
  if (threadIdx.x == 0) {
    int at = 0, t = 0;
    for (int e = 0; e < E; ++e) {
      offsets[e] = at;
      first_tile[e] = t;
      at += count[e];
      t += (count[e] + MOE_TILE - 1) / MOE_TILE;
    }
    offsets[E] = at;
    first_tile[E] = t;
    meta[0] = t;
  }
  __syncthreads();
  for (int e = threadIdx.x; e < E; e += 1024) {
    cursors[e] = 0;
    const int n = count[e], t0 = first_tile[e];
    for (int k = 0; k * MOE_TILE < n; ++k) {
      tiles[3 * (t0 + k)] = e;
      tiles[3 * (t0 + k) + 1] = offsets[e] + k * MOE_TILE;
      tiles[3 * (t0 + k) + 2] = min(MOE_TILE, n - k * MOE_TILE);
    }
  }
}

// A workgroup per 64 pairs: where[pair] = its row; rows[row] = bf16(s h[token]).  The workgroup counts its pairs per expert in
// LDS and takes a run of rows from every expert's cursor at once (one atomic per expert it met, not one per pair); inside the
// run a pair's place is its count in LDS.
__global__ void __launch_bounds__(256)
moe_place_kernel(const bf16_t* __restrict__ h, const int* __restrict__ ids, const float* __restrict__ wts, int* __restrict__ meta,
                 int E, int top, int W, int n_pairs, int* __restrict__ where, bf16_t* __restrict__ rows) {
  __shared__ int count[MOE_MAX_E];      // pairs of this workgroup per expert, then the first row of their run
  __shared__ int s_row[64];
  const int pair0 = blockIdx.x * 64;
  for (int e = threadIdx.x; e < E; e += 256) count[e] = 0;
  __syncthreads();
  int e_mine = -1, local = 0;
  if (threadIdx.x < 64 && pair0 + threadIdx.x < n_pairs) {
    e_mine = ids[pair0 + threadIdx.x];
    local = atomicAdd(&count[e_mine], 1);
  }
  __syncthreads();
  for (int e = threadIdx.x; e < E; e += 256)
    if (count[e] > 0) count[e] = meta[1 + e] + atomicAdd(&meta[1 + E + 1 + e], count[e]);
  __syncthreads();
  if (e_mine >= 0) {
    const int r = count[e_mine] + local;
    where[pair0 + threadIdx.x] = r;
    s_row[threadIdx.x] = r;
  }
  __syncthreads();
  // a wavefront copies 16 of the rows, a lane 16 bytes at a time (W is a multiple of 32)
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  for (int i = 0; i < 16; ++i) {
    const int pair = pair0 + wave * 16 + i;
    if (pair >= n_pairs) break;
    const float s = wts ? wts[pair] : 1.f;      // no weights: the rows as they are (the weights come in at the end)
    const bf16_t* src = h + (size_t)(pair / top) * W;
    bf16_t* dst = rows + (size_t)s_row[wave * 16 + i] * W;
    for (int c = lane * 8; c < W; c += 64 * 8) {
      const uint4 a = *reinterpret_cast<const uint4*>(src + c);
      const unsigned w[4] = {a.x, a.y, a.z, a.w};
      unsigned o[4];
#pragma unroll
      for (int k = 0; k < 4; ++k) o[k] = pack_bf16x2(__uint_as_float(w[k] << 16) * s, __uint_as_float(w[k] & 0xffff0000u) * s);
      *reinterpret_cast<uint4*>(dst + c) = make_uint4(o[0], o[1], o[2], o[3]);
    }
  }
}

// out[row][n] (op)= sum_k rows[row][k] w[e][n][k] over the tiles.  A workgroup: one tile of 128 rows x 128 outputs, its four
// wavefronts two by two, each 64 outputs (four blocks of 16) against 64 rows (four blocks of 16).  A step of 32 along k of both
// operands is fetched once by the workgroup (thread t the 16-byte pieces t, t + 256) into one of two LDS stages while the step
// before it is multiplied from the other; one barrier a step.  Rows of a stage are 80 bytes apart, so that the fragments'
// reads spread over the banks.  EPI 0: relu^2, bfloat16; 1: 32-bit.
#define MOE_LDS_ROW 40       // bfloat16 elements between rows of a stage (32 + 8)
template <int EPI>
__global__ void __launch_bounds__(256)
moe_grouped_kernel(const bf16_t* __restrict__ rows, const bf16_t* __restrict__ w, const int* __restrict__ meta, int E, void* __restrict__ out,
                   int N, int K) {
  __shared__ __attribute__((aligned(16))) bf16_t lds[2][2][128 * MOE_LDS_ROW];      // [stage][weights | rows]
  const int n_tiles = meta[0];
  if ((int)blockIdx.x >= n_tiles) return;
  const int* tile = meta + 1 + E + 1 + E + 3 * blockIdx.x;
  const int e = tile[0], row0 = tile[1], n_rows = tile[2];
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int r16 = lane & 15, quad = lane >> 4;
  const int wy = wave >> 1, wx = wave & 1;
  const int n_blk = blockIdx.y * 128;
  // what this thread fetches: rows u / 4 of both operands, 16 bytes from element 8 (u % 4) on
  const int u0 = threadIdx.x, u1 = threadIdx.x + 256;
  const bf16_t* const src_w0 = w + ((size_t)e * N + min(n_blk + (u0 >> 2), N - 1)) * K + (u0 & 3) * 8;
  const bf16_t* const src_w1 = w + ((size_t)e * N + min(n_blk + (u1 >> 2), N - 1)) * K + (u1 & 3) * 8;
  const bf16_t* const src_r0 = rows + (size_t)(row0 + min(u0 >> 2, n_rows - 1)) * K + (u0 & 3) * 8;
  const bf16_t* const src_r1 = rows + (size_t)(row0 + min(u1 >> 2, n_rows - 1)) * K + (u1 & 3) * 8;
  const int park0 = (u0 >> 2) * MOE_LDS_ROW + (u0 & 3) * 8, park1 = (u1 >> 2) * MOE_LDS_ROW + (u1 & 3) * 8;
  floatx4 acc[4][4];
#pragma unroll
  for (int a = 0; a < 4; ++a)
#pragma unroll
    for (int b = 0; b < 4; ++b) acc[a][b] = floatx4{0.f, 0.f, 0.f, 0.f};
  uint4 w0 = *reinterpret_cast<const uint4*>(src_w0), w1 = *reinterpret_cast<const uint4*>(src_w1);
  uint4 t0 = *reinterpret_cast<const uint4*>(src_r0), t1 = *reinterpret_cast<const uint4*>(src_r1);
  *reinterpret_cast<uint4*>(&lds[0][0][park0]) = w0;
  *reinterpret_cast<uint4*>(&lds[0][0][park1]) = w1;
  *reinterpret_cast<uint4*>(&lds[0][1][park0]) = t0;
  *reinterpret_cast<uint4*>(&lds[0][1][park1]) = t1;
  __syncthreads();
  int cur = 0;
  for (int k = 0; k < K; k += 32, cur ^= 1) {       // K is a multiple of 32
    const bool more = k + 32 < K;
    if (more) {
      w0 = *reinterpret_cast<const uint4*>(src_w0 + k + 32);
      w1 = *reinterpret_cast<const uint4*>(src_w1 + k + 32);
      t0 = *reinterpret_cast<const uint4*>(src_r0 + k + 32);
      t1 = *reinterpret_cast<const uint4*>(src_r1 + k + 32);
    }
    Frag8 fa[4], fb[4];
#pragma unroll
    for (int a = 0; a < 4; ++a) fa[a].u = *reinterpret_cast<const uint4*>(&lds[cur][0][(64 * wy + 16 * a + r16) * MOE_LDS_ROW + quad * 8]);
#pragma unroll
    for (int b = 0; b < 4; ++b) fb[b].u = *reinterpret_cast<const uint4*>(&lds[cur][1][(64 * wx + 16 * b + r16) * MOE_LDS_ROW + quad * 8]);
#pragma unroll
    for (int a = 0; a < 4; ++a)
#pragma unroll
      for (int b = 0; b < 4; ++b) acc[a][b] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(fa[a].v, fb[b].v, acc[a][b], 0, 0, 0);
    if (more) {
      *reinterpret_cast<uint4*>(&lds[cur ^ 1][0][park0]) = w0;
      *reinterpret_cast<uint4*>(&lds[cur ^ 1][0][park1]) = w1;
      *reinterpret_cast<uint4*>(&lds[cur ^ 1][1][park0]) = t0;
      *reinterpret_cast<uint4*>(&lds[cur ^ 1][1][park1]) = t1;
    }
    __syncthreads();
  }
  // lane: outputs n0 + 16 a + 4 quad + i of row 64 wx + 16 b + r16
  const int n0 = n_blk + 64 * wy;
#pragma unroll
  for (int b = 0; b < 4; ++b) {
    const int r = 64 * wx + 16 * b + r16;
    if (r >= n_rows) continue;
#pragma unroll
    for (int a = 0; a < 4; ++a) {
      const int n = n0 + 16 * a + 4 * quad;
      if (n >= N) continue;                 // N is a multiple of 4
      const floatx4 v = acc[a][b];
      if (EPI == 0) {
        float z[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          z[i] = fmaxf(v[i], 0.f);
          z[i] *= z[i];
        }
        *reinterpret_cast<uint2*>((bf16_t*)out + (size_t)(row0 + r) * N + n) = make_uint2(pack_bf16x2(z[0], z[1]), pack_bf16x2(z[2], z[3]));
      } else {
        *reinterpret_cast<float4*>((float*)out + (size_t)(row0 + r) * N + n) = make_float4(v[0], v[1], v[2], v[3]);
      }
    }
  }
}

// y[m] = sum_k out[where[m top + k]], k ascending
__global__ void moe_combine_kernel(const float* __restrict__ out, const int* __restrict__ where, float* __restrict__ y, int W, int top) {
  const int m = blockIdx.x;
  for (int c = threadIdx.x; c < W; c += blockDim.x) {
    float v = 0.f;
    for (int k = 0; k < top; ++k) v += out[(size_t)where[m * top + k] * W + c];
    y[(size_t)m * W + c] = v;
  }
}

extern "C" long ti_moe_grouped_meta_ints(int n_pairs, int E) { return 1 + (E + 1) + E + 3L * ((n_pairs + MOE_TILE - 1) / MOE_TILE + E); }

// h bf16 [M, W]; ids, wts [M top]; up [E][F][W], down [E][W][F] bf16.  Scratch: meta int32 [ti_moe_grouped_meta_ints],
// where int32 [M top], rows bf16 [M top][W], act bf16 [M top][F], out f32 [M top][W].  y (may be null): the tokens' sums;
// without it the caller adds the rows out[where[m top + k]] itself.  3: sizes not served (W, F multiples of 32, E <= 1024).
extern "C" int ti_moe_experts_grouped_bf16(const void* h, const int* ids, const float* wts, const void* up, const void* down,
                                           int* meta, int* where, void* rows, void* act, float* out, float* y, int M, int W, int F,
                                           int E, int top, int scale_input, hipStream_t stream) {
  if (W % 32 || F % 32 || E > MOE_MAX_E || !scale_input) {
    ti_set_error("moe_experts (grouped): W=%d, F=%d, %d experts are not served", W, F, E);
    return 3;
  }
  TI_REQUIRE(M >= 0 && top > 0 && E > 0, "moe_experts (grouped): bad sizes");
  if (M == 0) return 0;
  const int n_pairs = M * top;
  const int max_tiles = (n_pairs + MOE_TILE - 1) / MOE_TILE + E;
  moe_group_kernel<<<1, 1024, 0, stream>>>(ids, n_pairs, E, meta);
  moe_place_kernel<<<(n_pairs + 63) / 64, 256, 0, stream>>>((const bf16_t*)h, ids, wts, meta, E, top, W, n_pairs, where, (bf16_t*)rows);
  moe_grouped_kernel<0><<<dim3(max_tiles, (F + 127) / 128), 256, 0, stream>>>((const bf16_t*)rows, (const bf16_t*)up, meta, E, act, F, W);
  moe_grouped_kernel<1><<<dim3(max_tiles, (W + 127) / 128), 256, 0, stream>>>((const bf16_t*)act, (const bf16_t*)down, meta, E, out, W, F);
  if (y) moe_combine_kernel<<<M, 256, 0, stream>>>(out, where, y, W, top);
  TI_LAUNCH_CHECK();
  return 0;
}

// ------------------------------------------------------------ gated experts
// out = sum_k s_k down_e act(gate_e h, up_e h) with gate_up [E][2F][W]: the rows are placed unscaled, one grouped product leaves
// the sums of [gate | up] in 32-bit (z), the activation is taken in 32-bit and rounded once, the second grouped product
// leaves a pair's row, and a token's rows are added times their weights in the order of choice.
__global__ void moe_gate_rows_kernel(const float* __restrict__ z, bf16_t* __restrict__ act, long n_rows, int F, int kind, float limit,
                                     float alpha) {
  const long n = n_rows * F;
  for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (long)gridDim.x * blockDim.x) {
    const long row = i / F;
    const int f = (int)(i % F);
    float g = z[row * 2 * F + f], u = z[row * 2 * F + F + f];
    float y;
    if (kind == 0) {
      y = g / (1.0f + expf(-g)) * u;
    } else {
      g = fminf(g, limit);
      u = fminf(fmaxf(u, -limit), limit);
      y = g / (1.0f + expf(-alpha * g)) * (u + 1.0f);
    }
    act[i] = f2bf(y);
  }
}

// y[m] = sum_k wts[m top + k] out[where[m top + k]], k ascending
__global__ void moe_combine_weighted_kernel(const float* __restrict__ out, const int* __restrict__ where, const float* __restrict__ wts,
                                            float* __restrict__ y, int W, int top) {
  const int m = blockIdx.x;
  for (int c = threadIdx.x; c < W; c += blockDim.x) {
    float v = 0.f;
    for (int k = 0; k < top; ++k) v = fmaf(wts[m * top + k], out[(size_t)where[m * top + k] * W + c], v);
    y[(size_t)m * W + c] = v;
  }
}

// Scratch as ti_moe_experts_grouped_bf16, and z f32 [M top][2F].  3: sizes not served (W, F multiples of 32, E <= 1024).
extern "C" int ti_moe_experts_grouped_gated_bf16(const void* h, const int* ids, const float* wts, const void* gate_up, const void* down,
                                                 int* meta, int* where, void* rows, float* z, void* act, float* out, float* y, int M,
                                                 int W, int F, int E, int top, int act_kind, float limit, float alpha,
                                                 hipStream_t stream) {
  if (W % 32 || F % 32 || E > MOE_MAX_E) {
    ti_set_error("moe_experts (grouped, gated): W=%d, F=%d, %d experts are not served", W, F, E);
    return 3;
  }
  TI_REQUIRE(M >= 0 && top > 0 && E > 0 && y && (act_kind == 0 || act_kind == 1), "moe_experts (grouped, gated): bad arguments");
  if (M == 0) return 0;
  const int n_pairs = M * top;
  const int max_tiles = (n_pairs + MOE_TILE - 1) / MOE_TILE + E;
  moe_group_kernel<<<1, 1024, 0, stream>>>(ids, n_pairs, E, meta);
  moe_place_kernel<<<(n_pairs + 63) / 64, 256, 0, stream>>>((const bf16_t*)h, ids, nullptr, meta, E, top, W, n_pairs, where, (bf16_t*)rows);
  moe_grouped_kernel<1><<<dim3(max_tiles, (2 * F + 127) / 128), 256, 0, stream>>>((const bf16_t*)rows, (const bf16_t*)gate_up, meta, E, z, 2 * F, W);
  const long n_act = (long)n_pairs * F;
  const unsigned blocks = (unsigned)((n_act + 255) / 256 < 16384 ? (n_act + 255) / 256 : 16384);
  moe_gate_rows_kernel<<<blocks, 256, 0, stream>>>(z, (bf16_t*)act, n_pairs, F, act_kind, limit, alpha);
  moe_grouped_kernel<1><<<dim3(max_tiles, (W + 127) / 128), 256, 0, stream>>>((const bf16_t*)act, (const bf16_t*)down, meta, E, out, W, F);
  moe_combine_weighted_kernel<<<M, 256, 0, stream>>>(out, where, wts, y, W, top);
  TI_LAUNCH_CHECK();
  return 0;
}
