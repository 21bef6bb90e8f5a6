// libti_linear_attention: linear attention with a fixed decay per head as a scan over each request's tokens of the step, and
// the gated norm behind it.
//
//   q = silu(.), k = silu(.) (heads x dk), v = silu(.) (heads x dv) from the 32-bit sums of one stacked projection;
//   per head  S_t = decay_h S_(t-1) + k_t v_t^T,  o_t = S_t^T q_t;  S [dk][dv] is per-request state in 32-bit, from and
//   into the request's slot.  Everything here is 32-bit.
//
// A workgroup per (entry, head).  The state lives in registers: thread (rg, j) holds rows rg, rg + RG, ... of column j
// (RG = threads / padded dv).  Tokens are staged TB at a time in LDS (activations applied on the way); per token a thread
// updates its rows and leaves its share of o_t[j] in LDS; after the TB tokens the shares are added in ascending rg.  The
// order of every sum depends on the sizes alone, never on how the tokens were cut into steps.
#include "common.h"
#include "tinyinfer_kernels.h"

TI_ERROR_API

__device__ __forceinline__ float la_silu(float z) { return z / (1.0f + expf(-z)); }

template <int NT, int RPT, int TB>
__global__ void __launch_bounds__(NT)
decay_scan_kernel(const float* __restrict__ proj, int ld, int off_q, int off_k, int off_v, const float* __restrict__ decay,
                  float* __restrict__ state, long slot_stride, const int* __restrict__ entry_meta, float* __restrict__ o, int heads,
                  int dk, int dv, int dvp) {
  extern __shared__ float lds[];
  const int e = blockIdx.x, h = blockIdx.y;
  const int row0 = entry_meta[4 * e], n = entry_meta[4 * e + 1], slot = entry_meta[4 * e + 3];
  const int RG = NT / dvp;
  const int j = threadIdx.x % dvp, rg = threadIdx.x / dvp;
  const bool live = j < dv;
  float* s_q = lds;                               // [TB][dk]
  float* s_k = s_q + TB * dk;                     // [TB][dk]
  float* s_v = s_k + TB * dk;                     // [TB][dv]
  float* s_part = s_v + TB * dv;                  // [TB][RG][dvp] = [TB][NT]
  float* S = state + (size_t)slot * slot_stride + (size_t)h * dk * dv;
  const float a = decay[h];
  float reg[RPT];
#pragma unroll
  for (int r = 0; r < RPT; ++r) {
    const int i = rg + r * RG;
    reg[r] = (live && i < dk) ? S[(size_t)i * dv + j] : 0.f;
  }
  const int width = 2 * dk + dv;
  for (int t0 = 0; t0 < n; t0 += TB) {
    const int nt = min(TB, n - t0);
    __syncthreads();
    for (int x = threadIdx.x; x < nt * width; x += NT) {
      const int tt = x / width, c = x % width;
      const float* row = proj + (size_t)(row0 + t0 + tt) * ld;
      if (c < dk) s_q[tt * dk + c] = la_silu(row[off_q + h * dk + c]);
      else if (c < 2 * dk) s_k[tt * dk + c - dk] = la_silu(row[off_k + h * dk + c - dk]);
      else s_v[tt * dv + c - 2 * dk] = la_silu(row[off_v + h * dv + c - 2 * dk]);
    }
    __syncthreads();
    for (int tt = 0; tt < nt; ++tt) {
      const float vj = live ? s_v[tt * dv + j] : 0.f;
      float part = 0.f;
#pragma unroll
      for (int r = 0; r < RPT; ++r) {
        const int i = rg + r * RG;
        if (i < dk) {
          reg[r] = fmaf(a, reg[r], s_k[tt * dk + i] * vj);
          part = fmaf(reg[r], s_q[tt * dk + i], part);
        }
      }
      s_part[tt * NT + threadIdx.x] = part;
    }
    __syncthreads();
    for (int x = threadIdx.x; x < nt * dv; x += NT) {
      const int tt = x / dv, c = x % dv;
      float acc = 0.f;
      for (int g = 0; g < RG; ++g) acc += s_part[tt * NT + g * dvp + c];
      o[(size_t)(row0 + t0 + tt) * heads * dv + (size_t)h * dv + c] = acc;
    }
  }
#pragma unroll
  for (int r = 0; r < RPT; ++r) {
    const int i = rg + r * RG;
    if (live && i < dk) S[(size_t)i * dv + j] = reg[r];
  }
}

template <int NT, int TB>
static int launch_scan(int rpt, dim3 grid, size_t lds, hipStream_t stream, const float* proj, int ld, int off_q, int off_k, int off_v,
                       const float* decay, float* state, long slot_stride, const int* entry_meta, float* o, int heads, int dk,
                       int dv, int dvp) {
#define LA_CASE(R)                                                                                                            \
  case R:                                                                                                                     \
    decay_scan_kernel<NT, R, TB><<<grid, NT, lds, stream>>>(proj, ld, off_q, off_k, off_v, decay, state, slot_stride, entry_meta, o, \
                                                            heads, dk, dv, dvp);                                              \
    return 0;
  switch (rpt) {
    LA_CASE(1) LA_CASE(2) LA_CASE(4) LA_CASE(8) LA_CASE(16) LA_CASE(32) LA_CASE(64)
  }
#undef LA_CASE
  return 1;
}

// proj f32 [M, ld]: q, k (heads x dk) and v (heads x dv) before their activation from the given columns on; decay f32 [heads];
// state f32 [slots][heads][dk][dv] (slot_stride floats a slot); entry_meta [n_entries][4] = (row0, tokens, start, slot);
// o f32 [M, heads dv]
extern "C" int ti_decay_scan(const float* proj, int ld, int off_q, int off_k, int off_v, const float* decay, float* state,
                             long slot_stride, const int* entry_meta, int n_entries, float* o, int heads, int dk, int dv,
                             hipStream_t stream) {
  TI_REQUIRE(heads > 0 && heads <= 65535 && dk > 0 && dk <= 256 && dv > 0 && dv <= 256, "decay_scan: bad sizes heads=%d dk=%d dv=%d (up to 256)",
             heads, dk, dv);
  TI_REQUIRE(off_q >= 0 && off_k >= 0 && off_v >= 0 && off_q + heads * dk <= ld && off_k + heads * dk <= ld && off_v + heads * dv <= ld,
             "decay_scan: the columns do not lie inside rows of %d", ld);
  TI_REQUIRE(slot_stride >= (long)heads * dk * dv, "decay_scan: a slot of %ld floats does not hold the state", slot_stride);
  if (n_entries == 0) return 0;
  int dvp = 1;
  while (dvp < dv) dvp *= 2;
  const bool big = (long)dk * dvp > 64L * 256;
  const int nt = big ? 1024 : 256, tb = big ? 4 : 16;
  const int rgs = nt / dvp;
  int rpt = 1;
  while (rpt * rgs < dk) rpt *= 2;
  TI_REQUIRE(rpt <= 64, "decay_scan: a state of %d x %d is not served", dk, dv);
  const size_t lds = ((size_t)tb * (2 * dk + dv) + (size_t)tb * nt) * 4;
  const dim3 grid(n_entries, heads);
  const int rc = big ? launch_scan<1024, 4>(rpt, grid, lds, stream, proj, ld, off_q, off_k, off_v, decay, state, slot_stride, entry_meta,
                                            o, heads, dk, dv, dvp)
                     : launch_scan<256, 16>(rpt, grid, lds, stream, proj, ld, off_q, off_k, off_v, decay, state, slot_stride, entry_meta,
                                            o, heads, dk, dv, dvp);
  TI_REQUIRE(rc == 0, "decay_scan: no kernel for %d rows a thread", rpt);
  TI_LAUNCH_CHECK();
  return 0;
}

// out[m, :] = o[m, :] / sqrt(mean(o[m, :]^2) + eps) * w * sigmoid(gate[m, off_g + :]): one norm over the whole row (all heads
// together), in T.  A workgroup per row.
template <typename T>
__global__ void __launch_bounds__(256)
gated_row_norm_kernel(const float* __restrict__ o, const float* __restrict__ gate, int ld, int off_g, const float* __restrict__ w,
                      T* __restrict__ out, int W, float eps) {
  __shared__ float red[4];
  const int m = blockIdx.x;
  const float* src = o + (size_t)m * W;
  float ss = 0.f;
  for (int c = threadIdx.x; c < W; c += 256) ss = fmaf(src[c], src[c], ss);
  const float inv = 1.0f / sqrtf(block_sum<256>(ss, red) / (float)W + eps);
  const float* g = gate + (size_t)m * ld + off_g;
  for (int c = threadIdx.x; c < W; c += 256) st<T>(out + (size_t)m * W + c, src[c] * inv * w[c] * (1.0f / (1.0f + expf(-g[c]))));
}

extern "C" int ti_gated_row_norm(int out_dtype, const float* o, const float* gate, int ld, int off_g, const float* w, void* out, int M,
                                 int W, float eps, hipStream_t stream) {
  TI_REQUIRE(M >= 0 && W > 0 && off_g >= 0 && off_g + W <= ld, "gated_row_norm: bad sizes M=%d W=%d gate columns %d of %d", M, W, off_g, ld);
  if (M == 0) return 0;
  if (out_dtype == TI_F32) gated_row_norm_kernel<float><<<M, 256, 0, stream>>>(o, gate, ld, off_g, w, (float*)out, W, eps);
  else if (out_dtype == TI_BF16) gated_row_norm_kernel<bf16_t><<<M, 256, 0, stream>>>(o, gate, ld, off_g, w, (bf16_t*)out, W, eps);
  else TI_REQUIRE(false, "gated_row_norm: unknown dtype %d", out_dtype);
  TI_LAUNCH_CHECK();
  return 0;
}
