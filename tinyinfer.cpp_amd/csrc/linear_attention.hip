// libti_linear_attention: linear attention with a fixed decay per head as a scan over each request's tokens of the step, and
// the gated norm behind it.
//
//   q = silu(.), k = silu(.) (heads x dk), v = silu(.) (heads x dv) from the 32-bit sums of one stacked projection;
//   per head  S_t = decay_h S_(t-1) + k_t v_t^T,  o_t = S_t^T q_t;  S [dk][dv] is per-request state in 32-bit, from and
//   into the request's slot.  Everything here is 32-bit.
//
// A workgroup per (entry, head), or per (chunk, head) where long portions are cut into chunks that run side by side.  The
// state lives in registers: thread (rg, j) holds RPT neighbouring rows of column j (RG = threads / padded dv row groups).  Tokens are staged TB at a time in LDS (activations applied on the way); per token a thread
// updates its rows and leaves its share of o_t[j] in LDS; after the TB tokens the shares are added in ascending rg.  The
// order of every sum depends on the sizes alone, never on how the tokens were cut into steps.
#include "common.h"
#include "tinyinfer_kernels.h"

TI_ERROR_API

// z sigmoid(z) with the hardware's exponential and reciprocal (a few units of 32-bit rounding)
__device__ __forceinline__ float la_silu(float z) { return z * __frcp_rn(1.0f + __expf(-z)); }

// MODE 0: an entry's tokens from and into its slot.  MODE 1: a chunk alone from an empty state, no outputs, its state into
// `scratch` [chunk][head][dk][dv].  MODE 2: a chunk from the state `scratch` holds for it (what the carry kernel left there),
// with outputs; the state is not written.  chunks [n][4] = (entry, first row, tokens, 1: the entry's first chunk + 2: its last).
// A thread's rows are RPT neighbours rg RPT .., so that their k and q come in pieces of four from LDS (rows beyond dk are
// staged as zeros and cost nothing but their multiply-adds).
template <int NT, int RPT, int TB, int MODE>
__global__ void __launch_bounds__(NT)
decay_scan_kernel(const float* __restrict__ proj, int ld, int off_q, int off_k, int off_v, const float* __restrict__ decay,
                  float* __restrict__ state, long slot_stride, const int* __restrict__ entry_meta, const int* __restrict__ chunks,
                  float* __restrict__ scratch, float* __restrict__ o, int heads, int dk, int dv, int dvs, int dvp) {
  extern __shared__ __attribute__((aligned(16))) float lds[];
  const int h = blockIdx.y;
  int row0, n, slot = 0;
  if (MODE == 0) {
    row0 = entry_meta[4 * blockIdx.x];
    n = entry_meta[4 * blockIdx.x + 1];
    slot = entry_meta[4 * blockIdx.x + 3];
  } else {
    row0 = chunks[4 * blockIdx.x + 1];
    n = chunks[4 * blockIdx.x + 2];
  }
  const int RG = NT / dvp;
  const int dkp = RPT * RG;
  const int j = threadIdx.x % dvp, rg = threadIdx.x / dvp;
  const int i0 = rg * RPT;
  const int col0 = blockIdx.z * dvs, jg = col0 + j;      // this workgroup's slice of the state's columns: they never meet
  const bool live = j < dvs && jg < dv;
  float* s_q = lds;                               // [TB][dkp]
  float* s_k = s_q + TB * dkp;                    // [TB][dkp]
  float* s_v = s_k + TB * dkp;                    // [TB][dvs]
  float* s_part = s_v + TB * dvs;                 // [TB][RG][dvp] = [TB][NT]
  float* S = MODE == 0 ? state + (size_t)slot * slot_stride + (size_t)h * dk * dv
                       : scratch + ((size_t)blockIdx.x * heads + h) * dk * dv;
  const float a = decay[h];
  float reg[RPT];
#pragma unroll
  for (int r = 0; r < RPT; ++r) reg[r] = (MODE != 1 && live && i0 + r < dk) ? S[(size_t)(i0 + r) * dv + jg] : 0.f;
  const int width = 2 * dkp + dvs;
  for (int t0 = 0; t0 < n; t0 += TB) {
    const int nt = min(TB, n - t0);
    __syncthreads();
    for (int x = threadIdx.x; x < nt * width; x += NT) {
      const int tt = x / width, c = x % width;
      const float* row = proj + (size_t)(row0 + t0 + tt) * ld;
      if (c < dkp) s_q[tt * dkp + c] = c < dk ? la_silu(row[off_q + h * dk + c]) : 0.f;
      else if (c < 2 * dkp) s_k[tt * dkp + c - dkp] = c - dkp < dk ? la_silu(row[off_k + h * dk + c - dkp]) : 0.f;
      else s_v[tt * dvs + c - 2 * dkp] = col0 + c - 2 * dkp < dv ? la_silu(row[off_v + h * dv + col0 + c - 2 * dkp]) : 0.f;
    }
    __syncthreads();
    for (int tt = 0; tt < nt; ++tt) {
      const float vj = live ? s_v[tt * dvs + j] : 0.f;
      float part = 0.f;
      if constexpr (RPT % 4 == 0) {
        const float4* k4 = reinterpret_cast<const float4*>(s_k + tt * dkp + i0);
        const float4* q4 = reinterpret_cast<const float4*>(s_q + tt * dkp + i0);
#pragma unroll
        for (int r = 0; r < RPT / 4; ++r) {
          const float4 kk = k4[r];
          reg[4 * r] = fmaf(a, reg[4 * r], kk.x * vj);
          reg[4 * r + 1] = fmaf(a, reg[4 * r + 1], kk.y * vj);
          reg[4 * r + 2] = fmaf(a, reg[4 * r + 2], kk.z * vj);
          reg[4 * r + 3] = fmaf(a, reg[4 * r + 3], kk.w * vj);
          if (MODE != 1) {
            const float4 qq = q4[r];
            part = fmaf(reg[4 * r], qq.x, part);
            part = fmaf(reg[4 * r + 1], qq.y, part);
            part = fmaf(reg[4 * r + 2], qq.z, part);
            part = fmaf(reg[4 * r + 3], qq.w, part);
          }
        }
      } else {
#pragma unroll
        for (int r = 0; r < RPT; ++r) {
          reg[r] = fmaf(a, reg[r], s_k[tt * dkp + i0 + r] * vj);
          if (MODE != 1) part = fmaf(reg[r], s_q[tt * dkp + i0 + r], part);
        }
      }
      if (MODE != 1) s_part[tt * NT + threadIdx.x] = part;
    }
    if (MODE == 1) continue;
    __syncthreads();
    for (int x = threadIdx.x; x < nt * dvs; x += NT) {
      const int tt = x / dvs, c = x % dvs;
      if (col0 + c >= dv) continue;
      float acc = 0.f;
      for (int g = 0; g < RG; ++g) acc += s_part[tt * NT + g * dvp + c];
      o[(size_t)(row0 + t0 + tt) * heads * dv + (size_t)h * dv + col0 + c] = acc;
    }
  }
  if (MODE == 2) return;
#pragma unroll
  for (int r = 0; r < RPT; ++r)
    if (live && i0 + r < dk) S[(size_t)(i0 + r) * dv + jg] = reg[r];
}

// The states the chunks of an entry start from: with S the entry's state before the step (its slot) and A_c what chunk c adds
// to an empty state over its n_c tokens, chunk c starts from S and leaves decay^(n_c) S + A_c.  scratch [chunk][head][dk dv]
// holds A_c when the kernel starts and the chunk's start state when it ends; the slot gets the state behind the last chunk.
// A thread per element of the state; spans [entry][2] = (first chunk, chunks).
__global__ void decay_carry_kernel(float* __restrict__ scratch, const int* __restrict__ chunks, const int* __restrict__ spans,
                                   const int* __restrict__ entry_meta, const float* __restrict__ decay, float* __restrict__ state,
                                   long slot_stride, int heads, int per_head) {
  const int e = blockIdx.x, h = blockIdx.y;
  const int x = blockIdx.z * blockDim.x + threadIdx.x;
  if (x >= per_head) return;
  const int c0 = spans[2 * e], nc = spans[2 * e + 1];
  float* slot = state + (size_t)entry_meta[4 * e + 3] * slot_stride + (size_t)h * per_head + x;
  const float a = decay[h];
  float S = *slot;
  int f_len = -1;      // the power of the decay last worked out, and for how many tokens
  float f = 1.f;
  // eight chunks' shares are asked for together: the walk waits for memory once per eight chunks, not once per chunk
  for (int c = c0; c < c0 + nc; c += 8) {
    float add[8];
    int len[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int ci = min(c + i, c0 + nc - 1);
      add[i] = scratch[((size_t)ci * heads + h) * per_head + x];
      len[i] = chunks[4 * ci + 2];
    }
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      if (c + i >= c0 + nc) break;
      scratch[((size_t)(c + i) * heads + h) * per_head + x] = S;
      if (len[i] != f_len) {
        f = 1.f;
        for (int t = len[i]; t > 0; --t) f *= a;
        f_len = len[i];
      }
      S = fmaf(f, S, add[i]);
    }
  }
  *slot = S;
}

template <int NT, int TB, int MODE>
static int launch_scan(int rpt, dim3 grid, size_t lds, hipStream_t stream, const float* proj, int ld, int off_q, int off_k, int off_v,
                       const float* decay, float* state, long slot_stride, const int* entry_meta, const int* chunks, float* scratch,
                       float* o, int heads, int dk, int dv, int dvs, int dvp) {
#define LA_CASE(R)                                                                                                                   \
  case R:                                                                                                                            \
    decay_scan_kernel<NT, R, TB, MODE><<<grid, NT, lds, stream>>>(proj, ld, off_q, off_k, off_v, decay, state, slot_stride, entry_meta, \
                                                                  chunks, scratch, o, heads, dk, dv, dvs, dvp);                      \
    return 0;
  switch (rpt) {
    LA_CASE(1) LA_CASE(2) LA_CASE(4) LA_CASE(8) LA_CASE(16) LA_CASE(32) LA_CASE(64)
  }
#undef LA_CASE
  return 1;
}

// wide states are cut into slices of 64 columns, a workgroup each: more workgroups, and fewer rows a thread
struct ScanShape { int dvs, slices, dvp, nt, tb, rpt; size_t lds; bool big; };
static ScanShape scan_shape(int dk, int dv) {
  ScanShape s;
  s.dvs = dv > 64 ? 64 : dv;
  s.slices = (dv + s.dvs - 1) / s.dvs;
  s.dvp = 1;
  while (s.dvp < s.dvs) s.dvp *= 2;
  s.big = (long)dk * s.dvp > 64L * 256;
  s.nt = s.big ? 1024 : 256;
  s.tb = s.big ? 4 : 16;
  const int rgs = s.nt / s.dvp;
  s.rpt = 1;
  while (s.rpt * rgs < dk) s.rpt *= 2;
  s.lds = ((size_t)s.tb * (2 * s.rpt * rgs + s.dvs) + (size_t)s.tb * s.nt) * 4;
  return s;
}

static int check_scan(const char* what, int ld, int off_q, int off_k, int off_v, long slot_stride, int heads, int dk, int dv) {
  TI_REQUIRE(heads > 0 && heads <= 65535 && dk > 0 && dk <= 256 && dv > 0 && dv <= 256, "%s: bad sizes heads=%d dk=%d dv=%d (up to 256)",
             what, heads, dk, dv);
  TI_REQUIRE(off_q >= 0 && off_k >= 0 && off_v >= 0 && off_q + heads * dk <= ld && off_k + heads * dk <= ld && off_v + heads * dv <= ld,
             "%s: the columns do not lie inside rows of %d", what, ld);
  TI_REQUIRE(slot_stride >= (long)heads * dk * dv, "%s: a slot of %ld floats does not hold the state", what, slot_stride);
  return 0;
}

// proj f32 [M, ld]: q, k (heads x dk) and v (heads x dv) before their activation from the given columns on; decay f32 [heads];
// state f32 [slots][heads][dk][dv] (slot_stride floats a slot); entry_meta [n_entries][4] = (row0, tokens, start, slot);
// o f32 [M, heads dv]
extern "C" int ti_decay_scan(const float* proj, int ld, int off_q, int off_k, int off_v, const float* decay, float* state,
                             long slot_stride, const int* entry_meta, int n_entries, float* o, int heads, int dk, int dv,
                             hipStream_t stream) {
  if (check_scan("decay_scan", ld, off_q, off_k, off_v, slot_stride, heads, dk, dv)) return 1;
  if (n_entries == 0) return 0;
  const ScanShape s = scan_shape(dk, dv);
  TI_REQUIRE(s.rpt <= 64, "decay_scan: a state of %d x %d is not served", dk, dv);
  const dim3 grid(n_entries, heads, s.slices);
  const int rc = s.big ? launch_scan<1024, 4, 0>(s.rpt, grid, s.lds, stream, proj, ld, off_q, off_k, off_v, decay, state, slot_stride,
                                                 entry_meta, nullptr, nullptr, o, heads, dk, dv, s.dvs, s.dvp)
                       : launch_scan<256, 16, 0>(s.rpt, grid, s.lds, stream, proj, ld, off_q, off_k, off_v, decay, state, slot_stride,
                                                 entry_meta, nullptr, nullptr, o, heads, dk, dv, s.dvs, s.dvp);
  TI_REQUIRE(rc == 0, "decay_scan: no kernel for %d rows a thread", s.rpt);
  TI_LAUNCH_CHECK();
  return 0;
}

// The same with every entry's tokens cut into chunks that run side by side: every chunk alone from an empty state, the states
// carried from chunk to chunk element by element, every chunk again from the state it starts from, with outputs.
// chunks int [n_chunks][4] = (entry, first row, tokens, flags), spans int [n_entries][2] = (first chunk, chunks), both in
// device memory; scratch float [n_chunks][heads][dk dv]
extern "C" int ti_decay_scan_chunked(const float* proj, int ld, int off_q, int off_k, int off_v, const float* decay, float* state,
                                     long slot_stride, const int* entry_meta, int n_entries, const int* chunks, int n_chunks,
                                     const int* spans, float* scratch, float* o, int heads, int dk, int dv, hipStream_t stream) {
  if (check_scan("decay_scan", ld, off_q, off_k, off_v, slot_stride, heads, dk, dv)) return 1;
  TI_REQUIRE(chunks && spans && scratch && n_chunks >= n_entries, "decay_scan: chunks need their lists and scratch");
  if (n_entries == 0) return 0;
  const ScanShape s = scan_shape(dk, dv);
  TI_REQUIRE(s.rpt <= 64, "decay_scan: a state of %d x %d is not served", dk, dv);
  const dim3 grid(n_chunks, heads, s.slices);
  int rc = s.big ? launch_scan<1024, 4, 1>(s.rpt, grid, s.lds, stream, proj, ld, off_q, off_k, off_v, decay, state, slot_stride, entry_meta,
                                           chunks, scratch, o, heads, dk, dv, s.dvs, s.dvp)
                 : launch_scan<256, 16, 1>(s.rpt, grid, s.lds, stream, proj, ld, off_q, off_k, off_v, decay, state, slot_stride, entry_meta,
                                           chunks, scratch, o, heads, dk, dv, s.dvs, s.dvp);
  TI_REQUIRE(rc == 0, "decay_scan: no kernel for %d rows a thread", s.rpt);
  const int per_head = dk * dv;
  decay_carry_kernel<<<dim3(n_entries, heads, (per_head + 255) / 256), 256, 0, stream>>>(scratch, chunks, spans, entry_meta, decay, state,
                                                                                       slot_stride, heads, per_head);
  rc = s.big ? launch_scan<1024, 4, 2>(s.rpt, grid, s.lds, stream, proj, ld, off_q, off_k, off_v, decay, state, slot_stride, entry_meta,
                                       chunks, scratch, o, heads, dk, dv, s.dvs, s.dvp)
             : launch_scan<256, 16, 2>(s.rpt, grid, s.lds, stream, proj, ld, off_q, off_k, off_v, decay, state, slot_stride, entry_meta,
                                       chunks, scratch, o, heads, dk, dv, s.dvs, s.dvp);
  TI_REQUIRE(rc == 0, "decay_scan: no kernel for %d rows a thread", s.rpt);
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
