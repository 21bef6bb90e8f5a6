// Latent attention: a token keeps one normed latent c (R numbers) and one rotated key part (r numbers) shared by all heads;
// a head's unrotated key is W_uk c and its value W_uv c.  The kernels here never form keys or values per token.  With
// q = [q_plain (d) | q_rot (r)] per head:
//   score(i, j) = (q_plain . W_uk c_j + q_rot . kr_j) scale = ((W_uk^T q_plain) . c_j + q_rot . kr_j) scale,
//   out_i       = W_uv sum_j p_ij c_j,
// so every head attends over the cached rows [c | kr] with the absorbed query [W_uk^T q_plain | q_rot] (R + r numbers),
// its value is the first R entries of the same row, and W_uv maps the head's weighted latent to its output.  The softmax
// may hold a sink: exp(sink_h) in the denominator, with no key and no value.
//
//   latent_prep     proj f32 -> cache row [rms-normed c * w | rotated kr] (T), the heads' q_rot rotated in place; a page of
//                   P (2 R + r) elements also gets the latents transposed [R][P] behind its rows (the matrix-core kernels' operand)
//   latent_absorb   qa f32 [M, H, R + r] = [W_uk_h^T q_plain | q_rot]
//   latent_rows     o f32 [M, H, R]: a workgroup per (row, head) over the paged rows, scores and softmax in 32-bit
//   latent_expand   out T [M, H dv] = W_uv_h o
// All arithmetic is 32-bit with sums in a fixed order; T is the storage type of cache, weights and the result.
#include "common.h"
#include "tinyinfer_kernels.h"

TI_ERROR_API

__device__ __forceinline__ void latent_rotation(const float* __restrict__ inv_freq, const float* __restrict__ rope_table, int table_len,
                                                float mag, int half, int p, int i, float* c, float* s) {
  if (rope_table && p < table_len) {
    *c = rope_table[((size_t)p * half + i) * 2];
    *s = rope_table[((size_t)p * half + i) * 2 + 1];
  } else {
    const float a = (float)p * inv_freq[i];
    *c = cosf(a) * mag;
    *s = sinf(a) * mag;
  }
}

// ------------------------------------------------------------ preparation
// proj f32 [M, ld]: the heads' queries [H][d + r] from column 0, then the latent (R) and the shared key part (r) from
// column off_kv.  A workgroup per token.
template <typename T>
__global__ void __launch_bounds__(256)
latent_prep_kernel(float* __restrict__ proj, int ldp, int off_kv, const float* __restrict__ norm_w, float eps,
                   const float* __restrict__ inv_freq, const float* __restrict__ rope_table, int table_len, float mag, int rot_dims,
                   const int* __restrict__ pos, const int* __restrict__ slot, const int* __restrict__ table, int table_stride,
                   T* __restrict__ pool, size_t page_elems, int H, int d, int r, int R, int P) {
  __shared__ float red[4];
  const int m = blockIdx.x;
  const int p = pos[m];
  float* row = proj + (size_t)m * ldp;
  const float* c = row + off_kv;
  float ss = 0.f;
  for (int i = threadIdx.x; i < R; i += 256) ss = fmaf(c[i], c[i], ss);
  ss = block_sum<256>(ss, red);
  const float scale = 1.0f / sqrtf(ss / (float)R + eps);
  const int page = table[(size_t)slot[m] * table_stride + p / P];
  T* dst = pool + (size_t)max(page, 0) * page_elems + (size_t)(p % P) * (R + r);
  // a page that is longer than its P rows holds the latents a second time, transposed [R][P], behind them
  T* tdst = page_elems >= (size_t)P * (2 * R + r) ? pool + (size_t)max(page, 0) * page_elems + (size_t)P * (R + r) + p % P : nullptr;
  const int half = inv_freq ? rot_dims / 2 : 0;
  if (page >= 0) {      // the host reserves pages first; never write astray
    for (int i = threadIdx.x; i < R; i += 256) {
      const float v = c[i] * scale * norm_w[i];
      st<T>(dst + i, v);
      if (tdst) st<T>(tdst + (size_t)i * P, v);
    }
    const float* kr = c + R;
    for (int i = threadIdx.x; i < r; i += 256) {
      if (i >= half && i < 2 * half) continue;
      float u = kr[i];
      if (i < half) {
        float w = kr[i + half], cs, sn;
        latent_rotation(inv_freq, rope_table, table_len, mag, half, p, i, &cs, &sn);
        st<T>(dst + R + i + half, w * cs + u * sn);
        u = u * cs - w * sn;
      }
      st<T>(dst + R + i, u);
    }
  }
  // the heads' rotated parts, in place
  for (int e = threadIdx.x; e < H * half; e += 256) {
    const int h = e / half, i = e % half;
    float* q = row + (size_t)h * (d + r) + d;
    float cs, sn;
    latent_rotation(inv_freq, rope_table, table_len, mag, half, p, i, &cs, &sn);
    const float u = q[i], w = q[i + half];
    q[i] = u * cs - w * sn;
    q[i + half] = w * cs + u * sn;
  }
}

extern "C" int ti_latent_prep(int dtype, float* proj, int ldp, int off_kv, const float* norm_w, float eps, const float* inv_freq,
                              const float* rope_table, int table_len, float mag, int rot_dims, const int* pos, const int* slot,
                              const int* table, int table_stride, void* pool, long page_elems, int M, int H, int d, int r, int R,
                              int page_size, hipStream_t stream) {
  TI_REQUIRE(H > 0 && d >= 0 && r >= 0 && R > 0 && page_size > 0 && table_stride > 0 && off_kv >= H * (d + r) && ldp >= off_kv + R + r &&
                 page_elems >= (long)page_size * (R + r),
             "latent_prep: bad sizes heads=%d dim=%d rot=%d rank=%d ld=%d page=%ld", H, d, r, R, ldp, page_elems);
  TI_REQUIRE(!inv_freq || (rot_dims >= 0 && rot_dims % 2 == 0 && rot_dims <= r), "latent_prep: %d rotated entries do not fit %d", rot_dims, r);
  if (M == 0) return 0;
#define LATENT_PREP(T)                                                                                                              \
  latent_prep_kernel<T><<<M, 256, 0, stream>>>(proj, ldp, off_kv, norm_w, eps, inv_freq, rope_table, table_len, mag, rot_dims, pos, \
                                               slot, table, table_stride, (T*)pool, (size_t)page_elems, H, d, r, R, page_size)
  if (dtype == TI_F32) LATENT_PREP(float);
  else if (dtype == TI_BF16) LATENT_PREP(bf16_t);
  else TI_REQUIRE(false, "latent_prep: unknown dtype %d", dtype);
#undef LATENT_PREP
  TI_LAUNCH_CHECK();
  return 0;
}

// ------------------------------------------------------------ the absorbed query
// qa[m, h, c] = sum_k q[m, h, k] W_uk[h d + k, c] for c < R (k ascending), qa[m, h, R + j] = q_rot[m, h, j].
// Grid (tokens / TM, heads, R / 256): a thread owns a column for TM tokens, whose q lie in LDS; W_uk [H d][R] in T.
#define LATENT_TM 8
template <typename T>
__global__ void __launch_bounds__(256)
latent_absorb_kernel(const float* __restrict__ proj, int ldp, const T* __restrict__ w_uk, float* __restrict__ qa, int M, int H, int d,
                     int r, int R) {
  extern __shared__ float s_q[];      // [TM][d]
  const int m0 = blockIdx.x * LATENT_TM, h = blockIdx.y;
  const int n = min(LATENT_TM, M - m0);
  for (int e = threadIdx.x; e < LATENT_TM * d; e += 256) {
    const int t = e / d, k = e % d;
    s_q[e] = t < n ? proj[(size_t)(m0 + t) * ldp + (size_t)h * (d + r) + k] : 0.f;
  }
  __syncthreads();
  const int c = blockIdx.z * 256 + threadIdx.x;
  if (c < R) {
    float acc[LATENT_TM];
#pragma unroll
    for (int t = 0; t < LATENT_TM; ++t) acc[t] = 0.f;
    const T* w = w_uk + (size_t)h * d * R + c;
    for (int k = 0; k < d; ++k) {
      const float wv = ld<T>(w + (size_t)k * R);
#pragma unroll
      for (int t = 0; t < LATENT_TM; ++t) acc[t] = fmaf(s_q[t * d + k], wv, acc[t]);
    }
#pragma unroll
    for (int t = 0; t < LATENT_TM; ++t)
      if (t < n) qa[((size_t)(m0 + t) * H + h) * (R + r) + c] = acc[t];
  }
  if (blockIdx.z == 0)
    for (int e = threadIdx.x; e < n * r; e += 256) {
      const int t = e / r, j = e % r;
      qa[((size_t)(m0 + t) * H + h) * (R + r) + R + j] = proj[(size_t)(m0 + t) * ldp + (size_t)h * (d + r) + d + j];
    }
}

extern "C" int ti_latent_absorb(int dtype, const float* proj, int ldp, const void* w_uk, float* qa, int M, int H, int d, int r, int R,
                                hipStream_t stream) {
  TI_REQUIRE(H > 0 && d >= 0 && r >= 0 && R > 0 && ldp >= H * (d + r) && H <= 65535, "latent_absorb: bad sizes heads=%d dim=%d rot=%d rank=%d ld=%d", H, d, r,
             R, ldp);
  TI_REQUIRE((size_t)LATENT_TM * d * 4 <= 48 * 1024, "latent_absorb: a key size of %d is not served", d);
  if (M == 0) return 0;
  const dim3 grid((M + LATENT_TM - 1) / LATENT_TM, H, (R + 255) / 256);
  const size_t lds = (size_t)LATENT_TM * (d > 0 ? d : 1) * 4;
  if (dtype == TI_F32) latent_absorb_kernel<float><<<grid, 256, lds, stream>>>(proj, ldp, (const float*)w_uk, qa, M, H, d, r, R);
  else if (dtype == TI_BF16) latent_absorb_kernel<bf16_t><<<grid, 256, lds, stream>>>(proj, ldp, (const bf16_t*)w_uk, qa, M, H, d, r, R);
  else TI_REQUIRE(false, "latent_absorb: unknown dtype %d", dtype);
  TI_LAUNCH_CHECK();
  return 0;
}

// ------------------------------------------------------------ attention over the latent rows
// A workgroup per (row, head): 16 groups of 16 lanes; lane j of a group owns entries j, j + 16, ... of a cached row, group g
// walks the keys lo + g, lo + g + 16, ... with a running softmax; the 16 shares are merged through LDS in a fixed order, and the
// sink joins the denominator there.  A key's group depends on its position alone, so a row's sums do not depend on the step.
#define LA_GROUPS 16
#define LA_LANES 16
template <typename T, int DPL>
__global__ void __launch_bounds__(256)
latent_rows_kernel(const float* __restrict__ qa, const T* __restrict__ pool, const int* __restrict__ table, int table_stride,
                   const int* __restrict__ pos, const int* __restrict__ slot, const float* __restrict__ sink, float* __restrict__ out,
                   int H, int R, int r, int P, size_t page_elems, float scale, int window) {
  extern __shared__ float s_o[];      // [groups][R]
  __shared__ float s_m[LA_GROUPS], s_l[LA_GROUPS];
  const int m = blockIdx.x, h = blockIdx.y;
  const int g = threadIdx.x / LA_LANES, lane = threadIdx.x % LA_LANES;
  const int DK = R + r;
  const int p_q = pos[m];
  const int lo = (window > 0 && p_q - window + 1 > 0) ? p_q - window + 1 : 0;
  const int* tab = table + (size_t)slot[m] * table_stride;
  float qv[DPL], o[DPL];
  const float* qh = qa + ((size_t)m * H + h) * DK;
#pragma unroll
  for (int i = 0; i < DPL; ++i) {
    const int e = lane + i * LA_LANES;
    qv[i] = e < DK ? qh[e] : 0.f;
    o[i] = 0.f;
  }
  float mx = -INFINITY, l = 0.f;
  for (int p = lo + g; p <= p_q; p += LA_GROUPS) {
    const int page = tab[p / P];
    if (page < 0) continue;
    const T* kp = pool + (size_t)page * page_elems + (size_t)(p % P) * DK;
    float kv[DPL];
    float s = 0.f;
#pragma unroll
    for (int i = 0; i < DPL; ++i) {
      const int e = lane + i * LA_LANES;
      kv[i] = e < DK ? ld<T>(kp + e) : 0.f;
      s = fmaf(qv[i], kv[i], s);
    }
    s = group_sum<LA_LANES>(s) * scale;
    const float m_new = fmaxf(mx, s);
    const float alpha = expf(mx - m_new);
    const float w = expf(s - m_new);
    l = l * alpha + w;
#pragma unroll
    for (int i = 0; i < DPL; ++i) o[i] = o[i] * alpha + w * kv[i];
    mx = m_new;
  }
#pragma unroll
  for (int i = 0; i < DPL; ++i) {
    const int e = lane + i * LA_LANES;
    if (e < R) s_o[(size_t)g * R + e] = o[i];
  }
  if (lane == 0) {
    s_m[g] = mx;
    s_l[g] = l;
  }
  __syncthreads();
  float mm = sink ? sink[h] : -INFINITY;
#pragma unroll
  for (int j = 0; j < LA_GROUPS; ++j) mm = fmaxf(mm, s_m[j]);
  float lt = sink ? expf(sink[h] - mm) : 0.f;
  float wj[LA_GROUPS];
#pragma unroll
  for (int j = 0; j < LA_GROUPS; ++j) {
    wj[j] = (s_m[j] == -INFINITY) ? 0.f : expf(s_m[j] - mm);
    lt += s_l[j] * wj[j];
  }
  for (int e = threadIdx.x; e < R; e += 256) {
    float acc = 0.f;
#pragma unroll
    for (int j = 0; j < LA_GROUPS; ++j) acc += s_o[(size_t)j * R + e] * wj[j];
    out[((size_t)m * H + h) * R + e] = acc / lt;
  }
}

template <typename T>
static int launch_latent_rows(int dpl, dim3 grid, size_t lds, const float* qa, const void* pool, size_t page_elems, const int* table, int table_stride,
                              const int* pos, const int* slot, const float* sink, float* out, int H, int R, int r, int P, float scale,
                              int window, hipStream_t stream) {
#define LA_CASE(D)                                                                                                               \
  if (dpl <= D) {                                                                                                                \
    latent_rows_kernel<T, D><<<grid, 256, lds, stream>>>(qa, (const T*)pool, table, table_stride, pos, slot, sink, out, H, R, r, \
                                                         P, page_elems, scale, window);                                                      \
    return 0;                                                                                                                    \
  }
  LA_CASE(2) LA_CASE(4) LA_CASE(8) LA_CASE(12) LA_CASE(16) LA_CASE(24) LA_CASE(32) LA_CASE(40) LA_CASE(48)
#undef LA_CASE
  return 1;
}

// qa f32 [M, H, R + r]; pool T [pages][P][R + r]; sink f32 [H] (null: none); out f32 [M, H, R]
extern "C" int ti_latent_attention_rows(int dtype, const float* qa, const void* pool, long page_elems, const int* table, int table_stride,
                                        const int* pos, const int* slot, const float* sink, float* out, int M, int H, int R, int r,
                                        int page_size, float scale, int window, hipStream_t stream) {
  TI_REQUIRE(H > 0 && H <= 65535 && R > 0 && r >= 0 && R + r <= 48 * LA_LANES, "latent_attention: heads=%d, a latent of %d + %d is not served (up to %d)",
             H, R, r, 48 * LA_LANES);
  TI_REQUIRE(page_size > 0 && table_stride > 0 && page_elems >= (long)page_size * (R + r), "latent_attention: bad page_size %d / table_stride %d / page of %ld", page_size,
             table_stride, page_elems);
  if (M == 0) return 0;
  const dim3 grid(M, H);
  const int dpl = (R + r + LA_LANES - 1) / LA_LANES;
  const size_t lds = (size_t)LA_GROUPS * R * 4;
  int rc;
  if (dtype == TI_F32)
    rc = launch_latent_rows<float>(dpl, grid, lds, qa, pool, (size_t)page_elems, table, table_stride, pos, slot, sink, out, H, R, r, page_size, scale, window, stream);
  else if (dtype == TI_BF16)
    rc = launch_latent_rows<bf16_t>(dpl, grid, lds, qa, pool, (size_t)page_elems, table, table_stride, pos, slot, sink, out, H, R, r, page_size, scale, window, stream);
  else
    TI_REQUIRE(false, "latent_attention: unknown dtype %d", dtype);
  TI_REQUIRE(rc == 0, "latent_attention: no kernel for a latent of %d + %d", R, r);
  TI_LAUNCH_CHECK();
  return 0;
}

// ------------------------------------------------------------ a head's weighted latent to its output
// out[m, h dv + j] = sum_c o[m, h, c] W_uv[h dv + j, c].  Grid (tokens / TM, heads); the TM rows of o lie in LDS, a wavefront
// takes the outputs j = wave, wave + 4, ...: its lanes share the weight's row (lane l the entries l, l + 64, ... in ascending
// order, then a butterfly).
template <typename T>
__global__ void __launch_bounds__(256)
latent_expand_kernel(const float* __restrict__ o, const T* __restrict__ w_uv, T* __restrict__ out, int M, int H, int R, int dv) {
  extern __shared__ float s_r[];      // [TM][R]
  const int m0 = blockIdx.x * LATENT_TM, h = blockIdx.y;
  const int n = min(LATENT_TM, M - m0);
  for (int e = threadIdx.x; e < LATENT_TM * R; e += 256) {
    const int t = e / R, c = e % R;
    s_r[e] = t < n ? o[((size_t)(m0 + t) * H + h) * R + c] : 0.f;
  }
  __syncthreads();
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  for (int j = wave; j < dv; j += 4) {
    const T* w = w_uv + ((size_t)h * dv + j) * R;
    float acc[LATENT_TM];
#pragma unroll
    for (int t = 0; t < LATENT_TM; ++t) acc[t] = 0.f;
    for (int c = lane; c < R; c += 64) {
      const float wv = ld<T>(w + c);
#pragma unroll
      for (int t = 0; t < LATENT_TM; ++t) acc[t] = fmaf(s_r[t * R + c], wv, acc[t]);
    }
#pragma unroll
    for (int t = 0; t < LATENT_TM; ++t) acc[t] = group_sum<64>(acc[t]);
    if (lane == 0)
#pragma unroll
      for (int t = 0; t < LATENT_TM; ++t)
        if (t < n) st<T>(out + (size_t)(m0 + t) * H * dv + (size_t)h * dv + j, acc[t]);
  }
}

extern "C" int ti_latent_expand(int dtype, const float* o, const void* w_uv, void* out, int M, int H, int R, int dv, hipStream_t stream) {
  TI_REQUIRE(H > 0 && H <= 65535 && R > 0 && dv > 0 && (size_t)LATENT_TM * R * 4 <= 48 * 1024, "latent_expand: bad sizes heads=%d rank=%d vdim=%d", H, R, dv);
  if (M == 0) return 0;
  const dim3 grid((M + LATENT_TM - 1) / LATENT_TM, H);
  const size_t lds = (size_t)LATENT_TM * R * 4;
  if (dtype == TI_F32) latent_expand_kernel<float><<<grid, 256, lds, stream>>>(o, (const float*)w_uv, (float*)out, M, H, R, dv);
  else if (dtype == TI_BF16) latent_expand_kernel<bf16_t><<<grid, 256, lds, stream>>>(o, (const bf16_t*)w_uv, (bf16_t*)out, M, H, R, dv);
  else TI_REQUIRE(false, "latent_expand: unknown dtype %d", dtype);
  TI_LAUNCH_CHECK();
  return 0;
}

// ------------------------------------------------------------ a head's matrices transposed
// dst [H][cols][rows] = src [H][rows][cols]^T, head by head: what the matrix-core kernel of the absorbed query reads
template <typename T>
__global__ void __launch_bounds__(256)
latent_transpose_kernel(const T* __restrict__ src, T* __restrict__ dst, int rows, int cols) {
  const size_t base = (size_t)blockIdx.y * rows * cols;
  const int e = blockIdx.x * 256 + threadIdx.x;
  if (e < rows * cols) dst[base + (size_t)(e % cols) * rows + e / cols] = src[base + e];
}

extern "C" int ti_latent_transpose(int dtype, const void* src, void* dst, int H, int rows, int cols, hipStream_t stream) {
  TI_REQUIRE(H > 0 && H <= 65535 && rows > 0 && cols > 0, "latent_transpose: bad sizes %d x %d x %d", H, rows, cols);
  const dim3 grid((rows * cols + 255) / 256, H);
  if (dtype == TI_F32) latent_transpose_kernel<float><<<grid, 256, 0, stream>>>((const float*)src, (float*)dst, rows, cols);
  else if (dtype == TI_BF16) latent_transpose_kernel<bf16_t><<<grid, 256, 0, stream>>>((const bf16_t*)src, (bf16_t*)dst, rows, cols);
  else TI_REQUIRE(false, "latent_transpose: unknown dtype %d", dtype);
  TI_LAUNCH_CHECK();
  return 0;
}
