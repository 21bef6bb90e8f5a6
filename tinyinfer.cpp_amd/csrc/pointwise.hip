// Element-wise kernels of layers that are not the plain pre-norm transformer block: an additive
// sinusoidal position vector, a learned vector added to every row, the xIELU activation between the
// two products of a dense feed-forward, the per-channel scaled sum of a parallel block's branches
// into the residual, and the split of a fused q/k/v projection (keys and values of different sizes,
// a position-dependent factor on the query) into the paged cache.  All arithmetic is 32-bit; T is
// the storage type of activations and cache.
#include "common.h"
#include "tinyinfer_kernels.h"

TI_ERROR_API

// ------------------------------------------------------------ sinusoidal positions
// x[m, 2i] += sin(pos[m] * inv_freq[i]),  x[m, 2i + 1] += cos(pos[m] * inv_freq[i])
__global__ void add_sinusoid_kernel(float* __restrict__ x, const int* __restrict__ pos,
                                    const float* __restrict__ inv_freq, int H) {
  const int m = blockIdx.x;
  const float p = (float)pos[m];
  float* row = x + (size_t)m * H;
  for (int c = threadIdx.x; c < H; c += blockDim.x) {
    const float a = p * inv_freq[c >> 1];
    row[c] += (c & 1) ? cosf(a) : sinf(a);
  }
}

extern "C" int ti_add_sinusoid(float* x, const int* pos, const float* inv_freq, int M, int H, hipStream_t stream) {
  TI_REQUIRE(M >= 0 && H > 0, "add_sinusoid: bad sizes M=%d H=%d", M, H);
  if (M == 0) return 0;
  add_sinusoid_kernel<<<M, 256, 0, stream>>>(x, pos, inv_freq, H);
  TI_LAUNCH_CHECK();
  return 0;
}

// ------------------------------------------------------------ one vector onto every row
__global__ void add_row_kernel(float* __restrict__ x, const float* __restrict__ v, long n, int H) {
  for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (long)gridDim.x * blockDim.x) x[i] += v[i % H];
}

extern "C" int ti_add_row(float* x, const float* v, int M, int H, hipStream_t stream) {
  TI_REQUIRE(M >= 0 && H > 0, "add_row: bad sizes M=%d H=%d", M, H);
  if (M == 0) return 0;
  const long n = (long)M * H;
  const unsigned blocks = (unsigned)((n + 255) / 256 < 4096 ? (n + 255) / 256 : 4096);
  add_row_kernel<<<blocks, 256, 0, stream>>>(x, v, n, H);
  TI_LAUNCH_CHECK();
  return 0;
}

// ------------------------------------------------------------ xIELU
// act = (p, q), two learned numbers.  z > 0: softplus(p) z^2 + z / 2;  z <= 0: (1/2 + softplus(q))
// (exp(z) - 1 - z) + z / 2.
__device__ __forceinline__ float softplus_f(float z) { return fmaxf(z, 0.f) + log1pf(expf(-fabsf(z))); }
__device__ __forceinline__ float xielu_f(float z, float ap, float an) {
  return z > 0.f ? fmaf(ap * z, z, 0.5f * z) : fmaf(an, expm1f(z) - z, 0.5f * z);
}

template <typename T>
__global__ void xielu_kernel(const float* __restrict__ z, const float* __restrict__ act, T* __restrict__ out, long n) {
  const float ap = softplus_f(act[0]), an = 0.5f + softplus_f(act[1]);
  for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (long)gridDim.x * blockDim.x)
    st<T>(out + i, xielu_f(z[i], ap, an));
}

// The same, eight elements a thread (n a multiple of 8, 16-byte aligned operands).  Rounded to bfloat16 the
// result keeps 8 bits, so exp(z) - 1 from the hardware's exponential (absolute error 1e-7) serves there;
// 32-bit output keeps expm1.
template <typename T>
__global__ void __launch_bounds__(256)
xielu_wide_kernel(const float* __restrict__ z, const float* __restrict__ act, T* __restrict__ out, long n8) {
  const float ap = softplus_f(act[0]), an = 0.5f + softplus_f(act[1]);
  for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < n8; i += (long)gridDim.x * blockDim.x) {
    const float4 a = reinterpret_cast<const float4*>(z)[2 * i], b = reinterpret_cast<const float4*>(z)[2 * i + 1];
    const float v[8] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
    float y[8];
#pragma unroll
    for (int k = 0; k < 8; ++k) {
      if (sizeof(T) == 2) {
        const float e = __builtin_amdgcn_exp2f(fminf(v[k], 0.f) * 1.4426950408889634f) - 1.0f;
        y[k] = v[k] > 0.f ? fmaf(ap * v[k], v[k], 0.5f * v[k]) : fmaf(an, e - v[k], 0.5f * v[k]);
      } else {
        y[k] = xielu_f(v[k], ap, an);
      }
    }
    if (sizeof(T) == 2) {
      reinterpret_cast<uint4*>(out)[i] = make_uint4(pack_bf16x2(y[0], y[1]), pack_bf16x2(y[2], y[3]), pack_bf16x2(y[4], y[5]),
                                                    pack_bf16x2(y[6], y[7]));
    } else {
      reinterpret_cast<float4*>(out)[2 * i] = make_float4(y[0], y[1], y[2], y[3]);
      reinterpret_cast<float4*>(out)[2 * i + 1] = make_float4(y[4], y[5], y[6], y[7]);
    }
  }
}

extern "C" int ti_xielu(int out_dtype, const float* z, const float* act, void* out, long n, hipStream_t stream) {
  TI_REQUIRE(n >= 0, "xielu: bad count %ld", n);
  if (n == 0) return 0;
  TI_REQUIRE(out_dtype == TI_F32 || out_dtype == TI_BF16, "xielu: unknown dtype %d", out_dtype);
  if (n % 8 == 0 && (((uintptr_t)z | (uintptr_t)out) & 15) == 0) {
    const long n8 = n / 8;
    const unsigned blocks = (unsigned)((n8 + 255) / 256 < 8192 ? (n8 + 255) / 256 : 8192);
    if (out_dtype == TI_F32) xielu_wide_kernel<float><<<blocks, 256, 0, stream>>>(z, act, (float*)out, n8);
    else xielu_wide_kernel<bf16_t><<<blocks, 256, 0, stream>>>(z, act, (bf16_t*)out, n8);
    TI_LAUNCH_CHECK();
    return 0;
  }
  const unsigned blocks = (unsigned)((n + 255) / 256 < 16384 ? (n + 255) / 256 : 16384);
  if (out_dtype == TI_F32) xielu_kernel<float><<<blocks, 256, 0, stream>>>(z, act, (float*)out, n);
  else xielu_kernel<bf16_t><<<blocks, 256, 0, stream>>>(z, act, (bf16_t*)out, n);
  TI_LAUNCH_CHECK();
  return 0;
}

// ------------------------------------------------------------ scaled sum into the residual
// x[m, c] += a[m, c] * sa[c] + b[m, c] * sb[c]   (b may be null: one branch; a scale that is null is 1)
__global__ void scaled_add_kernel(float* __restrict__ x, const float* __restrict__ a, const float* __restrict__ sa,
                                  const float* __restrict__ b, const float* __restrict__ sb, long n, int H) {
  for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (long)gridDim.x * blockDim.x) {
    const int c = (int)(i % H);
    float y = a[i] * (sa ? sa[c] : 1.f);
    if (b) y = fmaf(b[i], sb ? sb[c] : 1.f, y);
    x[i] += y;
  }
}

// the same, four channels a thread (H a multiple of 4, 16-byte aligned operands): the same arithmetic, the same bits
__global__ void __launch_bounds__(256)
scaled_add_wide_kernel(float* __restrict__ x, const float* __restrict__ a, const float* __restrict__ sa,
                       const float* __restrict__ b, const float* __restrict__ sb, long n4, int H4) {
  for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < n4; i += (long)gridDim.x * blockDim.x) {
    const int c = (int)(i % H4);
    const float4 one = make_float4(1.f, 1.f, 1.f, 1.f);
    const float4 av = reinterpret_cast<const float4*>(a)[i], s1 = sa ? reinterpret_cast<const float4*>(sa)[c] : one;
    float4 y = make_float4(av.x * s1.x, av.y * s1.y, av.z * s1.z, av.w * s1.w);
    if (b) {
      const float4 bv = reinterpret_cast<const float4*>(b)[i], s2 = sb ? reinterpret_cast<const float4*>(sb)[c] : one;
      y = make_float4(fmaf(bv.x, s2.x, y.x), fmaf(bv.y, s2.y, y.y), fmaf(bv.z, s2.z, y.z), fmaf(bv.w, s2.w, y.w));
    }
    float4 xv = reinterpret_cast<float4*>(x)[i];
    xv.x += y.x;
    xv.y += y.y;
    xv.z += y.z;
    xv.w += y.w;
    reinterpret_cast<float4*>(x)[i] = xv;
  }
}

extern "C" int ti_scaled_add(float* x, const float* a, const float* sa, const float* b, const float* sb, int M, int H,
                             hipStream_t stream) {
  TI_REQUIRE(M >= 0 && H > 0 && a, "scaled_add: bad sizes M=%d H=%d", M, H);
  if (M == 0) return 0;
  const long n = (long)M * H;
  if (H % 4 == 0 && (((uintptr_t)x | (uintptr_t)a | (uintptr_t)sa | (uintptr_t)b | (uintptr_t)sb) & 15) == 0) {
    const long n4 = n / 4;
    const unsigned wide = (unsigned)((n4 + 255) / 256 < 8192 ? (n4 + 255) / 256 : 8192);
    scaled_add_wide_kernel<<<wide, 256, 0, stream>>>(x, a, sa, b, sb, n4, H / 4);
    TI_LAUNCH_CHECK();
    return 0;
  }
  const unsigned blocks = (unsigned)((n + 255) / 256 < 16384 ? (n + 255) / 256 : 16384);
  scaled_add_kernel<<<blocks, 256, 0, stream>>>(x, a, sa, b, sb, n, H);
  TI_LAUNCH_CHECK();
  return 0;
}

// ------------------------------------------------------------ q/k/v split with a query temperature
// qkv f32 [M, n_head dk + n_kv dk + n_kv dv].  q[m] times 1 + coef ln(floor((pos + 1) / every) + 1)
// goes to q_out (T) [M, n_head dk]; k and v into the page of the token's position,
// page = table[slot][pos / P], a page being  K [n_kv][P][dk] | V [n_kv][dv][P]  (values transposed).
template <typename T>
__global__ void qkv_split_write_kernel(const float* __restrict__ qkv, const int* __restrict__ pos,
                                       const int* __restrict__ slot, const int* __restrict__ table, int table_stride,
                                       T* __restrict__ pool, T* __restrict__ q_out, int n_head, int n_kv, int dk, int dv,
                                       int P, float coef, int every) {
  const int m = blockIdx.x;
  const int p = pos[m];
  const int nq = n_head * dk, nk = n_kv * dk, nv = n_kv * dv;
  const float* row = qkv + (size_t)m * (nq + nk + nv);
  const float temp = (coef != 0.f && every > 0) ? 1.f + coef * logf((float)((p + 1) / every) + 1.f) : 1.f;
  // four elements a thread where every run of them is aligned (the products are the same, so are the bits)
  const bool wide = (dk % 4 == 0) && (dv % 4 == 0) && (((uintptr_t)qkv | (uintptr_t)q_out | (uintptr_t)pool) & 15) == 0;
  const int page = table[(size_t)slot[m] * table_stride + p / P];
  const int r = p % P;
  T* base = pool + (size_t)max(page, 0) * ((size_t)n_kv * P * (dk + dv));
  if (wide) {
    for (int e = threadIdx.x * 4; e < nq; e += blockDim.x * 4) {
      const float4 v = *reinterpret_cast<const float4*>(row + e);
      T* dst = q_out + (size_t)m * nq + e;
      st<T>(dst, v.x * temp);
      st<T>(dst + 1, v.y * temp);
      st<T>(dst + 2, v.z * temp);
      st<T>(dst + 3, v.w * temp);
    }
    if (page < 0) return;   // the host reserves pages first; never write astray
    for (int e = threadIdx.x * 4; e < nk; e += blockDim.x * 4) {
      const int h = e / dk, d = e % dk;
      const float4 v = *reinterpret_cast<const float4*>(row + nq + e);
      T* dst = base + ((size_t)h * P + r) * dk + d;
      st<T>(dst, v.x);
      st<T>(dst + 1, v.y);
      st<T>(dst + 2, v.z);
      st<T>(dst + 3, v.w);
    }
  } else {
    for (int e = threadIdx.x; e < nq; e += blockDim.x) st<T>(q_out + (size_t)m * nq + e, row[e] * temp);
    if (page < 0) return;
    for (int e = threadIdx.x; e < nk; e += blockDim.x) {
      const int h = e / dk, d = e % dk;
      st<T>(base + ((size_t)h * P + r) * dk + d, row[nq + e]);
    }
  }
  T* vbase = base + (size_t)n_kv * P * dk;
  for (int e = threadIdx.x; e < nv; e += blockDim.x) {
    const int h = e / dv, d = e % dv;
    st<T>(vbase + ((size_t)h * dv + d) * P + r, row[nq + nk + e]);
  }
}

extern "C" int ti_qkv_split_write(int dtype, const float* qkv, const int* pos, const int* slot, const int* table,
                                  int table_stride, void* pool, void* q_out, int M, int n_head, int n_kv, int dk, int dv,
                                  int page_size, float coef, int every, hipStream_t stream) {
  TI_REQUIRE(n_head > 0 && n_kv > 0 && dk > 0 && dv > 0 && page_size > 0 && table_stride > 0,
             "qkv_split_write: bad sizes heads=%d kv_heads=%d dk=%d dv=%d page=%d table_stride=%d", n_head, n_kv, dk, dv,
             page_size, table_stride);
  if (M == 0) return 0;
  if (dtype == TI_F32)
    qkv_split_write_kernel<float><<<M, 256, 0, stream>>>(qkv, pos, slot, table, table_stride, (float*)pool, (float*)q_out,
                                                         n_head, n_kv, dk, dv, page_size, coef, every);
  else if (dtype == TI_BF16)
    qkv_split_write_kernel<bf16_t><<<M, 256, 0, stream>>>(qkv, pos, slot, table, table_stride, (bf16_t*)pool,
                                                          (bf16_t*)q_out, n_head, n_kv, dk, dv, page_size, coef, every);
  else
    TI_REQUIRE(false, "qkv_split_write: unknown dtype %d", dtype);
  TI_LAUNCH_CHECK();
  return 0;
}

// ------------------------------------------------------------ q/k/v split with biases and a partial rotation
// The same split with what a projection may still owe its rows: a bias on every column of qkv (null: none) and the
// rotation of the first rot_dims entries of every query and key head (entry i with entry i + rot_dims / 2 by the angle
// pos * inv_freq[i]; cosine and sine times mag; rope_table [table_len][rot_dims / 2][2] holds them ready for positions
// below table_len; inv_freq null: none).  Bias and rotation happen in 32-bit, before the query's factor.
__device__ __forceinline__ void rotation_of(const float* __restrict__ inv_freq, const float* __restrict__ rope_table, int table_len,
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

template <typename T>
__global__ void qkv_prep_write_kernel(const float* __restrict__ qkv, const float* __restrict__ bias,
                                      const float* __restrict__ inv_freq, const float* __restrict__ rope_table, int table_len,
                                      float mag, int rot_dims, const int* __restrict__ pos, const int* __restrict__ slot,
                                      const int* __restrict__ table, int table_stride, T* __restrict__ pool, T* __restrict__ q_out,
                                      int n_head, int n_kv, int dk, int dv, int P, float coef, int every) {
  const int m = blockIdx.x;
  const int p = pos[m];
  const int nq = n_head * dk, nk = n_kv * dk, nv = n_kv * dv;
  const float* row = qkv + (size_t)m * (nq + nk + nv);
  const float temp = (coef != 0.f && every > 0) ? 1.f + coef * logf((float)((p + 1) / every) + 1.f) : 1.f;
  const int page = table[(size_t)slot[m] * table_stride + p / P];
  const int r = p % P;
  T* base = pool + (size_t)max(page, 0) * ((size_t)n_kv * P * (dk + dv));
  const int half = inv_freq ? rot_dims / 2 : 0;
  // queries and keys: a thread takes entry d of a head, and with it entry d + half where d is turned (grid (token, pieces of
  // 256 entries): a decoded token's few thousand entries spread over workgroups)
  const int e = blockIdx.y * blockDim.x + threadIdx.x;
  if (e < nq + nk) {
    const int d = e % dk;
    if (d >= half && d < 2 * half) return;      // written by the thread of its partner
    const bool is_q = e < nq;
    float u = row[e] + (bias ? bias[e] : 0.f);
    float w = 0.f;
    if (d < half) {
      w = row[e + half] + (bias ? bias[e + half] : 0.f);
      float c, s;
      rotation_of(inv_freq, rope_table, table_len, mag, half, p, d, &c, &s);
      const float a = u * c - w * s;
      w = w * c + u * s;
      u = a;
    }
    if (is_q) {
      st<T>(q_out + (size_t)m * nq + e, u * temp);
      if (d < half) st<T>(q_out + (size_t)m * nq + e + half, w * temp);
    } else if (page >= 0) {      // the host reserves pages first; never write astray
      const int h = (e - nq) / dk;
      T* dst = base + ((size_t)h * P + r) * dk + d;
      st<T>(dst, u);
      if (d < half) st<T>(dst + half, w);
    }
  }
  else if (e < nq + nk + nv && page >= 0) {
    T* vbase = base + (size_t)n_kv * P * dk;
    const int ev = e - nq - nk;
    const int h = ev / dv, d = ev % dv;
    st<T>(vbase + ((size_t)h * dv + d) * P + r, row[e] + (bias ? bias[e] : 0.f));
  }
}

extern "C" int ti_qkv_prep_write(int dtype, const float* qkv, const float* bias, const float* inv_freq, const float* rope_table,
                                 int table_len, float mag, int rot_dims, const int* pos, const int* slot, const int* table,
                                 int table_stride, void* pool, void* q_out, int M, int n_head, int n_kv, int dk, int dv,
                                 int page_size, float coef, int every, hipStream_t stream) {
  TI_REQUIRE(n_head > 0 && n_kv > 0 && dk > 0 && dv > 0 && page_size > 0 && table_stride > 0,
             "qkv_prep_write: bad sizes heads=%d kv_heads=%d dk=%d dv=%d page=%d table_stride=%d", n_head, n_kv, dk, dv,
             page_size, table_stride);
  TI_REQUIRE(!inv_freq || (rot_dims >= 0 && rot_dims % 2 == 0 && rot_dims <= dk),
             "qkv_prep_write: %d rotated entries do not fit a head of %d (even, at most the head)", rot_dims, dk);
  if (M == 0) return 0;
  const dim3 grid(M, (n_head * dk + n_kv * (dk + dv) + 255) / 256);
  if (dtype == TI_F32)
    qkv_prep_write_kernel<float><<<grid, 256, 0, stream>>>(qkv, bias, inv_freq, rope_table, table_len, mag, rot_dims, pos, slot, table,
                                                        table_stride, (float*)pool, (float*)q_out, n_head, n_kv, dk, dv,
                                                        page_size, coef, every);
  else if (dtype == TI_BF16)
    qkv_prep_write_kernel<bf16_t><<<grid, 256, 0, stream>>>(qkv, bias, inv_freq, rope_table, table_len, mag, rot_dims, pos, slot, table,
                                                         table_stride, (bf16_t*)pool, (bf16_t*)q_out, n_head, n_kv, dk, dv,
                                                         page_size, coef, every);
  else
    TI_REQUIRE(false, "qkv_prep_write: unknown dtype %d", dtype);
  TI_LAUNCH_CHECK();
  return 0;
}

// ------------------------------------------------------------ Dynamic Tanh
// out[r, c] = tanh(alpha x[rows ? rows[r] : r, c]) * w[c] + b[c]: a norm that takes no mean and no variance.  alpha is one
// learned number (device memory).  32-bit arithmetic, rounded once to T.
template <typename T>
__global__ void dyt_kernel(const float* __restrict__ x, const float* __restrict__ alpha, const float* __restrict__ w,
                           const float* __restrict__ b, const int* __restrict__ rows, T* __restrict__ out, int H) {
  const int r = blockIdx.x;
  const float a = alpha[0];
  const float* src = x + (size_t)(rows ? rows[r] : r) * H;
  for (int c = threadIdx.x; c < H; c += blockDim.x) st<T>(out + (size_t)r * H + c, fmaf(tanhf(a * src[c]), w[c], b ? b[c] : 0.f));
}

extern "C" int ti_dyt(int out_dtype, const float* x, const float* alpha, const float* w, const float* b, const int* rows, void* out,
                      int n_rows, int H, hipStream_t stream) {
  TI_REQUIRE(n_rows >= 0 && H > 0 && alpha && w, "dyt: bad sizes rows=%d H=%d", n_rows, H);
  if (n_rows == 0) return 0;
  if (out_dtype == TI_F32) dyt_kernel<float><<<n_rows, 256, 0, stream>>>(x, alpha, w, b, rows, (float*)out, H);
  else if (out_dtype == TI_BF16) dyt_kernel<bf16_t><<<n_rows, 256, 0, stream>>>(x, alpha, w, b, rows, (bf16_t*)out, H);
  else TI_REQUIRE(false, "dyt: unknown dtype %d", out_dtype);
  TI_LAUNCH_CHECK();
  return 0;
}

// ------------------------------------------------------------ gated activations between a feed-forward's products
// z f32 [R, 2F] = [gate | up] (rows ldz floats apart), bias f32 [2F] (null: none) added first.
//   kind 0: out = silu(g) * u
//   kind 1: g = min(g, limit), u = clamp(u, -limit, limit); out = g * sigmoid(alpha g) * (u + 1)
//   kind 2: out = gelu(g) * u, gelu in its tanh form: g / 2 (1 + tanh(sqrt(2 / pi) (g + 0.044715 g^3)))
__device__ __forceinline__ float sigmoid_f(float z) { return 1.0f / (1.0f + expf(-z)); }

template <typename T>
__global__ void gated_act_kernel(const float* __restrict__ z, long ldz, const float* __restrict__ bias, T* __restrict__ out, long R,
                                 int F, int kind, float limit, float alpha) {
  const long n = R * F;
  for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (long)gridDim.x * blockDim.x) {
    const long r = i / F;
    const int f = (int)(i % F);
    float g = z[r * ldz + f], u = z[r * ldz + F + f];
    if (bias) {
      g += bias[f];
      u += bias[F + f];
    }
    float y;
    if (kind == 0) {
      y = g * sigmoid_f(g) * u;
    } else if (kind == 2) {
      y = 0.5f * g * (1.0f + tanhf(0.7978845608028654f * (g + 0.044715f * g * g * g))) * u;
    } else {
      g = fminf(g, limit);
      u = fminf(fmaxf(u, -limit), limit);
      y = g * sigmoid_f(alpha * g) * (u + 1.0f);
    }
    st<T>(out + i, y);
  }
}

extern "C" int ti_gated_act(int out_dtype, const float* z, long ldz, const float* bias, void* out, long R, int F, int kind,
                            float limit, float alpha, hipStream_t stream) {
  TI_REQUIRE(R >= 0 && F > 0 && ldz >= 2L * F && (kind >= 0 && kind <= 2), "gated_act: bad sizes R=%ld F=%d ld=%ld kind=%d", R, F, ldz, kind);
  if (R == 0) return 0;
  const long n = R * F;
  const unsigned blocks = (unsigned)((n + 255) / 256 < 16384 ? (n + 255) / 256 : 16384);
  if (out_dtype == TI_F32) gated_act_kernel<float><<<blocks, 256, 0, stream>>>(z, ldz, bias, (float*)out, R, F, kind, limit, alpha);
  else if (out_dtype == TI_BF16) gated_act_kernel<bf16_t><<<blocks, 256, 0, stream>>>(z, ldz, bias, (bf16_t*)out, R, F, kind, limit, alpha);
  else TI_REQUIRE(false, "gated_act: unknown dtype %d", out_dtype);
  TI_LAUNCH_CHECK();
  return 0;
}

// ------------------------------------------------------------ two streams side by side, rounded
// out T [M, 2H] = [a | b] for the product that mixes the residual with a stream kept from earlier in the step
template <typename T>
__global__ void concat_round_kernel(const float* __restrict__ a, const float* __restrict__ b, T* __restrict__ out, long M, int H) {
  const long n = M * 2 * H;
  for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (long)gridDim.x * blockDim.x) {
    const long m = i / (2 * H);
    const int c = (int)(i % (2 * H));
    st<T>(out + i, c < H ? a[m * H + c] : b[m * H + c - H]);
  }
}

extern "C" int ti_concat_round(int out_dtype, const float* a, const float* b, void* out, int M, int H, hipStream_t stream) {
  TI_REQUIRE(M >= 0 && H > 0, "concat_round: bad sizes M=%d H=%d", M, H);
  if (M == 0) return 0;
  const long n = (long)M * 2 * H;
  const unsigned blocks = (unsigned)((n + 255) / 256 < 16384 ? (n + 255) / 256 : 16384);
  if (out_dtype == TI_F32) concat_round_kernel<float><<<blocks, 256, 0, stream>>>(a, b, (float*)out, M, H);
  else if (out_dtype == TI_BF16) concat_round_kernel<bf16_t><<<blocks, 256, 0, stream>>>(a, b, (bf16_t*)out, M, H);
  else TI_REQUIRE(false, "concat_round: unknown dtype %d", out_dtype);
  TI_LAUNCH_CHECK();
  return 0;
}
