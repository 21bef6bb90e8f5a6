// libti_gated_attention: softmax attention with what sits around it in gated layers, for any sizes up to 256 and both
// storage types (the float32 path of such layers, and the path of sizes the matrix-core kernels do not take).
//
//   preparation   from the 32-bit sums of one stacked projection [q | k | v | ...]: per-head RMS norms of q and k (a weight
//                 of the head's size shared by all heads; before the rotation), rotation of the first rot_dims entries of
//                 every query and key head, values that are the keys as projected (no v columns), values mixed with the
//                 values another layer left for the same tokens, q out, k and v into the pages
//   attention     causal softmax over the pages with a learned number a head in the denominator (a sink: no key, no value,
//                 not scaled) and a sigmoid gate on the output, one number an entry or one a head, read from the 32-bit sums
//
// A page is K [n_kv][P][dk] | V [n_kv][dvr][P], as the other attention kernels of keys and values of their own sizes read it;
// dvr >= dv rows a value head: rows beyond dv are written as zeros (values padded to the keys' size, so that kernels that
// hold keys and values of one size can read the pages).
#include "common.h"
#include "tinyinfer_kernels.h"

TI_ERROR_API

#define GA_MAX_DPL 4      // entries of a head a lane holds: heads up to 256

__device__ __forceinline__ void ga_rotation(const float* __restrict__ inv_freq, const float* __restrict__ rope_table, int table_len,
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

// grid (token, heads + kv heads), a wavefront each: a query head, or a key head with its value head
template <typename T>
__global__ void __launch_bounds__(TI_WAVE)
gated_qkv_prep_kernel(const float* __restrict__ proj, int ld, int off_q, int off_k, int off_v, const float* __restrict__ q_w,
                      const float* __restrict__ k_w, float eps, const float* __restrict__ inv_freq,
                      const float* __restrict__ rope_table, int table_len, float mag, int rot_dims, int mix_mode,
                      const float* __restrict__ mix_lambda, float* __restrict__ v_kept, const int* __restrict__ pos,
                      const int* __restrict__ slot, const int* __restrict__ table, int table_stride, T* __restrict__ pool,
                      T* __restrict__ q_out, int n_head, int n_kv, int dk, int dv, int dvr, int P) {
  __shared__ float s_h[256];
  const int m = blockIdx.x, unit = blockIdx.y, lane = threadIdx.x;
  const int p = pos[m];
  const bool is_q = unit < n_head;
  const int h = is_q ? unit : unit - n_head;
  const float* row = proj + (size_t)m * ld;
  const float* src = row + (is_q ? off_q : off_k) + (size_t)h * dk;
  const float* nw = is_q ? q_w : k_w;
  const int page = table[(size_t)slot[m] * table_stride + p / P];
  const int r = p % P;
  T* base = pool + (size_t)max(page, 0) * ((size_t)n_kv * P * (dk + dvr));
  float v[GA_MAX_DPL];
  float ss = 0.f;
#pragma unroll
  for (int i = 0; i < GA_MAX_DPL; ++i) {
    const int d = lane + i * TI_WAVE;
    v[i] = d < dk ? src[d] : 0.f;
    ss = fmaf(v[i], v[i], ss);
  }
  if (!is_q && off_v < 0 && page >= 0) {
    // the values are the keys as projected: before norm and rotation
    T* vbase = base + (size_t)n_kv * P * dk + (size_t)h * dvr * P + r;
#pragma unroll
    for (int i = 0; i < GA_MAX_DPL; ++i) {
      const int d = lane + i * TI_WAVE;
      if (d < dv) st<T>(vbase + (size_t)d * P, v[i]);
    }
  }
  if (nw) {
    const float inv = 1.0f / sqrtf(group_sum<TI_WAVE>(ss) / (float)dk + eps);
#pragma unroll
    for (int i = 0; i < GA_MAX_DPL; ++i) {
      const int d = lane + i * TI_WAVE;
      if (d < dk) v[i] = v[i] * inv * nw[d];
    }
  }
  const int half = inv_freq ? rot_dims / 2 : 0;
  if (half > 0) {
#pragma unroll
    for (int i = 0; i < GA_MAX_DPL; ++i) {
      const int d = lane + i * TI_WAVE;
      if (d < dk) s_h[d] = v[i];
    }
    __syncthreads();
#pragma unroll
    for (int i = 0; i < GA_MAX_DPL; ++i) {
      const int d = lane + i * TI_WAVE;
      if (d < 2 * half) {
        float c, s;
        ga_rotation(inv_freq, rope_table, table_len, mag, half, p, d < half ? d : d - half, &c, &s);
        v[i] = d < half ? s_h[d] * c - s_h[d + half] * s : s_h[d] * c + s_h[d - half] * s;
      }
    }
  }
  if (is_q) {
    T* dst = q_out + ((size_t)m * n_head + h) * dk;
#pragma unroll
    for (int i = 0; i < GA_MAX_DPL; ++i) {
      const int d = lane + i * TI_WAVE;
      if (d < dk) st<T>(dst + d, v[i]);
    }
    return;
  }
  if (page >= 0) {      // the host reserves pages first; never write astray
    T* dst = base + ((size_t)h * P + r) * dk;
#pragma unroll
    for (int i = 0; i < GA_MAX_DPL; ++i) {
      const int d = lane + i * TI_WAVE;
      if (d < dk) st<T>(dst + d, v[i]);
    }
  }
  if (off_v < 0) return;
  const float* vs = row + off_v + (size_t)h * dv;
  float* kept = v_kept ? v_kept + ((size_t)m * n_kv + h) * dv : nullptr;
  const float lam = mix_mode == 2 ? mix_lambda[0] : 0.f;
  T* vbase = base + (size_t)n_kv * P * dk + (size_t)h * dvr * P + r;
  for (int d = lane; d < dvr; d += TI_WAVE) {
    float x = 0.f;                                                    // rows beyond the value's size: zeros
    if (d < dv) {
      x = vs[d];
      if (mix_mode == 1) kept[d] = x;                                 // the layer whose values the later ones mix in
      else if (mix_mode == 2) x = fmaf(lam, kept[d], (1.0f - lam) * x);
    }
    if (page >= 0) st<T>(vbase + (size_t)d * P, x);
  }
}

extern "C" int ti_gated_qkv_prep(int dtype, const float* proj, int ld, int off_q, int off_k, int off_v, const float* q_w,
                                 const float* k_w, float eps, const float* inv_freq, const float* rope_table, int table_len,
                                 float mag, int rot_dims, int mix_mode, const float* mix_lambda, float* v_kept, const int* pos,
                                 const int* slot, const int* table, int table_stride, void* pool, void* q_out, int M, int n_head,
                                 int n_kv, int dk, int dv, int dv_rows, int page_size, hipStream_t stream) {
  const int dvr = dv_rows > 0 ? dv_rows : dv;
  TI_REQUIRE(n_head > 0 && n_kv > 0 && dk > 0 && dk <= 256 && dv > 0 && dv <= 256 && dvr >= dv && dvr <= 256 && page_size > 0 &&
                 table_stride > 0 && n_head + n_kv <= 65535,
             "gated_qkv_prep: bad sizes heads=%d kv_heads=%d dk=%d dv=%d (%d rows) page=%d", n_head, n_kv, dk, dv, dvr, page_size);
  TI_REQUIRE(!inv_freq || (rot_dims >= 0 && rot_dims % 2 == 0 && rot_dims <= dk),
             "gated_qkv_prep: %d rotated entries do not fit a head of %d (even, at most the head)", rot_dims, dk);
  TI_REQUIRE(off_v >= 0 || dv == dk, "gated_qkv_prep: values that are the keys have the keys' size (%d, not %d)", dk, dv);
  TI_REQUIRE(mix_mode == 0 || (off_v >= 0 && v_kept && (mix_mode == 1 || (mix_mode == 2 && mix_lambda))),
             "gated_qkv_prep: mixing values (mode %d) needs value columns, the kept values and the factor", mix_mode);
  TI_REQUIRE(off_q >= 0 && off_k >= 0 && off_q + n_head * dk <= ld && off_k + n_kv * dk <= ld && (off_v < 0 || off_v + n_kv * dv <= ld),
             "gated_qkv_prep: the columns do not lie inside rows of %d", ld);
  if (M == 0) return 0;
  const dim3 grid(M, n_head + n_kv);
  if (dtype == TI_F32)
    gated_qkv_prep_kernel<float><<<grid, TI_WAVE, 0, stream>>>(proj, ld, off_q, off_k, off_v, q_w, k_w, eps, inv_freq, rope_table,
                                                               table_len, mag, rot_dims, mix_mode, mix_lambda, v_kept, pos, slot,
                                                               table, table_stride, (float*)pool, (float*)q_out, n_head, n_kv, dk,
                                                               dv, dvr, page_size);
  else if (dtype == TI_BF16)
    gated_qkv_prep_kernel<bf16_t><<<grid, TI_WAVE, 0, stream>>>(proj, ld, off_q, off_k, off_v, q_w, k_w, eps, inv_freq, rope_table,
                                                                table_len, mag, rot_dims, mix_mode, mix_lambda, v_kept, pos, slot,
                                                                table, table_stride, (bf16_t*)pool, (bf16_t*)q_out, n_head, n_kv,
                                                                dk, dv, dvr, page_size);
  else
    TI_REQUIRE(false, "gated_qkv_prep: unknown dtype %d", dtype);
  TI_LAUNCH_CHECK();
  return 0;
}

// The gate on its own, behind attention kernels that do not take it in: out[m, h dv + d] = src[m, h src_dv + d] times
// sigmoid(gate[m, h dv + d] or gate[m, h]) (gate null: times one).  src_dv > dv: the heads of src are padded and come out packed;
// src may be out where src_dv = dv.
template <typename T>
__global__ void sigmoid_gate_kernel(const T* __restrict__ src, int src_dv, T* __restrict__ out, const float* __restrict__ gate,
                                    int gate_ld, int gate_mode, long n, int n_head, int dv) {
  const int W = n_head * dv;
  for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (long)gridDim.x * blockDim.x) {
    const long m = i / W;
    const int c = (int)(i % W), h = c / dv;
    float y = ld<T>(src + m * ((long)n_head * src_dv) + (long)h * src_dv + (c - h * dv));
    if (gate) y *= 1.0f / (1.0f + expf(-gate[m * gate_ld + (gate_mode == 1 ? c : h)]));
    st<T>(out + i, y);
  }
}

extern "C" int ti_sigmoid_gate(int dtype, const void* src, int src_dv, void* out, const float* gate, int gate_ld, int gate_mode, int M,
                               int n_head, int dv, hipStream_t stream) {
  TI_REQUIRE(M >= 0 && n_head > 0 && dv > 0 && src_dv >= dv && (src != out || src_dv == dv) &&
                 (!gate || (gate_mode == 1 && gate_ld >= n_head * dv) || (gate_mode == 2 && gate_ld >= n_head)),
             "sigmoid_gate: bad sizes M=%d heads=%d dv=%d (from %d) gate mode %d in rows of %d", M, n_head, dv, src_dv, gate_mode, gate_ld);
  if (M == 0) return 0;
  const long n = (long)M * n_head * dv;
  const unsigned blocks = (unsigned)((n + 255) / 256 < 16384 ? (n + 255) / 256 : 16384);
  if (dtype == TI_F32)
    sigmoid_gate_kernel<float><<<blocks, 256, 0, stream>>>((const float*)src, src_dv, (float*)out, gate, gate_ld, gate_mode, n, n_head, dv);
  else if (dtype == TI_BF16)
    sigmoid_gate_kernel<bf16_t><<<blocks, 256, 0, stream>>>((const bf16_t*)src, src_dv, (bf16_t*)out, gate, gate_ld, gate_mode, n, n_head, dv);
  else
    TI_REQUIRE(false, "sigmoid_gate: unknown dtype %d", dtype);
  TI_LAUNCH_CHECK();
  return 0;
}

// ------------------------------------------------------------------------------------------------
// A workgroup per (row, head): sixteen groups of sixteen lanes, group g the keys at positions g, g + 16, ... with a running
// softmax each, merged in a fixed order (a key's group depends on its position alone, so every cut of the same tokens takes
// the same sums in the same order).  The sink joins the merge as a share of its own with maximum sink[h], weight 1 and no
// values.  gate (null: none): rows of gate_ld floats; gate_mode 1: entry h * dv + d of the row, 2: entry h.
#define GA_LANES 16
#define GA_GROUPS 16

template <typename T, int DPL>
__global__ void __launch_bounds__(256)
gated_attention_kernel(const T* __restrict__ q, const T* __restrict__ pool, const int* __restrict__ table, int table_stride,
                       const int* __restrict__ pos, const int* __restrict__ slot, const float* __restrict__ sink,
                       const float* __restrict__ gate, int gate_ld, int gate_mode, T* __restrict__ out, int n_head, int n_kv,
                       int dk, int dv, int dvr, int P, float scale, int window) {
  constexpr int HD = DPL * GA_LANES;
  __shared__ float s_o[GA_GROUPS][HD];
  __shared__ float s_m[GA_GROUPS], s_l[GA_GROUPS];
  const int m = blockIdx.x, h = blockIdx.y;
  const int g = threadIdx.x / GA_LANES, lane = threadIdx.x % GA_LANES;
  const int kvh = h / (n_head / n_kv);
  const int p_q = pos[m];
  const int lo = (window > 0 && p_q - window + 1 > 0) ? p_q - window + 1 : 0;
  const int* tab = table + (size_t)slot[m] * table_stride;
  const size_t page_elems = (size_t)n_kv * P * (dk + dvr);
  const size_t k_off = (size_t)kvh * P * dk;
  const size_t v_off = (size_t)n_kv * P * dk + (size_t)kvh * dvr * P;

  float qv[DPL], o[DPL];
  const T* qh = q + ((size_t)m * n_head + h) * dk;
#pragma unroll
  for (int i = 0; i < DPL; ++i) {
    const int d = lane + i * GA_LANES;
    qv[i] = d < dk ? ld<T>(qh + d) : 0.f;
    o[i] = 0.f;
  }
  float mx = -INFINITY, l = 0.f;
  for (int p = lo - lo % GA_GROUPS + g; p <= p_q; p += GA_GROUPS) {
    if (p < lo) continue;
    const int page = tab[p / P];
    if (page < 0) continue;
    const T* kp = pool + (size_t)page * page_elems + k_off + (size_t)(p % P) * dk;
    const T* vp = pool + (size_t)page * page_elems + v_off + (p % P);
    float s = 0.f;
#pragma unroll
    for (int i = 0; i < DPL; ++i) {
      const int d = lane + i * GA_LANES;
      if (d < dk) s = fmaf(qv[i], ld<T>(kp + d), s);
    }
    s = group_sum<GA_LANES>(s) * scale;
    const float m_new = fmaxf(mx, s);
    const float alpha = expf(mx - m_new);
    const float w = expf(s - m_new);
    l = l * alpha + w;
#pragma unroll
    for (int i = 0; i < DPL; ++i) {
      const int d = lane + i * GA_LANES;
      if (d < dv) o[i] = o[i] * alpha + w * ld<T>(vp + (size_t)d * P);
    }
    mx = m_new;
  }
#pragma unroll
  for (int i = 0; i < DPL; ++i) s_o[g][lane + i * GA_LANES] = o[i];
  if (lane == 0) {
    s_m[g] = mx;
    s_l[g] = l;
  }
  __syncthreads();
  const float sk = sink ? sink[h] : -INFINITY;
  const float* grow = gate ? gate + (size_t)m * gate_ld : nullptr;
  for (int d = threadIdx.x; d < dv; d += 256) {
    float mm = sk;
#pragma unroll
    for (int j = 0; j < GA_GROUPS; ++j) mm = fmaxf(mm, s_m[j]);
    float lt = sink ? expf(sk - mm) : 0.f, acc = 0.f;
#pragma unroll
    for (int j = 0; j < GA_GROUPS; ++j) {
      const float w = (s_m[j] == -INFINITY) ? 0.f : expf(s_m[j] - mm);
      lt += s_l[j] * w;
      acc += s_o[j][d] * w;
    }
    float y = acc / lt;
    if (grow) {
      const float z = grow[gate_mode == 1 ? h * dv + d : h];
      y *= 1.0f / (1.0f + expf(-z));
    }
    st<T>(out + ((size_t)m * n_head + h) * dv + d, y);
  }
}

template <typename T>
static int launch_gated(int dpl, dim3 grid, const void* q, const void* pool, const int* table, int table_stride, const int* pos,
                        const int* slot, const float* sink, const float* gate, int gate_ld, int gate_mode, void* out, int n_head,
                        int n_kv, int dk, int dv, int dvr, int P, float scale, int window, hipStream_t stream) {
#define GA_CASE(D)                                                                                                       \
  case D:                                                                                                                \
    gated_attention_kernel<T, D><<<grid, 256, 0, stream>>>((const T*)q, (const T*)pool, table, table_stride, pos, slot, sink, \
                                                           gate, gate_ld, gate_mode, (T*)out, n_head, n_kv, dk, dv, dvr, P, scale, \
                                                           window);                                                      \
    break;
  switch (dpl) {
    GA_CASE(1) GA_CASE(2) GA_CASE(3) GA_CASE(4) GA_CASE(5) GA_CASE(6) GA_CASE(7) GA_CASE(8)
    GA_CASE(9) GA_CASE(10) GA_CASE(11) GA_CASE(12) GA_CASE(13) GA_CASE(14) GA_CASE(15) GA_CASE(16)
    default:
      return 1;
  }
#undef GA_CASE
  return 0;
}

// q: [M, n_head, dk], out: [M, n_head, dv] in T
extern "C" int ti_gated_attention_rows(int dtype, const void* q, const void* pool, const int* table, int table_stride,
                                       const int* pos, const int* slot, const float* sink, const float* gate, int gate_ld,
                                       int gate_mode, void* out, int M, int n_head, int n_kv, int dk, int dv, int dv_rows, int page_size,
                                       float scale, int window, hipStream_t stream) {
  const int dvr = dv_rows > 0 ? dv_rows : dv;
  TI_REQUIRE(dvr >= dv && dvr <= 256, "gated attention: %d rows a value head do not hold values of %d", dvr, dv);
  TI_REQUIRE(dk >= 1 && dk <= 256 && dv >= 1 && dv <= 256, "gated attention: key size %d / value size %d are not served (up to 256)",
             dk, dv);
  TI_REQUIRE(n_head > 0 && n_kv > 0 && n_head % n_kv == 0 && n_head <= 65535, "gated attention: heads %d / kv_heads %d", n_head, n_kv);
  TI_REQUIRE(page_size > 0 && table_stride > 0, "gated attention: bad page_size %d / table_stride %d", page_size, table_stride);
  TI_REQUIRE(!gate || ((gate_mode == 1 && gate_ld >= n_head * dv) || (gate_mode == 2 && gate_ld >= n_head)),
             "gated attention: the gate (mode %d) does not fit rows of %d", gate_mode, gate_ld);
  if (M == 0) return 0;
  dim3 grid(M, n_head);
  const int big = dk > dv ? dk : dv;
  const int dpl = (big + GA_LANES - 1) / GA_LANES;
  int rc;
  if (dtype == TI_F32)
    rc = launch_gated<float>(dpl, grid, q, pool, table, table_stride, pos, slot, sink, gate, gate_ld, gate_mode, out, n_head, n_kv, dk,
                             dv, dvr, page_size, scale, window, stream);
  else if (dtype == TI_BF16)
    rc = launch_gated<bf16_t>(dpl, grid, q, pool, table, table_stride, pos, slot, sink, gate, gate_ld, gate_mode, out, n_head, n_kv,
                              dk, dv, dvr, page_size, scale, window, stream);
  else
    TI_REQUIRE(false, "gated attention: unknown dtype %d", dtype);
  TI_REQUIRE(rc == 0, "gated attention: no kernel for sizes %d / %d", dk, dv);
  TI_LAUNCH_CHECK();
  return 0;
}
