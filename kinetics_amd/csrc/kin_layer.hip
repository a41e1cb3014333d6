// Row-wise kernels of a decoder layer on either side of the attention path:
// RMSNorm with the residual add folded in, the q/k norm + split of the fused QKV
// projection, and the gated activation of the MLP.  All are HBM-bound: every
// element is read once and written once with 16-byte accesses, statistics are
// taken in fp32 inside lane groups (no LDS), and each replaces a chain of
// elementwise launches that would move the same rows through HBM several times.
// F16 = false: bfloat16 tensors; true: float16 (the kin_*_f16 entry points).
#include "kin_common.h"

namespace kin {

// 16-byte chunks one lane keeps in registers: a row of up to LPR * 8 * 16 elements.
constexpr int kNormMaxChunks = 16;

struct NormParams {
  const u32x4* x;
  u32x4* residual;      // [rows, hidden] contiguous, updated in place (RES only)
  const u32x4* weight;  // [hidden]
  u32x4* out;
  int64_t rows;
  int64_t x_stride, out_stride;  // row strides in 16-byte units
  int chunks;                    // hidden / (LPR * 8)
  float eps, inv_hidden;
};

template <bool F16>
__device__ __forceinline__ float sum_sq8(const u32x4& v) {
  float s = 0.f;
  const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const float a = elem_lo<F16>(w[i]), b = elem_hi<F16>(w[i]);
    s = fmaf(a, a, s);
    s = fmaf(b, b, s);
  }
  return s;
}

// round(a + b) per element, as a 16-bit tensor add computes it.
template <bool F16>
__device__ __forceinline__ uint32_t add_x2(uint32_t a, uint32_t b) {
  return f32_to_elem<F16>(elem_lo<F16>(a) + elem_lo<F16>(b)) | (f32_to_elem<F16>(elem_hi<F16>(a) + elem_hi<F16>(b)) << 16);
}

// round((x * r) * w) per element.
template <bool F16>
__device__ __forceinline__ uint32_t scale_x2(uint32_t x, float r, uint32_t w) {
  return f32_to_elem<F16>(elem_lo<F16>(x) * r * elem_lo<F16>(w)) |
         (f32_to_elem<F16>(elem_hi<F16>(x) * r * elem_hi<F16>(w)) << 16);
}

template <int LPR>
__device__ __forceinline__ float group_sum(float x) {
  if constexpr (LPR == 8) return row_sum<8>(x);
  x = row16_sum(x);
  if (LPR == 64) {
    x += __shfl_xor(x, 16);
    x += __shfl_xor(x, 32);
  }
  return x;
}

// LPR lanes (8, 16 or 64) own one row; a 256-thread workgroup covers 256 / LPR rows.
// Lane l holds the 16-byte chunks c * LPR + l, so every load instruction of a
// lane group covers LPR * 16 contiguous bytes.  MAXC bounds the chunks per lane
// (the row stays in registers between the two passes): the smaller
// instantiations need fewer registers, so that a grid of a few thousand rows is
// resident at once instead of running a nearly empty second round.
template <int LPR, int MAXC, bool RES, bool F16>
__global__ __launch_bounds__(256) void rms_norm_kernel(NormParams p) {
  const int sub = threadIdx.x / LPR, l = threadIdx.x % LPR;
  const int64_t row = (int64_t)blockIdx.x * (256 / LPR) + sub;
  if (row >= p.rows) return;  // whole lane groups leave together
  const u32x4* xr = p.x + row * p.x_stride;
  u32x4* rr = RES ? p.residual + row * ((int64_t)p.chunks * LPR) : nullptr;
  u32x4 v[MAXC], r[RES ? MAXC : 1];
#pragma unroll
  for (int c = 0; c < MAXC; ++c) {
    if (c < p.chunks) {
      v[c] = __builtin_nontemporal_load(xr + c * LPR + l);
      if (RES) r[c] = rr[c * LPR + l];
    }
  }
  float ss = 0.f;
#pragma unroll
  for (int c = 0; c < MAXC; ++c) {
    if (c < p.chunks) {
      if (RES) {
        v[c].x = add_x2<F16>(v[c].x, r[c].x);
        v[c].y = add_x2<F16>(v[c].y, r[c].y);
        v[c].z = add_x2<F16>(v[c].z, r[c].z);
        v[c].w = add_x2<F16>(v[c].w, r[c].w);
        rr[c * LPR + l] = v[c];
      }
      ss += sum_sq8<F16>(v[c]);
    }
  }
  ss = group_sum<LPR>(ss);
  const float rinv = rsqrtf(ss * p.inv_hidden + p.eps);
  u32x4* orow = p.out + row * p.out_stride;
#pragma unroll
  for (int c = 0; c < MAXC; ++c) {
    if (c < p.chunks) {
      const u32x4 w = p.weight[c * LPR + l];
      u32x4 o;
      o.x = scale_x2<F16>(v[c].x, rinv, w.x);
      o.y = scale_x2<F16>(v[c].y, rinv, w.y);
      o.z = scale_x2<F16>(v[c].z, rinv, w.z);
      o.w = scale_x2<F16>(v[c].w, rinv, w.w);
      orow[c * LPR + l] = o;
    }
  }
}

struct QkvParams {
  const u32x4* qkv;
  int64_t row_stride;  // 16-byte units
  const u32x4 *q_weight, *k_weight;
  u32x4 *q, *k, *v;
  int batch, hq, hkv;
  float eps;
};

// LPR lanes per head row of LPR * 8 elements (16 lanes for 128, 8 for 64): q and k heads are normalised, v heads
// copied, each to its own contiguous [batch, heads, head_dim] tensor.
template <bool F16, int LPR>
__global__ __launch_bounds__(256) void qkv_norm_split_kernel(QkvParams p) {
  const int heads = p.hq + 2 * p.hkv;
  const int64_t g = (int64_t)blockIdx.x * (256 / LPR) + (threadIdx.x / LPR);
  const int l = threadIdx.x & (LPR - 1);
  if (g >= (int64_t)p.batch * heads) return;
  const int64_t b = g / heads;
  const int j = (int)(g - b * heads);
  u32x4 x = __builtin_nontemporal_load(p.qkv + b * p.row_stride + j * LPR + l);
  u32x4* dst;
  if (j < p.hq + p.hkv) {
    const bool is_q = j < p.hq;
    const float ss = row_sum<LPR>(sum_sq8<F16>(x));
    const float rinv = rsqrtf(ss * (1.0f / (LPR * 8)) + p.eps);
    const u32x4 w = (is_q ? p.q_weight : p.k_weight)[l];
    x.x = scale_x2<F16>(x.x, rinv, w.x);
    x.y = scale_x2<F16>(x.y, rinv, w.y);
    x.z = scale_x2<F16>(x.z, rinv, w.z);
    x.w = scale_x2<F16>(x.w, rinv, w.w);
    dst = is_q ? p.q + (b * p.hq + j) * LPR : p.k + (b * p.hkv + (j - p.hq)) * LPR;
  } else {
    dst = p.v + (b * p.hkv + (j - p.hq - p.hkv)) * LPR;
  }
  dst[l] = x;
}

struct GateParams {
  const u32x4 *gate, *up;
  u32x4* out;
  int64_t rows;
  int64_t gate_stride, up_stride;  // 16-byte units
  int row_chunks;                  // inter / 8
};

// Each activation is rounded to the element format before the product, as the chain
// act(gate) * up over 16-bit tensors rounds it.
template <int ACT, bool F16>
__device__ __forceinline__ float act_rounded(float x) {
  float y;
  if (ACT == KIN_ACT_SILU) y = x / (1.0f + expf(-x));
  else if (ACT == KIN_ACT_GELU) y = 0.5f * x * erfcf(-x * 0.70710678118654752440f);  // = 1 + erf(x / sqrt 2), without its cancellation for x < 0
  else y = fmaxf(x, 0.f);
  return elem_lo<F16>(f32_to_elem<F16>(y));
}

template <int ACT, bool F16>
__device__ __forceinline__ uint32_t gate_x2(uint32_t g, uint32_t u) {
  return f32_to_elem<F16>(act_rounded<ACT, F16>(elem_lo<F16>(g)) * elem_lo<F16>(u)) |
         (f32_to_elem<F16>(act_rounded<ACT, F16>(elem_hi<F16>(g)) * elem_hi<F16>(u)) << 16);
}

template <int ACT, bool F16>
__global__ __launch_bounds__(256) void gated_act_kernel(GateParams p) {
  const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (idx >= p.rows * p.row_chunks) return;
  const int64_t row = idx / p.row_chunks;
  const int c = (int)(idx - row * p.row_chunks);
  const u32x4 g = __builtin_nontemporal_load(p.gate + row * p.gate_stride + c);
  const u32x4 u = __builtin_nontemporal_load(p.up + row * p.up_stride + c);
  u32x4 o;
  o.x = gate_x2<ACT, F16>(g.x, u.x);
  o.y = gate_x2<ACT, F16>(g.y, u.y);
  o.z = gate_x2<ACT, F16>(g.z, u.z);
  o.w = gate_x2<ACT, F16>(g.w, u.w);
  p.out[idx] = o;
}

static int check_row_stride(const char* fn, const char* name, int64_t stride, int width) {
  if (stride < width || stride % 8 != 0)
    return fail(KIN_ERR_BAD_SHAPE, "%s: %s=%lld must be a multiple of 8 and at least the row width %d", fn, name,
                (long long)stride, width);
  return KIN_OK;
}

}  // namespace kin

namespace kin {
static int rms_norm_impl(const char* fn, bool f16, const void* x, void* residual, const void* weight, void* out, int64_t rows,
                         int hidden, int64_t x_row_stride, int64_t out_row_stride, float eps, kin_stream_t stream) {
  if (!x || !weight || !out) return fail(KIN_ERR_NULL_POINTER, "%s: null pointer argument", fn);
  if (rows < 0 || hidden < 1) return fail(KIN_ERR_BAD_SHAPE, "%s: rows=%lld hidden=%d", fn, (long long)rows, hidden);
  int lpr;
  if (hidden % 512 == 0 && hidden <= 512 * kNormMaxChunks) lpr = 64;
  else if (hidden % 128 == 0 && hidden <= 128 * kNormMaxChunks) lpr = 16;
  else if (hidden == 64) lpr = 8;  // qk_norm over head rows of 64 elements
  else
    return fail(KIN_ERR_UNSUPPORTED, "%s: hidden=%d must be 64, a multiple of 128 up to %d or of 512 up to %d", fn, hidden,
                128 * kNormMaxChunks, 512 * kNormMaxChunks);
  if (int st = check_row_stride(fn, "x_row_stride", x_row_stride, hidden)) return st;
  if (int st = check_row_stride(fn, "out_row_stride", out_row_stride, hidden)) return st;
  if (!aligned16(x) || !aligned16(weight) || !aligned16(out) || !aligned16(residual))
    return fail(KIN_ERR_MISALIGNED, "%s: pointers must be 16-byte aligned", fn);
  if (!(eps >= 0.f)) return fail(KIN_ERR_BAD_SHAPE, "%s: eps must be non-negative", fn);
  const int rows_per_wg = 256 / lpr;
  const int64_t grid = (rows + rows_per_wg - 1) / rows_per_wg;
  if (grid > 0x7fffffffLL) return fail(KIN_ERR_UNSUPPORTED, "%s: rows=%lld is too many", fn, (long long)rows);
  if (rows == 0) return KIN_OK;
  NormParams p;
  p.x = static_cast<const u32x4*>(x);
  p.residual = static_cast<u32x4*>(residual);
  p.weight = static_cast<const u32x4*>(weight);
  p.out = static_cast<u32x4*>(out);
  p.rows = rows;
  p.x_stride = x_row_stride / 8;
  p.out_stride = out_row_stride / 8;
  p.chunks = hidden / (lpr * 8);
  p.eps = eps;
  p.inv_hidden = 1.0f / (float)hidden;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const unsigned g = (unsigned)grid;
#define KIN_NORM_LAUNCH(LPR, MAXC)                                                          \
  do {                                                                                      \
    if (f16) {                                                                              \
      if (residual) rms_norm_kernel<LPR, MAXC, true, true><<<g, 256, 0, s>>>(p);            \
      else rms_norm_kernel<LPR, MAXC, false, true><<<g, 256, 0, s>>>(p);                    \
    } else {                                                                                \
      if (residual) rms_norm_kernel<LPR, MAXC, true, false><<<g, 256, 0, s>>>(p);           \
      else rms_norm_kernel<LPR, MAXC, false, false><<<g, 256, 0, s>>>(p);                   \
    }                                                                                       \
  } while (0)
  if (lpr == 64) {
    if (p.chunks <= 4) KIN_NORM_LAUNCH(64, 4);
    else if (p.chunks <= 8) KIN_NORM_LAUNCH(64, 8);
    else KIN_NORM_LAUNCH(64, 16);
  } else if (lpr == 8) {
    KIN_NORM_LAUNCH(8, 1);
  } else {
    if (p.chunks <= 1) KIN_NORM_LAUNCH(16, 1);
    else if (p.chunks <= 4) KIN_NORM_LAUNCH(16, 4);
    else KIN_NORM_LAUNCH(16, 16);
  }
#undef KIN_NORM_LAUNCH
  return check_hip(hipGetLastError(), "rms_norm_kernel launch");
}

static int qkv_norm_split_impl(const char* fn, bool f16, const void* qkv, int64_t qkv_row_stride, const void* q_weight,
                               const void* k_weight, float eps, void* q, void* k, void* v, int batch, int num_q_heads,
                               int num_kv_heads, int head_dim, kin_stream_t stream) {
  if (!qkv || !q_weight || !k_weight || !q || !k || !v) return fail(KIN_ERR_NULL_POINTER, "%s: null pointer argument", fn);
  if (batch < 0 || num_q_heads < 1 || num_kv_heads < 1)
    return fail(KIN_ERR_BAD_SHAPE, "%s: batch=%d num_q_heads=%d num_kv_heads=%d", fn, batch, num_q_heads, num_kv_heads);
  if (!supported_head_dim(head_dim))
    return fail(KIN_ERR_UNSUPPORTED, "%s: head_dim=%d, only %d and %d are built", fn, head_dim, kHeadDimSmall, kHeadDim);
  const int64_t heads = (int64_t)num_q_heads + 2 * (int64_t)num_kv_heads;
  if (heads * head_dim > 0x7fffffffLL) return fail(KIN_ERR_UNSUPPORTED, "%s: too many heads", fn);
  if (int st = check_row_stride(fn, "qkv_row_stride", qkv_row_stride, (int)(heads * head_dim))) return st;
  if (!aligned16(qkv) || !aligned16(q_weight) || !aligned16(k_weight) || !aligned16(q) || !aligned16(k) || !aligned16(v))
    return fail(KIN_ERR_MISALIGNED, "%s: pointers must be 16-byte aligned", fn);
  if (!(eps >= 0.f)) return fail(KIN_ERR_BAD_SHAPE, "%s: eps must be non-negative", fn);
  const int rows_per_block = 256 / (head_dim / 8);
  const int64_t grid = ((int64_t)batch * heads + rows_per_block - 1) / rows_per_block;
  if (grid > 0x7fffffffLL) return fail(KIN_ERR_UNSUPPORTED, "%s: batch*heads is too large", fn);
  if (batch == 0) return KIN_OK;
  QkvParams p;
  p.qkv = static_cast<const u32x4*>(qkv);
  p.row_stride = qkv_row_stride / 8;
  p.q_weight = static_cast<const u32x4*>(q_weight);
  p.k_weight = static_cast<const u32x4*>(k_weight);
  p.q = static_cast<u32x4*>(q);
  p.k = static_cast<u32x4*>(k);
  p.v = static_cast<u32x4*>(v);
  p.batch = batch;
  p.hq = num_q_heads;
  p.hkv = num_kv_heads;
  p.eps = eps;
  hipStream_t hs = static_cast<hipStream_t>(stream);
  if (head_dim == kHeadDimSmall) {
    if (f16) qkv_norm_split_kernel<true, 8><<<(unsigned)grid, 256, 0, hs>>>(p);
    else qkv_norm_split_kernel<false, 8><<<(unsigned)grid, 256, 0, hs>>>(p);
  } else {
    if (f16) qkv_norm_split_kernel<true, 16><<<(unsigned)grid, 256, 0, hs>>>(p);
    else qkv_norm_split_kernel<false, 16><<<(unsigned)grid, 256, 0, hs>>>(p);
  }
  return check_hip(hipGetLastError(), "qkv_norm_split_kernel launch");
}

static int gated_act_impl(const char* fn, bool f16, const void* gate, const void* up, void* out, int64_t rows, int inter,
                          int64_t gate_row_stride, int64_t up_row_stride, int act, kin_stream_t stream) {
  if (!gate || !up || !out) return fail(KIN_ERR_NULL_POINTER, "%s: null pointer argument", fn);
  if (rows < 0 || inter < 1 || inter % 8 != 0)
    return fail(KIN_ERR_BAD_SHAPE, "%s: rows=%lld inter=%d (inter must be a positive multiple of 8)", fn, (long long)rows, inter);
  if (int st = check_row_stride(fn, "gate_row_stride", gate_row_stride, inter)) return st;
  if (int st = check_row_stride(fn, "up_row_stride", up_row_stride, inter)) return st;
  if (!aligned16(gate) || !aligned16(up) || !aligned16(out))
    return fail(KIN_ERR_MISALIGNED, "%s: pointers must be 16-byte aligned", fn);
  if (act != KIN_ACT_SILU && act != KIN_ACT_GELU && act != KIN_ACT_RELU)
    return fail(KIN_ERR_UNSUPPORTED, "%s: act=%d is not one of KIN_ACT_SILU/GELU/RELU", fn, act);
  GateParams p;
  p.gate = static_cast<const u32x4*>(gate);
  p.up = static_cast<const u32x4*>(up);
  p.out = static_cast<u32x4*>(out);
  p.rows = rows;
  p.gate_stride = gate_row_stride / 8;
  p.up_stride = up_row_stride / 8;
  p.row_chunks = inter / 8;
  const int64_t grid = (rows * p.row_chunks + 255) / 256;
  if (grid > 0x7fffffffLL) return fail(KIN_ERR_UNSUPPORTED, "%s: rows*inter is too large", fn);
  if (rows == 0) return KIN_OK;
  hipStream_t s = static_cast<hipStream_t>(stream);
#define KIN_GATE_LAUNCH(ACT)                                                       \
  do {                                                                             \
    if (f16) gated_act_kernel<ACT, true><<<(unsigned)grid, 256, 0, s>>>(p);        \
    else gated_act_kernel<ACT, false><<<(unsigned)grid, 256, 0, s>>>(p);           \
  } while (0)
  if (act == KIN_ACT_SILU) KIN_GATE_LAUNCH(KIN_ACT_SILU);
  else if (act == KIN_ACT_GELU) KIN_GATE_LAUNCH(KIN_ACT_GELU);
  else KIN_GATE_LAUNCH(KIN_ACT_RELU);
#undef KIN_GATE_LAUNCH
  return check_hip(hipGetLastError(), "gated_act_kernel launch");
}
}  // namespace kin

extern "C" {

int kin_rms_norm(const void* x, void* residual, const void* weight, void* out, int64_t rows, int hidden,
                 int64_t x_row_stride, int64_t out_row_stride, float eps, kin_stream_t stream) {
  return kin::rms_norm_impl("kin_rms_norm", false, x, residual, weight, out, rows, hidden, x_row_stride, out_row_stride, eps,
                            stream);
}
int kin_rms_norm_f16(const void* x, void* residual, const void* weight, void* out, int64_t rows, int hidden,
                     int64_t x_row_stride, int64_t out_row_stride, float eps, kin_stream_t stream) {
  return kin::rms_norm_impl("kin_rms_norm_f16", true, x, residual, weight, out, rows, hidden, x_row_stride, out_row_stride,
                            eps, stream);
}
int kin_qkv_norm_split(const void* qkv, int64_t qkv_row_stride, const void* q_weight, const void* k_weight, float eps,
                       void* q, void* k, void* v, int batch, int num_q_heads, int num_kv_heads, int head_dim,
                       kin_stream_t stream) {
  return kin::qkv_norm_split_impl("kin_qkv_norm_split", false, qkv, qkv_row_stride, q_weight, k_weight, eps, q, k, v, batch,
                                  num_q_heads, num_kv_heads, head_dim, stream);
}
int kin_qkv_norm_split_f16(const void* qkv, int64_t qkv_row_stride, const void* q_weight, const void* k_weight, float eps,
                           void* q, void* k, void* v, int batch, int num_q_heads, int num_kv_heads, int head_dim,
                           kin_stream_t stream) {
  return kin::qkv_norm_split_impl("kin_qkv_norm_split_f16", true, qkv, qkv_row_stride, q_weight, k_weight, eps, q, k, v, batch,
                                  num_q_heads, num_kv_heads, head_dim, stream);
}
int kin_gated_act(const void* gate, const void* up, void* out, int64_t rows, int inter, int64_t gate_row_stride,
                  int64_t up_row_stride, int act, kin_stream_t stream) {
  return kin::gated_act_impl("kin_gated_act", false, gate, up, out, rows, inter, gate_row_stride, up_row_stride, act, stream);
}
int kin_gated_act_f16(const void* gate, const void* up, void* out, int64_t rows, int inter, int64_t gate_row_stride,
                      int64_t up_row_stride, int act, kin_stream_t stream) {
  return kin::gated_act_impl("kin_gated_act_f16", true, gate, up, out, rows, inter, gate_row_stride, up_row_stride, act,
                             stream);
}

}  // extern "C"
