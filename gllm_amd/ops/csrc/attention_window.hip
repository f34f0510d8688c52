// Windowed attention with kept first tokens and a softmax sink, gfx950.
//
// Dtype-generic (T = bf16 or fp32 for q/k/v/cache/out; scores, softmax
// and accumulation are fp32 always) and shape-generic: any per-head
// query/key size D, value size Dv != D, any GQA ratio, any page size.
//
//   qk_norm_rope_store  per-head RMS norm of q and k (plain weight or
//                       none), rotary on the first rot_dims dims with a
//                       per-pair frequency table (YaRN or plain; angle =
//                       pos * f in fp64, so long positions lose
//                       nothing; pairs (2i, 2i+1) or, half layout,
//                       (i, i + rot_dims/2)), norm before or after the
//                       rotation (or no norm at all), then q in place
//                       and k, v scattered into the paged cache (v may
//                       be k as projected; with a value frequency table
//                       v is turned by its own position over all of Dv);
//                       span norm: ONE RMS over all heads of the token's
//                       q (k) row with row-sized weights; unit values:
//                       each value head divided by its RMS on the way in.
//                       The span form runs one workgroup per token
//                       (qk_span_rope_store_kernel) while the rows fit LDS
//   window_attention    ragged batch (prompt portions beside single
//                       decode tokens) over the paged cache: position i
//                       sees j <= i with i - j < window or j < keep_first;
//                       optional sink: softmax denominator 1 + sum exp(s)
//                       (a score-0 key with no value) or, with a per-head
//                       table, exp(sink_h) + sum exp(s); optional tanh cap
//                       cap * tanh(s / cap) on the scaled scores;
//                       optional fused sigmoid output gate
//   rotate_scale_rows   turn the pairs of every head row by sign * pos * f
//                       and scale (the inverse turn of rotated values)
//   rms_weight_store    weighted RMS norm of a row, also scattered into a
//                       single-head paged cache (a low-rank latent)
//
// A layer that shares another layer's keys and values calls
// qk_norm_rope_store with no k/v and attends over the owner's cache.

#include <torch/extension.h>
#include <ATen/cuda/CUDAContext.h>
#include "common.h"

namespace {

constexpr int QK_BLOCK = 64;
constexpr int ATT_BLOCK = 256;

// ------------------------------------------------------------------
// grid (tokens, H + 2G): y < H query head (in place), y < H+G key head
// (norm + rotary -> cache), else value head (plain copy -> cache)
template <typename T>
__global__ __launch_bounds__(QK_BLOCK) void qk_norm_rope_store_kernel(
    T *__restrict__ q, long q_stride, const T *__restrict__ k, long k_stride,
    const T *__restrict__ v, long v_stride, const T *__restrict__ q_w,
    const T *__restrict__ k_w, const long *__restrict__ positions,
    const long *__restrict__ slot_mapping, const double *__restrict__ freqs,
    float mag, int rot_dims, T *__restrict__ k_cache, T *__restrict__ v_cache,
    int H, int G, int D, int Dv, float eps, int half_layout, int norm_last,
    int do_norm, const double *__restrict__ v_freqs, int norm_span,
    int v_unit, T *__restrict__ q_out, long q_out_stride) {
  extern __shared__ float buf[];
  const int t = blockIdx.x;
  const int y = blockIdx.y;
  const int lane = threadIdx.x;
  if (y >= H + G) {  // value copy, or value turned by its own position
    const int g = y - H - G;
    const long slot = slot_mapping[t];
    const T *src = v + (long)t * v_stride + (long)g * Dv;
    T *dst = v_cache + (slot * G + g) * Dv;
    if (v_unit) {  // unit RMS per head (no rotation on this path)
      float vs = 0.f;
      for (int i = lane; i < Dv; i += QK_BLOCK) {
        const float x = ScalarOps<T>::to_f32(src[i]);
        vs += x * x;
      }
      const float vinv = 1.0f / sqrtf(wave_reduce_sum(vs) / Dv + eps);
      for (int i = lane; i < Dv; i += QK_BLOCK)
        dst[i] = ScalarOps<T>::from_f32(ScalarOps<T>::to_f32(src[i]) * vinv);
      return;
    }
    if (v_freqs == nullptr) {
      for (int i = lane; i < Dv; i += QK_BLOCK) dst[i] = src[i];
      return;
    }
    const double vpos = (double)positions[t];
    const int vhalf = Dv / 2;
    for (int p = lane; p < vhalf; p += QK_BLOCK) {
      double sn, cs;
      sincos(vpos * v_freqs[p], &sn, &cs);
      const float c = (float)cs, s = (float)sn;
      const int ia = half_layout ? p : 2 * p;
      const int ib = half_layout ? p + vhalf : 2 * p + 1;
      const float a = ScalarOps<T>::to_f32(src[ia]);
      const float b = ScalarOps<T>::to_f32(src[ib]);
      dst[ia] = ScalarOps<T>::from_f32(a * c - b * s);
      dst[ib] = ScalarOps<T>::from_f32(b * c + a * s);
    }
    return;
  }
  const bool is_q = y < H;
  const T *src = is_q ? q + (long)t * q_stride + (long)y * D
                      : k + (long)t * k_stride + (long)(y - H) * D;
  const T *w = is_q ? q_w : k_w;
  // span norm: the weights cover the row, this head reads its block
  if (norm_span && w) w += (long)(is_q ? y : y - H) * D;
  float ss = 0.f;
  for (int i = lane; i < D; i += QK_BLOCK) {
    const float x = ScalarOps<T>::to_f32(src[i]);
    buf[i] = x;
    ss += x * x;
  }
  __syncthreads();
  if (do_norm && !norm_last) {
    int n = D;
    if (norm_span) {
      // every head of the row sums the whole row, in the same order, so
      // all heads of a token scale by the same number (the host makes q
      // land in a buffer of its own: the row stays as it came in)
      const T *row = is_q ? q + (long)t * q_stride : k + (long)t * k_stride;
      n = (is_q ? H : G) * D;
      ss = 0.f;
      if (n % 8 == 0 && reinterpret_cast<uintptr_t>(row) % 16 == 0) {
        for (int i = lane * 8; i < n; i += QK_BLOCK * 8) {  // 16 B loads
          float x[8];
          ld8<T>(row + i, x);
#pragma unroll
          for (int e = 0; e < 8; ++e) ss += x[e] * x[e];
        }
      } else {
        for (int i = lane; i < n; i += QK_BLOCK) {
          const float x = ScalarOps<T>::to_f32(row[i]);
          ss += x * x;
        }
      }
    }
    ss = wave_reduce_sum(ss);
    const float inv = 1.0f / sqrtf(ss / n + eps);
    for (int i = lane; i < D; i += QK_BLOCK)
      buf[i] = buf[i] * inv * (w ? ScalarOps<T>::to_f32(w[i]) : 1.0f);
    __syncthreads();
  }
  const double pos = (double)positions[t];
  const int half = rot_dims / 2;
  for (int p = lane; p < half; p += QK_BLOCK) {
    double sn, cs;
    sincos(pos * freqs[p], &sn, &cs);
    const float c = (float)cs * mag, s = (float)sn * mag;
    const int ia = half_layout ? p : 2 * p;
    const int ib = half_layout ? p + half : 2 * p + 1;
    const float a = buf[ia], b = buf[ib];
    buf[ia] = a * c - b * s;
    buf[ib] = b * c + a * s;
  }
  __syncthreads();
  if (do_norm && norm_last) {
    ss = 0.f;
    for (int i = lane; i < D; i += QK_BLOCK) ss += buf[i] * buf[i];
    ss = wave_reduce_sum(ss);
    const float inv = 1.0f / sqrtf(ss / D + eps);
    for (int i = lane; i < D; i += QK_BLOCK)
      buf[i] = buf[i] * inv * (w ? ScalarOps<T>::to_f32(w[i]) : 1.0f);
    __syncthreads();
  }
  T *dst = is_q ? q_out + (long)t * q_out_stride + (long)y * D
                : k_cache + (slot_mapping[t] * G + (y - H)) * D;
  for (int i = lane; i < D; i += QK_BLOCK)
    dst[i] = ScalarOps<T>::from_f32(buf[i]);
}

// ------------------------------------------------------------------
// Row-wide form: one workgroup per token prepares the whole q row, the
// whole k row and all value heads. The token's cos / sin table is formed
// once (fp64 angle) and shared by every head; a row is read once, summed
// by the block for its one RMS, then normed (row-sized weights), turned
// and written. LDS: [2 * half] table + [max(H, G) * D] row as fp32.
// grid (tokens), block 256.
constexpr int SPAN_BLOCK = 256;

template <typename T>
DEV_INLINE void span_row(float *row, const float *cs, const float *sn,
                         float *red, const T *__restrict__ src,
                         const T *__restrict__ w, T *__restrict__ dst,
                         int heads, int D, int rot_dims, int half_layout,
                         float eps, bool vec) {
  const int n = heads * D, tid = threadIdx.x;
  float ss = 0.f;
  if (vec) {
    for (int i = tid * 8; i < n; i += SPAN_BLOCK * 8) {
      ld8<T>(src + i, row + i);
#pragma unroll
      for (int e = 0; e < 8; ++e) ss += row[i + e] * row[i + e];
    }
  } else {
    for (int i = tid; i < n; i += SPAN_BLOCK) {
      const float x = ScalarOps<T>::to_f32(src[i]);
      row[i] = x;
      ss += x * x;
    }
  }
  __syncthreads();  // red may still be read from the previous row
  const float inv =
      1.0f / sqrtf(block_reduce_sum<SPAN_BLOCK>(ss, red) / n + eps);
  const int half = rot_dims / 2;
  // the turned pairs of every head
  for (int idx = tid; idx < heads * half; idx += SPAN_BLOCK) {
    const int h = idx / half, p = idx % half;
    const int ia = h * D + (half_layout ? p : 2 * p);
    const int ib = h * D + (half_layout ? p + half : 2 * p + 1);
    const float a = row[ia] * inv * (w ? ScalarOps<T>::to_f32(w[ia]) : 1.0f);
    const float b = row[ib] * inv * (w ? ScalarOps<T>::to_f32(w[ib]) : 1.0f);
    dst[ia] = ScalarOps<T>::from_f32(a * cs[p] - b * sn[p]);
    dst[ib] = ScalarOps<T>::from_f32(b * cs[p] + a * sn[p]);
  }
  // the dims that pass unchanged
  const int rest = D - rot_dims;
  for (int idx = tid; idx < heads * rest; idx += SPAN_BLOCK) {
    const int i = (idx / rest) * D + rot_dims + idx % rest;
    dst[i] = ScalarOps<T>::from_f32(
        row[i] * inv * (w ? ScalarOps<T>::to_f32(w[i]) : 1.0f));
  }
}

template <typename T>
__global__ __launch_bounds__(SPAN_BLOCK) void qk_span_rope_store_kernel(
    const T *__restrict__ q, long q_stride, const T *__restrict__ k,
    long k_stride, const T *__restrict__ v, long v_stride,
    const T *__restrict__ q_w, const T *__restrict__ k_w,
    const long *__restrict__ positions, const long *__restrict__ slot_mapping,
    const double *__restrict__ freqs, float mag, int rot_dims,
    T *__restrict__ k_cache, T *__restrict__ v_cache, int H, int G, int D,
    int Dv, float eps, int half_layout, int v_unit, T *__restrict__ q_out,
    long q_out_stride, int vec_q, int vec_k) {
  extern __shared__ float span_lds[];
  __shared__ float red[SPAN_BLOCK / WAVE_SIZE];
  const int t = blockIdx.x, tid = threadIdx.x;
  const int half = rot_dims / 2;
  float *cs = span_lds, *sn = span_lds + half;
  float *row = span_lds + ((2 * half + 3) & ~3);
  const double pos = (double)positions[t];
  for (int p = tid; p < half; p += SPAN_BLOCK) {
    double s, c;
    sincos(pos * freqs[p], &s, &c);
    cs[p] = (float)c * mag;
    sn[p] = (float)s * mag;
  }
  // (span_row's first barrier publishes the table)
  span_row<T>(row, cs, sn, red, q + (long)t * q_stride, q_w,
              q_out + (long)t * q_out_stride, H, D, rot_dims, half_layout,
              eps, vec_q != 0);
  if (k == nullptr) return;
  const long slot = slot_mapping[t];
  __syncthreads();  // every thread is done with the q row
  span_row<T>(row, cs, sn, red, k + (long)t * k_stride, k_w,
              k_cache + slot * G * D, G, D, rot_dims, half_layout, eps,
              vec_k != 0);
  // values: a wave per head
  const int lane = tid & 63, wave = tid >> 6;
  for (int g = wave; g < G; g += SPAN_BLOCK / WAVE_SIZE) {
    const T *src = v + (long)t * v_stride + (long)g * Dv;
    T *dst = v_cache + (slot * G + g) * Dv;
    if (!v_unit) {
      for (int i = lane; i < Dv; i += 64) dst[i] = src[i];
      continue;
    }
    float vs = 0.f;
    for (int i = lane; i < Dv; i += 64) {
      const float x = ScalarOps<T>::to_f32(src[i]);
      vs += x * x;
    }
    const float vinv = 1.0f / sqrtf(wave_reduce_sum(vs) / Dv + eps);
    for (int i = lane; i < Dv; i += 64)
      dst[i] = ScalarOps<T>::from_f32(ScalarOps<T>::to_f32(src[i]) * vinv);
  }
}

// ------------------------------------------------------------------
// grid (tokens, H); one workgroup = one (query token, query head).
// Visible keys are enumerated as kept-first [0, n_keep) followed by the
// window [lo, i]; tiles of ATT_BLOCK keys: one score per thread, online
// softmax across tiles, then P.V with threads laid out as
// (key part) x (value column).
template <typename T, int CT>  // CT: column threads, pow2 >= min(Dv,256)
__global__ __launch_bounds__(ATT_BLOCK) void window_attention_kernel(
    T *__restrict__ out, long out_stride, const T *__restrict__ q,
    long q_stride,
    const T *__restrict__ gate, long gate_stride,
    const T *__restrict__ k_cache, const T *__restrict__ v_cache,
    const int *__restrict__ block_table, int bt_stride,
    const int *__restrict__ seq_lens, const int *__restrict__ qsl, int B,
    int H, int G, int D, int Dv, int page, float scale, int window,
    int keep_first, int sink, const float *__restrict__ sinks,
    float softcap) {
  constexpr int PARTS = ATT_BLOCK / CT;
  constexpr int NC = 2;  // columns per thread when Dv > CT (Dv <= 512)
  extern __shared__ float smem[];
  float *qs = smem;                 // [D]
  float *ps = qs + ((D + 3) & ~3);  // [ATT_BLOCK] probabilities
  long *rows = reinterpret_cast<long *>(ps + ATT_BLOCK);  // [ATT_BLOCK]
  float *accs = reinterpret_cast<float *>(rows + ATT_BLOCK);  // [PARTS][NC*CT]
  __shared__ float red[ATT_BLOCK / WAVE_SIZE];
  __shared__ float bcast;

  const int t = blockIdx.x, h = blockIdx.y;
  const int tid = threadIdx.x;
  // which sequence owns token t: largest b with qsl[b] <= t
  int lo_b = 0, hi_b = B - 1;
  while (lo_b < hi_b) {
    const int mid = (lo_b + hi_b + 1) >> 1;
    if (qsl[mid] <= t) lo_b = mid; else hi_b = mid - 1;
  }
  const int b = lo_b;
  // sequence b holds seq_lens[b] tokens after this step; its new tokens
  // are rows qsl[b]..qsl[b+1]-1, so row t sits at position
  const int i = seq_lens[b] - (qsl[b + 1] - t);
  const int g = h / (H / G);
  const int *bt = block_table + (long)b * bt_stride;

  for (int d = tid; d < D; d += ATT_BLOCK)
    qs[d] = ScalarOps<T>::to_f32(q[(long)t * q_stride + (long)h * D + d]);

  const int lo = (window > 0 && i - window + 1 > 0) ? i - window + 1 : 0;
  const int n_keep = keep_first < lo ? keep_first : lo;
  const int total = n_keep + (i - lo + 1);

  // the sink is an already-seen key (score 0, or the head's learned
  // score) that has no value
  float m = sinks ? sinks[h] : (sink ? 0.f : -INFINITY);
  float l = (sink || sinks) ? 1.f : 0.f;
  float acc[NC] = {0.f, 0.f};
  const int col = tid % CT, part = tid / CT;
  __syncthreads();

  for (int base = 0; base < total; base += ATT_BLOCK) {
    const int vi = base + tid;
    float s = -INFINITY;
    __syncthreads();  // the last tile's ps/rows/red are done with
    if (vi < total) {
      const int j = vi < n_keep ? vi : lo + (vi - n_keep);
      const long row = (long)bt[j / page] * page + j % page;
      rows[tid] = row;
      const T *kr = k_cache + (row * G + g) * D;
      float dot = 0.f;
      if (sizeof(T) == 2 && D % 8 == 0) {  // 16 B loads, rows 16 B aligned
        for (int d = 0; d < D; d += 8) {
          float kf[8];
          unpack8<T>(*reinterpret_cast<const shortx8 *>(kr + d), kf);
#pragma unroll
          for (int e = 0; e < 8; ++e) dot += qs[d + e] * kf[e];
        }
      } else if (sizeof(T) == 4 && D % 4 == 0) {
        for (int d = 0; d < D; d += 4) {
          const floatx4 kf = *reinterpret_cast<const floatx4 *>(kr + d);
#pragma unroll
          for (int e = 0; e < 4; ++e) dot += qs[d + e] * kf[e];
        }
      } else {
        for (int d = 0; d < D; ++d)
          dot += qs[d] * ScalarOps<T>::to_f32(kr[d]);
      }
      s = dot * scale;
      if (softcap > 0.f) s = softcap * tanhf(s / softcap);
    }
    // tile max -> new running max
    float tm = wave_reduce_max(s);
    if ((tid & 63) == 0) red[tid >> 6] = tm;
    __syncthreads();
    if (tid == 0) {
      float x = red[0];
      for (int w = 1; w < ATT_BLOCK / WAVE_SIZE; ++w) x = fmaxf(x, red[w]);
      bcast = fmaxf(m, x);
    }
    __syncthreads();
    const float m_new = bcast;
    const float p = vi < total ? expf(s - m_new) : 0.f;
    ps[tid] = p;
    float psum = wave_reduce_sum(p);
    __syncthreads();
    if ((tid & 63) == 0) red[tid >> 6] = psum;
    __syncthreads();
    float tsum = 0.f;
    for (int w = 0; w < ATT_BLOCK / WAVE_SIZE; ++w) tsum += red[w];
    const float corr = (m == -INFINITY) ? 0.f : expf(m - m_new);
    l = l * corr + tsum;
    m = m_new;
    const int n_tile = total - base < ATT_BLOCK ? total - base : ATT_BLOCK;
#pragma unroll
    for (int c = 0; c < NC; ++c) acc[c] *= corr;
    for (int jj = part; jj < n_tile; jj += PARTS) {
      const float pj = ps[jj];
      const T *vr = v_cache + (rows[jj] * G + g) * Dv;
#pragma unroll
      for (int c = 0; c < NC; ++c) {
        const int d = col + c * CT;
        if (d < Dv) acc[c] += pj * ScalarOps<T>::to_f32(vr[d]);
      }
    }
  }
  // reduce the key parts
  __syncthreads();
#pragma unroll
  for (int c = 0; c < NC; ++c) accs[(part * NC + c) * CT + col] = acc[c];
  __syncthreads();
  if (part == 0) {
    const float inv_l = 1.0f / l;
#pragma unroll
    for (int c = 0; c < NC; ++c) {
      const int d = col + c * CT;
      if (d >= Dv) continue;
      float o = 0.f;
      for (int pp = 0; pp < PARTS; ++pp) o += accs[(pp * NC + c) * CT + col];
      o *= inv_l;
      if (gate != nullptr) {
        const float z = ScalarOps<T>::to_f32(
            gate[(long)t * gate_stride + (long)h * Dv + d]);
        o *= 1.0f / (1.0f + expf(-z));
      }
      out[(long)t * out_stride + (long)h * Dv + d] = ScalarOps<T>::from_f32(o);
    }
  }
}

bool rows_ok(const torch::Tensor &t) {
  return t.dim() == 2 && t.stride(1) == 1;
}

}  // namespace

void qk_norm_rope_store(torch::Tensor q, c10::optional<torch::Tensor> k,
                        c10::optional<torch::Tensor> v,
                        c10::optional<torch::Tensor> q_w,
                        c10::optional<torch::Tensor> k_w,
                        torch::Tensor positions, torch::Tensor slot_mapping,
                        torch::Tensor freqs, double mag, long rot_dims,
                        c10::optional<torch::Tensor> k_cache,
                        c10::optional<torch::Tensor> v_cache, long H, long G,
                        long D, long Dv, double eps, bool half_layout,
                        bool norm_last, bool do_norm,
                        c10::optional<torch::Tensor> v_freqs, bool norm_span,
                        bool v_unit, c10::optional<torch::Tensor> q_out) {
  const long T = q.size(0);
  // span norm: other heads still read the incoming row while one head
  // writes, so the result needs a buffer of its own
  TORCH_CHECK(!norm_span || q_out.has_value(),
              "span norm writes q out of place");
  void *qop = q.data_ptr();
  long qos = q.stride(0);
  if (q_out.has_value()) {
    TORCH_CHECK(q_out->is_cuda() && rows_ok(*q_out) &&
                q_out->sizes() == q.sizes() &&
                q_out->scalar_type() == q.scalar_type() &&
                q_out->data_ptr() != q.data_ptr());
    qop = q_out->data_ptr();
    qos = q_out->stride(0);
  }
  TORCH_CHECK(!norm_span || (do_norm && !norm_last),
              "span norm runs before the rotation");
  TORCH_CHECK(!v_unit || !v_freqs.has_value(),
              "unit values and rotated values do not combine");
  if (T == 0) return;
  const auto st = q.scalar_type();
  TORCH_CHECK(q.is_cuda() && rows_ok(q) && q.size(1) == H * D);
  const void *qwp = nullptr;
  if (q_w.has_value()) {
    TORCH_CHECK(q_w->scalar_type() == st &&
                q_w->numel() == (norm_span ? H * D : D) &&
                q_w->is_contiguous());
    qwp = q_w->data_ptr();
  }
  TORCH_CHECK(positions.scalar_type() == at::kLong &&
              positions.is_contiguous() && positions.numel() >= T);
  TORCH_CHECK(freqs.scalar_type() == at::kDouble && freqs.is_contiguous() &&
              freqs.numel() * 2 >= rot_dims);
  TORCH_CHECK(rot_dims >= 0 && rot_dims <= D && rot_dims % 2 == 0,
              "rotary dims must be even and <= head dim");
  TORCH_CHECK(D * 4 <= 32 * 1024);
  const bool own = k.has_value();
  const void *kp = nullptr, *vp = nullptr, *kwp = nullptr;
  void *kcp = nullptr, *vcp = nullptr;
  long ks = 0, vs = 0;
  if (own) {
    TORCH_CHECK(v.has_value() && k_w.has_value() == q_w.has_value() &&
                k_cache.has_value() && v_cache.has_value());
    TORCH_CHECK(rows_ok(*k) && k->size(0) == T && k->size(1) == G * D &&
                k->scalar_type() == st);
    TORCH_CHECK(rows_ok(*v) && v->size(0) == T && v->size(1) == G * Dv &&
                v->scalar_type() == st);
    if (k_w.has_value()) {
      TORCH_CHECK(k_w->scalar_type() == st &&
                  k_w->numel() == (norm_span ? G * D : D) &&
                  k_w->is_contiguous());
      kwp = k_w->data_ptr();
    }
    TORCH_CHECK(k_cache->is_contiguous() && v_cache->is_contiguous() &&
                k_cache->scalar_type() == st && v_cache->scalar_type() == st);
    TORCH_CHECK(k_cache->dim() == 4 && k_cache->size(2) == G &&
                k_cache->size(3) == D && v_cache->size(2) == G &&
                v_cache->size(3) == Dv, "cache geometry mismatch");
    TORCH_CHECK(slot_mapping.scalar_type() == at::kLong &&
                slot_mapping.is_contiguous() && slot_mapping.numel() >= T);
    kp = k->data_ptr(); vp = v->data_ptr();
    kcp = k_cache->data_ptr(); vcp = v_cache->data_ptr();
    ks = k->stride(0); vs = v->stride(0);
  }
  const double *vfp = nullptr;
  if (v_freqs.has_value()) {
    TORCH_CHECK(v_freqs->scalar_type() == at::kDouble &&
                v_freqs->is_contiguous() && Dv % 2 == 0 &&
                v_freqs->numel() * 2 >= Dv, "value rotary table");
    vfp = v_freqs->data_ptr<double>();
  }
  const int gy = own ? H + 2 * G : H;
  auto stream = at::cuda::getCurrentCUDAStream();
  const long span_floats =
      ((rot_dims + 3) & ~3L) + std::max(H, own ? G : 0L) * D;
  if (norm_span && !vfp && span_floats * 4 <= 60 * 1024 && T >= 512) {
    // prompt-sized batches, one workgroup per token: one cos / sin table
    // and one read of each row for all heads (a handful of decode tokens
    // is served sooner by the workgroup-per-head form below, which
    // spreads a token over H + 2G workgroups)
    const size_t es = q.element_size();
    auto vec_ok = [&](const void *p, long stride, long n, const void *w) {
      return n % 8 == 0 && (stride * es) % 16 == 0 &&
             reinterpret_cast<uintptr_t>(p) % 16 == 0 ? 1 : 0;
    };
    const int vq = vec_ok(q.data_ptr(), q.stride(0), H * D, qwp);
    const int vk = own ? vec_ok(kp, ks, G * D, kwp) : 0;
#define RUNS(TT)                                                             \
  hipLaunchKernelGGL((qk_span_rope_store_kernel<TT>), dim3(T),               \
                     dim3(SPAN_BLOCK), span_floats * sizeof(float), stream,  \
                     (const TT *)q.data_ptr(), (long)q.stride(0),            \
                     (const TT *)kp, ks, (const TT *)vp, vs,                 \
                     (const TT *)qwp, (const TT *)kwp,                       \
                     positions.data_ptr<long>(),                             \
                     own ? slot_mapping.data_ptr<long>() : nullptr,          \
                     freqs.data_ptr<double>(), (float)mag, (int)rot_dims,    \
                     (TT *)kcp, (TT *)vcp, (int)H, (int)G, (int)D, (int)Dv,  \
                     (float)eps, half_layout ? 1 : 0, v_unit ? 1 : 0,        \
                     (TT *)qop, qos, vq, vk)
    if (st == at::kBFloat16) RUNS(__hip_bfloat16);
    else if (st == at::kFloat) RUNS(float);
    else TORCH_CHECK(false, "qk_norm_rope_store: bf16 or fp32");
#undef RUNS
    HIP_CHECK_KERNEL();
    return;
  }
#define RUN(TT)                                                              \
  hipLaunchKernelGGL((qk_norm_rope_store_kernel<TT>), dim3(T, gy),           \
                     dim3(QK_BLOCK), D * sizeof(float), stream,              \
                     (TT *)q.data_ptr(), (long)q.stride(0), (const TT *)kp,  \
                     ks, (const TT *)vp, vs, (const TT *)qwp,                \
                     (const TT *)kwp, positions.data_ptr<long>(),            \
                     own ? slot_mapping.data_ptr<long>() : nullptr,          \
                     freqs.data_ptr<double>(), (float)mag, (int)rot_dims,    \
                     (TT *)kcp, (TT *)vcp, (int)H, (int)G, (int)D, (int)Dv,  \
                     (float)eps, half_layout ? 1 : 0, norm_last ? 1 : 0,     \
                     do_norm ? 1 : 0, vfp, norm_span ? 1 : 0, v_unit ? 1 : 0, \
                     (TT *)qop, qos)
  if (st == at::kBFloat16) RUN(__hip_bfloat16);
  else if (st == at::kFloat) RUN(float);
  else TORCH_CHECK(false, "qk_norm_rope_store: bf16 or fp32");
#undef RUN
  HIP_CHECK_KERNEL();
}

void window_attention(torch::Tensor out, torch::Tensor q,
                      c10::optional<torch::Tensor> gate,
                      torch::Tensor k_cache, torch::Tensor v_cache,
                      torch::Tensor block_table, torch::Tensor seq_lens,
                      torch::Tensor query_start_loc, double scale,
                      long window, long keep_first, bool sink,
                      c10::optional<torch::Tensor> sinks, double softcap) {
  const long T = q.size(0);
  if (T == 0) return;
  const auto st = q.scalar_type();
  TORCH_CHECK(k_cache.dim() == 4 && v_cache.dim() == 4);
  const int page = k_cache.size(1), G = k_cache.size(2), D = k_cache.size(3);
  const int Dv = v_cache.size(3);
  TORCH_CHECK(rows_ok(q) && q.size(1) % D == 0);
  const int H = q.size(1) / D;
  TORCH_CHECK(H % G == 0, "query heads must be a multiple of kv heads");
  TORCH_CHECK(k_cache.is_contiguous() && v_cache.is_contiguous() &&
              k_cache.scalar_type() == st && v_cache.scalar_type() == st);
  TORCH_CHECK(v_cache.size(0) == k_cache.size(0) && v_cache.size(1) == page &&
              v_cache.size(2) == G);
  TORCH_CHECK(rows_ok(out) && out.scalar_type() == st && out.size(0) == T &&
              out.size(1) == (long)H * Dv,
              "out: [T, H*Dv] rows (a column block is fine)");
  TORCH_CHECK(block_table.scalar_type() == at::kInt && block_table.dim() == 2 &&
              block_table.stride(1) == 1);
  TORCH_CHECK(seq_lens.scalar_type() == at::kInt && seq_lens.is_contiguous());
  TORCH_CHECK(query_start_loc.scalar_type() == at::kInt &&
              query_start_loc.is_contiguous());
  const int B = seq_lens.numel();
  TORCH_CHECK(query_start_loc.numel() >= B + 1 && block_table.size(0) >= B);
  TORCH_CHECK(Dv <= 512, "window_attention: value size <= 512");
  const void *gp = nullptr;
  long gs = 0;
  if (gate.has_value()) {
    TORCH_CHECK(rows_ok(*gate) && gate->size(0) == T &&
                gate->size(1) == H * Dv && gate->scalar_type() == st);
    gp = gate->data_ptr();
    gs = gate->stride(0);
  }
  const float *sp = nullptr;
  if (sinks.has_value()) {
    TORCH_CHECK(sinks->scalar_type() == at::kFloat && sinks->is_contiguous() &&
                sinks->numel() == H, "sinks: fp32 [H]");
    sp = sinks->data_ptr<float>();
  }
  int ct = 16;
  while (ct < Dv && ct < 256) ct *= 2;
  const int parts = ATT_BLOCK / ct;
  const size_t lds = (((D + 3) & ~3) + ATT_BLOCK) * sizeof(float) +
                     ATT_BLOCK * sizeof(long) +
                     (size_t)parts * 2 * ct * sizeof(float);
  auto stream = at::cuda::getCurrentCUDAStream();
#define RUN(TT, CTV)                                                         \
  hipLaunchKernelGGL((window_attention_kernel<TT, CTV>), dim3(T, H),         \
                     dim3(ATT_BLOCK), lds, stream, (TT *)out.data_ptr(),     \
                     (long)out.stride(0), (const TT *)q.data_ptr(),          \
                     (long)q.stride(0),                                      \
                     (const TT *)gp, gs, (const TT *)k_cache.data_ptr(),     \
                     (const TT *)v_cache.data_ptr(),                         \
                     block_table.data_ptr<int>(), (int)block_table.stride(0), \
                     seq_lens.data_ptr<int>(),                               \
                     query_start_loc.data_ptr<int>(), B, H, G, D, Dv, page,  \
                     (float)scale, (int)window, (int)keep_first,             \
                     sink ? 1 : 0, sp, (float)softcap)
#define RUN_CT(TT)                                                           \
  switch (ct) {                                                              \
    case 16: RUN(TT, 16); break;                                             \
    case 32: RUN(TT, 32); break;                                             \
    case 64: RUN(TT, 64); break;                                             \
    case 128: RUN(TT, 128); break;                                           \
    default: RUN(TT, 256); break;                                            \
  }
  if (st == at::kBFloat16) { RUN_CT(__hip_bfloat16) }
  else if (st == at::kFloat) { RUN_CT(float) }
  else TORCH_CHECK(false, "window_attention: bf16 or fp32");
#undef RUN_CT
#undef RUN
  HIP_CHECK_KERNEL();
}

namespace {

// one workgroup per token: the cos/sin of the token's D/2 pair angles
// (sign * pos * freqs[m], fp64 angle) are formed once in LDS, then every
// head row is turned (pairs (2m, 2m+1), or (m, m + D/2) in the half
// layout) and scaled; out may be a column block of a wider buffer.
template <typename T>
__global__ __launch_bounds__(ATT_BLOCK) void rotate_scale_kernel(
    T *__restrict__ out, long out_stride, const T *__restrict__ x,
    long x_stride, const long *__restrict__ positions,
    const double *__restrict__ freqs, int heads, int D, float sign,
    float scale, int layout) {
  // layout 0: pairs (2m, 2m+1) moved as 32-bit words; 1: pairs
  // (m, m + D/2); 2: pairs (2m, 2m+1) element by element
  const bool half_layout = layout == 1;
  extern __shared__ float cs_tab[];  // [D/2] cos, [D/2] sin
  const int t = blockIdx.x;
  const int half = D / 2;
  const double pos = (double)positions[t];
  for (int p = threadIdx.x; p < half; p += ATT_BLOCK) {
    double sn, cs;
    sincos(pos * freqs[p], &sn, &cs);
    cs_tab[p] = (float)cs;
    cs_tab[half + p] = sign * (float)sn;
  }
  __syncthreads();
  const T *src = x + (long)t * x_stride;
  T *dst = out + (long)t * out_stride;
  const int total = heads * half;
  if (layout == 0 && sizeof(T) == 2) {
    // a pair is one aligned 32-bit word of the row
    for (int idx = threadIdx.x; idx < total; idx += ATT_BLOCK) {
      const int p = idx % half;
      const float c = cs_tab[p], s = cs_tab[half + p];
      T pr[2];
      *reinterpret_cast<unsigned *>(pr) =
          reinterpret_cast<const unsigned *>(src)[idx];
      const float a = ScalarOps<T>::to_f32(pr[0]);
      const float b = ScalarOps<T>::to_f32(pr[1]);
      pr[0] = ScalarOps<T>::from_f32((a * c - b * s) * scale);
      pr[1] = ScalarOps<T>::from_f32((b * c + a * s) * scale);
      reinterpret_cast<unsigned *>(dst)[idx] =
          *reinterpret_cast<unsigned *>(pr);
    }
    return;
  }
  for (int idx = threadIdx.x; idx < total; idx += ATT_BLOCK) {
    const int hd = idx / half, p = idx % half;
    const float c = cs_tab[p], s = cs_tab[half + p];
    const int ia = hd * D + (half_layout ? p : 2 * p);
    const int ib = hd * D + (half_layout ? p + half : 2 * p + 1);
    const float a = ScalarOps<T>::to_f32(src[ia]);
    const float b = ScalarOps<T>::to_f32(src[ib]);
    dst[ia] = ScalarOps<T>::from_f32((a * c - b * s) * scale);
    dst[ib] = ScalarOps<T>::from_f32((b * c + a * s) * scale);
  }
}

// one wave per row: out = x / rms(x) * w (row kept in the model dtype)
// and, with a cache, the same row scattered into its paged slot. VEC: 8
// elements per lane through 16 B accesses (n % 8 == 0, aligned rows).
template <typename T, bool VEC>
__global__ __launch_bounds__(ATT_BLOCK) void rms_weight_store_kernel(
    T *__restrict__ out, const T *__restrict__ x, long x_stride,
    const T *__restrict__ w, int n, float eps, T *__restrict__ cache,
    const long *__restrict__ slot_mapping, long rows) {
  const long r = (long)blockIdx.x * (ATT_BLOCK / WAVE_SIZE) + (threadIdx.x >> 6);
  const int lane = threadIdx.x & 63;
  if (r >= rows) return;
  const T *src = x + r * x_stride;
  T *crow = cache ? cache + slot_mapping[r] * n : nullptr;
  float ss = 0.f;
  if (VEC) {
    for (int i = lane * 8; i < n; i += WAVE_SIZE * 8) {
      float f[8];
      ld8<T>(src + i, f);
#pragma unroll
      for (int e = 0; e < 8; ++e) ss += f[e] * f[e];
    }
    ss = wave_reduce_sum(ss);
    const float inv = 1.0f / sqrtf(ss / n + eps);
    for (int i = lane * 8; i < n; i += WAVE_SIZE * 8) {
      float f[8], wf[8];
      ld8<T>(src + i, f);
      ld8<T>(w + i, wf);
#pragma unroll
      for (int e = 0; e < 8; ++e) f[e] = f[e] * inv * wf[e];
      st8<T>(out + r * n + i, f);
      if (crow) st8<T>(crow + i, f);
    }
    return;
  }
  for (int i = lane; i < n; i += WAVE_SIZE) {
    const float v = ScalarOps<T>::to_f32(src[i]);
    ss += v * v;
  }
  ss = wave_reduce_sum(ss);
  const float inv = 1.0f / sqrtf(ss / n + eps);
  for (int i = lane; i < n; i += WAVE_SIZE) {
    const T v = ScalarOps<T>::from_f32(ScalarOps<T>::to_f32(src[i]) * inv *
                                       ScalarOps<T>::to_f32(w[i]));
    out[r * n + i] = v;
    if (crow) crow[i] = v;
  }
}

}  // namespace

void rotate_scale_rows(torch::Tensor out, torch::Tensor x,
                       torch::Tensor positions, torch::Tensor freqs,
                       long heads, long D, double sign, double scale,
                       bool half_layout) {
  const long T = x.size(0);
  if (T == 0) return;
  const auto st = x.scalar_type();
  TORCH_CHECK(x.is_cuda() && rows_ok(x) && x.size(1) == heads * D &&
              D % 2 == 0);
  TORCH_CHECK(rows_ok(out) && out.size(0) == T && out.size(1) == heads * D &&
              out.scalar_type() == st);
  TORCH_CHECK(positions.scalar_type() == at::kLong &&
              positions.is_contiguous() && positions.numel() >= T);
  TORCH_CHECK(freqs.scalar_type() == at::kDouble && freqs.is_contiguous() &&
              freqs.numel() * 2 >= D);
  auto stream = at::cuda::getCurrentCUDAStream();
  // the word-wide path needs 4-byte aligned rows on both sides
  const bool words = x.element_size() == 2 &&
                     reinterpret_cast<uintptr_t>(x.data_ptr()) % 4 == 0 &&
                     reinterpret_cast<uintptr_t>(out.data_ptr()) % 4 == 0 &&
                     x.stride(0) % 2 == 0 && out.stride(0) % 2 == 0;
  const int layout = half_layout ? 1 : (words ? 0 : 2);
#define RUN(TT)                                                              \
  hipLaunchKernelGGL((rotate_scale_kernel<TT>), dim3(T), dim3(ATT_BLOCK),    \
                     D * sizeof(float), stream, (TT *)out.data_ptr(),        \
                     (long)out.stride(0), (const TT *)x.data_ptr(),          \
                     (long)x.stride(0), positions.data_ptr<long>(),          \
                     freqs.data_ptr<double>(), (int)heads, (int)D,           \
                     (float)sign, (float)scale, layout)
  if (st == at::kBFloat16) RUN(__hip_bfloat16);
  else if (st == at::kFloat) RUN(float);
  else TORCH_CHECK(false, "rotate_scale_rows: bf16 or fp32");
#undef RUN
  HIP_CHECK_KERNEL();
}

void rms_weight_store(torch::Tensor out, torch::Tensor x, torch::Tensor w,
                      double eps, c10::optional<torch::Tensor> cache,
                      c10::optional<torch::Tensor> slot_mapping) {
  const long rows = x.size(0);
  if (rows == 0) return;
  const auto st = x.scalar_type();
  const int n = x.size(1);
  TORCH_CHECK(x.is_cuda() && rows_ok(x));
  TORCH_CHECK(out.is_contiguous() && out.scalar_type() == st &&
              out.numel() == rows * n);
  TORCH_CHECK(w.scalar_type() == st && w.is_contiguous() && w.numel() == n);
  void *cp = nullptr;
  const long *sp = nullptr;
  if (cache.has_value()) {
    TORCH_CHECK(slot_mapping.has_value() &&
                slot_mapping->scalar_type() == at::kLong &&
                slot_mapping->is_contiguous() &&
                slot_mapping->numel() >= rows);
    TORCH_CHECK(cache->is_contiguous() && cache->scalar_type() == st &&
                cache->size(-1) == n && cache->numel() % n == 0 &&
                cache->dim() == 4 && cache->size(2) == 1,
                "latent cache: [pages, page, 1, n]");
    cp = cache->data_ptr();
    sp = slot_mapping->data_ptr<long>();
  }
  const int per = ATT_BLOCK / WAVE_SIZE;
  auto stream = at::cuda::getCurrentCUDAStream();
  const long esz = x.element_size();
  auto al16 = [](const void *p) {
    return p == nullptr || reinterpret_cast<uintptr_t>(p) % 16 == 0;
  };
  const bool vec = n % 8 == 0 && (x.stride(0) * esz) % 16 == 0 &&
                   al16(x.data_ptr()) && al16(out.data_ptr()) &&
                   al16(w.data_ptr()) && al16(cp);
#define RUN(TT, V)                                                           \
  hipLaunchKernelGGL((rms_weight_store_kernel<TT, V>),                       \
                     dim3((rows + per - 1) / per), dim3(ATT_BLOCK), 0,       \
                     stream, (TT *)out.data_ptr(), (const TT *)x.data_ptr(), \
                     (long)x.stride(0), (const TT *)w.data_ptr(), n,         \
                     (float)eps, (TT *)cp, sp, rows)
  if (st == at::kBFloat16) {
    if (vec) RUN(__hip_bfloat16, true); else RUN(__hip_bfloat16, false);
  } else if (st == at::kFloat) {
    if (vec) RUN(float, true); else RUN(float, false);
  } else {
    TORCH_CHECK(false, "rms_weight_store: bf16 or fp32");
  }
#undef RUN
  HIP_CHECK_KERNEL();
}
