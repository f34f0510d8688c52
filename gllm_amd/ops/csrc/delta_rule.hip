// Gated delta rule over ragged batches, any head geometry, gfx950.
//
// Dtype-generic (projections T = bf16 or fp32; unit norms, gates, decay
// and the recurrent state are fp32 always). One code path serves prompt
// portions of any length and single decode tokens in the same launch,
// so a position's result never depends on how its sequence was cut.
//
//   causal_conv_silu   short causal depthwise convolution over time with
//                      silu; the taps-1 inputs before a portion come from
//                      the per-slot conv state
//   conv_state_update  rolls the conv state to the portion's last inputs
//   delta_rule_varlen  per (sequence, value head): for each token
//                        S <- g S;  u = beta (v - S^T k);  S <- S + k u^T;
//                        o = S^T q
//                      with q, k unit-normalised per head (q also scaled),
//                      beta = sigmoid(b), g = exp(-exp(A_log) softplus(a + dt)).
//                      A wavefront owns 16 state columns; each column is
//                      shared by a quad of lanes that split the key axis,
//                      so reductions over it are two DPP quad swaps, and
//                      waves never meet at a barrier: the state column
//                      block lives in registers for the whole portion.
//                      Norms and gates come from a per-token pre-pass.
//   rms_gate           scale * o / rms(o) * w * act(z) per head, act silu
//                      or sigmoid, w shared by the heads or one per head
//   token_shift        h_t + (h_(t-1) - h_t) * mu over a ragged batch; the
//                      row before a portion comes from the per-slot state
//   general_delta_rule per (sequence, head): for each token
//                        d = k^T S;  S <- diag(w) S - ak d^T + k v^T;
//                        o = S^T r
//                      with w = exp(-c sigmoid(.)) per key channel and
//                      ak = sigmoid(.) k / (|k|^2 + 1e-6) (removal rate on
//                      the unit key, folded) from a per-token pre-pass;
//                      same lane layout as delta_rule_varlen
//
// State layouts: conv [slots, C, taps-1] (oldest first), recurrent
// [slots, H, Dk, Dv] fp32.

#include <torch/extension.h>
#include <ATen/cuda/CUDAContext.h>
#include "common.h"

namespace {

constexpr int MAX_TAPS = 8;

DEV_INLINE int find_seq(const int *__restrict__ qsl, int B, int t) {
  int lo = 0, hi = B - 1;
  while (lo < hi) {
    const int mid = (lo + hi + 1) >> 1;
    if (qsl[mid] <= t) lo = mid; else hi = mid - 1;
  }
  return lo;
}

DEV_INLINE float silu_f(float z) { return z / (1.0f + expf(-z)); }

// grid (tokens, ceil(C / 256))
template <typename T>
__global__ __launch_bounds__(256) void causal_conv_silu_kernel(
    T *__restrict__ out, const T *__restrict__ x, long x_stride,
    const T *__restrict__ w, T *__restrict__ state,
    const long *__restrict__ slots, const int *__restrict__ has_init,
    const int *__restrict__ qsl, int B, int C, int taps, int act,
    int store) {
  const int t = blockIdx.x;
  const int c = blockIdx.y * 256 + threadIdx.x;
  if (c >= C) return;
  const int b = find_seq(qsl, B, t);
  const int r = t - qsl[b];  // offset inside this portion
  const bool init = has_init[b] != 0;
  T *st = state + ((long)slots[b] * C + c) * (taps - 1);
  float acc = 0.f;
  for (int tap = 0; tap < taps; ++tap) {
    const int rel = r - (taps - 1 - tap);
    T raw;
    if (rel >= 0)
      raw = x[(long)(qsl[b] + rel) * x_stride + c];
    else
      raw = init ? st[taps - 1 + rel] : ScalarOps<T>::from_f32(0.f);
    // store != 0: every portion is one token, so this thread alone reads
    // and rolls its channel's history (slot i <- what tap i + 1 just read)
    if (store && tap > 0) st[tap - 1] = raw;
    acc += ScalarOps<T>::to_f32(raw) *
           ScalarOps<T>::to_f32(w[(long)c * taps + tap]);
  }
  // the activation output feeds 16-bit consumers in bf16 serving
  out[(long)t * C + c] = ScalarOps<T>::from_f32(act ? silu_f(acc) : acc);
}

// 8 channels per thread, 16 B accesses (C % 8 == 0, aligned rows);
// grid (tokens, ceil(C / 8 / 256)). The taps-1 first tokens of a portion
// read their history from the per-slot state with scalar loads.
template <typename T, int TAPS>
__global__ __launch_bounds__(256) void causal_conv_silu8_kernel(
    T *__restrict__ out, const T *__restrict__ x, long x_stride,
    const T *__restrict__ w, T *__restrict__ state,
    const long *__restrict__ slots, const int *__restrict__ has_init,
    const int *__restrict__ qsl, int B, int C, int act, int store) {
  const int t = blockIdx.x;
  const int c0 = (blockIdx.y * 256 + threadIdx.x) * 8;
  if (c0 >= C) return;
  const int b = find_seq(qsl, B, t);
  const int start = qsl[b];
  const int r = t - start;
  float wf[8 * TAPS];  // [channel][tap], contiguous in memory
#pragma unroll
  for (int j = 0; j < TAPS; ++j) ld8<T>(w + (long)c0 * TAPS + j * 8, wf + j * 8);
  float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int tap = 0; tap < TAPS; ++tap) {
    const int rel = r - (TAPS - 1 - tap);
    float xv[8];
    if (rel >= 0) {
      ld8<T>(x + (long)(start + rel) * x_stride + c0, xv);
    } else if (has_init[b] != 0) {
      const T *st = state + ((long)slots[b] * C + c0) * (TAPS - 1);
#pragma unroll
      for (int e = 0; e < 8; ++e)
        xv[e] = ScalarOps<T>::to_f32(st[e * (TAPS - 1) + TAPS - 1 + rel]);
    } else {
#pragma unroll
      for (int e = 0; e < 8; ++e) xv[e] = 0.f;
    }
#pragma unroll
    for (int e = 0; e < 8; ++e) acc[e] += xv[e] * wf[e * TAPS + tap];
    if (store && tap > 0) {
      // one-token portions: this thread alone reads and rolls its
      // channels' history (slot tap - 1 <- what tap just read; the
      // 16-bit values survive the trip through fp32 unchanged)
      T *st = state + ((long)slots[b] * C + c0) * (TAPS - 1);
#pragma unroll
      for (int e = 0; e < 8; ++e)
        st[e * (TAPS - 1) + tap - 1] = ScalarOps<T>::from_f32(xv[e]);
    }
  }
  if (act) {
#pragma unroll
    for (int e = 0; e < 8; ++e) acc[e] = silu_f(acc[e]);
  }
  st8<T>(out + (long)t * C + c0, acc);
}

// grid (B, ceil(C / 256)); each thread owns one (sequence, channel) state
template <typename T>
__global__ __launch_bounds__(256) void conv_state_update_kernel(
    T *__restrict__ state, const T *__restrict__ x, long x_stride,
    const long *__restrict__ slots, const int *__restrict__ has_init,
    const int *__restrict__ qsl, int C, int taps) {
  const int b = blockIdx.x;
  const int c = blockIdx.y * 256 + threadIdx.x;
  if (c >= C) return;
  const int start = qsl[b], n = qsl[b + 1] - qsl[b];
  const bool init = has_init[b] != 0;
  T *st = state + ((long)slots[b] * C + c) * (taps - 1);
  T next[MAX_TAPS];
  for (int i = 0; i < taps - 1; ++i) {
    const int rel = n - (taps - 1) + i;
    if (rel >= 0) next[i] = x[(long)(start + rel) * x_stride + c];
    else next[i] = init ? st[taps - 1 + rel] : ScalarOps<T>::from_f32(0.f);
  }
  for (int i = 0; i < taps - 1; ++i) st[i] = next[i];
}

// One lane's contiguous key slice [i0, i0 + KP) of a q or k row as fp32;
// 16 B vector loads when the host found every slice aligned and whole.
template <typename T, int KP>
DEV_INLINE void load_slice(const T *__restrict__ row, int i0, int Dk,
                           bool vec, float *out) {
  if (vec) {
    if (sizeof(T) == 2) {
#pragma unroll
      for (int r = 0; r < KP; r += 8)
        unpack8<T>(*reinterpret_cast<const shortx8 *>(row + i0 + r), out + r);
    } else {
#pragma unroll
      for (int r = 0; r < KP; r += 4) {
        const floatx4 f = *reinterpret_cast<const floatx4 *>(row + i0 + r);
        out[r] = f[0]; out[r + 1] = f[1]; out[r + 2] = f[2]; out[r + 3] = f[3];
      }
    }
  } else {
#pragma unroll
    for (int r = 0; r < KP; ++r)
      out[r] = (i0 + r < Dk) ? ScalarOps<T>::to_f32(row[i0 + r]) : 0.f;
  }
}

// Per-token scalars of the recurrence, computed once instead of by every
// wave that needs them: prep[t] = [ik(G) | iq(G) | decay(H) | beta(H)]
// with ik = 1/sqrt(|k|^2 + 1e-6), iq = q_scale/sqrt(|q|^2 + 1e-6),
// decay = exp(-exp(A_log) softplus(a + dt_bias)), beta = sigmoid(b).
// grid (tokens), block 64.
template <typename T>
__global__ __launch_bounds__(64) void delta_prep_kernel(
    float *__restrict__ prep, const T *__restrict__ q,
    const T *__restrict__ k, long qkv_stride, const T *__restrict__ a,
    const T *__restrict__ bproj, long ab_stride,
    const float *__restrict__ A_log, const float *__restrict__ dt_bias,
    int H, int G, int Dk, float q_scale) {
  const long t = blockIdx.x;
  const int lane = threadIdx.x;
  float *out = prep + t * (2 * G + 2 * H);
  for (int g = 0; g < G; ++g) {
    float sk = 0.f, sq = 0.f;
    for (int i = lane; i < Dk; i += 64) {
      const float kv = ScalarOps<T>::to_f32(k[t * qkv_stride + (long)g * Dk + i]);
      const float qv = ScalarOps<T>::to_f32(q[t * qkv_stride + (long)g * Dk + i]);
      sk += kv * kv;
      sq += qv * qv;
    }
    sk = wave_reduce_sum(sk);
    sq = wave_reduce_sum(sq);
    if (lane == 0) {
      out[g] = 1.0f / sqrtf(sk + 1e-6f);
      out[G + g] = q_scale / sqrtf(sq + 1e-6f);
    }
  }
  for (int h = lane; h < H; h += 64) {
    const float av = ScalarOps<T>::to_f32(a[t * ab_stride + h]) + dt_bias[h];
    const float bv = ScalarOps<T>::to_f32(bproj[t * ab_stride + h]);
    // softplus without overflow: max(x, 0) + log1p(exp(-|x|))
    const float sp_a = fmaxf(av, 0.f) + log1pf(expf(-fabsf(av)));
    out[2 * G + h] = expf(-expf(A_log[h]) * sp_a);
    out[2 * G + H + h] = 1.0f / (1.0f + expf(-bv));
  }
}

// sum over the 4 adjacent lanes of a quad (DPP quad_perm: no LDS trip)
DEV_INLINE float quad_sum(float v) {
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(
      0, __builtin_bit_cast(int, v), 0xB1, 0xF, 0xF, true));  // [1,0,3,2]
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(
      0, __builtin_bit_cast(int, v), 0x4E, 0xF, 0xF, true));  // [2,3,0,1]
  return v;
}

// grid (B, H, ceil(Dv / 64)), block 256 = 4 independent waves.
// A wave owns 16 state columns; a quad of adjacent lanes shares a column
// and splits the key axis in 4 contiguous slices of KP = ceil(Dk / 4)
// (rounded up to 8/16/32/64): lane (col, part) holds S[part * KP + r][col].
// With S' = g S the step is
//   d = ik g (S^T k);  u = beta (v - d);  S <- g S + k (u ik);  o = iq S^T q
// on raw (un-normalised) q, k; the next token's operands are loaded
// while the current one is computed.
template <typename T, int KP>
__global__ __launch_bounds__(256) void delta_rule_varlen_kernel(
    float *__restrict__ o, const T *__restrict__ q, const T *__restrict__ k,
    const T *__restrict__ v, long qkv_stride, const float *__restrict__ prep,
    float *__restrict__ state, const long *__restrict__ slots,
    const int *__restrict__ has_init, const int *__restrict__ qsl, int H,
    int G, int Dk, int Dv, int vec) {
  const int b = blockIdx.x, h = blockIdx.y;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int col = blockIdx.z * 64 + wave * 16 + (lane >> 2);
  const int part = lane & 3;
  const int i0 = part * KP;
  const int g = h / (H / G);
  const int start = qsl[b], end = qsl[b + 1];
  const bool live = col < Dv;
  const int colc = live ? col : Dv - 1;  // clamp loads, mask stores
  if (blockIdx.z * 64 + wave * 16 >= Dv) return;  // whole wave idle
  if (start >= end) return;
  const int PW = 2 * G + 2 * H;

  float *sp = state + ((long)slots[b] * H + h) * Dk * Dv;
  float S[KP];
  const bool init = has_init[b] != 0;
#pragma unroll
  for (int r = 0; r < KP; ++r) {
    const int i = i0 + r;
    S[r] = (init && i < Dk) ? sp[(long)i * Dv + colc] : 0.f;
  }

  float kc[KP], qc[KP];
  float vc, ikc, iqc, gc, bc;
  {
    const long t = start;
    load_slice<T, KP>(k + t * qkv_stride + (long)g * Dk, i0, Dk, vec, kc);
    load_slice<T, KP>(q + t * qkv_stride + (long)g * Dk, i0, Dk, vec, qc);
    vc = ScalarOps<T>::to_f32(v[t * qkv_stride + (long)h * Dv + colc]);
    const float *pp = prep + t * PW;
    ikc = pp[g]; iqc = pp[G + g]; gc = pp[2 * G + h]; bc = pp[2 * G + H + h];
  }
  for (int t = start; t < end; ++t) {
    // prefetch t + 1 (clamped: the last iteration re-reads row t)
    const long tn = t + 1 < end ? t + 1 : t;
    float kx[KP], qx[KP];
    load_slice<T, KP>(k + tn * qkv_stride + (long)g * Dk, i0, Dk, vec, kx);
    load_slice<T, KP>(q + tn * qkv_stride + (long)g * Dk, i0, Dk, vec, qx);
    const float vx =
        ScalarOps<T>::to_f32(v[tn * qkv_stride + (long)h * Dv + colc]);
    const float *pn = prep + tn * PW;
    const float ikx = pn[g], iqx = pn[G + g], gx = pn[2 * G + h],
                bx = pn[2 * G + H + h];

    float d0 = 0.f, d1 = 0.f, d2 = 0.f, d3 = 0.f;  // 4 chains, not one
#pragma unroll
    for (int r = 0; r < KP; r += 4) {
      d0 += S[r] * kc[r];
      d1 += S[r + 1] * kc[r + 1];
      d2 += S[r + 2] * kc[r + 2];
      d3 += S[r + 3] * kc[r + 3];
    }
    const float sk_dot = quad_sum((d0 + d1) + (d2 + d3)) * (ikc * gc);
    const float c = bc * (vc - sk_dot) * ikc;
    float e0 = 0.f, e1 = 0.f, e2 = 0.f, e3 = 0.f;
#pragma unroll
    for (int r = 0; r < KP; r += 4) {
      S[r] = S[r] * gc + kc[r] * c;
      S[r + 1] = S[r + 1] * gc + kc[r + 1] * c;
      S[r + 2] = S[r + 2] * gc + kc[r + 2] * c;
      S[r + 3] = S[r + 3] * gc + kc[r + 3] * c;
      e0 += S[r] * qc[r];
      e1 += S[r + 1] * qc[r + 1];
      e2 += S[r + 2] * qc[r + 2];
      e3 += S[r + 3] * qc[r + 3];
    }
    const float od = quad_sum((e0 + e1) + (e2 + e3)) * iqc;
    if (live && part == 0) o[((long)t * H + h) * Dv + col] = od;
#pragma unroll
    for (int r = 0; r < KP; ++r) {
      kc[r] = kx[r];
      qc[r] = qx[r];
    }
    vc = vx; ikc = ikx; iqc = iqx; gc = gx; bc = bx;
  }
  if (live) {
#pragma unroll
    for (int r = 0; r < KP; ++r) {
      const int i = i0 + r;
      if (i < Dk) sp[(long)i * Dv + col] = S[r];
    }
  }
}

// Prompt-portion form of the same recurrence: the 4 waves of a workgroup
// share q, k (one kv head) and the per-token scalars, so tiles of TT
// tokens are staged once per workgroup into LDS as fp32 (double buffered:
// the next tile's global loads are in flight while the current one is
// computed) and every lane reads its key slice with 16 B LDS loads. The
// arithmetic per token is exactly delta_rule_varlen_kernel's.
// grid (B, H, ceil(Dv / 64)), block 256.
template <typename T, int KP>
__global__ __launch_bounds__(256) void delta_rule_tiled_kernel(
    float *__restrict__ o, const T *__restrict__ q, const T *__restrict__ k,
    const T *__restrict__ v, long qkv_stride, const float *__restrict__ prep,
    float *__restrict__ state, const long *__restrict__ slots,
    const int *__restrict__ has_init, const int *__restrict__ qsl, int H,
    int G, int Dk, int Dv) {
  constexpr int TT = KP == 64 ? 8 : 16;   // tokens per tile
  constexpr int KPP = KP + 4;             // padded slice: no bank clash
  constexpr int DKP = 4 * KP;             // padded key size
  constexpr int KQ_T = 2 * 4 * KPP;       // floats per token: [k|q][part]
  constexpr int TOK_F = KQ_T + 64 + 4;    // + v columns + 4 scalars
  constexpr int PER = TT * 2 * DKP / 256; // k/q elements per thread, tile
  constexpr int VPER = TT * 64 / 256;
  __shared__ __attribute__((aligned(16))) float lds[2][TT * TOK_F];

  const int b = blockIdx.x, h = blockIdx.y;
  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int vcol = wave * 16 + (lane >> 2);  // column inside the 64 block
  const int col = blockIdx.z * 64 + vcol;
  const int part = lane & 3;
  const int i0 = part * KP;
  const int g = h / (H / G);
  const int start = qsl[b], end = qsl[b + 1];
  if (start >= end) return;
  const bool live = col < Dv;
  const int colc = live ? col : Dv - 1;
  const int PW = 2 * G + 2 * H;

  float *sp = state + ((long)slots[b] * H + h) * Dk * Dv;
  float S[KP];
  const bool init = has_init[b] != 0;
#pragma unroll
  for (int r = 0; r < KP; ++r) {
    const int i = i0 + r;
    S[r] = (init && i < Dk) ? sp[(long)i * Dv + colc] : 0.f;
  }

  T stg[PER];
  T stg_v[VPER];
  float stg_s = 0.f;
  auto stage_load = [&](int tile0) {
#pragma unroll
    for (int j = 0; j < PER; ++j) {
      const int idx = j * 256 + tid;
      const int tt = idx / (2 * DKP);
      const int w = (idx / DKP) & 1;
      const int i = idx % DKP;
      const long t = tile0 + tt;
      const T *src = w ? q : k;
      stg[j] = (i < Dk && t < end) ? src[t * qkv_stride + (long)g * Dk + i]
                                   : ScalarOps<T>::from_f32(0.f);
    }
#pragma unroll
    for (int j = 0; j < VPER; ++j) {
      const int idx = j * 256 + tid;
      const int tt = idx / 64, c = blockIdx.z * 64 + idx % 64;
      const long t = tile0 + tt;
      stg_v[j] = (c < Dv && t < end)
                     ? v[t * qkv_stride + (long)h * Dv + c]
                     : ScalarOps<T>::from_f32(0.f);
    }
    if (tid < TT * 4) {
      const int tt = tid >> 2, which = tid & 3;
      const long t = tile0 + tt < end ? tile0 + tt : end - 1;
      const float *pp = prep + t * PW;
      stg_s = which == 0 ? pp[g] : which == 1 ? pp[G + g]
              : which == 2 ? pp[2 * G + h] : pp[2 * G + H + h];
    }
  };
  auto stage_store = [&](float *buf) {
#pragma unroll
    for (int j = 0; j < PER; ++j) {
      const int idx = j * 256 + tid;
      const int tt = idx / (2 * DKP);
      const int w = (idx / DKP) & 1;
      const int i = idx % DKP;
      buf[tt * TOK_F + (w * 4 + i / KP) * KPP + i % KP] =
          ScalarOps<T>::to_f32(stg[j]);
    }
#pragma unroll
    for (int j = 0; j < VPER; ++j) {
      const int idx = j * 256 + tid;
      buf[(idx / 64) * TOK_F + KQ_T + idx % 64] =
          ScalarOps<T>::to_f32(stg_v[j]);
    }
    if (tid < TT * 4) buf[(tid >> 2) * TOK_F + KQ_T + 64 + (tid & 3)] = stg_s;
  };

  stage_load(start);
  stage_store(lds[0]);
  __syncthreads();
  int cur = 0;
  for (int tile0 = start; tile0 < end; tile0 += TT) {
    const bool more = tile0 + TT < end;
    if (more) stage_load(tile0 + TT);
    const int n = end - tile0 < TT ? end - tile0 : TT;
    const float *buf = lds[cur];
    for (int tt = 0; tt < n; ++tt) {
      const float *tok = buf + tt * TOK_F;
      const floatx4 *kp4 =
          reinterpret_cast<const floatx4 *>(tok + part * KPP);
      const floatx4 *qp4 =
          reinterpret_cast<const floatx4 *>(tok + (4 + part) * KPP);
      const float vc = tok[KQ_T + vcol];
      const float ikc = tok[KQ_T + 64], iqc = tok[KQ_T + 65];
      const float gc = tok[KQ_T + 66], bc = tok[KQ_T + 67];
      float kc[KP];
      float d0 = 0.f, d1 = 0.f, d2 = 0.f, d3 = 0.f;
#pragma unroll
      for (int r = 0; r < KP; r += 4) {
        const floatx4 kk = kp4[r / 4];
        kc[r] = kk[0]; kc[r + 1] = kk[1]; kc[r + 2] = kk[2]; kc[r + 3] = kk[3];
        d0 += S[r] * kk[0];
        d1 += S[r + 1] * kk[1];
        d2 += S[r + 2] * kk[2];
        d3 += S[r + 3] * kk[3];
      }
      const float sk_dot = quad_sum((d0 + d1) + (d2 + d3)) * (ikc * gc);
      const float c = bc * (vc - sk_dot) * ikc;
      float e0 = 0.f, e1 = 0.f, e2 = 0.f, e3 = 0.f;
#pragma unroll
      for (int r = 0; r < KP; r += 4) {
        const floatx4 qq = qp4[r / 4];
        S[r] = S[r] * gc + kc[r] * c;
        S[r + 1] = S[r + 1] * gc + kc[r + 1] * c;
        S[r + 2] = S[r + 2] * gc + kc[r + 2] * c;
        S[r + 3] = S[r + 3] * gc + kc[r + 3] * c;
        e0 += S[r] * qq[0];
        e1 += S[r + 1] * qq[1];
        e2 += S[r + 2] * qq[2];
        e3 += S[r + 3] * qq[3];
      }
      const float od = quad_sum((e0 + e1) + (e2 + e3)) * iqc;
      if (live && part == 0)
        o[((long)(tile0 + tt) * H + h) * Dv + col] = od;
    }
    if (more) stage_store(lds[cur ^ 1]);
    __syncthreads();
    cur ^= 1;
  }
  if (live) {
#pragma unroll
    for (int r = 0; r < KP; ++r) {
      const int i = i0 + r;
      if (i < Dk) sp[(long)i * Dv + col] = S[r];
    }
  }
}

DEV_INLINE float gate_act(float z, int sig) {
  return sig ? 1.0f / (1.0f + expf(-z)) : silu_f(z);
}

// grid (tokens * H); block 64: out = scale * o / rms(o) * w * act(z);
// w_hs = 0: one weight row for all heads, Dv: a row per head
template <typename T>
__global__ __launch_bounds__(64) void rms_gate_kernel(
    T *__restrict__ out, long out_stride, const float *__restrict__ o,
    const T *__restrict__ z, long z_stride, const T *__restrict__ w,
    int w_hs, int H, int Dv, float eps, int sig, float scale) {
  const long th = blockIdx.x;
  const long t = th / H;
  const int h = th % H;
  const float *orow = o + th * Dv;
  float ss = 0.f;
  for (int d = threadIdx.x; d < Dv; d += 64) ss += orow[d] * orow[d];
  ss = wave_reduce_sum(ss);
  const float inv = scale / sqrtf(ss / Dv + eps);
  for (int d = threadIdx.x; d < Dv; d += 64) {
    const float zz = ScalarOps<T>::to_f32(z[t * z_stride + (long)h * Dv + d]);
    out[t * out_stride + (long)h * Dv + d] = ScalarOps<T>::from_f32(
        orow[d] * inv * ScalarOps<T>::to_f32(w[(long)h * w_hs + d]) *
        gate_act(zz, sig));
  }
}

// 8 elements per lane, LPR = Dv / 8 lanes per (token, head) row;
// grid ceil(rows / (256 / LPR)), block 256
template <typename T, int LPR>
__global__ __launch_bounds__(256) void rms_gate8_kernel(
    T *__restrict__ out, long out_stride, const float *__restrict__ o,
    const T *__restrict__ z, long z_stride, const T *__restrict__ w,
    int w_hs, int H, long rows, float eps, int sig, float scale) {
  constexpr int Dv = LPR * 8;
  const long th = (long)blockIdx.x * (256 / LPR) + threadIdx.x / LPR;
  const int d0 = (threadIdx.x % LPR) * 8;
  const bool ok = th < rows;
  const long thc = ok ? th : rows - 1;  // whole groups take the reduction
  const long t = thc / H;
  const int h = thc % H;
  float of[8], zf[8], wf[8];
  ld8<float>(o + thc * Dv + d0, of);
  float ss = 0.f;
#pragma unroll
  for (int e = 0; e < 8; ++e) ss += of[e] * of[e];
  ss = group_reduce_sum<LPR>(ss);
  const float inv = scale / sqrtf(ss / Dv + eps);
  ld8<T>(z + t * z_stride + (long)h * Dv + d0, zf);
  ld8<T>(w + (long)h * w_hs + d0, wf);
#pragma unroll
  for (int e = 0; e < 8; ++e)
    of[e] = of[e] * inv * wf[e] * gate_act(zf[e], sig);
  if (ok) st8<T>(out + t * out_stride + (long)h * Dv + d0, of);
}

// ------------------------------------------------------------------
// Token shift. grid (tokens, ceil(W / (256 * EPT))), EPT = 8 (16 B
// accesses) or 1. Row t of sequence b reads row t - 1 of the same
// portion, or the slot's state row when it opens the portion (zeros when
// the sequence starts here). `store` != 0 (every portion is one token):
// the same thread then leaves its incoming values in the state, so one
// launch does both; longer portions roll the state in a second launch
// (another workgroup may still have to read the old row).
template <typename T, int EPT>
__global__ __launch_bounds__(256) void token_shift_kernel(
    T *__restrict__ out, const T *__restrict__ h, long h_stride,
    const T *__restrict__ mu, T *__restrict__ state,
    const long *__restrict__ slots, const int *__restrict__ has_init,
    const int *__restrict__ qsl, int B, int W, int store) {
  const int t = blockIdx.x;
  const int c0 = (blockIdx.y * 256 + threadIdx.x) * EPT;
  if (c0 >= W) return;
  const int b = find_seq(qsl, B, t);
  const bool first = t == qsl[b];
  T *st = state + (long)slots[b] * W + c0;
  float cur[EPT], prev[EPT], m[EPT];
  if (EPT == 8) {
    ld8<T>(h + (long)t * h_stride + c0, cur);
    ld8<T>(mu + c0, m);
    if (!first) ld8<T>(h + (long)(t - 1) * h_stride + c0, prev);
    else if (has_init[b] != 0) ld8<T>(st, prev);
    else {
#pragma unroll
      for (int e = 0; e < EPT; ++e) prev[e] = 0.f;
    }
  } else {
    cur[0] = ScalarOps<T>::to_f32(h[(long)t * h_stride + c0]);
    m[0] = ScalarOps<T>::to_f32(mu[c0]);
    prev[0] = !first ? ScalarOps<T>::to_f32(h[(long)(t - 1) * h_stride + c0])
              : has_init[b] != 0 ? ScalarOps<T>::to_f32(st[0]) : 0.f;
  }
  float res[EPT];
#pragma unroll
  for (int e = 0; e < EPT; ++e) res[e] = cur[e] + (prev[e] - cur[e]) * m[e];
  if (EPT == 8) {
    st8<T>(out + (long)t * W + c0, res);
    if (store) st8<T>(st, cur);
  } else {
    out[(long)t * W + c0] = ScalarOps<T>::from_f32(res[0]);
    if (store) st[0] = ScalarOps<T>::from_f32(cur[0]);
  }
}

// grid (B, ceil(W / 256)): state[slot] <- last incoming row of the portion
template <typename T>
__global__ __launch_bounds__(256) void shift_state_kernel(
    T *__restrict__ state, const T *__restrict__ h, long h_stride,
    const long *__restrict__ slots, const int *__restrict__ qsl, int W) {
  const int b = blockIdx.x;
  const int c = blockIdx.y * 256 + threadIdx.x;
  if (c >= W || qsl[b + 1] <= qsl[b]) return;
  state[(long)slots[b] * W + c] = h[(long)(qsl[b + 1] - 1) * h_stride + c];
}

// ------------------------------------------------------------------
// Per-token operands of the generalized delta rule, once per (token,
// head) instead of once per wave that needs them:
//   prep[t, 0, h, i] = w  = exp(-c * sigmoid(w_logit + w0))
//   prep[t, 1, h, i] = ak = sigmoid(a_logit) * k / (|k|^2 + 1e-6)
// (removal rate times the unit key, times the unit key's own 1/|k|, so
// the recurrence takes d = k^T S on the raw key). grid (tokens, H), block 64.
template <typename T>
__global__ __launch_bounds__(64) void general_delta_prep_kernel(
    float *__restrict__ prep, const T *__restrict__ k, long k_stride,
    const T *__restrict__ wl, long wl_stride, const T *__restrict__ al,
    long al_stride, const T *__restrict__ w0, int H, int D, float c) {
  const long t = blockIdx.x;
  const int h = blockIdx.y, lane = threadIdx.x;
  const T *kr = k + t * k_stride + (long)h * D;
  float ss = 0.f;
  for (int i = lane; i < D; i += 64) {
    const float kv = ScalarOps<T>::to_f32(kr[i]);
    ss += kv * kv;
  }
  const float ik2 = 1.0f / (wave_reduce_sum(ss) + 1e-6f);
  float *pw = prep + (t * 2 * H + h) * D;
  float *pa = pw + (long)H * D;
  for (int i = lane; i < D; i += 64) {
    const float z = ScalarOps<T>::to_f32(wl[t * wl_stride + (long)h * D + i]) +
                    ScalarOps<T>::to_f32(w0[(long)h * D + i]);
    pw[i] = expf(-c / (1.0f + expf(-z)));
    const float a = 1.0f / (1.0f + expf(-ScalarOps<T>::to_f32(
                                     al[t * al_stride + (long)h * D + i])));
    pa[i] = a * ScalarOps<T>::to_f32(kr[i]) * ik2;
  }
}

// grid (B, H, ceil(Dv / 64)), block 256 = 4 independent waves; lane layout
// of delta_rule_varlen_kernel: a wave owns 16 state columns, a quad of
// lanes shares a column and splits the key axis in 4 slices of KP. Per token
//   d = k^T S[:, col];  S[i, col] <- w_i S[i, col] - ak_i d + k_i v_col;
//   o_col = r^T S[:, col]
// This is the form for decode-only batches (one token per sequence; it
// walks longer portions too): no pre-pass, every lane forms decay and
// removal rate of its own key slice from the logits, and the quad that
// shares a column holds the whole key, so |k|^2 is one quad sum.
template <typename T, int KP>
__global__ __launch_bounds__(256) void general_delta_kernel(
    float *__restrict__ o, const T *__restrict__ r, const T *__restrict__ k,
    const T *__restrict__ v, long rkv_stride, const T *__restrict__ wl,
    long wl_stride, const T *__restrict__ al, long al_stride,
    const T *__restrict__ w0, float c, float *__restrict__ state,
    const long *__restrict__ slots, const int *__restrict__ has_init,
    const int *__restrict__ qsl, int H, int Dk, int Dv, int vec, int vec_l) {
  const int b = blockIdx.x, h = blockIdx.y;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int col = blockIdx.z * 64 + wave * 16 + (lane >> 2);
  const int part = lane & 3;
  const int i0 = part * KP;
  const int start = qsl[b], end = qsl[b + 1];
  const bool live = col < Dv;
  const int colc = live ? col : Dv - 1;  // clamp loads, mask stores
  if (blockIdx.z * 64 + wave * 16 >= Dv) return;  // whole wave idle
  if (start >= end) return;

  float *sp = state + ((long)slots[b] * H + h) * Dk * Dv;
  float S[KP];
  const bool init = has_init[b] != 0;
#pragma unroll
  for (int i = 0; i < KP; ++i)
    S[i] = (init && i0 + i < Dk) ? sp[(long)(i0 + i) * Dv + colc] : 0.f;
  float w0c[KP];
  load_slice<T, KP>(w0 + (long)h * Dk, i0, Dk, vec_l, w0c);

  for (int t = start; t < end; ++t) {
    float kc[KP], rc[KP], wc[KP], ac[KP];
    load_slice<T, KP>(k + t * rkv_stride + (long)h * Dk, i0, Dk, vec, kc);
    load_slice<T, KP>(r + t * rkv_stride + (long)h * Dk, i0, Dk, vec, rc);
    load_slice<T, KP>(wl + t * wl_stride + (long)h * Dk, i0, Dk, vec_l, wc);
    load_slice<T, KP>(al + t * al_stride + (long)h * Dk, i0, Dk, vec_l, ac);
    const float vc =
        ScalarOps<T>::to_f32(v[t * rkv_stride + (long)h * Dv + colc]);
    float ss = 0.f;
    float d0 = 0.f, d1 = 0.f, d2 = 0.f, d3 = 0.f;  // 4 chains, not one
#pragma unroll
    for (int i = 0; i < KP; i += 4) {
      ss += kc[i] * kc[i] + kc[i + 1] * kc[i + 1] + kc[i + 2] * kc[i + 2] +
            kc[i + 3] * kc[i + 3];
      d0 += S[i] * kc[i];
      d1 += S[i + 1] * kc[i + 1];
      d2 += S[i + 2] * kc[i + 2];
      d3 += S[i + 3] * kc[i + 3];
    }
    const float ik2 = 1.0f / (quad_sum(ss) + 1e-6f);
    const float d = quad_sum((d0 + d1) + (d2 + d3)) * ik2;
    float e0 = 0.f, e1 = 0.f;
#pragma unroll
    for (int i = 0; i < KP; i += 2) {
#pragma unroll
      for (int u = 0; u < 2; ++u) {
        const float w = expf(-c / (1.0f + expf(-(wc[i + u] + w0c[i + u]))));
        const float a = 1.0f / (1.0f + expf(-ac[i + u]));
        S[i + u] = S[i + u] * w - a * kc[i + u] * d + kc[i + u] * vc;
      }
      e0 += S[i] * rc[i];
      e1 += S[i + 1] * rc[i + 1];
    }
    const float od = quad_sum(e0 + e1);
    if (live && part == 0) o[((long)t * H + h) * Dv + col] = od;
  }
  if (live) {
#pragma unroll
    for (int i = 0; i < KP; ++i)
      if (i0 + i < Dk) sp[(long)(i0 + i) * Dv + col] = S[i];
  }
}

// Prompt-portion form of general_delta_kernel: the 4 waves of a workgroup
// share k, r and the fp32 decay / removal rows of their head, so tiles of
// TT tokens are staged once per workgroup into LDS as fp32 (double
// buffered: the next tile's global loads are in flight while the current
// one is computed) and every lane reads its key slice with 16 B LDS
// loads. The arithmetic per token is exactly general_delta_kernel's.
// grid (B, H, ceil(Dv / 64)), block 256.
template <typename T, int KP>
__global__ __launch_bounds__(256) void general_delta_tiled_kernel(
    float *__restrict__ o, const T *__restrict__ r, const T *__restrict__ k,
    const T *__restrict__ v, long rkv_stride, const float *__restrict__ prep,
    float *__restrict__ state, const long *__restrict__ slots,
    const int *__restrict__ has_init, const int *__restrict__ qsl, int H,
    int Dk, int Dv) {
  constexpr int TT = KP == 64 ? 4 : 8;     // tokens per tile
  constexpr int KPP = KP + 4;              // padded slice: no bank clash
  constexpr int DKP = 4 * KP;              // padded key size
  constexpr int ROW = 4 * KPP;             // one operand row in LDS
  constexpr int TOK_F = 4 * ROW + 64;      // k | r | w | ak | v columns
  constexpr int PER = TT * 2 * DKP / 256;  // k/r (and w/ak) per thread, tile
  constexpr int VPER = TT * 64 / 256;
  __shared__ __attribute__((aligned(16))) float lds[2][TT * TOK_F];

  const int b = blockIdx.x, h = blockIdx.y;
  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int vcol = wave * 16 + (lane >> 2);  // column inside the 64 block
  const int col = blockIdx.z * 64 + vcol;
  const int part = lane & 3;
  const int i0 = part * KP;
  const int start = qsl[b], end = qsl[b + 1];
  if (start >= end) return;
  const bool live = col < Dv;
  const int colc = live ? col : Dv - 1;
  const long PW = 2L * H * Dk;

  float *sp = state + ((long)slots[b] * H + h) * Dk * Dv;
  float S[KP];
  const bool init = has_init[b] != 0;
#pragma unroll
  for (int i = 0; i < KP; ++i)
    S[i] = (init && i0 + i < Dk) ? sp[(long)(i0 + i) * Dv + colc] : 0.f;

  T stg[PER];
  float stg_f[PER];
  T stg_v[VPER];
  auto stage_load = [&](int tile0) {
#pragma unroll
    for (int j = 0; j < PER; ++j) {
      const int idx = j * 256 + tid;
      const int tt = idx / (2 * DKP);
      const int w = (idx / DKP) & 1;
      const int i = idx % DKP;
      const long t = tile0 + tt;
      const bool ok = i < Dk && t < end;
      const T *src = w ? r : k;
      stg[j] = ok ? src[t * rkv_stride + (long)h * Dk + i]
                  : ScalarOps<T>::from_f32(0.f);
      stg_f[j] = ok ? prep[t * PW + ((long)w * H + h) * Dk + i] : 0.f;
    }
#pragma unroll
    for (int j = 0; j < VPER; ++j) {
      const int idx = j * 256 + tid;
      const int tt = idx / 64, c = blockIdx.z * 64 + idx % 64;
      const long t = tile0 + tt;
      stg_v[j] = (c < Dv && t < end)
                     ? v[t * rkv_stride + (long)h * Dv + c]
                     : ScalarOps<T>::from_f32(0.f);
    }
  };
  auto stage_store = [&](float *buf) {
#pragma unroll
    for (int j = 0; j < PER; ++j) {
      const int idx = j * 256 + tid;
      const int tt = idx / (2 * DKP);
      const int w = (idx / DKP) & 1;
      const int i = idx % DKP;
      float *tok = buf + tt * TOK_F + (i / KP) * KPP + i % KP;
      tok[w * ROW] = ScalarOps<T>::to_f32(stg[j]);   // k (w = 0) | r
      tok[(2 + w) * ROW] = stg_f[j];                 // decay | removal
    }
#pragma unroll
    for (int j = 0; j < VPER; ++j) {
      const int idx = j * 256 + tid;
      buf[(idx / 64) * TOK_F + 4 * ROW + idx % 64] =
          ScalarOps<T>::to_f32(stg_v[j]);
    }
  };

  stage_load(start);
  stage_store(lds[0]);
  __syncthreads();
  int cur = 0;
  for (int tile0 = start; tile0 < end; tile0 += TT) {
    const bool more = tile0 + TT < end;
    if (more) stage_load(tile0 + TT);
    const int n = end - tile0 < TT ? end - tile0 : TT;
    const float *buf = lds[cur];
    for (int tt = 0; tt < n; ++tt) {
      const float *tok = buf + tt * TOK_F + part * KPP;
      const floatx4 *kp4 = reinterpret_cast<const floatx4 *>(tok);
      const floatx4 *rp4 = reinterpret_cast<const floatx4 *>(tok + ROW);
      const floatx4 *wp4 = reinterpret_cast<const floatx4 *>(tok + 2 * ROW);
      const floatx4 *ap4 = reinterpret_cast<const floatx4 *>(tok + 3 * ROW);
      const float vc = buf[tt * TOK_F + 4 * ROW + vcol];
      float kc[KP];
      float d0 = 0.f, d1 = 0.f, d2 = 0.f, d3 = 0.f;
#pragma unroll
      for (int i = 0; i < KP; i += 4) {
        const floatx4 kk = kp4[i / 4];
        kc[i] = kk[0]; kc[i + 1] = kk[1]; kc[i + 2] = kk[2]; kc[i + 3] = kk[3];
        d0 += S[i] * kk[0];
        d1 += S[i + 1] * kk[1];
        d2 += S[i + 2] * kk[2];
        d3 += S[i + 3] * kk[3];
      }
      const float d = quad_sum((d0 + d1) + (d2 + d3));
      float e0 = 0.f, e1 = 0.f, e2 = 0.f, e3 = 0.f;
#pragma unroll
      for (int i = 0; i < KP; i += 4) {
        const floatx4 rr = rp4[i / 4];
        const floatx4 ww = wp4[i / 4];
        const floatx4 aa = ap4[i / 4];
        S[i] = S[i] * ww[0] - aa[0] * d + kc[i] * vc;
        S[i + 1] = S[i + 1] * ww[1] - aa[1] * d + kc[i + 1] * vc;
        S[i + 2] = S[i + 2] * ww[2] - aa[2] * d + kc[i + 2] * vc;
        S[i + 3] = S[i + 3] * ww[3] - aa[3] * d + kc[i + 3] * vc;
        e0 += S[i] * rr[0];
        e1 += S[i + 1] * rr[1];
        e2 += S[i + 2] * rr[2];
        e3 += S[i + 3] * rr[3];
      }
      const float od = quad_sum((e0 + e1) + (e2 + e3));
      if (live && part == 0)
        o[((long)(tile0 + tt) * H + h) * Dv + col] = od;
    }
    if (more) stage_store(lds[cur ^ 1]);
    __syncthreads();
    cur ^= 1;
  }
  if (live) {
#pragma unroll
    for (int i = 0; i < KP; ++i)
      if (i0 + i < Dk) sp[(long)(i0 + i) * Dv + col] = S[i];
  }
}

bool rows_ok(const torch::Tensor &t) {
  return t.dim() == 2 && t.stride(1) == 1;
}

}  // namespace

void causal_conv_silu(torch::Tensor out, torch::Tensor x, torch::Tensor w,
                      torch::Tensor conv_state, torch::Tensor slots,
                      torch::Tensor has_init, torch::Tensor query_start_loc,
                      bool activation, long max_query_len) {
  const long T = x.size(0);
  const int C = x.size(1);
  const int taps = w.size(1);
  const int act = activation ? 1 : 0;
  // one token per sequence: the convolution's launch also rolls the state
  const int store = (max_query_len == 1 && T == slots.numel() &&
                     w.size(1) > 1) ? 1 : 0;
  const int B = slots.numel();
  if (T == 0) return;
  const auto st = x.scalar_type();
  TORCH_CHECK(rows_ok(x) && out.is_contiguous() && out.scalar_type() == st &&
              out.numel() == T * C);
  TORCH_CHECK(w.is_contiguous() && w.size(0) == C && w.scalar_type() == st);
  TORCH_CHECK(taps >= 1 && taps <= MAX_TAPS, "conv taps must be 1..8");
  TORCH_CHECK(conv_state.is_contiguous() && conv_state.scalar_type() == st &&
              conv_state.dim() == 3 && conv_state.size(1) == C &&
              conv_state.size(2) == std::max(taps - 1, 1));
  TORCH_CHECK(slots.scalar_type() == at::kLong && slots.is_contiguous());
  TORCH_CHECK(has_init.scalar_type() == at::kInt && has_init.numel() == B);
  TORCH_CHECK(query_start_loc.scalar_type() == at::kInt &&
              query_start_loc.numel() >= B + 1);
  auto stream = at::cuda::getCurrentCUDAStream();
  const int cy = (C + 255) / 256;
  const size_t es = x.element_size();
  const bool vec8 =
      C % 8 == 0 && (x.stride(0) * es) % 16 == 0 &&
      reinterpret_cast<uintptr_t>(x.data_ptr()) % 16 == 0 &&
      reinterpret_cast<uintptr_t>(out.data_ptr()) % 16 == 0 &&
      reinterpret_cast<uintptr_t>(w.data_ptr()) % 16 == 0;
  const int cy8 = (C / 8 + 255) / 256;
#define CONV8(TT, TP)                                                        \
  hipLaunchKernelGGL((causal_conv_silu8_kernel<TT, TP>), dim3(T, cy8),       \
                     dim3(256), 0, stream, (TT *)out.data_ptr(),             \
                     (const TT *)x.data_ptr(), (long)x.stride(0),            \
                     (const TT *)w.data_ptr(), (TT *)conv_state.data_ptr(),  \
                     slots.data_ptr<long>(), has_init.data_ptr<int>(),       \
                     query_start_loc.data_ptr<int>(), B, C, act, store)
#define CONV8_T(TT)                                                          \
  switch (taps) {                                                            \
    case 1: CONV8(TT, 1); break;                                             \
    case 2: CONV8(TT, 2); break;                                             \
    case 3: CONV8(TT, 3); break;                                             \
    case 4: CONV8(TT, 4); break;                                             \
    case 5: CONV8(TT, 5); break;                                             \
    case 6: CONV8(TT, 6); break;                                             \
    case 7: CONV8(TT, 7); break;                                             \
    default: CONV8(TT, 8); break;                                            \
  }
#define RUN(TT)                                                              \
  if (vec8) {                                                                \
    CONV8_T(TT)                                                              \
  } else                                                                     \
    hipLaunchKernelGGL((causal_conv_silu_kernel<TT>), dim3(T, cy),           \
                       dim3(256), 0, stream, (TT *)out.data_ptr(),           \
                       (const TT *)x.data_ptr(), (long)x.stride(0),          \
                       (const TT *)w.data_ptr(), (TT *)conv_state.data_ptr(), \
                       slots.data_ptr<long>(), has_init.data_ptr<int>(),     \
                       query_start_loc.data_ptr<int>(), B, C, taps, act,     \
                       store);                                               \
  if (taps > 1 && !store)                                                              \
    hipLaunchKernelGGL((conv_state_update_kernel<TT>), dim3(B, cy),          \
                       dim3(256), 0, stream, (TT *)conv_state.data_ptr(),    \
                       (const TT *)x.data_ptr(), (long)x.stride(0),          \
                       slots.data_ptr<long>(), has_init.data_ptr<int>(),     \
                       query_start_loc.data_ptr<int>(), C, taps)
  if (st == at::kBFloat16) { RUN(__hip_bfloat16); }
  else if (st == at::kFloat) { RUN(float); }
  else TORCH_CHECK(false, "causal_conv_silu: bf16 or fp32");
#undef RUN
#undef CONV8_T
#undef CONV8
  HIP_CHECK_KERNEL();
}

void delta_rule_varlen(torch::Tensor o, torch::Tensor q, torch::Tensor k,
                       torch::Tensor v, torch::Tensor a, torch::Tensor b,
                       torch::Tensor A_log, torch::Tensor dt_bias,
                       torch::Tensor state, torch::Tensor slots,
                       torch::Tensor has_init, torch::Tensor query_start_loc,
                       double q_scale, long max_query_len) {
  const long T = q.size(0);
  if (T == 0) return;
  const auto st = q.scalar_type();
  TORCH_CHECK(state.dim() == 4 && state.scalar_type() == at::kFloat &&
              state.is_contiguous());
  const int H = state.size(1), Dk = state.size(2), Dv = state.size(3);
  TORCH_CHECK(rows_ok(q) && rows_ok(k) && rows_ok(v) && rows_ok(a) &&
              rows_ok(b));
  TORCH_CHECK(k.scalar_type() == st && v.scalar_type() == st &&
              a.scalar_type() == st && b.scalar_type() == st);
  TORCH_CHECK(q.size(1) % Dk == 0 && k.size(1) == q.size(1));
  const int G = q.size(1) / Dk;
  TORCH_CHECK(G > 0 && H % G == 0 && v.size(1) == (long)H * Dv);
  TORCH_CHECK(q.stride(0) == k.stride(0) && q.stride(0) == v.stride(0),
              "q, k, v must share a row stride (slices of one buffer)");
  TORCH_CHECK(a.size(1) == H && b.size(1) == H && a.stride(0) == b.stride(0));
  TORCH_CHECK(k.size(0) == T && v.size(0) == T && a.size(0) == T &&
              b.size(0) == T);
  TORCH_CHECK(A_log.scalar_type() == at::kFloat && A_log.numel() == H &&
              dt_bias.scalar_type() == at::kFloat && dt_bias.numel() == H);
  TORCH_CHECK(o.scalar_type() == at::kFloat && o.is_contiguous() &&
              o.numel() == T * H * Dv);
  const int B = slots.numel();
  TORCH_CHECK(slots.scalar_type() == at::kLong && slots.is_contiguous());
  TORCH_CHECK(has_init.scalar_type() == at::kInt && has_init.numel() == B);
  TORCH_CHECK(query_start_loc.scalar_type() == at::kInt &&
              query_start_loc.numel() >= B + 1);
  TORCH_CHECK(Dk <= 256, "delta rule: key size <= 256");
  auto stream = at::cuda::getCurrentCUDAStream();
  const dim3 grid(B, H, (Dv + 63) / 64);
  // 16 B vector loads of the per-lane key slices: every slice whole
  // (Dk = 4 KP) and every row / head / slice offset 16 B aligned
  const int kp = Dk <= 32 ? 8 : Dk <= 64 ? 16 : Dk <= 128 ? 32 : 64;
  const size_t es = q.element_size();
  const int vec =
      (Dk == 4 * kp && (q.stride(0) * es) % 16 == 0 && (Dk * es) % 16 == 0 &&
       reinterpret_cast<uintptr_t>(q.data_ptr()) % 16 == 0 &&
       reinterpret_cast<uintptr_t>(k.data_ptr()) % 16 == 0) ? 1 : 0;
  // per-token scalars first: [ik(G) | iq(G) | decay(H) | beta(H)]
  auto prep = torch::empty({T, 2 * G + 2 * H},
                           o.options().dtype(at::kFloat));
#define PREP(TT)                                                             \
  hipLaunchKernelGGL((delta_prep_kernel<TT>), dim3(T), dim3(64), 0, stream,  \
                     prep.data_ptr<float>(), (const TT *)q.data_ptr(),       \
                     (const TT *)k.data_ptr(), (long)q.stride(0),            \
                     (const TT *)a.data_ptr(), (const TT *)b.data_ptr(),     \
                     (long)a.stride(0), A_log.data_ptr<float>(),             \
                     dt_bias.data_ptr<float>(), H, G, Dk, (float)q_scale)
  if (st == at::kBFloat16) PREP(__hip_bfloat16);
  else if (st == at::kFloat) PREP(float);
  else TORCH_CHECK(false, "delta_rule_varlen: bf16 or fp32");
#undef PREP
#define RUN(TT, KPV)                                                         \
  hipLaunchKernelGGL((delta_rule_varlen_kernel<TT, KPV>), grid, dim3(256),   \
                     0, stream, o.data_ptr<float>(),                         \
                     (const TT *)q.data_ptr(), (const TT *)k.data_ptr(),     \
                     (const TT *)v.data_ptr(), (long)q.stride(0),            \
                     prep.data_ptr<float>(), state.data_ptr<float>(),        \
                     slots.data_ptr<long>(), has_init.data_ptr<int>(),       \
                     query_start_loc.data_ptr<int>(), H, G, Dk, Dv, vec)
#define RUNT(TT, KPV)                                                        \
  hipLaunchKernelGGL((delta_rule_tiled_kernel<TT, KPV>), grid, dim3(256),    \
                     0, stream, o.data_ptr<float>(),                         \
                     (const TT *)q.data_ptr(), (const TT *)k.data_ptr(),     \
                     (const TT *)v.data_ptr(), (long)q.stride(0),            \
                     prep.data_ptr<float>(), state.data_ptr<float>(),        \
                     slots.data_ptr<long>(), has_init.data_ptr<int>(),       \
                     query_start_loc.data_ptr<int>(), H, G, Dk, Dv)
  // batches that hold a prompt portion stage tiles through LDS; decode-
  // only batches (one token per sequence) keep everything in registers
  const bool tiled = max_query_len != 1;
#define RUN_KP(TT)                                                           \
  if (tiled) {                                                               \
    if (Dk <= 32) RUNT(TT, 8);                                               \
    else if (Dk <= 64) RUNT(TT, 16);                                         \
    else if (Dk <= 128) RUNT(TT, 32);                                        \
    else RUNT(TT, 64);                                                       \
  } else if (Dk <= 32) RUN(TT, 8);                                           \
  else if (Dk <= 64) RUN(TT, 16);                                            \
  else if (Dk <= 128) RUN(TT, 32);                                           \
  else RUN(TT, 64)
  if (st == at::kBFloat16) { RUN_KP(__hip_bfloat16); }
  else if (st == at::kFloat) { RUN_KP(float); }
  else TORCH_CHECK(false, "delta_rule_varlen: bf16 or fp32");
#undef RUN_KP
#undef RUNT
#undef RUN
  HIP_CHECK_KERNEL();
}

void rms_gate(torch::Tensor out, torch::Tensor o, torch::Tensor z,
              torch::Tensor w, long H, double eps, bool sigmoid_gate,
              double scale) {
  TORCH_CHECK(o.dim() == 3 && o.size(1) == H, "rms_gate: o [T, H, Dv]");
  const int Dv = o.size(2);
  const long rows = o.numel() / std::max(Dv, 1);
  if (rows == 0) return;
  const auto st = out.scalar_type();
  TORCH_CHECK(o.scalar_type() == at::kFloat && o.is_contiguous());
  TORCH_CHECK(rows_ok(out) && out.size(0) * H == rows &&
              out.size(1) == H * Dv, "rms_gate: out [T, H * Dv] rows");
  TORCH_CHECK(w.numel() == Dv || w.numel() == H * Dv,
              "rms_gate: weight [Dv] or [H * Dv]");
  const int w_hs = w.numel() == Dv ? 0 : Dv;
  const int sig = sigmoid_gate ? 1 : 0;
  const long os = out.stride(0);
  TORCH_CHECK(rows_ok(z) && z.scalar_type() == st && z.size(1) == H * Dv &&
              z.size(0) * H == rows);
  TORCH_CHECK(w.scalar_type() == st && w.is_contiguous());
  auto stream = at::cuda::getCurrentCUDAStream();
  const int lpr = Dv / 8;
  const bool vec8 =
      Dv % 8 == 0 && lpr <= 64 && (lpr & (lpr - 1)) == 0 &&
      (z.stride(0) * z.element_size()) % 16 == 0 &&
      reinterpret_cast<uintptr_t>(z.data_ptr()) % 16 == 0 &&
      reinterpret_cast<uintptr_t>(o.data_ptr()) % 16 == 0 &&
      reinterpret_cast<uintptr_t>(out.data_ptr()) % 16 == 0 &&
      (os * out.element_size()) % 16 == 0 &&
      reinterpret_cast<uintptr_t>(w.data_ptr()) % 16 == 0;
  if (vec8) {
    const long blocks = (rows * lpr + 255) / 256;
#define G8(TT, L)                                                            \
  hipLaunchKernelGGL((rms_gate8_kernel<TT, L>), dim3(blocks), dim3(256), 0,  \
                     stream, (TT *)out.data_ptr(), os, o.data_ptr<float>(),  \
                     (const TT *)z.data_ptr(), (long)z.stride(0),            \
                     (const TT *)w.data_ptr(), w_hs, (int)H, rows,           \
                     (float)eps, sig, (float)scale)
#define G8_L(TT)                                                             \
  switch (lpr) {                                                             \
    case 1: G8(TT, 1); break;                                                \
    case 2: G8(TT, 2); break;                                                \
    case 4: G8(TT, 4); break;                                                \
    case 8: G8(TT, 8); break;                                                \
    case 16: G8(TT, 16); break;                                              \
    case 32: G8(TT, 32); break;                                              \
    default: G8(TT, 64); break;                                              \
  }
    if (st == at::kBFloat16) { G8_L(__hip_bfloat16) }
    else if (st == at::kFloat) { G8_L(float) }
    else TORCH_CHECK(false, "rms_gate: bf16 or fp32");
#undef G8_L
#undef G8
    HIP_CHECK_KERNEL();
    return;
  }
#define RUN(TT)                                                              \
  hipLaunchKernelGGL((rms_gate_kernel<TT>), dim3(rows), dim3(64), 0, stream, \
                     (TT *)out.data_ptr(), os, o.data_ptr<float>(),          \
                     (const TT *)z.data_ptr(), (long)z.stride(0),            \
                     (const TT *)w.data_ptr(), w_hs, (int)H, Dv, (float)eps, \
                     sig, (float)scale)
  if (st == at::kBFloat16) RUN(__hip_bfloat16);
  else if (st == at::kFloat) RUN(float);
  else TORCH_CHECK(false, "rms_gate: bf16 or fp32");
#undef RUN
  HIP_CHECK_KERNEL();
}

void token_shift(torch::Tensor out, torch::Tensor h, torch::Tensor mu,
                 torch::Tensor state, torch::Tensor slots,
                 torch::Tensor has_init, torch::Tensor query_start_loc,
                 long max_query_len) {
  const long T = h.size(0);
  if (T == 0) return;
  const int W = h.size(1);
  const auto st = h.scalar_type();
  const int B = slots.numel();
  TORCH_CHECK(h.is_cuda() && rows_ok(h) && out.is_contiguous() &&
              out.scalar_type() == st && out.numel() == T * W);
  TORCH_CHECK(mu.is_contiguous() && mu.numel() == W && mu.scalar_type() == st);
  TORCH_CHECK(state.is_contiguous() && state.dim() == 2 &&
              state.size(1) == W && state.scalar_type() == st,
              "token_shift: state [slots, width] in the dtype of h");
  TORCH_CHECK(slots.scalar_type() == at::kLong && slots.is_contiguous());
  TORCH_CHECK(has_init.scalar_type() == at::kInt && has_init.numel() == B);
  TORCH_CHECK(query_start_loc.scalar_type() == at::kInt &&
              query_start_loc.numel() >= B + 1);
  auto stream = at::cuda::getCurrentCUDAStream();
  const size_t es = h.element_size();
  const bool vec8 =
      W % 8 == 0 && (h.stride(0) * es) % 16 == 0 &&
      reinterpret_cast<uintptr_t>(h.data_ptr()) % 16 == 0 &&
      reinterpret_cast<uintptr_t>(out.data_ptr()) % 16 == 0 &&
      reinterpret_cast<uintptr_t>(mu.data_ptr()) % 16 == 0 &&
      reinterpret_cast<uintptr_t>(state.data_ptr()) % 16 == 0;
  // one token per sequence: the launch that shifts also rolls the state
  const int store = (max_query_len == 1 && T == B) ? 1 : 0;
  const int cy = vec8 ? (W / 8 + 255) / 256 : (W + 255) / 256;
#define RUN(TT, E)                                                           \
  hipLaunchKernelGGL((token_shift_kernel<TT, E>), dim3(T, cy), dim3(256), 0, \
                     stream, (TT *)out.data_ptr(), (const TT *)h.data_ptr(), \
                     (long)h.stride(0), (const TT *)mu.data_ptr(),           \
                     (TT *)state.data_ptr(), slots.data_ptr<long>(),         \
                     has_init.data_ptr<int>(),                               \
                     query_start_loc.data_ptr<int>(), B, W, store)
#define RUN_ALL(TT)                                                          \
  if (vec8) RUN(TT, 8); else RUN(TT, 1);                                     \
  if (!store)                                                                \
    hipLaunchKernelGGL((shift_state_kernel<TT>), dim3(B, (W + 255) / 256),   \
                       dim3(256), 0, stream, (TT *)state.data_ptr(),         \
                       (const TT *)h.data_ptr(), (long)h.stride(0),          \
                       slots.data_ptr<long>(),                               \
                       query_start_loc.data_ptr<int>(), W)
  if (st == at::kBFloat16) { RUN_ALL(__hip_bfloat16); }
  else if (st == at::kFloat) { RUN_ALL(float); }
  else TORCH_CHECK(false, "token_shift: bf16 or fp32");
#undef RUN_ALL
#undef RUN
  HIP_CHECK_KERNEL();
}

void general_delta_rule(torch::Tensor o, torch::Tensor r, torch::Tensor k,
                        torch::Tensor v, torch::Tensor w_logit,
                        torch::Tensor a_logit, torch::Tensor w0,
                        double decay_scale, torch::Tensor state,
                        torch::Tensor slots, torch::Tensor has_init,
                        torch::Tensor query_start_loc, long max_query_len) {
  const long T = r.size(0);
  if (T == 0) return;
  const auto st = r.scalar_type();
  TORCH_CHECK(state.dim() == 4 && state.scalar_type() == at::kFloat &&
              state.is_contiguous());
  const int H = state.size(1), Dk = state.size(2), Dv = state.size(3);
  TORCH_CHECK(r.is_cuda() && rows_ok(r) && rows_ok(k) && rows_ok(v) &&
              rows_ok(w_logit) && rows_ok(a_logit));
  TORCH_CHECK(k.scalar_type() == st && v.scalar_type() == st &&
              w_logit.scalar_type() == st && a_logit.scalar_type() == st &&
              w0.scalar_type() == st);
  TORCH_CHECK(r.size(1) == (long)H * Dk && k.size(1) == (long)H * Dk &&
              v.size(1) == (long)H * Dv && w_logit.size(1) == (long)H * Dk &&
              a_logit.size(1) == (long)H * Dk && w0.numel() == (long)H * Dk &&
              w0.is_contiguous(), "general_delta_rule: operand widths");
  TORCH_CHECK(k.size(0) == T && v.size(0) == T && w_logit.size(0) == T &&
              a_logit.size(0) == T);
  TORCH_CHECK(r.stride(0) == k.stride(0) && r.stride(0) == v.stride(0),
              "r, k, v must share a row stride (slices of one buffer)");
  TORCH_CHECK(o.scalar_type() == at::kFloat && o.is_contiguous() &&
              o.numel() == T * H * Dv);
  const int B = slots.numel();
  TORCH_CHECK(slots.scalar_type() == at::kLong && slots.is_contiguous());
  TORCH_CHECK(has_init.scalar_type() == at::kInt && has_init.numel() == B);
  TORCH_CHECK(query_start_loc.scalar_type() == at::kInt &&
              query_start_loc.numel() >= B + 1);
  TORCH_CHECK(Dk <= 256, "general delta rule: key size <= 256");
  auto stream = at::cuda::getCurrentCUDAStream();
  // batches that hold a prompt portion stage tiles through LDS after a
  // per-token pre-pass; decode-only batches (one token per sequence) keep
  // everything in registers and form decay / removal rate in the lane
  const bool tiled = max_query_len != 1;
  torch::Tensor prep;
  if (tiled) {
    prep = torch::empty({T, 2, H, Dk}, o.options().dtype(at::kFloat));
#define PREP(TT)                                                             \
  hipLaunchKernelGGL((general_delta_prep_kernel<TT>), dim3(T, H), dim3(64),  \
                     0, stream, prep.data_ptr<float>(),                      \
                     (const TT *)k.data_ptr(), (long)k.stride(0),            \
                     (const TT *)w_logit.data_ptr(), (long)w_logit.stride(0), \
                     (const TT *)a_logit.data_ptr(), (long)a_logit.stride(0), \
                     (const TT *)w0.data_ptr(), H, Dk, (float)decay_scale)
    if (st == at::kBFloat16) PREP(__hip_bfloat16);
    else if (st == at::kFloat) PREP(float);
    else TORCH_CHECK(false, "general_delta_rule: bf16 or fp32");
#undef PREP
  }
  const dim3 grid(B, H, (Dv + 63) / 64);
  const int kp = Dk <= 32 ? 8 : Dk <= 64 ? 16 : Dk <= 128 ? 32 : 64;
  const size_t es = r.element_size();
  // 16 B vector loads of the per-lane slices: every slice whole and every
  // row / head / slice offset 16 B aligned (vec: r, k; vec_l: the logit
  // rows and w0)
  auto al16 = [](const torch::Tensor &t) {
    return reinterpret_cast<uintptr_t>(t.data_ptr()) % 16 == 0;
  };
  const bool whole = Dk == 4 * kp && (Dk * es) % 16 == 0;
  const int vec = (whole && (r.stride(0) * es) % 16 == 0 && al16(r) &&
                   al16(k)) ? 1 : 0;
  const int vec_l = (whole && (w_logit.stride(0) * es) % 16 == 0 &&
                     (a_logit.stride(0) * es) % 16 == 0 && al16(w_logit) &&
                     al16(a_logit) && al16(w0)) ? 1 : 0;
#define RUN(TT, KPV)                                                         \
  hipLaunchKernelGGL((general_delta_kernel<TT, KPV>), grid, dim3(256), 0,    \
                     stream, o.data_ptr<float>(), (const TT *)r.data_ptr(),  \
                     (const TT *)k.data_ptr(), (const TT *)v.data_ptr(),     \
                     (long)r.stride(0), (const TT *)w_logit.data_ptr(),      \
                     (long)w_logit.stride(0),                                \
                     (const TT *)a_logit.data_ptr(),                         \
                     (long)a_logit.stride(0), (const TT *)w0.data_ptr(),     \
                     (float)decay_scale, state.data_ptr<float>(),            \
                     slots.data_ptr<long>(), has_init.data_ptr<int>(),       \
                     query_start_loc.data_ptr<int>(), H, Dk, Dv, vec, vec_l)
#define RUNT(TT, KPV)                                                        \
  hipLaunchKernelGGL((general_delta_tiled_kernel<TT, KPV>), grid, dim3(256), \
                     0, stream, o.data_ptr<float>(),                         \
                     (const TT *)r.data_ptr(), (const TT *)k.data_ptr(),     \
                     (const TT *)v.data_ptr(), (long)r.stride(0),            \
                     prep.data_ptr<float>(), state.data_ptr<float>(),        \
                     slots.data_ptr<long>(), has_init.data_ptr<int>(),       \
                     query_start_loc.data_ptr<int>(), H, Dk, Dv)
#define RUN_KP(TT)                                                           \
  if (tiled) {                                                               \
    if (Dk <= 32) RUNT(TT, 8);                                               \
    else if (Dk <= 64) RUNT(TT, 16);                                         \
    else if (Dk <= 128) RUNT(TT, 32);                                        \
    else RUNT(TT, 64);                                                       \
  } else if (Dk <= 32) RUN(TT, 8);                                           \
  else if (Dk <= 64) RUN(TT, 16);                                            \
  else if (Dk <= 128) RUN(TT, 32);                                           \
  else RUN(TT, 64)
  if (st == at::kBFloat16) { RUN_KP(__hip_bfloat16); }
  else if (st == at::kFloat) { RUN_KP(float); }
  else TORCH_CHECK(false, "general_delta_rule: bf16 or fp32");
#undef RUN_KP
#undef RUNT
#undef RUN
  HIP_CHECK_KERNEL();
}
