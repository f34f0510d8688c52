// Hyper-connections over an fp32 multi-stream residual, gfx950.
//
// The residual of a token is S parallel streams x_1..x_S (fp32,
// xs [S, T, W]). A sublayer reads one mixture of them through an RMS
// norm whose gain is ONE number, and its result is written back into
// every stream while the streams are mixed among themselves:
//
//   hyper_read    h = g * u / sqrt(mean(u^2) + eps),  u = sum_s a[s] x_s
//   hyper_write   x_t <- sum_s M[s, t] x_s + b[t] * y   (all t at once,
//                 from the old streams), y = y1 [+ sigmoid(gate) * y2]
//                 with one gate logit per row; optionally followed, in
//                 the same launch, by the NEXT sublayer's hyper_read of
//                 the updated streams (a', g')
//
// S = 1 with a = b = M = 1 is the ordinary pre-norm residual. All
// arithmetic is fp32; y and h are in the model dtype (bf16 or fp32).
// One workgroup per token row; the row's read mixture is kept in LDS
// between the two passes of the norm.

#include <torch/extension.h>
#include <ATen/cuda/CUDAContext.h>
#include "common.h"

namespace {

constexpr int HY_BLOCK = 256;
constexpr int MAX_S = 8;

// 4 consecutive elements <-> fp32 (8 B for 16-bit types, 16 B for fp32)
template <typename T> DEV_INLINE void ld4(const T *p, float *f) {
  const shortx4 v = *reinterpret_cast<const shortx4 *>(p);
  const T *e = reinterpret_cast<const T *>(&v);
#pragma unroll
  for (int i = 0; i < 4; ++i) f[i] = ScalarOps<T>::to_f32(e[i]);
}
template <> DEV_INLINE void ld4<float>(const float *p, float *f) {
  const floatx4 v = *reinterpret_cast<const floatx4 *>(p);
  f[0] = v[0]; f[1] = v[1]; f[2] = v[2]; f[3] = v[3];
}
template <typename T> DEV_INLINE void st4(T *p, const float *f) {
  shortx4 v;
  T *e = reinterpret_cast<T *>(&v);
#pragma unroll
  for (int i = 0; i < 4; ++i) e[i] = ScalarOps<T>::from_f32(f[i]);
  *reinterpret_cast<shortx4 *>(p) = v;
}
template <> DEV_INLINE void st4<float>(float *p, const float *f) {
  *reinterpret_cast<floatx4 *>(p) = floatx4{f[0], f[1], f[2], f[3]};
}

// V = 4: four columns per thread through 8 / 16 B accesses (W % 4 == 0,
// aligned rows); V = 1: element by element.
template <typename T, int V>
__global__ __launch_bounds__(HY_BLOCK) void hyper_kernel(
    float *__restrict__ xs, long stream_stride, int S, int W,
    // write part (y == nullptr: read only)
    const T *__restrict__ y, long y_stride, const T *__restrict__ y2,
    long y2_stride, const T *__restrict__ gate, long gate_stride,
    const float *__restrict__ mix, const float *__restrict__ out_w,
    // read part (h == nullptr: write only)
    T *__restrict__ h, const float *__restrict__ in_w,
    const float *__restrict__ g, float eps) {
  extern __shared__ float u_row[];  // [W]
  __shared__ float red[HY_BLOCK / WAVE_SIZE];
  __shared__ float coef[MAX_S * MAX_S + 2 * MAX_S];
  const long t = blockIdx.x;
  const int tid = threadIdx.x;
  float *m_s = coef, *b_s = coef + MAX_S * MAX_S, *a_s = b_s + MAX_S;
  if (tid < S * S) m_s[tid] = y ? mix[tid] : 0.f;
  if (tid < S) {
    b_s[tid] = y ? out_w[tid] : 0.f;
    a_s[tid] = h ? in_w[tid] : 0.f;
  }
  __syncthreads();
  float gy = 1.f;
  if (y2 != nullptr && gate != nullptr) {
    const float z = ScalarOps<T>::to_f32(gate[t * gate_stride]);
    gy = 1.0f / (1.0f + expf(-z));
  }
  float ss = 0.f;
  for (int c = tid * V; c < W; c += HY_BLOCK * V) {
    float old[MAX_S][V];
#pragma unroll
    for (int s = 0; s < MAX_S; ++s)
      if (s < S) {
        if (V == 4) ld4<float>(xs + s * stream_stride + t * W + c, old[s]);
        else old[s][0] = xs[s * stream_stride + t * W + c];
      }
    float u[V];
#pragma unroll
    for (int e = 0; e < V; ++e) u[e] = 0.f;
    if (y != nullptr) {
      float yv[V];
      if (V == 4) ld4<T>(y + t * y_stride + c, yv);
      else yv[0] = ScalarOps<T>::to_f32(y[t * y_stride + c]);
      if (y2 != nullptr) {
        float y2v[V];
        if (V == 4) ld4<T>(y2 + t * y2_stride + c, y2v);
        else y2v[0] = ScalarOps<T>::to_f32(y2[t * y2_stride + c]);
#pragma unroll
        for (int e = 0; e < V; ++e) yv[e] += gy * y2v[e];
      }
#pragma unroll
      for (int to = 0; to < MAX_S; ++to) {
        if (to >= S) break;
        float nv[V];
#pragma unroll
        for (int e = 0; e < V; ++e) nv[e] = b_s[to] * yv[e];
#pragma unroll
        for (int s = 0; s < MAX_S; ++s)
          if (s < S) {
#pragma unroll
            for (int e = 0; e < V; ++e) nv[e] += m_s[s * S + to] * old[s][e];
          }
        if (V == 4) st4<float>(xs + to * stream_stride + t * W + c, nv);
        else xs[to * stream_stride + t * W + c] = nv[0];
#pragma unroll
        for (int e = 0; e < V; ++e) u[e] += a_s[to] * nv[e];
      }
    } else {
#pragma unroll
      for (int s = 0; s < MAX_S; ++s)
        if (s < S) {
#pragma unroll
          for (int e = 0; e < V; ++e) u[e] += a_s[s] * old[s][e];
        }
    }
    if (h != nullptr) {
#pragma unroll
      for (int e = 0; e < V; ++e) {
        u_row[c + e] = u[e];
        ss += u[e] * u[e];
      }
    }
  }
  if (h == nullptr) return;
  ss = block_reduce_sum<HY_BLOCK>(ss, red);
  const float k = g[0] / sqrtf(ss / W + eps);
  for (int c = tid * V; c < W; c += HY_BLOCK * V) {
    if (V == 4) {
      float o[4];
#pragma unroll
      for (int e = 0; e < 4; ++e) o[e] = u_row[c + e] * k;
      st4<T>(h + t * W + c, o);
    } else {
      h[t * W + c] = ScalarOps<T>::from_f32(u_row[c] * k);
    }
  }
}

const float *f32_vec(const c10::optional<torch::Tensor> &t, long n,
                     const char *what) {
  TORCH_CHECK(t.has_value(), what, " is required");
  TORCH_CHECK(t->is_cuda() && t->scalar_type() == at::kFloat &&
              t->is_contiguous() && t->numel() == n, what,
              ": fp32, contiguous, ", n, " numbers");
  return t->data_ptr<float>();
}

}  // namespace

// xs [S, T, W] fp32 (updated in place when y is given). y / y2 [T, W]
// row-strided, gate [T, 1] row-strided; h [T, W] contiguous.
void hyper_streams(torch::Tensor xs, c10::optional<torch::Tensor> y,
                   c10::optional<torch::Tensor> y2,
                   c10::optional<torch::Tensor> gate,
                   c10::optional<torch::Tensor> mix,
                   c10::optional<torch::Tensor> out_w,
                   c10::optional<torch::Tensor> h,
                   c10::optional<torch::Tensor> in_w,
                   c10::optional<torch::Tensor> g, double eps) {
  TORCH_CHECK(xs.is_cuda() && xs.dim() == 3 && xs.is_contiguous() &&
              xs.scalar_type() == at::kFloat, "xs: fp32 [S, T, W]");
  const int S = xs.size(0), W = xs.size(2);
  const long T = xs.size(1);
  if (T == 0) return;
  TORCH_CHECK(S >= 1 && S <= MAX_S, "1..", MAX_S, " streams");
  TORCH_CHECK((size_t)W * sizeof(float) <= 64 * 1024,
              "row wider than the 64 KB of LDS a launch gets by default");
  TORCH_CHECK(y.has_value() || h.has_value());
  auto st = y.has_value() ? y->scalar_type() : h->scalar_type();
  const void *yp = nullptr, *y2p = nullptr, *gp = nullptr;
  long ys = 0, y2s = 0, gs = 0;
  const float *mp = nullptr, *bp = nullptr, *ap = nullptr, *gnp = nullptr;
  if (y.has_value()) {
    TORCH_CHECK(y->dim() == 2 && y->stride(1) == 1 && y->size(0) == T &&
                y->size(1) == W, "y: [T, W] rows");
    yp = y->data_ptr();
    ys = y->stride(0);
    if (y2.has_value()) {
      TORCH_CHECK(y2->dim() == 2 && y2->stride(1) == 1 && y2->size(0) == T &&
                  y2->size(1) == W && y2->scalar_type() == st);
      y2p = y2->data_ptr();
      y2s = y2->stride(0);
      if (gate.has_value()) {
        TORCH_CHECK(gate->dim() == 2 && gate->size(0) == T &&
                    gate->size(1) == 1 && gate->scalar_type() == st);
        gp = gate->data_ptr();
        gs = gate->stride(0);
      }
    }
    mp = f32_vec(mix, (long)S * S, "mix");
    bp = f32_vec(out_w, S, "out weights");
  }
  void *hp = nullptr;
  if (h.has_value()) {
    TORCH_CHECK(h->is_contiguous() && h->scalar_type() == st &&
                h->numel() == T * W);
    hp = h->data_ptr();
    ap = f32_vec(in_w, S, "in weights");
    gnp = f32_vec(g, 1, "norm gain");
  }
  auto stream = at::cuda::getCurrentCUDAStream();
  // four columns per thread when every row is 16 B (fp32) / 8 B (16-bit)
  // aligned
  const long esz = st == at::kFloat ? 4 : 2;
  auto row_ok = [&](const void *p, long stride) {
    return p == nullptr ||
           (reinterpret_cast<uintptr_t>(p) % (4 * esz) == 0 &&
            (stride * esz) % (4 * esz) == 0);
  };
  const bool vec = W % 4 == 0 &&
                   reinterpret_cast<uintptr_t>(xs.data_ptr()) % 16 == 0 &&
                   row_ok(yp, ys) && row_ok(y2p, y2s) && row_ok(hp, W);
#define RUN(TT, V)                                                          \
  hipLaunchKernelGGL((hyper_kernel<TT, V>), dim3(T), dim3(HY_BLOCK),        \
                     W * sizeof(float), stream, xs.data_ptr<float>(),       \
                     (long)xs.stride(0), S, W, (const TT *)yp, ys,          \
                     (const TT *)y2p, y2s, (const TT *)gp, gs, mp, bp,      \
                     (TT *)hp, ap, gnp, (float)eps)
  if (st == at::kBFloat16) {
    if (vec) RUN(__hip_bfloat16, 4); else RUN(__hip_bfloat16, 1);
  } else if (st == at::kFloat) {
    if (vec) RUN(float, 4); else RUN(float, 1);
  } else {
    TORCH_CHECK(false, "hyper_streams: bf16 or fp32");
  }
#undef RUN
  HIP_CHECK_KERNEL();
}
