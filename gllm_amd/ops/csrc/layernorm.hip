// LayerNorm (weight + optional bias) over an fp32 residual stream, gfx950.
//
// The residual stream of a sandwich-norm decoder (norm before AND after
// every sublayer) is kept in fp32 while the sublayers run in the model
// dtype T (bf16 or fp32). Two kernels cover a whole layer boundary:
//
//   layernorm_f32:      h = LN_pre(x)                       x fp32 -> h T
//   residual_layernorm: x += LN_post(y); h = LN_pre(x)      y T, x fp32
//                       with a gate: LN_post sees y * sigmoid(gate)
//   stream_rmsnorm:     the RMS form (plain weight, eps inside the root,
//                       no mean): x += mult * RMS(s (y + y2)) w_post;
//                       x += add; h = RMS(x) w_pre — every part optional
//
// One workgroup per token row; the row lives in LDS as fp32 between the
// mean, variance (mean of squared deviations, two passes: no E[x^2] -
// E[x]^2 cancellation) and normalize passes, so HBM sees each operand
// once. Statistics and the residual sum are fp32 whatever T is.

#include <torch/extension.h>
#include <ATen/cuda/CUDAContext.h>
#include "common.h"

namespace {

constexpr int LN_BLOCK = 256;

DEV_INLINE float ln_block_sum(float v, float *red) {
  __syncthreads();  // red may still be read from a previous reduction
  return block_reduce_sum<LN_BLOCK>(v, red);
}

// row <- src (vec: width % 8 == 0 and 16 B aligned rows)
template <typename T>
DEV_INLINE void row_load(float *row, const T *src, int width, bool vec) {
  if (vec) {
    for (int i = threadIdx.x * 8; i < width; i += LN_BLOCK * 8)
      ld8<T>(src + i, row + i);
  } else {
    for (int i = threadIdx.x; i < width; i += LN_BLOCK)
      row[i] = ScalarOps<T>::to_f32(src[i]);
  }
}

template <typename T>
DEV_INLINE void row_store(T *dst, const float *row, int width, bool vec) {
  if (vec) {
    for (int i = threadIdx.x * 8; i < width; i += LN_BLOCK * 8)
      st8<T>(dst + i, row + i);
  } else {
    for (int i = threadIdx.x; i < width; i += LN_BLOCK)
      dst[i] = ScalarOps<T>::from_f32(row[i]);
  }
}

// normalize the LDS row in place: row = (row - mean) / sqrt(var + eps) * w + b
// Callers put a barrier between filling the row and this call (the
// reductions walk the row with another thread-to-element mapping than
// the 8-wide loads); the trailing barrier publishes the result.
template <typename T>
DEV_INLINE void ln_row(float *row, const T *__restrict__ w,
                       const T *__restrict__ b, float eps, int width,
                       float *red, bool vec) {
  float s = 0.f;
  for (int i = threadIdx.x; i < width; i += LN_BLOCK) s += row[i];
  const float mean = ln_block_sum(s, red) / width;
  float ss = 0.f;
  for (int i = threadIdx.x; i < width; i += LN_BLOCK) {
    const float d = row[i] - mean;
    ss += d * d;
  }
  const float var = ln_block_sum(ss, red) / width;
  const float inv = 1.0f / sqrtf(var + eps);
  if (vec) {
    for (int i = threadIdx.x * 8; i < width; i += LN_BLOCK * 8) {
      float wf[8], bf[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
      ld8<T>(w + i, wf);
      if (b) ld8<T>(b + i, bf);
#pragma unroll
      for (int e = 0; e < 8; ++e)
        row[i + e] = (row[i + e] - mean) * inv * wf[e] + bf[e];
    }
  } else {
    for (int i = threadIdx.x; i < width; i += LN_BLOCK)
      row[i] = (row[i] - mean) * inv * ScalarOps<T>::to_f32(w[i]) +
               (b ? ScalarOps<T>::to_f32(b[i]) : 0.f);
  }
  __syncthreads();
}

DEV_INLINE float sigmoid_f32(float z) { return 1.0f / (1.0f + expf(-z)); }

// row *= sigmoid(gate row); same thread-to-element mapping as row_load
template <typename T>
DEV_INLINE void row_gate(float *row, const T *g, int width, bool vec) {
  if (vec) {
    for (int i = threadIdx.x * 8; i < width; i += LN_BLOCK * 8) {
      float gf[8];
      ld8<T>(g + i, gf);
#pragma unroll
      for (int e = 0; e < 8; ++e) row[i + e] *= sigmoid_f32(gf[e]);
    }
  } else {
    for (int i = threadIdx.x; i < width; i += LN_BLOCK)
      row[i] *= sigmoid_f32(ScalarOps<T>::to_f32(g[i]));
  }
}

template <typename T>
__global__ __launch_bounds__(LN_BLOCK) void layernorm_f32_kernel(
    T *__restrict__ out, const float *__restrict__ x,
    const T *__restrict__ w, const T *__restrict__ b, float eps, int width,
    int vec) {
  extern __shared__ float row[];
  __shared__ float red[LN_BLOCK / WAVE_SIZE];
  const long base = (long)blockIdx.x * width;
  row_load<float>(row, x + base, width, vec);
  __syncthreads();
  ln_row<T>(row, w, b, eps, width, red, vec);
  row_store<T>(out + base, row, width, vec);
}

// x += LN(y; w_post, b_post); optionally h = LN(x; w_pre, b_pre)
template <typename T>
__global__ __launch_bounds__(LN_BLOCK) void residual_layernorm_kernel(
    float *__restrict__ x, const T *__restrict__ y, long y_stride,
    const T *__restrict__ w_post, const T *__restrict__ b_post,
    T *__restrict__ h, const T *__restrict__ w_pre,
    const T *__restrict__ b_pre, float eps, int width, int vec,
    const T *__restrict__ gate, long gate_stride) {
  extern __shared__ float row[];
  __shared__ float red[LN_BLOCK / WAVE_SIZE];
  const long base = (long)blockIdx.x * width;
  row_load<T>(row, y + (long)blockIdx.x * y_stride, width, vec);
  if (gate) row_gate<T>(row, gate + (long)blockIdx.x * gate_stride, width, vec);
  __syncthreads();
  ln_row<T>(row, w_post, b_post, eps, width, red, vec);
  if (vec) {
    for (int i = threadIdx.x * 8; i < width; i += LN_BLOCK * 8) {
      float xf[8];
      ld8<float>(x + base + i, xf);
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        xf[e] += row[i + e];
        row[i + e] = xf[e];
      }
      st8<float>(x + base + i, xf);
    }
  } else {
    for (int i = threadIdx.x; i < width; i += LN_BLOCK) {
      const float r = x[base + i] + row[i];
      x[base + i] = r;
      row[i] = r;
    }
  }
  if (h == nullptr) return;
  __syncthreads();
  ln_row<T>(row, w_pre, b_pre, eps, width, red, vec);
  row_store<T>(h + base, row, width, vec);
}

// Wave-per-row form of residual_layernorm for 8-aligned widths up to
// 512 * NCH: the row stays in registers (NCH chunks of 8 per lane), the
// four statistics are wave reductions, and there is no LDS traffic or
// barrier at all. 4 rows per workgroup.
template <typename T, int NCH>
__global__ __launch_bounds__(LN_BLOCK) void residual_layernorm_wave_kernel(
    float *__restrict__ x, const T *__restrict__ y, long y_stride,
    const T *__restrict__ w_post, const T *__restrict__ b_post,
    T *__restrict__ h, const T *__restrict__ w_pre,
    const T *__restrict__ b_pre, float eps, int width, long rows,
    const T *__restrict__ gate, long gate_stride) {
  const int lane = threadIdx.x & 63;
  const long row = (long)blockIdx.x * (LN_BLOCK / 64) + (threadIdx.x >> 6);
  if (row >= rows) return;
  const long base = row * width;
  const T *yr = y + row * y_stride;
  float r[NCH][8];
  float s = 0.f;
#pragma unroll
  for (int c = 0; c < NCH; ++c) {
    const int i = (c * 64 + lane) * 8;
    if (i < width) {
      ld8<T>(yr + i, r[c]);
      if (gate) {
        float gf[8];
        ld8<T>(gate + row * gate_stride + i, gf);
#pragma unroll
        for (int e = 0; e < 8; ++e) r[c][e] *= sigmoid_f32(gf[e]);
      }
    } else {
#pragma unroll
      for (int e = 0; e < 8; ++e) r[c][e] = 0.f;
    }
#pragma unroll
    for (int e = 0; e < 8; ++e) s += r[c][e];
  }
  float mean = wave_reduce_sum(s) / width;
  float ss = 0.f;
#pragma unroll
  for (int c = 0; c < NCH; ++c) {
    if ((c * 64 + lane) * 8 < width) {
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const float d = r[c][e] - mean;
        ss += d * d;
      }
    }
  }
  float inv = 1.0f / sqrtf(wave_reduce_sum(ss) / width + eps);
  s = 0.f;
#pragma unroll
  for (int c = 0; c < NCH; ++c) {
    const int i = (c * 64 + lane) * 8;
    if (i < width) {
      float wf[8], bf[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f}, xf[8];
      ld8<T>(w_post + i, wf);
      if (b_post) ld8<T>(b_post + i, bf);
      ld8<float>(x + base + i, xf);
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        xf[e] += (r[c][e] - mean) * inv * wf[e] + bf[e];
        r[c][e] = xf[e];
        s += xf[e];
      }
      st8<float>(x + base + i, xf);
    }
  }
  if (h == nullptr) return;
  mean = wave_reduce_sum(s) / width;
  ss = 0.f;
#pragma unroll
  for (int c = 0; c < NCH; ++c) {
    if ((c * 64 + lane) * 8 < width) {
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const float d = r[c][e] - mean;
        ss += d * d;
      }
    }
  }
  inv = 1.0f / sqrtf(wave_reduce_sum(ss) / width + eps);
#pragma unroll
  for (int c = 0; c < NCH; ++c) {
    const int i = (c * 64 + lane) * 8;
    if (i < width) {
      float wf[8], bf[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f}, of[8];
      ld8<T>(w_pre + i, wf);
      if (b_pre) ld8<T>(b_pre + i, bf);
#pragma unroll
      for (int e = 0; e < 8; ++e)
        of[e] = (r[c][e] - mean) * inv * wf[e] + bf[e];
      st8<T>(h + base + i, of);
    }
  }
}

bool aligned16(const void *p) {
  return reinterpret_cast<uintptr_t>(p) % 16 == 0;
}

void check_vec(const torch::Tensor &t, int width, at::ScalarType st) {
  TORCH_CHECK(t.is_cuda() && t.is_contiguous() && t.numel() == width &&
              t.scalar_type() == st, "layernorm: bad weight/bias");
}

}  // namespace

void layernorm_f32(torch::Tensor out, torch::Tensor x, torch::Tensor w,
                   c10::optional<torch::Tensor> b, double eps) {
  TORCH_CHECK(x.scalar_type() == at::kFloat && x.is_contiguous());
  TORCH_CHECK(out.is_contiguous() && out.sizes() == x.sizes());
  const int width = x.size(-1);
  const long rows = x.numel() / std::max(width, 1);
  if (rows == 0) return;
  TORCH_CHECK(width > 0 && width * 4 <= 64 * 1024);
  check_vec(w, width, out.scalar_type());
  const void *bp = nullptr;
  if (b.has_value()) {
    check_vec(*b, width, out.scalar_type());
    bp = b->data_ptr();
  }
  const int vec = (width % 8 == 0 && aligned16(x.data_ptr()) &&
                   aligned16(out.data_ptr()) && aligned16(w.data_ptr()) &&
                   aligned16(bp)) ? 1 : 0;
  auto stream = at::cuda::getCurrentCUDAStream();
#define RUN(T)                                                             \
  hipLaunchKernelGGL((layernorm_f32_kernel<T>), dim3(rows), dim3(LN_BLOCK), \
                     width * sizeof(float), stream, (T *)out.data_ptr(),   \
                     x.data_ptr<float>(), (const T *)w.data_ptr(),         \
                     (const T *)bp, (float)eps, width, vec)
  if (out.scalar_type() == at::kBFloat16) RUN(__hip_bfloat16);
  else if (out.scalar_type() == at::kFloat) RUN(float);
  else TORCH_CHECK(false, "layernorm_f32: bf16 or fp32 output");
#undef RUN
  HIP_CHECK_KERNEL();
}

void residual_layernorm(torch::Tensor x, torch::Tensor y,
                        torch::Tensor w_post,
                        c10::optional<torch::Tensor> b_post,
                        c10::optional<torch::Tensor> h,
                        c10::optional<torch::Tensor> w_pre,
                        c10::optional<torch::Tensor> b_pre, double eps,
                        c10::optional<torch::Tensor> gate) {
  TORCH_CHECK(x.scalar_type() == at::kFloat && x.is_contiguous());
  const int width = x.size(-1);
  const long rows = x.numel() / std::max(width, 1);
  if (rows == 0) return;
  TORCH_CHECK(width > 0 && width * 4 <= 64 * 1024);
  TORCH_CHECK(y.dim() == 2 && y.size(0) == rows && y.size(1) == width &&
              y.stride(1) == 1, "residual_layernorm: y must be [rows, width]");
  const auto st = y.scalar_type();
  check_vec(w_post, width, st);
  const void *bpost = nullptr;
  if (b_post.has_value()) {
    check_vec(*b_post, width, st);
    bpost = b_post->data_ptr();
  }
  void *hp = nullptr;
  const void *wp = nullptr, *bp = nullptr;
  if (h.has_value()) {
    TORCH_CHECK(w_pre.has_value());
    TORCH_CHECK(h->is_contiguous() && h->numel() == x.numel() &&
                h->scalar_type() == st);
    check_vec(*w_pre, width, st);
    hp = h->data_ptr();
    wp = w_pre->data_ptr();
    if (b_pre.has_value()) {
      check_vec(*b_pre, width, st);
      bp = b_pre->data_ptr();
    }
  }
  const void *gp = nullptr;
  long gs = 0;
  if (gate.has_value()) {
    TORCH_CHECK(gate->is_cuda() && gate->dim() == 2 &&
                gate->size(0) == rows && gate->size(1) == width &&
                gate->stride(1) == 1 && gate->scalar_type() == st,
                "residual_layernorm: gate must be [rows, width]");
    gp = gate->data_ptr();
    gs = gate->stride(0);
  }
  const int vec =
      (width % 8 == 0 && aligned16(x.data_ptr()) && aligned16(y.data_ptr()) &&
       (y.stride(0) * y.element_size()) % 16 == 0 &&
       aligned16(w_post.data_ptr()) && aligned16(bpost) &&
       aligned16(hp) && aligned16(wp) && aligned16(bp) && aligned16(gp) &&
       (gs * y.element_size()) % 16 == 0) ? 1 : 0;
  auto stream = at::cuda::getCurrentCUDAStream();
  if (vec && width <= 8192) {
    const int nch = width <= 512 ? 1 : width <= 1024 ? 2 : width <= 2048 ? 4
                    : width <= 4096 ? 8 : 16;
    const long blocks = (rows + LN_BLOCK / 64 - 1) / (LN_BLOCK / 64);
#define RUNW(T, N)                                                          \
  hipLaunchKernelGGL((residual_layernorm_wave_kernel<T, N>), dim3(blocks),  \
                     dim3(LN_BLOCK), 0, stream, x.data_ptr<float>(),        \
                     (const T *)y.data_ptr(), (long)y.stride(0),            \
                     (const T *)w_post.data_ptr(),                          \
                     (const T *)bpost, (T *)hp, (const T *)wp,              \
                     (const T *)bp, (float)eps, width, rows,                \
                     (const T *)gp, gs)
#define RUNW_N(T)                                                           \
  switch (nch) {                                                            \
    case 1: RUNW(T, 1); break;                                              \
    case 2: RUNW(T, 2); break;                                              \
    case 4: RUNW(T, 4); break;                                              \
    case 8: RUNW(T, 8); break;                                              \
    default: RUNW(T, 16); break;                                            \
  }
    if (st == at::kBFloat16) { RUNW_N(__hip_bfloat16) }
    else if (st == at::kFloat) { RUNW_N(float) }
    else TORCH_CHECK(false, "residual_layernorm: bf16 or fp32");
#undef RUNW_N
#undef RUNW
    HIP_CHECK_KERNEL();
    return;
  }
#define RUN(T)                                                              \
  hipLaunchKernelGGL((residual_layernorm_kernel<T>), dim3(rows),            \
                     dim3(LN_BLOCK), width * sizeof(float), stream,         \
                     x.data_ptr<float>(), (const T *)y.data_ptr(),          \
                     (long)y.stride(0), (const T *)w_post.data_ptr(),       \
                     (const T *)bpost, (T *)hp, (const T *)wp,              \
                     (const T *)bp, (float)eps, width, vec,                 \
                     (const T *)gp, gs)
  if (st == at::kBFloat16) RUN(__hip_bfloat16);
  else if (st == at::kFloat) RUN(float);
  else TORCH_CHECK(false, "residual_layernorm: bf16 or fp32 sublayer output");
#undef RUN
  HIP_CHECK_KERNEL();
}

namespace {

// RMS sandwich boundary, one workgroup per token row, the row in LDS:
//   z = y_scale * (y + y2);  x += mult * z / sqrt(mean z^2 + eps) * w_post
//   x += add (one fp32 row for all tokens);  h = x / sqrt(mean x^2 + eps) * w_pre
// y == nullptr skips the first line, h == nullptr the last.
template <typename T>
__global__ __launch_bounds__(LN_BLOCK) void stream_rmsnorm_kernel(
    float *__restrict__ x, const T *__restrict__ y, long y_stride,
    const T *__restrict__ y2, long y2_stride, const T *__restrict__ w_post,
    const float *__restrict__ add, T *__restrict__ h,
    const T *__restrict__ w_pre, float eps, float mult, float y_scale,
    int width, int vec) {
  extern __shared__ float row[];
  __shared__ float red[LN_BLOCK / WAVE_SIZE];
  const long base = (long)blockIdx.x * width;
  const int tid = threadIdx.x;
  float ss = 0.f;
  if (y) {
    const T *yr = y + (long)blockIdx.x * y_stride;
    const T *y2r = y2 ? y2 + (long)blockIdx.x * y2_stride : nullptr;
    if (vec) {
      for (int i = tid * 8; i < width; i += LN_BLOCK * 8) {
        float a[8], b[8];
        ld8<T>(yr + i, a);
        if (y2r) {
          ld8<T>(y2r + i, b);
#pragma unroll
          for (int e = 0; e < 8; ++e) a[e] += b[e];
        }
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          a[e] *= y_scale;
          row[i + e] = a[e];
          ss += a[e] * a[e];
        }
      }
    } else {
      for (int i = tid; i < width; i += LN_BLOCK) {
        float a = ScalarOps<T>::to_f32(yr[i]);
        if (y2r) a += ScalarOps<T>::to_f32(y2r[i]);
        a *= y_scale;
        row[i] = a;
        ss += a * a;
      }
    }
    const float inv = mult / sqrtf(ln_block_sum(ss, red) / width + eps);
    ss = 0.f;
    // each thread revisits exactly the elements it wrote above
    if (vec) {
      for (int i = tid * 8; i < width; i += LN_BLOCK * 8) {
        float wf[8], xf[8], af[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
        ld8<T>(w_post + i, wf);
        ld8<float>(x + base + i, xf);
        if (add) ld8<float>(add + i, af);
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          xf[e] += row[i + e] * inv * wf[e];
          xf[e] += af[e];
          row[i + e] = xf[e];
          ss += xf[e] * xf[e];
        }
        st8<float>(x + base + i, xf);
      }
    } else {
      for (int i = tid; i < width; i += LN_BLOCK) {
        float r = x[base + i] + row[i] * inv * ScalarOps<T>::to_f32(w_post[i]);
        if (add) r += add[i];
        x[base + i] = r;
        row[i] = r;
        ss += r * r;
      }
    }
  } else {
    if (vec) {
      for (int i = tid * 8; i < width; i += LN_BLOCK * 8) {
        float xf[8], af[8];
        ld8<float>(x + base + i, xf);
        if (add) {
          ld8<float>(add + i, af);
#pragma unroll
          for (int e = 0; e < 8; ++e) xf[e] += af[e];
          st8<float>(x + base + i, xf);
        }
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          row[i + e] = xf[e];
          ss += xf[e] * xf[e];
        }
      }
    } else {
      for (int i = tid; i < width; i += LN_BLOCK) {
        float r = x[base + i];
        if (add) {
          r += add[i];
          x[base + i] = r;
        }
        row[i] = r;
        ss += r * r;
      }
    }
  }
  if (h == nullptr) return;
  const float inv = 1.0f / sqrtf(ln_block_sum(ss, red) / width + eps);
  if (vec) {
    for (int i = tid * 8; i < width; i += LN_BLOCK * 8) {
      float wf[8], of[8];
      ld8<T>(w_pre + i, wf);
#pragma unroll
      for (int e = 0; e < 8; ++e) of[e] = row[i + e] * inv * wf[e];
      st8<T>(h + base + i, of);
    }
  } else {
    for (int i = tid; i < width; i += LN_BLOCK)
      h[base + i] = ScalarOps<T>::from_f32(row[i] * inv *
                                           ScalarOps<T>::to_f32(w_pre[i]));
  }
}

}  // namespace

void stream_rmsnorm(torch::Tensor x, c10::optional<torch::Tensor> y,
                    c10::optional<torch::Tensor> y2,
                    c10::optional<torch::Tensor> w_post,
                    c10::optional<torch::Tensor> add,
                    c10::optional<torch::Tensor> h,
                    c10::optional<torch::Tensor> w_pre, double eps,
                    double mult, double y_scale) {
  TORCH_CHECK(x.is_cuda() && x.scalar_type() == at::kFloat &&
              x.is_contiguous());
  const int width = x.size(-1);
  const long rows = x.numel() / std::max(width, 1);
  if (rows == 0) return;
  TORCH_CHECK(width > 0 && width * 4 <= 64 * 1024);
  TORCH_CHECK(y.has_value() || h.has_value() || add.has_value());
  at::ScalarType st = at::kFloat;
  if (y.has_value()) st = y->scalar_type();
  else if (h.has_value()) st = h->scalar_type();
  const size_t es = st == at::kFloat ? 4 : 2;
  const void *yp = nullptr, *y2p = nullptr, *wpost = nullptr, *wpre = nullptr;
  const float *addp = nullptr;
  void *hp = nullptr;
  long ys = 0, y2s = 0;
  bool vec = width % 8 == 0 && aligned16(x.data_ptr());
  auto rows_of = [&](const torch::Tensor &t, const char *what) {
    TORCH_CHECK(t.is_cuda() && t.dim() == 2 && t.size(0) == rows &&
                t.size(1) == width && t.stride(1) == 1 &&
                t.scalar_type() == st, "stream_rmsnorm: ", what,
                " must be [rows, width] in the sublayer dtype");
    vec = vec && aligned16(t.data_ptr()) && (t.stride(0) * es) % 16 == 0;
  };
  if (y.has_value()) {
    rows_of(*y, "y");
    TORCH_CHECK(w_post.has_value());
    check_vec(*w_post, width, st);
    yp = y->data_ptr(); ys = y->stride(0);
    wpost = w_post->data_ptr();
    vec = vec && aligned16(wpost);
    if (y2.has_value()) {
      rows_of(*y2, "y2");
      y2p = y2->data_ptr(); y2s = y2->stride(0);
    }
  }
  if (add.has_value()) {
    TORCH_CHECK(add->is_cuda() && add->scalar_type() == at::kFloat &&
                add->is_contiguous() && add->numel() == width,
                "stream_rmsnorm: add must be fp32 [width]");
    addp = add->data_ptr<float>();
    vec = vec && aligned16(addp);
  }
  if (h.has_value()) {
    TORCH_CHECK(w_pre.has_value());
    TORCH_CHECK(h->is_contiguous() && h->numel() == x.numel() &&
                h->scalar_type() == st);
    check_vec(*w_pre, width, st);
    hp = h->data_ptr();
    wpre = w_pre->data_ptr();
    vec = vec && aligned16(hp) && aligned16(wpre);
  }
  auto stream = at::cuda::getCurrentCUDAStream();
#define RUN(T)                                                              \
  hipLaunchKernelGGL((stream_rmsnorm_kernel<T>), dim3(rows), dim3(LN_BLOCK), \
                     width * sizeof(float), stream, x.data_ptr<float>(),    \
                     (const T *)yp, ys, (const T *)y2p, y2s,                \
                     (const T *)wpost, addp, (T *)hp, (const T *)wpre,      \
                     (float)eps, (float)mult, (float)y_scale, width,        \
                     vec ? 1 : 0)
  if (st == at::kBFloat16) RUN(__hip_bfloat16);
  else if (st == at::kFloat) RUN(float);
  else TORCH_CHECK(false, "stream_rmsnorm: bf16 or fp32");
#undef RUN
  HIP_CHECK_KERNEL();
}
