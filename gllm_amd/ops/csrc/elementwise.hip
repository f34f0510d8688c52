// silu_and_mul + RoPE + reshape_and_cache for gfx950.
// All memory-bound: grid-stride, 16 B/lane vector loads.

#include <torch/extension.h>
#include <ATen/cuda/CUDAContext.h>
#include "common.h"

namespace {

// out[t, i] = silu(x[t, i]) * x[t, d + i],  x: [T, 2d]
template <typename T>
__global__ void silu_and_mul_kernel(T *__restrict__ out,
                                    const T *__restrict__ x, long rows,
                                    int d) {
  const int nvec = d / 8;
  const long total = rows * nvec;
  for (long idx = blockIdx.x * (long)blockDim.x + threadIdx.x; idx < total;
       idx += (long)gridDim.x * blockDim.x) {
    const long row = idx / nvec;
    const int i = idx % nvec;
    shortx8 a = reinterpret_cast<const shortx8 *>(x + row * 2 * d)[i];
    shortx8 b = reinterpret_cast<const shortx8 *>(x + row * 2 * d + d)[i];
    float va[8], vb[8];
    unpack8<T>(a, va);
    unpack8<T>(b, vb);
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      float s = va[j] / (1.f + __expf(-va[j]));
      va[j] = s * vb[j];
    }
    reinterpret_cast<shortx8 *>(out + row * d)[i] = pack8<T>(va);
  }
}

// gelu(x[:, :d]) * x[:, d:] — erf-based GELU (reference gelu_and_mul,
// the MoE activation="gelu" path in fused_moe.py:943).
template <typename T>
__global__ void gelu_and_mul_kernel(T *__restrict__ out,
                                    const T *__restrict__ x, long rows,
                                    int d) {
  const int nvec = d / 8;
  const long total = rows * nvec;
  for (long idx = blockIdx.x * (long)blockDim.x + threadIdx.x; idx < total;
       idx += (long)gridDim.x * blockDim.x) {
    const long row = idx / nvec;
    const int i = idx % nvec;
    shortx8 a = reinterpret_cast<const shortx8 *>(x + row * 2 * d)[i];
    shortx8 b = reinterpret_cast<const shortx8 *>(x + row * 2 * d + d)[i];
    float va[8], vb[8];
    unpack8<T>(a, va);
    unpack8<T>(b, vb);
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const float g = 0.5f * va[j] * (1.f + erff(va[j] * 0.70710678f));
      va[j] = g * vb[j];
    }
    reinterpret_cast<shortx8 *>(out + row * d)[i] = pack8<T>(va);
  }
}

// In-place neox / interleaved RoPE on q [T, Hq*D] and k [T, Hk*D].
// cos_sin_cache: [max_pos, rot_dim] fp32, [cos | sin] halves (host-built
// — no device trig, guide App. B). One block per token.
template <typename T, bool NEOX>
__global__ void rope_kernel(const long *__restrict__ positions,
                            T *__restrict__ q, T *__restrict__ k,
                            const float *__restrict__ cache, int rot_dim,
                            int head_dim, int num_q_heads, int num_k_heads,
                            long q_stride, long k_stride) {
  const long t = blockIdx.x;
  const float *cs = cache + positions[t] * rot_dim;
  const int half = rot_dim / 2;
  const int total = (num_q_heads + num_k_heads) * half;
  for (int idx = threadIdx.x; idx < total; idx += blockDim.x) {
    const int h = idx / half;
    const int p = idx % half;           // rotation pair index
    T *base = (h < num_q_heads)
                  ? q + t * q_stride + h * head_dim
                  : k + t * k_stride + (h - num_q_heads) * head_dim;
    const float c = cs[p], s = cs[half + p];
    int i1, i2;
    if (NEOX) { i1 = p; i2 = p + half; }
    else      { i1 = 2 * p; i2 = 2 * p + 1; }
    const float x1 = ScalarOps<T>::to_f32(base[i1]);
    const float x2 = ScalarOps<T>::to_f32(base[i2]);
    base[i1] = ScalarOps<T>::from_f32(x1 * c - x2 * s);
    base[i2] = ScalarOps<T>::from_f32(x2 * c + x1 * s);
  }
}

// Scatter per-token K/V [T, H, D] into paged caches [P, page, H, D].
// One block per token; row copy is H*D*2 bytes, vectorized.
template <typename T>
__global__ void reshape_and_cache_kernel(
    const T *__restrict__ k, const T *__restrict__ v, T *__restrict__ k_cache,
    T *__restrict__ v_cache, const long *__restrict__ slot_mapping,
    int k_row_elems /* H*Dk */, int v_row_elems /* H*Dv (MLA: != k) */,
    int page_size, long k_stride, long v_stride) {
  const long t = blockIdx.x;
  const long slot = slot_mapping[t];
  const long page = slot / page_size, off = slot % page_size;
  const long tok = page * page_size + off;
  const int knvec = k_row_elems / 8, vnvec = v_row_elems / 8;
  const shortx8 *ks = reinterpret_cast<const shortx8 *>(k + t * k_stride);
  const shortx8 *vs = reinterpret_cast<const shortx8 *>(v + t * v_stride);
  shortx8 *kd = reinterpret_cast<shortx8 *>(k_cache + tok * (long)k_row_elems);
  shortx8 *vd = reinterpret_cast<shortx8 *>(v_cache + tok * (long)v_row_elems);
  for (int i = threadIdx.x; i < knvec; i += blockDim.x) kd[i] = ks[i];
  for (int i = threadIdx.x; i < vnvec; i += blockDim.x) vd[i] = vs[i];
}

// fp32 variant: floatx4 (16 B) vector loads instead of shortx8.
__global__ void silu_and_mul_f32_kernel(float *__restrict__ out,
                                        const float *__restrict__ x,
                                        long rows, int d) {
  const int nvec = d / 4;
  const long total = rows * nvec;
  for (long idx = blockIdx.x * (long)blockDim.x + threadIdx.x; idx < total;
       idx += (long)gridDim.x * blockDim.x) {
    const long row = idx / nvec;
    const int i = idx % nvec;
    floatx4 a = reinterpret_cast<const floatx4 *>(x + row * 2 * d)[i];
    floatx4 b = reinterpret_cast<const floatx4 *>(x + row * 2 * d + d)[i];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      float s = a[j] / (1.f + __expf(-a[j]));
      a[j] = s * b[j];
    }
    reinterpret_cast<floatx4 *>(out + row * d)[i] = a;
  }
}

}  // namespace

void silu_and_mul(torch::Tensor out, torch::Tensor x) {
  const int d = x.size(-1) / 2;
  const long rows = x.numel() / (2 * d);
  TORCH_CHECK(d % 8 == 0);
  TORCH_CHECK(x.is_contiguous() && out.is_contiguous());
  const long total = rows * (d / 8);
  const int block = 256;
  const long grid = std::min<long>((total + block - 1) / block, 2048);
  auto stream = at::cuda::getCurrentCUDAStream();
  if (x.scalar_type() == at::kBFloat16) {
    hipLaunchKernelGGL((silu_and_mul_kernel<__hip_bfloat16>), dim3(grid),
                       dim3(block), 0, stream,
                       (__hip_bfloat16 *)out.data_ptr(),
                       (const __hip_bfloat16 *)x.data_ptr(), rows, d);
  } else if (x.scalar_type() == at::kHalf) {
    hipLaunchKernelGGL((silu_and_mul_kernel<__half>), dim3(grid), dim3(block),
                       0, stream, (__half *)out.data_ptr(),
                       (const __half *)x.data_ptr(), rows, d);
  } else if (x.scalar_type() == at::kFloat) {
    hipLaunchKernelGGL((silu_and_mul_f32_kernel), dim3(grid), dim3(block),
                       0, stream, out.data_ptr<float>(),
                       x.data_ptr<float>(), rows, d);
  } else {
    TORCH_CHECK(false, "silu_and_mul: unsupported dtype");
  }
  HIP_CHECK_KERNEL();
}

void gelu_and_mul(torch::Tensor out, torch::Tensor x) {
  const int d = x.size(-1) / 2;
  const long rows = x.numel() / (2 * d);
  TORCH_CHECK(d % 8 == 0);
  TORCH_CHECK(x.is_contiguous() && out.is_contiguous());
  const long total = rows * (d / 8);
  const int block = 256;
  const long grid = std::min<long>((total + block - 1) / block, 2048);
  auto stream = at::cuda::getCurrentCUDAStream();
  if (x.scalar_type() == at::kBFloat16) {
    hipLaunchKernelGGL((gelu_and_mul_kernel<__hip_bfloat16>), dim3(grid),
                       dim3(block), 0, stream,
                       (__hip_bfloat16 *)out.data_ptr(),
                       (const __hip_bfloat16 *)x.data_ptr(), rows, d);
  } else if (x.scalar_type() == at::kHalf) {
    hipLaunchKernelGGL((gelu_and_mul_kernel<__half>), dim3(grid), dim3(block),
                       0, stream, (__half *)out.data_ptr(),
                       (const __half *)x.data_ptr(), rows, d);
  } else {
    TORCH_CHECK(false, "gelu_and_mul: unsupported dtype");
  }
  HIP_CHECK_KERNEL();
}

void rotary_embedding(torch::Tensor positions, torch::Tensor q,
                      torch::Tensor k, long head_dim,
                      torch::Tensor cos_sin_cache, bool is_neox) {
  const long T = positions.size(0);
  const int rot_dim = cos_sin_cache.size(-1);
  const int hq = q.size(-1) / head_dim, hk = k.size(-1) / head_dim;
  TORCH_CHECK(q.stride(-1) == 1 && k.stride(-1) == 1,
              "rope: innermost dim must be contiguous");
  const long qs = q.stride(0), ks = k.stride(0);
  TORCH_CHECK(q.scalar_type() == at::kBFloat16,
              "rope: bf16 only for now");
  TORCH_CHECK(cos_sin_cache.scalar_type() == at::kFloat);
  auto stream = at::cuda::getCurrentCUDAStream();
  if (is_neox) {
    hipLaunchKernelGGL((rope_kernel<__hip_bfloat16, true>), dim3(T),
                       dim3(256), 0, stream,
                       positions.data_ptr<long>(),
                       (__hip_bfloat16 *)q.data_ptr(),
                       (__hip_bfloat16 *)k.data_ptr(),
                       cos_sin_cache.data_ptr<float>(), rot_dim,
                       (int)head_dim, hq, hk, qs, ks);
  } else {
    hipLaunchKernelGGL((rope_kernel<__hip_bfloat16, false>), dim3(T),
                       dim3(256), 0, stream,
                       positions.data_ptr<long>(),
                       (__hip_bfloat16 *)q.data_ptr(),
                       (__hip_bfloat16 *)k.data_ptr(),
                       cos_sin_cache.data_ptr<float>(), rot_dim,
                       (int)head_dim, hq, hk, qs, ks);
  }
  HIP_CHECK_KERNEL();
}

void reshape_and_cache(torch::Tensor k, torch::Tensor v,
                       torch::Tensor k_cache, torch::Tensor v_cache,
                       torch::Tensor slot_mapping) {
  const long T = k.size(0);
  if (T == 0) return;
  const int k_row = k.size(1) * k.size(2);
  const int v_row = v.size(1) * v.size(2);
  const int page_size = k_cache.size(1);
  TORCH_CHECK(k_row % 8 == 0 && v_row % 8 == 0);
  TORCH_CHECK(k.stride(-1) == 1 && v.stride(-1) == 1 &&
              k.stride(1) == k.size(2) && v.stride(1) == v.size(2),
              "reshape_and_cache: per-token row must be contiguous");
  TORCH_CHECK(k_cache.is_contiguous() && v_cache.is_contiguous());
  TORCH_CHECK(k_cache.size(2) * k_cache.size(3) == k_row &&
              v_cache.size(2) * v_cache.size(3) == v_row,
              "cache row dims must match inputs");
  TORCH_CHECK(slot_mapping.scalar_type() == at::kLong);
  TORCH_CHECK(k.scalar_type() == at::kBFloat16);
  auto stream = at::cuda::getCurrentCUDAStream();
  const int block = std::min(256, std::max(64, k_row / 8));
  hipLaunchKernelGGL((reshape_and_cache_kernel<__hip_bfloat16>), dim3(T),
                     dim3(block), 0, stream,
                     (const __hip_bfloat16 *)k.data_ptr(),
                     (const __hip_bfloat16 *)v.data_ptr(),
                     (__hip_bfloat16 *)k_cache.data_ptr(),
                     (__hip_bfloat16 *)v_cache.data_ptr(),
                     slot_mapping.data_ptr<long>(), k_row, v_row,
                     page_size, k.stride(0), v.stride(0));
  HIP_CHECK_KERNEL();
}

// ------------------------------------------------------------------
// Ungated feed-forward activations: out[r, i] = act(x[r, i]) for a
// row-strided x (a column slice of a merged projection) and a
// contiguous out. fp32 arithmetic whatever the I/O type is.
namespace {

struct XieluOp {
  float a_pos, a_neg;
  // z > 0: a_pos z^2 + z/2; z <= 0: a_neg (e^z - 1 - z) + z/2
  DEV_INLINE float operator()(float z) const {
    return z > 0.f ? a_pos * z * z + 0.5f * z
                   : a_neg * (expm1f(z) - z) + 0.5f * z;
  }
};

struct Relu2Op {
  DEV_INLINE float operator()(float z) const {
    const float r = fmaxf(z, 0.f);
    return r * r;
  }
};

template <typename T, typename Op, bool VEC>
__global__ __launch_bounds__(256) void unary_rows_kernel(
    T *__restrict__ out, const T *__restrict__ x, long x_stride, long rows,
    int n, Op op) {
  if (VEC) {
    const int nvec = n / 8;
    const long total = rows * nvec;
    for (long idx = blockIdx.x * (long)blockDim.x + threadIdx.x; idx < total;
         idx += (long)gridDim.x * blockDim.x) {
      const long r = idx / nvec;
      const int i = (idx % nvec) * 8;
      float f[8];
      ld8<T>(x + r * x_stride + i, f);
#pragma unroll
      for (int e = 0; e < 8; ++e) f[e] = op(f[e]);
      st8<T>(out + r * n + i, f);
    }
  } else {
    const long total = rows * n;
    for (long idx = blockIdx.x * (long)blockDim.x + threadIdx.x; idx < total;
         idx += (long)gridDim.x * blockDim.x) {
      const long r = idx / n;
      const int i = idx % n;
      out[r * n + i] = ScalarOps<T>::from_f32(
          op(ScalarOps<T>::to_f32(x[r * x_stride + i])));
    }
  }
}

template <typename Op>
void launch_unary_rows(torch::Tensor &out, torch::Tensor &x, Op op,
                       const char *name) {
  TORCH_CHECK(x.is_cuda() && x.dim() == 2 && x.stride(1) == 1, name,
              ": x must be [rows, n] with unit inner stride");
  TORCH_CHECK(out.is_contiguous() && out.sizes() == x.sizes() &&
              out.scalar_type() == x.scalar_type());
  const long rows = x.size(0);
  const int n = x.size(1);
  if (rows == 0 || n == 0) return;
  const long esz = x.element_size();
  const bool vec = n % 8 == 0 &&
                   reinterpret_cast<uintptr_t>(x.data_ptr()) % 16 == 0 &&
                   reinterpret_cast<uintptr_t>(out.data_ptr()) % 16 == 0 &&
                   (x.stride(0) * esz) % 16 == 0;
  const long work = vec ? rows * (n / 8) : rows * (long)n;
  const int grid = (int)std::min<long>((work + 255) / 256, 65535);
  auto stream = at::cuda::getCurrentCUDAStream();
#define RUN(TT, V)                                                          \
  hipLaunchKernelGGL((unary_rows_kernel<TT, Op, V>), dim3(grid), dim3(256), \
                     0, stream, (TT *)out.data_ptr(),                       \
                     (const TT *)x.data_ptr(), (long)x.stride(0), rows, n, op)
  if (x.scalar_type() == at::kBFloat16) {
    if (vec) RUN(__hip_bfloat16, true); else RUN(__hip_bfloat16, false);
  } else if (x.scalar_type() == at::kFloat) {
    if (vec) RUN(float, true); else RUN(float, false);
  } else {
    TORCH_CHECK(false, name, ": bf16 or fp32");
  }
#undef RUN
  HIP_CHECK_KERNEL();
}

}  // namespace

void xielu(torch::Tensor out, torch::Tensor x, double a_pos, double a_neg) {
  launch_unary_rows(out, x, XieluOp{(float)a_pos, (float)a_neg}, "xielu");
}

void relu2(torch::Tensor out, torch::Tensor x) {
  launch_unary_rows(out, x, Relu2Op{}, "relu2");
}

namespace {

// out[r, i] = g * sigmoid(alpha g) * (u + 1), g = min(x[r, i], limit),
// u = clamp(x[r, d + i], -limit, limit); x rows may be strided. VEC: 8
// elements per thread through 16 B accesses (d % 8 == 0, aligned rows).
template <typename T, bool VEC>
__global__ __launch_bounds__(256) void clamp_swiglu_kernel(
    T *__restrict__ out, const T *__restrict__ x, long x_stride, long rows,
    int d, float limit, float alpha) {
  if (VEC) {
    const int nvec = d / 8;
    const long total = rows * nvec;
    for (long idx = blockIdx.x * (long)blockDim.x + threadIdx.x; idx < total;
         idx += (long)gridDim.x * blockDim.x) {
      const long r = idx / nvec;
      const int i = (idx % nvec) * 8;
      float g[8], u[8];
      ld8<T>(x + r * x_stride + i, g);
      ld8<T>(x + r * x_stride + d + i, u);
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const float gv = fminf(g[e], limit);
        const float uv = fminf(fmaxf(u[e], -limit), limit);
        g[e] = gv / (1.0f + (sizeof(T) == 4 ? expf(-alpha * gv)
                                            : __expf(-alpha * gv))) *
               (uv + 1.0f);
      }
      st8<T>(out + r * d + i, g);
    }
    return;
  }
  const long total = rows * d;
  for (long idx = blockIdx.x * (long)blockDim.x + threadIdx.x; idx < total;
       idx += (long)gridDim.x * blockDim.x) {
    const long r = idx / d;
    const int i = idx % d;
    const float g = fminf(ScalarOps<T>::to_f32(x[r * x_stride + i]), limit);
    const float u = fminf(fmaxf(ScalarOps<T>::to_f32(x[r * x_stride + d + i]),
                                -limit), limit);
    out[r * d + i] =
        ScalarOps<T>::from_f32(g / (1.0f + expf(-alpha * g)) * (u + 1.0f));
  }
}

}  // namespace

void clamp_swiglu(torch::Tensor out, torch::Tensor x, double limit,
                  double alpha) {
  TORCH_CHECK(x.is_cuda() && x.dim() == 2 && x.stride(1) == 1 &&
              x.size(1) % 2 == 0, "clamp_swiglu: x [rows, 2d] rows");
  const long rows = x.size(0);
  const int d = x.size(1) / 2;
  TORCH_CHECK(out.is_contiguous() && out.scalar_type() == x.scalar_type() &&
              out.numel() == rows * d);
  if (rows == 0 || d == 0) return;
  const long esz = x.element_size();
  const bool vec = d % 8 == 0 &&
                   reinterpret_cast<uintptr_t>(x.data_ptr()) % 16 == 0 &&
                   reinterpret_cast<uintptr_t>(out.data_ptr()) % 16 == 0 &&
                   (x.stride(0) * esz) % 16 == 0;
  const long work = vec ? rows * (d / 8) : rows * (long)d;
  const int grid = (int)std::min<long>((work + 255) / 256, 8192);
  auto stream = at::cuda::getCurrentCUDAStream();
#define RUN(TT, V)                                                          \
  hipLaunchKernelGGL((clamp_swiglu_kernel<TT, V>), dim3(grid), dim3(256),   \
                     0, stream, (TT *)out.data_ptr(),                       \
                     (const TT *)x.data_ptr(), (long)x.stride(0), rows, d,  \
                     (float)limit, (float)alpha)
  if (x.scalar_type() == at::kBFloat16) {
    if (vec) RUN(__hip_bfloat16, true); else RUN(__hip_bfloat16, false);
  } else if (x.scalar_type() == at::kFloat) {
    if (vec) RUN(float, true); else RUN(float, false);
  } else {
    TORCH_CHECK(false, "clamp_swiglu: bf16 or fp32");
  }
#undef RUN
  HIP_CHECK_KERNEL();
}

namespace {

DEV_INLINE float gelu_tanh_f(float z) {
  // 0.5 z (1 + tanh(sqrt(2/pi) (z + 0.044715 z^3)))
  const float u = 0.7978845608028654f * (z + 0.044715f * z * z * z);
  return 0.5f * z * (1.0f + tanhf(u));
}

// out[r, i] = act(x[r, i]) * x[r, d + i], ACT 0: silu, 1: tanh-form gelu;
// x rows may be strided, any d. VEC: 8 elements per thread through 16 B
// accesses (d % 8 == 0, aligned rows).
template <typename T, int ACT, bool VEC>
__global__ __launch_bounds__(256) void gated_act_mul_kernel(
    T *__restrict__ out, const T *__restrict__ x, long x_stride, long rows,
    int d) {
  if (VEC) {
    const int nvec = d / 8;
    const long total = rows * nvec;
    for (long idx = blockIdx.x * (long)blockDim.x + threadIdx.x; idx < total;
         idx += (long)gridDim.x * blockDim.x) {
      const long r = idx / nvec;
      const int i = (idx % nvec) * 8;
      float g[8], u[8];
      ld8<T>(x + r * x_stride + i, g);
      ld8<T>(x + r * x_stride + d + i, u);
#pragma unroll
      for (int e = 0; e < 8; ++e)
        g[e] = (ACT == 0 ? g[e] / (1.0f + expf(-g[e])) : gelu_tanh_f(g[e])) *
               u[e];
      st8<T>(out + r * d + i, g);
    }
    return;
  }
  const long total = rows * d;
  for (long idx = blockIdx.x * (long)blockDim.x + threadIdx.x; idx < total;
       idx += (long)gridDim.x * blockDim.x) {
    const long r = idx / d;
    const int i = idx % d;
    const float g = ScalarOps<T>::to_f32(x[r * x_stride + i]);
    const float u = ScalarOps<T>::to_f32(x[r * x_stride + d + i]);
    out[r * d + i] = ScalarOps<T>::from_f32(
        (ACT == 0 ? g / (1.0f + expf(-g)) : gelu_tanh_f(g)) * u);
  }
}

}  // namespace

// act: 0 silu, 1 gelu (tanh form)
void gated_act_mul(torch::Tensor out, torch::Tensor x, long act) {
  TORCH_CHECK(x.is_cuda() && x.dim() == 2 && x.stride(1) == 1 &&
              x.size(1) % 2 == 0, "gated_act_mul: x [rows, 2d] rows");
  TORCH_CHECK(act == 0 || act == 1, "gated_act_mul: act 0 (silu) or 1 (gelu)");
  const long rows = x.size(0);
  const int d = x.size(1) / 2;
  TORCH_CHECK(out.is_contiguous() && out.scalar_type() == x.scalar_type() &&
              out.numel() == rows * d);
  if (rows == 0 || d == 0) return;
  const long esz = x.element_size();
  const bool vec = d % 8 == 0 &&
                   reinterpret_cast<uintptr_t>(x.data_ptr()) % 16 == 0 &&
                   reinterpret_cast<uintptr_t>(out.data_ptr()) % 16 == 0 &&
                   (x.stride(0) * esz) % 16 == 0;
  const long work = vec ? rows * (d / 8) : rows * (long)d;
  const int grid = (int)std::min<long>((work + 255) / 256, 8192);
  auto stream = at::cuda::getCurrentCUDAStream();
#define RUN(TT, A, V)                                                        \
  hipLaunchKernelGGL((gated_act_mul_kernel<TT, A, V>), dim3(grid),           \
                     dim3(256), 0, stream, (TT *)out.data_ptr(),            \
                     (const TT *)x.data_ptr(), (long)x.stride(0), rows, d)
#define RUN_AV(TT)                                                           \
  if (act == 0) { if (vec) RUN(TT, 0, true); else RUN(TT, 0, false); }       \
  else { if (vec) RUN(TT, 1, true); else RUN(TT, 1, false); }
  if (x.scalar_type() == at::kBFloat16) { RUN_AV(__hip_bfloat16) }
  else if (x.scalar_type() == at::kFloat) { RUN_AV(float) }
  else TORCH_CHECK(false, "gated_act_mul: bf16 or fp32");
#undef RUN_AV
#undef RUN
  HIP_CHECK_KERNEL();
}

namespace {

// out[r, i] = tanh(x[r, i]) over strided rows (a column block of a merged
// projection), any width; the function is taken in fp32.
template <typename T>
__global__ __launch_bounds__(256) void tanh_rows_kernel(
    T *__restrict__ out, const T *__restrict__ x, long x_stride, long rows,
    int n) {
  const long total = rows * n;
  for (long idx = blockIdx.x * (long)blockDim.x + threadIdx.x; idx < total;
       idx += (long)gridDim.x * blockDim.x) {
    const long r = idx / n;
    const int i = idx % n;
    out[idx] = ScalarOps<T>::from_f32(
        tanhf(ScalarOps<T>::to_f32(x[r * x_stride + i])));
  }
}

}  // namespace

void tanh_rows(torch::Tensor out, torch::Tensor x) {
  TORCH_CHECK(x.is_cuda() && x.dim() == 2 && x.stride(1) == 1,
              "tanh_rows: x [rows, n] rows");
  const long rows = x.size(0);
  const int n = x.size(1);
  TORCH_CHECK(out.is_contiguous() && out.scalar_type() == x.scalar_type() &&
              out.numel() == rows * n);
  if (rows == 0 || n == 0) return;
  const int grid = (int)std::min<long>((rows * n + 255) / 256, 8192);
  auto stream = at::cuda::getCurrentCUDAStream();
#define RUN(TT)                                                              \
  hipLaunchKernelGGL((tanh_rows_kernel<TT>), dim3(grid), dim3(256), 0,       \
                     stream, (TT *)out.data_ptr(), (const TT *)x.data_ptr(), \
                     (long)x.stride(0), rows, n)
  if (x.scalar_type() == at::kBFloat16) RUN(__hip_bfloat16);
  else if (x.scalar_type() == at::kFloat) RUN(float);
  else TORCH_CHECK(false, "tanh_rows: bf16 or fp32");
#undef RUN
  HIP_CHECK_KERNEL();
}
