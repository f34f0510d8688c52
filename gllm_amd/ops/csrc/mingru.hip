// minGRU: a gated linear recurrence whose gates read only the current
// token, over a ragged batch, gfx950.
//
//   z_t = sigmoid(zp_t)              update gate
//   c_t = up_t + 1/2  (up_t >= 0),  sigmoid(up_t)  (up_t < 0)
//   S_t = (1 - z_t) S_{t-1} + z_t c_t            (element by element)
//   out_t = scale * S_t * silu(gp_t)
//
// zp | up arrive as one row-strided projection [T, 2C] (biases already
// added), gp as [T, C]; the state pool [slots, C] is fp32 and is carried
// per sequence (has_init[b] == 0: the sequence starts from zero, whatever
// the slot held). Gates, candidate and state are fp32; out is in the
// model dtype and may be a column block of a wider buffer.
//
// S_t = a_t S_{t-1} + b_t is an affine map per step, and affine maps
// compose: a workgroup owns (sequence, CH channels) and splits the
// sequence's new tokens into NSEG contiguous segments, one per thread
// row. Pass 1 folds each segment into one map (A, B); the maps of the
// earlier segments applied to the carried state give the segment's
// start state; pass 2 replays the segment from there and writes the
// outputs. A decode-only batch runs NSEG = 1 (one pass, nothing folded).
// CH x NSEG is 64 x 16, or 32 x 32 / 16 x 64 for small batches, so that a
// few long sequences still give every compute unit a workgroup.

#include <torch/extension.h>
#include <ATen/cuda/CUDAContext.h>
#include "common.h"

namespace {

template <typename T>
DEV_INLINE void gru_step(const T *__restrict__ zx, int C, int c, float &a,
                         float &b) {
  const float zp = ScalarOps<T>::to_f32(zx[c]);
  const float up = ScalarOps<T>::to_f32(zx[C + c]);
  const float z = 1.0f / (1.0f + expf(-zp));
  const float cand = up >= 0.f ? up + 0.5f : 1.0f / (1.0f + expf(-up));
  a = 1.0f - z;
  b = z * cand;
}

template <typename T, int CH, int NSEG>
__global__ __launch_bounds__(CH *NSEG) void mingru_kernel(
    T *__restrict__ out, long out_stride, const T *__restrict__ zx,
    long zx_stride, const T *__restrict__ gp, long gp_stride,
    float *__restrict__ state, const long *__restrict__ slots,
    const int *__restrict__ has_init, const int *__restrict__ qsl, int C,
    float scale) {
  __shared__ float fa[NSEG > 1 ? NSEG : 1][CH];
  __shared__ float fb[NSEG > 1 ? NSEG : 1][CH];
  const int b = blockIdx.x;
  const int cx = threadIdx.x % CH, seg = threadIdx.x / CH;
  const int c = blockIdx.y * CH + cx;
  const int t0 = qsl[b], t1 = qsl[b + 1];
  const int n = t1 - t0;
  if (n <= 0) return;
  const bool live = c < C;
  const long slot = slots[b];
  float S = (live && has_init[b]) ? state[slot * C + c] : 0.f;
  // this thread's tokens: [lo, hi)
  const int per = (n + NSEG - 1) / NSEG;
  const int lo = t0 + min(seg * per, n), hi = t0 + min((seg + 1) * per, n);
  if (NSEG > 1) {
    float A = 1.f, B = 0.f;
    if (live)
#pragma unroll 4
      for (int t = lo; t < hi; ++t) {
        float a, bb;
        gru_step<T>(zx + (long)t * zx_stride, C, c, a, bb);
        A *= a;
        B = a * B + bb;
      }
    fa[seg][cx] = A;
    fb[seg][cx] = B;
    __syncthreads();
    for (int s = 0; s < seg; ++s) S = fa[s][cx] * S + fb[s][cx];
  }
  if (!live) return;
#pragma unroll 4
  for (int t = lo; t < hi; ++t) {
    float a, bb;
    gru_step<T>(zx + (long)t * zx_stride, C, c, a, bb);
    S = a * S + bb;
    const float gv = ScalarOps<T>::to_f32(gp[(long)t * gp_stride + c]);
    out[(long)t * out_stride + c] =
        ScalarOps<T>::from_f32(scale * S * (gv / (1.0f + expf(-gv))));
  }
  // the thread that holds the sequence's last new token
  if (hi == t1 && lo < hi) state[slot * C + c] = S;
}

}  // namespace

void mingru_varlen(torch::Tensor out, torch::Tensor zx, torch::Tensor gp,
                   torch::Tensor state, torch::Tensor slots,
                   torch::Tensor has_init, torch::Tensor query_start_loc,
                   double scale, long max_query_len) {
  const long T = zx.size(0);
  if (T == 0) return;
  const auto st = zx.scalar_type();
  TORCH_CHECK(zx.is_cuda() && zx.dim() == 2 && zx.stride(1) == 1 &&
              zx.size(1) % 2 == 0);
  const int C = zx.size(1) / 2;
  TORCH_CHECK(gp.dim() == 2 && gp.stride(1) == 1 && gp.size(0) == T &&
              gp.size(1) == C && gp.scalar_type() == st);
  TORCH_CHECK(out.dim() == 2 && out.stride(1) == 1 && out.size(0) == T &&
              out.size(1) == C && out.scalar_type() == st);
  TORCH_CHECK(state.scalar_type() == at::kFloat && state.is_contiguous() &&
              state.numel() % C == 0 && state.size(-1) == C,
              "state pool: fp32 [slots, C]");
  const int B = slots.numel();
  TORCH_CHECK(slots.scalar_type() == at::kLong && slots.is_contiguous());
  TORCH_CHECK(has_init.scalar_type() == at::kInt && has_init.is_contiguous() &&
              has_init.numel() >= B);
  TORCH_CHECK(query_start_loc.scalar_type() == at::kInt &&
              query_start_loc.is_contiguous() &&
              query_start_loc.numel() >= B + 1);
  auto stream = at::cuda::getCurrentCUDAStream();
#define RUN(TT, CH, NSEG)                                                   \
  hipLaunchKernelGGL((mingru_kernel<TT, CH, NSEG>),                         \
                     dim3(B, (C + CH - 1) / CH), dim3(CH * NSEG), 0,        \
                     stream, (TT *)out.data_ptr(), (long)out.stride(0),     \
                     (const TT *)zx.data_ptr(), (long)zx.stride(0),         \
                     (const TT *)gp.data_ptr(), (long)gp.stride(0),         \
                     state.data_ptr<float>(), slots.data_ptr<long>(),       \
                     has_init.data_ptr<int>(),                              \
                     query_start_loc.data_ptr<int>(), C, (float)scale)
  // batches with prompt portions: 1024 threads = CH channels x NSEG
  // segments; fewer channels per workgroup (more, shorter segments) when
  // 64 would leave compute units without a workgroup
  const long wg64 = (long)B * ((C + 63) / 64);
  const int ch = wg64 >= 256 ? 64 : (2 * wg64 >= 256 ? 32 : 16);
#define RUN_T(TT)                                                           \
  if (max_query_len > 0 && max_query_len <= 8) RUN(TT, 256, 1);             \
  else if (ch == 64) RUN(TT, 64, 16);                                       \
  else if (ch == 32) RUN(TT, 32, 32);                                       \
  else RUN(TT, 16, 64)
  if (st == at::kBFloat16) { RUN_T(__hip_bfloat16); }
  else if (st == at::kFloat) { RUN_T(float); }
  else TORCH_CHECK(false, "mingru_varlen: bf16 or fp32");
#undef RUN_T
#undef RUN
  HIP_CHECK_KERNEL();
}
