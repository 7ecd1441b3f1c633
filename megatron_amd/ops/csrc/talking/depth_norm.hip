// Residual updates of layers that norm a sublayer's OUTPUT and hand on a
// weighted sum over depth, and the tanh form of GELU.
#include "../ragged/ragged_common.h"

// ---------------------------------------------------------------------------
// x[t] <- x[t] + y[t] / sqrt(mean(y[t]^2) + eps) * (1 + w)          (y given)
// hist[depth][t] <- x[t];  x[t] <- sum_{j <= depth} dwa[j] hist[j][t]  (hist given)
// h[t] <- x[t] in the next GEMM's input type (TO = float: x itself is that input).
// Workgroup = token.  x, hist fp32; the row of y is read twice (second time from L1/L2).
// ---------------------------------------------------------------------------
template <typename TY, typename TO>
__global__ __launch_bounds__(256) void post_norm_add_kernel(
    float* __restrict__ x, const TY* __restrict__ y, const float* __restrict__ w, float eps, TO* __restrict__ h,
    float* __restrict__ hist, int depth, const float* __restrict__ dwa, long TW, int W) {
  __shared__ float red[256 / WAVE];
  const long t = blockIdx.x;
  float* xr = x + t * W;
  float r = 0.f;
  if (y != nullptr) {
    const TY* yr = y + t * W;
    float ss = 0.f;
    for (int c = threadIdx.x; c < W; c += 256) {
      const float v = ldf(yr + c);
      ss += v * v;
    }
    r = 1.f / sqrtf(block_reduce_sum<256>(ss, red) / (float)W + eps);
  }
  for (int c = threadIdx.x; c < W; c += 256) {
    float v = xr[c];
    if (y != nullptr) v += ldf(y + t * W + c) * r * (1.f + w[c]);
    if (hist != nullptr) {
      hist[(long)depth * TW + t * W + c] = v;
      float a = dwa[depth] * v;
      for (int j = depth - 1; j >= 0; --j) a += dwa[j] * hist[(long)j * TW + t * W + c];
      v = a;
    }
    if (y != nullptr || hist != nullptr) xr[c] = v;
    if (sizeof(TO) == 2) stf(h + t * W + c, v);
  }
}

torch::Tensor post_norm_add(torch::Tensor x, torch::Tensor y, torch::Tensor w, double eps, bool out_bf16,
                            torch::Tensor hist, int64_t depth, torch::Tensor dwa) {
  check_f32(x, "residual");
  TORCH_CHECK(x.dim() == 2);
  const int T_ = x.size(0), W = x.size(1);
  const bool has_y = y.numel() > 0, has_h = hist.numel() > 0;
  if (has_y) {
    TORCH_CHECK(y.is_cuda() && y.is_contiguous() && y.dim() == 2 && y.size(0) == T_ && y.size(1) == W);
    check_f32(w, "norm weight");
    TORCH_CHECK(w.numel() == W);
  }
  if (has_h) {
    check_f32(hist, "depth history"); check_f32(dwa, "depth weights");
    TORCH_CHECK(hist.dim() == 3 && hist.size(1) == T_ && hist.size(2) == W && depth >= 0 && depth < hist.size(0) &&
                dwa.numel() == depth + 1, "depth history [layers + 1, T, W] and one weight per entry up to depth");
  }
  torch::Tensor h = out_bf16 ? torch::empty({T_, W}, x.options().dtype(at::kBFloat16)) : x;
  if (T_ == 0) return h;
  auto stream = at::cuda::getCurrentHIPStream();
  const float* wp = has_y ? w.data_ptr<float>() : nullptr;
  float* hp = has_h ? hist.data_ptr<float>() : nullptr;
  const float* dp = has_h ? dwa.data_ptr<float>() : nullptr;
#define PN_LAUNCH(TY, TO)                                                                                        \
  hipLaunchKernelGGL((post_norm_add_kernel<TY, TO>), dim3(T_), dim3(256), 0, stream, x.data_ptr<float>(),        \
      has_y ? (const TY*)y.data_ptr() : nullptr, wp, (float)eps, out_bf16 ? (TO*)h.data_ptr() : nullptr, hp,     \
      (int)depth, dp, (long)T_ * W, W)
  const bool y16 = has_y && y.scalar_type() == at::kBFloat16;
  TORCH_CHECK(!has_y || y16 || y.scalar_type() == at::kFloat, "sublayer output is float32 or bfloat16");
  if (y16 && out_bf16) PN_LAUNCH(bf16, bf16);
  else if (y16) PN_LAUNCH(bf16, float);
  else if (out_bf16) PN_LAUNCH(float, bf16);
  else PN_LAUNCH(float, float);
#undef PN_LAUNCH
  return h;
}

// ---------------------------------------------------------------------------
// 0.5 z (1 + tanh(sqrt(2/pi) (z + 0.044715 z^3)))
// ---------------------------------------------------------------------------
template <typename T>
__global__ void gelu_tanh_kernel(const T* __restrict__ z, T* __restrict__ y, long N) {
  for (long i = blockIdx.x * (long)blockDim.x + threadIdx.x; i < N; i += (long)gridDim.x * blockDim.x) {
    const float v = ldf(z + i);
    stf(y + i, 0.5f * v * (1.f + tanhf(0.7978845608028654f * (v + 0.044715f * v * v * v))));
  }
}

torch::Tensor gelu_tanh(torch::Tensor z) {
  TORCH_CHECK(z.is_cuda() && z.is_contiguous());
  auto y = torch::empty_like(z);
  const long N = z.numel();
  if (N == 0) return y;
  auto stream = at::cuda::getCurrentHIPStream();
  RAGGED_DISPATCH(z, hipLaunchKernelGGL((gelu_tanh_kernel<T>), dim3(grid_for(N, 256)), dim3(256), 0, stream,
      (const T*)z.data_ptr(), (T*)y.data_ptr(), N));
  return y;
}
