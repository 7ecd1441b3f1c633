// Residual updates of layers that norm a sublayer's OUTPUT and hand on a
// weighted sum over depth, and the tanh form of GELU.
#include "../ragged/ragged_common.h"

// ---------------------------------------------------------------------------
// x[t] <- x[t] + y[t] / sqrt(mean(y[t]^2) + eps) * (1 + w)          (y given)
// hist[depth][t] <- x[t];  x[t] <- sum_{j <= depth} dwa[j] hist[j][t]  (hist given)
// h[t] <- x[t] in the next GEMM's input type (TO = float: x itself is that input).
// Workgroup = token.  x, hist fp32; the row of y is read twice (second time from L1/L2).
// ---------------------------------------------------------------------------
template <typename T>
__device__ __forceinline__ void ld4(const T* p, float* v);
template <>
__device__ __forceinline__ void ld4<float>(const float* p, float* v) {
  const float4v a = *reinterpret_cast<const float4v*>(p);
  v[0] = a[0]; v[1] = a[1]; v[2] = a[2]; v[3] = a[3];
}
template <>
__device__ __forceinline__ void ld4<bf16>(const bf16* p, float* v) {
  typedef short short4v __attribute__((ext_vector_type(4)));
  const short4v a = *reinterpret_cast<const short4v*>(p);
  v[0] = sbf2f(a[0]); v[1] = sbf2f(a[1]); v[2] = sbf2f(a[2]); v[3] = sbf2f(a[3]);
}
__device__ __forceinline__ void st4(float* p, const float* v) {
  *reinterpret_cast<float4v*>(p) = float4v{v[0], v[1], v[2], v[3]};
}
__device__ __forceinline__ void st4(bf16* p, const float* v) {
  typedef short short4v __attribute__((ext_vector_type(4)));
  *reinterpret_cast<short4v*>(p) = short4v{f2sbf(v[0]), f2sbf(v[1]), f2sbf(v[2]), f2sbf(v[3])};
}

// VEC: rows are a multiple of four wide, every access moves four elements
template <typename TY, typename TO, bool VEC>
__global__ __launch_bounds__(256) void post_norm_add_kernel(
    float* __restrict__ x, const TY* __restrict__ y, const float* __restrict__ w, float eps, TO* __restrict__ h,
    float* __restrict__ hist, int depth, const float* __restrict__ dwa, long TW, int W) {
  __shared__ float red[256 / WAVE];
  const long t = blockIdx.x;
  float* xr = x + t * W;
  constexpr int STEP = VEC ? 4 : 1;
  float r = 0.f;
  if (y != nullptr) {
    const TY* yr = y + t * W;
    float ss = 0.f;
    for (int c = threadIdx.x * STEP; c < W; c += 256 * STEP) {
      float v[4] = {0.f, 0.f, 0.f, 0.f};
      if (VEC) ld4<TY>(yr + c, v);
      else v[0] = ldf(yr + c);
      ss += (v[0] * v[0] + v[1] * v[1]) + (v[2] * v[2] + v[3] * v[3]);
    }
    r = 1.f / sqrtf(block_reduce_sum<256>(ss, red) / (float)W + eps);
  }
  for (int c = threadIdx.x * STEP; c < W; c += 256 * STEP) {
    float v[4] = {0.f, 0.f, 0.f, 0.f};
    if (VEC) ld4<float>(xr + c, v);
    else v[0] = xr[c];
    if (y != nullptr) {
      float yv[4] = {0.f, 0.f, 0.f, 0.f}, wv[4] = {0.f, 0.f, 0.f, 0.f};
      if (VEC) { ld4<TY>(y + t * W + c, yv); ld4<float>(w + c, wv); }
      else { yv[0] = ldf(y + t * W + c); wv[0] = w[c]; }
#pragma unroll
      for (int i = 0; i < STEP; ++i) v[i] += yv[i] * r * (1.f + wv[i]);
    }
    if (hist != nullptr) {
      float* hr = hist + t * W + c;
      if (VEC) st4(hr + (long)depth * TW, v);
      else hr[(long)depth * TW] = v[0];
      const float dd = dwa[depth];
#pragma unroll
      for (int i = 0; i < STEP; ++i) v[i] *= dd;
      for (int j = depth - 1; j >= 0; --j) {
        float hv[4] = {0.f, 0.f, 0.f, 0.f};
        if (VEC) ld4<float>(hr + (long)j * TW, hv);
        else hv[0] = hr[(long)j * TW];
        const float dj = dwa[j];
#pragma unroll
        for (int i = 0; i < STEP; ++i) v[i] += dj * hv[i];
      }
    }
    if (y != nullptr || hist != nullptr) {
      if (VEC) st4(xr + c, v);
      else xr[c] = v[0];
    }
    if (sizeof(TO) == 2) {
      if (VEC) st4(h + t * W + c, v);
      else stf(h + t * W + c, v[0]);
    }
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
#define PN_LAUNCH1(TY, TO, VEC)                                                                                  \
  hipLaunchKernelGGL((post_norm_add_kernel<TY, TO, VEC>), dim3(T_), dim3(256), 0, stream, x.data_ptr<float>(),   \
      has_y ? (const TY*)y.data_ptr() : nullptr, wp, (float)eps, out_bf16 ? (TO*)h.data_ptr() : nullptr, hp,     \
      (int)depth, dp, (long)T_ * W, W)
#define PN_LAUNCH(TY, TO)            \
  do {                               \
    if (W % 4 == 0) PN_LAUNCH1(TY, TO, true); \
    else PN_LAUNCH1(TY, TO, false);  \
  } while (0)
  const bool y16 = has_y && y.scalar_type() == at::kBFloat16;
  TORCH_CHECK(!has_y || y16 || y.scalar_type() == at::kFloat, "sublayer output is float32 or bfloat16");
  if (y16 && out_bf16) PN_LAUNCH(bf16, bf16);
  else if (y16) PN_LAUNCH(bf16, float);
  else if (out_bf16) PN_LAUNCH(float, bf16);
  else PN_LAUNCH(float, float);
#undef PN_LAUNCH
#undef PN_LAUNCH1
  return h;
}

// ---------------------------------------------------------------------------
// 0.5 z (1 + tanh(sqrt(2/pi) (z + 0.044715 z^3)))
// ---------------------------------------------------------------------------
__device__ __forceinline__ float gelu_tanh_(float v) {
  return 0.5f * v * (1.f + tanhf(0.7978845608028654f * (v + 0.044715f * v * v * v)));
}

// four elements a thread and turn; the tail (N % 4) by single elements
template <typename T>
__global__ void gelu_tanh_kernel(const T* __restrict__ z, T* __restrict__ y, long N) {
  const long n4 = N / 4;
  for (long i = blockIdx.x * (long)blockDim.x + threadIdx.x; i < n4; i += (long)gridDim.x * blockDim.x) {
    float v[4];
    ld4<T>(z + 4 * i, v);
#pragma unroll
    for (int k = 0; k < 4; ++k) v[k] = gelu_tanh_(v[k]);
    st4(y + 4 * i, v);
  }
  for (long i = 4 * n4 + blockIdx.x * (long)blockDim.x + threadIdx.x; i < N; i += (long)gridDim.x * blockDim.x)
    stf(y + i, gelu_tanh_(ldf(z + i)));
}

torch::Tensor gelu_tanh(torch::Tensor z) {
  TORCH_CHECK(z.is_cuda() && z.is_contiguous());
  auto y = torch::empty_like(z);
  const long N = z.numel();
  if (N == 0) return y;
  auto stream = at::cuda::getCurrentHIPStream();
  RAGGED_DISPATCH(z, hipLaunchKernelGGL((gelu_tanh_kernel<T>), dim3(grid_for((N + 3) / 4, 256)), dim3(256), 0, stream,
      (const T*)z.data_ptr(), (T*)y.data_ptr(), N));
  return y;
}
