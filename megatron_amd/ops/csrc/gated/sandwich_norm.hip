// Row kernels of layers that norm a sublayer on BOTH sides, x <- x + norm_b(f(norm_a(x))):
// the output norm of one sublayer, the residual add and the input norm of the next in one
// pass over the row; the restart of a repeated block of layers; the finishing steps of
// gated and of differential attention; squared ReLU.
#include "../ragged/ragged_common.h"

template <typename T>
__device__ __forceinline__ void ld4g(const T* p, float* v);
template <>
__device__ __forceinline__ void ld4g<float>(const float* p, float* v) {
  const float4v a = *reinterpret_cast<const float4v*>(p);
  v[0] = a[0]; v[1] = a[1]; v[2] = a[2]; v[3] = a[3];
}
template <>
__device__ __forceinline__ void ld4g<bf16>(const bf16* p, float* v) {
  typedef short short4v __attribute__((ext_vector_type(4)));
  const short4v a = *reinterpret_cast<const short4v*>(p);
  v[0] = sbf2f(a[0]); v[1] = sbf2f(a[1]); v[2] = sbf2f(a[2]); v[3] = sbf2f(a[3]);
}
__device__ __forceinline__ void st4g(float* p, const float* v) {
  *reinterpret_cast<float4v*>(p) = float4v{v[0], v[1], v[2], v[3]};
}
__device__ __forceinline__ void st4g(bf16* p, const float* v) {
  typedef short short4v __attribute__((ext_vector_type(4)));
  *reinterpret_cast<short4v*>(p) = short4v{f2sbf(v[0]), f2sbf(v[1]), f2sbf(v[2]), f2sbf(v[3])};
}

// ---------------------------------------------------------------------------
// RESTART = false:  x[t] <- x[t] + y[t] / sqrt(mean(y[t]^2) + eps) * wpost        (y given)
// RESTART = true:   x[t] <- y[t] + wpost                    (wpost = a bias row, x is written only)
// copy[t] <- x[t] in the GEMM type (row stride cstride)                           (copy given)
// h[t]    <- x[t] / sqrt(mean(x[t]^2) + eps) * wpre  in the GEMM type             (wpre given)
// Workgroup = token.  The row is read from memory once and kept in LDS as fp32.
// VEC: rows are a multiple of four wide and every access moves four elements.
// ---------------------------------------------------------------------------
template <typename TY, typename TO, bool VEC, bool RESTART>
__global__ __launch_bounds__(256) void sandwich_norm_kernel(
    float* __restrict__ x, const TY* __restrict__ y, const float* __restrict__ wpost,
    const float* __restrict__ wpre, float eps, TO* __restrict__ h, TO* __restrict__ copy, long cstride, int W) {
  extern __shared__ __align__(16) float row[];
  __shared__ float red_a[256 / WAVE], red_b[256 / WAVE];
  const long t = blockIdx.x;
  float* xr = x + t * W;
  constexpr int STEP = VEC ? 4 : 1;
  float ry = 0.f;
  if (y != nullptr && !RESTART) {
    const TY* yr = y + t * W;
    float ss = 0.f;
    for (int c = threadIdx.x * STEP; c < W; c += 256 * STEP) {
      float v[4] = {0.f, 0.f, 0.f, 0.f};
      if (VEC) ld4g<TY>(yr + c, v);
      else v[0] = ldf(yr + c);
#pragma unroll
      for (int i = 0; i < STEP; ++i) row[c + i] = v[i];
      ss += (v[0] * v[0] + v[1] * v[1]) + (v[2] * v[2] + v[3] * v[3]);
    }
    ry = 1.f / sqrtf(block_reduce_sum<256>(ss, red_a) / (float)W + eps);
  }
  float sx = 0.f;
  for (int c = threadIdx.x * STEP; c < W; c += 256 * STEP) {
    float v[4] = {0.f, 0.f, 0.f, 0.f}, wv[4] = {0.f, 0.f, 0.f, 0.f};
    if (RESTART) {
      if (VEC) { ld4g<TY>(y + t * W + c, v); ld4g<float>(wpost + c, wv); }
      else { v[0] = ldf(y + t * W + c); wv[0] = wpost[c]; }
#pragma unroll
      for (int i = 0; i < STEP; ++i) v[i] += wv[i];
    } else {
      if (VEC) ld4g<float>(xr + c, v);
      else v[0] = xr[c];
      if (y != nullptr) {
        if (VEC) ld4g<float>(wpost + c, wv);
        else wv[0] = wpost[c];
#pragma unroll
        for (int i = 0; i < STEP; ++i) v[i] += row[c + i] * ry * wv[i];   // this thread's own entries
      }
    }
    if (RESTART || y != nullptr) {
      if (VEC) st4g(xr + c, v);
      else xr[c] = v[0];
    }
    if (copy != nullptr) {
      if (VEC) st4g(copy + t * cstride + c, v);
      else stf(copy + t * cstride + c, v[0]);
    }
#pragma unroll
    for (int i = 0; i < STEP; ++i) row[c + i] = v[i];
    sx += (v[0] * v[0] + v[1] * v[1]) + (v[2] * v[2] + v[3] * v[3]);
  }
  if (wpre == nullptr) return;
  const float rx = 1.f / sqrtf(block_reduce_sum<256>(sx, red_b) / (float)W + eps);
  for (int c = threadIdx.x * STEP; c < W; c += 256 * STEP) {
    float v[4] = {0.f, 0.f, 0.f, 0.f}, wv[4] = {0.f, 0.f, 0.f, 0.f};
    if (VEC) ld4g<float>(wpre + c, wv);
    else wv[0] = wpre[c];
#pragma unroll
    for (int i = 0; i < STEP; ++i) v[i] = row[c + i] * rx * wv[i];
    if (VEC) st4g(h + t * W + c, v);
    else stf(h + t * W + c, v[0]);
  }
}

#define SN_LAUNCH1(TY, TO, VEC, RESTART)                                                                        \
  hipLaunchKernelGGL((sandwich_norm_kernel<TY, TO, VEC, RESTART>), dim3(T_), dim3(256), (size_t)W * sizeof(float), \
      stream, x.data_ptr<float>(), has_y ? (const TY*)y.data_ptr() : (const TY*)nullptr, wpost_p, wpre_p,        \
      (float)eps, has_pre ? (TO*)h.data_ptr() : (TO*)nullptr, has_c ? (TO*)copy_to.data_ptr() : (TO*)nullptr,    \
      cstride, W)
#define SN_LAUNCH(TY, TO, RESTART)                   \
  do {                                               \
    if (vec) SN_LAUNCH1(TY, TO, true, RESTART);      \
    else SN_LAUNCH1(TY, TO, false, RESTART);         \
  } while (0)
#define SN_DISPATCH(RESTART)                                 \
  do {                                                       \
    if (y16 && out_bf16) SN_LAUNCH(bf16, bf16, RESTART);     \
    else if (y16) SN_LAUNCH(bf16, float, RESTART);           \
    else if (out_bf16) SN_LAUNCH(float, bf16, RESTART);      \
    else SN_LAUNCH(float, float, RESTART);                   \
  } while (0)

torch::Tensor sandwich_norm_add(torch::Tensor x, torch::Tensor y, torch::Tensor w_post, torch::Tensor w_pre,
                                double eps, bool out_bf16, torch::Tensor copy_to) {
  check_f32(x, "residual");
  TORCH_CHECK(x.dim() == 2);
  const int T_ = x.size(0), W = x.size(1);
  const bool has_y = y.numel() > 0, has_pre = w_pre.numel() > 0, has_c = copy_to.numel() > 0;
  const auto out_t = out_bf16 ? at::kBFloat16 : at::kFloat;
  if (has_y) {
    TORCH_CHECK(y.is_cuda() && y.is_contiguous() && y.dim() == 2 && y.size(0) == T_ && y.size(1) == W);
    TORCH_CHECK(y.scalar_type() == at::kFloat || y.scalar_type() == at::kBFloat16, "sublayer output is float32 or bfloat16");
    check_f32(w_post, "output norm weight");
    TORCH_CHECK(w_post.numel() == W);
  }
  if (has_pre) {
    check_f32(w_pre, "input norm weight");
    TORCH_CHECK(w_pre.numel() == W);
  }
  long cstride = 0;
  if (has_c) {
    TORCH_CHECK(copy_to.is_cuda() && copy_to.dim() == 2 && copy_to.size(0) == T_ && copy_to.size(1) == W &&
                copy_to.stride(1) == 1 && copy_to.scalar_type() == out_t, "copy target [T, W] in the GEMM type");
    cstride = copy_to.stride(0);
  }
  TORCH_CHECK((size_t)W * sizeof(float) <= 60 * 1024, "row too wide for the norm kernel");
  auto h = has_pre ? torch::empty({T_, W}, x.options().dtype(out_t)) : torch::empty({0}, x.options().dtype(out_t));
  if (T_ == 0 || (!has_y && !has_pre && !has_c)) return h;
  const bool vec = W % 4 == 0 && (!has_c || (cstride % 4 == 0 && copy_to.storage_offset() % 4 == 0));
  const bool y16 = has_y && y.scalar_type() == at::kBFloat16;
  const float* wpost_p = has_y ? w_post.data_ptr<float>() : nullptr;
  const float* wpre_p = has_pre ? w_pre.data_ptr<float>() : nullptr;
  auto stream = at::cuda::getCurrentHIPStream();
  SN_DISPATCH(false);
  return h;
}

// x = y + bias (fresh fp32 residual), h = x / rms(x) * w_pre
std::vector<torch::Tensor> restart_norm(torch::Tensor y, torch::Tensor bias, torch::Tensor w_pre, double eps,
                                        bool out_bf16) {
  TORCH_CHECK(y.is_cuda() && y.is_contiguous() && y.dim() == 2);
  TORCH_CHECK(y.scalar_type() == at::kFloat || y.scalar_type() == at::kBFloat16);
  const int T_ = y.size(0), W = y.size(1);
  check_f32(bias, "bias row"); check_f32(w_pre, "input norm weight");
  TORCH_CHECK(bias.numel() == W && w_pre.numel() == W);
  TORCH_CHECK((size_t)W * sizeof(float) <= 60 * 1024, "row too wide for the norm kernel");
  const auto out_t = out_bf16 ? at::kBFloat16 : at::kFloat;
  auto x = torch::empty({T_, W}, y.options().dtype(at::kFloat));
  auto h = torch::empty({T_, W}, y.options().dtype(out_t));
  if (T_ == 0) return {x, h};
  const bool has_y = true, has_pre = true, has_c = false, vec = W % 4 == 0;
  const bool y16 = y.scalar_type() == at::kBFloat16;
  const long cstride = 0;
  torch::Tensor copy_to;
  const float* wpost_p = bias.data_ptr<float>();
  const float* wpre_p = w_pre.data_ptr<float>();
  auto stream = at::cuda::getCurrentHIPStream();
  SN_DISPATCH(true);
  return {x, h};
}
#undef SN_DISPATCH
#undef SN_LAUNCH
#undef SN_LAUNCH1

// ---------------------------------------------------------------------------
// out[t, c] = A[t, c] * sigmoid(gate[t, c])      (A fp32, gate a strided view)
// ---------------------------------------------------------------------------
template <typename T>
__global__ void gate_finish_kernel(const float* __restrict__ A, const T* __restrict__ gate, long gstride,
                                   T* __restrict__ out, long Tn, int N) {
  const long total = Tn * N;
  for (long i = blockIdx.x * (long)blockDim.x + threadIdx.x; i < total; i += (long)gridDim.x * blockDim.x) {
    const long t = i / N;
    const int c = (int)(i % N);
    stf(out + i, A[i] * sigmoidf_(ldf(gate + t * gstride + c)));
  }
}

torch::Tensor gate_finish(torch::Tensor A, torch::Tensor gate, bool out_bf16) {
  check_f32(A, "attention result");
  TORCH_CHECK(A.dim() == 2 && gate.is_cuda() && gate.dim() == 2 && gate.stride(1) == 1 && gate.sizes() == A.sizes());
  TORCH_CHECK(gate.scalar_type() == (out_bf16 ? at::kBFloat16 : at::kFloat), "gate in the compute type");
  const long Tn = A.size(0);
  const int N = A.size(1);
  auto out = torch::empty({Tn, N}, gate.options());
  if (Tn == 0) return out;
  auto stream = at::cuda::getCurrentHIPStream();
  RAGGED_DISPATCH(gate, hipLaunchKernelGGL((gate_finish_kernel<T>), dim3(grid_for(Tn * N, 256)), dim3(256), 0, stream,
      A.data_ptr<float>(), (const T*)gate.data_ptr(), (long)gate.stride(0), (T*)out.data_ptr(), Tn, N));
  return out;
}

// ---------------------------------------------------------------------------
// A [T, H, 2, V] fp32 -> out[t, h, :] = o / sqrt(mean(o^2) + eps) * (1 - diff) * sigmoid(gate[t, h]),
// o = A[t, h, 0] - lam * A[t, h, 1].  Workgroup = token, a wave takes heads in turn.
// ---------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void differential_finish_kernel(
    const float* __restrict__ A, const T* __restrict__ gate, long gstride, const float* __restrict__ lam,
    float diff, float eps, T* __restrict__ out, int H, int V) {
  const long t = blockIdx.x;
  const int wave = threadIdx.x / WAVE, lane = threadIdx.x % WAVE;
  const float lm = lam[0];
  for (int hd = wave; hd < H; hd += 256 / WAVE) {
    const float* a1 = A + ((t * H + hd) * 2) * V;
    const float* a2 = a1 + V;
    float ss = 0.f;
    for (int d = lane; d < V; d += WAVE) {
      const float o = a1[d] - lm * a2[d];
      ss += o * o;
    }
    const float r = 1.f / sqrtf(wave_reduce_sum(ss) / (float)V + eps) * (1.f - diff) *
                    sigmoidf_(ldf(gate + t * gstride + hd));
    for (int d = lane; d < V; d += WAVE) stf(out + (t * H + hd) * V + d, (a1[d] - lm * a2[d]) * r);
  }
}

torch::Tensor differential_finish(torch::Tensor A, torch::Tensor gate, torch::Tensor lam, double diff, double eps,
                                  int64_t H, int64_t V, bool out_bf16) {
  check_f32(A, "attention result"); check_f32(lam, "lambda");
  TORCH_CHECK(A.dim() == 2 && A.size(1) == H * 2 * V && lam.numel() == 1);
  const long Tn = A.size(0);
  TORCH_CHECK(gate.is_cuda() && gate.dim() == 2 && gate.stride(1) == 1 && gate.size(0) == Tn && gate.size(1) == H);
  TORCH_CHECK(gate.scalar_type() == (out_bf16 ? at::kBFloat16 : at::kFloat), "gate in the compute type");
  auto out = torch::empty({Tn, H * V}, gate.options());
  if (Tn == 0) return out;
  auto stream = at::cuda::getCurrentHIPStream();
  RAGGED_DISPATCH(gate, hipLaunchKernelGGL((differential_finish_kernel<T>), dim3(Tn), dim3(256), 0, stream,
      A.data_ptr<float>(), (const T*)gate.data_ptr(), (long)gate.stride(0), lam.data_ptr<float>(), (float)diff,
      (float)eps, (T*)out.data_ptr(), (int)H, (int)V));
  return out;
}

// ---------------------------------------------------------------------------
// max(z, 0)^2
// ---------------------------------------------------------------------------
template <typename T>
__global__ void relu2_kernel(const T* __restrict__ z, T* __restrict__ y, long N) {
  const long n4 = N / 4;
  for (long i = blockIdx.x * (long)blockDim.x + threadIdx.x; i < n4; i += (long)gridDim.x * blockDim.x) {
    float v[4];
    ld4g<T>(z + 4 * i, v);
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const float r = fmaxf(v[k], 0.f);
      v[k] = r * r;
    }
    st4g(y + 4 * i, v);
  }
  for (long i = 4 * n4 + blockIdx.x * (long)blockDim.x + threadIdx.x; i < N; i += (long)gridDim.x * blockDim.x) {
    const float r = fmaxf(ldf(z + i), 0.f);
    stf(y + i, r * r);
  }
}

torch::Tensor relu2(torch::Tensor z) {
  TORCH_CHECK(z.is_cuda() && z.is_contiguous());
  auto y = torch::empty_like(z);
  const long N = z.numel();
  if (N == 0) return y;
  auto stream = at::cuda::getCurrentHIPStream();
  RAGGED_DISPATCH(z, hipLaunchKernelGGL((relu2_kernel<T>), dim3(grid_for((N + 3) / 4, 256)), dim3(256), 0, stream,
      (const T*)z.data_ptr(), (T*)y.data_ptr(), N));
  return y;
}
