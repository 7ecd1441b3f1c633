// Routed GLU experts (clamped, kind 0, SiLU, kind 1, tanh-GELU, kind 2) and experts without a gate
// matrix (squared ReLU) for steps with few (token, choice) pairs
// (decoding): every pair reads its expert's matrices directly, no sorting, no
// host read.  Two kernels:
//   y[pair, f]   = act(W_gate[e][f] . x, W_up[e][f] . x)     grid (pair, tiles of rows f)
//   out[pair, w] = W_down[e][w] . y[pair]                    grid (pair, tiles of rows w)
// A wave computes one output row at a time: lanes stride over the input in
// 8-element pieces (16 B of bf16), shuffle-reduce; the input vector is staged
// in LDS as fp32.  Memory-bound: each pair streams 3 F W weights once.
#include "../ragged/ragged_common.h"

constexpr int EP_ROWS = 32;          // output rows per workgroup (8 per wave)

template <typename T>
__device__ __forceinline__ void load8(const T* p, float* v);
template <>
__device__ __forceinline__ void load8<bf16>(const bf16* p, float* v) {
  const short8 x = *reinterpret_cast<const short8*>(p);
#pragma unroll
  for (int i = 0; i < 8; ++i) v[i] = sbf2f(x[i]);
}
template <>
__device__ __forceinline__ void load8<float>(const float* p, float* v) {
  const float4v a = *reinterpret_cast<const float4v*>(p), b = *reinterpret_cast<const float4v*>(p + 4);
#pragma unroll
  for (int i = 0; i < 4; ++i) { v[i] = a[i]; v[4 + i] = b[i]; }
}

template <typename T>
__global__ __launch_bounds__(256) void expert_gate_up_kernel(
    const T* __restrict__ h, const int* __restrict__ ids, const T* __restrict__ wgu, T* __restrict__ y, int K,
    int W, int F, float limit, float alpha, int kind) {
  extern __shared__ float xs[];                  // the token's input, fp32
  const int pair = blockIdx.x, t = pair / K;
  const long e = ids[pair];
  for (int i = threadIdx.x; i < W; i += 256) xs[i] = ldf(h + (long)t * W + i);
  __syncthreads();
  const int wave = threadIdx.x / WAVE, lane = threadIdx.x % WAVE;
  const T* base = wgu + e * 2L * F * W;
  for (int fi = wave; fi < EP_ROWS; fi += 4) {
    const int f = blockIdx.y * EP_ROWS + fi;
    if (f >= F) break;
    const T* gr = base + (long)f * W;
    const T* ur = base + (long)(F + f) * W;
    float ag = 0.f, au = 0.f;
    for (int d = lane * 8; d < W; d += WAVE * 8) {
      float a[8], b[8];
      load8<T>(gr + d, a);
      load8<T>(ur + d, b);
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        ag += a[i] * xs[d + i];
        au += b[i] * xs[d + i];
      }
    }
    ag = wave_reduce_sum(ag);
    au = wave_reduce_sum(au);
    if (lane == 0) {
      // the products' results take the storage type's rounding, as a GEMM's output would
      float g = ag, u = au;
      if (sizeof(T) == 2) { g = sbf2f(f2sbf(g)); u = sbf2f(f2sbf(u)); }
      if (kind == 0) {
        g = fminf(g, limit);
        u = fminf(fmaxf(u, -limit), limit);
        stf(y + (long)pair * F + f, g * sigmoidf_(alpha * g) * (u + 1.f));
      } else if (kind == 1) {
        stf(y + (long)pair * F + f, g * sigmoidf_(g) * u);
      } else {
        stf(y + (long)pair * F + f, 0.5f * g * (1.f + tanhf(0.7978845608028654f * (g + 0.044715f * g * g * g))) * u);
      }
    }
  }
}

template <typename T>
__global__ __launch_bounds__(256) void expert_down_kernel(const T* __restrict__ y, const int* __restrict__ ids,
                                                          const T* __restrict__ wd, T* __restrict__ out, int W,
                                                          int F) {
  extern __shared__ float ys[];
  const int pair = blockIdx.x;
  const long e = ids[pair];
  for (int i = threadIdx.x; i < F; i += 256) ys[i] = ldf(y + (long)pair * F + i);
  __syncthreads();
  const int wave = threadIdx.x / WAVE, lane = threadIdx.x % WAVE;
  const T* base = wd + e * (long)W * F;
  // two rows in flight a wave: rows wi and wi + 4 of the workgroup's EP_ROWS
  for (int wi = wave; wi < EP_ROWS; wi += 8) {
    const int w0 = blockIdx.y * EP_ROWS + wi, w1 = w0 + 4;
    if (w0 >= W) break;
    const bool two = w1 < W && wi + 4 < EP_ROWS;
    const T* r0 = base + (long)w0 * F;
    const T* r1 = base + (long)(two ? w1 : w0) * F;
    float a0 = 0.f, a1 = 0.f;
    for (int d = lane * 8; d < F; d += WAVE * 8) {
      float b0[8], b1[8];
      load8<T>(r0 + d, b0);
      load8<T>(r1 + d, b1);
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        a0 += b0[i] * ys[d + i];
        a1 += b1[i] * ys[d + i];
      }
    }
    a0 = wave_reduce_sum(a0);
    a1 = wave_reduce_sum(a1);
    if (lane == 0) {
      stf(out + (long)pair * W + w0, a0);
      if (two) stf(out + (long)pair * W + w1, a1);
    }
  }
}

// experts WITHOUT a gate matrix: y[pair, f] = max(W_up[e][f] . x, 0)^2
template <typename T>
__global__ __launch_bounds__(256) void expert_up_relu2_kernel(
    const T* __restrict__ h, const int* __restrict__ ids, const T* __restrict__ wu, T* __restrict__ y, int K,
    int W, int F) {
  extern __shared__ float xs[];                  // the token's input, fp32
  const int pair = blockIdx.x, t = pair / K;
  const long e = ids[pair];
  for (int i = threadIdx.x; i < W; i += 256) xs[i] = ldf(h + (long)t * W + i);
  __syncthreads();
  const int wave = threadIdx.x / WAVE, lane = threadIdx.x % WAVE;
  const T* base = wu + e * (long)F * W;
  // two rows in flight a wave: rows fi and fi + 4 of the workgroup's EP_ROWS
  for (int fi = wave; fi < EP_ROWS; fi += 8) {
    const int f0 = blockIdx.y * EP_ROWS + fi, f1 = f0 + 4;
    if (f0 >= F) break;
    const bool two = f1 < F && fi + 4 < EP_ROWS;
    const T* r0 = base + (long)f0 * W;
    const T* r1 = base + (long)(two ? f1 : f0) * W;
    float a0 = 0.f, a1 = 0.f;
    for (int d = lane * 8; d < W; d += WAVE * 8) {
      float b0[8], b1[8];
      load8<T>(r0 + d, b0);
      load8<T>(r1 + d, b1);
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        a0 += b0[i] * xs[d + i];
        a1 += b1[i] * xs[d + i];
      }
    }
    a0 = wave_reduce_sum(a0);
    a1 = wave_reduce_sum(a1);
    if (lane == 0) {
      // the product's result takes the storage type's rounding, as a GEMM's output would
      float u0 = a0, u1 = a1;
      if (sizeof(T) == 2) { u0 = sbf2f(f2sbf(u0)); u1 = sbf2f(f2sbf(u1)); }
      u0 = fmaxf(u0, 0.f);
      u1 = fmaxf(u1, 0.f);
      stf(y + (long)pair * F + f0, u0 * u0);
      if (two) stf(y + (long)pair * F + f1, u1 * u1);
    }
  }
}

// h [T, W], ids [T, K], w_up [E, F, W], w_down [E, W, F] -> rows [T * K, W] in pair order (token-major)
torch::Tensor expert_pairs_plain(torch::Tensor h, torch::Tensor ids, torch::Tensor wu, torch::Tensor wd) {
  TORCH_CHECK(h.is_cuda() && h.dim() == 2 && h.is_contiguous());
  check_i32(ids, "ids");
  TORCH_CHECK(wu.is_contiguous() && wu.dim() == 3 && wd.is_contiguous() && wd.dim() == 3);
  TORCH_CHECK(wu.scalar_type() == h.scalar_type() && wd.scalar_type() == h.scalar_type());
  const int T_ = h.size(0), W = h.size(1), E = wu.size(0), F = wu.size(1);
  TORCH_CHECK(ids.dim() == 2 && ids.size(0) == T_);
  const int K = ids.size(1);
  TORCH_CHECK(wu.size(2) == W && wd.size(0) == E && wd.size(1) == W && wd.size(2) == F);
  TORCH_CHECK(W % 8 == 0 && F % 8 == 0, "pair kernels take widths that are multiples of 8");
  TORCH_CHECK((size_t)std::max(W, F) * sizeof(float) <= 60 * 1024, "input vector above the LDS staging size");
  const int N = T_ * K;
  auto out = torch::empty({N, W}, h.options());
  if (N == 0) return out;
  auto y = torch::empty({N, F}, h.options());
  auto stream = at::cuda::getCurrentHIPStream();
  RAGGED_DISPATCH(h, {
    hipLaunchKernelGGL((expert_up_relu2_kernel<T>), dim3(N, (F + EP_ROWS - 1) / EP_ROWS), dim3(256),
        (size_t)W * sizeof(float), stream, (const T*)h.data_ptr(), ids.data_ptr<int>(), (const T*)wu.data_ptr(),
        (T*)y.data_ptr(), K, W, F);
    hipLaunchKernelGGL((expert_down_kernel<T>), dim3(N, (W + EP_ROWS - 1) / EP_ROWS), dim3(256),
        (size_t)F * sizeof(float), stream, (const T*)y.data_ptr(), ids.data_ptr<int>(), (const T*)wd.data_ptr(),
        (T*)out.data_ptr(), W, F);
  });
  return out;
}

// h [T, W], ids [T, K] -> rows [T * K, W] in pair order (token-major)
torch::Tensor expert_pairs(torch::Tensor h, torch::Tensor ids, torch::Tensor wgu, torch::Tensor wd, double limit,
                           double alpha, int64_t kind) {
  TORCH_CHECK(kind >= 0 && kind <= 2, "GLU kind: 0 clamped, 1 SiLU, 2 tanh-GELU");
  TORCH_CHECK(h.is_cuda() && h.dim() == 2 && h.is_contiguous());
  check_i32(ids, "ids");
  TORCH_CHECK(wgu.is_contiguous() && wgu.dim() == 3 && wd.is_contiguous() && wd.dim() == 3);
  TORCH_CHECK(wgu.scalar_type() == h.scalar_type() && wd.scalar_type() == h.scalar_type());
  const int T_ = h.size(0), W = h.size(1), E = wgu.size(0), F = wgu.size(1) / 2;
  TORCH_CHECK(ids.dim() == 2 && ids.size(0) == T_);
  const int K = ids.size(1);
  TORCH_CHECK(wgu.size(1) == 2 * F && wgu.size(2) == W && wd.size(0) == E && wd.size(1) == W && wd.size(2) == F);
  TORCH_CHECK(W % 8 == 0 && F % 8 == 0, "pair kernels take widths that are multiples of 8");
  TORCH_CHECK((size_t)std::max(W, F) * sizeof(float) <= 60 * 1024, "input vector above the LDS staging size");
  const int N = T_ * K;
  auto out = torch::empty({N, W}, h.options());
  if (N == 0) return out;
  auto y = torch::empty({N, F}, h.options());
  auto stream = at::cuda::getCurrentHIPStream();
  RAGGED_DISPATCH(h, {
    hipLaunchKernelGGL((expert_gate_up_kernel<T>), dim3(N, (F + EP_ROWS - 1) / EP_ROWS), dim3(256),
        (size_t)W * sizeof(float), stream, (const T*)h.data_ptr(), ids.data_ptr<int>(), (const T*)wgu.data_ptr(),
        (T*)y.data_ptr(), K, W, F, (float)limit, (float)alpha, (int)kind);
    hipLaunchKernelGGL((expert_down_kernel<T>), dim3(N, (W + EP_ROWS - 1) / EP_ROWS), dim3(256),
        (size_t)F * sizeof(float), stream, (const T*)y.data_ptr(), ids.data_ptr<int>(), (const T*)wd.data_ptr(),
        (T*)out.data_ptr(), W, F);
  });
  return out;
}
