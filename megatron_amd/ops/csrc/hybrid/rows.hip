// Row kernels of the plain-residual serving path: embedding gather into the
// fp32 residual, residual add fused with grouped RMS norm (one or two normed
// copies of the same row), and the elementwise / per-token parts of routed
// clamped-GLU experts (routing, activation, weighted combine).
#include "../ragged/ragged_common.h"

// ---------------------------------------------------------------------------
// x[t] = embed[token[t]]  (fp32)
// ---------------------------------------------------------------------------
template <typename T>
__global__ void embed_plain_kernel(const long* __restrict__ tokens, const T* __restrict__ embed,
                                   float* __restrict__ x, int W) {
  const long t = blockIdx.x;
  const T* row = embed + tokens[t] * (long)W;
  for (int c = threadIdx.x; c < W; c += blockDim.x) x[t * W + c] = ldf(row + c);
}

torch::Tensor embed_plain(torch::Tensor tokens, torch::Tensor embed) {
  TORCH_CHECK(tokens.is_cuda() && tokens.scalar_type() == at::kLong && tokens.is_contiguous() && tokens.dim() == 1);
  TORCH_CHECK(embed.is_cuda() && embed.dim() == 2 && embed.is_contiguous());
  const int T_ = tokens.numel(), W = embed.size(1);
  auto x = torch::empty({T_, W}, embed.options().dtype(at::kFloat));
  if (T_ == 0) return x;
  auto stream = at::cuda::getCurrentHIPStream();
  RAGGED_DISPATCH(embed, hipLaunchKernelGGL((embed_plain_kernel<T>), dim3(T_), dim3(256), 0, stream,
      tokens.data_ptr<long>(), (const T*)embed.data_ptr(), x.data_ptr<float>(), W));
  return x;
}

// ---------------------------------------------------------------------------
// x += y ; n = x / rms(x) per group ; h_a = n * w_a ; h_b = n * w_b
// One workgroup per token; the row is staged in LDS, wave w reduces the
// groups w, w + 4, ...
// ---------------------------------------------------------------------------
constexpr int GN_MAX_GROUPS = 256;

template <typename TY, typename TO>
__global__ __launch_bounds__(256) void residual_group_norm_kernel(
    float* __restrict__ x, const TY* __restrict__ y, const float* __restrict__ wa, const float* __restrict__ wb,
    TO* __restrict__ ha, TO* __restrict__ hb, int W, int groups, float eps) {
  extern __shared__ float row[];
  __shared__ float rs[GN_MAX_GROUPS];
  const long t = blockIdx.x;
  float* xp = x + t * W;
  for (int c = threadIdx.x; c < W; c += 256) {
    float v = xp[c];
    if (y != nullptr) {
      v += ldf(y + t * W + c);
      xp[c] = v;
    }
    row[c] = v;
  }
  __syncthreads();
  const int gs = W / groups, wave = threadIdx.x / WAVE, lane = threadIdx.x % WAVE;
  for (int g = wave; g < groups; g += 4) {
    float ss = 0.f;
    for (int i = lane; i < gs; i += WAVE) {
      const float v = row[g * gs + i];
      ss += v * v;
    }
    ss = wave_reduce_sum(ss);
    if (lane == 0) rs[g] = 1.f / sqrtf(ss / (float)gs + eps);
  }
  __syncthreads();
  for (int c = threadIdx.x; c < W; c += 256) {
    const float n = row[c] * rs[c / gs];
    stf(ha + t * W + c, n * wa[c]);
    if (hb != nullptr) stf(hb + t * W + c, n * wb[c]);
  }
}

std::vector<torch::Tensor> residual_group_norm(torch::Tensor x, torch::Tensor y, torch::Tensor wa, torch::Tensor wb,
                                               int64_t groups, double eps, bool out_bf16) {
  check_f32(x, "x"); check_f32(wa, "w_a");
  TORCH_CHECK(x.dim() == 2);
  const int T_ = x.size(0), W = x.size(1);
  const bool has_y = y.numel() > 0, has_b = wb.numel() > 0;
  TORCH_CHECK(groups >= 1 && groups <= GN_MAX_GROUPS && W % groups == 0, "norm groups divide the width");
  TORCH_CHECK(wa.numel() == W && (!has_b || (wb.numel() == W && wb.scalar_type() == at::kFloat && wb.is_cuda())));
  if (has_y) {
    TORCH_CHECK(y.is_cuda() && y.is_contiguous() && y.dim() == 2 && y.size(0) == T_ && y.size(1) == W);
    TORCH_CHECK(y.scalar_type() == at::kFloat || y.scalar_type() == at::kBFloat16);
  }
  auto ho = x.options().dtype(out_bf16 ? at::kBFloat16 : at::kFloat);
  auto ha = torch::empty({T_, W}, ho);
  auto hb = has_b ? torch::empty({T_, W}, ho) : torch::empty({0}, ho);
  if (T_ == 0) return {ha, hb};
  auto stream = at::cuda::getCurrentHIPStream();
  const size_t smem = (size_t)W * sizeof(float);
  TORCH_CHECK(smem <= 60 * 1024, "row too wide for the norm kernel");
#define GN_LAUNCH(TY, TO)                                                                                        \
  hipLaunchKernelGGL((residual_group_norm_kernel<TY, TO>), dim3(T_), dim3(256), smem, stream, x.data_ptr<float>(), \
      has_y ? (const TY*)y.data_ptr() : (const TY*)nullptr, wa.data_ptr<float>(),                                \
      has_b ? wb.data_ptr<float>() : (const float*)nullptr, (TO*)ha.data_ptr(),                                  \
      has_b ? (TO*)hb.data_ptr() : (TO*)nullptr, W, (int)groups, (float)eps)
  const bool y_bf = has_y && y.scalar_type() == at::kBFloat16;
  if (y_bf && out_bf16) GN_LAUNCH(bf16, bf16);
  else if (y_bf) GN_LAUNCH(bf16, float);
  else if (out_bf16) GN_LAUNCH(float, bf16);
  else GN_LAUNCH(float, float);
#undef GN_LAUNCH
  return {ha, hb};
}

// ---------------------------------------------------------------------------
// routing: sigmoid scores, group-limited top-k, normalised weights.
// One thread per token.
// ---------------------------------------------------------------------------
constexpr int RT_MAX_TOP = 16, RT_MAX_GROUPS = 64;

__global__ void moe_route_kernel(const float* __restrict__ logits, long stride, int Tn, int E, int top, int groups,
                                 int keep, float scale, int* __restrict__ ids, float* __restrict__ wts) {
  const int t = blockIdx.x * blockDim.x + threadIdx.x;
  if (t >= Tn) return;
  const float* z = logits + (long)t * stride;
  unsigned long long allowed = ~0ull;             // bit g: group g may be chosen from
  const int per = E / groups;
  if (groups > 1) {
    float gsc[RT_MAX_GROUPS];
    for (int g = 0; g < groups; ++g) {
      float a = -1.f, b = -1.f;                   // two largest scores of the group (scores lie in (0, 1))
      for (int i = 0; i < per; ++i) {
        const float s = sigmoidf_(z[g * per + i]);
        if (s > a) { b = a; a = s; }
        else if (s > b) b = s;
      }
      gsc[g] = a + (per > 1 ? b : 0.f);
    }
    allowed = 0ull;
    for (int n = 0; n < keep; ++n) {
      int best = -1;
      float bv = -INFINITY;
      for (int g = 0; g < groups; ++g)
        if (!((allowed >> g) & 1ull) && gsc[g] > bv) { bv = gsc[g]; best = g; }
      if (best >= 0) allowed |= 1ull << best;
    }
  }
  int chosen[RT_MAX_TOP];
  float cs[RT_MAX_TOP];
  float sum = 0.f;
  for (int n = 0; n < top; ++n) {
    int best = -1;
    float bv = -INFINITY;
    for (int e = 0; e < E; ++e) {
      if (groups > 1 && !((allowed >> (e / per)) & 1ull)) continue;
      bool taken = false;
      for (int m = 0; m < n; ++m) taken |= chosen[m] == e;
      if (taken) continue;
      const float s = sigmoidf_(z[e]);
      if (s > bv) { bv = s; best = e; }
    }
    chosen[n] = best < 0 ? 0 : best;
    cs[n] = best < 0 ? 0.f : bv;
    sum += cs[n];
  }
  for (int n = 0; n < top; ++n) {
    ids[(long)t * top + n] = chosen[n];
    wts[(long)t * top + n] = cs[n] / (sum + 1e-20f) * scale;
  }
}

std::vector<torch::Tensor> moe_route(torch::Tensor logits, int64_t E, int64_t top, int64_t groups, int64_t keep,
                                     double scale) {
  TORCH_CHECK(logits.is_cuda() && logits.scalar_type() == at::kFloat && logits.dim() == 2 && logits.stride(1) == 1);
  TORCH_CHECK(E >= 1 && E <= logits.size(1) && top >= 1 && top <= RT_MAX_TOP && top <= E, "experts chosen per token");
  TORCH_CHECK(groups >= 1 && groups <= RT_MAX_GROUPS && E % groups == 0 && keep >= 1 && keep <= groups);
  TORCH_CHECK(groups == 1 || keep * (E / groups) >= top, "the kept groups hold fewer experts than are chosen");
  const int T_ = logits.size(0);
  auto ids = torch::empty({T_, top}, logits.options().dtype(at::kInt));
  auto wts = torch::empty({T_, top}, logits.options());
  if (T_ == 0) return {ids, wts};
  auto stream = at::cuda::getCurrentHIPStream();
  hipLaunchKernelGGL(moe_route_kernel, dim3((T_ + 63) / 64), dim3(64), 0, stream, logits.data_ptr<float>(),
                     (long)logits.stride(0), T_, (int)E, (int)top, (int)groups, (int)keep, (float)scale,
                     ids.data_ptr<int>(), wts.data_ptr<float>());
  return {ids, wts};
}

// ---------------------------------------------------------------------------
// router in one kernel: logits = W_r h (+ bias) in fp32 (W_r fp32, h from its
// storage type), then either sigmoid scores, group-limited top-k and weights =
// chosen scores / their sum * scale (score 0), or the largest logits and
// weights = softmax over the chosen logits (score 1) or their softmax over ALL
// experts (score 2: the weights do not sum to one); rows beyond the experts
// (a shared expert's gate vector) are returned as raw logits.
// One workgroup per token: its eight waves take the rows of W_r in turn (16 B
// loads, four partial sums), one thread selects from the scores in LDS.
// ---------------------------------------------------------------------------
constexpr int RF_MAX_ROWS = 512;

constexpr int RF_THREADS = 512;

template <typename T>
__global__ __launch_bounds__(RF_THREADS) void moe_router_kernel(
    const T* __restrict__ h, const float* __restrict__ wr, const float* __restrict__ bias, int W, int rows, int E,
    int top, int groups, int keep, float scale, int score, int* __restrict__ ids, float* __restrict__ wts,
    float* __restrict__ extra) {
  extern __shared__ __align__(16) float xs[];    // the token's input, fp32
  __shared__ float sc[RF_MAX_ROWS];
  const long t = blockIdx.x;
  for (int i = threadIdx.x; i < W; i += RF_THREADS) xs[i] = ldf(h + t * W + i);
  __syncthreads();
  const int wave = threadIdx.x / WAVE, lane = threadIdx.x % WAVE;
  const int W4 = (W % 4 == 0) ? W : 0;           // 16 B pieces when rows stay aligned
  for (int e = wave; e < rows; e += RF_THREADS / WAVE) {
    const float* row = wr + (long)e * W;
    float a0 = 0.f, a1 = 0.f, a2 = 0.f, a3 = 0.f;
#pragma unroll 4
    for (int d = lane * 4; d < W4; d += WAVE * 4) {
      const float4v w = *reinterpret_cast<const float4v*>(row + d);
      const float4v x = *reinterpret_cast<const float4v*>(xs + d);
      a0 += w[0] * x[0]; a1 += w[1] * x[1]; a2 += w[2] * x[2]; a3 += w[3] * x[3];
    }
    for (int d = W4 + lane; d < W; d += WAVE) a0 += row[d] * xs[d];
    float a = wave_reduce_sum((a0 + a1) + (a2 + a3));
    if (lane == 0) {
      if (bias != nullptr) a += bias[e];
      if (e < E) sc[e] = score == 0 ? sigmoidf_(a) : a;
      else extra[t * (rows - E) + (e - E)] = a;
    }
  }
  __syncthreads();
  if (threadIdx.x != 0) return;
  unsigned long long allowed = ~0ull;
  const int per = E / groups;
  if (groups > 1) {
    float gsc[RT_MAX_GROUPS];
    for (int g = 0; g < groups; ++g) {
      float a = -1.f, b = -1.f;
      for (int i = 0; i < per; ++i) {
        const float s = sc[g * per + i];
        if (s > a) { b = a; a = s; }
        else if (s > b) b = s;
      }
      gsc[g] = a + (per > 1 ? b : 0.f);
    }
    allowed = 0ull;
    for (int n = 0; n < keep; ++n) {
      int best = -1;
      float bv = -INFINITY;
      for (int g = 0; g < groups; ++g)
        if (!((allowed >> g) & 1ull) && gsc[g] > bv) { bv = gsc[g]; best = g; }
      if (best >= 0) allowed |= 1ull << best;
    }
  }
  float cs[RT_MAX_TOP];
  int chosen[RT_MAX_TOP];
  float sum = 0.f;
  for (int n = 0; n < top; ++n) {
    int best = -1;
    float bv = -INFINITY;
    for (int e = 0; e < E; ++e) {
      if (groups > 1 && !((allowed >> (e / per)) & 1ull)) continue;
      const float s = sc[e];
      if (s > bv) { bv = s; best = e; }
    }
    chosen[n] = best < 0 ? 0 : best;
    cs[n] = best < 0 ? 0.f : bv;
    if (best >= 0) sc[best] = -INFINITY;          // taken
    sum += cs[n];
  }
  if (score == 2) {                               // softmax over all experts; cs[0] is the largest logit
    const float top0 = cs[0];
    sum = 0.f;
    for (int n = 0; n < top; ++n) sum += expf(cs[n] - top0);
    for (int e = 0; e < E; ++e)                   // the chosen entries of sc were overwritten with -inf
      if (sc[e] != -INFINITY) sum += expf(sc[e] - top0);
    for (int n = 0; n < top; ++n) {
      ids[t * top + n] = chosen[n];
      wts[t * top + n] = expf(cs[n] - top0) / sum;
    }
    return;
  }
  if (score != 0) {                               // softmax over the chosen logits; cs[0] is the largest
    sum = 0.f;
    const float top0 = cs[0];
    for (int n = 0; n < top; ++n) {
      cs[n] = expf(cs[n] - top0);
      sum += cs[n];
    }
    for (int n = 0; n < top; ++n) {
      ids[t * top + n] = chosen[n];
      wts[t * top + n] = cs[n] / sum;
    }
    return;
  }
  for (int n = 0; n < top; ++n) {
    ids[t * top + n] = chosen[n];
    wts[t * top + n] = cs[n] / (sum + 1e-20f) * scale;
  }
}

std::vector<torch::Tensor> moe_router(torch::Tensor h, torch::Tensor wr, torch::Tensor bias, int64_t E, int64_t top,
                                      int64_t groups, int64_t keep, double scale, int64_t score) {
  TORCH_CHECK(h.is_cuda() && h.dim() == 2 && h.is_contiguous());
  check_f32(wr, "router weight");
  const bool has_bias = bias.numel() > 0;
  if (has_bias) {
    check_f32(bias, "router bias");
    TORCH_CHECK(bias.numel() == wr.size(0), "one bias per router row");
  }
  TORCH_CHECK(score == 0 || ((score == 1 || score == 2) && groups == 1),
              "score: 0 sigmoid (groups allowed), 1 softmax over the chosen, 2 softmax over all experts");
  const int T_ = h.size(0), W = h.size(1), rows = wr.size(0);
  TORCH_CHECK(wr.dim() == 2 && wr.size(1) == W && E >= 1 && E <= rows && rows <= RF_MAX_ROWS);
  TORCH_CHECK(top >= 1 && top <= RT_MAX_TOP && top <= E, "experts chosen per token");
  TORCH_CHECK(groups >= 1 && groups <= RT_MAX_GROUPS && E % groups == 0 && keep >= 1 && keep <= groups);
  TORCH_CHECK(groups == 1 || keep * (E / groups) >= top, "the kept groups hold fewer experts than are chosen");
  TORCH_CHECK((size_t)W * sizeof(float) <= 60 * 1024, "row too wide for the router kernel");
  auto ids = torch::empty({T_, top}, h.options().dtype(at::kInt));
  auto wts = torch::empty({T_, top}, h.options().dtype(at::kFloat));
  auto extra = torch::empty({T_, rows - E}, h.options().dtype(at::kFloat));
  if (T_ == 0) return {ids, wts, extra};
  auto stream = at::cuda::getCurrentHIPStream();
  RAGGED_DISPATCH(h, hipLaunchKernelGGL((moe_router_kernel<T>), dim3(T_), dim3(RF_THREADS), (size_t)W * sizeof(float), stream,
      (const T*)h.data_ptr(), wr.data_ptr<float>(), has_bias ? bias.data_ptr<float>() : nullptr, W, rows, (int)E,
      (int)top, (int)groups, (int)keep, (float)scale, (int)score, ids.data_ptr<int>(), wts.data_ptr<float>(),
      extra.data_ptr<float>()));
  return {ids, wts, extra};
}

template <typename T>
__device__ __forceinline__ void load8_(const T* p, float* v);
template <>
__device__ __forceinline__ void load8_<bf16>(const bf16* p, float* v) {
  const short8 x = *reinterpret_cast<const short8*>(p);
#pragma unroll
  for (int i = 0; i < 8; ++i) v[i] = sbf2f(x[i]);
}
template <>
__device__ __forceinline__ void load8_<float>(const float* p, float* v) {
  const float4v a = *reinterpret_cast<const float4v*>(p), b = *reinterpret_cast<const float4v*>(p + 4);
#pragma unroll
  for (int i = 0; i < 4; ++i) { v[i] = a[i]; v[4 + i] = b[i]; }
}

template <typename T>
__device__ __forceinline__ void store8_(T* p, const float* v);
template <>
__device__ __forceinline__ void store8_<bf16>(bf16* p, const float* v) {
  short8 x;
#pragma unroll
  for (int i = 0; i < 8; ++i) x[i] = f2sbf(v[i]);
  *reinterpret_cast<short8*>(p) = x;
}
template <>
__device__ __forceinline__ void store8_<float>(float* p, const float* v) {
  float4v* q = reinterpret_cast<float4v*>(p);
  q[0] = float4v{v[0], v[1], v[2], v[3]};
  q[1] = float4v{v[4], v[5], v[6], v[7]};
}

// ---------------------------------------------------------------------------
// kind 0: y = g sigmoid(alpha g) (u + 1),  g = min(gate, limit), u = clamp(up, -limit, limit)
// kind 1: y = gate sigmoid(gate) up
// kind 2: y = gelu_tanh(gate) up,  gelu_tanh(z) = 0.5 z (1 + tanh(sqrt(2/pi) (z + 0.044715 z^3)))
// ---------------------------------------------------------------------------
__device__ __forceinline__ float glu_value_(float g, float u, float limit, float alpha, int kind) {
  if (kind == 0) {
    g = fminf(g, limit);
    u = fminf(fmaxf(u, -limit), limit);
    return g * sigmoidf_(alpha * g) * (u + 1.f);
  }
  if (kind == 1) return g * sigmoidf_(g) * u;
  return 0.5f * g * (1.f + tanhf(0.7978845608028654f * (g + 0.044715f * g * g * g))) * u;
}

// VEC: F and the row stride are multiples of 8 and the rows 16-byte aligned: 8 elements a thread and turn
template <typename T, bool VEC>
__global__ void clamped_glu_kernel(const T* __restrict__ gu, long stride, T* __restrict__ y, long N, int F,
                                   float limit, float alpha, int kind) {
  if (VEC) {
    const int F8 = F / 8;
    const long total = N * F8;
    for (long i = blockIdx.x * (long)blockDim.x + threadIdx.x; i < total; i += (long)gridDim.x * blockDim.x) {
      const long n = i / F8;
      const int f = (int)(i % F8) * 8;
      float g[8], u[8];
      load8_<T>(gu + n * stride + f, g);
      load8_<T>(gu + n * stride + F + f, u);
#pragma unroll
      for (int k = 0; k < 8; ++k) g[k] = glu_value_(g[k], u[k], limit, alpha, kind);
      store8_<T>(y + n * F + f, g);
    }
    return;
  }
  const long total = N * F;
  for (long i = blockIdx.x * (long)blockDim.x + threadIdx.x; i < total; i += (long)gridDim.x * blockDim.x) {
    const long n = i / F;
    const int f = (int)(i % F);
    stf(y + i, glu_value_(ldf(gu + n * stride + f), ldf(gu + n * stride + F + f), limit, alpha, kind));
  }
}

torch::Tensor clamped_glu(torch::Tensor gu, double limit, double alpha, int64_t kind) {
  TORCH_CHECK(kind >= 0 && kind <= 2, "GLU kind: 0 clamped, 1 SiLU, 2 tanh-GELU");
  TORCH_CHECK(gu.is_cuda() && gu.dim() == 2 && gu.stride(1) == 1 && gu.size(1) % 2 == 0);
  const long N = gu.size(0);
  const int F = gu.size(1) / 2;
  auto y = torch::empty({N, F}, gu.options());
  if (N == 0) return y;
  auto stream = at::cuda::getCurrentHIPStream();
  const bool vec = F % 8 == 0 && gu.stride(0) % 8 == 0 &&
                   reinterpret_cast<uintptr_t>(gu.data_ptr()) % 16 == 0;
#define GLU_LAUNCH(VEC, COUNT)                                                                                   \
  RAGGED_DISPATCH(gu, hipLaunchKernelGGL((clamped_glu_kernel<T, VEC>), dim3(grid_for(COUNT, 256)), dim3(256), 0, \
      stream, (const T*)gu.data_ptr(), (long)gu.stride(0), (T*)y.data_ptr(), N, F, (float)limit, (float)alpha,   \
      (int)kind))
  if (vec) GLU_LAUNCH(true, N * (F / 8));
  else GLU_LAUNCH(false, N * F);
#undef GLU_LAUNCH
  return y;
}

// ---------------------------------------------------------------------------
// y[t] = sum_k w[t,k] down[inv[t,k]] + sigmoid(gate[t]) shared[t] + add[t]   (fp32)
// ---------------------------------------------------------------------------
// VEC: 8 elements per thread and pass with 16/32-byte accesses (W a multiple of 8), else one
template <typename T, bool VEC>
__global__ __launch_bounds__(256) void moe_combine_kernel(
    const T* __restrict__ down, const int* __restrict__ inv, const float* __restrict__ wts,
    const T* __restrict__ shared, const float* __restrict__ gate, const T* __restrict__ add,
    float* __restrict__ y, int W, int K) {
  const long t = blockIdx.x;
  const float sg = shared != nullptr ? sigmoidf_(gate[t]) : 0.f;
  if (VEC) {
    for (int c = threadIdx.x * 8; c < W; c += 256 * 8) {
      float a[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f}, v[8];
      for (int k = 0; k < K; ++k) {
        const float w = wts[t * K + k];
        load8_<T>(down + (long)inv[t * K + k] * W + c, v);
#pragma unroll
        for (int i = 0; i < 8; ++i) a[i] += w * v[i];
      }
      if (shared != nullptr) {
        load8_<T>(shared + t * W + c, v);
#pragma unroll
        for (int i = 0; i < 8; ++i) a[i] += sg * v[i];
      }
      if (add != nullptr) {
        load8_<T>(add + t * W + c, v);
#pragma unroll
        for (int i = 0; i < 8; ++i) a[i] += v[i];
      }
      float4v* yp = reinterpret_cast<float4v*>(y + t * W + c);
      yp[0] = float4v{a[0], a[1], a[2], a[3]};
      yp[1] = float4v{a[4], a[5], a[6], a[7]};
    }
    return;
  }
  for (int c = threadIdx.x; c < W; c += 256) {
    float a = 0.f;
    for (int k = 0; k < K; ++k) a += wts[t * K + k] * ldf(down + (long)inv[t * K + k] * W + c);
    if (shared != nullptr) a += sg * ldf(shared + t * W + c);
    if (add != nullptr) a += ldf(add + t * W + c);
    y[t * W + c] = a;
  }
}

torch::Tensor moe_combine(torch::Tensor down, torch::Tensor inv, torch::Tensor wts, torch::Tensor shared,
                          torch::Tensor gate, torch::Tensor add) {
  TORCH_CHECK(down.is_cuda() && down.dim() == 2 && down.is_contiguous());
  check_i32(inv, "inv"); check_f32(wts, "weights");
  TORCH_CHECK(wts.dim() == 2 && inv.sizes() == wts.sizes());
  const int T_ = wts.size(0), K = wts.size(1), W = down.size(1);
  TORCH_CHECK(down.size(0) == (long)T_ * K);
  const bool has_s = shared.numel() > 0, has_a = add.numel() > 0;
  if (has_s) {
    TORCH_CHECK(shared.is_contiguous() && shared.scalar_type() == down.scalar_type() && shared.size(0) == T_ &&
                shared.size(1) == W);
    check_f32(gate, "shared gate");
    TORCH_CHECK(gate.numel() == T_);
  }
  if (has_a) TORCH_CHECK(add.is_contiguous() && add.scalar_type() == down.scalar_type() && add.size(0) == T_ && add.size(1) == W);
  auto y = torch::empty({T_, W}, down.options().dtype(at::kFloat));
  if (T_ == 0) return y;
  auto stream = at::cuda::getCurrentHIPStream();
#define MC_LAUNCH(VEC)                                                                                          \
  hipLaunchKernelGGL((moe_combine_kernel<T, VEC>), dim3(T_), dim3(256), 0, stream, (const T*)down.data_ptr(),    \
      inv.data_ptr<int>(), wts.data_ptr<float>(), has_s ? (const T*)shared.data_ptr() : (const T*)nullptr,       \
      has_s ? gate.data_ptr<float>() : (const float*)nullptr, has_a ? (const T*)add.data_ptr() : (const T*)nullptr, \
      y.data_ptr<float>(), W, K)
  RAGGED_DISPATCH(down, {
    if (W % 8 == 0) MC_LAUNCH(true);
    else MC_LAUNCH(false);
  });
#undef MC_LAUNCH
  return y;
}
