// Causal softmax attention with M softmax maps a head over shared values, on a paged cache of
// rows [G*M*D keys | G*V values], in fp32 arithmetic for any storage type.
// q row (t, h, m) reads key head (h / rep) * M + m and value head h / rep (rep = H / G).
// s = q . k * scale;  cap > 0: s <- cap * tanh(s / cap).
#include "../ragged/ragged_common.h"

// ---------------------------------------------------------------------------
// Workgroup = (token, query row h * M + m), 4 waves.  A wave scores one cache row at a time
// (lanes split the head dim, shuffle-reduce the dot product), keeps an online softmax and the
// weighted sum of the values in registers; the waves' partial results merge through LDS.
// A[t, h * M + m, :] fp32.
// ---------------------------------------------------------------------------
template <typename T, int MAXI>
__global__ __launch_bounds__(256) void map_attn_kernel(
    const T* __restrict__ q, const T* __restrict__ pool, float scale, float cap,
    const int* __restrict__ tok_req, const int* __restrict__ tok_pos, const int* __restrict__ tables, int maxb,
    int bs, float* __restrict__ A, int H, int G, int M, int D, int V) {
  __shared__ float s_m[4], s_l[4];
  __shared__ float s_acc[4][MAXI * WAVE];
  const int t = blockIdx.x, qh = blockIdx.y;
  const int rep = H / G;
  const int kh = (qh / (rep * M)) * M + qh % M, vh = qh / (rep * M);
  const int wave = threadIdx.x / WAVE, lane = threadIdx.x % WAVE;
  const int kw = G * M * D, width = kw + G * V;
  float qv[MAXI], acc[MAXI];
  const T* qp = q + ((long)t * H * M + qh) * D;
#pragma unroll
  for (int i = 0; i < MAXI; ++i) {
    const int d = lane + WAVE * i;
    qv[i] = (d < D) ? ldf(qp + d) : 0.f;
    acc[i] = 0.f;
  }
  const int p = tok_pos[t];
  const float inv_cap = cap > 0.f ? 1.f / cap : 0.f;
  const int* tab = tables + (long)tok_req[t] * maxb;
  float m = -INFINITY, l = 0.f;
  for (int j = wave; j <= p; j += 4) {
    const T* row = pool + ((long)tab[j / bs] * bs + (j % bs)) * width;
    const T* kr = row + kh * D;
    const T* vr = row + kw + vh * V;
    float dot = 0.f;
#pragma unroll
    for (int i = 0; i < MAXI; ++i) {
      const int d = lane + WAVE * i;
      if (d < D) dot += ldf(kr + d) * qv[i];
    }
    dot = wave_reduce_sum(dot) * scale;
    if (cap > 0.f) dot = cap * tanhf(dot * inv_cap);
    const float mn = fmaxf(m, dot);
    const float corr = expf(m - mn), pj = expf(dot - mn);
    l = l * corr + pj;
#pragma unroll
    for (int i = 0; i < MAXI; ++i) {
      const int d = lane + WAVE * i;
      const float vv = (d < V) ? ldf(vr + d) : 0.f;
      acc[i] = acc[i] * corr + pj * vv;
    }
    m = mn;
  }
  if (lane == 0) {
    s_m[wave] = m;
    s_l[wave] = l;
  }
#pragma unroll
  for (int i = 0; i < MAXI; ++i) s_acc[wave][lane + WAVE * i] = acc[i];
  __syncthreads();
  float Mx = -INFINITY;
#pragma unroll
  for (int w = 0; w < 4; ++w) Mx = fmaxf(Mx, s_m[w]);
  float L = 0.f;
  float f[4];
#pragma unroll
  for (int w = 0; w < 4; ++w) {
    f[w] = (s_m[w] == -INFINITY) ? 0.f : expf(s_m[w] - Mx);
    L += s_l[w] * f[w];
  }
  float* op = A + ((long)t * H * M + qh) * V;
  for (int d = threadIdx.x; d < V; d += 256) {
    float a = 0.f;
#pragma unroll
    for (int w = 0; w < 4; ++w) a += s_acc[w][d] * f[w];
    op[d] = a / L;
  }
}

torch::Tensor map_attention(torch::Tensor q, torch::Tensor pool, int64_t H, int64_t G, int64_t M, int64_t D, int64_t V,
                            double scale, double cap, torch::Tensor tok_req, torch::Tensor tok_pos,
                            torch::Tensor tables, int64_t bs) {
  TORCH_CHECK(q.is_cuda() && q.dim() == 2 && q.is_contiguous() && q.size(1) == H * M * D);
  TORCH_CHECK(pool.is_contiguous() && pool.dim() == 2 && pool.scalar_type() == q.scalar_type() &&
              pool.size(1) == G * (M * D + V));
  check_i32(tok_req, "tok_req"); check_i32(tok_pos, "tok_pos"); check_i32(tables, "tables");
  const int T_ = q.size(0);
  TORCH_CHECK(G >= 1 && M >= 1 && H % G == 0 && bs >= 1 && H * M <= 65535 && cap >= 0.0);
  TORCH_CHECK(pool.size(0) % bs == 0);
  TORCH_CHECK(tok_req.numel() == T_ && tok_pos.numel() == T_ && tables.dim() == 2);
  const int wide = (int)std::max(D, V);
  TORCH_CHECK(wide <= 8 * WAVE, "head dim above ", 8 * WAVE);
  auto A = torch::empty({T_, H * M * V}, q.options().dtype(at::kFloat));
  if (T_ == 0) return A;
  auto stream = at::cuda::getCurrentHIPStream();
#define MA_LAUNCH(MAXI)                                                                                          \
  RAGGED_DISPATCH(q, hipLaunchKernelGGL((map_attn_kernel<T, MAXI>), dim3(T_, (unsigned)(H * M)), dim3(256), 0,   \
      stream, (const T*)q.data_ptr(), (const T*)pool.data_ptr(), (float)scale, (float)cap,                       \
      tok_req.data_ptr<int>(), tok_pos.data_ptr<int>(), tables.data_ptr<int>(), (int)tables.size(1), (int)bs,    \
      A.data_ptr<float>(), (int)H, (int)G, (int)M, (int)D, (int)V))
  if (wide <= WAVE) MA_LAUNCH(1);
  else if (wide <= 2 * WAVE) MA_LAUNCH(2);
  else if (wide <= 4 * WAVE) MA_LAUNCH(4);
  else MA_LAUNCH(8);
#undef MA_LAUNCH
  return A;
}
