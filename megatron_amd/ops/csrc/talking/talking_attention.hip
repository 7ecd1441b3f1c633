// Chunked talking-heads attention on a paged cache of rows
// [kv_heads * dim keys | kv_heads * vdim values]: per-head q/k norm with
// pairwise rotation, value mixing and cache store; the attention itself in
// fp32 arithmetic for any storage type; the head mixing after the softmax.
#include "../ragged/ragged_common.h"

// ---------------------------------------------------------------------------
// proj [T, H*D | G*D | G*V] -> q_out [T, H*D], cache row [k | v].
// Every q head and k head: x / sqrt(mean(x^2) + eps) * w (w [D], shared by the
// heads), then entries (2i, 2i+1), i < nrot, rotated by pos * freqs[i].
// v <- (1 - lam) v + lam v_first when v_first is given.
// Workgroup = token; its four waves take the H + G heads in turn, a lane a pair.
// ---------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void head_norm_rope_store_kernel(
    const T* __restrict__ proj, long stride, int H, int G, int D, int V, const float* __restrict__ wq,
    const float* __restrict__ wk, float eps, const float* __restrict__ freqs, int nrot,
    const T* __restrict__ v_first, long vf_stride, const float* __restrict__ lam, T* __restrict__ q_out,
    T* __restrict__ pool, const int* __restrict__ tok_pos, const long* __restrict__ tok_row) {
  const long t = blockIdx.x;
  const T* x = proj + t * stride;
  const int wave = threadIdx.x / WAVE, lane = threadIdx.x % WAVE;
  const float pos = (float)tok_pos[t];
  T* row = pool + tok_row[t] * (long)(G * (D + V));
  const int pairs = D / 2;
  for (int u = wave; u < H + G; u += 256 / WAVE) {
    const bool is_q = u < H;
    const T* src = x + (long)u * D;              // q heads, then k heads, lie one after the other
    T* dst = is_q ? q_out + (t * H + u) * D : row + (long)(u - H) * D;
    const float* w = is_q ? wq : wk;
    float ss = 0.f;
    for (int d = lane; d < D; d += WAVE) {
      const float v = ldf(src + d);
      ss += v * v;
    }
    const float r = 1.f / sqrtf(wave_reduce_sum(ss) / (float)D + eps);
    for (int i = lane; i < pairs; i += WAVE) {
      float a = ldf(src + 2 * i) * r * w[2 * i], b = ldf(src + 2 * i + 1) * r * w[2 * i + 1];
      if (i < nrot) {
        float sn, cs;
        sincosf(pos * freqs[i], &sn, &cs);
        const float ra = a * cs - b * sn, rb = b * cs + a * sn;
        a = ra;
        b = rb;
      }
      stf(dst + 2 * i, a);
      stf(dst + 2 * i + 1, b);
    }
    if ((D & 1) && lane == 0) stf(dst + D - 1, ldf(src + D - 1) * r * w[D - 1]);
  }
  const T* vs = x + (long)(H + G) * D;
  T* vd = row + (long)G * D;
  if (v_first != nullptr) {
    const float lm = lam[0];
    const T* vf = v_first + t * vf_stride;
    for (int c = threadIdx.x; c < G * V; c += 256) stf(vd + c, (1.f - lm) * ldf(vs + c) + lm * ldf(vf + c));
  } else {
    for (int c = threadIdx.x; c < G * V; c += 256) vd[c] = vs[c];
  }
}

torch::Tensor head_norm_rope_store(torch::Tensor proj, int64_t H, int64_t G, int64_t D, int64_t V, torch::Tensor wq,
                                   torch::Tensor wk, double eps, torch::Tensor freqs, torch::Tensor v_first,
                                   torch::Tensor lam, torch::Tensor pool, torch::Tensor tok_pos,
                                   torch::Tensor tok_row) {
  TORCH_CHECK(proj.is_cuda() && proj.dim() == 2 && proj.stride(1) == 1);
  check_f32(wq, "q norm"); check_f32(wk, "k norm"); check_i32(tok_pos, "tok_pos");
  TORCH_CHECK(tok_row.is_cuda() && tok_row.scalar_type() == at::kLong && tok_row.is_contiguous());
  const int T_ = proj.size(0);
  TORCH_CHECK(H >= 1 && G >= 1 && D >= 1 && V >= 1 && proj.size(1) == (H + G) * D + G * V, "fused projection width");
  TORCH_CHECK(wq.numel() == D && wk.numel() == D && tok_row.numel() == T_ && tok_pos.numel() == T_);
  const int nrot = freqs.numel();
  if (nrot > 0) check_f32(freqs, "freqs");
  TORCH_CHECK(2 * nrot <= D, "rotated entries lie inside a head");
  TORCH_CHECK(pool.is_contiguous() && pool.dim() == 2 && pool.size(1) == G * (D + V) &&
              pool.scalar_type() == proj.scalar_type());
  const bool mix = v_first.numel() > 0;
  if (mix) {
    TORCH_CHECK(v_first.is_cuda() && v_first.dim() == 2 && v_first.stride(1) == 1 && v_first.size(0) == T_ &&
                v_first.size(1) == G * V && v_first.scalar_type() == proj.scalar_type(), "first values [T, G*V]");
    check_f32(lam, "lam");
    TORCH_CHECK(lam.numel() == 1);
  }
  auto q = torch::empty({T_, H * D}, proj.options());
  if (T_ == 0) return q;
  auto stream = at::cuda::getCurrentHIPStream();
  RAGGED_DISPATCH(proj, hipLaunchKernelGGL((head_norm_rope_store_kernel<T>), dim3(T_), dim3(256), 0, stream,
      (const T*)proj.data_ptr(), (long)proj.stride(0), (int)H, (int)G, (int)D, (int)V, wq.data_ptr<float>(),
      wk.data_ptr<float>(), (float)eps, nrot > 0 ? freqs.data_ptr<float>() : nullptr, nrot,
      mix ? (const T*)v_first.data_ptr() : nullptr, mix ? (long)v_first.stride(0) : 0L,
      mix ? lam.data_ptr<float>() : nullptr, (T*)q.data_ptr(), (T*)pool.data_ptr(), tok_pos.data_ptr<int>(),
      tok_row.data_ptr<long>()));
  return q;
}

// ---------------------------------------------------------------------------
// attention, any storage type.  Workgroup = (token, query head g, value head c),
// 4 waves.  The keys of positions chunk_start(p) .. p: a wave scores one row at
// a time (lanes split the head dim, shuffle-reduce the dot product), keeps an
// online softmax and the weighted sum of value head c in registers; the waves'
// partial results merge through LDS.  A[t, g, c, :] fp32.
// ---------------------------------------------------------------------------
template <typename T, int MAXI>
__global__ __launch_bounds__(256) void talking_attn_kernel(
    const T* __restrict__ q, const T* __restrict__ pool, float scale, const float* __restrict__ temp, int chunk,
    const int* __restrict__ tok_req, const int* __restrict__ tok_pos, const int* __restrict__ tables, int maxb,
    int bs, float* __restrict__ A, int H, int G, int D, int V) {
  __shared__ float s_m[4], s_l[4];
  __shared__ float s_acc[4][MAXI * WAVE];
  const int t = blockIdx.x, hd = blockIdx.y, vh = blockIdx.z;
  const int g = hd / (H / G);
  const int wave = threadIdx.x / WAVE, lane = threadIdx.x % WAVE;
  const int width = G * (D + V);
  float qv[MAXI], acc[MAXI];
  const T* qp = q + ((long)t * H + hd) * D;
#pragma unroll
  for (int i = 0; i < MAXI; ++i) {
    const int d = lane + WAVE * i;
    qv[i] = (d < D) ? ldf(qp + d) : 0.f;
    acc[i] = 0.f;
  }
  const int p = tok_pos[t];
  const int lo = chunk > 0 ? (p / chunk) * chunk : 0;
  const float sc = scale * temp[hd];
  const int* tab = tables + (long)tok_req[t] * maxb;
  float m = -INFINITY, l = 0.f;
  for (int j = lo + wave; j <= p; j += 4) {
    const T* row = pool + ((long)tab[j / bs] * bs + (j % bs)) * width;
    const T* kr = row + g * D;
    const T* vr = row + G * D + vh * V;
    float dot = 0.f;
#pragma unroll
    for (int i = 0; i < MAXI; ++i) {
      const int d = lane + WAVE * i;
      if (d < D) dot += ldf(kr + d) * qv[i];
    }
    dot = wave_reduce_sum(dot) * sc;
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
  float M = -INFINITY;
#pragma unroll
  for (int w = 0; w < 4; ++w) M = fmaxf(M, s_m[w]);
  float L = 0.f;
  float f[4];
#pragma unroll
  for (int w = 0; w < 4; ++w) {
    f[w] = (s_m[w] == -INFINITY) ? 0.f : expf(s_m[w] - M);
    L += s_l[w] * f[w];
  }
  float* op = A + (((long)t * H + hd) * G + vh) * V;
  for (int d = threadIdx.x; d < V; d += 256) {
    float a = 0.f;
#pragma unroll
    for (int w = 0; w < 4; ++w) a += s_acc[w][d] * f[w];
    op[d] = a / L;
  }
}

// ---------------------------------------------------------------------------
// out[t, h, :] = sum_g talk[h, g] A[t, g, kv(h), :]   (A fp32 [T, H, G, V])
// Workgroup = token; the mixing matrix sits in LDS.
// ---------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void talk_mix_kernel(const float* __restrict__ A, const float* __restrict__ talk,
                                                       T* __restrict__ out, int H, int G, int V) {
  extern __shared__ float s_talk[];              // [H][H]
  for (int i = threadIdx.x; i < H * H; i += 256) s_talk[i] = talk[i];
  __syncthreads();
  const long t = blockIdx.x;
  const int rep = H / G;
  const float* At = A + t * H * G * V;
  if (V % 4 == 0) {                              // 16 B reads of A
    const int V4 = V / 4;
    for (int i = threadIdx.x; i < H * V4; i += 256) {
      const int h = i / V4, d = (i % V4) * 4, c = h / rep;
      float4v a = float4v{0.f, 0.f, 0.f, 0.f};
      for (int g = 0; g < H; ++g)
        a += s_talk[h * H + g] * *reinterpret_cast<const float4v*>(At + ((long)g * G + c) * V + d);
      T* op = out + t * H * V + (long)h * V + d;
#pragma unroll
      for (int k = 0; k < 4; ++k) stf(op + k, a[k]);
    }
    return;
  }
  for (int i = threadIdx.x; i < H * V; i += 256) {
    const int h = i / V, d = i % V, c = h / rep;
    float a = 0.f;
    for (int g = 0; g < H; ++g) a += s_talk[h * H + g] * At[((long)g * G + c) * V + d];
    stf(out + t * H * V + i, a);
  }
}

void talk_mix_launch(const torch::Tensor& A, const torch::Tensor& talk, torch::Tensor& out, int H, int G, int V) {
  const int T_ = out.size(0);
  TORCH_CHECK((size_t)H * H * sizeof(float) <= 60 * 1024, "head-mixing matrix above the LDS staging size");
  auto stream = at::cuda::getCurrentHIPStream();
  RAGGED_DISPATCH(out, hipLaunchKernelGGL((talk_mix_kernel<T>), dim3(T_), dim3(256), (size_t)H * H * sizeof(float),
      stream, A.data_ptr<float>(), talk.data_ptr<float>(), (T*)out.data_ptr(), H, G, V));
}

torch::Tensor talking_attention(torch::Tensor q, torch::Tensor pool, int64_t H, int64_t G, int64_t D, int64_t V,
                                double scale, torch::Tensor temp, torch::Tensor talk, int64_t chunk,
                                torch::Tensor tok_req, torch::Tensor tok_pos, torch::Tensor tables, int64_t bs) {
  TORCH_CHECK(q.is_cuda() && q.dim() == 2 && q.is_contiguous() && q.size(1) == H * D);
  TORCH_CHECK(pool.is_contiguous() && pool.dim() == 2 && pool.scalar_type() == q.scalar_type() &&
              pool.size(1) == G * (D + V));
  check_i32(tok_req, "tok_req"); check_i32(tok_pos, "tok_pos"); check_i32(tables, "tables");
  check_f32(temp, "temp"); check_f32(talk, "talk");
  const int T_ = q.size(0);
  TORCH_CHECK(G >= 1 && H % G == 0 && bs >= 1 && chunk >= 0 && H <= 65535 && G <= 65535);
  TORCH_CHECK(temp.numel() == H && talk.numel() == H * H);
  TORCH_CHECK(pool.size(0) % bs == 0);
  TORCH_CHECK(tok_req.numel() == T_ && tok_pos.numel() == T_ && tables.dim() == 2);
  const int wide = (int)std::max(D, V);
  TORCH_CHECK(wide <= 8 * WAVE, "head dim above ", 8 * WAVE);
  auto out = torch::empty({T_, H * V}, q.options());
  if (T_ == 0) return out;
  auto A = torch::empty({(long)T_ * H * G, V}, q.options().dtype(at::kFloat));
  auto stream = at::cuda::getCurrentHIPStream();
#define TK_LAUNCH(MAXI)                                                                                          \
  RAGGED_DISPATCH(q, hipLaunchKernelGGL((talking_attn_kernel<T, MAXI>), dim3(T_, (unsigned)H, (unsigned)G),      \
      dim3(256), 0, stream, (const T*)q.data_ptr(), (const T*)pool.data_ptr(), (float)scale,                     \
      temp.data_ptr<float>(), (int)chunk, tok_req.data_ptr<int>(), tok_pos.data_ptr<int>(),                      \
      tables.data_ptr<int>(), (int)tables.size(1), (int)bs, A.data_ptr<float>(), (int)H, (int)G, (int)D, (int)V))
  if (wide <= WAVE) TK_LAUNCH(1);
  else if (wide <= 2 * WAVE) TK_LAUNCH(2);
  else if (wide <= 4 * WAVE) TK_LAUNCH(4);
  else TK_LAUNCH(8);
#undef TK_LAUNCH
  talk_mix_launch(A, talk, out, (int)H, (int)G, (int)V);
  return out;
}
