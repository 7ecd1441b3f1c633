// Rotation of q and k heads by position (entry pairs (2i, 2i+1) or (i, i + n)), an optional
// unit norm AFTER the rotation, and the paged store of [k | v]; q goes to a dense buffer.
#include "../ragged/ragged_common.h"

// ---------------------------------------------------------------------------
// proj [T, QH*D | KH*D | VW | ...] (row stride given; later columns are not read)
// -> q_out [T, QH*D], cache row [KH*D | VW].
// Every head: entries of pair i < nrot rotated by pos * freqs[i] (float64 product, fp32 sine and cosine); layout 0 pairs
// (2i, 2i+1), layout 1 pairs (i, i + nrot); with unit: x / sqrt(mean(x^2) + eps).
// Workgroup = token; its four waves take the QH + KH heads in turn and keep the
// rotated head in LDS as fp32 between the two passes.
// ---------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void rope_norm_store_kernel(
    const T* __restrict__ proj, long stride, int QH, int KH, int D, int VW, const double* __restrict__ freqs,
    int nrot, int layout, int unit, float eps, T* __restrict__ q_out, T* __restrict__ pool,
    const int* __restrict__ tok_pos, const long* __restrict__ tok_row) {
  extern __shared__ float heads_lds[];           // [4][D]
  const long t = blockIdx.x;
  const T* x = proj + t * stride;
  const int wave = threadIdx.x / WAVE, lane = threadIdx.x % WAVE;
  const double pos = (double)tok_pos[t];
  T* row = pool + tok_row[t] * (long)(KH * D + VW);
  float* buf = heads_lds + wave * D;
  for (int u0 = 0; u0 < QH + KH; u0 += 256 / WAVE) {          // the same trip count for every wave
    const int u = u0 + wave;
    const bool on = u < QH + KH;
    const T* src = x + (long)(on ? u : 0) * D;   // q heads, then k heads, lie one after the other
    float ss = 0.f;
    if (on) {
      for (int i = lane; i < nrot; i += WAVE) {
        const int ia = layout == 0 ? 2 * i : i, ib = layout == 0 ? 2 * i + 1 : i + nrot;
        const float a = ldf(src + ia), b = ldf(src + ib);
        float sn, cs;
        // the angle in float64, reduced to [-pi, pi] before it is rounded: far positions keep their precision
        double turns = pos * freqs[i] * 0.15915494309189535;      // angle / 2 pi
        turns -= rint(turns);
        sincosf((float)(turns * 6.283185307179586), &sn, &cs);
        const float ra = a * cs - b * sn, rb = b * cs + a * sn;
        buf[ia] = ra;
        buf[ib] = rb;
        ss += ra * ra + rb * rb;
      }
      for (int d = 2 * nrot + lane; d < D; d += WAVE) {
        const float v = ldf(src + d);
        buf[d] = v;
        ss += v * v;
      }
    }
    const float r = unit ? 1.f / sqrtf(wave_reduce_sum(ss) / (float)D + eps) : 1.f;
    __syncthreads();
    if (on) {
      T* dst = u < QH ? q_out + (t * QH + u) * D : row + (long)(u - QH) * D;
      for (int d = lane; d < D; d += WAVE) stf(dst + d, buf[d] * r);
    }
    __syncthreads();
  }
  const T* vs = x + (long)(QH + KH) * D;
  T* vd = row + (long)KH * D;
  for (int c = threadIdx.x; c < VW; c += 256) vd[c] = vs[c];
}

torch::Tensor rope_norm_store(torch::Tensor proj, int64_t QH, int64_t KH, int64_t D, int64_t VW, torch::Tensor freqs,
                              int64_t layout, bool unit, double eps, torch::Tensor pool, torch::Tensor tok_pos,
                              torch::Tensor tok_row) {
  TORCH_CHECK(proj.is_cuda() && proj.dim() == 2 && proj.stride(1) == 1);
  check_i32(tok_pos, "tok_pos");
  TORCH_CHECK(tok_row.is_cuda() && tok_row.scalar_type() == at::kLong && tok_row.is_contiguous());
  const int T_ = proj.size(0);
  TORCH_CHECK(QH >= 1 && KH >= 1 && D >= 1 && VW >= 1 && proj.size(1) >= (QH + KH) * D + VW, "fused projection width");
  TORCH_CHECK(tok_row.numel() == T_ && tok_pos.numel() == T_);
  TORCH_CHECK(layout == 0 || layout == 1, "layout: 0 neighbouring pairs, 1 halves");
  const int nrot = freqs.numel();
  if (nrot > 0)
    TORCH_CHECK(freqs.is_cuda() && freqs.scalar_type() == at::kDouble && freqs.is_contiguous(), "freqs: float64 device tensor");
  TORCH_CHECK(2 * nrot <= D, "rotated entries lie inside a head");
  TORCH_CHECK(pool.is_contiguous() && pool.dim() == 2 && pool.size(1) == KH * D + VW &&
              pool.scalar_type() == proj.scalar_type());
  TORCH_CHECK((size_t)4 * D * sizeof(float) <= 60 * 1024, "head too wide for the rotation kernel");
  auto q = torch::empty({T_, QH * D}, proj.options());
  if (T_ == 0) return q;
  auto stream = at::cuda::getCurrentHIPStream();
  RAGGED_DISPATCH(proj, hipLaunchKernelGGL((rope_norm_store_kernel<T>), dim3(T_), dim3(256),
      (size_t)4 * D * sizeof(float), stream, (const T*)proj.data_ptr(), (long)proj.stride(0), (int)QH, (int)KH,
      (int)D, (int)VW, nrot > 0 ? freqs.data_ptr<double>() : nullptr, nrot, (int)layout, unit ? 1 : 0, (float)eps,
      (T*)q.data_ptr(), (T*)pool.data_ptr(), tok_pos.data_ptr<int>(), tok_row.data_ptr<long>()));
  return q;
}
