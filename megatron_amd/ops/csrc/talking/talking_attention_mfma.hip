// Chunked talking-heads attention on the matrix cores (bf16 storage).
//
// The head mixing after the softmax is linear in the per-head results:
//   o_h(i) = sum_g talk[h, g] A[g, kv(h)](i),   A[g, c](i) = sum_j P_g(i, j) v_c(j)
// so this kernel computes A for every query head g and EVERY value head c, in
// fp32, and talk_mix_kernel (talking_attention.hip) forms the sums.
//
// The value heads lie side by side in a cache row, so A[g, c0 .. c0+CG-1] is ONE
// product with a value CG * V wide: a workgroup takes as many value heads as its
// accumulators hold (up to 512 columns), and the scores and the softmax are
// computed once per group of CG value heads instead of once per value head.
//
// Rows of the problem are (token, query head) pairs of ONE request and ONE key
// head (the rep = H / G query heads that share it), 64 per workgroup (16 per
// wave), numbered token-major; blockIdx.z = key head * groups + value group picks
// the key columns and the value columns of the cache row that are staged, in
// tiles of 32 positions, as [key | values] in LDS.  A row at position p sees
// positions chunk_start(p) .. p, chunk_start(p) = floor(p / chunk) * chunk
// (0 without chunks); the tiles run from the chunk start of the workgroup's
// FIRST token to its last token and the rest of a tile is masked per row.
//
// Both products run transposed so that a query row is a lane column (lane & 15)
// from the first MFMA to the last and softmax statistics never cross lanes
// except over the four 16-lane groups:
//   S^T[kv][q] = sum_d K[kv][d] Q[q][d]          A = K tile rows (LDS, 16 B reads), B = Q (registers)
//   O^T[d][q] += sum_kv V^T[d][kv] P^T[kv][q]    A = V^T gathered from the LDS tile, B = P^T
// The D fragment of S^T (lane (c, g4): kv = 4 g4 + r of two 16-key sub-tiles) is
// used directly as the B fragment of the second product by numbering that MFMA's
// k slots (g4, j) -> kv = 4 g4 + j (j < 4), 16 + 4 g4 + j - 4 (j >= 4); the A
// fragment gathers V in the same order, so no register relayout is needed.
// Wave w computes S^T and the softmax of row tile w and publishes P^T (bf16, in
// B-fragment order) and its rows' rescale factors in LDS; for the second
// product wave w owns the value tiles n = w, w + 4, ... of ALL four row tiles.
//
// Steps with few rows (decode) split the tile list over gridDim.y; partial
// (O, m, l) go to fp32 scratch and a combine kernel normalises.
#include "../ragged/ragged_common.h"

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

constexpr int TK_KT = 32;     // keys per tile
constexpr int TK_ROWS = 64;   // rows per workgroup
constexpr float TK_NEG = -1e30f;
constexpr int TK_MAX_SPLIT = 64;

template <int NKS, int NT>
__global__ __launch_bounds__(256) void talking_attn_mfma_kernel(
    const bf16* __restrict__ q, const bf16* __restrict__ pool, float scale, const float* __restrict__ temp,
    int chunk, const int* __restrict__ tiles, const int* __restrict__ cu, const int* __restrict__ start_pos,
    const int* __restrict__ tables, int maxb, int bs, float* __restrict__ out, float* __restrict__ part_o,
    float* __restrict__ part_m, float* __restrict__ part_l, int nsplit, int Tn, int H, int G, int D, int V,
    int CG) {
  static_assert(NT % 4 == 0, "value tiles are dealt to four waves");
  constexpr int NTW = NT / 4;                    // value tiles per wave
  constexpr int KW = NKS * 32;                   // staged key columns (zero-padded)
  constexpr int ldk = KW + NT * 16 + 8;          // LDS row stride (bf16), padded against bank conflicts
  extern __shared__ __align__(16) short lds[];   // [TK_KT][ldk] key|value tile | P^T [64][32] | factors [64]
  short* const p_lds = lds + TK_KT * ldk;
  float* const f_lds = reinterpret_cast<float*>(p_lds + TK_ROWS * TK_KT);
  const int req = tiles[2 * blockIdx.x], row0 = tiles[2 * blockIdx.x + 1];
  const int NVG = (G + CG - 1) / CG;              // groups of value heads
  const int kvh = blockIdx.z / NVG, vg = blockIdx.z % NVG, rep = H / G;
  const int vcol0 = vg * CG * V;                  // first value column of the group, among the G * V of a row
  const int VW = min(CG, G - vg * CG) * V;        // its width
  const int t0 = cu[req], n_rows = (cu[req + 1] - t0) * rep, start = start_pos[req];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, c = lane & 15, g4 = lane >> 4;
  const int width = G * (D + V);

  // first product and softmax: wave w owns rows row0 + 16 w + (0..15), one per lane column c
  const int my_row = row0 + wave * 16 + c;
  const bool row_ok = my_row < n_rows;
  const int my_tok = row_ok ? my_row / rep : 0, my_head = kvh * rep + (row_ok ? my_row % rep : 0);
  const int my_p = row_ok ? start + my_tok : -1;                    // the row's position
  const int my_lo = (chunk > 0 && my_p >= 0) ? (my_p / chunk) * chunk : 0;   // first position it sees
  const float my_scale = scale * temp[my_head];
  const int last_row = min(row0 + TK_ROWS, n_rows) - 1;
  const int p_max = start + last_row / rep, p_min = start + row0 / rep;
  const int lo_min = chunk > 0 ? (p_min / chunk) * chunk : 0;
  int rt_pmax[4], rt_lomin[4];                                      // the same per row tile of 16
#pragma unroll
  for (int rt = 0; rt < 4; ++rt) {
    const int first = row0 + rt * 16;
    if (first < n_rows) {
      rt_pmax[rt] = start + (min(first + 16, n_rows) - 1) / rep;
      const int pf = start + first / rep;
      rt_lomin[rt] = chunk > 0 ? (pf / chunk) * chunk : 0;
    } else {
      rt_pmax[rt] = -1; rt_lomin[rt] = 0;
    }
  }

  bf16x8 qb[NKS];
  {
    const bf16* qp = q + ((long)(t0 + my_tok) * H + my_head) * D;
#pragma unroll
    for (int ks = 0; ks < NKS; ++ks) {
      short8 v = short8{0, 0, 0, 0, 0, 0, 0, 0};
      const int d = ks * 32 + 8 * g4;
      if (row_ok && d < D) v = *reinterpret_cast<const short8*>(qp + d);
      qb[ks] = *reinterpret_cast<bf16x8*>(&v);
    }
  }
  f32x4 oacc[NTW][4];
#pragma unroll
  for (int i = 0; i < NTW; ++i)
#pragma unroll
    for (int rt = 0; rt < 4; ++rt) oacc[i][rt] = f32x4{0.f, 0.f, 0.f, 0.f};
  float m = TK_NEG, l = 0.f;

  const int jt0 = lo_min / TK_KT;
  const int ntiles = p_max / TK_KT - jt0 + 1;
  int tile_lo = 0, tile_hi = ntiles;
  if (nsplit > 1) {
    const int per = (ntiles + nsplit - 1) / nsplit;
    tile_lo = blockIdx.y * per;
    tile_hi = min(ntiles, tile_lo + per);
  }
  const int* tab = tables + (long)req * maxb;
  constexpr int cpr = (KW + NT * 16) / 8;         // 16 B chunks per staged row
  constexpr int NSTG = (TK_KT * cpr + 255) / 256;
  short8 stg[NSTG];
  int s_row[NSTG], s_lds[NSTG], s_col[NSTG];      // s_col: column in the cache row, -1: zero fill
#pragma unroll
  for (int k = 0; k < NSTG; ++k) {
    const int i = threadIdx.x + k * 256;
    const int r = i / cpr, d = (i % cpr) * 8;
    s_row[k] = (i < TK_KT * cpr) ? r : -1;
    s_lds[k] = r * ldk + d;
    int col = -1;
    if (d < KW) {
      if (d < D) col = kvh * D + d;
    } else if (d - KW < VW) {
      col = G * D + vcol0 + (d - KW);
    }
    s_col[k] = (i < TK_KT * cpr) ? col : -1;
  }
  // Register-staged tile pipeline: the global loads of tile t+1 are issued right
  // after tile t became visible in LDS and are waited for when they are written
  // to LDS at the top of the next iteration.  Pages that are a multiple of the key
  // tile hold a tile in one piece: one scalar page lookup per tile.
  const bool whole = (bs % TK_KT) == 0;
  long s_off[NSTG];
#pragma unroll
  for (int k = 0; k < NSTG; ++k) s_off[k] = (long)s_row[k] * width + s_col[k];
  auto issue = [&](int tile) {
    const int base = (jt0 + tile) * TK_KT;
    if (whole) {
      const bf16* rows = pool + ((long)tab[base / bs] * bs + (base % bs)) * width;
#pragma unroll
      for (int k = 0; k < NSTG; ++k) {
        short8 v = short8{0, 0, 0, 0, 0, 0, 0, 0};
        if (s_col[k] >= 0 && base + s_row[k] <= p_max) v = *reinterpret_cast<const short8*>(rows + s_off[k]);
        stg[k] = v;
      }
      return;
    }
#pragma unroll
    for (int k = 0; k < NSTG; ++k) {
      short8 v = short8{0, 0, 0, 0, 0, 0, 0, 0};
      if (s_col[k] >= 0) {
        const int e = base + s_row[k];
        if (e <= p_max)
          v = *reinterpret_cast<const short8*>(pool + ((long)tab[e / bs] * bs + (e % bs)) * width + s_col[k]);
      }
      stg[k] = v;
    }
  };
  if (tile_lo < tile_hi) issue(tile_lo);
  for (int tile = tile_lo; tile < tile_hi; ++tile) {
    const int base = (jt0 + tile) * TK_KT;
#pragma unroll
    for (int k = 0; k < NSTG; ++k)
      if (s_row[k] >= 0) *reinterpret_cast<short8*>(lds + s_lds[k]) = stg[k];
    __syncthreads();
    if (tile + 1 < tile_hi) issue(tile + 1);
    bool act[4];                                  // does row tile rt see anything of this key tile
#pragma unroll
    for (int rt = 0; rt < 4; ++rt) act[rt] = base <= rt_pmax[rt] && base + TK_KT - 1 >= rt_lomin[rt];
    if (act[wave]) {                              // wave-uniform
      f32x4 st[2], st2[2];
#pragma unroll
      for (int kvt = 0; kvt < 2; ++kvt) {
        st[kvt] = f32x4{0.f, 0.f, 0.f, 0.f};
        st2[kvt] = f32x4{0.f, 0.f, 0.f, 0.f};
      }
#pragma unroll
      for (int ks = 0; ks < NKS; ++ks) {
#pragma unroll
        for (int kvt = 0; kvt < 2; ++kvt) {
          short8 tmp = *reinterpret_cast<const short8*>(lds + (kvt * 16 + c) * ldk + 8 * g4 + ks * 32);
          if (ks & 1)
            st2[kvt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(*reinterpret_cast<bf16x8*>(&tmp), qb[ks], st2[kvt],
                                                               0, 0, 0);
          else
            st[kvt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(*reinterpret_cast<bf16x8*>(&tmp), qb[ks], st[kvt],
                                                              0, 0, 0);
        }
      }
      st[0] += st2[0];
      st[1] += st2[1];
      float s[8];
      bool ok[8];
      float mx = TK_NEG;
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const int e = base + (i >> 2) * 16 + 4 * g4 + (i & 3);
        ok[i] = e <= my_p && e >= my_lo;
        s[i] = st[i >> 2][i & 3] * my_scale;
        if (ok[i]) mx = fmaxf(mx, s[i]);
      }
      mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
      mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
      const float m_new = fmaxf(m, mx);
      const float corr = __expf(m - m_new);
      m = m_new;
      float psum = 0.f;
      short8 pk;
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const float p = ok[i] ? __expf(s[i] - m_new) : 0.f;
        psum += p;
        pk[i] = f2sbf(p);
      }
      l = l * corr + psum;
      *reinterpret_cast<short8*>(p_lds + (wave * 16 + c) * TK_KT + g4 * 8) = pk;
      if (g4 == 0) f_lds[wave * 16 + c] = corr;
    }
    __syncthreads();
    {
      bf16x8 pb[4];
      float cr[4];
      bool rescale = false;
#pragma unroll
      for (int rt = 0; rt < 4; ++rt) {
        // a row tile that sees nothing of this key tile contributes P = 0 with factor 1
        short8 tmp = *reinterpret_cast<const short8*>(p_lds + (rt * 16 + c) * TK_KT + g4 * 8);
        const float f = f_lds[rt * 16 + c];
        if (!act[rt]) tmp = short8{0, 0, 0, 0, 0, 0, 0, 0};
        cr[rt] = act[rt] ? f : 1.f;
        rescale |= cr[rt] != 1.f;
        pb[rt] = *reinterpret_cast<bf16x8*>(&tmp);
      }
      if (__any(rescale)) {
#pragma unroll
        for (int i = 0; i < NTW; ++i)
#pragma unroll
          for (int rt = 0; rt < 4; ++rt) oacc[i][rt] *= cr[rt];
      }
#pragma unroll
      for (int i = 0; i < NTW; ++i) {
        short8 av;
        const short* vcol = lds + KW + (wave + 4 * i) * 16 + c;
#pragma unroll
        for (int j = 0; j < 8; ++j) av[j] = vcol[((j >> 2) * 16 + 4 * g4 + (j & 3)) * ldk];
        const bf16x8 a = *reinterpret_cast<bf16x8*>(&av);
#pragma unroll
        for (int rt = 0; rt < 4; ++rt)
          oacc[i][rt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, pb[rt], oacc[i][rt], 0, 0, 0);
      }
    }
    __syncthreads();
  }
  l += __shfl_xor(l, 16, 64);
  l += __shfl_xor(l, 32, 64);
  if (nsplit == 1) {
    if (g4 == 0) f_lds[wave * 16 + c] = (row_ok && l > 0.f) ? 1.f / l : 0.f;
    __syncthreads();
#pragma unroll
    for (int rt = 0; rt < 4; ++rt) {
      const int row = row0 + rt * 16 + c;
      if (row < n_rows) {
        const float inv = f_lds[rt * 16 + c];
        float* op = out + ((long)(t0 + row / rep) * H + kvh * rep + row % rep) * G * V + vcol0;
#pragma unroll
        for (int i = 0; i < NTW; ++i) {
          const int d = (wave + 4 * i) * 16 + 4 * g4;
          if (d < VW) *reinterpret_cast<f32x4*>(op + d) = oacc[i][rt] * inv;
        }
      }
    }
  } else {
    const long rows_all = (long)Tn * H;
    if (g4 == 0 && row_ok) {
      const long grow = (long)(t0 + my_tok) * H + my_head;
      part_m[(blockIdx.y * rows_all + grow) * NVG + vg] = m;
      part_l[(blockIdx.y * rows_all + grow) * NVG + vg] = l;
    }
#pragma unroll
    for (int rt = 0; rt < 4; ++rt) {
      const int row = row0 + rt * 16 + c;
      if (row < n_rows) {
        const long grow = (long)(t0 + row / rep) * H + kvh * rep + row % rep;
        float* po = part_o + (blockIdx.y * rows_all + grow) * G * V + vcol0;
#pragma unroll
        for (int i = 0; i < NTW; ++i) {
          const int d = (wave + 4 * i) * 16 + 4 * g4;
          if (d < VW) *reinterpret_cast<f32x4*>(po + d) = oacc[i][rt];
        }
      }
    }
  }
}

// merge of the key splits: one workgroup per (token, query head, value head) row of A;
// rows = tokens * heads, the statistics are kept per (row, group of value heads)
__global__ void talking_combine_kernel(const float* __restrict__ part_o, const float* __restrict__ part_m,
                                       const float* __restrict__ part_l, float* __restrict__ out, int nsplit,
                                       long rows, int G, int V, int CG) {
  __shared__ float s_m[TK_MAX_SPLIT], s_l[TK_MAX_SPLIT];
  const long grow = blockIdx.x / G;
  const int c = blockIdx.x % G, NVG = (G + CG - 1) / CG, vg = c / CG;
  if (threadIdx.x < nsplit) {
    s_m[threadIdx.x] = part_m[(threadIdx.x * rows + grow) * NVG + vg];
    s_l[threadIdx.x] = part_l[(threadIdx.x * rows + grow) * NVG + vg];
  }
  __syncthreads();
  float M = TK_NEG;
  for (int s = 0; s < nsplit; ++s) M = fmaxf(M, s_m[s]);
  float L = 0.f;
  for (int s = 0; s < nsplit; ++s) L += s_l[s] * expf(s_m[s] - M);
  const float inv = L > 0.f ? 1.f / L : 0.f;
  for (int d = threadIdx.x; d < V; d += blockDim.x) {
    float a = 0.f;
#pragma unroll 4
    for (int s = 0; s < nsplit; ++s) a += part_o[((s * rows + grow) * G + c) * V + d] * expf(s_m[s] - M);
    out[(grow * G + c) * V + d] = a * inv;
  }
}

void talk_mix_launch(const torch::Tensor& A, const torch::Tensor& talk, torch::Tensor& out, int H, int G, int V);

torch::Tensor talking_attention_mfma(torch::Tensor q, torch::Tensor pool, int64_t H, int64_t G, int64_t D, int64_t V,
                                     double scale, torch::Tensor temp, torch::Tensor talk, int64_t chunk,
                                     torch::Tensor tiles, torch::Tensor cu, torch::Tensor start_pos,
                                     torch::Tensor tables, int64_t bs, int64_t nsplit) {
  TORCH_CHECK(q.is_cuda() && q.dim() == 2 && q.is_contiguous() && q.scalar_type() == at::kBFloat16 && q.size(1) == H * D);
  TORCH_CHECK(pool.is_contiguous() && pool.dim() == 2 && pool.scalar_type() == at::kBFloat16 && pool.size(1) == G * (D + V));
  check_i32(tiles, "tiles"); check_i32(cu, "cu"); check_i32(start_pos, "start_pos"); check_i32(tables, "tables");
  check_f32(temp, "temp"); check_f32(talk, "talk");
  const int T_ = q.size(0), R = start_pos.numel();
  TORCH_CHECK(G >= 1 && H % G == 0 && bs >= 1 && chunk >= 0 && G * G <= 65535 && (long)T_ * H * G < (1L << 31));
  TORCH_CHECK(temp.numel() == H && talk.numel() == H * H);
  TORCH_CHECK(D % 8 == 0 && V % 8 == 0 && D <= 256 && V <= 256, "MFMA path: head dims multiples of 8, at most 256");
  TORCH_CHECK(pool.size(0) % bs == 0);
  TORCH_CHECK(cu.numel() == R + 1 && tiles.dim() == 2 && tiles.size(1) == 2 && tables.dim() == 2 && tables.size(0) == R);
  TORCH_CHECK(nsplit >= 1 && nsplit <= TK_MAX_SPLIT);
  auto out = torch::empty({T_, H * V}, q.options());
  const int nblk = tiles.size(0);
  if (T_ == 0 || nblk == 0) return out;
  // value heads per workgroup: as many as the widest instantiation for this key size holds
  const int nks = ((int)D + 31) / 32;
  const int wide = nks <= 4 ? 512 : 256;          // measured: 512 columns beat 256 and 128 at 128-wide heads
  int CG = std::max(1, std::min((int)G, wide / (int)V));
  // steps with few rows (decoding) keep one value head a workgroup: more workgroups, shorter ones
  if ((long)nblk * G * ((G + CG - 1) / CG) < 256) CG = 1;
  const int NVG = ((int)G + CG - 1) / CG, nt = (CG * (int)V + 15) / 16;
  auto fo = q.options().dtype(at::kFloat);
  auto A = torch::empty({(long)T_ * H * G, V}, fo);      // every row is written by a workgroup or the combine
  auto stream = at::cuda::getCurrentHIPStream();
  torch::Tensor po, pm, pl;
  float *pop = nullptr, *pmp = nullptr, *plp = nullptr;
  if (nsplit > 1) {
    po = torch::empty({nsplit, (long)T_ * H * G, V}, fo);
    pm = torch::empty({nsplit, (long)T_ * H * NVG}, fo);
    pl = torch::empty({nsplit, (long)T_ * H * NVG}, fo);
    pop = po.data_ptr<float>(); pmp = pm.data_ptr<float>(); plp = pl.data_ptr<float>();
  }
  const dim3 grid(nblk, (unsigned)nsplit, (unsigned)(G * NVG));
#define TK_MFMA(NKS, NT)                                                                                        \
  hipLaunchKernelGGL((talking_attn_mfma_kernel<NKS, NT>), grid, dim3(256),                                      \
      ((size_t)TK_KT * (NKS * 32 + NT * 16 + 8) + TK_ROWS * TK_KT) * sizeof(short) + TK_ROWS * sizeof(float),   \
      stream, (const bf16*)q.data_ptr(), (const bf16*)pool.data_ptr(), (float)scale, temp.data_ptr<float>(),    \
      (int)chunk, tiles.data_ptr<int>(), cu.data_ptr<int>(), start_pos.data_ptr<int>(), tables.data_ptr<int>(), \
      (int)tables.size(1), (int)bs, A.data_ptr<float>(), pop, pmp, plp, (int)nsplit, T_, (int)H, (int)G,        \
      (int)D, (int)V, CG)
  if (nks <= 2 && nt <= 4) TK_MFMA(2, 4);
  else if (nks <= 4 && nt <= 8) TK_MFMA(4, 8);
  else if (nks <= 4) TK_MFMA(4, 32);
  else TK_MFMA(8, 16);
#undef TK_MFMA
  if (nsplit > 1)
    hipLaunchKernelGGL(talking_combine_kernel, dim3((unsigned)((long)T_ * H * G)), dim3(128), 0, stream, pop, pmp,
                       plp, A.data_ptr<float>(), (int)nsplit, (long)T_ * H, (int)G, (int)V, CG);
  talk_mix_launch(A, talk, out, (int)H, (int)G, (int)V);
  return out;
}
