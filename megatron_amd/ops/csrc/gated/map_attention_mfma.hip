// Causal softmax attention with M softmax maps a head over shared values, on the matrix cores
// (bf16 storage), over a paged cache of rows [G*M*D keys | G*V values].
//
// Rows of the problem are (token, query head of the group) pairs of ONE request, ONE key/value
// group g and ONE map m, i.e. the rep = H / G query rows (h, m), h in group g, that read key head
// g * M + m and value head g; 64 * RT per workgroup (RT tiles of 16 per wave), numbered token-major
// (RT = 2 for steps with many rows: every staged tile, key fragment and gathered value fragment
// then feeds twice the MFMAs; RT = 1 for steps with few rows).
// blockIdx.z = g * M + m picks the key columns and the value columns of the cache row that are
// staged, in tiles of 32 positions, as [key | value] in LDS.  A row at position p sees 0 .. p; the
// tiles run to the workgroup's last token and the rest of a tile is masked per row.
//
// Both products run transposed so that a query row is a lane column (lane & 15) from the first
// MFMA to the last and softmax statistics never cross lanes except over the four 16-lane groups:
//   S^T[kv][q] = sum_d K[kv][d] Q[q][d]          A = K tile rows (LDS, 16 B reads), B = Q (registers)
//   O^T[d][q] += sum_kv V^T[d][kv] P^T[kv][q]    A = V^T gathered from the LDS tile, B = P^T
// The D fragment of S^T (lane (c, g4): kv = 4 g4 + r of two 16-key sub-tiles) is used directly as
// the B fragment of the second product by numbering that MFMA's k slots (g4, j) -> kv = 4 g4 + j
// (j < 4), 16 + 4 g4 + j - 4 (j >= 4); the A fragment gathers V in the same order.
// Wave w computes S^T, the cap and the softmax of row tiles w RT .. w RT + RT - 1 and publishes P^T
// (bf16, in B-fragment order) and its rows' rescale factors in LDS; for the second product wave w
// owns the value tiles n = w, w + 4, ... of ALL 4 RT row tiles.
//
// Scores: s = q . k * scale; cap > 0: s <- cap * tanh(s / cap), tanh(x) = 1 - 2 / (exp(2x) + 1).
// Result: with a gate (M = 1), out[t, h, :] = o * sigmoid(gate[t, h, :]) in bf16; without, the fp32
// result of every (head, map) row for a finishing kernel.
// Steps with few rows (decode) split the tile list over gridDim.y; partial (O, m, l) go to fp32
// scratch and a combine kernel normalises (and applies the gate).
#include "../ragged/ragged_common.h"

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

constexpr int MA_KT = 32;     // keys per tile
constexpr int MA_ROWS = 64;   // rows per workgroup and row tile of a wave
constexpr float MA_NEG = -1e30f;
constexpr int MA_MAX_SPLIT = 64;

__device__ __forceinline__ float fast_cap(float s, float cap, float two_inv_cap) {
  // cap * tanh(s / cap); exp overflow gives 1 - 0, underflow 1 - 2: both exact limits
  return cap * (1.f - 2.f / (__expf(s * two_inv_cap) + 1.f));
}

template <int NKS, int NT, int RT>
__global__ __launch_bounds__(256) void map_attn_mfma_kernel(
    const bf16* __restrict__ q, const bf16* __restrict__ gate, long gstride, const bf16* __restrict__ pool,
    float scale, float cap, const int* __restrict__ tiles, const int* __restrict__ cu,
    const int* __restrict__ start_pos, const int* __restrict__ tables, int maxb, int bs, float* __restrict__ out,
    bf16* __restrict__ gated, float* __restrict__ part_o, float* __restrict__ part_m, float* __restrict__ part_l,
    int nsplit, int Tn, int H, int G, int M, int D, int V) {
  static_assert(NT % 4 == 0, "value tiles are dealt to four waves");
  constexpr int NTW = NT / 4;                    // value tiles per wave
  constexpr int KW = NKS * 32;                   // staged key columns (zero-padded)
  constexpr int ldk = KW + NT * 16 + 8;          // LDS row stride (bf16), padded against bank conflicts
  constexpr int ROWS = MA_ROWS * RT, NRT = 4 * RT;   // rows and row tiles of the workgroup
  extern __shared__ __align__(16) short lds[];   // [MA_KT][ldk] key|value tile | P^T [ROWS][32] | factors [ROWS]
  short* const p_lds = lds + MA_KT * ldk;
  float* const f_lds = reinterpret_cast<float*>(p_lds + ROWS * MA_KT);
  const int req = tiles[2 * blockIdx.x], row0 = tiles[2 * blockIdx.x + 1];
  const int kz = blockIdx.z, grp = kz / M, mp = kz % M, rep = H / G, HM = H * M;
  const int t0 = cu[req], n_rows = (cu[req + 1] - t0) * rep, start = start_pos[req];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, c = lane & 15, g4 = lane >> 4;
  const int kcols = G * M * D, width = kcols + G * V;

  // first product and softmax: wave w owns rows row0 + 16 (w RT + j) + (0..15), one per lane column c
  int my_tok[RT], my_qh[RT], my_p[RT];
  bool row_ok[RT];
#pragma unroll
  for (int j = 0; j < RT; ++j) {
    const int my_row = row0 + (wave * RT + j) * 16 + c;
    row_ok[j] = my_row < n_rows;
    my_tok[j] = row_ok[j] ? my_row / rep : 0;
    my_qh[j] = (grp * rep + (row_ok[j] ? my_row % rep : 0)) * M + mp;
    my_p[j] = row_ok[j] ? start + my_tok[j] : -1;                   // the row's position
  }
  const float two_inv_cap = cap > 0.f ? 2.f / cap : 0.f;
  const int last_row = min(row0 + ROWS, n_rows) - 1;
  const int p_max = start + last_row / rep;
  int rt_pmax[NRT];                                                 // last position per row tile of 16
#pragma unroll
  for (int rt = 0; rt < NRT; ++rt) {
    const int first = row0 + rt * 16;
    rt_pmax[rt] = first < n_rows ? start + (min(first + 16, n_rows) - 1) / rep : -1;
  }

  bf16x8 qb[RT][NKS];
#pragma unroll
  for (int j = 0; j < RT; ++j) {
    const bf16* qp = q + ((long)(t0 + my_tok[j]) * HM + my_qh[j]) * D;
#pragma unroll
    for (int ks = 0; ks < NKS; ++ks) {
      short8 v = short8{0, 0, 0, 0, 0, 0, 0, 0};
      const int d = ks * 32 + 8 * g4;
      if (row_ok[j] && d < D) v = *reinterpret_cast<const short8*>(qp + d);
      qb[j][ks] = *reinterpret_cast<bf16x8*>(&v);
    }
  }
  f32x4 oacc[NTW][NRT];
#pragma unroll
  for (int i = 0; i < NTW; ++i)
#pragma unroll
    for (int rt = 0; rt < NRT; ++rt) oacc[i][rt] = f32x4{0.f, 0.f, 0.f, 0.f};
  float m[RT], l[RT];
#pragma unroll
  for (int j = 0; j < RT; ++j) { m[j] = MA_NEG; l[j] = 0.f; }

  const int ntiles = p_max / MA_KT + 1;
  int tile_lo = 0, tile_hi = ntiles;
  if (nsplit > 1) {
    const int per = (ntiles + nsplit - 1) / nsplit;
    tile_lo = blockIdx.y * per;
    tile_hi = min(ntiles, tile_lo + per);
  }
  const int* tab = tables + (long)req * maxb;
  constexpr int cpr = (KW + NT * 16) / 8;         // 16 B chunks per staged row
  constexpr int NSTG = (MA_KT * cpr + 255) / 256;
  short8 stg[NSTG];
  int s_row[NSTG], s_lds[NSTG], s_col[NSTG];      // s_col: column in the cache row, -1: zero fill
#pragma unroll
  for (int k = 0; k < NSTG; ++k) {
    const int i = threadIdx.x + k * 256;
    const int r = i / cpr, d = (i % cpr) * 8;
    s_row[k] = (i < MA_KT * cpr) ? r : -1;
    s_lds[k] = r * ldk + d;
    int col = -1;
    if (d < KW) {
      if (d < D) col = kz * D + d;
    } else if (d - KW < V) {
      col = kcols + grp * V + (d - KW);
    }
    s_col[k] = (i < MA_KT * cpr) ? col : -1;
  }
  // Register-staged tile pipeline: the global loads of tile t+1 are issued right after tile t
  // became visible in LDS and are waited for when they are written to LDS at the top of the next
  // iteration.  Pages that are a multiple of the key tile hold a tile in one piece.
  const bool whole = (bs % MA_KT) == 0;
  long s_off[NSTG];
#pragma unroll
  for (int k = 0; k < NSTG; ++k) s_off[k] = (long)s_row[k] * width + s_col[k];
  auto issue = [&](int tile) {
    const int base = tile * MA_KT;
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
    const int base = tile * MA_KT;
#pragma unroll
    for (int k = 0; k < NSTG; ++k)
      if (s_row[k] >= 0) *reinterpret_cast<short8*>(lds + s_lds[k]) = stg[k];
    __syncthreads();
    if (tile + 1 < tile_hi) issue(tile + 1);
    bool act[NRT];                                // does row tile rt see anything of this key tile
#pragma unroll
    for (int rt = 0; rt < NRT; ++rt) act[rt] = base <= rt_pmax[rt];
    bool mine = false;                            // does any row tile of this wave see the key tile (wave-uniform)
#pragma unroll
    for (int j = 0; j < RT; ++j) mine |= act[wave * RT + j];
    if (mine) {
      f32x4 st[RT][2], st2[RT][2];
#pragma unroll
      for (int j = 0; j < RT; ++j)
#pragma unroll
        for (int kvt = 0; kvt < 2; ++kvt) {
          st[j][kvt] = f32x4{0.f, 0.f, 0.f, 0.f};
          st2[j][kvt] = f32x4{0.f, 0.f, 0.f, 0.f};
        }
#pragma unroll
      for (int ks = 0; ks < NKS; ++ks) {
#pragma unroll
        for (int kvt = 0; kvt < 2; ++kvt) {
          short8 tmp = *reinterpret_cast<const short8*>(lds + (kvt * 16 + c) * ldk + 8 * g4 + ks * 32);
          const bf16x8 kf = *reinterpret_cast<bf16x8*>(&tmp);
#pragma unroll
          for (int j = 0; j < RT; ++j) {
            if (!act[wave * RT + j]) continue;
            if (ks & 1) st2[j][kvt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf, qb[j][ks], st2[j][kvt], 0, 0, 0);
            else st[j][kvt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf, qb[j][ks], st[j][kvt], 0, 0, 0);
          }
        }
      }
#pragma unroll
      for (int j = 0; j < RT; ++j) {
        if (!act[wave * RT + j]) continue;
        st[j][0] += st2[j][0];
        st[j][1] += st2[j][1];
        float sc[8];
        bool ok[8];
        float mx = MA_NEG;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          const int e = base + (i >> 2) * 16 + 4 * g4 + (i & 3);
          ok[i] = e <= my_p[j];
          sc[i] = st[j][i >> 2][i & 3] * scale;
          if (cap > 0.f) sc[i] = fast_cap(sc[i], cap, two_inv_cap);
          if (ok[i]) mx = fmaxf(mx, sc[i]);
        }
        mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
        mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
        const float m_new = fmaxf(m[j], mx);
        const float corr = __expf(m[j] - m_new);
        m[j] = m_new;
        float psum = 0.f;
        short8 pk;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          const float p = ok[i] ? __expf(sc[i] - m_new) : 0.f;
          psum += p;
          pk[i] = f2sbf(p);
        }
        l[j] = l[j] * corr + psum;
        const int prow = (wave * RT + j) * 16 + c;
        *reinterpret_cast<short8*>(p_lds + prow * MA_KT + g4 * 8) = pk;
        if (g4 == 0) f_lds[prow] = corr;
      }
    }
    __syncthreads();
    {
      bf16x8 pb[NRT];
      float cr[NRT];
      bool rescale = false;
#pragma unroll
      for (int rt = 0; rt < NRT; ++rt) {
        // a row tile that sees nothing of this key tile contributes P = 0 with factor 1
        short8 tmp = *reinterpret_cast<const short8*>(p_lds + (rt * 16 + c) * MA_KT + g4 * 8);
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
          for (int rt = 0; rt < NRT; ++rt) oacc[i][rt] *= cr[rt];
      }
#pragma unroll
      for (int i = 0; i < NTW; ++i) {
        short8 av;
        const short* vcol = lds + KW + (wave + 4 * i) * 16 + c;
#pragma unroll
        for (int j = 0; j < 8; ++j) av[j] = vcol[((j >> 2) * 16 + 4 * g4 + (j & 3)) * ldk];
        const bf16x8 a = *reinterpret_cast<bf16x8*>(&av);
#pragma unroll
        for (int rt = 0; rt < NRT; ++rt)
          if (act[rt]) oacc[i][rt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, pb[rt], oacc[i][rt], 0, 0, 0);
      }
    }
    __syncthreads();
  }
#pragma unroll
  for (int j = 0; j < RT; ++j) {
    l[j] += __shfl_xor(l[j], 16, 64);
    l[j] += __shfl_xor(l[j], 32, 64);
  }
  if (nsplit == 1) {
#pragma unroll
    for (int j = 0; j < RT; ++j)
      if (g4 == 0) f_lds[(wave * RT + j) * 16 + c] = (row_ok[j] && l[j] > 0.f) ? 1.f / l[j] : 0.f;
    __syncthreads();
#pragma unroll
    for (int rt = 0; rt < NRT; ++rt) {
      const int row = row0 + rt * 16 + c;
      if (row < n_rows) {
        const float inv = f_lds[rt * 16 + c];
        const long grow = (long)(t0 + row / rep) * HM + (grp * rep + row % rep) * M + mp;
#pragma unroll
        for (int i = 0; i < NTW; ++i) {
          const int d = (wave + 4 * i) * 16 + 4 * g4;
          if (d < V) {
            const f32x4 o = oacc[i][rt] * inv;
            if (gated != nullptr) {
              const bf16* gp = gate + (long)(t0 + row / rep) * gstride + (long)(grow % HM) * V + d;
              typedef short short4v __attribute__((ext_vector_type(4)));
              short4v pk;
#pragma unroll
              for (int k = 0; k < 4; ++k) pk[k] = f2sbf(o[k] * sigmoidf_(__bfloat162float(gp[k])));
              *reinterpret_cast<short4v*>(gated + grow * V + d) = pk;
            } else {
              *reinterpret_cast<f32x4*>(out + grow * V + d) = o;
            }
          }
        }
      }
    }
  } else {
    const long rows_all = (long)Tn * HM;
#pragma unroll
    for (int j = 0; j < RT; ++j)
      if (g4 == 0 && row_ok[j]) {
        const long grow = (long)(t0 + my_tok[j]) * HM + my_qh[j];
        part_m[blockIdx.y * rows_all + grow] = m[j];
        part_l[blockIdx.y * rows_all + grow] = l[j];
      }
#pragma unroll
    for (int rt = 0; rt < NRT; ++rt) {
      const int row = row0 + rt * 16 + c;
      if (row < n_rows) {
        const long grow = (long)(t0 + row / rep) * HM + (grp * rep + row % rep) * M + mp;
        float* po = part_o + (blockIdx.y * rows_all + grow) * V;
#pragma unroll
        for (int i = 0; i < NTW; ++i) {
          const int d = (wave + 4 * i) * 16 + 4 * g4;
          if (d < V) *reinterpret_cast<f32x4*>(po + d) = oacc[i][rt];
        }
      }
    }
  }
}

// merge of the key splits: one workgroup per (token, head, map) row; with a gate the row leaves as
// o * sigmoid(gate) in bf16
__global__ void map_combine_kernel(const float* __restrict__ part_o, const float* __restrict__ part_m,
                                   const float* __restrict__ part_l, float* __restrict__ out,
                                   bf16* __restrict__ gated, const bf16* __restrict__ gate, long gstride,
                                   int nsplit, long rows, int HM, int V) {
  __shared__ float s_m[MA_MAX_SPLIT], s_l[MA_MAX_SPLIT];
  const long grow = blockIdx.x;
  if (threadIdx.x < nsplit) {
    s_m[threadIdx.x] = part_m[threadIdx.x * rows + grow];
    s_l[threadIdx.x] = part_l[threadIdx.x * rows + grow];
  }
  __syncthreads();
  float Mx = MA_NEG;
  for (int s = 0; s < nsplit; ++s) Mx = fmaxf(Mx, s_m[s]);
  float L = 0.f;
  for (int s = 0; s < nsplit; ++s) L += s_l[s] * expf(s_m[s] - Mx);
  const float inv = L > 0.f ? 1.f / L : 0.f;
  for (int d = threadIdx.x; d < V; d += blockDim.x) {
    float a = 0.f;
#pragma unroll 4
    for (int s = 0; s < nsplit; ++s) a += part_o[(s * rows + grow) * V + d] * expf(s_m[s] - Mx);
    a *= inv;
    if (gated != nullptr) {
      const float gv = __bfloat162float(gate[(grow / HM) * gstride + (grow % HM) * V + d]);
      gated[grow * V + d] = __float2bfloat16(a * sigmoidf_(gv));
    } else {
      out[grow * V + d] = a;
    }
  }
}

// gate [T, H*V] (any row stride) with M = 1: -> bf16 [T, H*V], the gated result;
// gate empty: -> fp32 [T, H*M*V], every map's result
torch::Tensor map_attention_mfma(torch::Tensor q, torch::Tensor gate, torch::Tensor pool, int64_t H, int64_t G,
                                 int64_t M, int64_t D, int64_t V, double scale, double cap, torch::Tensor tiles,
                                 torch::Tensor cu, torch::Tensor start_pos, torch::Tensor tables, int64_t bs,
                                 int64_t nsplit, int64_t tile_rows) {
  TORCH_CHECK(tile_rows == MA_ROWS || tile_rows == 2 * MA_ROWS, "rows a workgroup: 64 or 128 (what the tile list was made for)");
  TORCH_CHECK(q.is_cuda() && q.dim() == 2 && q.is_contiguous() && q.scalar_type() == at::kBFloat16 &&
              q.size(1) == H * M * D);
  TORCH_CHECK(pool.is_contiguous() && pool.dim() == 2 && pool.scalar_type() == at::kBFloat16 &&
              pool.size(1) == G * (M * D + V));
  check_i32(tiles, "tiles"); check_i32(cu, "cu"); check_i32(start_pos, "start_pos"); check_i32(tables, "tables");
  const int T_ = q.size(0), R = start_pos.numel();
  TORCH_CHECK(G >= 1 && M >= 1 && H % G == 0 && bs >= 1 && G * M <= 65535 && cap >= 0.0 &&
              (long)T_ * H * M * V < (1L << 40));
  TORCH_CHECK(D % 8 == 0 && V % 8 == 0 && D <= 256 && V <= 256, "MFMA path: head dims multiples of 8, at most 256");
  TORCH_CHECK(pool.size(0) % bs == 0);
  TORCH_CHECK(cu.numel() == R + 1 && tiles.dim() == 2 && tiles.size(1) == 2 && tables.dim() == 2 && tables.size(0) == R);
  TORCH_CHECK(nsplit >= 1 && nsplit <= MA_MAX_SPLIT);
  const bool has_gate = gate.numel() > 0;
  long gstride = 0;
  if (has_gate) {
    TORCH_CHECK(M == 1, "the fused gate is elementwise on the heads of a one-map attention");
    TORCH_CHECK(gate.is_cuda() && gate.dim() == 2 && gate.stride(1) == 1 && gate.size(0) == T_ &&
                gate.size(1) == H * V && gate.scalar_type() == at::kBFloat16, "gate [T, H*V] bf16");
    gstride = gate.stride(0);
  }
  auto fo = q.options().dtype(at::kFloat);
  auto out = has_gate ? torch::empty({T_, H * V}, q.options()) : torch::empty({T_, H * M * V}, fo);
  const int nblk = tiles.size(0);
  if (T_ == 0 || nblk == 0) return out;
  const int nks = ((int)D + 31) / 32, nt = ((int)V + 15) / 16;
  auto stream = at::cuda::getCurrentHIPStream();
  torch::Tensor po, pm, pl;
  float *pop = nullptr, *pmp = nullptr, *plp = nullptr;
  if (nsplit > 1) {
    po = torch::empty({nsplit, (long)T_ * H * M, V}, fo);
    pm = torch::empty({nsplit, (long)T_ * H * M}, fo);
    pl = torch::empty({nsplit, (long)T_ * H * M}, fo);
    pop = po.data_ptr<float>(); pmp = pm.data_ptr<float>(); plp = pl.data_ptr<float>();
  }
  float* outp = has_gate ? nullptr : out.data_ptr<float>();
  bf16* gatedp = has_gate ? (bf16*)out.data_ptr() : nullptr;
  const bf16* gatep = has_gate ? (const bf16*)gate.data_ptr() : nullptr;
  const dim3 grid(nblk, (unsigned)nsplit, (unsigned)(G * M));
#define MA_MFMA1(NKS, NT, RT)                                                                                   \
  hipLaunchKernelGGL((map_attn_mfma_kernel<NKS, NT, RT>), grid, dim3(256),                                      \
      ((size_t)MA_KT * (NKS * 32 + NT * 16 + 8) + MA_ROWS * RT * MA_KT) * sizeof(short) +                       \
          MA_ROWS * RT * sizeof(float),                                                                         \
      stream, (const bf16*)q.data_ptr(), gatep, gstride, (const bf16*)pool.data_ptr(), (float)scale, (float)cap, \
      tiles.data_ptr<int>(), cu.data_ptr<int>(), start_pos.data_ptr<int>(), tables.data_ptr<int>(),             \
      (int)tables.size(1), (int)bs, outp, gatedp, pop, pmp, plp, (int)nsplit, T_, (int)H, (int)G, (int)M,       \
      (int)D, (int)V)
#define MA_MFMA(NKS, NT)                        \
  do {                                          \
    if (tile_rows == MA_ROWS) MA_MFMA1(NKS, NT, 1); \
    else MA_MFMA1(NKS, NT, 2);                  \
  } while (0)
  if (nks <= 2 && nt <= 4) MA_MFMA(2, 4);
  else if (nks <= 2 && nt <= 8) MA_MFMA(2, 8);
  else if (nks <= 4 && nt <= 8) MA_MFMA(4, 8);
  else if (nks <= 4) MA_MFMA(4, 16);
  else MA_MFMA(8, 16);
#undef MA_MFMA1
#undef MA_MFMA
  if (nsplit > 1)
    hipLaunchKernelGGL(map_combine_kernel, dim3((unsigned)((long)T_ * H * M)), dim3(128), 0, stream, pop, pmp, plp,
                       outp, gatedp, gatep, gstride, (int)nsplit, (long)T_ * H * M, (int)(H * M), (int)V);
  return out;
}
