// Pooled-window grouped-query attention on the matrix cores (bf16 storage).
//
// Rows of the problem are (token, query head) pairs of ONE request and ONE
// key/value head (the rep = H / G query heads that share it), 64 per workgroup
// (16 per wave), numbered token-major.  The keys a workgroup walks are, in
// tiles of 32 staged in LDS as [key of the kv head | value of the kv head]:
//   * pooled tiles: the pooled rows of blocks 0 .. nb_max-1 (nb_max: blocks visible
//     to the workgroup's LAST token),
//   * token tiles: cache rows of positions lo_min .. p_max (window start of its
//     FIRST token .. its last token).
// A row at position p sees pooled entry e iff e < max(0, p - window + 1) / P and
// token j iff p - window < j <= p; the rest of a tile is masked per row.
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

constexpr int PW_KT = 32;     // keys per tile
constexpr int PW_ROWS = 64;   // rows per workgroup
constexpr float PW_NEG = -1e30f;
constexpr int PW_MAX_SPLIT = 64;

template <int NKS, int NT>
__global__ __launch_bounds__(256) void pooled_window_attn_mfma_kernel(
    const bf16* __restrict__ q, const bf16* __restrict__ pool, const bf16* __restrict__ pooled, float scale,
    int window, int P, int rpp, const int* __restrict__ tiles, const int* __restrict__ cu,
    const int* __restrict__ start_pos, const int* __restrict__ tables, int maxb, int bs, bf16* __restrict__ out,
    long out_stride, int out_col, float out_scale, float* __restrict__ part_o, float* __restrict__ part_m,
    float* __restrict__ part_l, int nsplit, int Tn, int H, int G, int D, int V) {
  static_assert(NT % 4 == 0, "value tiles are dealt to four waves");
  constexpr int NTW = NT / 4;                    // value tiles per wave
  constexpr int KW = NKS * 32;                   // staged key columns (zero-padded)
  constexpr int ldk = KW + NT * 16 + 8;          // LDS row stride (bf16), padded against bank conflicts
  extern __shared__ __align__(16) short lds[];   // [PW_KT][ldk] key|value tile | P^T [64][32] | factors [64]
  short* const p_lds = lds + PW_KT * ldk;
  float* const f_lds = reinterpret_cast<float*>(p_lds + PW_ROWS * PW_KT);
  const int req = tiles[2 * blockIdx.x], row0 = tiles[2 * blockIdx.x + 1];
  const int kvh = blockIdx.z, rep = H / G;
  const int t0 = cu[req], n_rows = (cu[req + 1] - t0) * rep, start = start_pos[req];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, c = lane & 15, g4 = lane >> 4;
  const int width = G * (D + V);

  // first product and softmax: wave w owns rows row0 + 16 w + (0..15), one per lane column c
  const int my_row = row0 + wave * 16 + c;
  const bool row_ok = my_row < n_rows;
  const int my_tok = row_ok ? my_row / rep : 0, my_head = kvh * rep + (row_ok ? my_row % rep : 0);
  const int my_p = row_ok ? start + my_tok : -1;                    // the row's position
  const int my_lo = max(0, my_p - window + 1);                      // first token of its window
  const int my_nb = my_lo / P;                                      // pooled blocks it sees
  const int last_row = min(row0 + PW_ROWS, n_rows) - 1;
  const int p_max = start + last_row / rep, p_min = start + row0 / rep;
  const int lo_min = max(0, p_min - window + 1);
  const int nb_max = max(0, p_max - window + 1) / P;
  int rt_pmax[4], rt_lomin[4], rt_nb[4];                            // the same per row tile of 16
#pragma unroll
  for (int rt = 0; rt < 4; ++rt) {
    const int first = row0 + rt * 16;
    if (first < n_rows) {
      rt_pmax[rt] = start + (min(first + 16, n_rows) - 1) / rep;
      rt_lomin[rt] = max(0, start + first / rep - window + 1);
      rt_nb[rt] = max(0, rt_pmax[rt] - window + 1) / P;
    } else {
      rt_pmax[rt] = -1; rt_lomin[rt] = 0; rt_nb[rt] = 0;
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
  float m = PW_NEG, l = 0.f;

  // tile list: pooled tiles, then token tiles
  const int npt = (nb_max + PW_KT - 1) / PW_KT;
  const int jt0 = lo_min / PW_KT;
  const int ntiles = npt + (p_max / PW_KT - jt0 + 1);
  int tile_lo = 0, tile_hi = ntiles;
  if (nsplit > 1) {
    const int per = (ntiles + nsplit - 1) / nsplit;
    tile_lo = blockIdx.y * per;
    tile_hi = min(ntiles, tile_lo + per);
  }
  const int* tab = tables + (long)req * maxb;
  constexpr int cpr = (KW + NT * 16) / 8;         // 16 B chunks per staged row
  constexpr int NSTG = (PW_KT * cpr + 255) / 256;
  short8 stg[NSTG];
  int s_row[NSTG], s_lds[NSTG], s_col[NSTG];      // s_col: column in the cache row, -1: zero fill
#pragma unroll
  for (int k = 0; k < NSTG; ++k) {
    const int i = threadIdx.x + k * 256;
    const int r = i / cpr, d = (i % cpr) * 8;
    s_row[k] = (i < PW_KT * cpr) ? r : -1;
    s_lds[k] = r * ldk + d;
    int col = -1;
    if (d < KW) {
      if (d < D) col = kvh * D + d;
    } else if (d - KW < V) {
      col = G * D + kvh * V + (d - KW);
    }
    s_col[k] = (i < PW_KT * cpr) ? col : -1;
  }
  // Register-staged tile pipeline: the global loads of tile t+1 are issued right
  // after tile t became visible in LDS and are waited for when they are written
  // to LDS at the top of the next iteration.
  // pages that are a multiple of the key tile hold a token tile in one piece: one scalar
  // page lookup per tile instead of two divisions per staged row
  const bool whole = (bs % PW_KT) == 0;
  long s_off[NSTG];                               // offset inside a tile whose rows are consecutive
#pragma unroll
  for (int k = 0; k < NSTG; ++k) s_off[k] = (long)s_row[k] * width + s_col[k];
  auto issue = [&](int tile) {
    const bool is_pooled = tile < npt;
    const int base = is_pooled ? tile * PW_KT : (jt0 + tile - npt) * PW_KT;
    if (!is_pooled && whole) {
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
        if (is_pooled) {
          if (e < nb_max)
            v = *reinterpret_cast<const short8*>(pooled + ((long)tab[e / rpp] * rpp + (e % rpp)) * width + s_col[k]);
        } else if (e <= p_max) {
          v = *reinterpret_cast<const short8*>(pool + ((long)tab[e / bs] * bs + (e % bs)) * width + s_col[k]);
        }
      }
      stg[k] = v;
    }
  };
  if (tile_lo < tile_hi) issue(tile_lo);
  for (int tile = tile_lo; tile < tile_hi; ++tile) {
    const bool is_pooled = tile < npt;
    const int base = is_pooled ? tile * PW_KT : (jt0 + tile - npt) * PW_KT;
#pragma unroll
    for (int k = 0; k < NSTG; ++k)
      if (s_row[k] >= 0) *reinterpret_cast<short8*>(lds + s_lds[k]) = stg[k];
    __syncthreads();
    if (tile + 1 < tile_hi) issue(tile + 1);
    bool act[4];                                  // does row tile rt see anything of this key tile
#pragma unroll
    for (int rt = 0; rt < 4; ++rt)
      act[rt] = is_pooled ? (base < rt_nb[rt]) : (base <= rt_pmax[rt] && base + PW_KT - 1 >= rt_lomin[rt]);
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
      float mx = PW_NEG;
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const int e = base + (i >> 2) * 16 + 4 * g4 + (i & 3);
        ok[i] = is_pooled ? (e < my_nb) : (e <= my_p && e >= my_lo);
        s[i] = st[i >> 2][i & 3] * scale;
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
      *reinterpret_cast<short8*>(p_lds + (wave * 16 + c) * PW_KT + g4 * 8) = pk;
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
        short8 tmp = *reinterpret_cast<const short8*>(p_lds + (rt * 16 + c) * PW_KT + g4 * 8);
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
    if (g4 == 0) f_lds[wave * 16 + c] = (row_ok && l > 0.f) ? out_scale / l : 0.f;
    __syncthreads();
#pragma unroll
    for (int rt = 0; rt < 4; ++rt) {
      const int row = row0 + rt * 16 + c;
      if (row < n_rows) {
        const float inv = f_lds[rt * 16 + c];
        bf16* op = out + (long)(t0 + row / rep) * out_stride + out_col + (long)(kvh * rep + row % rep) * V;
#pragma unroll
        for (int i = 0; i < NTW; ++i) {
          const int d = (wave + 4 * i) * 16 + 4 * g4;
          if (d < V) {
#pragma unroll
            for (int r = 0; r < 4; ++r) op[d + r] = __float2bfloat16(oacc[i][rt][r] * inv);
          }
        }
      }
    }
  } else {
    const long rows_all = (long)Tn * H;
    if (g4 == 0 && row_ok) {
      const long grow = (long)(t0 + my_tok) * H + my_head;
      part_m[blockIdx.y * rows_all + grow] = m;
      part_l[blockIdx.y * rows_all + grow] = l;
    }
#pragma unroll
    for (int rt = 0; rt < 4; ++rt) {
      const int row = row0 + rt * 16 + c;
      if (row < n_rows) {
        const long grow = (long)(t0 + row / rep) * H + kvh * rep + row % rep;
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

__global__ void pooled_window_combine_kernel(const float* __restrict__ part_o, const float* __restrict__ part_m,
                                             const float* __restrict__ part_l, bf16* __restrict__ out,
                                             long out_stride, int out_col, float out_scale, int nsplit, int Tn, int H,
                                             int V) {
  __shared__ float s_m[PW_MAX_SPLIT], s_l[PW_MAX_SPLIT];
  const long grow = blockIdx.x;                 // token * H + head
  const int head = (int)(grow % H);
  const long tok = grow / H;
  const long rows = (long)Tn * H;
  if (threadIdx.x < nsplit) {
    s_m[threadIdx.x] = part_m[threadIdx.x * rows + grow];
    s_l[threadIdx.x] = part_l[threadIdx.x * rows + grow];
  }
  __syncthreads();
  float M = PW_NEG;
  for (int s = 0; s < nsplit; ++s) M = fmaxf(M, s_m[s]);
  float L = 0.f;
  for (int s = 0; s < nsplit; ++s) L += s_l[s] * expf(s_m[s] - M);
  const float inv = L > 0.f ? out_scale / L : 0.f;
  for (int d = threadIdx.x; d < V; d += blockDim.x) {
    float a = 0.f;
#pragma unroll 4
    for (int s = 0; s < nsplit; ++s) a += part_o[(s * rows + grow) * V + d] * expf(s_m[s] - M);
    out[tok * out_stride + out_col + (long)head * V + d] = __float2bfloat16(a * inv);
  }
}

void pooled_window_attention_mfma(torch::Tensor q, torch::Tensor pool, torch::Tensor pooled, int64_t H, int64_t G,
                                  int64_t D, int64_t V, double scale, int64_t window, int64_t P, int64_t rpp,
                                  torch::Tensor tiles, torch::Tensor cu, torch::Tensor start_pos,
                                  torch::Tensor tables, int64_t bs, int64_t nsplit, torch::Tensor out,
                                  int64_t out_col, double out_scale) {
  TORCH_CHECK(q.is_cuda() && q.dim() == 2 && q.is_contiguous() && q.scalar_type() == at::kBFloat16 && q.size(1) == H * D);
  TORCH_CHECK(pool.is_contiguous() && pool.dim() == 2 && pool.scalar_type() == at::kBFloat16 && pool.size(1) == G * (D + V));
  TORCH_CHECK(pooled.is_contiguous() && pooled.dim() == 2 && pooled.scalar_type() == at::kBFloat16 &&
              pooled.size(1) == pool.size(1));
  check_i32(tiles, "tiles"); check_i32(cu, "cu"); check_i32(start_pos, "start_pos"); check_i32(tables, "tables");
  const int T_ = q.size(0), R = start_pos.numel();
  TORCH_CHECK(G >= 1 && H % G == 0 && window >= 1 && P >= 1 && bs >= 1 && rpp * P >= bs);
  TORCH_CHECK(D % 8 == 0 && V % 8 == 0 && D <= 256 && V <= 256, "MFMA path: head dims multiples of 8, at most 256");
  TORCH_CHECK(pool.size(0) % bs == 0 && pooled.size(0) / rpp >= pool.size(0) / bs);
  TORCH_CHECK(cu.numel() == R + 1 && tiles.dim() == 2 && tiles.size(1) == 2 && tables.dim() == 2 && tables.size(0) == R);
  TORCH_CHECK(nsplit >= 1 && nsplit <= PW_MAX_SPLIT);
  TORCH_CHECK(out.is_cuda() && out.dim() == 2 && out.stride(1) == 1 && out.size(0) == T_ &&
              out.scalar_type() == at::kBFloat16 && out_col >= 0 && out_col + H * V <= out.size(1));
  const int nblk = tiles.size(0);
  if (T_ == 0 || nblk == 0) return;
  auto stream = at::cuda::getCurrentHIPStream();
  torch::Tensor po, pm, pl;
  float *pop = nullptr, *pmp = nullptr, *plp = nullptr;
  if (nsplit > 1) {
    auto fo = q.options().dtype(at::kFloat);
    // every (split, row) entry is written by the kernel: no fill needed
    po = torch::empty({nsplit, (long)T_ * H, V}, fo);
    pm = torch::empty({nsplit, (long)T_ * H}, fo);
    pl = torch::empty({nsplit, (long)T_ * H}, fo);
    pop = po.data_ptr<float>(); pmp = pm.data_ptr<float>(); plp = pl.data_ptr<float>();
  }
  const dim3 grid(nblk, (unsigned)nsplit, (unsigned)G);
#define PW_MFMA(NKS, NT)                                                                                        \
  hipLaunchKernelGGL((pooled_window_attn_mfma_kernel<NKS, NT>), grid, dim3(256),                                \
      ((size_t)PW_KT * (NKS * 32 + NT * 16 + 8) + PW_ROWS * PW_KT) * sizeof(short) + PW_ROWS * sizeof(float),   \
      stream, (const bf16*)q.data_ptr(), (const bf16*)pool.data_ptr(), (const bf16*)pooled.data_ptr(),          \
      (float)scale, (int)window, (int)P, (int)rpp, tiles.data_ptr<int>(), cu.data_ptr<int>(),                   \
      start_pos.data_ptr<int>(), tables.data_ptr<int>(), (int)tables.size(1), (int)bs, (bf16*)out.data_ptr(),   \
      (long)out.stride(0), (int)out_col, (float)out_scale, pop, pmp, plp, (int)nsplit, T_, (int)H, (int)G,      \
      (int)D, (int)V)
  const int nks = ((int)D + 31) / 32, nt = ((int)V + 15) / 16;
  if (nks <= 2 && nt <= 4) PW_MFMA(2, 4);
  else if (nks <= 4 && nt <= 8) PW_MFMA(4, 8);
  else PW_MFMA(8, 16);
#undef PW_MFMA
  if (nsplit > 1)
    hipLaunchKernelGGL(pooled_window_combine_kernel, dim3(T_ * (unsigned)H), dim3(128), 0, stream, pop, pmp, plp,
                       (bf16*)out.data_ptr(), (long)out.stride(0), (int)out_col, (float)out_scale, (int)nsplit, T_,
                       (int)H, (int)V);
}
