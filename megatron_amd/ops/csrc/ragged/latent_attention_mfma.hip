// Latent-cache attention with sink on the matrix cores (bf16 storage).
//
// Rows of the problem are (token, head) pairs of one request, 64 per
// workgroup (16 per wave); all rows of a request share the cached rows
// [latent | rotated key part], which serve as keys (all Dk entries) and as
// values (first `rank` entries).  Keys are walked in tiles of 32 staged in LDS.
//
// Both products run transposed so that a query row is a lane column (q = lane&15)
// from the first MFMA to the last and softmax statistics never cross lanes
// except over the four 16-lane groups:
//   S^T[kv][q] = sum_d K[kv][d] Q[q][d]     A = K tile rows (LDS, 16 B reads), B = Q (registers)
//   O^T[d][q] += sum_kv V^T[d][kv] P^T[kv][q]   A = V^T gathered from the same LDS tile, B = P^T
// The D fragment of S^T (lane (c, g): kv = 4g + r of two 16-key sub-tiles) is used
// directly as the B fragment of the second product by numbering the k slots of
// that MFMA (g, j) -> kv = 4g + j (j < 4), 16 + 4g + j - 4 (j >= 4); the A fragment
// gathers V in the same order, so no register relayout is needed.
//
// Work split inside a workgroup: wave w computes S^T and the softmax of row tile w
// (16 rows) and publishes P^T (bf16, already in B-fragment order) and the
// rescale factor of its rows in LDS; for the second product wave w owns the value
// tiles n = w, w+4, ... of ALL four row tiles, so every V^T fragment gathered
// from LDS (eight 2-byte reads) feeds four MFMAs instead of one.
//
// Long contexts with few rows (decode) split the key range over gridDim.y;
// partial (O, m, l) go to fp32 scratch and a combine kernel applies the sink
// and the normalisation.
#include "ragged_common.h"

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

constexpr int LA_KT = 32;     // keys per tile
constexpr int LA_ROWS = 64;   // rows per workgroup
constexpr float LA_NEG = -1e30f;

template <int NKS, int NT>
__global__ __launch_bounds__(256) void latent_attn_mfma_kernel(
    const bf16* __restrict__ q, const bf16* __restrict__ pool, const float* __restrict__ sink, float scale,
    const int* __restrict__ tiles, const int* __restrict__ cu, const int* __restrict__ start_pos,
    const int* __restrict__ tables, int maxb, int bs, bf16* __restrict__ out, float* __restrict__ part_o,
    float* __restrict__ part_m, float* __restrict__ part_l, int nsplit, int Tn, int H, int Dk, int rank) {
  // NKS (32-wide k steps over the row) and NT (16-wide value tiles) are compile-time
  // and the MFMA loops carry no run-time guards: staged rows are zero-padded to
  // NKS * 32 columns, so surplus steps add zeros and surplus value tiles are
  // simply not stored.  Guards inside the unrolled loops would keep the compiler
  // from issuing LDS reads ahead of the MFMAs that consume them, and at one wave
  // per SIMD nothing else hides that latency.
  static_assert(NT % 4 == 0 && NT * 16 <= NKS * 32, "value tiles are dealt to four waves and lie inside a row");
  constexpr int NTW = NT / 4;                    // value tiles per wave
  constexpr int ldk = NKS * 32 + 8;              // LDS row stride (bf16), padded against bank conflicts
  extern __shared__ __align__(16) short lds[];   // [LA_KT][ldk] key tile | P^T [64][32] | factors [64]
  short* const p_lds = lds + LA_KT * ldk;
  float* const f_lds = reinterpret_cast<float*>(p_lds + LA_ROWS * LA_KT);
  const int req = tiles[2 * blockIdx.x], row0 = tiles[2 * blockIdx.x + 1];
  const int t0 = cu[req], n_rows = (cu[req + 1] - t0) * H, start = start_pos[req];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, c = lane & 15, g = lane >> 4;

  // first product and softmax: wave w owns rows row0 + 16 w + (0..15), one per lane column c
  const int my_row = row0 + wave * 16 + c;
  const bool row_ok = my_row < n_rows;
  const int my_tok = row_ok ? my_row / H : 0, my_head = row_ok ? my_row % H : 0;
  const int my_bound = row_ok ? start + my_tok : -1;            // last key position this row sees
  const int kend_blk = start + (min(row0 + LA_ROWS, n_rows) - 1) / H;
  int rt_kend[4];                                               // last key any row of row tile rt sees
#pragma unroll
  for (int rt = 0; rt < 4; ++rt) {
    const int first = row0 + rt * 16;
    rt_kend[rt] = (first < n_rows) ? start + (min(first + 16, n_rows) - 1) / H : -1;
  }
  const int kend_wave = rt_kend[wave];

  bf16x8 qb[NKS];
  {
    const bf16* qp = q + ((long)(t0 + my_tok) * H + my_head) * Dk;
#pragma unroll
    for (int ks = 0; ks < NKS; ++ks) {
      short8 v = short8{0, 0, 0, 0, 0, 0, 0, 0};
      const int d = ks * 32 + 8 * g;
      if (row_ok && d < Dk) v = *reinterpret_cast<const short8*>(qp + d);
      qb[ks] = *reinterpret_cast<bf16x8*>(&v);
    }
  }
  // second product: wave w owns value tiles n = w, w + 4, ... for ALL four row tiles
  f32x4 oacc[NTW][4];
#pragma unroll
  for (int i = 0; i < NTW; ++i)
#pragma unroll
    for (int rt = 0; rt < 4; ++rt) oacc[i][rt] = f32x4{0.f, 0.f, 0.f, 0.f};
  float m = LA_NEG, l = 0.f;

  const int ntiles = kend_blk / LA_KT + 1;
  int tile_lo = 0, tile_hi = ntiles;
  if (nsplit > 1) {
    const int per = (ntiles + nsplit - 1) / nsplit;
    tile_lo = blockIdx.y * per;
    tile_hi = min(ntiles, tile_lo + per);
  }
  const int* tab = tables + (long)req * maxb;
  constexpr int cpr = NKS * 4;                    // 16 B chunks per staged row
  // Register-staged tile pipeline: the global loads of tile t+1 are issued
  // right after tile t became visible in LDS and are only waited for when
  // they are written to LDS at the top of the next iteration, so their latency
  // hides behind tile t's MFMA work (the kernel runs at one wave per SIMD at
  // the large instantiation; nothing else would hide it).
  constexpr int NSTG = (LA_KT * NKS * 4 + 255) / 256;
  short8 stg[NSTG];
  int s_row[NSTG], s_lds[NSTG];
  long s_off[NSTG];                               // element offset inside the tile's rows, -1: zero fill
#pragma unroll
  for (int k = 0; k < NSTG; ++k) {
    const int i = threadIdx.x + k * 256;
    const int r = i / cpr, d = (i % cpr) * 8;
    s_row[k] = (i < LA_KT * cpr) ? r : -1;
    s_lds[k] = r * ldk + d;
    s_off[k] = (i < LA_KT * cpr && d < Dk) ? (long)r * Dk + d : -1;
  }
  // pages that are a multiple of the key tile hold a tile in one piece: one scalar
  // page lookup per tile instead of a division per staged row
  const bool whole = (bs % LA_KT) == 0;
  auto issue = [&](int tile) {
    const int j0 = tile * LA_KT;
    if (whole) {
      const bf16* base = pool + ((long)tab[j0 / bs] * bs + (j0 % bs)) * Dk;
#pragma unroll
      for (int k = 0; k < NSTG; ++k) {
        short8 v = short8{0, 0, 0, 0, 0, 0, 0, 0};
        if (s_off[k] >= 0 && j0 + s_row[k] <= kend_blk) v = *reinterpret_cast<const short8*>(base + s_off[k]);
        stg[k] = v;
      }
    } else {
#pragma unroll
      for (int k = 0; k < NSTG; ++k) {
        const int j = j0 + s_row[k];
        short8 v = short8{0, 0, 0, 0, 0, 0, 0, 0};
        if (s_off[k] >= 0 && j <= kend_blk)
          v = *reinterpret_cast<const short8*>(pool + ((long)tab[j / bs] * bs + (j % bs)) * Dk +
                                               (s_off[k] - (long)s_row[k] * Dk));
        stg[k] = v;
      }
    }
  };
  if (tile_lo < tile_hi) issue(tile_lo);
  for (int tile = tile_lo; tile < tile_hi; ++tile) {
    const int j0 = tile * LA_KT;
#pragma unroll
    for (int k = 0; k < NSTG; ++k)
      if (s_row[k] >= 0) *reinterpret_cast<short8*>(lds + s_lds[k]) = stg[k];
    __syncthreads();
    if (tile + 1 < tile_hi) issue(tile + 1);
    if (j0 <= kend_wave) {                        // wave-uniform: later tiles are all masked for this wave's rows
      // two independent accumulation chains per key sub-tile (even / odd k steps):
      // four MFMAs in flight instead of two dependent ones
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
          short8 tmp = *reinterpret_cast<const short8*>(lds + (kvt * 16 + c) * ldk + 8 * g + ks * 32);
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
      float mx = LA_NEG;
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const int kv = j0 + (i >> 2) * 16 + 4 * g + (i & 3);
        ok[i] = kv <= my_bound;
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
      // P^T in B-fragment order (k slot (g, i) of column c) and the rescale factor, for all waves
      *reinterpret_cast<short8*>(p_lds + (wave * 16 + c) * LA_KT + g * 8) = pk;
      if (g == 0) f_lds[wave * 16 + c] = corr;
    }
    __syncthreads();
    {
      bf16x8 pb[4];
      float cr[4];
      bool rescale = false;
#pragma unroll
      for (int rt = 0; rt < 4; ++rt) {
        // a row tile that sees nothing of this key tile contributes P = 0 with factor 1
        const bool act = j0 <= rt_kend[rt];
        short8 tmp = *reinterpret_cast<const short8*>(p_lds + (rt * 16 + c) * LA_KT + g * 8);
        const float f = f_lds[rt * 16 + c];
        if (!act) tmp = short8{0, 0, 0, 0, 0, 0, 0, 0};
        cr[rt] = act ? f : 1.f;
        rescale |= cr[rt] != 1.f;
        pb[rt] = *reinterpret_cast<bf16x8*>(&tmp);
      }
      // the running maxima settle after the first tiles: skip the pass over the
      // accumulators (they live in accumulation registers) when no factor differs from 1
      if (__any(rescale)) {
#pragma unroll
        for (int i = 0; i < NTW; ++i)
#pragma unroll
          for (int rt = 0; rt < 4; ++rt) oacc[i][rt] *= cr[rt];
      }
#pragma unroll
      for (int i = 0; i < NTW; ++i) {
        short8 av;
        const short* vcol = lds + (wave + 4 * i) * 16 + c;
#pragma unroll
        for (int j = 0; j < 8; ++j) av[j] = vcol[((j >> 2) * 16 + 4 * g + (j & 3)) * ldk];
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
    // owner waves publish 1 / denominator (with the sink) per row
    if (g == 0) {
      float inv = 0.f;
      if (row_ok) {
        const float sk = sink[my_head];
        const float M = fmaxf(m, sk);
        const float f = expf(m - M);
        inv = f / (l * f + expf(sk - M));
      }
      f_lds[wave * 16 + c] = inv;
    }
    __syncthreads();
#pragma unroll
    for (int rt = 0; rt < 4; ++rt) {
      const int row = row0 + rt * 16 + c;
      if (row < n_rows) {
        const float inv = f_lds[rt * 16 + c];
        bf16* op = out + ((long)(row % H) * Tn + t0 + row / H) * rank;
#pragma unroll
        for (int i = 0; i < NTW; ++i) {
          const int d = (wave + 4 * i) * 16 + 4 * g;
          if (d < rank) {
#pragma unroll
            for (int r = 0; r < 4; ++r) op[d + r] = __float2bfloat16(oacc[i][rt][r] * inv);
          }
        }
      }
    }
  } else {
    const long base = (long)blockIdx.y * Tn * H + (long)t0 * H;
    if (g == 0 && row_ok) {
      part_m[base + my_row] = m;
      part_l[base + my_row] = l;
    }
#pragma unroll
    for (int rt = 0; rt < 4; ++rt) {
      const int row = row0 + rt * 16 + c;
      if (row < n_rows) {
        float* po = part_o + (base + row) * rank;
#pragma unroll
        for (int i = 0; i < NTW; ++i) {
          const int d = (wave + 4 * i) * 16 + 4 * g;
          if (d < rank) *reinterpret_cast<f32x4*>(po + d) = oacc[i][rt];
        }
      }
    }
  }
}

constexpr int LA_MAX_SPLIT = 64;

__global__ void latent_attn_combine_kernel(const float* __restrict__ part_o, const float* __restrict__ part_m,
                                           const float* __restrict__ part_l, const float* __restrict__ sink,
                                           bf16* __restrict__ out, int nsplit, int Tn, int H, int rank) {
  __shared__ float s_m[LA_MAX_SPLIT], s_l[LA_MAX_SPLIT];
  const long grow = blockIdx.x;                 // token * H + head
  const int head = (int)(grow % H);
  const long tok = grow / H;
  const long rows = (long)Tn * H;
  if (threadIdx.x < nsplit) {
    s_m[threadIdx.x] = part_m[threadIdx.x * rows + grow];
    s_l[threadIdx.x] = part_l[threadIdx.x * rows + grow];
  }
  __syncthreads();
  const float sk = sink[head];
  float M = sk;
  for (int s = 0; s < nsplit; ++s) M = fmaxf(M, s_m[s]);
  float L = expf(sk - M);
  for (int s = 0; s < nsplit; ++s) L += s_l[s] * expf(s_m[s] - M);
  const float inv = 1.f / L;
  for (int d = threadIdx.x; d < rank; d += blockDim.x) {
    float a = 0.f;
#pragma unroll 4
    for (int s = 0; s < nsplit; ++s) a += part_o[(s * rows + grow) * rank + d] * expf(s_m[s] - M);
    out[((long)head * Tn + tok) * rank + d] = __float2bfloat16(a * inv);
  }
}

torch::Tensor latent_sink_attention_mfma(torch::Tensor q, torch::Tensor pool, int64_t rank, torch::Tensor sink,
                                         double scale, torch::Tensor tiles, torch::Tensor cu, torch::Tensor start_pos,
                                         torch::Tensor tables, int64_t bs, int64_t nsplit) {
  TORCH_CHECK(q.is_cuda() && q.dim() == 3 && q.is_contiguous() && q.scalar_type() == at::kBFloat16);
  TORCH_CHECK(pool.is_contiguous() && pool.dim() == 2 && pool.scalar_type() == at::kBFloat16);
  check_f32(sink, "sink"); check_i32(tiles, "tiles"); check_i32(cu, "cu"); check_i32(start_pos, "start_pos");
  check_i32(tables, "tables");
  const int T_ = q.size(0), H = q.size(1), Dk = q.size(2);
  const int R = start_pos.numel();
  TORCH_CHECK(pool.size(1) == Dk && rank <= Dk && sink.numel() == H && cu.numel() == R + 1);
  TORCH_CHECK(Dk % 8 == 0 && rank % 4 == 0, "MFMA path: row width a multiple of 8, rank of 4");
  TORCH_CHECK(tiles.dim() == 2 && tiles.size(1) == 2 && tables.dim() == 2 && tables.size(0) == R);
  TORCH_CHECK(bs > 0 && pool.size(0) % bs == 0 && nsplit >= 1 && nsplit <= LA_MAX_SPLIT);
  const int nks = (Dk + 31) / 32, nt = ((int)rank + 15) / 16;
  TORCH_CHECK(nks <= 18 && nt <= 32, "MFMA path: row width <= 576, rank <= 512");
  auto out = torch::empty({H, T_, rank}, q.options());
  const int nblk = tiles.size(0);
  if (T_ == 0 || nblk == 0) return out.transpose(0, 1);
  auto stream = at::cuda::getCurrentHIPStream();
  torch::Tensor po, pm, pl;
  float *pop = nullptr, *pmp = nullptr, *plp = nullptr;
  if (nsplit > 1) {
    auto fo = q.options().dtype(at::kFloat);
    // every (split, valid row) entry is written by the kernel: no fill needed
    po = torch::empty({nsplit, (long)T_ * H, rank}, fo);
    pm = torch::empty({nsplit, (long)T_ * H}, fo);
    pl = torch::empty({nsplit, (long)T_ * H}, fo);
    pop = po.data_ptr<float>(); pmp = pm.data_ptr<float>(); plp = pl.data_ptr<float>();
  }
  const dim3 grid(nblk, (unsigned)nsplit);
#define LAUNCH_MFMA(NKS, NT)                                                                                   \
  hipLaunchKernelGGL((latent_attn_mfma_kernel<NKS, NT>), grid, dim3(256),                                      \
      ((size_t)LA_KT * (NKS * 32 + 8) + LA_ROWS * LA_KT) * sizeof(short) + LA_ROWS * sizeof(float), stream,    \
      (const bf16*)q.data_ptr(), (const bf16*)pool.data_ptr(), sink.data_ptr<float>(), (float)scale,           \
      tiles.data_ptr<int>(), cu.data_ptr<int>(), start_pos.data_ptr<int>(), tables.data_ptr<int>(),            \
      (int)tables.size(1), (int)bs, (bf16*)out.data_ptr(), pop, pmp, plp, (int)nsplit, T_, H, Dk, (int)rank)
  if (nks <= 5 && nt <= 8) LAUNCH_MFMA(5, 8);
  else if (nks <= 9 && nt <= 16) LAUNCH_MFMA(9, 16);
  else if (nks <= 12 && nt <= 20) LAUNCH_MFMA(12, 20);
  else LAUNCH_MFMA(18, 32);
#undef LAUNCH_MFMA
  if (nsplit > 1)
    hipLaunchKernelGGL(latent_attn_combine_kernel, dim3(T_ * H), dim3(128), 0, stream, pop, pmp, plp,
                       sink.data_ptr<float>(), (bf16*)out.data_ptr(), (int)nsplit, T_, H, (int)rank);
  return out.transpose(0, 1);
}
