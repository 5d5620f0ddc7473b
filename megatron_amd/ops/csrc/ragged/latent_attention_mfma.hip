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
    float* __restrict__ part_m, float* __restrict__ part_l, int nsplit, int Tn, int H, int Dk, int rank,
    int nks, int nt, int ldk) {
  extern __shared__ __align__(16) short lds[];   // [LA_KT][ldk]
  const int req = tiles[2 * blockIdx.x], row0 = tiles[2 * blockIdx.x + 1];
  const int t0 = cu[req], n_rows = (cu[req + 1] - t0) * H, start = start_pos[req];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, c = lane & 15, g = lane >> 4;

  const int my_row = row0 + wave * 16 + c;
  const bool row_ok = my_row < n_rows;
  const int my_tok = row_ok ? my_row / H : 0, my_head = row_ok ? my_row % H : 0;
  const int my_bound = row_ok ? start + my_tok : -1;            // last key position this row sees
  const int kend_blk = start + (min(row0 + LA_ROWS, n_rows) - 1) / H;
  const int wave_first = row0 + wave * 16;
  const int kend_wave = (wave_first < n_rows) ? start + (min(wave_first + 16, n_rows) - 1) / H : -1;

  bf16x8 qb[NKS];
  {
    const bf16* qp = q + ((long)(t0 + my_tok) * H + my_head) * Dk;
#pragma unroll
    for (int ks = 0; ks < NKS; ++ks) {
      short8 v = short8{0, 0, 0, 0, 0, 0, 0, 0};
      const int d = ks * 32 + 8 * g;
      if (ks < nks && row_ok && d < Dk) v = *reinterpret_cast<const short8*>(qp + d);
      qb[ks] = *reinterpret_cast<bf16x8*>(&v);
    }
  }
  f32x4 oacc[NT];
#pragma unroll
  for (int n = 0; n < NT; ++n) oacc[n] = f32x4{0.f, 0.f, 0.f, 0.f};
  float m = LA_NEG, l = 0.f;

  const int ntiles = kend_blk / LA_KT + 1;
  int tile_lo = 0, tile_hi = ntiles;
  if (nsplit > 1) {
    const int per = (ntiles + nsplit - 1) / nsplit;
    tile_lo = blockIdx.y * per;
    tile_hi = min(ntiles, tile_lo + per);
  }
  const int* tab = tables + (long)req * maxb;
  const int cpr = nks * 4;                        // 16 B chunks per staged row
  for (int tile = tile_lo; tile < tile_hi; ++tile) {
    const int j0 = tile * LA_KT;
    for (int i = threadIdx.x; i < LA_KT * cpr; i += 256) {
      const int r = i / cpr, d = (i % cpr) * 8, j = j0 + r;
      short8 v = short8{0, 0, 0, 0, 0, 0, 0, 0};
      if (j <= kend_blk && d < Dk)
        v = *reinterpret_cast<const short8*>(pool + ((long)tab[j / bs] * bs + (j % bs)) * Dk + d);
      *reinterpret_cast<short8*>(lds + r * ldk + d) = v;
    }
    __syncthreads();
    if (j0 <= kend_wave) {                        // wave-uniform: later tiles are all masked for this wave
      f32x4 st[2];
#pragma unroll
      for (int kvt = 0; kvt < 2; ++kvt) {
        st[kvt] = f32x4{0.f, 0.f, 0.f, 0.f};
        const short* krow = lds + (kvt * 16 + c) * ldk + 8 * g;
#pragma unroll
        for (int ks = 0; ks < NKS; ++ks) {
          if (ks < nks) {
            short8 tmp = *reinterpret_cast<const short8*>(krow + ks * 32);
            st[kvt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(*reinterpret_cast<bf16x8*>(&tmp), qb[ks], st[kvt],
                                                              0, 0, 0);
          }
        }
      }
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
      const float corr = expf(m - m_new);
      m = m_new;
      float psum = 0.f;
      short8 pk;
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const float p = ok[i] ? expf(s[i] - m_new) : 0.f;
        psum += p;
        pk[i] = f2sbf(p);
      }
      l = l * corr + psum;
      const bf16x8 pb = *reinterpret_cast<bf16x8*>(&pk);
#pragma unroll
      for (int n = 0; n < NT; ++n) {
        if (n < nt) {
          oacc[n] *= corr;
          short8 av;
          const short* vcol = lds + n * 16 + c;
#pragma unroll
          for (int j = 0; j < 8; ++j) av[j] = vcol[((j >> 2) * 16 + 4 * g + (j & 3)) * ldk];
          oacc[n] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(*reinterpret_cast<bf16x8*>(&av), pb, oacc[n], 0, 0, 0);
        }
      }
    }
    __syncthreads();
  }
  l += __shfl_xor(l, 16, 64);
  l += __shfl_xor(l, 32, 64);
  if (!row_ok) return;
  if (nsplit == 1) {
    const float sk = sink[my_head];
    const float M = fmaxf(m, sk);
    const float f = expf(m - M);
    const float inv = f / (l * f + expf(sk - M));
    bf16* op = out + ((long)my_head * Tn + t0 + my_tok) * rank;
#pragma unroll
    for (int n = 0; n < NT; ++n) {
      const int d = n * 16 + 4 * g;
      if (n < nt && d < rank) {
#pragma unroll
        for (int r = 0; r < 4; ++r) op[d + r] = __float2bfloat16(oacc[n][r] * inv);
      }
    }
  } else {
    const long grow = (long)blockIdx.y * Tn * H + (long)t0 * H + my_row;
    float* po = part_o + grow * rank;
#pragma unroll
    for (int n = 0; n < NT; ++n) {
      const int d = n * 16 + 4 * g;
      if (n < nt && d < rank) *reinterpret_cast<f32x4*>(po + d) = oacc[n];
    }
    if (g == 0) {
      part_m[grow] = m;
      part_l[grow] = l;
    }
  }
}

__global__ void latent_attn_combine_kernel(const float* __restrict__ part_o, const float* __restrict__ part_m,
                                           const float* __restrict__ part_l, const float* __restrict__ sink,
                                           bf16* __restrict__ out, int nsplit, int Tn, int H, int rank) {
  const long grow = blockIdx.x;                 // token * H + head
  const int head = (int)(grow % H);
  const long tok = grow / H;
  const long rows = (long)Tn * H;
  const float sk = sink[head];
  float M = sk;
  for (int s = 0; s < nsplit; ++s) M = fmaxf(M, part_m[s * rows + grow]);
  float L = expf(sk - M);
  for (int s = 0; s < nsplit; ++s) L += part_l[s * rows + grow] * expf(part_m[s * rows + grow] - M);
  for (int d = threadIdx.x; d < rank; d += blockDim.x) {
    float a = 0.f;
    for (int s = 0; s < nsplit; ++s) a += part_o[(s * rows + grow) * rank + d] * expf(part_m[s * rows + grow] - M);
    out[((long)head * Tn + tok) * rank + d] = __float2bfloat16(a / L);
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
  TORCH_CHECK(bs > 0 && pool.size(0) % bs == 0 && nsplit >= 1);
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
    po = torch::zeros({nsplit, (long)T_ * H, rank}, fo);
    pm = torch::full({nsplit, (long)T_ * H}, LA_NEG, fo);
    pl = torch::zeros({nsplit, (long)T_ * H}, fo);
    pop = po.data_ptr<float>(); pmp = pm.data_ptr<float>(); plp = pl.data_ptr<float>();
  }
  const int ldk = nks * 32 + 8;
  const size_t smem = (size_t)LA_KT * ldk * sizeof(short);
  const dim3 grid(nblk, (unsigned)nsplit);
#define LAUNCH_MFMA(NKS, NT)                                                                                   \
  hipLaunchKernelGGL((latent_attn_mfma_kernel<NKS, NT>), grid, dim3(256), smem, stream,                        \
      (const bf16*)q.data_ptr(), (const bf16*)pool.data_ptr(), sink.data_ptr<float>(), (float)scale,           \
      tiles.data_ptr<int>(), cu.data_ptr<int>(), start_pos.data_ptr<int>(), tables.data_ptr<int>(),            \
      (int)tables.size(1), (int)bs, (bf16*)out.data_ptr(), pop, pmp, plp, (int)nsplit, T_, H, Dk, (int)rank,   \
      nks, nt, ldk)
  if (nks <= 5 && nt <= 8) LAUNCH_MFMA(5, 8);
  else if (nks <= 10 && nt <= 16) LAUNCH_MFMA(10, 16);
  else LAUNCH_MFMA(18, 32);
#undef LAUNCH_MFMA
  if (nsplit > 1)
    hipLaunchKernelGGL(latent_attn_combine_kernel, dim3(T_ * H), dim3(128), 0, stream, pop, pmp, plp,
                       sink.data_ptr<float>(), (bf16*)out.data_ptr(), (int)nsplit, T_, H, (int)rank);
  return out.transpose(0, 1);
}
