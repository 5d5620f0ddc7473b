// Grouped-query attention over a sliding window plus mean-pooled blocks, on a
// paged cache of rows [kv_heads * dim normed keys | kv_heads * vdim values]:
// whole-projection query/key norm + cache store, completion of pooled rows,
// and the attention itself (any storage type; fp32 arithmetic).
#include "../ragged/ragged_common.h"

// ---------------------------------------------------------------------------
// q <- rms(q) * wq over ALL query heads at once; cache row <- [rms(k) * wk | v]
// ---------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void qk_norm_store_kernel(
    const T* __restrict__ proj, long stride, int q_off, int qw, int k_off, int kw, int v_off, int vw,
    const float* __restrict__ wq, const float* __restrict__ wk, float eps, T* __restrict__ q_out,
    T* __restrict__ pool, const long* __restrict__ tok_row) {
  __shared__ float red[256 / WAVE];
  const long t = blockIdx.x;
  const T* x = proj + t * stride;
  float ss = 0.f;
  for (int c = threadIdx.x; c < qw; c += 256) {
    const float v = ldf(x + q_off + c);
    ss += v * v;
  }
  const float rq = 1.f / sqrtf(block_reduce_sum<256>(ss, red) / (float)qw + eps);
  for (int c = threadIdx.x; c < qw; c += 256) stf(q_out + t * qw + c, ldf(x + q_off + c) * rq * wq[c]);
  __syncthreads();                               // the reduction buffer is used again
  ss = 0.f;
  for (int c = threadIdx.x; c < kw; c += 256) {
    const float v = ldf(x + k_off + c);
    ss += v * v;
  }
  const float rk = 1.f / sqrtf(block_reduce_sum<256>(ss, red) / (float)kw + eps);
  T* dst = pool + tok_row[t] * (long)(kw + vw);
  for (int c = threadIdx.x; c < kw; c += 256) stf(dst + c, ldf(x + k_off + c) * rk * wk[c]);
  for (int c = threadIdx.x; c < vw; c += 256) dst[kw + c] = x[v_off + c];
}

torch::Tensor qk_norm_store(torch::Tensor proj, int64_t q_off, int64_t qw, int64_t k_off, int64_t kw, int64_t v_off,
                            int64_t vw, torch::Tensor wq, torch::Tensor wk, double eps, torch::Tensor pool,
                            torch::Tensor tok_row) {
  TORCH_CHECK(proj.is_cuda() && proj.dim() == 2 && proj.stride(1) == 1);
  check_f32(wq, "q norm"); check_f32(wk, "k norm");
  TORCH_CHECK(tok_row.is_cuda() && tok_row.scalar_type() == at::kLong && tok_row.is_contiguous());
  const int T_ = proj.size(0), C = proj.size(1);
  TORCH_CHECK(q_off >= 0 && q_off + qw <= C && k_off >= 0 && k_off + kw <= C && v_off >= 0 && v_off + vw <= C);
  TORCH_CHECK(wq.numel() == qw && wk.numel() == kw && tok_row.numel() == T_);
  TORCH_CHECK(pool.is_contiguous() && pool.dim() == 2 && pool.size(1) == kw + vw &&
              pool.scalar_type() == proj.scalar_type());
  auto q = torch::empty({T_, qw}, proj.options());
  if (T_ == 0) return q;
  auto stream = at::cuda::getCurrentHIPStream();
  RAGGED_DISPATCH(proj, hipLaunchKernelGGL((qk_norm_store_kernel<T>), dim3(T_), dim3(256), 0, stream,
      (const T*)proj.data_ptr(), (long)proj.stride(0), (int)q_off, (int)qw, (int)k_off, (int)kw, (int)v_off, (int)vw,
      wq.data_ptr<float>(), wk.data_ptr<float>(), (float)eps, (T*)q.data_ptr(), (T*)pool.data_ptr(),
      tok_row.data_ptr<long>()));
  return q;
}

// ---------------------------------------------------------------------------
// pooled row of every block of P tokens whose last position this step wrote:
// the mean of the P cache rows as the cache holds them
// ---------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void pool_blocks_kernel(
    const T* __restrict__ pool, T* __restrict__ pooled, int P, int rpp, const int* __restrict__ cu,
    const int* __restrict__ start_pos, const int* __restrict__ tables, int maxb, int bs, int width) {
  const int r = blockIdx.x;
  const int start = start_pos[r], n = cu[r + 1] - cu[r];
  const int b = start / P + blockIdx.y;          // blocks [start / P, (start + n) / P) complete in this step
  if (b >= (start + n) / P) return;
  const int* tab = tables + (long)r * maxb;
  T* dst = pooled + ((long)tab[b / rpp] * rpp + (b % rpp)) * width;
  for (int c = threadIdx.x; c < width; c += 256) {
    float s = 0.f;
    for (int i = 0; i < P; ++i) {
      const int j = b * P + i;
      s += ldf(pool + ((long)tab[j / bs] * bs + (j % bs)) * width + c);
    }
    stf(dst + c, s / (float)P);
  }
}

void pool_blocks(torch::Tensor pool, torch::Tensor pooled, int64_t P, int64_t rpp, torch::Tensor cu,
                 torch::Tensor start_pos, torch::Tensor tables, int64_t bs, int64_t max_new) {
  TORCH_CHECK(pool.is_cuda() && pool.is_contiguous() && pool.dim() == 2 && pooled.is_contiguous() &&
              pooled.dim() == 2 && pooled.size(1) == pool.size(1) && pooled.scalar_type() == pool.scalar_type());
  check_i32(cu, "cu"); check_i32(start_pos, "start_pos"); check_i32(tables, "tables");
  const int R = start_pos.numel();
  TORCH_CHECK(P >= 1 && bs >= 1 && rpp * P >= bs, "a page's pooled rows cover the page");
  TORCH_CHECK(pool.size(0) % bs == 0 && pooled.size(0) / rpp >= pool.size(0) / bs, "pooled pool has a page per cache page");
  TORCH_CHECK(cu.numel() == R + 1 && tables.dim() == 2 && tables.size(0) == R);
  if (R == 0 || max_new <= 0) return;
  auto stream = at::cuda::getCurrentHIPStream();
  const dim3 grid(R, (unsigned)(max_new / P + 1));
  RAGGED_DISPATCH(pool, hipLaunchKernelGGL((pool_blocks_kernel<T>), grid, dim3(256), 0, stream,
      (const T*)pool.data_ptr(), (T*)pooled.data_ptr(), (int)P, (int)rpp, cu.data_ptr<int>(),
      start_pos.data_ptr<int>(), tables.data_ptr<int>(), (int)tables.size(1), (int)bs, (int)pool.size(1)));
}

// ---------------------------------------------------------------------------
// attention.  Workgroup = (token, query head), 4 waves.  The keys a query sees
// form one list: the pooled rows of blocks 0 .. nb-1, nb = max(0, p - window + 1) / P,
// then the cache rows of positions max(0, p - window + 1) .. p.  A wave scores
// one row at a time (lanes split the head dim, shuffle-reduce the dot product),
// keeps an online softmax and the weighted value sum in registers; the waves'
// partial results merge through LDS.
// ---------------------------------------------------------------------------
template <typename T, int MAXI>
__global__ __launch_bounds__(256) void pooled_window_attn_kernel(
    const T* __restrict__ q, const T* __restrict__ pool, const T* __restrict__ pooled, float scale, int window,
    int P, int rpp, const int* __restrict__ tok_req, const int* __restrict__ tok_pos,
    const int* __restrict__ tables, int maxb, int bs, T* __restrict__ out, long out_stride, int out_col,
    float out_scale, int H, int G, int D, int V) {
  __shared__ float s_m[4], s_l[4];
  __shared__ float s_acc[4][MAXI * WAVE];
  const int t = blockIdx.x, hd = blockIdx.y;
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
  const int lo = max(0, p - window + 1);
  const int nb = lo / P;                          // blocks that end at or before p - window
  const int total = nb + (p - lo + 1);
  const int* tab = tables + (long)tok_req[t] * maxb;
  float m = -INFINITY, l = 0.f;
  for (int idx = wave; idx < total; idx += 4) {
    const T* row;
    if (idx < nb) {
      row = pooled + ((long)tab[idx / rpp] * rpp + (idx % rpp)) * width;
    } else {
      const int j = lo + (idx - nb);
      row = pool + ((long)tab[j / bs] * bs + (j % bs)) * width;
    }
    const T* kr = row + g * D;
    const T* vr = row + G * D + g * V;
    float dot = 0.f;
#pragma unroll
    for (int i = 0; i < MAXI; ++i) {
      const int d = lane + WAVE * i;
      if (d < D) dot += ldf(kr + d) * qv[i];
    }
    dot = wave_reduce_sum(dot) * scale;
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
  T* op = out + (long)t * out_stride + out_col + (long)hd * V;
  for (int d = threadIdx.x; d < V; d += 256) {
    float a = 0.f;
#pragma unroll
    for (int w = 0; w < 4; ++w) a += s_acc[w][d] * f[w];
    stf(op + d, a / L * out_scale);
  }
}

void pooled_window_attention(torch::Tensor q, torch::Tensor pool, torch::Tensor pooled, int64_t H, int64_t G,
                             int64_t D, int64_t V, double scale, int64_t window, int64_t P, int64_t rpp,
                             torch::Tensor tok_req, torch::Tensor tok_pos, torch::Tensor tables, int64_t bs,
                             torch::Tensor out, int64_t out_col, double out_scale) {
  TORCH_CHECK(q.is_cuda() && q.dim() == 2 && q.is_contiguous() && q.size(1) == H * D);
  TORCH_CHECK(pool.is_contiguous() && pool.dim() == 2 && pool.scalar_type() == q.scalar_type() &&
              pool.size(1) == G * (D + V));
  TORCH_CHECK(pooled.is_contiguous() && pooled.dim() == 2 && pooled.scalar_type() == q.scalar_type() &&
              pooled.size(1) == pool.size(1));
  check_i32(tok_req, "tok_req"); check_i32(tok_pos, "tok_pos"); check_i32(tables, "tables");
  const int T_ = q.size(0);
  TORCH_CHECK(G >= 1 && H % G == 0 && window >= 1 && P >= 1 && bs >= 1 && rpp * P >= bs);
  TORCH_CHECK(pool.size(0) % bs == 0 && pooled.size(0) / rpp >= pool.size(0) / bs);
  TORCH_CHECK(tok_req.numel() == T_ && tok_pos.numel() == T_ && tables.dim() == 2);
  TORCH_CHECK(out.is_cuda() && out.dim() == 2 && out.stride(1) == 1 && out.size(0) == T_ &&
              out.scalar_type() == q.scalar_type() && out_col >= 0 && out_col + H * V <= out.size(1));
  const int wide = (int)std::max(D, V);
  TORCH_CHECK(wide <= 8 * WAVE, "head dim above ", 8 * WAVE);
  if (T_ == 0) return;
  auto stream = at::cuda::getCurrentHIPStream();
#define PW_LAUNCH(MAXI)                                                                                          \
  RAGGED_DISPATCH(q, hipLaunchKernelGGL((pooled_window_attn_kernel<T, MAXI>), dim3(T_, (unsigned)H), dim3(256), 0, \
      stream, (const T*)q.data_ptr(), (const T*)pool.data_ptr(), (const T*)pooled.data_ptr(), (float)scale,       \
      (int)window, (int)P, (int)rpp, tok_req.data_ptr<int>(), tok_pos.data_ptr<int>(), tables.data_ptr<int>(),    \
      (int)tables.size(1), (int)bs, (T*)out.data_ptr(), (long)out.stride(0), (int)out_col, (float)out_scale,      \
      (int)H, (int)G, (int)D, (int)V))
  if (wide <= WAVE) PW_LAUNCH(1);
  else if (wide <= 2 * WAVE) PW_LAUNCH(2);
  else if (wide <= 4 * WAVE) PW_LAUNCH(4);
  else PW_LAUNCH(8);
#undef PW_LAUNCH
}
