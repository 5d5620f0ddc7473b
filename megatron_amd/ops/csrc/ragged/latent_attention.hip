// Latent-cache attention over ragged batches: cache-row store (RMS-normed
// latent + rotated shared key part), query assembly (absorbed part + rotated
// part) and causal attention with a softmax sink over the paged pool.
#include "ragged_common.h"

// ---------------------------------------------------------------------------
// cache row of each token: [rms(c) * w | rope(k_rot)]
// ---------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void latent_kv_store_kernel(
    const T* __restrict__ dkv, long stride, const float* __restrict__ w, float eps, const float* __restrict__ cosv,
    const float* __restrict__ sinv, int rot_dims, int rank, int rd, T* __restrict__ pool,
    const int* __restrict__ tok_pos, const long* __restrict__ tok_row) {
  __shared__ float red[256 / WAVE];
  const long t = blockIdx.x;
  const T* x = dkv + t * stride;
  T* dst = pool + tok_row[t] * (long)(rank + rd);
  float ss = 0.f;
  for (int c = threadIdx.x; c < rank; c += 256) {
    const float v = ldf(x + c);
    ss += v * v;
  }
  const float rs = rsqrtf(block_reduce_sum<256>(ss, red) / (float)rank + eps);
  for (int c = threadIdx.x; c < rank; c += 256) stf(dst + c, ldf(x + c) * rs * w[c]);
  const int half = rot_dims / 2;
  const long p = tok_pos[t];
  for (int i = threadIdx.x; i < rd; i += 256) {
    float v;
    if (i < rot_dims) {
      const int j = (i < half) ? i : i - half;
      const float cs = cosv[p * half + j], sn = sinv[p * half + j];
      const float a = ldf(x + rank + j), b = ldf(x + rank + j + half);
      v = (i < half) ? (a * cs - b * sn) : (b * cs + a * sn);
    } else {
      v = ldf(x + rank + i);
    }
    stf(dst + rank + i, v);
  }
}

void latent_kv_store(torch::Tensor dkv, torch::Tensor w, double eps, torch::Tensor cosv, torch::Tensor sinv,
                     int64_t rot_dims, int64_t rank, torch::Tensor pool, torch::Tensor tok_pos,
                     torch::Tensor tok_row) {
  TORCH_CHECK(dkv.is_cuda() && dkv.dim() == 2 && dkv.stride(1) == 1);
  check_f32(w, "w"); check_f32(cosv, "cos"); check_f32(sinv, "sin"); check_i32(tok_pos, "tok_pos");
  TORCH_CHECK(tok_row.is_cuda() && tok_row.scalar_type() == at::kLong && tok_row.is_contiguous());
  const int T_ = dkv.size(0);
  const int rd = dkv.size(1) - rank;
  TORCH_CHECK(rd >= 0 && rot_dims <= rd && rot_dims % 2 == 0 && w.numel() == rank);
  TORCH_CHECK(pool.is_contiguous() && pool.dim() == 2 && pool.size(1) == rank + rd &&
              pool.scalar_type() == dkv.scalar_type());
  TORCH_CHECK(cosv.dim() == 2 && cosv.size(1) == rot_dims / 2 && sinv.sizes() == cosv.sizes());
  TORCH_CHECK(tok_pos.numel() == T_ && tok_row.numel() == T_);
  if (T_ == 0) return;
  auto stream = at::cuda::getCurrentHIPStream();
  RAGGED_DISPATCH(dkv, hipLaunchKernelGGL((latent_kv_store_kernel<T>), dim3(T_), dim3(256), 0, stream,
      (const T*)dkv.data_ptr(), (long)dkv.stride(0), w.data_ptr<float>(), (float)eps, cosv.data_ptr<float>(),
      sinv.data_ptr<float>(), (int)rot_dims, (int)rank, rd, (T*)pool.data_ptr(), tok_pos.data_ptr<int>(),
      tok_row.data_ptr<long>()));
}

// ---------------------------------------------------------------------------
// query rows: [q_abs (rank) | rope(q_rot) (rd)] per (token, head)
// ---------------------------------------------------------------------------
template <typename T>
__global__ void assemble_q_kernel(const T* __restrict__ qa, long as_t, long as_h, const T* __restrict__ qr,
                                  long rs_t, long rs_h, const float* __restrict__ cosv,
                                  const float* __restrict__ sinv, int rot_dims, const int* __restrict__ tok_pos,
                                  T* __restrict__ out, int H, int rank, int rd) {
  const long t = blockIdx.x;
  const int hd = blockIdx.y;
  const int Dk = rank + rd, half = rot_dims / 2;
  const long p = tok_pos[t];
  const T* a = qa + t * as_t + hd * as_h;
  const T* x = qr + t * rs_t + hd * rs_h;
  T* dst = out + (t * H + hd) * Dk;
  for (int d = threadIdx.x; d < Dk; d += blockDim.x) {
    float v;
    if (d < rank) {
      v = ldf(a + d);
    } else {
      const int e = d - rank;
      if (e < rot_dims) {
        const int j = (e < half) ? e : e - half;
        const float cs = cosv[p * half + j], sn = sinv[p * half + j];
        const float u = ldf(x + j), w = ldf(x + j + half);
        v = (e < half) ? (u * cs - w * sn) : (w * cs + u * sn);
      } else {
        v = ldf(x + e);
      }
    }
    stf(dst + d, v);
  }
}

torch::Tensor assemble_latent_q(torch::Tensor qa, torch::Tensor qr, torch::Tensor cosv, torch::Tensor sinv,
                                int64_t rot_dims, torch::Tensor tok_pos) {
  TORCH_CHECK(qa.is_cuda() && qa.dim() == 3 && qa.stride(2) == 1 && qr.dim() == 3 && qr.stride(2) == 1);
  TORCH_CHECK(qa.size(0) == qr.size(0) && qa.size(1) == qr.size(1) && qa.scalar_type() == qr.scalar_type());
  check_f32(cosv, "cos"); check_f32(sinv, "sin"); check_i32(tok_pos, "tok_pos");
  const int T_ = qa.size(0), H = qa.size(1), rank = qa.size(2), rd = qr.size(2);
  TORCH_CHECK(rot_dims <= rd && rot_dims % 2 == 0 && cosv.size(1) == rot_dims / 2 && tok_pos.numel() == T_);
  auto out = torch::empty({T_, H, rank + rd}, qa.options());
  if (T_ == 0) return out;
  auto stream = at::cuda::getCurrentHIPStream();
  RAGGED_DISPATCH(qa, hipLaunchKernelGGL((assemble_q_kernel<T>), dim3(T_, H), dim3(128), 0, stream,
      (const T*)qa.data_ptr(), (long)qa.stride(0), (long)qa.stride(1), (const T*)qr.data_ptr(),
      (long)qr.stride(0), (long)qr.stride(1), cosv.data_ptr<float>(), sinv.data_ptr<float>(), (int)rot_dims,
      tok_pos.data_ptr<int>(), (T*)out.data_ptr(), H, rank, rd));
  return out;
}

// ---------------------------------------------------------------------------
// attention with sink.  Workgroup = (token, head), 4 waves; a wave scores one
// cached row at a time (lanes split the row, shuffle-reduce the dot product),
// keeps an online softmax and the weighted sum of the row's latent part in
// registers; the waves' partial results and the sink logit merge through LDS.
// ---------------------------------------------------------------------------
template <typename T, int MAXI>
__global__ __launch_bounds__(256) void latent_attn_kernel(
    const T* __restrict__ q, const T* __restrict__ pool, const float* __restrict__ sink, float scale,
    const int* __restrict__ tok_req, const int* __restrict__ tok_pos, const int* __restrict__ tables, int maxb,
    int bs, T* __restrict__ out, int Tn, int H, int Dk, int rank) {
  __shared__ float s_m[4], s_l[4];
  __shared__ float s_acc[4][MAXI * WAVE];
  const int t = blockIdx.x, hd = blockIdx.y;
  const int wave = threadIdx.x / WAVE, lane = threadIdx.x % WAVE;
  float qv[MAXI], acc[MAXI];
  const T* qp = q + ((long)t * H + hd) * Dk;
#pragma unroll
  for (int i = 0; i < MAXI; ++i) {
    const int d = lane + WAVE * i;
    qv[i] = (d < Dk) ? ldf(qp + d) : 0.f;
    acc[i] = 0.f;
  }
  const int p = tok_pos[t];
  const int* tab = tables + (long)tok_req[t] * maxb;
  float m = -INFINITY, l = 0.f;
  for (int j = wave; j <= p; j += 4) {
    const T* kr = pool + ((long)tab[j / bs] * bs + (j % bs)) * Dk;
    float kv[MAXI];
    float dot = 0.f;
#pragma unroll
    for (int i = 0; i < MAXI; ++i) {
      const int d = lane + WAVE * i;
      kv[i] = (d < Dk) ? ldf(kr + d) : 0.f;
      dot += kv[i] * qv[i];
    }
    dot = wave_reduce_sum(dot) * scale;
    const float mn = fmaxf(m, dot);
    const float corr = expf(m - mn), pj = expf(dot - mn);
    l = l * corr + pj;
#pragma unroll
    for (int i = 0; i < MAXI; ++i) acc[i] = acc[i] * corr + pj * kv[i];
    m = mn;
  }
  if (lane == 0) {
    s_m[wave] = m;
    s_l[wave] = l;
  }
#pragma unroll
  for (int i = 0; i < MAXI; ++i) s_acc[wave][lane + WAVE * i] = acc[i];
  __syncthreads();
  const float sk = sink[hd];
  float M = sk;
#pragma unroll
  for (int w = 0; w < 4; ++w) M = fmaxf(M, s_m[w]);
  float L = expf(sk - M);
  float f[4];
#pragma unroll
  for (int w = 0; w < 4; ++w) {
    f[w] = (s_m[w] == -INFINITY) ? 0.f : expf(s_m[w] - M);
    L += s_l[w] * f[w];
  }
  T* op = out + ((long)hd * Tn + t) * rank;
  for (int d = threadIdx.x; d < rank; d += 256) {
    float a = 0.f;
#pragma unroll
    for (int w = 0; w < 4; ++w) a += s_acc[w][d] * f[w];
    stf(op + d, a / L);
  }
}

torch::Tensor latent_sink_attention(torch::Tensor q, torch::Tensor pool, int64_t rank, torch::Tensor sink,
                                    double scale, torch::Tensor tok_req, torch::Tensor tok_pos,
                                    torch::Tensor tables, int64_t bs) {
  TORCH_CHECK(q.is_cuda() && q.dim() == 3 && q.is_contiguous());
  TORCH_CHECK(pool.is_contiguous() && pool.dim() == 2 && pool.scalar_type() == q.scalar_type());
  check_f32(sink, "sink"); check_i32(tok_req, "tok_req"); check_i32(tok_pos, "tok_pos"); check_i32(tables, "tables");
  const int T_ = q.size(0), H = q.size(1), Dk = q.size(2);
  TORCH_CHECK(pool.size(1) == Dk && rank <= Dk && sink.numel() == H && tok_req.numel() == T_ && tok_pos.numel() == T_);
  TORCH_CHECK(tables.dim() == 2 && bs > 0 && pool.size(0) % bs == 0);
  TORCH_CHECK(Dk <= 10 * WAVE, "latent row wider than ", 10 * WAVE);
  // [H, T, rank] so the per-head value up-projection is a plain batched GEMM
  auto out = torch::empty({H, T_, rank}, q.options());
  if (T_ == 0) return out.transpose(0, 1);
  auto stream = at::cuda::getCurrentHIPStream();
  const int maxb = tables.size(1);
#define LAUNCH_ATTN(MAXI)                                                                                   \
  RAGGED_DISPATCH(q, hipLaunchKernelGGL((latent_attn_kernel<T, MAXI>), dim3(T_, H), dim3(256), 0, stream,   \
      (const T*)q.data_ptr(), (const T*)pool.data_ptr(), sink.data_ptr<float>(), (float)scale,               \
      tok_req.data_ptr<int>(), tok_pos.data_ptr<int>(), tables.data_ptr<int>(), maxb, (int)bs,               \
      (T*)out.data_ptr(), T_, H, Dk, (int)rank))
  if (Dk <= 3 * WAVE) LAUNCH_ATTN(3);
  else if (Dk <= 5 * WAVE) LAUNCH_ATTN(5);
  else LAUNCH_ATTN(10);
#undef LAUNCH_ATTN
  return out.transpose(0, 1);
}
