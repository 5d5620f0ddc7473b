// Generalized delta rule over ragged batches with a per-request fp32 state:
//   S <- diag(w) S - (a u)(u^T S) + k v^T ,  o = S^T r      (per head; both terms read the old S)
//   w = exp(-e^{-1/2} sigmoid(W2 tanh(b) + w0)),  a = sigmoid(a_pre + a_b),  u = k / sqrt(sum k^2 + 1e-6)
// The update is independent per value column: S[:, c] needs u . S[:, c] and
// r . S[:, c] only.  Workgroup = (request, head, tile of 64 value columns), four
// waves of 16 columns x 4 row groups.  A request's new tokens are walked in
// order; operands are staged in LDS a chunk of tokens at a time, where all the
// non-linearities are evaluated in parallel.
#include "../ragged/ragged_common.h"

constexpr int DR_COLS = 64;          // value columns per workgroup
constexpr int DR_RG = 4;             // row groups: a column's rows are dealt to 4 lanes of one wave
constexpr int DR_NT = DR_COLS * DR_RG;
constexpr int DR_MAX_RANK = 128;     // decay bottleneck

// x summed over the four 16-lane rows of a wave, in every lane: two register
// swaps between lane halves / neighbouring rows (VALU, no LDS round trip) and two adds
__device__ __forceinline__ float sum_row_groups(float x) {
  const int xi = __float_as_int(x);
  auto a = __builtin_amdgcn_permlane32_swap(xi, xi, false, false);      // lanes l and l ^ 32 exchanged
  const float y = __int_as_float(a[0]) + __int_as_float(a[1]);
  const int yi = __float_as_int(y);
  auto b = __builtin_amdgcn_permlane16_swap(yi, yi, false, false);      // rows r and r ^ 1 exchanged
  return __int_as_float(b[0]) + __int_as_float(b[1]);
}

// Thread mapping: wave w holds columns 16 w .. 16 w + 15 of the tile; inside a
// wave lane = rg * 16 + c, so the four partial sums of a column sit in lanes
// c, c + 16, c + 32, c + 48 and are reduced with two register swaps: the token loop
// has no barrier.  Thread (column, rg) keeps rows rg * RPT .. rg * RPT + RPT - 1
// of its column in registers.
template <typename T, int DMAX, int CH>
__global__ __launch_bounds__(DR_NT) void delta_rule_kernel(
    const T* __restrict__ proj, long stride, int r_off, int k_off, int v_off, int a_off, int w_off, int rank,
    const float* __restrict__ w2, const float* __restrict__ w0, const float* __restrict__ a_b,
    float* __restrict__ state, const int* __restrict__ cu, const int* __restrict__ slots, float* __restrict__ o,
    int H, int D, int w2_in_lds) {
  constexpr int RPT = DMAX / DR_RG;
  __shared__ __align__(16) float s_r[CH][DMAX], s_k[CH][DMAX], s_u[CH][DMAX], s_au[CH][DMAX], s_w[CH][DMAX];
  __shared__ float s_v[CH][DR_COLS], s_b[CH][DR_MAX_RANK], s_inv[CH];
  extern __shared__ float s_w2[];                  // [rank][D] (transposed), when it fits
  const int r = blockIdx.x, hd = blockIdx.y, ct = blockIdx.z;
  const int wave = threadIdx.x / WAVE, lane = threadIdx.x % WAVE;
  const int c = wave * 16 + (lane & 15), rg = lane >> 4;
  const int col = ct * DR_COLS + c;
  const bool colok = col < D;
  const long slot = slots[r];
  float* sp = state + ((slot * H + hd) * D) * (long)D;
  float S[RPT];
#pragma unroll
  for (int i = 0; i < RPT; ++i) {
    const int row = rg * RPT + i;
    S[i] = (row < D && colok) ? sp[(long)row * D + col] : 0.f;
  }
  // rows D .. DMAX-1 of the operand buffers are read by the token loop (against zero state): keep them zero
  for (int i = threadIdx.x; i < CH * DMAX; i += DR_NT) {
    (&s_r[0][0])[i] = 0.f; (&s_k[0][0])[i] = 0.f; (&s_u[0][0])[i] = 0.f; (&s_au[0][0])[i] = 0.f; (&s_w[0][0])[i] = 0.f;
  }
  if (w2_in_lds)
    for (int i = threadIdx.x; i < D * rank; i += DR_NT) s_w2[(i % rank) * D + i / rank] = w2[(long)hd * D * rank + i];
  __syncthreads();
  const int t0 = cu[r], t1 = cu[r + 1];
  const float decay_c = -0.60653065971263342f;     // -e^{-1/2}
  for (int tc = t0; tc < t1; tc += CH) {
    const int nc = min(CH, t1 - tc);
    for (int i = threadIdx.x; i < nc * rank; i += DR_NT) {
      const int tt = i / rank, j = i % rank;
      s_b[tt][j] = tanhf(ldf(proj + (long)(tc + tt) * stride + w_off + j));
    }
    for (int i = threadIdx.x; i < nc * DR_COLS; i += DR_NT) {
      const int tt = i / DR_COLS, cc = ct * DR_COLS + i % DR_COLS;
      s_v[tt][i % DR_COLS] = (cc < D) ? ldf(proj + (long)(tc + tt) * stride + v_off + hd * D + cc) : 0.f;
    }
    __syncthreads();
    for (int i = threadIdx.x; i < nc * D; i += DR_NT) {
      const int tt = i / D, d = i % D, ch = hd * D + d;
      const T* row = proj + (long)(tc + tt) * stride;
      s_r[tt][d] = ldf(row + r_off + ch);
      s_k[tt][d] = ldf(row + k_off + ch);
      float z = w0[ch];
      if (w2_in_lds) {
        for (int j = 0; j < rank; ++j) z += s_w2[j * D + d] * s_b[tt][j];
      } else {
        const float* w2r = w2 + (long)ch * rank;
        for (int j = 0; j < rank; ++j) z += w2r[j] * s_b[tt][j];
      }
      s_w[tt][d] = expf(decay_c * sigmoidf_(z));
      s_au[tt][d] = sigmoidf_(ldf(row + a_off + ch) + a_b[ch]);          // a for now, a * u below
    }
    __syncthreads();
    for (int tt = wave; tt < nc; tt += DR_NT / WAVE) {   // one wave per token: squared norm of the key
      float ss = 0.f;
      for (int d = lane; d < D; d += WAVE) ss += s_k[tt][d] * s_k[tt][d];
      ss = wave_reduce_sum(ss);
      if (lane == 0) s_inv[tt] = 1.f / sqrtf(ss + 1e-6f);
    }
    __syncthreads();
    for (int i = threadIdx.x; i < nc * D; i += DR_NT) {
      const int tt = i / D, d = i % D;
      const float u = s_k[tt][d] * s_inv[tt];
      s_u[tt][d] = u;
      s_au[tt][d] *= u;
    }
    __syncthreads();
#pragma unroll 2
    for (int tt = 0; tt < nc; ++tt) {
      const float vv = s_v[tt][c];
      const float* pu = &s_u[tt][rg * RPT];
      const float* pw = &s_w[tt][rg * RPT];
      const float* pa = &s_au[tt][rg * RPT];
      const float* pk = &s_k[tt][rg * RPT];
      const float* pr = &s_r[tt][rg * RPT];
      float d0 = 0.f, d1 = 0.f, d2 = 0.f, d3 = 0.f;
#pragma unroll
      for (int i = 0; i < RPT; i += 4) {
        d0 += pu[i] * S[i]; d1 += pu[i + 1] * S[i + 1]; d2 += pu[i + 2] * S[i + 2]; d3 += pu[i + 3] * S[i + 3];
      }
      const float dot = sum_row_groups((d0 + d1) + (d2 + d3));
      float p0 = 0.f, p1 = 0.f, p2 = 0.f, p3 = 0.f;
#pragma unroll
      for (int i = 0; i < RPT; i += 4) {
        S[i] = pw[i] * S[i] - pa[i] * dot + pk[i] * vv;
        S[i + 1] = pw[i + 1] * S[i + 1] - pa[i + 1] * dot + pk[i + 1] * vv;
        S[i + 2] = pw[i + 2] * S[i + 2] - pa[i + 2] * dot + pk[i + 2] * vv;
        S[i + 3] = pw[i + 3] * S[i + 3] - pa[i + 3] * dot + pk[i + 3] * vv;
        p0 += pr[i] * S[i]; p1 += pr[i + 1] * S[i + 1]; p2 += pr[i + 2] * S[i + 2]; p3 += pr[i + 3] * S[i + 3];
      }
      const float part = sum_row_groups((p0 + p1) + (p2 + p3));
      if (rg == 0 && colok) o[((long)(tc + tt) * H + hd) * D + col] = part;
    }
    __syncthreads();                                // the chunk buffers are rewritten next
  }
#pragma unroll
  for (int i = 0; i < RPT; ++i) {
    const int row = rg * RPT + i;
    if (row < D && colok) sp[(long)row * D + col] = S[i];
  }
}

// per-head RMS norm of o, learned weight, sigmoid output gate, output scale; one wave per (token, head)
template <typename T>
__global__ __launch_bounds__(256) void delta_out_kernel(const float* __restrict__ o, const T* __restrict__ proj,
                                                        long stride, int g_off, const float* __restrict__ w,
                                                        float eps, T* __restrict__ out, long out_stride, int out_col,
                                                        float out_scale, int TH, int H, int D) {
  const int wid = blockIdx.x * (256 / WAVE) + threadIdx.x / WAVE;
  const int lane = threadIdx.x % WAVE;
  if (wid >= TH) return;
  const int t = wid / H, hd = wid % H;
  const float* op = o + (long)wid * D;
  float ss = 0.f;
  for (int d = lane; d < D; d += WAVE) ss += op[d] * op[d];
  const float rs = 1.f / sqrtf(wave_reduce_sum(ss) / (float)D + eps);
  const T* gp = proj + (long)t * stride + g_off + (long)hd * D;
  T* dst = out + (long)t * out_stride + out_col + (long)hd * D;
  for (int d = lane; d < D; d += WAVE)
    stf(dst + d, op[d] * rs * w[hd * D + d] * sigmoidf_(ldf(gp + d)) * out_scale);
}

void delta_rule_scan(torch::Tensor proj, int64_t r_off, int64_t k_off, int64_t v_off, int64_t g_off, int64_t a_off,
                     int64_t w_off, int64_t rank, torch::Tensor w2, torch::Tensor w0, torch::Tensor a_b,
                     torch::Tensor norm_w, int64_t H, int64_t D, double eps, torch::Tensor state, torch::Tensor cu,
                     torch::Tensor slots, torch::Tensor out, int64_t out_col, double out_scale) {
  TORCH_CHECK(proj.is_cuda() && proj.dim() == 2 && proj.stride(1) == 1);
  check_f32(w2, "w2"); check_f32(w0, "w0"); check_f32(a_b, "a bias"); check_f32(norm_w, "norm"); check_f32(state, "S");
  check_i32(cu, "cu"); check_i32(slots, "slots");
  const int T_ = proj.size(0), C = proj.size(1), R = slots.numel();
  const long HD = H * D;
  for (int64_t off : {r_off, k_off, v_off, g_off, a_off}) TORCH_CHECK(off >= 0 && off + HD <= C, "column slice");
  TORCH_CHECK(w_off >= 0 && w_off + rank <= C && rank >= 1 && rank <= DR_MAX_RANK, "decay bottleneck above ", DR_MAX_RANK);
  TORCH_CHECK(w2.numel() == HD * rank && w0.numel() == HD && a_b.numel() == HD && norm_w.numel() == HD);
  TORCH_CHECK(state.dim() == 4 && state.size(1) == H && state.size(2) == D && state.size(3) == D && cu.numel() == R + 1);
  TORCH_CHECK(D <= 256, "delta-rule head dim above 256");
  TORCH_CHECK(out.is_cuda() && out.dim() == 2 && out.stride(1) == 1 && out.size(0) == T_ &&
              out.scalar_type() == proj.scalar_type() && out_col >= 0 && out_col + HD <= out.size(1));
  if (T_ == 0 || R == 0) return;
  auto o = torch::empty({T_, H, D}, proj.options().dtype(at::kFloat));
  auto stream = at::cuda::getCurrentHIPStream();
  const dim3 grid(R, (unsigned)H, (unsigned)((D + DR_COLS - 1) / DR_COLS));
  // the head's second decay matrix is kept in LDS (transposed) when it fits beside the operand buffers
  const size_t w2_bytes = (size_t)D * rank * sizeof(float);
  const int w2_in_lds = w2_bytes <= 16 * 1024;
  const size_t smem = w2_in_lds ? w2_bytes : 0;
#define DR_LAUNCH(DMAX, CH)                                                                                    \
  hipLaunchKernelGGL((delta_rule_kernel<T, DMAX, CH>), grid, dim3(DR_NT), smem, stream,                        \
      (const T*)proj.data_ptr(), (long)proj.stride(0), (int)r_off, (int)k_off, (int)v_off, (int)a_off,         \
      (int)w_off, (int)rank, w2.data_ptr<float>(), w0.data_ptr<float>(), a_b.data_ptr<float>(),                \
      state.data_ptr<float>(), cu.data_ptr<int>(), slots.data_ptr<int>(), o.data_ptr<float>(), (int)H, (int)D, \
      w2_in_lds)
  RAGGED_DISPATCH(proj, {
    if (D <= 64) DR_LAUNCH(64, 16);
    else if (D <= 128) DR_LAUNCH(128, 8);
    else DR_LAUNCH(256, 8);
    const int TH = T_ * H;
    hipLaunchKernelGGL((delta_out_kernel<T>), dim3((TH + 3) / 4), dim3(256), 0, stream, o.data_ptr<float>(),
        (const T*)proj.data_ptr(), (long)proj.stride(0), (int)g_off, norm_w.data_ptr<float>(), (float)eps,
        (T*)out.data_ptr(), (long)out.stride(0), (int)out_col, (float)out_scale, TH, (int)H, (int)D);
  });
#undef DR_LAUNCH
}
