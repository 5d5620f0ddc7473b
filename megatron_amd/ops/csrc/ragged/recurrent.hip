// Recurrent mixers over ragged batches with per-request fp32 state slots:
// minGRU (elementwise gated recurrence) and mLSTM (matrix memory with the
// running-maximum stabiliser).  A request's new tokens are walked in order by
// the workgroups that own its state; requests, channels, heads and value
// columns run in parallel.
#include "ragged_common.h"

// ---------------------------------------------------------------------------
// minGRU: S <- (1 - z) S + z cand ; out = S * silu(g)
// ---------------------------------------------------------------------------
template <typename T>
__global__ void mingru_kernel(const T* __restrict__ zxg, long stride, const float* __restrict__ bz,
                              const float* __restrict__ bx, float* __restrict__ state,
                              const int* __restrict__ cu, const int* __restrict__ slots,
                              T* __restrict__ out, int C) {
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  if (c >= C) return;
  const int r = blockIdx.y;
  const int t0 = cu[r], t1 = cu[r + 1];
  float* sp = state + (long)slots[r] * C + c;
  float S = *sp;
  const float bzc = bz[c], bxc = bx[c];
#pragma unroll 4
  for (int t = t0; t < t1; ++t) {
    const T* row = zxg + (long)t * stride;
    const float z = sigmoidf_(ldf(row + c) + bzc);
    const float u = ldf(row + C + c) + bxc;
    const float g = ldf(row + 2 * C + c);
    const float cand = (u >= 0.f) ? (u + 0.5f) : sigmoidf_(u);
    S = (1.f - z) * S + z * cand;
    stf(out + (long)t * C + c, S * (g * sigmoidf_(g)));
  }
  *sp = S;
}

torch::Tensor mingru_scan(torch::Tensor zxg, torch::Tensor bz, torch::Tensor bx, torch::Tensor state,
                          torch::Tensor cu, torch::Tensor slots) {
  TORCH_CHECK(zxg.is_cuda() && zxg.dim() == 2 && zxg.stride(1) == 1 && zxg.size(1) % 3 == 0);
  check_f32(bz, "bz"); check_f32(bx, "bx"); check_f32(state, "state");
  check_i32(cu, "cu"); check_i32(slots, "slots");
  const int T_ = zxg.size(0), C = zxg.size(1) / 3, R = slots.numel();
  TORCH_CHECK(bz.numel() == C && bx.numel() == C && state.dim() == 2 && state.size(1) == C && cu.numel() == R + 1);
  auto out = torch::empty({T_, C}, zxg.options());
  if (T_ == 0 || R == 0) return out;
  auto stream = at::cuda::getCurrentHIPStream();
  RAGGED_DISPATCH(zxg, hipLaunchKernelGGL((mingru_kernel<T>), dim3((C + 63) / 64, R), dim3(64), 0, stream,
      (const T*)zxg.data_ptr(), (long)zxg.stride(0), bz.data_ptr<float>(), bx.data_ptr<float>(),
      state.data_ptr<float>(), cu.data_ptr<int>(), slots.data_ptr<int>(), (T*)out.data_ptr(), C));
  return out;
}

// ---------------------------------------------------------------------------
// mLSTM.  Workgroup = (request, head, tile of VT value columns); 256 threads as
// RG row groups x VT columns, each thread holding the rows {rg, rg+RG, ...} of
// its column of S in registers (and the matching rows of n, redundantly per
// column).  Per token: q, k, the v tile and the two log gates are staged in
// LDS, the state is decayed and updated in registers, and S^T q / n.q are
// reduced over row groups through LDS.
// ---------------------------------------------------------------------------
constexpr int ML_VT = 16, ML_RG = 16, ML_RPT = 16;   // dim <= RG * RPT = 256
constexpr int ML_CH = 16;                             // tokens staged per chunk

// Tokens are taken in chunks of ML_CH: q, k, the v tile and the gate
// pre-activations of a whole chunk are loaded at once (one global latency per
// chunk instead of one per token), the capped log gates are evaluated in
// parallel (one thread per token) and the scalar stabiliser chain m, e^{f+m-m'},
// e^{i-m'}, e^{-m'} is run once by one thread; the serial loop over the chunk
// then only does the state update and the two reductions, with one barrier per
// token (the reduction buffer is double-buffered).
template <typename T>
__global__ __launch_bounds__(256) void mlstm_kernel(
    const T* __restrict__ qkvg, long stride, const float* __restrict__ gates, const float* __restrict__ bi,
    const float* __restrict__ bfg, float* __restrict__ stS, float* __restrict__ stn, float* __restrict__ stm,
    const int* __restrict__ cu, const int* __restrict__ slots, float* __restrict__ o, int H, int D, int V,
    float cap) {
  __shared__ float sq[ML_CH][ML_RG * ML_RPT], sk[ML_CH][ML_RG * ML_RPT], sv[ML_CH][ML_VT];
  __shared__ float s_ig[ML_CH], s_fg[ML_CH], s_da[ML_CH], s_db[ML_CH], s_em[ML_CH], s_m;
  __shared__ float red[2][ML_RG][ML_VT + 1];
  const int r = blockIdx.x, hd = blockIdx.y, vt = blockIdx.z;
  const int c = threadIdx.x % ML_VT, rg = threadIdx.x / ML_VT;
  const int col = vt * ML_VT + c;
  const bool colok = col < V;
  const long slot = slots[r];
  float S[ML_RPT], n[ML_RPT];
#pragma unroll
  for (int i = 0; i < ML_RPT; ++i) {
    const int row = rg + i * ML_RG;
    S[i] = (row < D && colok) ? stS[((slot * H + hd) * D + row) * V + col] : 0.f;
    n[i] = (row < D) ? stn[(slot * H + hd) * D + row] : 0.f;
  }
  if (threadIdx.x == 0) s_m = stm[slot * H + hd];
  const float qscale = 1.f / sqrtf((float)D);
  const float bih = bi[hd], bfh = bfg[hd];
  const int t0 = cu[r], t1 = cu[r + 1];
  int step = 0;
  for (int tc = t0; tc < t1; tc += ML_CH) {
    const int nc = min(ML_CH, t1 - tc);
    if ((int)threadIdx.x < D) {                  // D <= 256 = blockDim: one q and one k element per thread and token
#pragma unroll 4
      for (int tt = 0; tt < nc; ++tt) {
        const T* row = qkvg + (long)(tc + tt) * stride;
        sq[tt][threadIdx.x] = ldf(row + hd * D + threadIdx.x) * qscale;
        sk[tt][threadIdx.x] = ldf(row + (long)H * D + hd * D + threadIdx.x);
      }
    }
    {
      const int tt = threadIdx.x / ML_VT, cc = vt * ML_VT + threadIdx.x % ML_VT;   // 16 x 16 = 256 threads
      if (tt < nc) sv[tt][threadIdx.x % ML_VT] = (cc < V) ? ldf(qkvg + (long)(tc + tt) * stride + 2L * H * D + (long)hd * V + cc) : 0.f;
    }
    if ((int)threadIdx.x < nc) {
      const long t = tc + threadIdx.x;
      s_ig[threadIdx.x] = cap * tanhf((gates[t * 2 * H + hd] + bih) / cap);
      const float fc = cap * tanhf((gates[t * 2 * H + H + hd] + bfh) / cap);
      s_fg[threadIdx.x] = -softplusf_(-fc);      // log sigmoid
    }
    __syncthreads();
    if (threadIdx.x == 0) {
      float mm = s_m;
      for (int tt = 0; tt < nc; ++tt) {
        const float mn = fmaxf(s_fg[tt] + mm, s_ig[tt]);
        s_da[tt] = expf(s_fg[tt] + mm - mn);
        s_db[tt] = expf(s_ig[tt] - mn);
        s_em[tt] = expf(-mn);
        mm = mn;
      }
      s_m = mm;
    }
    __syncthreads();
    for (int tt = 0; tt < nc; ++tt, ++step) {
      const float da = s_da[tt], db = s_db[tt], vv = sv[tt][c];
      float part = 0.f, npart = 0.f;
#pragma unroll
      for (int i = 0; i < ML_RPT; ++i) {
        const int rr = rg + i * ML_RG;
        if (rr < D) {
          const float kk = sk[tt][rr], qq = sq[tt][rr];
          S[i] = da * S[i] + db * kk * vv;
          n[i] = da * n[i] + db * kk;
          part += S[i] * qq;
          npart += n[i] * qq;
        }
      }
      float(*rb)[ML_VT + 1] = red[step & 1];
      rb[rg][c] = part;
      if (c == 0) rb[rg][ML_VT] = npart;
      __syncthreads();
      if (rg == 0 && colok) {
        float num = 0.f, nq = 0.f;
#pragma unroll
        for (int g = 0; g < ML_RG; ++g) {
          num += rb[g][c];
          nq += rb[g][ML_VT];
        }
        o[((long)(tc + tt) * H + hd) * V + col] = num / (fmaxf(fabsf(nq), s_em[tt]) + 1e-6f);
      }
    }
    __syncthreads();                             // the chunk buffers are rewritten next
  }
#pragma unroll
  for (int i = 0; i < ML_RPT; ++i) {
    const int row = rg + i * ML_RG;
    if (row < D) {
      if (colok) stS[((slot * H + hd) * D + row) * V + col] = S[i];
      if (vt == 0 && c == 0) stn[(slot * H + hd) * D + row] = n[i];
    }
  }
  if (vt == 0 && threadIdx.x == 0) stm[slot * H + hd] = s_m;
}

// per-head RMS norm of o, learned weight, sigmoid output gate; one wave per (token, head)
template <typename T>
__global__ __launch_bounds__(256) void mlstm_out_kernel(const float* __restrict__ o, const T* __restrict__ qkvg,
                                                        long stride, long g_off, const float* __restrict__ w,
                                                        float eps, T* __restrict__ out, int TH, int H, int V) {
  const int wid = blockIdx.x * (256 / WAVE) + threadIdx.x / WAVE;
  const int lane = threadIdx.x % WAVE;
  if (wid >= TH) return;
  const int t = wid / H, hd = wid % H;
  const float* op = o + (long)wid * V;
  float ss = 0.f;
  for (int v = lane; v < V; v += WAVE) ss += op[v] * op[v];
  const float rs = rsqrtf(wave_reduce_sum(ss) / (float)V + eps);
  const T* gp = qkvg + (long)t * stride + g_off + (long)hd * V;
  for (int v = lane; v < V; v += WAVE)
    stf(out + (long)wid * V + v, op[v] * rs * w[hd * V + v] * sigmoidf_(ldf(gp + v)));
}

torch::Tensor mlstm_scan(torch::Tensor qkvg, torch::Tensor gates, torch::Tensor bi, torch::Tensor bfg,
                         torch::Tensor norm_w, int64_t H, int64_t D, int64_t V, double cap, double eps,
                         torch::Tensor stS, torch::Tensor stn, torch::Tensor stm, torch::Tensor cu,
                         torch::Tensor slots) {
  TORCH_CHECK(qkvg.is_cuda() && qkvg.dim() == 2 && qkvg.stride(1) == 1);
  TORCH_CHECK(qkvg.size(1) == 2 * H * D + 2 * H * V, "fused projection width");
  TORCH_CHECK(D <= ML_RG * ML_RPT, "mlstm head dim above ", ML_RG * ML_RPT);
  check_f32(gates, "gates"); check_f32(bi, "bias_i"); check_f32(bfg, "bias_f"); check_f32(norm_w, "norm_w");
  check_f32(stS, "S"); check_f32(stn, "n"); check_f32(stm, "m"); check_i32(cu, "cu"); check_i32(slots, "slots");
  const int T_ = qkvg.size(0), R = slots.numel();
  TORCH_CHECK(gates.dim() == 2 && gates.size(0) == T_ && gates.size(1) == 2 * H);
  TORCH_CHECK(bi.numel() == H && bfg.numel() == H && norm_w.numel() == H * V && cu.numel() == R + 1);
  TORCH_CHECK(stS.dim() == 4 && stS.size(1) == H && stS.size(2) == D && stS.size(3) == V);
  TORCH_CHECK(stn.numel() == stS.size(0) * H * D && stm.numel() == stS.size(0) * H);
  auto out = torch::empty({T_, H * V}, qkvg.options());
  if (T_ == 0 || R == 0) return out;
  auto o = torch::empty({T_, H, V}, qkvg.options().dtype(at::kFloat));
  auto stream = at::cuda::getCurrentHIPStream();
  const dim3 grid(R, H, (V + ML_VT - 1) / ML_VT);
  RAGGED_DISPATCH(qkvg, {
    hipLaunchKernelGGL((mlstm_kernel<T>), grid, dim3(256), 0, stream, (const T*)qkvg.data_ptr(),
        (long)qkvg.stride(0), gates.data_ptr<float>(), bi.data_ptr<float>(), bfg.data_ptr<float>(),
        stS.data_ptr<float>(), stn.data_ptr<float>(), stm.data_ptr<float>(), cu.data_ptr<int>(),
        slots.data_ptr<int>(), o.data_ptr<float>(), (int)H, (int)D, (int)V, (float)cap);
    const int TH = T_ * H;
    hipLaunchKernelGGL((mlstm_out_kernel<T>), dim3((TH + 3) / 4), dim3(256), 0, stream, o.data_ptr<float>(),
        (const T*)qkvg.data_ptr(), (long)qkvg.stride(0), (long)(2 * H * D + H * V), norm_w.data_ptr<float>(),
        (float)eps, (T*)out.data_ptr(), TH, (int)H, (int)V);
  });
  return out;
}
