// Generalized delta rule over ragged batches with a per-request fp32 state:
//   S <- diag(w) S - (a u)(u^T S) + k v^T ,  o = S^T r      (per head; both terms read the old S)
//   w = exp(-e^{-1/2} sigmoid(W2 tanh(b) + w0)),  a = sigmoid(a_pre + a_b),  u = k / sqrt(sum k^2 + 1e-6)
// Three kernels:
//   delta_prep_kernel   everything that does not depend on the state, in parallel over
//                       (token, head): r, k, u, a u, w as fp32 planes
//   delta_rule_kernel   the serial walk over a request's new tokens.  The update is
//                       independent per value column (S[:, c] needs u . S[:, c] and
//                       r . S[:, c] only): workgroup = (request, head, 16 value columns)
//   delta_out_kernel    per-head RMS norm, weight, sigmoid gate, output scale
#include "../ragged/ragged_common.h"

constexpr int DR_COLS = 16;          // value columns per workgroup
constexpr int DR_RG = 16;            // row groups: a column's rows are dealt to the 16 lanes of one wave row
constexpr int DR_CONS = DR_COLS * DR_RG;        // consumer threads (4 waves): the token loop
constexpr int DR_PW = 4;             // producer waves
constexpr int DR_CH = 8;             // tokens per chunk
constexpr int DR_MAX_RANK = 128;     // decay bottleneck
constexpr int DP_TOK = 16;           // tokens per workgroup of the prep kernel (4 per wave)

// x summed over the 16 lanes of its wave row, in every lane: four rotations inside
// the row (DPP modifiers of the adds: VALU only, nothing passes through LDS)
__device__ __forceinline__ float sum_row(float x) {
  x += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(x), 0x128, 0xf, 0xf, false));   // row_ror:8
  x += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(x), 0x124, 0xf, 0xf, false));   // row_ror:4
  x += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(x), 0x122, 0xf, 0xf, false));   // row_ror:2
  x += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(x), 0x121, 0xf, 0xf, false));   // row_ror:1
  return x;
}

__device__ __forceinline__ float lane_value(float x, int src_lane) {     // src_lane is wave-uniform
  return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(x), src_lane));
}

// ---------------------------------------------------------------------------
// operands of the recurrence.  One wave per (token, head), lanes over the
// channels; the head's second decay matrix sits in LDS (transposed) when it
// fits, the bottleneck's tanh values pass between lanes in registers.
// planes: [5][T][H][D] fp32 = r, k, u, a u, w
// ---------------------------------------------------------------------------
template <typename T, int EPL>
__global__ __launch_bounds__(256) void delta_prep_kernel(
    const T* __restrict__ proj, long stride, int r_off, int k_off, int a_off, int w_off, int rank,
    const float* __restrict__ w2, const float* __restrict__ w0, const float* __restrict__ a_b,
    float* __restrict__ planes, int Tn, int H, int D, int w2_in_lds) {
  extern __shared__ float s_w2[];                  // [rank][D]
  const int hd = blockIdx.y;
  const int wave = threadIdx.x / WAVE, lane = threadIdx.x % WAVE;
  if (w2_in_lds) {
    for (int i = threadIdx.x; i < D * rank; i += 256) s_w2[(i % rank) * D + i / rank] = w2[(long)hd * D * rank + i];
    __syncthreads();
  }
  const float decay_c = -0.60653065971263342f;     // -e^{-1/2}
  const long plane = (long)Tn * H * D;
  for (int ti = wave; ti < DP_TOK; ti += 4) {
    const long t = (long)blockIdx.x * DP_TOK + ti;
    if (t >= Tn) break;
    const T* row = proj + t * stride;
    const float tb0 = (lane < rank) ? tanhf(ldf(row + w_off + lane)) : 0.f;          // entry j in lane j % 64
    const float tb1 = (lane + WAVE < rank) ? tanhf(ldf(row + w_off + lane + WAVE)) : 0.f;
    float kk[EPL], rr[EPL], aa[EPL], zz[EPL];
    float ss = 0.f;
#pragma unroll
    for (int e = 0; e < EPL; ++e) {
      const int d = lane + WAVE * e;
      const bool ok = d < D;
      const int ch = hd * D + (ok ? d : 0);
      kk[e] = ok ? ldf(row + k_off + ch) : 0.f;
      rr[e] = ok ? ldf(row + r_off + ch) : 0.f;
      aa[e] = ok ? sigmoidf_(ldf(row + a_off + ch) + a_b[ch]) : 0.f;
      zz[e] = ok ? w0[ch] : 0.f;
      ss += kk[e] * kk[e];
    }
    const int r0 = min(rank, WAVE);
    for (int j = 0; j < r0; ++j) {
      const float tj = lane_value(tb0, j);
#pragma unroll
      for (int e = 0; e < EPL; ++e) {
        const int d = lane + WAVE * e;
        if (d < D) zz[e] += (w2_in_lds ? s_w2[j * D + d] : w2[(long)(hd * D + d) * rank + j]) * tj;
      }
    }
    for (int j = WAVE; j < rank; ++j) {
      const float tj = lane_value(tb1, j - WAVE);
#pragma unroll
      for (int e = 0; e < EPL; ++e) {
        const int d = lane + WAVE * e;
        if (d < D) zz[e] += (w2_in_lds ? s_w2[j * D + d] : w2[(long)(hd * D + d) * rank + j]) * tj;
      }
    }
    const float inv = 1.f / sqrtf(wave_reduce_sum(ss) + 1e-6f);
    float* dst = planes + (t * H + hd) * D;
#pragma unroll
    for (int e = 0; e < EPL; ++e) {
      const int d = lane + WAVE * e;
      if (d < D) {
        const float u = kk[e] * inv;
        dst[d] = rr[e];
        dst[plane + d] = kk[e];
        dst[2 * plane + d] = u;
        dst[3 * plane + d] = aa[e] * u;
        dst[4 * plane + d] = expf(decay_c * sigmoidf_(zz[e]));
      }
    }
  }
}

// ---------------------------------------------------------------------------
// the walk.  Waves with two roles.  Consumer waves 0-3 run the token loop: wave
// w holds columns 4 w .. 4 w + 3 of the tile; inside a wave lane = 16 cw + rg owns
// rows rg * RPT .. rg * RPT + RPT - 1 of column 4 w + cw in registers; the sixteen
// partial sums of a column sit in one wave row and are reduced in registers: the
// token loop has no barrier and a few dozen instructions per token.  Producer
// waves copy the operand rows of the NEXT chunk of tokens from the planes into
// the other half of a double buffer meanwhile (the reads of the chunk after
// next are already in flight).  One workgroup barrier per chunk.
// ---------------------------------------------------------------------------
template <typename T, int DMAX>
__global__ __launch_bounds__(DR_CONS + DR_PW * WAVE) void delta_rule_kernel(
    const float* __restrict__ planes, const T* __restrict__ proj, long stride, int v_off,
    float* __restrict__ state, const int* __restrict__ cu, const int* __restrict__ slots, float* __restrict__ o,
    int Tn, int H, int D) {
  constexpr int RPT = DMAX / DR_RG;
  constexpr int EPL = DMAX / WAVE;                 // channels per producer lane
  constexpr int CH = DR_CH, TPW = DR_CH / DR_PW;
  __shared__ __align__(16) float s_op[2][5][CH][DMAX];      // r, k, u, a u, w
  __shared__ float s_v[2][CH][DR_COLS];
  const int r = blockIdx.x, hd = blockIdx.y, ct = blockIdx.z;
  const int wave = threadIdx.x / WAVE, lane = threadIdx.x % WAVE;
  const bool producer = wave >= DR_CONS / WAVE;   // wave-uniform
  const int t0 = cu[r], t1 = cu[r + 1];
  const int nchunks = (t1 - t0 + CH - 1) / CH;
  const long plane = (long)Tn * H * D;

  // ---- producer: a wave owns tokens pw, pw + DR_PW, ... of a chunk; load() issues the global
  // reads into registers, store() writes buffer b (rows D .. DMAX-1 as zeros)
  const int pw = wave - DR_CONS / WAVE;
  float reg[TPW][5][EPL], vr[TPW];
  auto load = [&](int ci) {
    const int tc = t0 + ci * CH;
    const int nc = min(CH, t1 - tc);
#pragma unroll
    for (int s = 0; s < TPW; ++s) {
      const int tt = pw + DR_PW * s;
      if (tt < nc) {
        const float* src = planes + ((long)(tc + tt) * H + hd) * D;
#pragma unroll
        for (int q = 0; q < 5; ++q)
#pragma unroll
          for (int e = 0; e < EPL; ++e) {
            const int d = lane + WAVE * e;
            reg[s][q][e] = (d < D) ? src[q * plane + d] : 0.f;
          }
        const int cc = ct * DR_COLS + lane;
        vr[s] = (lane < DR_COLS && cc < D) ? ldf(proj + (long)(tc + tt) * stride + v_off + hd * D + cc) : 0.f;
      }
    }
  };
  auto store = [&](int ci, int b) {
    const int nc = min(CH, t1 - (t0 + ci * CH));
#pragma unroll
    for (int s = 0; s < TPW; ++s) {
      const int tt = pw + DR_PW * s;
      if (tt < nc) {
#pragma unroll
        for (int q = 0; q < 5; ++q)
#pragma unroll
          for (int e = 0; e < EPL; ++e) s_op[b][q][tt][lane + WAVE * e] = reg[s][q][e];
        if (lane < DR_COLS) s_v[b][tt][lane] = vr[s];
      }
    }
  };

  // ---- consumer state ----
  const int rg = lane & 15, c = (wave & 3) * 4 + (lane >> 4);
  const int col = ct * DR_COLS + c;
  const bool colok = col < D;
  const long slot = slots[r];
  float* sp = state + ((slot * H + hd) * D) * (long)D;
  float S[RPT];
  if (!producer) {
#pragma unroll
    for (int i = 0; i < RPT; ++i) {
      const int row = rg * RPT + i;
      S[i] = (row < D && colok) ? sp[(long)row * D + col] : 0.f;
    }
  } else if (nchunks > 0) {
    load(0);
    store(0, 0);
    if (nchunks > 1) load(1);
  }
  __syncthreads();
  for (int ci = 0; ci < nchunks; ++ci) {
    const int b = ci & 1;
    if (producer) {
      if (ci + 1 < nchunks) {
        store(ci + 1, b ^ 1);
        if (ci + 2 < nchunks) load(ci + 2);
      }
    } else {
      const int tc = t0 + ci * CH;
      const int nc = min(CH, t1 - tc);
#pragma unroll 2
      for (int tt = 0; tt < nc; ++tt) {
        const float vv = s_v[b][tt][c];
        const float* pr = &s_op[b][0][tt][rg * RPT];
        const float* pk = &s_op[b][1][tt][rg * RPT];
        const float* pu = &s_op[b][2][tt][rg * RPT];
        const float* pa = &s_op[b][3][tt][rg * RPT];
        const float* pw_ = &s_op[b][4][tt][rg * RPT];
        float d0 = 0.f, d1 = 0.f;
#pragma unroll
        for (int i = 0; i < RPT; i += 2) {
          d0 += pu[i] * S[i];
          d1 += pu[i + 1] * S[i + 1];
        }
        const float dot = sum_row(d0 + d1);
        float p0 = 0.f, p1 = 0.f;
#pragma unroll
        for (int i = 0; i < RPT; i += 2) {
          S[i] = pw_[i] * S[i] - pa[i] * dot + pk[i] * vv;
          S[i + 1] = pw_[i + 1] * S[i + 1] - pa[i + 1] * dot + pk[i + 1] * vv;
          p0 += pr[i] * S[i];
          p1 += pr[i + 1] * S[i + 1];
        }
        const float part = sum_row(p0 + p1);
        if (rg == 0 && colok) o[((long)(tc + tt) * H + hd) * D + col] = part;
      }
    }
    __syncthreads();
  }
  if (!producer) {
#pragma unroll
    for (int i = 0; i < RPT; ++i) {
      const int row = rg * RPT + i;
      if (row < D && colok) sp[(long)row * D + col] = S[i];
    }
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
  auto planes = torch::empty({5, T_, H, D}, proj.options().dtype(at::kFloat));
  auto stream = at::cuda::getCurrentHIPStream();
  // the head's second decay matrix is kept in LDS (transposed) when it fits
  const size_t w2_bytes = (size_t)D * rank * sizeof(float);
  const int w2_in_lds = w2_bytes <= 48 * 1024;
  const size_t smem = w2_in_lds ? w2_bytes : 0;
  const dim3 pgrid((T_ + DP_TOK - 1) / DP_TOK, (unsigned)H);
  const dim3 grid(R, (unsigned)H, (unsigned)((D + DR_COLS - 1) / DR_COLS));
#define DR_LAUNCH(DMAX)                                                                                        \
  do {                                                                                                         \
  hipLaunchKernelGGL((delta_prep_kernel<T, DMAX / WAVE>), pgrid, dim3(256), smem, stream,                      \
      (const T*)proj.data_ptr(), (long)proj.stride(0), (int)r_off, (int)k_off, (int)a_off, (int)w_off,         \
      (int)rank, w2.data_ptr<float>(), w0.data_ptr<float>(), a_b.data_ptr<float>(), planes.data_ptr<float>(),  \
      T_, (int)H, (int)D, w2_in_lds);                                                                          \
  hipLaunchKernelGGL((delta_rule_kernel<T, DMAX>), grid, dim3(DR_CONS + DR_PW * WAVE), 0, stream,              \
      planes.data_ptr<float>(), (const T*)proj.data_ptr(), (long)proj.stride(0), (int)v_off,                   \
      state.data_ptr<float>(), cu.data_ptr<int>(), slots.data_ptr<int>(), o.data_ptr<float>(), T_, (int)H, (int)D); \
  } while (0)
  RAGGED_DISPATCH(proj, {
    if (D <= 64) DR_LAUNCH(64);
    else if (D <= 128) DR_LAUNCH(128);
    else DR_LAUNCH(256);
    const int TH = T_ * H;
    hipLaunchKernelGGL((delta_out_kernel<T>), dim3((TH + 3) / 4), dim3(256), 0, stream, o.data_ptr<float>(),
        (const T*)proj.data_ptr(), (long)proj.stride(0), (int)g_off, norm_w.data_ptr<float>(), (float)eps,
        (T*)out.data_ptr(), (long)out.stride(0), (int)out_col, (float)out_scale, TH, (int)H, (int)D);
  });
#undef DR_LAUNCH
}
