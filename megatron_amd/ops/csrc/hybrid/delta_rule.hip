// Generalized delta rule over ragged batches with a per-request fp32 state:
//   S <- diag(w) S - (a u)(u^T S) + k v^T ,  o = S^T r      (per head; both terms read the old S)
//   w = exp(-e^{-1/2} sigmoid(W2 tanh(b) + w0)),  a = sigmoid(a_pre + a_b),  u = k / sqrt(sum k^2 + 1e-6)
// The update is independent per value column: S[:, c] needs u . S[:, c] and
// r . S[:, c] only.  Workgroup = (request, head, tile of 16 value columns).  A
// request's new tokens are walked in order by four consumer waves while the
// producer waves prepare the next chunk's operands (all the non-linearities)
// in LDS.
#include "../ragged/ragged_common.h"

constexpr int DR_COLS = 16;          // value columns per workgroup
constexpr int DR_RG = 16;            // row groups: a column's rows are dealt to the 16 lanes of one wave row
constexpr int DR_CONS = DR_COLS * DR_RG;        // consumer threads (4 waves): the token loop
constexpr int DR_MAX_RANK = 128;     // decay bottleneck

// x summed over the 16 lanes of its wave row, in every lane: four rotations inside
// the row (DPP modifiers of the adds: VALU only, no LDS round trip)
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

// Waves with two roles.  Consumer waves 0-3 run the token loop: wave w holds
// columns 4 w .. 4 w + 3 of the tile; inside a wave lane = 16 cw + rg owns rows
// rg * RPT .. rg * RPT + RPT - 1 of column 4 w + cw in registers; the sixteen partial
// sums of a column sit in one wave row and are reduced in registers: the token
// loop has no barrier and a few dozen instructions per token.
// Producer waves stage the operands of the NEXT chunk of tokens into the other
// half of a double buffer meanwhile, one wave per token, lanes over the
// channels: projections read, bottleneck tanh and second decay matrix, decay,
// removal rate, unit key; values pass between lanes in registers, so a
// producer needs no barrier either.  One workgroup barrier per chunk.  (The
// column tiles of a head repeat the staging; they run on different CUs.)
template <typename T, int DMAX, int CH, int PW>
__global__ __launch_bounds__(DR_CONS + PW * WAVE) void delta_rule_kernel(
    const T* __restrict__ proj, long stride, int r_off, int k_off, int v_off, int a_off, int w_off, int rank,
    const float* __restrict__ w2, const float* __restrict__ w0, const float* __restrict__ a_b,
    float* __restrict__ state, const int* __restrict__ cu, const int* __restrict__ slots, float* __restrict__ o,
    int H, int D, int w2_in_lds) {
  constexpr int RPT = DMAX / DR_RG;
  constexpr int EPL = DMAX / WAVE;                 // channels per producer lane
  __shared__ __align__(16) float s_r[2][CH][DMAX], s_k[2][CH][DMAX], s_u[2][CH][DMAX], s_au[2][CH][DMAX],
      s_w[2][CH][DMAX];
  __shared__ float s_v[2][CH][DR_COLS];
  extern __shared__ float s_w2[];                  // [rank][D] (transposed), when it fits
  const int r = blockIdx.x, hd = blockIdx.y, ct = blockIdx.z;
  const int wave = threadIdx.x / WAVE, lane = threadIdx.x % WAVE;
  const bool producer = wave >= DR_CONS / WAVE;   // wave-uniform
  const int t0 = cu[r], t1 = cu[r + 1];
  const int nchunks = (t1 - t0 + CH - 1) / CH;
  if (w2_in_lds)
    for (int i = threadIdx.x; i < D * rank; i += DR_CONS + PW * WAVE) s_w2[(i % rank) * D + i / rank] = w2[(long)hd * D * rank + i];
  __syncthreads();

  // ---- producer: a wave owns tokens pw, pw + PW, ... of a chunk.  load() only issues the
  // global reads of a chunk into registers; finish() does the arithmetic and writes buffer b
  // (rows D .. DMAX-1 as zeros).  The reads of chunk ci + 2 are issued right after chunk ci + 1
  // was finished, so their latency passes while the consumers walk chunk ci.
  constexpr int TPW = CH / PW;
  static_assert(CH % PW == 0, "a chunk is dealt evenly to the producer waves");
  const int pw = wave - DR_CONS / WAVE;
  float kk[TPW][EPL], rr[TPW][EPL], ar[TPW][EPL], b0[TPW], b1[TPW], vr[TPW];
  auto load = [&](int ci) {
    const int tc = t0 + ci * CH;
    const int nc = min(CH, t1 - tc);
#pragma unroll
    for (int s = 0; s < TPW; ++s) {
      const int tt = pw + PW * s;
      if (tt < nc) {
        const T* row = proj + (long)(tc + tt) * stride;
        b0[s] = (lane < rank) ? ldf(row + w_off + lane) : 0.f;
        b1[s] = (lane + WAVE < rank) ? ldf(row + w_off + lane + WAVE) : 0.f;
#pragma unroll
        for (int e = 0; e < EPL; ++e) {
          const int d = lane + WAVE * e;
          const bool ok = d < D;
          const int ch = hd * D + (ok ? d : 0);
          kk[s][e] = ok ? ldf(row + k_off + ch) : 0.f;
          rr[s][e] = ok ? ldf(row + r_off + ch) : 0.f;
          ar[s][e] = ok ? ldf(row + a_off + ch) : 0.f;
        }
        const int cc = ct * DR_COLS + lane;
        vr[s] = (lane < DR_COLS && cc < D) ? ldf(row + v_off + hd * D + cc) : 0.f;
      }
    }
  };
  auto finish = [&](int ci, int b) {
    const int tc = t0 + ci * CH;
    const int nc = min(CH, t1 - tc);
    const float decay_c = -0.60653065971263342f;   // -e^{-1/2}
#pragma unroll
    for (int s = 0; s < TPW; ++s) {
      const int tt = pw + PW * s;
      if (tt < nc) {
        const float tb0 = tanhf(b0[s]), tb1 = tanhf(b1[s]);   // tanh of the bottleneck, entry j in lane j % 64
        float zz[EPL];
        float ss = 0.f;
#pragma unroll
        for (int e = 0; e < EPL; ++e) {
          const int d = lane + WAVE * e;
          zz[e] = (d < D) ? w0[hd * D + d] : 0.f;
          ss += kk[s][e] * kk[s][e];
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
#pragma unroll
        for (int e = 0; e < EPL; ++e) {
          const int d = lane + WAVE * e;
          const bool ok = d < D;
          const float u = kk[s][e] * inv;
          const float a = ok ? sigmoidf_(ar[s][e] + a_b[hd * D + d]) : 0.f;
          s_r[b][tt][d] = rr[s][e];
          s_k[b][tt][d] = kk[s][e];
          s_u[b][tt][d] = u;
          s_au[b][tt][d] = a * u;
          s_w[b][tt][d] = ok ? expf(decay_c * sigmoidf_(zz[e])) : 0.f;
        }
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
    finish(0, 0);
    if (nchunks > 1) load(1);
  }
  __syncthreads();
  for (int ci = 0; ci < nchunks; ++ci) {
    const int b = ci & 1;
    if (producer) {
      if (ci + 1 < nchunks) {
        finish(ci + 1, b ^ 1);
        if (ci + 2 < nchunks) load(ci + 2);
      }
    } else {
      const int tc = t0 + ci * CH;
      const int nc = min(CH, t1 - tc);
#pragma unroll 2
      for (int tt = 0; tt < nc; ++tt) {
        const float vv = s_v[b][tt][c];
        const float* pu = &s_u[b][tt][rg * RPT];
        const float* pw_ = &s_w[b][tt][rg * RPT];
        const float* pa = &s_au[b][tt][rg * RPT];
        const float* pk = &s_k[b][tt][rg * RPT];
        const float* pr = &s_r[b][tt][rg * RPT];
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
  auto stream = at::cuda::getCurrentHIPStream();
  const dim3 grid(R, (unsigned)H, (unsigned)((D + DR_COLS - 1) / DR_COLS));
  // the head's second decay matrix is kept in LDS (transposed) when it fits beside the operand buffers
  const size_t w2_bytes = (size_t)D * rank * sizeof(float);
  const int w2_in_lds = w2_bytes <= 16 * 1024;
  const size_t smem = w2_in_lds ? w2_bytes : 0;
#define DR_LAUNCH(DMAX, CH, PW)                                                                                \
  hipLaunchKernelGGL((delta_rule_kernel<T, DMAX, CH, PW>), grid, dim3(DR_CONS + PW * WAVE), smem, stream,      \
      (const T*)proj.data_ptr(), (long)proj.stride(0), (int)r_off, (int)k_off, (int)v_off, (int)a_off,         \
      (int)w_off, (int)rank, w2.data_ptr<float>(), w0.data_ptr<float>(), a_b.data_ptr<float>(),                \
      state.data_ptr<float>(), cu.data_ptr<int>(), slots.data_ptr<int>(), o.data_ptr<float>(), (int)H, (int)D, \
      w2_in_lds)
  RAGGED_DISPATCH(proj, {
    if (D <= 64) DR_LAUNCH(64, 8, 8);
    else if (D <= 128) DR_LAUNCH(128, 8, 8);
    else DR_LAUNCH(256, 4, 4);
    const int TH = T_ * H;
    hipLaunchKernelGGL((delta_out_kernel<T>), dim3((TH + 3) / 4), dim3(256), 0, stream, o.data_ptr<float>(),
        (const T*)proj.data_ptr(), (long)proj.stride(0), (int)g_off, norm_w.data_ptr<float>(), (float)eps,
        (T*)out.data_ptr(), (long)out.stride(0), (int)out_col, (float)out_scale, TH, (int)H, (int)D);
  });
#undef DR_LAUNCH
}
