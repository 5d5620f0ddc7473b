// Token-local kernels of the ragged path: embedding gather with hashed bigrams,
// hyper-connection stream update fused with the next read and its RMS norm,
// residual causal convolution with carried taps, xIELU, per-head gating and a
// plain-weight RMS norm over rows.
#include "ragged_common.h"

// ---------------------------------------------------------------------------
// embedding: x[t] = embed[tok] (+ bigram[row]) (+ pos[p]) in fp32
// ---------------------------------------------------------------------------
template <typename T>
__global__ void embed_kernel(const long* __restrict__ tokens, const int* __restrict__ cu,
                             const int* __restrict__ slots, const int* __restrict__ tok_req,
                             const int* __restrict__ tok_pos, const T* __restrict__ embed,
                             const T* __restrict__ bigram, const T* __restrict__ pos,
                             const int* __restrict__ prev_state, long mul_prev, long mul_cur,
                             long buckets, float* __restrict__ x, int W) {
  const int t = blockIdx.x;
  const long tok = tokens[t];
  const int r = tok_req[t], p = tok_pos[t];
  long brow = -1;
  if (bigram != nullptr) {
    if (p == 0) {
      brow = buckets;
    } else {
      long prev = (t == cu[r]) ? (long)prev_state[slots[r]] : tokens[t - 1];
      brow = (prev * mul_prev + tok * mul_cur) % buckets;
    }
  }
  for (int c = threadIdx.x; c < W; c += blockDim.x) {
    float v = ldf(embed + tok * W + c);
    if (brow >= 0) v += ldf(bigram + brow * W + c);
    if (pos != nullptr) v += ldf(pos + (long)p * W + c);
    x[(long)t * W + c] = v;
  }
}

__global__ void prev_token_kernel(const long* __restrict__ tokens, const int* __restrict__ cu,
                                  const int* __restrict__ slots, int* __restrict__ prev_state, int R) {
  int r = blockIdx.x * blockDim.x + threadIdx.x;
  if (r < R) prev_state[slots[r]] = (int)tokens[cu[r + 1] - 1];
}

torch::Tensor embed_tokens(torch::Tensor tokens, torch::Tensor cu, torch::Tensor slots, torch::Tensor tok_req,
                           torch::Tensor tok_pos, torch::Tensor embed, torch::Tensor bigram, torch::Tensor pos,
                           torch::Tensor prev_state, int64_t mul_prev, int64_t mul_cur, int64_t buckets) {
  TORCH_CHECK(tokens.is_cuda() && tokens.scalar_type() == at::kLong && tokens.is_contiguous());
  check_i32(cu, "cu"); check_i32(slots, "slots"); check_i32(tok_req, "tok_req"); check_i32(tok_pos, "tok_pos");
  const int T_ = tokens.numel(), R = slots.numel(), W = embed.size(1);
  TORCH_CHECK(cu.numel() == R + 1 && tok_req.numel() == T_ && tok_pos.numel() == T_);
  TORCH_CHECK(embed.is_contiguous() && embed.dim() == 2);
  const bool has_bg = bigram.numel() > 0, has_pos = pos.numel() > 0;
  if (has_bg) {
    TORCH_CHECK(bigram.is_contiguous() && bigram.size(1) == W && bigram.size(0) == buckets + 1 &&
                bigram.scalar_type() == embed.scalar_type());
    check_i32(prev_state, "prev_state");
  }
  if (has_pos) TORCH_CHECK(pos.is_contiguous() && pos.size(1) == W && pos.scalar_type() == embed.scalar_type());
  auto x = torch::empty({T_, W}, embed.options().dtype(at::kFloat));
  auto stream = at::cuda::getCurrentHIPStream();
  RAGGED_DISPATCH(embed, hipLaunchKernelGGL((embed_kernel<T>), dim3(T_), dim3(256), 0, stream,
      tokens.data_ptr<long>(), cu.data_ptr<int>(), slots.data_ptr<int>(), tok_req.data_ptr<int>(),
      tok_pos.data_ptr<int>(), (const T*)embed.data_ptr(), has_bg ? (const T*)bigram.data_ptr() : nullptr,
      has_pos ? (const T*)pos.data_ptr() : nullptr, has_bg ? prev_state.data_ptr<int>() : nullptr,
      (long)mul_prev, (long)mul_cur, (long)buckets, x.data_ptr<float>(), W));
  if (has_bg)
    hipLaunchKernelGGL(prev_token_kernel, dim3((R + 63) / 64), dim3(64), 0, stream, tokens.data_ptr<long>(),
                       cu.data_ptr<int>(), slots.data_ptr<int>(), prev_state.data_ptr<int>(), R);
  return x;
}

// ---------------------------------------------------------------------------
// hyper-connections: x_t <- sum_s mix[s,t] x_s + out[t] y ; u = sum_s in[s] x_s ;
// h = u * rsqrt(mean(u^2) + eps) * (1 + w).  One workgroup per token.
// ---------------------------------------------------------------------------
constexpr int HC_MAX_STREAMS = 8;

// BLOCK = 1024 for steps with few tokens (decode): one workgroup owns a token, so
// more threads are the only way to have more loads in flight.
template <typename TY, int BLOCK>
__global__ __launch_bounds__(BLOCK) void hc_mix_norm_kernel(
    float* __restrict__ streams, const TY* __restrict__ y, long y_stride, const float* __restrict__ mix,
    const float* __restrict__ out_w, const float* __restrict__ in_w, const float* __restrict__ norm_w,
    float eps, float* __restrict__ h, int S, int W) {
  __shared__ float red[BLOCK / WAVE];
  __shared__ float s_mix[HC_MAX_STREAMS * HC_MAX_STREAMS], s_out[HC_MAX_STREAMS], s_in[HC_MAX_STREAMS];
  const int t = blockIdx.x;
  if (threadIdx.x < S * S && y != nullptr) s_mix[threadIdx.x] = mix[threadIdx.x];
  if (threadIdx.x < S) {
    if (y != nullptr) s_out[threadIdx.x] = out_w[threadIdx.x];
    if (in_w != nullptr) s_in[threadIdx.x] = in_w[threadIdx.x];
  }
  __syncthreads();
  float* xs_base = streams + (long)t * S * W;
  float ss = 0.f;
  for (int c = threadIdx.x; c < W; c += BLOCK) {
    float xs[HC_MAX_STREAMS];
#pragma unroll
    for (int s = 0; s < HC_MAX_STREAMS; ++s) xs[s] = (s < S) ? xs_base[(long)s * W + c] : 0.f;
    if (y != nullptr) {
      const float yv = ldf(y + (long)t * y_stride + c);
      float ns[HC_MAX_STREAMS];
#pragma unroll
      for (int d = 0; d < HC_MAX_STREAMS; ++d) {
        float a = 0.f;
        if (d < S) {
#pragma unroll
          for (int s = 0; s < HC_MAX_STREAMS; ++s)
            if (s < S) a += s_mix[s * S + d] * xs[s];
          a += s_out[d] * yv;
          xs_base[(long)d * W + c] = a;
        }
        ns[d] = a;
      }
#pragma unroll
      for (int d = 0; d < HC_MAX_STREAMS; ++d) xs[d] = ns[d];
    }
    if (in_w != nullptr) {
      float u = 0.f;
#pragma unroll
      for (int s = 0; s < HC_MAX_STREAMS; ++s)
        if (s < S) u += s_in[s] * xs[s];
      h[(long)t * W + c] = u;
      ss += u * u;
    }
  }
  if (in_w == nullptr) return;
  const float total = block_reduce_sum<BLOCK>(ss, red);
  const float rs = rsqrtf(total / (float)W + eps);
  for (int c = threadIdx.x; c < W; c += BLOCK) {
    const long i = (long)t * W + c;
    h[i] = h[i] * rs * (1.f + norm_w[c]);   // same thread wrote h[i] above
  }
}

torch::Tensor hc_mix_norm(torch::Tensor streams, torch::Tensor y, torch::Tensor mix, torch::Tensor out_w,
                          torch::Tensor in_w, torch::Tensor norm_w, double eps) {
  check_f32(streams, "streams");
  TORCH_CHECK(streams.dim() == 3);
  const int T_ = streams.size(0), S = streams.size(1), W = streams.size(2);
  TORCH_CHECK(S >= 1 && S <= HC_MAX_STREAMS, "at most ", HC_MAX_STREAMS, " residual streams");
  const bool has_y = y.numel() > 0, has_in = in_w.numel() > 0;
  if (has_y) {
    TORCH_CHECK(y.is_cuda() && y.dim() == 2 && y.size(0) == T_ && y.size(1) == W && y.stride(1) == 1);
    check_f32(mix, "mix"); check_f32(out_w, "out_w");
    TORCH_CHECK(mix.numel() == S * S && out_w.numel() == S);
  }
  torch::Tensor h;
  if (has_in) {
    check_f32(in_w, "in_w"); check_f32(norm_w, "norm_w");
    TORCH_CHECK(in_w.numel() == S && norm_w.numel() == W);
    h = torch::empty({T_, W}, streams.options());
  } else {
    h = torch::empty({0}, streams.options());
  }
  if (T_ == 0 || (!has_y && !has_in)) return h;
  auto stream = at::cuda::getCurrentHIPStream();
  float* hp = has_in ? h.data_ptr<float>() : nullptr;
  const float* inp = has_in ? in_w.data_ptr<float>() : nullptr;
  const float* nwp = has_in ? norm_w.data_ptr<float>() : nullptr;
  const bool wide = T_ < 512 && W >= 1024;
#define HC_LAUNCH(TY, BLOCK, YP, YS, MP, OP)                                                              \
  hipLaunchKernelGGL((hc_mix_norm_kernel<TY, BLOCK>), dim3(T_), dim3(BLOCK), 0, stream,                   \
                     streams.data_ptr<float>(), YP, YS, MP, OP, inp, nwp, (float)eps, hp, S, W)
  if (has_y) {
    RAGGED_DISPATCH(y, {
      if (wide) HC_LAUNCH(T, 1024, (const T*)y.data_ptr(), (long)y.stride(0), mix.data_ptr<float>(), out_w.data_ptr<float>());
      else HC_LAUNCH(T, 256, (const T*)y.data_ptr(), (long)y.stride(0), mix.data_ptr<float>(), out_w.data_ptr<float>());
    });
  } else {
    if (wide) HC_LAUNCH(float, 1024, (const float*)nullptr, 0L, (const float*)nullptr, (const float*)nullptr);
    else HC_LAUNCH(float, 256, (const float*)nullptr, 0L, (const float*)nullptr, (const float*)nullptr);
  }
#undef HC_LAUNCH
  return h;
}

// ---------------------------------------------------------------------------
// residual causal depthwise conv with carried taps
// ---------------------------------------------------------------------------
constexpr int CANON_MAX_TAPS = 16;

template <typename TO>
__global__ void canon_conv_kernel(const float* __restrict__ h, const float* __restrict__ w,
                                  const float* __restrict__ state, const int* __restrict__ cu,
                                  const int* __restrict__ slots, const int* __restrict__ tok_req,
                                  TO* __restrict__ out, long total, int W, int taps) {
  for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (long)gridDim.x * blockDim.x) {
    const int t = (int)(i / W), c = (int)(i % W);
    const int r = tok_req[t];
    const int first = cu[r], local = t - first;
    const float* st = state + (long)slots[r] * (taps - 1) * W;
    float acc = h[i];
    for (int j = 0; j < taps; ++j) {
      const int src = local - (taps - 1) + j;
      const float v = (src >= 0) ? h[(long)(first + src) * W + c] : st[(long)(taps - 1 + src) * W + c];
      acc += w[c * taps + j] * v;
    }
    stf(out + i, acc);
  }
}

__global__ void canon_state_kernel(const float* __restrict__ h, float* __restrict__ state,
                                   const int* __restrict__ cu, const int* __restrict__ slots, int R, int W,
                                   int taps) {
  const long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= (long)R * W) return;
  const int r = (int)(i / W), c = (int)(i % W);
  const int first = cu[r], n = cu[r + 1] - first;
  float* st = state + (long)slots[r] * (taps - 1) * W;
  float nv[CANON_MAX_TAPS];
  for (int k = 0; k < taps - 1; ++k) {
    const int src = n - (taps - 1) + k;
    nv[k] = (src >= 0) ? h[(long)(first + src) * W + c] : st[(long)(taps - 1 + src) * W + c];
  }
  for (int k = 0; k < taps - 1; ++k) st[(long)k * W + c] = nv[k];
}

torch::Tensor canon_conv(torch::Tensor h, torch::Tensor w, torch::Tensor state, torch::Tensor cu,
                         torch::Tensor slots, torch::Tensor tok_req, bool out_bf16) {
  check_f32(h, "h"); check_f32(w, "w"); check_f32(state, "state");
  check_i32(cu, "cu"); check_i32(slots, "slots"); check_i32(tok_req, "tok_req");
  const int T_ = h.size(0), W = h.size(1), taps = w.size(1), R = slots.numel();
  TORCH_CHECK(w.size(0) == W && taps >= 1 && taps <= CANON_MAX_TAPS);
  TORCH_CHECK(state.dim() == 3 && state.size(1) == taps - 1 && state.size(2) == W);
  TORCH_CHECK(tok_req.numel() == T_ && cu.numel() == R + 1);
  auto out = torch::empty({T_, W}, h.options().dtype(out_bf16 ? at::kBFloat16 : at::kFloat));
  if (T_ == 0) return out;
  auto stream = at::cuda::getCurrentHIPStream();
  const long total = (long)T_ * W;
  const int grid = grid_for(total, 256);
  if (out_bf16)
    hipLaunchKernelGGL((canon_conv_kernel<bf16>), dim3(grid), dim3(256), 0, stream, h.data_ptr<float>(),
                       w.data_ptr<float>(), state.data_ptr<float>(), cu.data_ptr<int>(), slots.data_ptr<int>(),
                       tok_req.data_ptr<int>(), (bf16*)out.data_ptr(), total, W, taps);
  else
    hipLaunchKernelGGL((canon_conv_kernel<float>), dim3(grid), dim3(256), 0, stream, h.data_ptr<float>(),
                       w.data_ptr<float>(), state.data_ptr<float>(), cu.data_ptr<int>(), slots.data_ptr<int>(),
                       tok_req.data_ptr<int>(), out.data_ptr<float>(), total, W, taps);
  if (taps > 1)
    hipLaunchKernelGGL(canon_state_kernel, dim3(((long)R * W + 255) / 256), dim3(256), 0, stream,
                       h.data_ptr<float>(), state.data_ptr<float>(), cu.data_ptr<int>(), slots.data_ptr<int>(),
                       R, W, taps);
  return out;
}

// ---------------------------------------------------------------------------
// xIELU
// ---------------------------------------------------------------------------
template <typename T>
__global__ void xielu_kernel(const T* __restrict__ z, const float* __restrict__ act, T* __restrict__ out, long n) {
  const float ap = softplusf_(act[0]);
  const float aq = 0.5f + softplusf_(act[1]);
  for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (long)gridDim.x * blockDim.x) {
    const float v = ldf(z + i);
    const float r = (v > 0.f) ? (ap * v * v + 0.5f * v) : (aq * (expm1f(v) - v) + 0.5f * v);
    stf(out + i, r);
  }
}

torch::Tensor xielu(torch::Tensor z, torch::Tensor act) {
  TORCH_CHECK(z.is_cuda() && z.is_contiguous());
  check_f32(act, "act");
  TORCH_CHECK(act.numel() == 2);
  auto out = torch::empty_like(z);
  const long n = z.numel();
  if (n == 0) return out;
  auto stream = at::cuda::getCurrentHIPStream();
  RAGGED_DISPATCH(z, hipLaunchKernelGGL((xielu_kernel<T>), dim3(grid_for(n, 256)), dim3(256), 0, stream,
      (const T*)z.data_ptr(), act.data_ptr<float>(), (T*)out.data_ptr(), n));
  return out;
}

// ---------------------------------------------------------------------------
// per-head sigmoid gate: out[t, h*d + i] = x[t, h, i] * sigmoid(g[t, h])
// ---------------------------------------------------------------------------
template <typename T>
__global__ void gate_heads_kernel(const T* __restrict__ x, long xs_t, long xs_h, const T* __restrict__ g,
                                  long gs_t, T* __restrict__ out, long total, int H, int d) {
  for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (long)gridDim.x * blockDim.x) {
    const int e = (int)(i % d);
    const int hh = (int)((i / d) % H);
    const long t = i / ((long)d * H);
    const float gv = sigmoidf_(ldf(g + t * gs_t + hh));
    stf(out + i, ldf(x + t * xs_t + hh * xs_h + e) * gv);
  }
}

torch::Tensor gate_heads(torch::Tensor x, torch::Tensor g, int64_t H) {
  TORCH_CHECK(x.is_cuda() && x.dim() == 3 && x.size(1) == H && x.stride(2) == 1);
  TORCH_CHECK(g.is_cuda() && g.dim() == 2 && g.size(0) == x.size(0) && g.size(1) == H && g.stride(1) == 1 &&
              g.scalar_type() == x.scalar_type());
  const int T_ = x.size(0), d = x.size(2);
  auto out = torch::empty({T_, (long)H * d}, x.options());
  const long total = out.numel();
  if (total == 0) return out;
  auto stream = at::cuda::getCurrentHIPStream();
  RAGGED_DISPATCH(x, hipLaunchKernelGGL((gate_heads_kernel<T>), dim3(grid_for(total, 256)), dim3(256), 0, stream,
      (const T*)x.data_ptr(), (long)x.stride(0), (long)x.stride(1), (const T*)g.data_ptr(), (long)g.stride(0),
      (T*)out.data_ptr(), total, (int)H, d));
  return out;
}

// ---------------------------------------------------------------------------
// RMS norm over rows with a plain fp32 weight (strided rows in, contiguous out)
// ---------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void rmsnorm_rows_kernel(const T* __restrict__ x, long xs, const float* __restrict__ w,
                                                           float eps, T* __restrict__ out, int n) {
  __shared__ float red[256 / WAVE];
  const long t = blockIdx.x;
  float ss = 0.f;
  for (int c = threadIdx.x; c < n; c += 256) {
    const float v = ldf(x + t * xs + c);
    ss += v * v;
  }
  const float rs = rsqrtf(block_reduce_sum<256>(ss, red) / (float)n + eps);
  for (int c = threadIdx.x; c < n; c += 256) stf(out + t * n + c, ldf(x + t * xs + c) * rs * w[c]);
}

torch::Tensor rmsnorm_rows(torch::Tensor x, torch::Tensor w, double eps) {
  TORCH_CHECK(x.is_cuda() && x.dim() == 2 && x.stride(1) == 1);
  check_f32(w, "w");
  const int T_ = x.size(0), n = x.size(1);
  TORCH_CHECK(w.numel() == n);
  auto out = torch::empty({T_, n}, x.options());
  if (T_ == 0) return out;
  auto stream = at::cuda::getCurrentHIPStream();
  RAGGED_DISPATCH(x, hipLaunchKernelGGL((rmsnorm_rows_kernel<T>), dim3(T_), dim3(256), 0, stream,
      (const T*)x.data_ptr(), (long)x.stride(0), w.data_ptr<float>(), (float)eps, (T*)out.data_ptr(), n));
  return out;
}
