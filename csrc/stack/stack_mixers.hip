// gfx950 kernels of the layers whose norm sits on the sublayer's output (interface: stack_ops.h): the cast of
// the stream into the matrix dtype, the post-norm residual update, latent attention's cache row / folded
// queries / value expansion, the short causal convolution with its carried inputs, the gated state scan that
// serves the mLSTM matrix memory and the Mamba-2 state space layer, the grouped RMS norm of their outputs,
// the dense feed-forward's activation and the score router with expert groups and identity experts.
// Everything but the matrix operands and the cached latent is float32. Wave = 64 lanes.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "stack_device.h"
#include "stack_ops.h"

namespace omx {
namespace stack {

// ------------------------------------------------------------------------------------------------ cast
template <typename T>
__global__ __launch_bounds__(256) void cast_rows_kernel(const float* __restrict__ x, long long n, T* __restrict__ out) {
  const long long i = (long long)blockIdx.x * 256 + threadIdx.x;
  if (i < n) st(out + i, x[i]);
}
void cast_rows(const float* x, int rows, int E, void* out, int f32, hipStream_t s) {
  check(rows > 0 && E > 0 && x && out, "cast_rows: bad operands");
  const long long n = (long long)rows * E;
  const dim3 grid((unsigned)((n + 255) / 256));
  if (f32)
    hipLaunchKernelGGL(cast_rows_kernel<float>, grid, dim3(256), 0, s, x, n, (float*)out);
  else
    hipLaunchKernelGGL(cast_rows_kernel<bf16>, grid, dim3(256), 0, s, x, n, (bf16*)out);
  launched("cast_rows");
}

// ------------------------------------------------------------------------------------------------ post-norm residual
// x[r] += layer_norm(y[r] + (idw ? idw[r] * x[r] : 0)) * w + b; the variance is the mean of the squared deviations.
// With hout the updated row also leaves in the matrix dtype (the next sublayer's operand).
template <typename T>
__global__ __launch_bounds__(256) void post_norm_add_kernel(float* __restrict__ x, const float* __restrict__ y, int E,
                                                            const float* __restrict__ w, const float* __restrict__ b,
                                                            float eps, const float* __restrict__ idw, T* __restrict__ hout) {
  __shared__ float red[4];
  const long long r = blockIdx.x;
  float* xr = x + r * E;
  const float* yr = y + r * E;
  const float iw = idw ? idw[r] : 0.f;
  float sum = 0.f;
  for (int i = threadIdx.x; i < E; i += 256) sum += yr[i] + iw * xr[i];
  const float mean = block_sum256(sum, red) / (float)E;
  float sq = 0.f;
  for (int i = threadIdx.x; i < E; i += 256) {
    const float d = yr[i] + iw * xr[i] - mean;
    sq += d * d;
  }
  const float inv = 1.f / sqrtf(block_sum256(sq, red) / (float)E + eps);
  for (int i = threadIdx.x; i < E; i += 256) {
    const float v = xr[i] + ((yr[i] + iw * xr[i] - mean) * inv * w[i] + b[i]);
    xr[i] = v;
    if (hout) st(hout + r * E + i, v);
  }
}
void post_norm_add(float* x, const float* y, int rows, int E, const float* w, const float* b, float eps, const float* idw,
                   void* hout, int f32, hipStream_t s) {
  check(rows > 0 && E > 0 && x && y && w && b, "post_norm_add: bad operands");
  if (f32)
    hipLaunchKernelGGL(post_norm_add_kernel<float>, dim3(rows), dim3(256), 0, s, x, y, E, w, b, eps, idw, (float*)hout);
  else
    hipLaunchKernelGGL(post_norm_add_kernel<bf16>, dim3(rows), dim3(256), 0, s, x, y, E, w, b, eps, idw, (bf16*)hout);
  launched("post_norm_add");
}

// ------------------------------------------------------------------------------------------------ latent attention
// Keys and values of every head are linear maps of one latent c per token, so attention runs in latent space:
//   score_h(t, s) = (W_uk_h^T q_plain_h(t)) . c(s) + q_rot_h(t) . k_rot(s),   o_h(t) = W_uv_h sum_s p_h(t, s) c(s).
// The cached row of a token is [c | k_rot] (one row serves all heads, and its first C elements are the value).
// latent_prepare: grid (row groups of LAT_RB, H + 1). Blocks y < H fold LAT_RB queries of head y onto the latent
// (thread r owns output r: W_uk is read along its contiguous axis) and rotate their rotated part; blocks y == H
// write the rows' cache entries: c = rms_norm(first C outputs) * w, the last R outputs rotated.
// Rotation: dims (2i, 2i + 1), i < rot_dims / 2, turn by pos * inv_freq[i]; the angle and its sine / cosine are
// computed in float64 (a float32 angle at position 10^3 is already off by 10^-4).
constexpr int LAT_RB = 8;
constexpr int LAT_MAXD = 256, LAT_MAXC = 512;
__device__ __forceinline__ float rotate_pair_elem(const float* v, int j, int rot_dims, int pos, const double* inv_freq) {
  if (j >= rot_dims) return v[j];
  const double ang = (double)pos * inv_freq[j >> 1];
  const float c = (float)cos(ang), sn = (float)sin(ang);
  const float a = v[j & ~1], b = v[j | 1];
  return (j & 1) ? b * c + a * sn : a * c - b * sn;
}
template <typename T>
__global__ __launch_bounds__(256) void latent_prepare_kernel(LatentParams P, StepRows R) {
  __shared__ float qs[LAT_RB][LAT_MAXD];
  __shared__ float red[4];
  const int r0 = blockIdx.x * LAT_RB, h = blockIdx.y, tid = threadIdx.x;
  const int nr = min(LAT_RB, R.B - r0);
  const int C = P.C, Rr = P.R, D = P.D, W = C + Rr;
  if (h == P.H) {  // the rows' cache entries
    T* cache = (T*)P.cache;
    for (int i = 0; i < nr; ++i) {
      const int b = r0 + i;
      const float* dkv = P.proj + (long long)b * P.ld + P.off_k;
      float sq = 0.f;
      for (int c = tid; c < C; c += 256) sq += dkv[c] * dkv[c];
      const float inv = 1.f / sqrtf(block_sum256(sq, red) / (float)C + P.eps);
      T* dst = cache + (long long)R.slot[b] * W;
      for (int c = tid; c < C; c += 256) st(dst + c, dkv[c] * inv * P.norm_w[c]);
      for (int j = tid; j < Rr; j += 256) st(dst + C + j, rotate_pair_elem(dkv + C, j, P.rot_dims, R.pos[b], P.inv_freq));
    }
    return;
  }
  for (int idx = tid; idx < nr * D; idx += 256) {
    const int i = idx / D, d = idx % D;
    qs[i][d] = P.proj[(long long)(r0 + i) * P.ld + P.off_q + h * (D + Rr) + d];
  }
  __syncthreads();
  const T* wk = (const T*)P.w_uk + (long long)h * D * C;
  for (int c = tid; c < C; c += 256) {
    float acc[LAT_RB];
#pragma unroll
    for (int i = 0; i < LAT_RB; ++i) acc[i] = 0.f;
    for (int d = 0; d < D; ++d) {
      const float wv = ld(wk + (long long)d * C + c);
#pragma unroll
      for (int i = 0; i < LAT_RB; ++i) acc[i] += qs[i][d] * wv;
    }
#pragma unroll
    for (int i = 0; i < LAT_RB; ++i)
      if (i < nr) P.qa[(long long)(r0 + i) * P.ld_qa + h * W + c] = acc[i];
  }
  for (int idx = tid; idx < nr * Rr; idx += 256) {
    const int i = idx / Rr, j = idx % Rr, b = r0 + i;
    const float* qr = P.proj + (long long)b * P.ld + P.off_q + h * (D + Rr) + D;
    P.qa[(long long)b * P.ld_qa + h * W + C + j] = rotate_pair_elem(qr, j, P.rot_dims, R.pos[b], P.inv_freq);
  }
}
// out[b][h * Dv + j] = (sum_c W_uvT[h][c][j] lat[b][h * C + c]) * sigmoid(g[b][h * Dv + j]); grid (row groups, H)
template <typename T>
__global__ __launch_bounds__(256) void latent_expand_kernel(LatentParams P, int B) {
  __shared__ float ls[LAT_RB][LAT_MAXC];
  const int r0 = blockIdx.x * LAT_RB, h = blockIdx.y, tid = threadIdx.x;
  const int nr = min(LAT_RB, B - r0);
  const int C = P.C, Dv = P.Dv;
  for (int idx = tid; idx < nr * C; idx += 256) {
    const int i = idx / C, c = idx % C;
    ls[i][c] = ld((const T*)P.lat + (long long)(r0 + i) * P.ld_lat + h * C + c);
  }
  __syncthreads();
  const T* wv = (const T*)P.w_uvT + (long long)h * C * Dv;
  for (int j = tid; j < Dv; j += 256) {
    float acc[LAT_RB];
#pragma unroll
    for (int i = 0; i < LAT_RB; ++i) acc[i] = 0.f;
    for (int c = 0; c < C; ++c) {
      const float w = ld(wv + (long long)c * Dv + j);
#pragma unroll
      for (int i = 0; i < LAT_RB; ++i) acc[i] += ls[i][c] * w;
    }
#pragma unroll
    for (int i = 0; i < LAT_RB; ++i)
      if (i < nr) {
        const float g = P.proj[(long long)(r0 + i) * P.ld + P.off_g + h * Dv + j];
        st((T*)P.out + (long long)(r0 + i) * P.ld_out + h * Dv + j, acc[i] * sigmoidf(g));
      }
  }
}
bool latent_supported(int D, int R, int C, int Dv) {
  return D > 0 && D <= LAT_MAXD && R >= 0 && C > 0 && C <= LAT_MAXC && Dv > 0 && C + R <= 256;
}
static void check_latent(const LatentParams& P) {
  check(P.proj && P.cache && P.qa && P.lat && P.out && P.w_uk && P.w_uvT && P.norm_w &&
            latent_supported(P.D, P.R, P.C, P.Dv) && P.rot_dims % 2 == 0 && P.rot_dims <= P.R && (P.rot_dims == 0 || P.inv_freq),
        "latent attention: operands or sizes (dim <= 256, kv_rank <= 512, kv_rank + rot_dim <= 256)");
}
void latent_prepare(const LatentParams& P, const StepRows& R, hipStream_t s) {
  check_latent(P);
  const dim3 grid((R.B + LAT_RB - 1) / LAT_RB, P.H + 1);
  if (P.f32)
    hipLaunchKernelGGL(latent_prepare_kernel<float>, grid, dim3(256), 0, s, P, R);
  else
    hipLaunchKernelGGL(latent_prepare_kernel<bf16>, grid, dim3(256), 0, s, P, R);
  launched("latent_prepare");
}
void latent_expand(const LatentParams& P, int B, hipStream_t s) {
  check_latent(P);
  const dim3 grid((B + LAT_RB - 1) / LAT_RB, P.H);
  if (P.f32)
    hipLaunchKernelGGL(latent_expand_kernel<float>, grid, dim3(256), 0, s, P, B);
  else
    hipLaunchKernelGGL(latent_expand_kernel<bf16>, grid, dim3(256), 0, s, P, B);
  launched("latent_expand");
}

// ------------------------------------------------------------------------------------------------ short convolution
// out[r][c] = silu(bias[c] + sum_j w[c][j] in(p_r - (taps - 1) + j)[c]): tap taps - 1 is the current token's.
// Inputs before the step's first row of the sequence come from its carried window (the last taps - 1 inputs,
// oldest first; zero for a new sequence). One block per row. A second launch advances the windows: the block of
// a sequence's LAST row of the step writes them (ascending, so a thread never reads what it has overwritten).
__global__ __launch_bounds__(256) void conv_silu_kernel(ConvParams P, StepRows R) {
  const int r = blockIdx.x, K = P.taps;
  const int seq = R.q_seq[r];
  int nb = 0;  // rows of the same sequence right before r, up to taps - 1
  while (nb < K - 1 && r - nb - 1 >= 0 && R.q_seq[r - nb - 1] == seq) ++nb;
  const float* win = P.state + (long long)seq * P.state_stride;
  for (int c = threadIdx.x; c < P.ch; c += 256) {
    float acc = P.bias[c];
    for (int j = 0; j < K; ++j) {
      const int back = K - 1 - j;
      const float v = back <= nb ? P.proj[(long long)(r - back) * P.ld + P.off_in + c]
                                 : win[(long long)(K - 1 - (back - nb)) * P.ch + c];
      acc += P.w[(long long)c * K + j] * v;
    }
    P.out[(long long)r * P.ld_out + c] = silu(acc);
  }
}
__global__ __launch_bounds__(256) void conv_window_kernel(ConvParams P, StepRows R) {
  const int r = blockIdx.x, K = P.taps;
  const int seq = R.q_seq[r];
  if (r + 1 < R.B && R.q_seq[r + 1] == seq) return;  // not the sequence's last row of this step
  int n = 1;  // rows of the sequence in this step, up to taps - 1
  while (n < K - 1 && r - n >= 0 && R.q_seq[r - n] == seq) ++n;
  float* win = P.state + (long long)seq * P.state_stride;
  for (int c = threadIdx.x; c < P.ch; c += 256)
    for (int sidx = 0; sidx < K - 1; ++sidx) {
      const int back = K - 2 - sidx;
      win[(long long)sidx * P.ch + c] = back < n ? P.proj[(long long)(r - back) * P.ld + P.off_in + c]
                                                 : win[(long long)(sidx + n) * P.ch + c];
    }
}
void conv_silu(const ConvParams& P, const StepRows& R, hipStream_t s) {
  check(R.B > 0 && P.proj && P.w && P.bias && P.out && P.ch > 0 && P.taps >= 1 && (P.taps == 1 || P.state),
        "conv_silu: bad operands");
  hipLaunchKernelGGL(conv_silu_kernel, dim3(R.B), dim3(256), 0, s, P, R);
  launched("conv_silu");
  if (P.taps > 1) {
    hipLaunchKernelGGL(conv_window_kernel, dim3(R.B), dim3(256), 0, s, P, R);
    launched("conv_window");
  }
}

// ------------------------------------------------------------------------------------------------ gated state scan
// S_t = a_t S_(t-1) + b_t k_t v_t^T (S is D x Dv per head), o_t = S_t^T q_t, with per-row scalars
//   SCAN_MLSTM: i = cap tanh((i_raw + i_b) / cap), f = logsigmoid(cap tanh((f_raw + f_b) / cap)),
//               m_t = max(f + m_(t-1), i), a = exp(f + m_(t-1) - m_t), b = exp(i - m_t); q scaled by D^(-1/2); a
//               normaliser n_t = a n_(t-1) + b k_t rides along as one more column of S (v = 1), and
//               y = o / (max(|n_t . q|, exp(-m_t)) + 1e-6)
//   SCAN_SSD:   dt = softplus(dt_raw + dt_bias), a = exp(-exp(A_log) dt), b = dt; q = C_t, k = B_t of the head's
//               group, v = x_t (all three from the convolution's output); y = (o + D x_t) silu(z_t)
// One block per (sequence segment of the step, head), as the retention kernel: the block of the segment's first
// row walks its rows; thread (g, j) = (tid / Dvp, tid % Dvp) keeps S[i][j], i = g, g + NG, ..., in registers
// (Dvp = Dv columns + the normaliser's), so the update needs no exchange and o is a sum of NG partials per column.
// The slot's state (S, then for the mLSTM n and m) is read once and written back once per step.
__device__ __forceinline__ float softplusf(float z) { return z > 20.f ? z : log1pf(expf(z)); }
__device__ __forceinline__ float logsigmoidf(float z) { return fminf(z, 0.f) - log1pf(expf(-fabsf(z))); }
template <int MODE, int MAXI>
__global__ __launch_bounds__(256) void gated_scan_kernel(ScanParams P, StepRows R) {
  __shared__ float qs[256], ks[256], vs[260], po[256], os[260];
  const int r0 = blockIdx.x, h = blockIdx.y, tid = threadIdx.x;
  const int seq = R.q_seq[r0];
  if (r0 > 0 && R.q_seq[r0 - 1] == seq) return;  // not the first row of its segment (uniform per block)
  const int D = P.D, Dv = P.Dv;
  const int Dvp = Dv + (MODE == SCAN_MLSTM ? 1 : 0);
  const int NG = 256 / Dvp;
  const int g = tid / Dvp, j = tid % Dvp;
  const bool act = g < NG;
  const int hg = h / (P.H / P.G);
  float* sbase = P.state + (long long)seq * P.state_stride;
  float* S0 = sbase + (long long)h * D * Dv;
  float* nvec = sbase + (long long)P.H * D * Dv + (long long)h * D;   // mLSTM only
  float* mptr = sbase + (long long)P.H * D * (Dv + 1) + h;            // mLSTM only
  float S[MAXI];
#pragma unroll
  for (int ii = 0; ii < MAXI; ++ii) {
    const int i = g + ii * NG;
    S[ii] = (act && i < D) ? (j < Dv ? S0[(long long)i * Dv + j] : nvec[i]) : 0.f;
  }
  float m = MODE == SCAN_MLSTM ? *mptr : 0.f;
  const float qscale = MODE == SCAN_MLSTM ? 1.f / sqrtf((float)D) : 1.f;
  for (int r = r0; r < R.B && R.q_seq[r] == seq; ++r) {
    const float* row = P.proj + (long long)r * P.ld;
    const float* src = MODE == SCAN_MLSTM ? row : P.conv + (long long)r * P.ld_conv;
    if (tid < D) {
      qs[tid] = src[P.off_q + hg * D + tid] * qscale;
      ks[tid] = src[P.off_k + hg * D + tid];
    }
    if (tid < Dv) vs[tid] = src[P.off_v + h * Dv + tid];
    if (MODE == SCAN_MLSTM && tid == Dv) vs[Dv] = 1.f;
    float a, b;
    if (MODE == SCAN_MLSTM) {
      const float ig = P.cap * tanhf((row[P.off_i + h] + P.i_b[h]) / P.cap);
      const float fg = logsigmoidf(P.cap * tanhf((row[P.off_f + h] + P.f_b[h]) / P.cap));
      const float mn = fmaxf(fg + m, ig);
      a = expf(fg + m - mn);
      b = expf(ig - mn);
      m = mn;
    } else {
      const float dt = softplusf(row[P.off_i + h] + P.dt_bias[h]);
      a = expf(-expf(P.a_log[h]) * dt);
      b = dt;
    }
    __syncthreads();
    float part = 0.f;
    if (act) {
      const float bv = b * vs[j];
#pragma unroll
      for (int ii = 0; ii < MAXI; ++ii) {
        const int i = g + ii * NG;
        if (i < D) {
          S[ii] = a * S[ii] + ks[i] * bv;
          part += S[ii] * qs[i];
        }
      }
    }
    po[tid] = part;
    __syncthreads();
    if (tid < Dvp) {
      float o = 0.f;
      for (int gg = 0; gg < NG; ++gg) o += po[gg * Dvp + tid];
      os[tid] = o;
    }
    __syncthreads();
    if (tid < Dv) {
      float y;
      if (MODE == SCAN_MLSTM)
        y = os[tid] / (fmaxf(fabsf(os[Dv]), expf(-m)) + 1e-6f);
      else
        y = (os[tid] + P.d_skip[h] * vs[tid]) * silu(row[P.off_g + h * Dv + tid]);
      P.y[(long long)r * P.ld_y + h * Dv + tid] = y;
    }
    __syncthreads();
  }
#pragma unroll
  for (int ii = 0; ii < MAXI; ++ii) {
    const int i = g + ii * NG;
    if (act && i < D) {
      if (j < Dv)
        S0[(long long)i * Dv + j] = S[ii];
      else
        nvec[i] = S[ii];
    }
  }
  if (MODE == SCAN_MLSTM && tid == 0) *mptr = m;
}
bool gated_scan_supported(int mode, int D, int Dv) {
  const int dvp = Dv + (mode == SCAN_MLSTM ? 1 : 0);
  if (D <= 0 || Dv <= 0 || D > 256 || dvp > 256) return false;
  const int ng = 256 / dvp;
  return (D + ng - 1) / ng <= 64;
}
template <int MODE>
static void launch_gated_scan(const ScanParams& P, const StepRows& R, hipStream_t s) {
  const int dvp = P.Dv + (MODE == SCAN_MLSTM ? 1 : 0);
  const int ng = 256 / dvp, ni = (P.D + ng - 1) / ng;
  const dim3 grid(R.B, P.H);
  if (ni <= 8)
    hipLaunchKernelGGL((gated_scan_kernel<MODE, 8>), grid, dim3(256), 0, s, P, R);
  else if (ni <= 16)
    hipLaunchKernelGGL((gated_scan_kernel<MODE, 16>), grid, dim3(256), 0, s, P, R);
  else if (ni <= 32)
    hipLaunchKernelGGL((gated_scan_kernel<MODE, 32>), grid, dim3(256), 0, s, P, R);
  else
    hipLaunchKernelGGL((gated_scan_kernel<MODE, 64>), grid, dim3(256), 0, s, P, R);
}
void gated_scan(const ScanParams& P, const StepRows& R, hipStream_t s) {
  check(R.B > 0 && P.proj && P.state && P.y && P.H > 0 && P.G > 0 && P.H % P.G == 0 && gated_scan_supported(P.mode, P.D, P.Dv),
        "gated scan: operands or head sizes (key size <= 256, value size <= 255, state within the registers)");
  if (P.mode == SCAN_MLSTM) {
    check(P.i_b && P.f_b && P.cap > 0.f && P.G == P.H, "gated scan: mLSTM gate operands");
    launch_gated_scan<SCAN_MLSTM>(P, R, s);
  } else {
    check(P.conv && P.dt_bias && P.a_log && P.d_skip, "gated scan: state space operands");
    launch_gated_scan<SCAN_SSD>(P, R, s);
  }
  launched("gated_scan");
}

// ------------------------------------------------------------------------------------------------ grouped RMS norm
// out[r][i] = y[r][i] / sqrt(mean over i's part of y^2 + eps) * w[i] * (gate ? sigmoid(gate[r][i]) : 1), the row in
// `groups` equal parts; grid (rows, groups)
template <typename T>
__global__ __launch_bounds__(256) void group_rms_kernel(const float* __restrict__ y, int ld_y, int n, int groups,
                                                        const float* __restrict__ w, float eps, const float* __restrict__ gate,
                                                        int ld_gate, T* __restrict__ out, int ld_out) {
  __shared__ float red[4];
  const long long r = blockIdx.x;
  const int per = n / groups, i0 = blockIdx.y * per;
  const float* yr = y + r * ld_y + i0;
  float sq = 0.f;
  for (int i = threadIdx.x; i < per; i += 256) sq += yr[i] * yr[i];
  const float inv = 1.f / sqrtf(block_sum256(sq, red) / (float)per + eps);
  for (int i = threadIdx.x; i < per; i += 256) {
    float v = yr[i] * inv * w[i0 + i];
    if (gate) v *= sigmoidf(gate[r * ld_gate + i0 + i]);
    st(out + r * ld_out + i0 + i, v);
  }
}
void group_rms_cast(const float* y, int ld_y, int rows, int n, int groups, const float* w, float eps, const float* gate,
                    int ld_gate, void* out, int ld_out, int f32, hipStream_t s) {
  check(rows > 0 && n > 0 && groups > 0 && n % groups == 0 && y && w && out, "group_rms_cast: bad operands");
  const dim3 grid(rows, groups);
  if (f32)
    hipLaunchKernelGGL(group_rms_kernel<float>, grid, dim3(256), 0, s, y, ld_y, n, groups, w, eps, gate, ld_gate, (float*)out,
                       ld_out);
  else
    hipLaunchKernelGGL(group_rms_kernel<bf16>, grid, dim3(256), 0, s, y, ld_y, n, groups, w, eps, gate, ld_gate, (bf16*)out,
                       ld_out);
  launched("group_rms_cast");
}

// ------------------------------------------------------------------------------------------------ dense feed-forward
// out[r][f] = relu(z[r][f])^2 in the matrix dtype
template <typename T>
__global__ __launch_bounds__(256) void relu2_kernel(const float* __restrict__ z, int ld, int rows, int F, T* __restrict__ out,
                                                    int ld_out) {
  const long long i = (long long)blockIdx.x * 256 + threadIdx.x;
  if (i >= (long long)rows * F) return;
  const long long r = i / F;
  const int f = (int)(i % F);
  const float v = fmaxf(z[r * ld + f], 0.f);
  st(out + r * ld_out + f, v * v);
}
void relu2_cast(const float* z, int ld, int rows, int F, void* out, int ld_out, int f32, hipStream_t s) {
  check(rows > 0 && F > 0 && z && out, "relu2_cast: bad operands");
  const long long n = (long long)rows * F;
  const dim3 grid((unsigned)((n + 255) / 256));
  if (f32)
    hipLaunchKernelGGL(relu2_kernel<float>, grid, dim3(256), 0, s, z, ld, rows, F, (float*)out, ld_out);
  else
    hipLaunchKernelGGL(relu2_kernel<bf16>, grid, dim3(256), 0, s, z, ld, rows, F, (bf16*)out, ld_out);
  launched("relu2_cast");
}

// ------------------------------------------------------------------------------------------------ score router
// Per row: s = softmax of the X + I router logits; choice = s + correction; the outputs form group_count groups of
// neighbours, a group ranks by its largest choice score and only outputs of the best group_keep groups can be
// chosen; the `top` largest choice scores among them are taken (ties: the lower index), weighted by their s (not
// renormalised). Outputs X .. X + I - 1 are identity experts: their weight is summed into idw[r] (the post-norm
// update adds idw * x) and their place in the expert list points at expert 0 with weight 0. The shared expert
// has no gate (sgate = 1); its activation silu(gate) * up is written behind the routed ones, as moe_route does.
constexpr int ROUTE_MAX = 256;
template <typename T>
__global__ __launch_bounds__(256) void moe_route_scores_kernel(MoeParams P) {
  __shared__ float sc[ROUTE_MAX], ch[ROUTE_MAX];
  const int b = blockIdx.x, NR = P.X + P.identity;
  const float* row = P.proj + (long long)b * P.ld;
  if (threadIdx.x == 0) {
    float mx = -INFINITY;
    for (int e = 0; e < NR; ++e) mx = fmaxf(mx, row[P.off_router + e]);
    float sum = 0.f;
    for (int e = 0; e < NR; ++e) {
      sc[e] = expf(row[P.off_router + e] - mx);
      sum += sc[e];
    }
    for (int e = 0; e < NR; ++e) {
      sc[e] /= sum;
      ch[e] = sc[e] + P.router_b[e];
    }
    if (P.group_count > 1) {  // drop the groups outside the best group_keep
      const int per = NR / P.group_count;
      unsigned long long kept = 0ull;
      for (int q = 0; q < P.group_keep; ++q) {
        int best = -1;
        float bv = -INFINITY;
        for (int gi = 0; gi < P.group_count; ++gi) {
          if (kept >> gi & 1ull) continue;
          float gm = -INFINITY;
          for (int e = gi * per; e < (gi + 1) * per; ++e) gm = fmaxf(gm, ch[e]);
          if (best < 0 || gm > bv) {
            best = gi;
            bv = gm;
          }
        }
        kept |= 1ull << best;
      }
      for (int gi = 0; gi < P.group_count; ++gi)
        if (!(kept >> gi & 1ull))
          for (int e = gi * per; e < (gi + 1) * per; ++e) ch[e] = -INFINITY;
    }
    float idw = 0.f;
    for (int jj = 0; jj < P.top; ++jj) {
      int best = 0;
      float bv = -INFINITY;
      bool any = false;
      for (int e = 0; e < NR; ++e) {
        if (ch[e] == -INFINITY) continue;  // outside the kept groups, or taken
        if (!any || ch[e] > bv) {
          best = e;
          bv = ch[e];
          any = true;
        }
      }
      if (any) ch[best] = -INFINITY;
      const bool real = any && best < P.X;
      P.eids[(long long)b * P.ld_top + jj] = real ? best : 0;
      P.ew[(long long)b * P.ld_top + jj] = real ? sc[best] : 0.f;
      if (any && !real) idw += sc[best];
    }
    P.idw[b] = idw;
    if (P.Fs > 0) P.sgate[b] = 1.f;
  }
  T* hm = (T*)P.hmid + (long long)b * P.ld_hmid + P.top * P.F;
  for (int f = threadIdx.x; f < P.Fs; f += 256) st(hm + f, silu(row[P.off_sgate + f]) * row[P.off_sup + f]);
}
void moe_route_scores(const MoeParams& P, hipStream_t s) {
  check(P.B > 0 && P.proj && P.eids && P.ew && P.idw && P.router_b && P.X + P.identity <= ROUTE_MAX && P.top > 0 &&
            P.top <= MOE_MAX_TOP && P.group_count >= 1 && P.group_count <= 64 && (P.X + P.identity) % P.group_count == 0 &&
            P.group_keep >= 1 && P.group_keep <= P.group_count && (P.Fs == 0 || (P.sgate && P.hmid)),
        "score router: operands or sizes (up to 256 outputs in up to 64 groups)");
  if (P.f32)
    hipLaunchKernelGGL(moe_route_scores_kernel<float>, dim3(P.B), dim3(256), 0, s, P);
  else
    hipLaunchKernelGGL(moe_route_scores_kernel<bf16>, dim3(P.B), dim3(256), 0, s, P);
  launched("moe_route_scores");
}

}  // namespace stack
}  // namespace omx
