// Layer glue around the mixed operator, forward: the depthwise causal short convolution with its activation, and the
// RMS / L2 normalisation of head rows.  Both are HBM-bound and work on the layer's own token-major tensors ([B,T,D] and
// [rows,D]): no transposed copies, one read and one write of the activations.
//
//   short_conv_kernel   y[b,t,d] = act(bias[d] + sum_j w[d,j] e[b, t-(W-1)+j, d]),  e = the W-1 inputs before the
//                       sequence (from a cached state, else zeros) followed by x.  This is what the reference's
//                       ShortConvolution (flash-linear-attention, called at src/nats/layers/natsl_attn_gdn.py:425-491)
//                       computes: a causal cross-correlation with the kernel's last tap on the current token.
//   row_norm_kernel     y = x * rsqrt(mean(x^2) + eps) * weight   (RMSNorm, src/nats/layers/natsl_attn_gdn.py:504-505)
//                       y = x * rsqrt(sum(x^2) + eps)             (L2Norm of the Mamba layer's B and C)
#include "natsl_device.h"
#include "natsl_host.h"

namespace natsl {

NATSL_DEVICE void unpack8_bf16(const u32x4 w, float* f) {
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    f[2 * j] = __uint_as_float(w[j] << 16);
    f[2 * j + 1] = __uint_as_float(w[j] & 0xffff0000u);
  }
}

// eight adjacent channels of one row, as floats
template <bool F32>
NATSL_DEVICE void load8(const void* base, const size_t elem, float* f) {
  if constexpr (F32) {
    const f32x4 a = *reinterpret_cast<const f32x4*>(reinterpret_cast<const float*>(base) + elem);
    const f32x4 b = *reinterpret_cast<const f32x4*>(reinterpret_cast<const float*>(base) + elem + 4);
#pragma unroll
    for (int j = 0; j < 4; ++j) { f[j] = a[j]; f[4 + j] = b[j]; }
  } else {
    unpack8_bf16(*reinterpret_cast<const u32x4*>(reinterpret_cast<const bf16_t*>(base) + elem), f);
  }
}
template <bool F32>
NATSL_DEVICE void store8(void* base, const size_t elem, const float* f) {
  if constexpr (F32) {
    *reinterpret_cast<f32x4*>(reinterpret_cast<float*>(base) + elem) = (f32x4){f[0], f[1], f[2], f[3]};
    *reinterpret_cast<f32x4*>(reinterpret_cast<float*>(base) + elem + 4) = (f32x4){f[4], f[5], f[6], f[7]};
  } else {
    u32x4 w;
#pragma unroll
    for (int j = 0; j < 4; ++j) w[j] = pack_bf16x2(f[2 * j], f[2 * j + 1]);
    *reinterpret_cast<u32x4*>(reinterpret_cast<bf16_t*>(base) + elem) = w;
  }
}
NATSL_DEVICE float ld1(const void* p, const bool f32, const size_t i) {
  return f32 ? reinterpret_cast<const float*>(p)[i] : bf16_to_f32(reinterpret_cast<const bf16_t*>(p)[i]);
}

// A thread owns 8 adjacent channels for a run of `run` consecutive tokens of one sequence and slides a window of the last
// W-1 rows through registers: every row is read once (plus W-1 rows at the start of each run).  Adjacent threads take
// adjacent channel groups, so a row is read and written in whole 16-byte (bf16) or 32-byte (fp32) pieces side by side.
template <int W, bool F32>
__global__ __launch_bounds__(256) void short_conv_kernel(const void* x, const void* w, const void* bias, const void* state,
                                                         void* y, void* state_out, const int B, const int T, const int D, const int run,
                                                         const int silu, const bool w_f32, const bool state_f32) {
  const int groups = D / 8, runs = (T + run - 1) / run;
  const long long gid = (long long)blockIdx.x * 256 + threadIdx.x;
  if (gid >= (long long)B * runs * groups) return;
  const int cg = (int)(gid % groups);
  const int r = (int)((gid / groups) % runs), b = (int)(gid / ((long long)groups * runs));
  const int d0 = 8 * cg, t0 = r * run, t1 = min(T, t0 + run);
  float wt[W][8], bs[8], win[W][8];   // win[j] = the input W-1-j rows back; win[W-1] is the current row
#pragma unroll
  for (int c = 0; c < 8; ++c) {
#pragma unroll
    for (int j = 0; j < W; ++j) wt[j][c] = ld1(w, w_f32, (size_t)(d0 + c) * W + j);
    bs[c] = bias ? ld1(bias, w_f32, d0 + c) : 0.f;
  }
  // the W-1 rows before the run: earlier tokens, else the cached state [B,D,W] (its last W-1 entries), else zeros
#pragma unroll
  for (int j = 0; j < W - 1; ++j) {
    const int s = t0 - (W - 1) + j;
    if (s >= 0) {
      load8<F32>(x, ((size_t)b * T + s) * D + d0, win[j]);
    } else {
#pragma unroll
      for (int c = 0; c < 8; ++c) win[j][c] = state ? ld1(state, state_f32, ((size_t)b * D + d0 + c) * W + (W + s)) : 0.f;
    }
  }
  // the state the next call starts from: the last W inputs of (state ++ x), [B,D,W] in x's dtype, by the thread that owns
  // the sequence's last run
  if (state_out && r == runs - 1) {
#pragma unroll
    for (int j = 0; j < W; ++j) {
      const int s = T - W + j;
      float e[8];
      if (s >= 0) {
        load8<F32>(x, ((size_t)b * T + s) * D + d0, e);
      } else {
#pragma unroll
        for (int c = 0; c < 8; ++c) e[c] = state ? ld1(state, state_f32, ((size_t)b * D + d0 + c) * W + (W + s)) : 0.f;
      }
#pragma unroll
      for (int c = 0; c < 8; ++c) {
        const size_t o = ((size_t)b * D + d0 + c) * W + j;
        if constexpr (F32) reinterpret_cast<float*>(state_out)[o] = e[c];
        else reinterpret_cast<bf16_t*>(state_out)[o] = f32_to_bf16(e[c]);
      }
    }
  }
  // eight rows are requested before the first of them is used: a thread's loads are otherwise one dependent round trip
  // to memory per row
  constexpr int AHEAD = 8;
  auto one_row = [&](const float* in, const int t) __attribute__((always_inline)) {
    float o[8];
#pragma unroll
    for (int c = 0; c < 8; ++c) {
      win[W - 1][c] = in[c];
      float acc = bs[c];
#pragma unroll
      for (int j = 0; j < W; ++j) acc += wt[j][c] * win[j][c];
      o[c] = silu ? acc / (1.f + __expf(-acc)) : acc;
    }
    store8<F32>(y, ((size_t)b * T + t) * D + d0, o);
#pragma unroll
    for (int j = 0; j < W - 1; ++j)
#pragma unroll
      for (int c = 0; c < 8; ++c) win[j][c] = win[j + 1][c];
  };
  int tb = t0;
  for (; tb + AHEAD <= t1; tb += AHEAD) {   // (no conditions around the loads: they all go out before the first wait)
    float rows[AHEAD][8];
#pragma unroll
    for (int a = 0; a < AHEAD; ++a) load8<F32>(x, ((size_t)b * T + tb + a) * D + d0, rows[a]);
#pragma unroll
    for (int a = 0; a < AHEAD; ++a) one_row(rows[a], tb + a);
  }
  for (; tb < t1; ++tb) {
    float row[8];
    load8<F32>(x, ((size_t)b * T + tb) * D + d0, row);
    one_row(row, tb);
  }
}

// Backward of the short convolution.  With pre[t] = bias + sum_j w[j] e[t-(W-1)+j] and y = act(pre):
//   dpre[t] = dy[t] act'(pre[t]);   dx[s] = sum_i w[W-1-i] dpre[s+i];   dw[j] = sum_{b,t} dpre[t] e[t-(W-1)+j];   dbias = sum dpre.
// Same decomposition as the forward: a thread owns 8 channels for a run of tokens, recomputes pre from a sliding window of
// inputs, keeps the last W dpre rows, and emits dx[s] once dpre[s .. s+W-1] exist (it reads W-1 rows past its run for that,
// without adding them to its weight sums).  Its weight / bias sums go to part[run id][W+1][D] (fp32) and are added up by
// conv_wgrad_reduce_kernel in a fixed order: no atomics, the same bits on every run.
template <int W, bool F32>
__global__ __launch_bounds__(256) void short_conv_bwd_kernel(const void* x, const void* w, const void* bias, const void* state,
                                                             const void* dy, void* dx, float* part, const int B, const int T,
                                                             const int D, const int run, const int silu, const bool w_f32,
                                                             const bool state_f32) {
  const int groups = D / 8, runs = (T + run - 1) / run;
  const long long gid = (long long)blockIdx.x * 256 + threadIdx.x;
  if (gid >= (long long)B * runs * groups) return;
  const int cg = (int)(gid % groups);
  const int r = (int)((gid / groups) % runs), b = (int)(gid / ((long long)groups * runs));
  const int d0 = 8 * cg, t0 = r * run, t1 = min(T, t0 + run);
  float wt[W][8], bs[8], win[W][8], dwin[W][8], dws[W + 1][8];
#pragma unroll
  for (int c = 0; c < 8; ++c) {
#pragma unroll
    for (int j = 0; j < W; ++j) { wt[j][c] = ld1(w, w_f32, (size_t)(d0 + c) * W + j); dws[j][c] = 0.f; dwin[j][c] = 0.f; }
    bs[c] = bias ? ld1(bias, w_f32, d0 + c) : 0.f;
    dws[W][c] = 0.f;
  }
#pragma unroll
  for (int j = 0; j < W - 1; ++j) {
    const int s = t0 - (W - 1) + j;
    if (s >= 0) {
      load8<F32>(x, ((size_t)b * T + s) * D + d0, win[j]);
    } else {
#pragma unroll
      for (int c = 0; c < 8; ++c) win[j][c] = state ? ld1(state, state_f32, ((size_t)b * D + d0 + c) * W + (W + s)) : 0.f;
    }
  }
  // t runs W-1 rows past the run: dx of the run's last tokens needs the dpre of the next run's first ones
  const int t_end = min(T, t1 + W - 1);
  for (int t = t0; t < t1 + W - 1; ++t) {
    float dp[8];
    if (t < t_end) {
      float g[8];
      load8<F32>(x, ((size_t)b * T + t) * D + d0, win[W - 1]);
      load8<F32>(dy, ((size_t)b * T + t) * D + d0, g);
#pragma unroll
      for (int c = 0; c < 8; ++c) {
        float acc = bs[c];
#pragma unroll
        for (int j = 0; j < W; ++j) acc += wt[j][c] * win[j][c];
        float da = 1.f;
        if (silu) {
          const float sg = 1.f / (1.f + __expf(-acc));
          da = sg * (1.f + acc * (1.f - sg));
        }
        dp[c] = g[c] * da;
        if (t < t1) {   // this run's own tokens: weight and bias sums
#pragma unroll
          for (int j = 0; j < W; ++j) dws[j][c] += dp[c] * win[j][c];
          dws[W][c] += dp[c];
        }
      }
    } else {
#pragma unroll
      for (int c = 0; c < 8; ++c) dp[c] = 0.f;
    }
    // dwin[i] = dpre[t-(W-1)+i]
#pragma unroll
    for (int c = 0; c < 8; ++c) dwin[W - 1][c] = dp[c];
    const int sx = t - (W - 1);
    if (sx >= t0) {
      float o[8];
#pragma unroll
      for (int c = 0; c < 8; ++c) {
        float acc = 0.f;
#pragma unroll
        for (int i = 0; i < W; ++i) acc += wt[W - 1 - i][c] * dwin[i][c];
        o[c] = acc;
      }
      store8<F32>(dx, ((size_t)b * T + sx) * D + d0, o);
    }
#pragma unroll
    for (int j = 0; j < W - 1; ++j)
#pragma unroll
      for (int c = 0; c < 8; ++c) { win[j][c] = win[j + 1][c]; dwin[j][c] = dwin[j + 1][c]; }
  }
  float* pr = part + ((size_t)(b * runs + r) * (W + 1)) * D + d0;
#pragma unroll
  for (int j = 0; j <= W; ++j) {
    *reinterpret_cast<f32x4*>(pr + (size_t)j * D) = (f32x4){dws[j][0], dws[j][1], dws[j][2], dws[j][3]};
    *reinterpret_cast<f32x4*>(pr + (size_t)j * D + 4) = (f32x4){dws[j][4], dws[j][5], dws[j][6], dws[j][7]};
  }
}

// dw[d][j] = sum over run ids of part[id][j][d], dbias[d] = the same of part[id][W][d].  A workgroup takes 64 adjacent
// (j, d) columns; its 16 thread rows each add up every 16th run id (eight loads in flight), then the 16 row sums are added
// in a fixed order: the same bits on every run.
__global__ __launch_bounds__(1024) void conv_wgrad_reduce_kernel(const float* part, float* dw, float* dbias, const int n_part, const int D,
                                                                 const int W) {
  __shared__ float sums[16][64];
  const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
  const int i = blockIdx.x * 64 + tx, n_col = (W + 1) * D;
  float acc = 0.f;
  if (i < n_col) {
    const float* src = part + i;
    int k = ty;
    for (; k + 7 * 16 < n_part; k += 8 * 16) {
      float v[8];
#pragma unroll
      for (int u = 0; u < 8; ++u) v[u] = src[(size_t)(k + 16 * u) * n_col];
#pragma unroll
      for (int u = 0; u < 8; ++u) acc += v[u];
    }
    for (; k < n_part; k += 16) acc += src[(size_t)k * n_col];
  }
  sums[ty][tx] = acc;
  __syncthreads();
  if (ty == 0 && i < n_col) {
    float t = 0.f;
#pragma unroll
    for (int r = 0; r < 16; ++r) t += sums[r][tx];
    const int j = i / D, d = i % D;
    if (j < W) dw[(size_t)d * W + j] = t;
    else if (dbias) dbias[d] = t;
  }
}

// A row is handled by LANES adjacent lanes with PER pieces of 8 elements each (D = 8 LANES PER).
template <int LANES, int PER, bool F32>
__global__ __launch_bounds__(256) void row_norm_kernel(const void* x, const void* weight, void* y, const long long rows, const float eps,
                                                       const int l2, const bool w_f32) {
  constexpr int D = LANES * PER * 8;
  const long long row = ((long long)blockIdx.x * 256 + threadIdx.x) / LANES;
  const int seg = threadIdx.x % LANES;
  if (row >= rows) return;  // whole row groups exit together: LANES divides 64
  float v[PER][8];
  float ss = 0.f;
#pragma unroll
  for (int u = 0; u < PER; ++u) {
    load8<F32>(x, (size_t)row * D + (u * LANES + seg) * 8, v[u]);
#pragma unroll
    for (int j = 0; j < 8; ++j) ss += v[u][j] * v[u][j];
  }
#pragma unroll
  for (int d = 1; d < LANES; d <<= 1) ss += __shfl_xor(ss, d);
  const float rs = rsqrtf((l2 ? ss : ss / D) + eps);
#pragma unroll
  for (int u = 0; u < PER; ++u) {
    const int col = (u * LANES + seg) * 8;
    float o[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) o[j] = v[u][j] * rs * (weight ? ld1(weight, w_f32, col + j) : 1.f);
    store8<F32>(y, (size_t)row * D + col, o);
  }
}

// Backward of row_norm_kernel: with n = x r (r = rsqrt(mean x^2 + eps), or rsqrt(sum x^2 + eps) for the L2 form) and
// a = dy w:  dx = r (a - n mean(a n))  (L2: the sum instead of the mean),  dw = sum over rows of dy n.  A workgroup takes ROWS
// consecutive rows; the lane groups' shares of dw are added in a fixed order through LDS and leave as one partial row per
// workgroup (part[workgroup][D]), which row_norm_wgrad_reduce_kernel adds up.
template <int LANES, int PER, bool F32>
__global__ __launch_bounds__(256) void row_norm_bwd_kernel(const void* x, const void* weight, const void* dy, void* dx, float* part,
                                                           const long long rows, const int rows_per_wg, const float eps, const int l2,
                                                           const bool w_f32) {
  constexpr int D = LANES * PER * 8, G = 256 / LANES;
  __shared__ float acc_s[G][D];
  const int grp = threadIdx.x / LANES, seg = threadIdx.x % LANES;
  float w[PER][8], dw[PER][8];
#pragma unroll
  for (int u = 0; u < PER; ++u)
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      w[u][j] = weight ? ld1(weight, w_f32, (u * LANES + seg) * 8 + j) : 1.f;
      dw[u][j] = 0.f;
    }
  const long long first = (long long)blockIdx.x * rows_per_wg;
  for (int it = 0; it * G < rows_per_wg; ++it) {
    const long long row = first + it * G + grp;
    if (it * G + grp >= rows_per_wg || row >= rows) continue;   // (a lane group leaves as a whole)
    float v[PER][8], d[PER][8];
    float ss = 0.f;
#pragma unroll
    for (int u = 0; u < PER; ++u) {
      load8<F32>(x, (size_t)row * D + (u * LANES + seg) * 8, v[u]);
      load8<F32>(dy, (size_t)row * D + (u * LANES + seg) * 8, d[u]);
#pragma unroll
      for (int j = 0; j < 8; ++j) ss += v[u][j] * v[u][j];
    }
#pragma unroll
    for (int dd = 1; dd < LANES; dd <<= 1) ss += __shfl_xor(ss, dd);
    const float rs = rsqrtf((l2 ? ss : ss / D) + eps);
    float an = 0.f;
#pragma unroll
    for (int u = 0; u < PER; ++u)
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        v[u][j] *= rs;                       // n
        dw[u][j] += d[u][j] * v[u][j];
        d[u][j] *= w[u][j];                  // a
        an += d[u][j] * v[u][j];
      }
#pragma unroll
    for (int dd = 1; dd < LANES; dd <<= 1) an += __shfl_xor(an, dd);
    const float m = l2 ? an : an / D;
#pragma unroll
    for (int u = 0; u < PER; ++u) {
      float o[8];
#pragma unroll
      for (int j = 0; j < 8; ++j) o[j] = rs * (d[u][j] - v[u][j] * m);
      store8<F32>(dx, (size_t)row * D + (u * LANES + seg) * 8, o);
    }
  }
  if (part == nullptr) return;
#pragma unroll
  for (int u = 0; u < PER; ++u)
#pragma unroll
    for (int j = 0; j < 8; ++j) acc_s[grp][(u * LANES + seg) * 8 + j] = dw[u][j];
  __syncthreads();
  for (int i = threadIdx.x; i < D; i += 256) {
    float t = 0.f;
#pragma unroll
    for (int q = 0; q < G; ++q) t += acc_s[q][i];
    part[(size_t)blockIdx.x * D + i] = t;
  }
}

// out[c] = sum over k of part[k][c] (64 columns x 16 partial-sum slices per workgroup, fixed order)
__global__ __launch_bounds__(1024) void row_norm_wgrad_reduce_kernel(const float* part, float* out, const int n_part, const int n_col) {
  __shared__ float sums[16][64];
  const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
  const int i = blockIdx.x * 64 + tx;
  float acc = 0.f;
  if (i < n_col)
    for (int k = ty; k < n_part; k += 16) acc += part[(size_t)k * n_col + i];
  sums[ty][tx] = acc;
  __syncthreads();
  if (ty == 0 && i < n_col) {
    float t = 0.f;
#pragma unroll
    for (int r = 0; r < 16; ++r) t += sums[r][tx];
    out[i] = t;
  }
}

constexpr int RN_BWD_ROWS = 128;   // rows per workgroup of the row norms' backward

}  // namespace natsl

using namespace natsl;

static int conv_run_length(int B, int T, int D) {
  // long runs read the fewest rows twice; short ones are needed to give every CU work on small inputs
  int run = 32;
  while (run > 8 && (long long)B * cdiv(T, run) * (D / 8) < 256 * 256) run >>= 1;
  return run;
}

extern "C" int natsl_short_conv_fwd(const void* x, const void* weight, const void* bias, const void* state, void* y, void* state_out,
                                    int B, int T, int D, int W, int activation, int dtype, int w_dtype, int state_dtype,
                                    natsl_stream_t stream) {
  const char* what = "natsl_short_conv_fwd";
  if (!x || !weight || !y) return fail(NATSL_ERR_INVALID, "%s: null pointer argument", what);
  if (dtype != NATSL_BF16 && dtype != NATSL_F32) return fail(NATSL_ERR_UNSUPPORTED, "%s: activations must be f32 or bf16", what);
  if (w_dtype != NATSL_BF16 && w_dtype != NATSL_F32) return fail(NATSL_ERR_UNSUPPORTED, "%s: weights must be f32 or bf16", what);
  if (state && state_dtype != NATSL_BF16 && state_dtype != NATSL_F32) return fail(NATSL_ERR_UNSUPPORTED, "%s: the state must be f32 or bf16", what);
  if (B <= 0 || T <= 0 || D <= 0) return fail(NATSL_ERR_INVALID, "%s: non-positive dimension", what);
  if (D % 8) return fail(NATSL_ERR_UNSUPPORTED, "%s: D=%d must be a multiple of 8", what, D);
  if (activation != 0 && activation != 1) return fail(NATSL_ERR_INVALID, "%s: activation must be 0 (none) or 1 (silu)", what);
  if (state_out && state_out == state) return fail(NATSL_ERR_INVALID, "%s: state_out must not alias state (other threads still read it)", what);
  const int run = conv_run_length(B, T, D);
  const long long threads = (long long)B * cdiv(T, run) * (D / 8);
  const dim3 grid((unsigned)((threads + 255) / 256));
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  const bool f32 = dtype == NATSL_F32;
#define NATSL_CONV(WW)                                                                                                        \
  {                                                                                                                           \
    if (f32) hipLaunchKernelGGL((short_conv_kernel<WW, true>), grid, dim3(256), 0, s, x, weight, bias, state, y, state_out, B, T, D, run, \
                                activation, w_dtype == NATSL_F32, state_dtype == NATSL_F32);                                   \
    else hipLaunchKernelGGL((short_conv_kernel<WW, false>), grid, dim3(256), 0, s, x, weight, bias, state, y, state_out, B, T, D, run,    \
                            activation, w_dtype == NATSL_F32, state_dtype == NATSL_F32);                                       \
    return check_launch(what);                                                                                                \
  }
  switch (W) {
    case 2: NATSL_CONV(2)
    case 3: NATSL_CONV(3)
    case 4: NATSL_CONV(4)
    default: return fail(NATSL_ERR_UNSUPPORTED, "%s: kernel size %d not built (2, 3, 4)", what, W);
  }
#undef NATSL_CONV
}

extern "C" size_t natsl_short_conv_bwd_workspace_bytes(int B, int T, int D, int W) {
  if (B <= 0 || T <= 0 || D <= 0 || W <= 0) return 0;
  return (size_t)B * cdiv(T, conv_run_length(B, T, D)) * (W + 1) * D * sizeof(float);
}

extern "C" int natsl_short_conv_bwd(const void* x, const void* weight, const void* bias, const void* state, const void* dy, void* dx,
                                    float* dweight, float* dbias, void* workspace, size_t workspace_bytes, int B, int T, int D, int W,
                                    int activation, int dtype, int w_dtype, int state_dtype, natsl_stream_t stream) {
  const char* what = "natsl_short_conv_bwd";
  if (!x || !weight || !dy || !dx || !dweight) return fail(NATSL_ERR_INVALID, "%s: null pointer argument", what);
  if (dtype != NATSL_BF16 && dtype != NATSL_F32) return fail(NATSL_ERR_UNSUPPORTED, "%s: activations must be f32 or bf16", what);
  if (w_dtype != NATSL_BF16 && w_dtype != NATSL_F32) return fail(NATSL_ERR_UNSUPPORTED, "%s: weights must be f32 or bf16", what);
  if (state && state_dtype != NATSL_BF16 && state_dtype != NATSL_F32) return fail(NATSL_ERR_UNSUPPORTED, "%s: the state must be f32 or bf16", what);
  if (B <= 0 || T <= 0 || D <= 0) return fail(NATSL_ERR_INVALID, "%s: non-positive dimension", what);
  if (D % 8) return fail(NATSL_ERR_UNSUPPORTED, "%s: D=%d must be a multiple of 8", what, D);
  if (activation != 0 && activation != 1) return fail(NATSL_ERR_INVALID, "%s: activation must be 0 (none) or 1 (silu)", what);
  if (W < 2 || W > 4) return fail(NATSL_ERR_UNSUPPORTED, "%s: kernel size %d not built (2, 3, 4)", what, W);
  const size_t need = natsl_short_conv_bwd_workspace_bytes(B, T, D, W);
  if (!workspace || workspace_bytes < need) return fail(NATSL_ERR_WORKSPACE, "%s: workspace of %zu bytes needed, %zu given", what, need, workspace_bytes);
  if (reinterpret_cast<uintptr_t>(workspace) & 15) return fail(NATSL_ERR_INVALID, "%s: workspace must be 16-byte aligned", what);
  const int run = conv_run_length(B, T, D), runs = cdiv(T, run);
  const long long threads = (long long)B * runs * (D / 8);
  const dim3 grid((unsigned)((threads + 255) / 256));
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  float* part = reinterpret_cast<float*>(workspace);
  const bool f32 = dtype == NATSL_F32;
#define NATSL_CONVB(WW)                                                                                                            \
  {                                                                                                                                \
    if (f32) hipLaunchKernelGGL((short_conv_bwd_kernel<WW, true>), grid, dim3(256), 0, s, x, weight, bias, state, dy, dx, part, B, T, \
                                D, run, activation, w_dtype == NATSL_F32, state_dtype == NATSL_F32);                                \
    else hipLaunchKernelGGL((short_conv_bwd_kernel<WW, false>), grid, dim3(256), 0, s, x, weight, bias, state, dy, dx, part, B, T,    \
                            D, run, activation, w_dtype == NATSL_F32, state_dtype == NATSL_F32);                                    \
  }
  if (W == 2) NATSL_CONVB(2) else if (W == 3) NATSL_CONVB(3) else NATSL_CONVB(4)
#undef NATSL_CONVB
  int rc = check_launch(what);
  if (rc != NATSL_OK) return rc;
  hipLaunchKernelGGL(conv_wgrad_reduce_kernel, dim3((unsigned)(((W + 1) * D + 63) / 64)), dim3(1024), 0, s, part, dweight, dbias, B * runs, D, W);
  return check_launch(what);
}

extern "C" int natsl_row_norm_fwd(const void* x, const void* weight, void* y, int64_t rows, int D, float eps, int l2, int dtype,
                                  int w_dtype, natsl_stream_t stream) {
  const char* what = "natsl_row_norm_fwd";
  if (!x || !y) return fail(NATSL_ERR_INVALID, "%s: null pointer argument", what);
  if (dtype != NATSL_BF16 && dtype != NATSL_F32) return fail(NATSL_ERR_UNSUPPORTED, "%s: activations must be f32 or bf16", what);
  if (weight && w_dtype != NATSL_BF16 && w_dtype != NATSL_F32) return fail(NATSL_ERR_UNSUPPORTED, "%s: weights must be f32 or bf16", what);
  if (rows <= 0) return NATSL_OK;
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  const bool f32 = dtype == NATSL_F32;
#define NATSL_RN(L, P)                                                                                                          \
  {                                                                                                                             \
    const long long threads = rows * (L);                                                                                       \
    const dim3 grid((unsigned)((threads + 255) / 256));                                                                         \
    if (f32) hipLaunchKernelGGL((row_norm_kernel<L, P, true>), grid, dim3(256), 0, s, x, weight, y, (long long)rows, eps, l2,    \
                                w_dtype == NATSL_F32);                                                                           \
    else hipLaunchKernelGGL((row_norm_kernel<L, P, false>), grid, dim3(256), 0, s, x, weight, y, (long long)rows, eps, l2,       \
                            w_dtype == NATSL_F32);                                                                               \
    return check_launch(what);                                                                                                  \
  }
  switch (D) {
    case 32: NATSL_RN(4, 1)
    case 64: NATSL_RN(8, 1)
    case 96: NATSL_RN(4, 3)
    case 128: NATSL_RN(16, 1)
    case 192: NATSL_RN(8, 3)
    case 256: NATSL_RN(32, 1)
    case 384: NATSL_RN(16, 3)
    case 512: NATSL_RN(64, 1)
    default: return fail(NATSL_ERR_UNSUPPORTED, "%s: row width %d not built (32, 64, 96, 128, 192, 256, 384, 512)", what, D);
  }
#undef NATSL_RN
}

extern "C" size_t natsl_row_norm_bwd_workspace_bytes(int64_t rows, int D) {
  if (rows <= 0 || D <= 0) return 0;
  return (size_t)((rows + RN_BWD_ROWS - 1) / RN_BWD_ROWS) * (size_t)D * sizeof(float);
}

extern "C" int natsl_row_norm_bwd(const void* x, const void* weight, const void* dy, void* dx, float* dweight, void* workspace,
                                  size_t workspace_bytes, int64_t rows, int D, float eps, int l2, int dtype, int w_dtype,
                                  natsl_stream_t stream) {
  const char* what = "natsl_row_norm_bwd";
  if (!x || !dy || !dx || (weight && !dweight)) return fail(NATSL_ERR_INVALID, "%s: null pointer argument", what);
  if (dtype != NATSL_BF16 && dtype != NATSL_F32) return fail(NATSL_ERR_UNSUPPORTED, "%s: activations must be f32 or bf16", what);
  if (weight && w_dtype != NATSL_BF16 && w_dtype != NATSL_F32) return fail(NATSL_ERR_UNSUPPORTED, "%s: weights must be f32 or bf16", what);
  if (rows <= 0) return NATSL_OK;
  float* part = nullptr;
  if (weight) {
    const size_t need = natsl_row_norm_bwd_workspace_bytes(rows, D);
    if (!workspace || workspace_bytes < need) return fail(NATSL_ERR_WORKSPACE, "%s: workspace of %zu bytes needed, %zu given", what, need, workspace_bytes);
    part = reinterpret_cast<float*>(workspace);
  }
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  const bool f32 = dtype == NATSL_F32;
  const unsigned wgs = (unsigned)((rows + RN_BWD_ROWS - 1) / RN_BWD_ROWS);
#define NATSL_RNB(L, P)                                                                                                         \
  if (f32) hipLaunchKernelGGL((row_norm_bwd_kernel<L, P, true>), dim3(wgs), dim3(256), 0, s, x, weight, dy, dx, part,            \
                              (long long)rows, RN_BWD_ROWS, eps, l2, w_dtype == NATSL_F32);                                      \
  else hipLaunchKernelGGL((row_norm_bwd_kernel<L, P, false>), dim3(wgs), dim3(256), 0, s, x, weight, dy, dx, part,               \
                          (long long)rows, RN_BWD_ROWS, eps, l2, w_dtype == NATSL_F32);                                          \
  break;
  switch (D) {
    case 32: NATSL_RNB(4, 1)
    case 64: NATSL_RNB(8, 1)
    case 96: NATSL_RNB(4, 3)
    case 128: NATSL_RNB(16, 1)
    case 192: NATSL_RNB(8, 3)
    case 256: NATSL_RNB(32, 1)
    case 384: NATSL_RNB(16, 3)
    case 512: NATSL_RNB(64, 1)
    default: return fail(NATSL_ERR_UNSUPPORTED, "%s: row width %d not built (32, 64, 96, 128, 192, 256, 384, 512)", what, D);
  }
#undef NATSL_RNB
  int rc = check_launch(what);
  if (rc != NATSL_OK || !weight) return rc;
  hipLaunchKernelGGL(row_norm_wgrad_reduce_kernel, dim3((unsigned)((D + 63) / 64)), dim3(1024), 0, s, part, dweight, (int)wgs, D);
  return check_launch(what);
}
