// Layer tail: two-input RMSNorm with per-head mix weights and a swish gate, forward.
//   y = (rms(x1)*w1*xw[0] + rms(x2)*w2*xw[1]) * gate*sigmoid(gate),  rms(x) = x*rsqrt(mean(x^2)+eps)
// HBM-bound: 3 reads + 1 write of [rows, D]; a row is handled by a group of adjacent lanes, 16 bytes per lane and piece.
#include "natsl_device.h"
#include "natsl_host.h"

namespace natsl {

NATSL_DEVICE void unpack8(const u32x4 w, float* f) {
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    f[2 * j] = __uint_as_float(w[j] << 16);
    f[2 * j + 1] = __uint_as_float(w[j] & 0xffff0000u);
  }
}

template <int LANES, int PER>  // a row is handled by LANES adjacent lanes, PER 16-byte pieces each: D = 8 LANES PER
__global__ __launch_bounds__(256) void norm_gate_kernel(const bf16_t* x1, const bf16_t* x2, const bf16_t* gate, const bf16_t* xw,
                                                        const void* w1, const void* w2, bf16_t* y, long long rows, float eps,
                                                        int w_dtype) {
  constexpr int D = LANES * PER * 8;
  const long long row = ((long long)blockIdx.x * 256 + threadIdx.x) / LANES;
  const int seg = threadIdx.x % LANES;
  if (row >= rows) return;  // whole row groups exit together: LANES divides 64
  float a[PER][8], b[PER][8];
  float sa = 0.f, sb = 0.f;
#pragma unroll
  for (int u = 0; u < PER; ++u) {
    // piece u of the row: lanes side by side read adjacent 16-byte pieces
    const size_t off = (size_t)row * D + (u * LANES + seg) * 8;
    unpack8(*reinterpret_cast<const u32x4*>(x1 + off), a[u]);
    unpack8(*reinterpret_cast<const u32x4*>(x2 + off), b[u]);
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      sa += a[u][j] * a[u][j];
      sb += b[u][j] * b[u][j];
    }
  }
#pragma unroll
  for (int d = 1; d < LANES; d <<= 1) {
    sa += __shfl_xor(sa, d);
    sb += __shfl_xor(sb, d);
  }
  const float ra = rsqrtf(sa / D + eps) * bf16_to_f32(xw[row * 2]);
  const float rb = rsqrtf(sb / D + eps) * bf16_to_f32(xw[row * 2 + 1]);
#pragma unroll
  for (int u = 0; u < PER; ++u) {
    const int col = (u * LANES + seg) * 8;
    const size_t off = (size_t)row * D + col;
    float g[8], wa[8], wb[8];
    unpack8(*reinterpret_cast<const u32x4*>(gate + off), g);
    if (w_dtype == NATSL_BF16) {
      unpack8(*reinterpret_cast<const u32x4*>(reinterpret_cast<const bf16_t*>(w1) + col), wa);
      unpack8(*reinterpret_cast<const u32x4*>(reinterpret_cast<const bf16_t*>(w2) + col), wb);
    } else {
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        wa[j] = reinterpret_cast<const float*>(w1)[col + j];
        wb[j] = reinterpret_cast<const float*>(w2)[col + j];
      }
    }
    u32x4 out;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      float r[2];
#pragma unroll
      for (int e = 0; e < 2; ++e) {
        const int i = 2 * j + e;
        const float mix = a[u][i] * ra * wa[i] + b[u][i] * rb * wb[i];
        r[e] = mix * g[i] / (1.f + __expf(-g[i]));
      }
      out[j] = pack_bf16x2(r[0], r[1]);
    }
    *reinterpret_cast<u32x4*>(y + off) = out;
  }
}

// Backward of the same formula.  Per row, with n = x * rsqrt(mean(x^2) + eps), y = n * w, mix = y1 xw0 + y2 xw1, s = sigmoid(g):
//   dmix = dy g s,   dgate = dy mix s (1 + g (1 - s)),   dxw0 = sum_d dmix y1,   dxw1 = sum_d dmix y2,
//   a1 = dmix xw0 w1,   dx1 = r1 (a1 - n1 mean_d(a1 n1))  with  sum_d a1 n1 = xw0 dxw0   (and the same for input 2),
//   dw1 = sum over rows of dmix xw0 n1.
// A workgroup takes ROWS consecutive rows; a lane group keeps its columns' share of dw1, dw2 in registers over the rows it
// handles, the groups' shares are added in a fixed order through LDS, and one row of partial sums per workgroup goes to
// part[workgroup][2][D]; colsum_reduce_kernel adds those up (no atomics: the same bits on every run).
template <int LANES, int PER>
__global__ __launch_bounds__(256) void norm_gate_bwd_kernel(const bf16_t* x1, const bf16_t* x2, const bf16_t* gate, const bf16_t* xw,
                                                            const void* w1, const void* w2, const bf16_t* dy, bf16_t* dx1, bf16_t* dx2,
                                                            bf16_t* dgate, float* dxw, float* part, long long rows, int rows_per_wg,
                                                            float eps, int w_dtype) {
  constexpr int D = LANES * PER * 8, G = 256 / LANES;
  __shared__ float acc_s[G][2][D];
  const int grp = threadIdx.x / LANES, seg = threadIdx.x % LANES;
  float wa[PER][8], wb[PER][8], dwa[PER][8], dwb[PER][8];
#pragma unroll
  for (int u = 0; u < PER; ++u) {
    const int col = (u * LANES + seg) * 8;
    if (w_dtype == NATSL_BF16) {
      unpack8(*reinterpret_cast<const u32x4*>(reinterpret_cast<const bf16_t*>(w1) + col), wa[u]);
      unpack8(*reinterpret_cast<const u32x4*>(reinterpret_cast<const bf16_t*>(w2) + col), wb[u]);
    } else {
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        wa[u][j] = reinterpret_cast<const float*>(w1)[col + j];
        wb[u][j] = reinterpret_cast<const float*>(w2)[col + j];
      }
    }
#pragma unroll
    for (int j = 0; j < 8; ++j) { dwa[u][j] = 0.f; dwb[u][j] = 0.f; }
  }
  const long long first = (long long)blockIdx.x * rows_per_wg;
  for (int it = 0; it * G < rows_per_wg; ++it) {
    const long long row = first + it * G + grp;
    // (a lane group leaves the loop as a whole: the shuffles below stay inside a group)
    if (it * G + grp >= rows_per_wg || row >= rows) continue;
    float a[PER][8], b[PER][8], g[PER][8], d[PER][8];
    float sa = 0.f, sb = 0.f;
#pragma unroll
    for (int u = 0; u < PER; ++u) {
      const size_t off = (size_t)row * D + (u * LANES + seg) * 8;
      unpack8(*reinterpret_cast<const u32x4*>(x1 + off), a[u]);
      unpack8(*reinterpret_cast<const u32x4*>(x2 + off), b[u]);
      unpack8(*reinterpret_cast<const u32x4*>(gate + off), g[u]);
      unpack8(*reinterpret_cast<const u32x4*>(dy + off), d[u]);
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        sa += a[u][j] * a[u][j];
        sb += b[u][j] * b[u][j];
      }
    }
#pragma unroll
    for (int dd = 1; dd < LANES; dd <<= 1) {
      sa += __shfl_xor(sa, dd);
      sb += __shfl_xor(sb, dd);
    }
    const float ra = rsqrtf(sa / D + eps), rb = rsqrtf(sb / D + eps);
    const float xa = bf16_to_f32(xw[row * 2]), xb = bf16_to_f32(xw[row * 2 + 1]);
    // pass 2: a, b become the normalised inputs, d becomes dmix, g becomes dgate / mix's factor
    float pa = 0.f, pb = 0.f;
#pragma unroll
    for (int u = 0; u < PER; ++u)
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const float n1 = a[u][j] * ra, n2 = b[u][j] * rb;
        const float y1 = n1 * wa[u][j], y2 = n2 * wb[u][j];
        const float sg = 1.f / (1.f + __expf(-g[u][j]));
        const float mix = y1 * xa + y2 * xb;
        const float dmix = d[u][j] * g[u][j] * sg;
        g[u][j] = d[u][j] * mix * sg * (1.f + g[u][j] * (1.f - sg));
        pa += dmix * y1;
        pb += dmix * y2;
        a[u][j] = n1;
        b[u][j] = n2;
        d[u][j] = dmix;
      }
#pragma unroll
    for (int dd = 1; dd < LANES; dd <<= 1) {
      pa += __shfl_xor(pa, dd);
      pb += __shfl_xor(pb, dd);
    }
    if (seg == 0) {
      dxw[row * 2] = pa;
      dxw[row * 2 + 1] = pb;
    }
    const float ma = xa * pa / D, mb = xb * pb / D;   // mean_d(a1 n1), mean_d(a2 n2)
#pragma unroll
    for (int u = 0; u < PER; ++u) {
      const size_t off = (size_t)row * D + (u * LANES + seg) * 8;
      u32x4 o1, o2, og;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        float r1[2], r2[2];
#pragma unroll
        for (int e = 0; e < 2; ++e) {
          const int i = 2 * j + e;
          const float t1 = d[u][i] * xa, t2 = d[u][i] * xb;
          dwa[u][i] += t1 * a[u][i];
          dwb[u][i] += t2 * b[u][i];
          r1[e] = ra * (t1 * wa[u][i] - a[u][i] * ma);
          r2[e] = rb * (t2 * wb[u][i] - b[u][i] * mb);
        }
        o1[j] = pack_bf16x2(r1[0], r1[1]);
        o2[j] = pack_bf16x2(r2[0], r2[1]);
        og[j] = pack_bf16x2(g[u][2 * j], g[u][2 * j + 1]);
      }
      *reinterpret_cast<u32x4*>(dx1 + off) = o1;
      *reinterpret_cast<u32x4*>(dx2 + off) = o2;
      *reinterpret_cast<u32x4*>(dgate + off) = og;
    }
  }
#pragma unroll
  for (int u = 0; u < PER; ++u)
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      acc_s[grp][0][(u * LANES + seg) * 8 + j] = dwa[u][j];
      acc_s[grp][1][(u * LANES + seg) * 8 + j] = dwb[u][j];
    }
  __syncthreads();
  for (int i = threadIdx.x; i < 2 * D; i += 256) {
    float t = 0.f;
#pragma unroll
    for (int q = 0; q < G; ++q) t += acc_s[q][i / D][i % D];
    part[(size_t)blockIdx.x * 2 * D + i] = t;
  }
}

// out[c] = sum over k of part[k][c]: 64 adjacent columns per workgroup, 16 thread rows that each add up every 16th k
// (eight loads in flight), the 16 row sums added in a fixed order.
__global__ __launch_bounds__(1024) void colsum_reduce_kernel(const float* part, float* out, const int n_part, const int n_col) {
  __shared__ float sums[16][64];
  const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
  const int i = blockIdx.x * 64 + tx;
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
    out[i] = t;
  }
}

constexpr int NG_BWD_ROWS = 128;   // rows per workgroup of the backward

}  // namespace natsl

using namespace natsl;

extern "C" int natsl_norm_gate_fwd(const void* x1, const void* x2, const void* gate, const void* x_weights, const void* w1,
                                   const void* w2, void* y, int64_t rows, int D, int dtype, float eps, int w_dtype,
                                   natsl_stream_t stream) {
  if (!x1 || !x2 || !gate || !x_weights || !w1 || !w2 || !y) return fail(NATSL_ERR_INVALID, "norm_gate: null pointer argument");
  if (dtype != NATSL_BF16) return fail(NATSL_ERR_UNSUPPORTED, "norm_gate: only bf16 activations are supported");
  if (w_dtype != NATSL_BF16 && w_dtype != NATSL_F32) return fail(NATSL_ERR_UNSUPPORTED, "norm_gate: weights must be f32 or bf16");
  if (rows <= 0) return NATSL_OK;
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
#define NATSL_NG(L, P)                                                                                                      \
  {                                                                                                                         \
    const long long threads = rows * (L);                                                                                   \
    hipLaunchKernelGGL((norm_gate_kernel<L, P>), dim3((unsigned)((threads + 255) / 256)), dim3(256), 0, s, (const bf16_t*)x1,    \
                       (const bf16_t*)x2, (const bf16_t*)gate, (const bf16_t*)x_weights, w1, w2, (bf16_t*)y, (long long)rows, \
                       eps, w_dtype);                                                                                       \
    return check_launch("natsl_norm_gate_fwd");                                                                             \
  }
  switch (D) {
    case 32: NATSL_NG(4, 1)
    case 64: NATSL_NG(8, 1)
    case 96: NATSL_NG(4, 3)
    case 128: NATSL_NG(16, 1)
    case 192: NATSL_NG(8, 3)
    case 256: NATSL_NG(32, 1)
    case 384: NATSL_NG(16, 3)
    case 512: NATSL_NG(64, 1)
    default: return fail(NATSL_ERR_UNSUPPORTED, "norm_gate: head dim %d not built (32, 64, 96, 128, 192, 256, 384, 512)", D);
  }
#undef NATSL_NG
}

extern "C" size_t natsl_norm_gate_bwd_workspace_bytes(int64_t rows, int D) {
  if (rows <= 0 || D <= 0) return 0;
  return (size_t)((rows + NG_BWD_ROWS - 1) / NG_BWD_ROWS) * 2 * (size_t)D * sizeof(float);
}

extern "C" int natsl_norm_gate_bwd(const void* x1, const void* x2, const void* gate, const void* x_weights, const void* w1,
                                   const void* w2, const void* dy, void* dx1, void* dx2, void* dgate, float* dx_weights, float* dw1,
                                   float* dw2, void* workspace, size_t workspace_bytes, int64_t rows, int D, int dtype, float eps,
                                   int w_dtype, natsl_stream_t stream) {
  const char* what = "natsl_norm_gate_bwd";
  if (!x1 || !x2 || !gate || !x_weights || !w1 || !w2 || !dy || !dx1 || !dx2 || !dgate || !dx_weights || !dw1 || !dw2)
    return fail(NATSL_ERR_INVALID, "%s: null pointer argument", what);
  if (dtype != NATSL_BF16) return fail(NATSL_ERR_UNSUPPORTED, "%s: only bf16 activations are supported", what);
  if (w_dtype != NATSL_BF16 && w_dtype != NATSL_F32) return fail(NATSL_ERR_UNSUPPORTED, "%s: weights must be f32 or bf16", what);
  if (dw2 != dw1 + D) return fail(NATSL_ERR_INVALID, "%s: dw1, dw2 must be the two rows of one [2][D] tensor", what);
  if (rows <= 0) return NATSL_OK;
  const size_t need = natsl_norm_gate_bwd_workspace_bytes(rows, D);
  if (!workspace || workspace_bytes < need) return fail(NATSL_ERR_WORKSPACE, "%s: workspace of %zu bytes needed, %zu given", what, need, workspace_bytes);
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  const unsigned wgs = (unsigned)((rows + NG_BWD_ROWS - 1) / NG_BWD_ROWS);
  float* part = reinterpret_cast<float*>(workspace);
#define NATSL_NGB(L, P)                                                                                                          \
  hipLaunchKernelGGL((norm_gate_bwd_kernel<L, P>), dim3(wgs), dim3(256), 0, s, (const bf16_t*)x1, (const bf16_t*)x2,              \
                     (const bf16_t*)gate, (const bf16_t*)x_weights, w1, w2, (const bf16_t*)dy, (bf16_t*)dx1, (bf16_t*)dx2,       \
                     (bf16_t*)dgate, dx_weights, part, (long long)rows, NG_BWD_ROWS, eps, w_dtype);                              \
  break;
  switch (D) {
    case 32: NATSL_NGB(4, 1)
    case 64: NATSL_NGB(8, 1)
    case 96: NATSL_NGB(4, 3)
    case 128: NATSL_NGB(16, 1)
    case 192: NATSL_NGB(8, 3)
    case 256: NATSL_NGB(32, 1)
    case 384: NATSL_NGB(16, 3)
    case 512: NATSL_NGB(64, 1)
    default: return fail(NATSL_ERR_UNSUPPORTED, "%s: head dim %d not built (32, 64, 96, 128, 192, 256, 384, 512)", what, D);
  }
#undef NATSL_NGB
  int rc = check_launch(what);
  if (rc != NATSL_OK) return rc;
  hipLaunchKernelGGL(colsum_reduce_kernel, dim3((unsigned)((2 * D + 63) / 64)), dim3(1024), 0, s, part, dw1, (int)wgs, 2 * D);
  return check_launch(what);
}
