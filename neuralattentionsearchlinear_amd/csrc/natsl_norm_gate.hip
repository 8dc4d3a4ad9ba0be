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
