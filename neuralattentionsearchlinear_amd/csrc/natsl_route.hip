// Selector and routing kernels: block mean pooling, hard selection, routing tables.
// Integer / byte work, HBM-bound and tiny except for the pooling pass over the hidden states.
#include "natsl_device.h"
#include "natsl_host.h"

namespace natsl {

static thread_local char g_error[512] = "";
char* error_buffer() { return g_error; }

NATSL_DEVICE float load_as_f32(const void* p, int dtype, size_t i) {
  return dtype == NATSL_F32 ? reinterpret_cast<const float*>(p)[i] : bf16_to_f32(reinterpret_cast<const bf16_t*>(p)[i]);
}
NATSL_DEVICE void store_from_f32(void* p, int dtype, size_t i, float x) {
  if (dtype == NATSL_F32) reinterpret_cast<float*>(p)[i] = x;
  else reinterpret_cast<bf16_t*>(p)[i] = f32_to_bf16(x);
}

// ---------------------------------------------------------------------------------------------
// mean pooling: grid (ceil(D/(256*VEC)), total_blocks); each thread sums one column slice.
// ---------------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void mean_pool_kernel(const void* x, void* out, int B, int T, int D, int block, int dtype,
                                                        const SeqRow* seqs, int n_seqs, int nb_per_seq) {
  const int gb = blockIdx.y;  // flat output block index
  int bos, len, c;
  if (seqs == nullptr) {
    const int n = gb / nb_per_seq;
    c = gb - n * nb_per_seq;
    bos = n * T;
    len = T;
  } else {
    int n = 0;
    for (int i = 1; i < n_seqs; ++i)
      if (seqs[i].bos_nats <= gb) n = i;
    c = gb - seqs[n].bos_nats;
    bos = seqs[n].bos;
    len = seqs[n].eos - bos;
  }
  const int lo = c * block, hi = min(len, lo + block);
  const float inv = 1.0f / (float)(hi - lo);
  if (dtype == NATSL_BF16 && (D & 7) == 0) {
    const int d8 = (blockIdx.x * 256 + threadIdx.x) * 8;
    if (d8 >= D) return;
    float s[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    const bf16_t* xp = reinterpret_cast<const bf16_t*>(x) + (size_t)(bos + lo) * D + d8;
    for (int t = lo; t < hi; ++t, xp += D) {
      const u32x4 w = *reinterpret_cast<const u32x4*>(xp);
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        s[2 * j] += __uint_as_float(w[j] << 16);
        s[2 * j + 1] += __uint_as_float(w[j] & 0xffff0000u);
      }
    }
    u32x4 o;
#pragma unroll
    for (int j = 0; j < 4; ++j) o[j] = pack_bf16x2(s[2 * j] * inv, s[2 * j + 1] * inv);
    *reinterpret_cast<u32x4*>(reinterpret_cast<bf16_t*>(out) + (size_t)gb * D + d8) = o;
  } else {
    for (int d = blockIdx.x * 256 * 8 + threadIdx.x; d < min(D, (int)(blockIdx.x + 1) * 256 * 8); d += 256) {
      float s = 0.f;
      for (int t = lo; t < hi; ++t) s += load_as_f32(x, dtype, (size_t)(bos + t) * D + d);
      store_from_f32(out, dtype, (size_t)gb * D + d, s * inv);
    }
  }
}

// ---------------------------------------------------------------------------------------------
// hard selection.  The softmax is evaluated the way an fp32 library softmax does (subtract the
// maximum, exponentiate, divide by the sum, round to the logits dtype) with a correctly rounded
// exponential, then the FIRST maximum of the rounded probabilities wins.  For two ops the
// straight-through value y_hard - y_soft + y_soft is exactly {0,1}.
// ---------------------------------------------------------------------------------------------
NATSL_DEVICE int select_first_max(float x0, float x1, int dtype) {
  const float mx = fmaxf(x0, x1);
  const float e0 = (float)exp((double)(x0 - mx)), e1 = (float)exp((double)(x1 - mx));
  const float s = e0 + e1;
  float y0 = e0 / s, y1 = e1 / s;
  if (dtype == NATSL_BF16) {
    y0 = bf16_to_f32(f32_to_bf16(y0));
    y1 = bf16_to_f32(f32_to_bf16(y1));
  }
  return y1 > y0 ? 1 : 0;  // ties (and NaN, outside the contract) go to the first index
}

// one workgroup per (sequence, selector head)
__global__ __launch_bounds__(256) void hard_select_kernel(const void* logits, void* types, int32_t* nblk, int TN, int HN, int dtype,
                                                          int force_last, const SeqRow* seqs, int n_seqs, int block_unused) {
  const int n = blockIdx.x / HN, hn = blockIdx.x % HN;
  int bos_nats, tn;
  if (seqs == nullptr) {
    bos_nats = n * TN;
    tn = TN;
  } else {
    bos_nats = seqs[n].bos_nats;
    tn = (n + 1 < n_seqs ? seqs[n + 1].bos_nats : TN) - bos_nats;
  }
  int c0 = 0, c1 = 0;
  for (int c = threadIdx.x; c < tn; c += 256) {
    const size_t i = ((size_t)(bos_nats + c) * HN + hn) * 2;
    const int sel = select_first_max(load_as_f32(logits, dtype, i), load_as_f32(logits, dtype, i + 1), dtype);
    float t0 = sel == 0 ? 1.f : 0.f, t1 = sel == 1 ? 1.f : 0.f;
    if (force_last && c == tn - 1) t0 = t1 = 1.f;
    store_from_f32(types, dtype, i, t0);
    store_from_f32(types, dtype, i + 1, t1);
    c0 += (int)t0;
    c1 += (int)t1;
  }
  if (nblk == nullptr) return;
  __shared__ int red[2][256];
  red[0][threadIdx.x] = c0;
  red[1][threadIdx.x] = c1;
  __syncthreads();
  for (int s = 128; s > 0; s >>= 1) {
    if ((int)threadIdx.x < s) {
      red[0][threadIdx.x] += red[0][threadIdx.x + s];
      red[1][threadIdx.x] += red[1][threadIdx.x + s];
    }
    __syncthreads();
  }
  if (threadIdx.x == 0) {
    nblk[((size_t)n * HN + hn) * 2] = red[0][0];
    nblk[((size_t)n * HN + hn) * 2 + 1] = red[1][0];
  }
}

// ---------------------------------------------------------------------------------------------
// routing tables.  One workgroup per (sequence, selector head) builds, for both ops, the sorted
// list of selected block ids (a stable compaction == the reference's where + sort), the counts,
// and the two prefix-count tables; a second single-workgroup kernel turns the per-(b,hn)
// linear chunk counts into offsets and fills the (flat_bh, j) index rows.
// ---------------------------------------------------------------------------------------------
constexpr int ROUTE_MAX_TN = 16384;

__global__ __launch_bounds__(256) void route_kernel(const void* types, int dtype, int TN, int HN, int T, int block, int32_t* idx,
                                                    int32_t* nblk, int64_t* starting_h_idx, int64_t* attn_n_iters,
                                                    const SeqRow* seqs, int n_seqs) {
  extern __shared__ int dyn[];  // [2][tn+1] exclusive prefix counts
  const int n = blockIdx.x / HN, hn = blockIdx.x % HN;
  int bos_nats, tn, len;
  if (seqs == nullptr) {
    bos_nats = n * TN;
    tn = TN;
    len = T;
  } else {
    bos_nats = seqs[n].bos_nats;
    tn = (n + 1 < n_seqs ? seqs[n + 1].bos_nats : TN) - bos_nats;
    len = seqs[n].eos - seqs[n].bos;
  }
  int* pa = dyn;            // attention prefix, tn+1 entries
  int* pl = dyn + (tn + 1); // linear prefix
  // each thread owns a contiguous segment of blocks
  const int seg = (tn + 255) / 256;
  const int lo = min(tn, (int)threadIdx.x * seg), hi = min(tn, lo + seg);
  int ca = 0, cl = 0;
  for (int c = lo; c < hi; ++c) {
    const size_t i = ((size_t)(bos_nats + c) * HN + hn) * 2;
    ca += rintf(load_as_f32(types, dtype, i)) == 1.f;
    cl += rintf(load_as_f32(types, dtype, i + 1)) == 1.f;
  }
  __shared__ int sa[257], sl[257];
  sa[threadIdx.x + 1] = ca;
  sl[threadIdx.x + 1] = cl;
  if (threadIdx.x == 0) sa[0] = sl[0] = 0;
  __syncthreads();
  if (threadIdx.x == 0)
    for (int i = 1; i <= 256; ++i) {
      sa[i] += sa[i - 1];
      sl[i] += sl[i - 1];
    }
  __syncthreads();
  int ra = sa[threadIdx.x], rl = sl[threadIdx.x];
  const int na = sa[256], nl = sl[256];
  for (int c = lo; c < hi; ++c) {
    const size_t i = ((size_t)(bos_nats + c) * HN + hn) * 2;
    pa[c] = ra;
    pl[c] = rl;
    if (rintf(load_as_f32(types, dtype, i)) == 1.f) {
      if (idx) idx[((size_t)(bos_nats + ra) * HN + hn) * 2] = c;
      ++ra;
    }
    if (rintf(load_as_f32(types, dtype, i + 1)) == 1.f) {
      if (idx) idx[((size_t)(bos_nats + rl) * HN + hn) * 2 + 1] = c;
      ++rl;
    }
  }
  if (threadIdx.x == 0) {
    pa[tn] = na;
    pl[tn] = nl;
    if (nblk) {
      nblk[((size_t)n * HN + hn) * 2] = na;
      nblk[((size_t)n * HN + hn) * 2 + 1] = nl;
    }
  }
  // sentinel padding
  if (idx)
    for (int c = threadIdx.x; c < tn; c += 256) {
      if (c >= na) idx[((size_t)(bos_nats + c) * HN + hn) * 2] = tn;
      if (c >= nl) idx[((size_t)(bos_nats + c) * HN + hn) * 2 + 1] = tn;
    }
  __syncthreads();
  if (seqs != nullptr) return;
  if (starting_h_idx) {
    const int NT = (len + 63) / 64;
    for (int c = threadIdx.x; c < NT; c += 256) {
      // linear blocks j with j*block < c*64  <=>  j < ceil(c*64/block)
      const int jmax = min(tn, (c * 64 + block - 1) / block);
      starting_h_idx[((size_t)n * NT + c) * HN + hn] = pl[jmax];
    }
  }
  if (attn_n_iters) {
    const int NQ = (len + 127) / 128;
    for (int i = threadIdx.x; i < NQ; i += 256) {
      // attention blocks j with (j+1)*block <= i*128  <=>  j < floor(i*128/block)
      const int jmax = min(tn, (i * 128) / block);
      attn_n_iters[((size_t)n * NQ + i) * HN + hn] = pa[jmax];
    }
  }
}

__global__ __launch_bounds__(256) void route_offsets_kernel(const int32_t* nblk, int n_bh, int block, int64_t* offsets, int32_t* chunk_indices) {
  __shared__ long long run;
  if (threadIdx.x == 0) run = 0;
  __syncthreads();
  // serial over (b,hn) pairs (a few hundred), parallel over each pair's rows
  for (int bh = 0; bh < n_bh; ++bh) {
    const long long base = run;
    const int cnt = (int)(((long long)nblk[2 * bh + 1] * block + 63) / 64);
    if (chunk_indices)
      for (int j = threadIdx.x; j < cnt; j += 256) {
        chunk_indices[(base + j) * 2] = bh;
        chunk_indices[(base + j) * 2 + 1] = j;
      }
    __syncthreads();
    if (threadIdx.x == 0) {
      if (offsets) offsets[bh] = base;
      run = base + cnt;
    }
    __syncthreads();
  }
  if (threadIdx.x == 0 && offsets) offsets[n_bh] = run;
}

}  // namespace natsl

using namespace natsl;

extern "C" int natsl_version(void) { return 100; }
extern "C" const char* natsl_last_error(void) { return error_buffer(); }

extern "C" int natsl_mean_pool(const void* hidden, void* pooled, int B, int T, int D, int block, int dtype,
                               const natsl_seq_row* seqs, int n_seqs, int total_units, natsl_stream_t stream) {
  if (!hidden || !pooled) return fail(NATSL_ERR_INVALID, "mean_pool: null pointer argument");
  if (B <= 0 || T <= 0 || D <= 0 || block <= 0) return fail(NATSL_ERR_INVALID, "mean_pool: non-positive dimension");
  if (dtype != NATSL_BF16 && dtype != NATSL_F32) return fail(NATSL_ERR_UNSUPPORTED, "mean_pool: dtype %d", dtype);
  if (seqs && (B != 1 || n_seqs <= 0 || total_units <= 0)) return fail(NATSL_ERR_INVALID, "mean_pool: packed input needs B == 1 and total_units = number of blocks");
  const int nb = cdiv(T, block);
  const int total = seqs ? total_units : B * nb;
  dim3 grid(cdiv(D, 256 * 8), total);
  hipLaunchKernelGGL(mean_pool_kernel, grid, dim3(256), 0, reinterpret_cast<hipStream_t>(stream), hidden, pooled, B, T, D, block,
                     dtype, reinterpret_cast<const SeqRow*>(seqs), n_seqs, nb);
  return check_launch("natsl_mean_pool");
}

extern "C" int natsl_hard_select(const void* logits, void* types, int32_t* n_nats_blocks, int B, int TN, int HN, int dtype,
                                 int force_last, const natsl_seq_row* seqs, int n_seqs, int total_units,
                                 natsl_stream_t stream) {
  (void)total_units;
  if (!logits || !types) return fail(NATSL_ERR_INVALID, "hard_select: null pointer argument");
  if (B <= 0 || TN <= 0 || HN <= 0) return fail(NATSL_ERR_INVALID, "hard_select: non-positive dimension");
  if (dtype != NATSL_BF16 && dtype != NATSL_F32) return fail(NATSL_ERR_UNSUPPORTED, "hard_select: dtype %d", dtype);
  if (seqs && (B != 1 || n_seqs <= 0)) return fail(NATSL_ERR_INVALID, "hard_select: packed input needs B == 1");
  const int n = seqs ? n_seqs : B;
  hipLaunchKernelGGL(hard_select_kernel, dim3(n * HN), dim3(256), 0, reinterpret_cast<hipStream_t>(stream), logits, types,
                     n_nats_blocks, TN, HN, dtype, force_last, reinterpret_cast<const SeqRow*>(seqs), n_seqs, 0);
  return check_launch("natsl_hard_select");
}

extern "C" int natsl_route(const void* types, int types_dtype, int B, int TN, int HN, int T, int block,
                           int32_t* nats_block_indices, int32_t* n_nats_blocks, int64_t* linear_chunk_offsets,
                           int32_t* chunk_indices_linear, int64_t* starting_h_idx, int64_t* attn_n_iters,
                           const natsl_seq_row* seqs, int n_seqs, int total_units, natsl_stream_t stream) {
  (void)total_units;
  if (!types) return fail(NATSL_ERR_INVALID, "route: null types pointer");
  if (B <= 0 || TN <= 0 || HN <= 0 || T <= 0) return fail(NATSL_ERR_INVALID, "route: non-positive dimension");
  if (types_dtype != NATSL_BF16 && types_dtype != NATSL_F32) return fail(NATSL_ERR_UNSUPPORTED, "route: dtype %d", types_dtype);
  if (block < 64 || block % 64) return fail(NATSL_ERR_UNSUPPORTED, "route: block size %d must be a multiple of 64", block);
  if (TN > ROUTE_MAX_TN) return fail(NATSL_ERR_UNSUPPORTED, "route: more than %d selector blocks per sequence", ROUTE_MAX_TN);
  if (seqs && (B != 1 || n_seqs <= 0)) return fail(NATSL_ERR_INVALID, "route: packed input needs B == 1");
  if (seqs && (starting_h_idx || attn_n_iters)) return fail(NATSL_ERR_UNSUPPORTED, "route: starting_h_idx / attn_n_iters are defined for regular batches only");
  if ((linear_chunk_offsets || chunk_indices_linear) && !n_nats_blocks)
    return fail(NATSL_ERR_INVALID, "route: offsets need n_nats_blocks as well");
  const int n = seqs ? n_seqs : B;
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  const size_t lds = (size_t)2 * (TN + 1) * sizeof(int);
  hipLaunchKernelGGL(route_kernel, dim3(n * HN), dim3(256), lds, s, types, types_dtype, TN, HN, T, block, nats_block_indices,
                     n_nats_blocks, starting_h_idx, attn_n_iters, reinterpret_cast<const SeqRow*>(seqs), n_seqs);
  int rc = check_launch("natsl_route");
  if (rc != NATSL_OK) return rc;
  if (linear_chunk_offsets || chunk_indices_linear) {
    hipLaunchKernelGGL(route_offsets_kernel, dim3(1), dim3(256), 0, s, n_nats_blocks, n * HN, block, linear_chunk_offsets, chunk_indices_linear);
    rc = check_launch("natsl_route(offsets)");
  }
  return rc;
}
