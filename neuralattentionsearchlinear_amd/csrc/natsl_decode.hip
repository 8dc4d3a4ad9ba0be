// Decode-time kernels of the NAtS-L hybrid layer for gfx950: tokens that continue the current
// (incomplete) selector block of a sequence whose state is cached.
//
//   gdn_recurrent_kernel   the gated delta rule token by token on a cached state
//                          (src/nats/ops/gated_delta_rule/fused_recurrent.py:28-358, the branch the
//                          reference takes at decode: UPDATE_HS_FOR_EACH_ITER with one selector block)
//   attn_masked_kernel     softmax attention of a few queries over cached keys/values under an explicit
//                          visibility mask (the scaled_dot_product_attention call at
//                          src/nats/ops/mixed_ops/mixed_attn_gdn.py:475-481)
//
// Both are memory-bound: the first reads and writes the fp32 state once, the second reads K and V once per
// query.  No matrix cores: per token the delta rule is two K-long dot products and one rank-1 update.
#include "natsl_device.h"
#include "natsl_host.h"
#include "../../include/natsl.h"

namespace natsl {

NATSL_DEVICE float ld_any(const void* p, int dtype, size_t i) {
  return dtype == NATSL_F32 ? reinterpret_cast<const float*>(p)[i] : bf16_to_f32(reinterpret_cast<const bf16_t*>(p)[i]);
}
NATSL_DEVICE void st_any(void* p, int dtype, size_t i, float x) {
  if (dtype == NATSL_F32) reinterpret_cast<float*>(p)[i] = x;
  else reinterpret_cast<bf16_t*>(p)[i] = f32_to_bf16(x);
}

// ---------------------------------------------------------------------------------------------
// gated delta rule, recurrent form
// ---------------------------------------------------------------------------------------------
// One wave owns the state slice S[0:K][16 columns] of one (sequence, head): lane = (kq, col) with
// kq = lane/16 the quarter of the K rows it keeps in registers (K/4 floats) and col = lane%16.  Sums over
// K are K/4 in-lane terms plus two cross-lane steps; no LDS, no barriers.  A workgroup is four such waves
// (64 columns).
struct RecurrentParams {
  const void* q; const void* k; const void* v; const float* g; const float* g_cumsum; const void* beta;
  const float* h0; float* hcur; void* o; float* ht;
  const void* types; int types_dtype; const int32_t* n_in_block;
  int N, T, H, HN, V, block, dtype;
  float scale; int decay, l2norm, n_in_block_scalar;
  int query_only;   // outputs from the decayed block-start state, no state update (the 'attn' mode of decode)
};

// DELTA = false is the Mamba form (src/nats/ops/mamba/fused_recurrent.py:150-178): S += k v^T, no beta, no norms.
template <int DK, bool DELTA>
__global__ __launch_bounds__(256) void gdn_recurrent_kernel(const RecurrentParams p) {
  constexpr int R = DK / 4;  // state rows per lane
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int kq = lane >> 4, col = lane & 15;
  const int nh = blockIdx.y, n = nh / p.H, h = nh % p.H;
  const int vc = (blockIdx.x * 4 + wave) * 16 + col;
  if (vc >= p.V) return;  // V is a multiple of 16: whole waves leave together
  const int hn = h / (p.H / p.HN);

  float S[R], Scur[R];
#pragma unroll
  for (int r = 0; r < R; ++r) {
    const size_t i = ((size_t)nh * DK + kq * R + r) * p.V + vc;
    S[r] = p.h0 ? p.h0[i] : 0.f;
    Scur[r] = p.hcur[i];
  }
  float gcum = p.g_cumsum ? p.g_cumsum[nh] : 0.f;
  const int n_in = p.n_in_block ? p.n_in_block[n] : p.n_in_block_scalar;
  const int n_tok = min(p.T, p.block - n_in);  // fused_recurrent.py:144
  if (p.query_only) {
    // The mode in which the linear operator does not run on the incomplete block: a token reads the state that entered
    // the block, decayed by the block's g up to and including itself (what the chunked forward without its intra-chunk
    // term gives, and what the reference's UPDATE_HS_FOR_EACH_ITER = False branch gives for a one-token step,
    // fused_recurrent.py:156-201 as called at mixed_attn_gdn.py:510-527); nothing is written back.
    const float e0 = __expf(gcum);
#pragma unroll
    for (int r = 0; r < R; ++r) S[r] = Scur[r] * e0;
    for (int t = 0; t < n_tok; ++t) {
      const size_t tok = (size_t)n * p.T + t;
      float qq[R];
      float sq = 0.f;
#pragma unroll
      for (int r = 0; r < R; ++r) {
        qq[r] = ld_any(p.q, p.dtype, (tok * p.H + h) * DK + kq * R + r);
        sq += qq[r] * qq[r];
      }
      float rq = 1.f;
      if (DELTA && p.l2norm) {
        sq += __shfl_xor(sq, 16); sq += __shfl_xor(sq, 32);
        rq = 1.f / sqrtf(sq + 1e-6f);
      }
      const float eg = __expf(p.g[tok * p.H + h]);
      float hq = 0.f;
#pragma unroll
      for (int r = 0; r < R; ++r) {
        S[r] *= eg;
        hq += S[r] * qq[r];
      }
      hq += __shfl_xor(hq, 16); hq += __shfl_xor(hq, 32);
      if (kq == 0) st_any(p.o, p.dtype, (tok * p.H + h) * p.V + vc, hq * rq * p.scale);
    }
    return;
  }

  for (int t = 0; t < n_tok; ++t) {
    const size_t tok = (size_t)n * p.T + t;
    float kk[R], qq[R];
    float sk = 0.f, sq = 0.f;
#pragma unroll
    for (int r = 0; r < R; ++r) {
      kk[r] = ld_any(p.k, p.dtype, (tok * p.H + h) * DK + kq * R + r);
      qq[r] = ld_any(p.q, p.dtype, (tok * p.H + h) * DK + kq * R + r);
      sk += kk[r] * kk[r];
      sq += qq[r] * qq[r];
    }
    if (DELTA && p.l2norm) {
      sk += __shfl_xor(sk, 16); sk += __shfl_xor(sk, 32);
      sq += __shfl_xor(sq, 16); sq += __shfl_xor(sq, 32);
      const float rk = 1.f / sqrtf(sk + 1e-6f), rq = 1.f / sqrtf(sq + 1e-6f);  // :165-169
#pragma unroll
      for (int r = 0; r < R; ++r) { kk[r] *= rk; qq[r] *= rq; }
    }
    const float gt = p.g[tok * p.H + h];
    const float eg = __expf(gt);
    if (p.decay) gcum += gt;                                    // :183-184
    const float bt = DELTA ? ld_any(p.beta, p.dtype, tok * p.H + h) : 1.f;
    const float vt = ld_any(p.v, p.dtype, (tok * p.H + h) * p.V + vc);
    float hk = 0.f;
#pragma unroll
    for (int r = 0; r < R; ++r) {
      S[r] *= eg;                                               // :182
      hk += S[r] * kk[r];
    }
    hk += __shfl_xor(hk, 16); hk += __shfl_xor(hk, 32);
    const float dv = DELTA ? bt * (vt - hk) : vt;               // :195
    float hq = 0.f;
#pragma unroll
    for (int r = 0; r < R; ++r) {
      S[r] += kk[r] * dv;                                       // :196
      hq += S[r] * qq[r];
    }
    hq += __shfl_xor(hq, 16); hq += __shfl_xor(hq, 32);
    if (kq == 0) st_any(p.o, p.dtype, (tok * p.H + h) * p.V + vc, hq * p.scale);  // :199-201
  }
  // the selector block is complete: a block not typed linear restores the state it started from
  // (times the block's total decay when asked), and that becomes the next block's start (:343-352)
  if (n_in + p.T >= p.block) {
    const size_t ti = ((size_t)n * p.HN + hn) * 2 + 1;
    const float ty = ld_any(p.types, p.types_dtype, ti);
    const bool is_delta = rintf(ty) == 1.0f;
    const float f = p.decay ? __expf(gcum) : 1.f;
#pragma unroll
    for (int r = 0; r < R; ++r) {
      if (!is_delta) S[r] = Scur[r] * f;
      p.hcur[((size_t)nh * DK + kq * R + r) * p.V + vc] = S[r];
    }
  }
  if (p.ht) {
#pragma unroll
    for (int r = 0; r < R; ++r) p.ht[((size_t)nh * DK + kq * R + r) * p.V + vc] = S[r];
  }
}

// ---------------------------------------------------------------------------------------------
// masked attention of a few queries
// ---------------------------------------------------------------------------------------------
// One workgroup of ATTN_WAVES waves per (sequence, query head, query); the waves take the 64-key chunks
// round-robin and keep their own running (max, sum, accumulator), joined through LDS at the end.  Within a
// chunk: 16 lanes per key row for the scores (coalesced), lane = key for the softmax, lane = DV/64 adjacent value
// columns for the output (a row of V is one coalesced read per wave; ATTN_VROWS rows are requested before they are
// used, and each key's probability is broadcast with a lane read).  Hidden keys get probability 0; a query that
// sees no key gives 0.
constexpr int ATTN_WAVES = 16;
constexpr int ATTN_VROWS = 16;  // rows of V requested before any is used

struct MaskedAttnParams {
  const void* q; const void* k; const void* v; const uint8_t* mask; void* o;
  int B, TQ, TK, HQ, HKV, HM, dtype;
  float scale_log2;
  int nsplit;        // workgroups per query, each owning every nsplit-th group of ATTN_WAVES chunks
  float* partials;   // nsplit > 1: [B, TQ, HQ, nsplit, 2 + DV] running (max, sum, accumulator) of each split
  size_t k_bs, v_bs; // elements from one sequence's keys / values to the next (TK * HKV * D when dense)
};

template <int DK, int DV>
__global__ __launch_bounds__(64 * ATTN_WAVES) void attn_masked_kernel(const MaskedAttnParams p) {
  constexpr int CPL = DV / 64;  // value columns per lane (DV = 64 or 128)
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int tq = blockIdx.x, hq = blockIdx.y, b = blockIdx.z / p.nsplit, split = blockIdx.z % p.nsplit;
  const int hkv = hq / (p.HQ / p.HKV), hm = hq / (p.HQ / p.HM);
  __shared__ float qs[DK];
  __shared__ float part_m[ATTN_WAVES], part_l[ATTN_WAVES], part_acc[ATTN_WAVES][DV];
  __shared__ float sc[ATTN_WAVES][64];
  for (int i = threadIdx.x; i < DK; i += 64 * ATTN_WAVES) qs[i] = ld_any(p.q, p.dtype, (((size_t)b * p.TQ + tq) * p.HQ + hq) * DK + i);
  __syncthreads();
  const uint8_t* mrow = p.mask + (((size_t)b * p.HM + hm) * p.TQ + tq) * p.TK;

  float m_run = -INFINITY, l_run = 0.f, acc[CPL];
#pragma unroll
  for (int j = 0; j < CPL; ++j) acc[j] = 0.f;
  // bf16 values are read like the keys, 16 lanes per row and 16 (8) bytes per lane, four rows per instruction: a lane then
  // sums DV/16 adjacent columns over every fourth row, and the four row groups are added up once, at the end.  (One row
  // per instruction with 4 bytes per lane, the f32 path below, keeps the memory pipe well below its rate.)
  constexpr int EV = DV / 16;
  float acc16[EV];
#pragma unroll
  for (int j = 0; j < EV; ++j) acc16[j] = 0.f;
  const bool wide_v = p.dtype == NATSL_BF16;
  for (int k0 = 64 * (split * ATTN_WAVES + wave); k0 < p.TK; k0 += 64 * ATTN_WAVES * p.nsplit) {
    // scores: 16 lanes share a key row (16 bytes = 8 (bf16) or 4 (f32) elements each, one coalesced 256/512-byte
    // read per row), four rows per pass; the 16 partial dot products are summed across the lanes and the row's
    // score is handed to lane = key through LDS
    {
      const int sub = lane & 15, rowg = lane >> 4;
      constexpr int EPL = DK / 16;  // elements of a row per lane
#pragma unroll 4
      for (int pass = 0; pass < 16; ++pass) {
        const int kidx = min(k0 + 4 * pass + rowg, p.TK - 1);
        const size_t kb = (size_t)b * p.k_bs + ((size_t)kidx * p.HKV + hkv) * DK + EPL * sub;
        float d = 0.f;
        if (p.dtype == NATSL_BF16) {
          if (EPL == 8) {
            const u32x4 kv = *reinterpret_cast<const u32x4*>(reinterpret_cast<const bf16_t*>(p.k) + kb);
#pragma unroll
            for (int e = 0; e < 4; ++e) {
              d += qs[8 * sub + 2 * e] * __uint_as_float(kv[e] << 16);
              d += qs[8 * sub + 2 * e + 1] * __uint_as_float(kv[e] & 0xffff0000u);
            }
          } else {
            const u32x2 kv = *reinterpret_cast<const u32x2*>(reinterpret_cast<const bf16_t*>(p.k) + kb);
#pragma unroll
            for (int e = 0; e < 2; ++e) {
              d += qs[4 * sub + 2 * e] * __uint_as_float(kv[e] << 16);
              d += qs[4 * sub + 2 * e + 1] * __uint_as_float(kv[e] & 0xffff0000u);
            }
          }
        } else {
#pragma unroll
          for (int e = 0; e < EPL; ++e) d += qs[EPL * sub + e] * reinterpret_cast<const float*>(p.k)[kb + e];
        }
        d += __shfl_xor(d, 1); d += __shfl_xor(d, 2); d += __shfl_xor(d, 4); d += __shfl_xor(d, 8);
        if (sub == 0) sc[wave][4 * pass + rowg] = d;
      }
    }
    __builtin_amdgcn_s_waitcnt(0xc07f);  // this wave's LDS writes have landed
    __builtin_amdgcn_wave_barrier();
    const int key = k0 + lane;
    const bool vis = key < p.TK && mrow[key] != 0;
    const float s = vis ? sc[wave][lane] * p.scale_log2 : -INFINITY;
    __builtin_amdgcn_wave_barrier();
    float m_new = s;
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) m_new = fmaxf(m_new, __shfl_xor(m_new, off));
    if (m_new == -INFINITY) continue;  // no visible key in this chunk (wave-uniform)
    m_new = fmaxf(m_new, m_run);
    const float alpha = __builtin_amdgcn_exp2f(m_run - m_new);  // 0 on the first visible chunk
    const float pr = vis ? __builtin_amdgcn_exp2f(s - m_new) : 0.f;
    float ps = pr;
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) ps += __shfl_xor(ps, off);
    l_run = l_run * alpha + ps;
    m_run = m_new;
#pragma unroll
    for (int j = 0; j < CPL; ++j) acc[j] *= alpha;
    if (wide_v) {
#pragma unroll
      for (int j = 0; j < EV; ++j) acc16[j] *= alpha;
      // the probabilities go to LDS (lane = key there) and come back to the lanes of their rows
      sc[wave][lane] = pr;
      __builtin_amdgcn_s_waitcnt(0xc07f);
      __builtin_amdgcn_wave_barrier();
      const int sub = lane & 15, rowg = lane >> 4;
#pragma unroll 4
      for (int pass = 0; pass < 16; ++pass) {
        const int kidx = min(k0 + 4 * pass + rowg, p.TK - 1);   // keys past the end are clamped (their probability is 0)
        const bf16_t* vrow = reinterpret_cast<const bf16_t*>(p.v) + (size_t)b * p.v_bs + ((size_t)kidx * p.HKV + hkv) * DV + EV * sub;
        const float pk = sc[wave][4 * pass + rowg];
        u32x4 w;
        if (EV == 8) {
          w = *reinterpret_cast<const u32x4*>(vrow);
        } else {
          const u32x2 w2 = *reinterpret_cast<const u32x2*>(vrow);
          w = u32x4{w2[0], w2[1], 0u, 0u};
        }
#pragma unroll
        for (int e = 0; e < EV / 2; ++e) {
          acc16[2 * e] += pk * __uint_as_float(w[e] << 16);
          acc16[2 * e + 1] += pk * __uint_as_float(w[e] & 0xffff0000u);
        }
      }
      __builtin_amdgcn_wave_barrier();   // sc[wave] is written again by the next chunk's scores
      continue;
    }
    // rows of V: keys past the end are clamped (their probability is 0)
    for (int kk = 0; kk < 64; kk += ATTN_VROWS) {
      float vv[ATTN_VROWS][CPL];
#pragma unroll
      for (int u = 0; u < ATTN_VROWS; ++u) {
        const int kidx = min(k0 + kk + u, p.TK - 1);
        const size_t vb = (size_t)b * p.v_bs + ((size_t)kidx * p.HKV + hkv) * DV + CPL * lane;
        if (p.dtype == NATSL_BF16) {
          if (CPL == 2) {
            const unsigned w = *reinterpret_cast<const unsigned*>(reinterpret_cast<const bf16_t*>(p.v) + vb);
            vv[u][0] = __uint_as_float(w << 16);
            vv[u][CPL - 1] = __uint_as_float(w & 0xffff0000u);
          } else {
            vv[u][0] = bf16_to_f32(reinterpret_cast<const bf16_t*>(p.v)[vb]);
          }
        } else {
#pragma unroll
          for (int j = 0; j < CPL; ++j) vv[u][j] = reinterpret_cast<const float*>(p.v)[vb + j];
        }
      }
#pragma unroll
      for (int u = 0; u < ATTN_VROWS; ++u) {
        const float pk = __uint_as_float(__builtin_amdgcn_readlane(__float_as_uint(pr), kk + u));
#pragma unroll
        for (int j = 0; j < CPL; ++j) acc[j] += pk * vv[u][j];
      }
    }
  }
  // join the waves
  if (lane == 0) { part_m[wave] = m_run; part_l[wave] = l_run; }
  if (wide_v) {
#pragma unroll
    for (int j = 0; j < EV; ++j) {
      acc16[j] += __shfl_xor(acc16[j], 16);
      acc16[j] += __shfl_xor(acc16[j], 32);
    }
    if (lane < 16) {
#pragma unroll
      for (int j = 0; j < EV; ++j) part_acc[wave][EV * lane + j] = acc16[j];
    }
  } else {
#pragma unroll
    for (int j = 0; j < CPL; ++j) part_acc[wave][CPL * lane + j] = acc[j];
  }
  __syncthreads();
  if (wave == 0) {
    float m = -INFINITY;
#pragma unroll
    for (int w = 0; w < ATTN_WAVES; ++w) m = fmaxf(m, part_m[w]);
    float l = 0.f, o[CPL];
#pragma unroll
    for (int j = 0; j < CPL; ++j) o[j] = 0.f;
#pragma unroll
    for (int w = 0; w < ATTN_WAVES; ++w) {
      const float f = part_m[w] == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(part_m[w] - m);
      l += f * part_l[w];
#pragma unroll
      for (int j = 0; j < CPL; ++j) o[j] += f * part_acc[w][CPL * lane + j];
    }
    if (p.nsplit > 1) {
      float* dst = p.partials + ((((size_t)b * p.TQ + tq) * p.HQ + hq) * p.nsplit + split) * (2 + DV);
      if (lane == 0) { dst[0] = m; dst[1] = l; }
#pragma unroll
      for (int j = 0; j < CPL; ++j) dst[2 + CPL * lane + j] = o[j];
      return;
    }
    const float inv = l > 0.f ? 1.f / l : 0.f;
#pragma unroll
    for (int j = 0; j < CPL; ++j) st_any(p.o, p.dtype, (((size_t)b * p.TQ + tq) * p.HQ + hq) * DV + CPL * lane + j, o[j] * inv);
  }
}

// joins the splits of one query: one wave per (sequence, query, head)
template <int DV>
__global__ __launch_bounds__(64) void attn_masked_join_kernel(const MaskedAttnParams p) {
  constexpr int CPL = DV / 64;
  const int lane = threadIdx.x;
  const size_t row = ((size_t)blockIdx.z * p.TQ + blockIdx.x) * p.HQ + blockIdx.y;
  const float* src = p.partials + row * p.nsplit * (2 + DV);
  float m = -INFINITY;
  for (int sidx = 0; sidx < p.nsplit; ++sidx) m = fmaxf(m, src[sidx * (2 + DV)]);
  float l = 0.f, o[CPL];
#pragma unroll
  for (int j = 0; j < CPL; ++j) o[j] = 0.f;
  for (int sidx = 0; sidx < p.nsplit; ++sidx) {
    const float* ps = src + sidx * (2 + DV);
    const float f = ps[0] == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(ps[0] - m);
    l += f * ps[1];
#pragma unroll
    for (int j = 0; j < CPL; ++j) o[j] += f * ps[2 + CPL * lane + j];
  }
  const float inv = l > 0.f ? 1.f / l : 0.f;
#pragma unroll
  for (int j = 0; j < CPL; ++j) st_any(p.o, p.dtype, row * DV + CPL * lane + j, o[j] * inv);
}

}  // namespace natsl

using namespace natsl;

static int recurrent_fwd(bool delta, const char* what, const void* q, const void* k, const void* v, const float* g,
                         const float* g_cumsum, const void* beta, const float* h0, float* h_block_start, void* o, float* ht,
                         const void* types, int types_dtype, const int32_t* n_tokens_in_block, int n_tokens_in_block_scalar,
                         int N, int T, int H, int HN, int K, int V, int block, float scale, int flags, int dtype,
                         natsl_stream_t stream) {
  const bool query_only = (flags & NATSL_QUERY_ONLY) != 0;
  if (!q || !g || !h_block_start || !o || !types || (!query_only && (!k || !v || (delta && !beta))))
    return fail(NATSL_ERR_INVALID, "%s: null pointer argument", what);
  if (dtype != NATSL_BF16 && dtype != NATSL_F32) return fail(NATSL_ERR_UNSUPPORTED, "%s: tensors must be f32 or bf16", what);
  if (types_dtype != NATSL_BF16 && types_dtype != NATSL_F32) return fail(NATSL_ERR_UNSUPPORTED, "%s: block types must be f32 or bf16", what);
  if (N <= 0 || T <= 0 || H <= 0 || HN <= 0 || block <= 0) return fail(NATSL_ERR_INVALID, "%s: non-positive dimension", what);
  if (H % HN) return fail(NATSL_ERR_INVALID, "%s: H=%d must be a multiple of HN=%d", what, H, HN);
  if (V <= 0 || V % 16) return fail(NATSL_ERR_UNSUPPORTED, "%s: V=%d must be a multiple of 16", what, V);
  if ((long long)N * H > 65535) return fail(NATSL_ERR_UNSUPPORTED, "%s: N*H=%lld above 65535", what, (long long)N * H);
  if (!n_tokens_in_block && (n_tokens_in_block_scalar < 0 || n_tokens_in_block_scalar >= block))
    return fail(NATSL_ERR_INVALID, "%s: n_tokens_in_current_block=%d outside [0, %d)", what, n_tokens_in_block_scalar, block);
  RecurrentParams p;
  p.q = q; p.k = k; p.v = v; p.g = g; p.g_cumsum = g_cumsum; p.beta = beta; p.h0 = h0; p.hcur = h_block_start; p.o = o; p.ht = ht;
  p.types = types; p.types_dtype = types_dtype; p.n_in_block = n_tokens_in_block; p.n_in_block_scalar = n_tokens_in_block_scalar;
  p.N = N; p.T = T; p.H = H; p.HN = HN; p.V = V; p.block = block; p.dtype = dtype; p.scale = scale;
  p.decay = (flags & NATSL_DECAY_NON_LINEAR) != 0; p.l2norm = (flags & NATSL_QK_L2NORM) != 0; p.query_only = query_only ? 1 : 0;
  const dim3 grid(cdiv(V, 64), N * H);
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  if (K == 128 && delta) hipLaunchKernelGGL((gdn_recurrent_kernel<128, true>), grid, dim3(256), 0, s, p);
  else if (K == 64 && delta) hipLaunchKernelGGL((gdn_recurrent_kernel<64, true>), grid, dim3(256), 0, s, p);
  else if (K == 128) hipLaunchKernelGGL((gdn_recurrent_kernel<128, false>), grid, dim3(256), 0, s, p);
  else if (K == 64) hipLaunchKernelGGL((gdn_recurrent_kernel<64, false>), grid, dim3(256), 0, s, p);
  else if (K == 192 && delta) hipLaunchKernelGGL((gdn_recurrent_kernel<192, true>), grid, dim3(256), 0, s, p);
  else if (K == 192) hipLaunchKernelGGL((gdn_recurrent_kernel<192, false>), grid, dim3(256), 0, s, p);
  else return fail(NATSL_ERR_UNSUPPORTED, "%s: K=%d not built (supported: 64, 128, 192)", what, K);
  return check_launch(what);
}

extern "C" int natsl_gdn_recurrent_fwd(const void* q, const void* k, const void* v, const float* g, const float* g_cumsum,
                                       const void* beta, const float* h0, float* h_block_start, void* o, float* ht,
                                       const void* types, int types_dtype, const int32_t* n_tokens_in_block,
                                       int n_tokens_in_block_scalar, int N, int T, int H, int HN, int K, int V, int block,
                                       float scale, int flags, int dtype, natsl_stream_t stream) {
  return recurrent_fwd(true, "natsl_gdn_recurrent_fwd", q, k, v, g, g_cumsum, beta, h0, h_block_start, o, ht, types, types_dtype,
                       n_tokens_in_block, n_tokens_in_block_scalar, N, T, H, HN, K, V, block, scale, flags, dtype, stream);
}

extern "C" int natsl_mamba_recurrent_fwd(const void* q, const void* k, const void* v, const float* g, const float* g_cumsum,
                                         const float* h0, float* h_block_start, void* o, float* ht, const void* types,
                                         int types_dtype, const int32_t* n_tokens_in_block, int n_tokens_in_block_scalar, int N,
                                         int T, int H, int HN, int K, int V, int block, float scale, int flags, int dtype,
                                         natsl_stream_t stream) {
  return recurrent_fwd(false, "natsl_mamba_recurrent_fwd", q, k, v, g, g_cumsum, nullptr, h0, h_block_start, o, ht, types,
                       types_dtype, n_tokens_in_block, n_tokens_in_block_scalar, N, T, H, HN, K, V, block, scale, flags, dtype, stream);
}

// splits per query: enough workgroups to cover the CUs twice, at least two chunk groups per split
static int attn_masked_splits(int B, int TQ, int TK, int HQ) {
  const long long queries = (long long)B * TQ * HQ;
  const int groups = cdiv(TK, 64 * ATTN_WAVES);
  long long want = cdiv(512, (int)(queries < 512 ? queries : 512));
  if (want > groups) want = groups;
  if (want > 16) want = 16;
  return want < 1 ? 1 : (int)want;
}

extern "C" size_t natsl_attn_masked_workspace_bytes(int B, int TQ, int TK, int HQ, int V) {
  const int ns = attn_masked_splits(B, TQ, TK, HQ);
  return ns > 1 ? (size_t)B * TQ * HQ * ns * (2 + V) * sizeof(float) : 0;
}

// The one implementation behind both entry points.  `strict`: a workspace smaller than the split needs is an error
// instead of a silent fall-back to one workgroup per query.
static int attn_masked_run(const char* what, const void* q, const void* k, const void* v, const uint8_t* mask, void* o, int B, int TQ,
                           int TK, int HQ, int HKV, int HM, int K, int V, float scale, int dtype, void* workspace,
                           size_t workspace_bytes, bool strict, long long k_batch_stride, long long v_batch_stride,
                           natsl_stream_t stream) {
  if (!q || !k || !v || !mask || !o) return fail(NATSL_ERR_INVALID, "%s: null pointer argument", what);
  if (dtype != NATSL_BF16 && dtype != NATSL_F32) return fail(NATSL_ERR_UNSUPPORTED, "%s: tensors must be f32 or bf16", what);
  if (B <= 0 || TQ <= 0 || TK <= 0 || HQ <= 0 || HKV <= 0 || HM <= 0) return fail(NATSL_ERR_INVALID, "%s: non-positive dimension", what);
  if (HQ % HKV || HQ % HM) return fail(NATSL_ERR_INVALID, "%s: HQ=%d must be a multiple of HKV=%d and of the mask heads %d", what, HQ, HKV, HM);
  MaskedAttnParams p;
  p.q = q; p.k = k; p.v = v; p.mask = mask; p.o = o;
  p.B = B; p.TQ = TQ; p.TK = TK; p.HQ = HQ; p.HKV = HKV; p.HM = HM; p.dtype = dtype;
  p.scale_log2 = scale * 1.4426950408889634f;
  if ((k_batch_stride && k_batch_stride < (long long)TK * HKV * K) || (v_batch_stride && v_batch_stride < (long long)TK * HKV * V) ||
      k_batch_stride % 8 || v_batch_stride % 8)
    return fail(NATSL_ERR_INVALID, "%s: a batch stride must be 0 (dense) or at least TK*HKV*D, and a multiple of 8 elements", what);
  p.k_bs = k_batch_stride ? (size_t)k_batch_stride : (size_t)TK * HKV * K;
  p.v_bs = v_batch_stride ? (size_t)v_batch_stride : (size_t)TK * HKV * V;
  // without a workspace (or with one that is too small) every query is handled by one workgroup
  p.nsplit = attn_masked_splits(B, TQ, TK, HQ);
  const size_t need = natsl_attn_masked_workspace_bytes(B, TQ, TK, HQ, V);
  if (!workspace || workspace_bytes < need) {
    if (strict && need > 0)
      return fail(NATSL_ERR_WORKSPACE, "%s: this shape needs %zu bytes of split scratch, the built-in buffer holds %zu", what, need, workspace_bytes);
    p.nsplit = 1;
  }
  p.partials = reinterpret_cast<float*>(workspace);
  if (TQ > 65535 || HQ > 65535 || (long long)B * p.nsplit > 65535) return fail(NATSL_ERR_UNSUPPORTED, "%s: grid dimension above 65535", what);
  const dim3 grid(TQ, HQ, B * p.nsplit), jgrid(TQ, HQ, B);
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
#define NATSL_MA(KK, VV)                                                                                \
  if (K == KK && V == VV) {                                                                             \
    hipLaunchKernelGGL((attn_masked_kernel<KK, VV>), grid, dim3(64 * ATTN_WAVES), 0, s, p);             \
    if (p.nsplit > 1) hipLaunchKernelGGL((attn_masked_join_kernel<VV>), jgrid, dim3(64), 0, s, p);      \
    return check_launch(what);                                                                          \
  }
  NATSL_MA(128, 128)
  NATSL_MA(64, 64)
  NATSL_MA(64, 128)
  NATSL_MA(128, 64)
#undef NATSL_MA
  return fail(NATSL_ERR_UNSUPPORTED, "%s: head dims K=%d, V=%d not built (supported: 64/128 x 64/128)", what, K, V);
}

extern "C" int natsl_attn_masked_fwd(const void* q, const void* k, const void* v, const uint8_t* mask, void* o, int B, int TQ,
                                     int TK, int HQ, int HKV, int HM, int K, int V, float scale, int dtype, void* workspace,
                                     size_t workspace_bytes, int64_t k_batch_stride, int64_t v_batch_stride,
                                     natsl_stream_t stream) {
  return attn_masked_run("natsl_attn_masked_fwd", q, k, v, mask, o, B, TQ, TK, HQ, HKV, HM, K, V, scale, dtype, workspace,
                         workspace_bytes, false, k_batch_stride, v_batch_stride, stream);
}

// ---- the variant that allocates nothing -----------------------------------------------------------------------------
// The split scratch (per query and split: running maximum, sum and DV partial outputs, fp32) lives in a device array
// of this library instead of a caller's workspace.  Every GPU holds its own copy at its own address until the process
// ends; the array's name is a host-side handle, so its device address is looked up once per device and only that
// pointer is ever handed to a kernel.  Nothing in it has to start at zero: every (query, split) slot that the join
// kernel reads is written by the split kernel of the same call.  Calls that overlap on one GPU share the array and race.
#define NATSL_ATTN_STATIC_SCRATCH_BYTES (256u << 10)
static __device__ __align__(256) unsigned char scratch[NATSL_ATTN_STATIC_SCRATCH_BYTES];

#include <mutex>
static void* scratch_device_address(const char* what, int* rc) {
  constexpr int MAX_DEVICES = 64;
  static void* ptr[MAX_DEVICES];
  static std::mutex mu;
  *rc = NATSL_OK;
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess || dev < 0 || dev >= MAX_DEVICES) {
    *rc = fail(NATSL_ERR_LAUNCH, "%s: cannot name the current device (%s)", what, hipGetErrorString(e));
    return nullptr;
  }
  std::lock_guard<std::mutex> lock(mu);
  if (!ptr[dev]) {
    void* a = nullptr;
    e = hipGetSymbolAddress(&a, HIP_SYMBOL(scratch));   // with device `dev` current: that device's copy
    if (e != hipSuccess || !a) {
      *rc = fail(NATSL_ERR_LAUNCH, "%s: hipGetSymbolAddress failed on device %d (%s)", what, dev, hipGetErrorString(e));
      return nullptr;
    }
    ptr[dev] = a;
  }
  return ptr[dev];
}

extern "C" size_t natsl_attn_masked_static_scratch_bytes(void) { return NATSL_ATTN_STATIC_SCRATCH_BYTES; }

extern "C" int natsl_attn_masked_fwd_static(const void* q, const void* k, const void* v, const uint8_t* mask, void* o, int B,
                                            int TQ, int TK, int HQ, int HKV, int HM, int K, int V, float scale, int dtype,
                                            natsl_stream_t stream) {
  const char* what = "natsl_attn_masked_fwd_static";
  int rc;
  void* ws = scratch_device_address(what, &rc);
  if (!ws) return rc;
  return attn_masked_run(what, q, k, v, mask, o, B, TQ, TK, HQ, HKV, HM, K, V, scale, dtype, ws, NATSL_ATTN_STATIC_SCRATCH_BYTES,
                         true, 0, 0, stream);
}
