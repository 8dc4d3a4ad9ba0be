// Softmax branch: sparse-KV causal flash attention for gfx950.
//
// One workgroup (4 waves) owns a tile of 256 queries of one (sequence, query head); each wave
// owns 64 of them.  Key/value chunks of 64 tokens stream through LDS (double buffered):
// first every earlier block typed "attention" (taken from the sorted block list), then the
// tile's own four chunks with the causal / same-block rules.  Scores are computed transposed,
// S^T = K Q^T, so that a lane owns one query column: the online-softmax statistics are per-lane
// scalars and the probabilities already sit in the B-operand layout of the second product
// O^T = V^T P^T.  V^T is read from the row-major V tile with the transposing LDS load.
#include "natsl_device.h"
#include "natsl_host.h"

namespace natsl {

struct SoftmaxParams {
  const bf16_t* q;
  const bf16_t* k;
  const bf16_t* v;
  bf16_t* o;
  float* lse;
  const void* types;
  int types_dtype;
  const int32_t* idx;
  const int32_t* nblk;
  const SeqRow* seqs;
  int n_seqs;
  int B, T, HQ, HKV, HN, TN, block;
  int nq_tiles;
  int total_tiles;
  float scale_log2;
  int same_block;
};

NATSL_DEVICE bool type_is_one(const void* types, int dtype, size_t i) {
  float x = dtype == NATSL_F32 ? reinterpret_cast<const float*>(types)[i]
                               : bf16_to_f32(reinterpret_cast<const bf16_t*>(types)[i]);
  return rintf(x) == 1.0f;
}

constexpr int QTILE = 256;

template <int DK, int DV>
__global__ __launch_bounds__(256, 1) void softmax_sparse_fwd_kernel(const SoftmaxParams p) {
  constexpr int KP = DK + 8, VP = DV + 8;  // LDS row pitch in elements (16-byte multiple)
  constexpr int KSTEPS = DK / 16, VT = DV / 32, KL = DK / 32, VL = DV / 32;
  extern __shared__ __align__(16) unsigned char smem[];
  bf16_t* Ks = reinterpret_cast<bf16_t*>(smem);  // [2][64][KP]
  bf16_t* Vs = Ks + 2 * 64 * KP;                 // [2][64][VP]

  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int l32 = lane & 31, hf = lane >> 5;

  // ---- which (sequence, head, tile) ------------------------------------------------------
  int n, tile, hq, bos, len, bos_nats;
  if (p.seqs == nullptr) {
    const int per = p.B * p.HQ;
    tile = p.nq_tiles - 1 - (int)blockIdx.x / per;  // heaviest tiles first
    const int rem = (int)blockIdx.x % per;
    n = rem / p.HQ;
    hq = rem % p.HQ;
    bos = n * p.T;
    len = p.T;
    bos_nats = n * p.TN;
  } else {
    const int gt = p.total_tiles - 1 - (int)blockIdx.x / p.HQ;
    hq = (int)blockIdx.x % p.HQ;
    n = 0;
    for (int i = 1; i < p.n_seqs; ++i)
      if (p.seqs[i].qtile_off <= gt) n = i;
    tile = gt - p.seqs[n].qtile_off;
    bos = p.seqs[n].bos;
    len = p.seqs[n].eos - bos;
    bos_nats = p.seqs[n].bos_nats;
  }
  const int Bs = p.block, per_blk = Bs >> 6;
  const int hkv = hq / (p.HQ / p.HKV), hn = hq / (p.HQ / p.HN);
  const int tile_start = tile * QTILE;
  const int q0 = tile_start + wave * 64;
  const bool wave_valid = q0 < len;

  const bf16_t* qp = p.q + ((size_t)bos * p.HQ + hq) * DK;
  const bf16_t* kp = p.k + ((size_t)bos * p.HKV + hkv) * DK;
  const bf16_t* vp = p.v + ((size_t)bos * p.HKV + hkv) * DV;
  const size_t krow = (size_t)p.HKV * DK, vrow = (size_t)p.HKV * DV;
  const int32_t* list = p.idx + ((size_t)bos_nats * p.HN + hn) * 2;  // element j at list[j*HN*2]
  const size_t list_stride = (size_t)p.HN * 2;
  const int n_attn = p.nblk[((size_t)n * p.HN + hn) * 2];

  // number of attention blocks that end at or before the tile's first query
  int n_prior;
  {
    int lo = 0, hi = n_attn;
    while (lo < hi) {
      const int mid = (lo + hi) >> 1;
      if ((list[mid * list_stride] + 1) * Bs <= tile_start) lo = mid + 1; else hi = mid;
    }
    n_prior = lo;
  }
  const int n_prior_chunks = n_prior * per_blk;
  const int n_diag = min(4, (len - tile_start + 63) >> 6);
  const int n_iters = n_prior_chunks + n_diag;

  auto key_start = [&](int it) -> int {
    if (it < n_prior_chunks) {
      const int j = it / per_blk;
      return list[j * list_stride] * Bs + (it - j * per_blk) * 64;
    }
    return tile_start + (it - n_prior_chunks) * 64;
  };
  auto attn_block = [&](int blk) -> bool {
    return type_is_one(p.types, p.types_dtype, ((size_t)(bos_nats + blk) * p.HN + hn) * 2);
  };

  // ---- Q as the B operand of S^T = K Q^T: lane = query column ----------------------------
  bf16x8 QB[2][KSTEPS];
#pragma unroll
  for (int qt = 0; qt < 2; ++qt) {
    const int qi = q0 + 32 * qt + l32;
    const bf16_t* qr = qp + (size_t)qi * p.HQ * DK + 8 * hf;
#pragma unroll
    for (int s = 0; s < KSTEPS; ++s) QB[qt][s] = qi < len ? ld8(qr + 16 * s) : zero8();
  }

  f32x16 acc[VT][2];
#pragma unroll
  for (int vt = 0; vt < VT; ++vt)
#pragma unroll
    for (int qt = 0; qt < 2; ++qt)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[vt][qt][r] = 0.f;
  float m_run[2] = {-INFINITY, -INFINITY}, l_run[2] = {0.f, 0.f};

  // ---- global -> register -> LDS staging of one 64-key chunk -----------------------------
  u32x4 kreg[KL], vreg[VL];
  const int ld_row = tid >> 2, ld_seg = tid & 3;
  auto gload = [&](int ks) {
    const int tok = ks + ld_row;
    const bool ok = tok < len;
    const u32x4* kr = reinterpret_cast<const u32x4*>(kp + (size_t)tok * krow);
    const u32x4* vr = reinterpret_cast<const u32x4*>(vp + (size_t)tok * vrow);
    const u32x4 z = {0u, 0u, 0u, 0u};
#pragma unroll
    for (int i = 0; i < KL; ++i) kreg[i] = ok ? kr[ld_seg + 4 * i] : z;
#pragma unroll
    for (int i = 0; i < VL; ++i) vreg[i] = ok ? vr[ld_seg + 4 * i] : z;
  };
  auto lstore = [&](int buf) {
    bf16_t* kd = Ks + (buf * 64 + ld_row) * KP;
    bf16_t* vd = Vs + (buf * 64 + ld_row) * VP;
#pragma unroll
    for (int i = 0; i < KL; ++i) *reinterpret_cast<u32x4*>(kd + (ld_seg + 4 * i) * 8) = kreg[i];
#pragma unroll
    for (int i = 0; i < VL; ++i) *reinterpret_cast<u32x4*>(vd + (ld_seg + 4 * i) * 8) = vreg[i];
  };

  if (n_iters > 0) {
    gload(key_start(0));
    lstore(0);
  }
  __syncthreads();

  const int my_blk = q0 / Bs;
  for (int it = 0; it < n_iters; ++it) {
    const int buf = it & 1;
    if (it + 1 < n_iters) gload(key_start(it + 1));

    bool active = wave_valid, causal = false;
    if (it >= n_prior_chunks) {
      const int jc = it - n_prior_chunks;
      const int kblk = (tile_start + jc * 64) / Bs;
      if (p.same_block) {
        if (jc > wave) active = false;
        else if (jc == wave) causal = true;
        else active = active && (kblk == my_blk || attn_block(kblk));
      } else {
        active = active && jc < wave && kblk < my_blk && attn_block(kblk);
      }
    }

    if (active) {
      const bf16_t* Kb = Ks + buf * 64 * KP;
      const bf16_t* Vb = Vs + buf * 64 * VP;
      f32x16 s[2][2];
#pragma unroll
      for (int kt = 0; kt < 2; ++kt)
#pragma unroll
        for (int qt = 0; qt < 2; ++qt)
#pragma unroll
          for (int r = 0; r < 16; ++r) s[kt][qt][r] = 0.f;
#pragma unroll
      for (int st = 0; st < KSTEPS; ++st) {
        const bf16x8 ka0 = ld8(Kb + l32 * KP + 16 * st + 8 * hf);
        const bf16x8 ka1 = ld8(Kb + (32 + l32) * KP + 16 * st + 8 * hf);
        s[0][0] = mfma32(ka0, QB[0][st], s[0][0]);
        s[0][1] = mfma32(ka0, QB[1][st], s[0][1]);
        s[1][0] = mfma32(ka1, QB[0][st], s[1][0]);
        s[1][1] = mfma32(ka1, QB[1][st], s[1][1]);
      }
      // online softmax; acc register r of key tile kt is key 32kt + 8(r/4) + 4hf + r%4
#pragma unroll
      for (int qt = 0; qt < 2; ++qt) {
        const int qloc = 32 * qt + l32;
        float mx = -INFINITY;
#pragma unroll
        for (int kt = 0; kt < 2; ++kt)
#pragma unroll
          for (int r = 0; r < 16; ++r) {
            float x = s[kt][qt][r] * p.scale_log2;
            if (causal) {
              const int kloc = 32 * kt + 8 * (r >> 2) + 4 * hf + (r & 3);
              if (kloc > qloc) x = -INFINITY;
            }
            s[kt][qt][r] = x;
            mx = fmaxf(mx, x);
          }
        mx = xhalf_max(mx);
        const float m_new = fmaxf(m_run[qt], mx);
        const float m_safe = m_new == -INFINITY ? 0.f : m_new;
        const float alpha = __builtin_amdgcn_exp2f(m_run[qt] - m_safe);
        float rs = 0.f;
#pragma unroll
        for (int kt = 0; kt < 2; ++kt)
#pragma unroll
          for (int r = 0; r < 16; ++r) {
            const float e = __builtin_amdgcn_exp2f(s[kt][qt][r] - m_safe);
            s[kt][qt][r] = e;
            rs += e;
          }
        l_run[qt] = l_run[qt] * alpha + rs;  // partial over this lane's keys; halves are joined at the end
        m_run[qt] = m_new;
#pragma unroll
        for (int vt = 0; vt < VT; ++vt)
#pragma unroll
          for (int r = 0; r < 16; ++r) acc[vt][qt][r] *= alpha;
      }
      // O^T += V^T P^T, 16 keys per step; MFMA k-slot (hf, j) <-> key base + 8(j/4) + 4hf + j%4
      const int i16 = lane & 15, colsel = 16 * ((lane >> 4) & 1);
#pragma unroll
      for (int sidx = 0; sidx < 4; ++sidx) {
        const int kt = sidx >> 1, ss = sidx & 1;
        bf16x8 PB[2];
#pragma unroll
        for (int qt = 0; qt < 2; ++qt) {
          u32x4 w;
#pragma unroll
          for (int j = 0; j < 4; ++j) w[j] = pack_bf16x2(s[kt][qt][8 * ss + 2 * j], s[kt][qt][8 * ss + 2 * j + 1]);
          PB[qt] = __builtin_bit_cast(bf16x8, w);
        }
        const int base = 32 * kt + 16 * ss + 4 * hf;
        const bf16_t* vrow0 = Vb + (base + (i16 >> 2)) * VP + colsel + 4 * (i16 & 3);
#pragma unroll
        for (int vt = 0; vt < VT; ++vt) {
          const bf16x8 va = join4(lds_tr4(vrow0 + 32 * vt), lds_tr4(vrow0 + 8 * VP + 32 * vt));
          acc[vt][0] = mfma32(va, PB[0], acc[vt][0]);
          acc[vt][1] = mfma32(va, PB[1], acc[vt][1]);
        }
      }
    }

    if (it + 1 < n_iters) lstore(buf ^ 1);
    __syncthreads();
  }

  // ---- epilogue: normalise, transpose through LDS, coalesced stores ------------------------
  bf16_t* Os = reinterpret_cast<bf16_t*>(smem) + wave * 64 * VP;  // this wave's [64][VP]
#pragma unroll
  for (int qt = 0; qt < 2; ++qt) {
    const float l_tot = xhalf_sum(l_run[qt]);
    const bool has = l_tot > 0.f;
    const float inv = has ? 1.f / l_tot : 0.f;
    const int qi = q0 + 32 * qt + l32;
    if (hf == 0 && qi < len)
      p.lse[((size_t)(bos + qi)) * p.HQ + hq] = has ? m_run[qt] + __builtin_amdgcn_logf(l_tot) : 0.f;
#pragma unroll
    for (int vt = 0; vt < VT; ++vt)
#pragma unroll
      for (int rg = 0; rg < 4; ++rg) {
        u32x2 w;
        w[0] = pack_bf16x2(acc[vt][qt][4 * rg] * inv, acc[vt][qt][4 * rg + 1] * inv);
        w[1] = pack_bf16x2(acc[vt][qt][4 * rg + 2] * inv, acc[vt][qt][4 * rg + 3] * inv);
        *reinterpret_cast<u32x2*>(Os + (32 * qt + l32) * VP + 32 * vt + 8 * rg + 4 * hf) = w;
      }
  }
  __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0): this wave's LDS writes have landed
  __builtin_amdgcn_wave_barrier();
  constexpr int SEGS = DV / 8;           // 16-byte segments per row
  constexpr int ROWS_PER_PASS = 64 / SEGS;
#pragma unroll
  for (int pass = 0; pass < 64 / ROWS_PER_PASS; ++pass) {
    const int row = pass * ROWS_PER_PASS + lane / SEGS, seg = lane % SEGS;
    const int qi = q0 + row;
    if (qi < len) {
      const u32x4 w = *reinterpret_cast<const u32x4*>(Os + row * VP + seg * 8);
      *reinterpret_cast<u32x4*>(p.o + ((size_t)(bos + qi) * p.HQ + hq) * DV + seg * 8) = w;
    }
  }
}

template <int DK, int DV>
static int launch_softmax(const SoftmaxParams& p, hipStream_t stream) {
  constexpr int KP = DK + 8, VP = DV + 8;
  size_t lds = (size_t)2 * 64 * (KP + VP) * sizeof(bf16_t);
  const size_t epi = (size_t)QTILE * VP * sizeof(bf16_t);
  if (epi > lds) lds = epi;
  auto kern = softmax_sparse_fwd_kernel<DK, DV>;
  hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
  if (e != hipSuccess) return fail(NATSL_ERR_LAUNCH, "softmax: cannot reserve %zu bytes of LDS: %s", lds, hipGetErrorString(e));
  const long long grid = (long long)p.total_tiles * p.HQ;
  if (grid <= 0) return NATSL_OK;
  hipLaunchKernelGGL(kern, dim3((unsigned)grid), dim3(256), lds, stream, p);
  return check_launch("natsl_softmax_sparse_fwd");
}

}  // namespace natsl

using namespace natsl;

extern "C" int natsl_softmax_sparse_fwd(const void* q, const void* k, const void* v, void* o, float* lse,
                                        const void* types, int types_dtype, const int32_t* nats_block_indices,
                                        const int32_t* n_nats_blocks, int B, int T, int HQ, int HKV, int HN, int K,
                                        int V, int TN, int block, float scale, int same_block_visible, int dtype,
                                        const natsl_seq_row* seqs, int n_seqs, int total_units,
                                        natsl_stream_t stream) {
  if (!q || !k || !v || !o || !lse || !types || !nats_block_indices || !n_nats_blocks)
    return fail(NATSL_ERR_INVALID, "softmax: null pointer argument");
  if (dtype != NATSL_BF16) return fail(NATSL_ERR_UNSUPPORTED, "softmax: only bf16 tensors are supported (got dtype %d)", dtype);
  if (types_dtype != NATSL_BF16 && types_dtype != NATSL_F32) return fail(NATSL_ERR_UNSUPPORTED, "softmax: block types must be f32 or bf16");
  if (B <= 0 || T <= 0 || HQ <= 0 || HKV <= 0 || HN <= 0 || TN <= 0) return fail(NATSL_ERR_INVALID, "softmax: non-positive dimension");
  if (HQ % HKV || HQ % HN) return fail(NATSL_ERR_INVALID, "softmax: HQ=%d must be a multiple of HKV=%d and HN=%d", HQ, HKV, HN);
  if (block < 64 || block % 64) return fail(NATSL_ERR_UNSUPPORTED, "softmax: block size %d must be a multiple of 64", block);
  if (seqs ? (B != 1 || n_seqs <= 0) : (TN != cdiv(T, block)))
    return fail(NATSL_ERR_INVALID, "softmax: TN=%d does not match T=%d, block=%d (or packed input with B != 1)", TN, T, block);

  SoftmaxParams p;
  p.q = (const bf16_t*)q; p.k = (const bf16_t*)k; p.v = (const bf16_t*)v; p.o = (bf16_t*)o; p.lse = lse;
  p.types = types; p.types_dtype = types_dtype; p.idx = nats_block_indices; p.nblk = n_nats_blocks;
  p.seqs = reinterpret_cast<const SeqRow*>(seqs); p.n_seqs = seqs ? n_seqs : 0;
  p.B = B; p.T = T; p.HQ = HQ; p.HKV = HKV; p.HN = HN; p.TN = TN; p.block = block;
  p.nq_tiles = cdiv(T, QTILE);
  p.total_tiles = seqs ? total_units : B * p.nq_tiles;
  p.scale_log2 = scale * 1.4426950408889634f;
  p.same_block = same_block_visible ? 1 : 0;
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  if (K == 128 && V == 128) return launch_softmax<128, 128>(p, s);
  if (K == 64 && V == 64) return launch_softmax<64, 64>(p, s);
  if (K == 64 && V == 128) return launch_softmax<64, 128>(p, s);
  if (K == 128 && V == 64) return launch_softmax<128, 64>(p, s);
  return fail(NATSL_ERR_UNSUPPORTED, "softmax: head dims K=%d, V=%d not built (supported: 64/128 x 64/128)", K, V);
}
