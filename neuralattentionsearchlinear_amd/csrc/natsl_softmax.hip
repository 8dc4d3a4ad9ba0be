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
#ifdef NATSL_ABLATE
#include <stdlib.h>  // development build only: getenv for the ablation switches
#endif

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
  int variant;  // 1: 128-query tile on 4 waves, 8: 256-query tile on 8 waves, 4: 256-query tile, 64 queries per wave
  int dbg;      // ablation bits, always 0 unless built with NATSL_ABLATE
};

NATSL_DEVICE bool type_is_one(const void* types, int dtype, size_t i) {
  float x = dtype == NATSL_F32 ? reinterpret_cast<const float*>(types)[i]
                               : bf16_to_f32(reinterpret_cast<const bf16_t*>(types)[i]);
  return rintf(x) == 1.0f;
}

constexpr int QTILE_TABLE = 256;  // query tile the packed-sequence table counts in
constexpr int VT_PITCH = 68;          // elements per row of the transposed V tile (64 keys + 4): conflict-free operand reads
constexpr float RESCALE_SLACK = 8.f;  // log2 units: probabilities may reach 2^8 before the reference maximum moves
constexpr int MAX_LDS_LIST = 2048;    // prior attention blocks whose ids are kept in LDS (more are re-read from memory)

// One 64-key chunk for one wave owning NQ column tiles of 32 queries, in three pieces:
//   scores      S^T = K Q^T (key tile kt x query tile qt) and the scaled row maxima
//   rescale     move the reference maximum m_ref and rescale the accumulators.  It is needed only
//               when some row's maximum has grown by more than RESCALE_SLACK since m_ref was set,
//               so the hot loop never touches the accumulators with vector ALU instructions.
//   exp_pv      P = exp2(S*c - m_ref), row sums, O^T += V^T P^T, 16 keys per step.
//               Accumulator register r of key tile kt is key 32kt + 8(r/4) + 4hf + r%4; the same
//               order is used for the k-slots of the V^T operand, so P needs no data movement.
//               V is staged TRANSPOSED in LDS (VT[v][key]): that operand is two 8-byte reads.
template <int DK, int NQ, bool CAUSAL>
NATSL_DEVICE void scores(const bf16_t* Kb, const bf16x8 (&QB)[NQ][DK / 16], f32x16 (&s)[2][NQ], float (&mx)[NQ], const float c,
                         const int lane, const int qloc0) {
  constexpr int KP = DK + 8, KSTEPS = DK / 16;
  const int l32 = lane & 31, hf = lane >> 5;
#pragma unroll
  for (int kt = 0; kt < 2; ++kt)
#pragma unroll
    for (int qt = 0; qt < NQ; ++qt)
#pragma unroll
      for (int r = 0; r < 16; ++r) s[kt][qt][r] = 0.f;
  // K operand reads run two k-steps ahead of the matrix instructions that consume them
  constexpr int AHEAD = 2;
  bf16x8 ka[KSTEPS][2];
#pragma unroll
  for (int st = 0; st < AHEAD; ++st) {
    ka[st][0] = ld8(Kb + l32 * KP + 16 * st + 8 * hf);
    ka[st][1] = ld8(Kb + (32 + l32) * KP + 16 * st + 8 * hf);
  }
#pragma unroll
  for (int st = 0; st < KSTEPS; ++st) {
    if (st + AHEAD < KSTEPS) {
      ka[st + AHEAD][0] = ld8(Kb + l32 * KP + 16 * (st + AHEAD) + 8 * hf);
      ka[st + AHEAD][1] = ld8(Kb + (32 + l32) * KP + 16 * (st + AHEAD) + 8 * hf);
    }
#pragma unroll
    for (int qt = 0; qt < NQ; ++qt) {
      s[0][qt] = mfma32(ka[st][0], QB[qt][st], s[0][qt]);
      s[1][qt] = mfma32(ka[st][1], QB[qt][st], s[1][qt]);
    }
  }
  // pin that order: 2*AHEAD reads, then {2 NQ matrix instructions, 2 reads} per k-step
  __builtin_amdgcn_sched_group_barrier(0x100, 2 * AHEAD, 0);
#pragma unroll
  for (int st = 0; st < KSTEPS - AHEAD; ++st) {
    __builtin_amdgcn_sched_group_barrier(0x008, 2 * NQ, 0);
    __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
  }
  __builtin_amdgcn_sched_group_barrier(0x008, 2 * NQ * AHEAD, 0);
#pragma unroll
  for (int qt = 0; qt < NQ; ++qt) {
    float m = -INFINITY;
#pragma unroll
    for (int kt = 0; kt < 2; ++kt)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        if (CAUSAL) {
          const int kloc = 32 * kt + 8 * (r >> 2) + 4 * hf + (r & 3), qloc = qloc0 + 32 * qt + l32;
          if (kloc > qloc) s[kt][qt][r] = -INFINITY;
        }
        m = fmaxf(m, s[kt][qt][r]);
      }
    mx[qt] = xhalf_max(m) * c;
  }
}

template <int NQ>
NATSL_DEVICE bool needs_rescale(const float (&mx)[NQ], const float (&m_ref)[NQ]) {
  bool need = false;
#pragma unroll
  for (int qt = 0; qt < NQ; ++qt) need = need || mx[qt] > m_ref[qt] + RESCALE_SLACK;
  return __any(need) != 0;
}

template <int DV, int NQ>
NATSL_DEVICE void rescale(f32x16 (&acc)[DV / 32][NQ], float (&m_ref)[NQ], float (&l_run)[NQ], const float (&mx)[NQ]) {
#pragma unroll
  for (int qt = 0; qt < NQ; ++qt) {
    const float m_new = fmaxf(m_ref[qt], mx[qt]);
    const float alpha = __builtin_amdgcn_exp2f(m_ref[qt] - (m_new == -INFINITY ? 0.f : m_new));
    m_ref[qt] = m_new;
    l_run[qt] *= alpha;
#pragma unroll
    for (int vt = 0; vt < DV / 32; ++vt)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[vt][qt][r] *= alpha;
  }
}

template <int DV, int NQ>
NATSL_DEVICE void exp_pv(const bf16_t* VTb, f32x16 (&s)[2][NQ], f32x16 (&acc)[DV / 32][NQ], const float (&m_ref)[NQ],
                         float (&l_run)[NQ], const float c, const int lane) {
  constexpr int TP = VT_PITCH, VT = DV / 32;
  const int l32 = lane & 31, hf = lane >> 5;
  float neg[NQ], rs[NQ];
#pragma unroll
  for (int qt = 0; qt < NQ; ++qt) {
    neg[qt] = m_ref[qt] == -INFINITY ? 0.f : -m_ref[qt];
    rs[qt] = 0.f;
  }
#pragma unroll
  for (int sidx = 0; sidx < 4; ++sidx) {
    const int kt = sidx >> 1, ss = sidx & 1;
    bf16x8 PB[NQ];
#pragma unroll
    for (int qt = 0; qt < NQ; ++qt) {
      float e[8];
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        e[j] = __builtin_amdgcn_exp2f(fmaf(s[kt][qt][8 * ss + j], c, neg[qt]));
        rs[qt] += e[j];
      }
      u32x4 w;
#pragma unroll
      for (int j = 0; j < 4; ++j) w[j] = pack_bf16x2(e[2 * j], e[2 * j + 1]);
      PB[qt] = __builtin_bit_cast(bf16x8, w);
    }
#pragma unroll
    for (int vt = 0; vt < VT; ++vt) {
      // this lane's keys: kbase..kbase+3 and kbase+8..kbase+11; 16-key groups of odd value tiles are stored swapped
      const int kbase = 16 * (sidx ^ (vt & 1)) + 4 * hf;
      const bf16_t* vr = VTb + (32 * vt + l32) * TP + kbase;
      const u32x2 lo = *reinterpret_cast<const u32x2*>(vr), hi = *reinterpret_cast<const u32x2*>(vr + 8);
      const u32x4 w = {lo[0], lo[1], hi[0], hi[1]};
      const bf16x8 va = __builtin_bit_cast(bf16x8, w);
#pragma unroll
      for (int qt = 0; qt < NQ; ++qt) acc[vt][qt] = mfma32(va, PB[qt], acc[vt][qt]);
    }
  }
#pragma unroll
  for (int qt = 0; qt < NQ; ++qt) l_run[qt] += rs[qt];  // partial over this lane's keys; halves are joined in the epilogue
}

// ---- the same work in halves of 32 keys, for the software-pipelined hot loop (one 32-query tile per wave) ----
// qk_half    S^T tile of key half kt (8 matrix instructions on one accumulator), K reads two steps ahead
// half_max   scaled row maximum of one half (both lane halves joined)
// probs_half P = exp2(S*c - m_ref) for one half, packed to bf16 in the B-operand order; adds the row sums
// pv_half    O^T += V^T P^T for one half
template <int DK>
NATSL_DEVICE void qk_half(const bf16_t* Kb, const int kt, const bf16x8 (&QB)[DK / 16], f32x16& s, const int lane) {
  constexpr int KP = DK + 8, KSTEPS = DK / 16, AHEAD = 2;
  const bf16_t* kr = Kb + (32 * kt + (lane & 31)) * KP + 8 * (lane >> 5);
  bf16x8 ka[KSTEPS];
#pragma unroll
  for (int st = 0; st < AHEAD; ++st) ka[st] = ld8(kr + 16 * st);
#pragma unroll
  for (int r = 0; r < 16; ++r) s[r] = 0.f;
#pragma unroll
  for (int st = 0; st < KSTEPS; ++st) {
    if (st + AHEAD < KSTEPS) ka[st + AHEAD] = ld8(kr + 16 * (st + AHEAD));
    s = mfma32(ka[st], QB[st], s);
  }
}

template <bool CAUSAL>
NATSL_DEVICE float half_max(f32x16& s, const int kt, const float c, const int lane, const int qloc0) {
  const int l32 = lane & 31, hf = lane >> 5;
  float m = -INFINITY;
#pragma unroll
  for (int r = 0; r < 16; ++r) {
    if (CAUSAL) {
      const int kloc = 32 * kt + 8 * (r >> 2) + 4 * hf + (r & 3), qloc = qloc0 + l32;
      if (kloc > qloc) s[r] = -INFINITY;
    }
    m = fmaxf(m, s[r]);
  }
  return xhalf_max(m) * c;
}

NATSL_DEVICE void probs_half(const f32x16& s, const float c, const float neg, float& rs, bf16x8 (&PB)[2]) {
#pragma unroll
  for (int ss = 0; ss < 2; ++ss) {
    float e[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      e[j] = __builtin_amdgcn_exp2f(fmaf(s[8 * ss + j], c, neg));
      rs += e[j];
    }
    u32x4 w;
#pragma unroll
    for (int j = 0; j < 4; ++j) w[j] = pack_bf16x2(e[2 * j], e[2 * j + 1]);
    PB[ss] = __builtin_bit_cast(bf16x8, w);
  }
}

template <int DV>
NATSL_DEVICE void pv_half(const bf16_t* VTb, const int kt, const bf16x8 (&PB)[2], f32x16 (&acc)[DV / 32][1], const int lane) {
  constexpr int TP = VT_PITCH, VT = DV / 32;
  const int l32 = lane & 31, hf = lane >> 5;
#pragma unroll
  for (int ss = 0; ss < 2; ++ss) {
#pragma unroll
    for (int vt = 0; vt < VT; ++vt) {
      const int kbase = 16 * ((2 * kt + ss) ^ (vt & 1)) + 4 * hf;  // 16-key groups of odd value tiles are stored swapped
      const bf16_t* vr = VTb + (32 * vt + l32) * TP + kbase;
      const u32x2 lo = *reinterpret_cast<const u32x2*>(vr), hi = *reinterpret_cast<const u32x2*>(vr + 8);
      const u32x4 w = {lo[0], lo[1], hi[0], hi[1]};
      acc[vt][0] = mfma32(__builtin_bit_cast(bf16x8, w), PB[ss], acc[vt][0]);
    }
  }
}

// NQ = 32-query column tiles per wave, NWAVES waves: the workgroup owns QTILE = 32*NQ*NWAVES queries.
template <int DK, int DV, int NQ, int NWAVES>
__global__ __launch_bounds__(64 * NWAVES, (NQ == 1 && NWAVES == 4) ? 2 : 1) void softmax_sparse_fwd_kernel(const SoftmaxParams p) {
  constexpr int NTHREADS = 64 * NWAVES, QW = 32 * NQ, QTILE = QW * NWAVES;  // QW = queries per wave
  constexpr int KP = DK + 8, VP = DV + 8;  // row pitch (elements) of the K tile and of the epilogue tile
  constexpr int TP = VT_PITCH;
  constexpr int KSTEPS = DK / 16, VT = DV / 32;
  extern __shared__ __align__(16) unsigned char smem[];
  bf16_t* Ks = reinterpret_cast<bf16_t*>(smem);  // [2][64][KP]   keys, row-major
  bf16_t* Vs = Ks + 2 * 64 * KP;                 // [2][DV][TP]   values, transposed
  __shared__ int lds_list[MAX_LDS_LIST];
  __shared__ int lds_count;

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // wave-uniform, so everything derived from it stays scalar
  const int l32 = lane & 31, hf = lane >> 5;

  // ---- which (sequence, head, tile) ------------------------------------------------------
  int n, tile, hq, bos, len, bos_nats;
  if (p.seqs == nullptr) {
    // Workgroup ids are dealt round-robin to the 8 XCDs; give each XCD whole (batch, head) pairs,
    // heaviest tile first, so the tiles that share one pair's K/V run together on one L2.
    const int n_pairs = p.B * p.HQ;
    const int xcd = (int)blockIdx.x & 7, j = (int)blockIdx.x >> 3;
    const int nq_tiles = (p.T + QTILE - 1) / QTILE;
    const int pair = (j / nq_tiles) * 8 + xcd;
    if (pair >= n_pairs) return;
    tile = nq_tiles - 1 - j % nq_tiles;
    n = pair / p.HQ;
    hq = pair % p.HQ;
    bos = n * p.T;
    len = p.T;
    bos_nats = n * p.TN;
  } else {
    const int tiles_per_256 = QTILE_TABLE / QTILE;
    const int gt = p.total_tiles * tiles_per_256 - 1 - (int)blockIdx.x / p.HQ;
    hq = (int)blockIdx.x % p.HQ;
    n = 0;
    for (int i = 1; i < p.n_seqs; ++i)
      if (p.seqs[i].qtile_off * tiles_per_256 <= gt) n = i;
    tile = gt - p.seqs[n].qtile_off * tiles_per_256;
    bos = p.seqs[n].bos;
    len = p.seqs[n].eos - bos;
    bos_nats = p.seqs[n].bos_nats;
  }
  const int Bs = p.block, per_blk = Bs >> 6;
  const int hkv = hq / (p.HQ / p.HKV), hn = hq / (p.HQ / p.HN);
  const int tile_start = tile * QTILE;
  const int q0 = tile_start + wave * QW;      // this wave's first query
  const int my_chunk = q0 >> 6;               // the 64-key chunk of the sequence that holds them
  const int qloc0 = q0 & 63;                  // ... and where in that chunk
  // keys from here on are handled chunk by chunk with the same-block / causal rules: the start of
  // the tile, or of the selector block it falls into when blocks are larger than the tile
  const int dstart = (tile_start / p.block) * p.block;
  const bool wave_valid = q0 < len;

  const bf16_t* qp = p.q + ((size_t)bos * p.HQ + hq) * DK;
  const bf16_t* kp = p.k + ((size_t)bos * p.HKV + hkv) * DK;
  const bf16_t* vp = p.v + ((size_t)bos * p.HKV + hkv) * DV;
  const size_t krow = (size_t)p.HKV * DK, vrow = (size_t)p.HKV * DV;
  const int32_t* list = p.idx + ((size_t)bos_nats * p.HN + hn) * 2;  // element j at list[j*HN*2]
  const size_t list_stride = (size_t)p.HN * 2;
  const int n_attn = p.nblk[((size_t)n * p.HN + hn) * 2];

  // ---- Q as the B operand of S^T = K Q^T: lane = query column ----------------------------
  bf16x8 QB[NQ][KSTEPS];
#pragma unroll
  for (int qt = 0; qt < NQ; ++qt) {
    const int qi = min(q0 + 32 * qt + l32, len - 1);  // rows past the end are computed on a copy and never stored
    const bf16_t* qr = qp + (size_t)qi * p.HQ * DK + 8 * hf;
#pragma unroll
    for (int s = 0; s < KSTEPS; ++s) QB[qt][s] = ld8(qr + 16 * s);
  }

  if (tile_start >= len) return;  // packed input: a sequence's last 256-row table slot may hold no tile of this size

  f32x16 acc[VT][NQ];
#pragma unroll
  for (int vt = 0; vt < VT; ++vt)
#pragma unroll
    for (int qt = 0; qt < NQ; ++qt)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[vt][qt][r] = 0.f;
  float m_ref[NQ], l_run[NQ];
#pragma unroll
  for (int qt = 0; qt < NQ; ++qt) {
    m_ref[qt] = -INFINITY;
    l_run[qt] = 0.f;
  }

  // ---- global -> register -> LDS staging of one 64-key chunk -----------------------------
  // 256 threads stage K (16-byte segments, whole rows per load instruction; stored row-major), 256 threads stage V
  // (thread = group of 4 keys x 8 value columns; the 4x8 block is transposed in registers and
  // stored as 8 rows of 4 keys).  With 4 waves every thread does both.
  static_assert(NTHREADS == 256 || NTHREADS == 512, "staging is written for 4 or 8 waves");
  constexpr bool SPLIT = NTHREADS == 512;
  constexpr int KL = DK / 32;
  const int st = SPLIT ? (tid & 255) : tid;
  const bool do_k = !SPLIT || tid < 256, do_v_role = !SPLIT || tid >= 256;
  u32x4 kreg[KL], vreg[4];
  // K: KSEGS lanes share a row, so one load instruction covers whole rows (full cache lines): a wave's loads
  // return in order, and an instruction that touches many half-used lines holds back everything behind it
  constexpr int KSEGS = DK / 8, KROWS = 256 / KSEGS;   // 16-byte segments per row; rows per pass (KL passes)
  const int ld_row = st / KSEGS, ld_seg = st % KSEGS;
  constexpr int VSEGS = DV / 8;                    // 8-column segments per V row
  // V: 8 lanes share 128 bytes (a full line) of a row; a thread owns keys 4*v_kg .. 4*v_kg+3 of one 8-column
  // segment.  In the transposed tile the 16-key groups of value rows with bit 5 set are swapped pairwise
  // (group ^ 1), which keeps the 8-byte transposed stores of one instruction on distinct banks.
  const int v_seg = VSEGS == 16 ? (st & 7) + 8 * ((st >> 6) & 1) : (st & 7);
  const int v_kg = VSEGS == 16 ? ((st >> 3) & 7) + 8 * (st >> 7) : (st >> 3);
  const bool v_on = do_v_role && v_seg < VSEGS && v_kg < 16;
  // per-thread byte offsets inside a chunk; the chunk's base address is wave-uniform
  const unsigned k_off = (unsigned)(((size_t)ld_row * krow + ld_seg * 8) * sizeof(bf16_t));
  const size_t k_pass = (size_t)KROWS * krow * sizeof(bf16_t);
  const unsigned v_off = (unsigned)(((size_t)(4 * v_kg) * vrow + 8 * v_seg) * sizeof(bf16_t));
  auto gload_full = [&](int ks) {
    // a chunk that lies wholly inside the sequence (every prior attention block): scalar base + lane offset
    if (do_k) {
      const char* kb = reinterpret_cast<const char*>(kp + (size_t)ks * krow) + k_off;
#pragma unroll
      for (int i = 0; i < KL; ++i) kreg[i] = *reinterpret_cast<const u32x4*>(kb + i * k_pass);
    }
    if (v_on) {
#pragma unroll
      for (int j = 0; j < 4; ++j)
        vreg[j] = *reinterpret_cast<const u32x4*>(reinterpret_cast<const char*>(vp + ((size_t)ks + j) * vrow) + v_off);
    }
  };
  auto gload_clamped = [&](int ks) {
    // Rows past the end of the sequence are clamped to its last row: such keys are always hidden
    // by the causal rule (a valid query precedes them), so only finite values are needed there.
    if (do_k) {
#pragma unroll
      for (int i = 0; i < KL; ++i) {
        const int tok = min(ks + ld_row + KROWS * i, len - 1);
        kreg[i] = *reinterpret_cast<const u32x4*>(kp + (size_t)tok * krow + 8 * ld_seg);
      }
    }
    if (v_on) {
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int vt_ = min(ks + 4 * v_kg + j, len - 1);
        vreg[j] = *reinterpret_cast<const u32x4*>(vp + (size_t)vt_ * vrow + 8 * v_seg);
      }
    }
  };
  auto gload = [&](int ks) {
    if (ks + 64 <= len) gload_full(ks);
    else gload_clamped(ks);
  };
  auto lstore = [&](int buf) {
    if (do_k) {
      bf16_t* kd = Ks + (buf * 64 + ld_row) * KP + 8 * ld_seg;
#pragma unroll
      for (int i = 0; i < KL; ++i) *reinterpret_cast<u32x4*>(kd + KROWS * i * KP) = kreg[i];
    }
    if (v_on) {
      bf16_t* vd = Vs + (buf * DV + 8 * v_seg) * TP + 4 * (v_kg ^ (4 * ((v_seg >> 2) & 1)));
#pragma unroll
      for (int d = 0; d < 4; ++d) {
        // value columns 2d (low halves) and 2d+1 (high halves) of the four keys
        u32x2 lo, hi;
        lo[0] = __builtin_amdgcn_perm(vreg[1][d], vreg[0][d], 0x05040100u);
        lo[1] = __builtin_amdgcn_perm(vreg[3][d], vreg[2][d], 0x05040100u);
        hi[0] = __builtin_amdgcn_perm(vreg[1][d], vreg[0][d], 0x07060302u);
        hi[1] = __builtin_amdgcn_perm(vreg[3][d], vreg[2][d], 0x07060302u);
        *reinterpret_cast<u32x2*>(vd + (2 * d) * TP) = lo;
        *reinterpret_cast<u32x2*>(vd + (2 * d + 1) * TP) = hi;
      }
    }
  };

  // ---- prologue: everything the tile needs first is requested at once -----------------------
  // The chunks from dstart on (same-block / causal rules) come FIRST: their addresses need no
  // routing table, so their loads, the Q loads above and the reads of the block list are all in
  // flight together.  The chunks of the prior attention blocks follow.
  const int n_diag = (min(len, tile_start + QTILE) - dstart + 63) >> 6;  // >= 1
  gload(dstart);
  if (tid == 0) lds_count = 0;
  __syncthreads();
  {
    // attention blocks that end at or before dstart: ids into LDS, count.  The list is sorted and
    // holds distinct block ids, so entry j >= j: only the first dstart/Bs entries can qualify.
    const int jmax = min(dstart / Bs, p.TN);
    int cnt = 0;
    for (int j = tid; j < jmax; j += NTHREADS) {
      const int e = list[j * list_stride];
      if (j < n_attn && (e + 1) * Bs <= dstart) {
        ++cnt;
        if (j < MAX_LDS_LIST) lds_list[j] = e;
      }
    }
    if (cnt) atomicAdd(&lds_count, cnt);
  }
  // types of the blocks the chunks from dstart on fall into, as a bit mask (bit i = block dstart/Bs + i)
  unsigned long long diag_attn;
  {
    const int blk = dstart / Bs + lane;
    const bool in_range = lane < n_diag && (size_t)blk * Bs < (size_t)min(len, tile_start + QTILE);
    diag_attn = __ballot(in_range && type_is_one(p.types, p.types_dtype, ((size_t)(bos_nats + blk) * p.HN + hn) * 2));
  }
  lstore(0);
  __syncthreads();
  const int n_prior_chunks = __builtin_amdgcn_readfirstlane(lds_count) * per_blk;
  const int n_iters = n_diag + n_prior_chunks;

  // Chunk iterator, all wave-uniform (scalar registers): the chunks from dstart on, then the
  // 64-key chunks of the prior attention blocks in list order.
  int nx_it = 1, nx_j = 0, nx_sub = 0;  // chunk 0 is already staged
  auto next_key_start = [&]() -> int {
    int ks;
    if (nx_it < n_diag) {
      ks = dstart + nx_it * 64;
    } else {
      int e;
      if (nx_j < MAX_LDS_LIST) e = __builtin_amdgcn_readfirstlane(lds_list[nx_j]);
      else e = __builtin_amdgcn_readfirstlane(list[nx_j * list_stride]);
      ks = e * Bs + nx_sub * 64;
      if (++nx_sub == per_blk) {
        nx_sub = 0;
        ++nx_j;
      }
    }
    ++nx_it;
    return ks;
  };
  int ks_fetch = 0;  // key start of the chunk the next gload brings in (known one iteration ahead)
  if (n_iters > 1) ks_fetch = next_key_start();

  const float c = p.scale_log2;
  f32x16 s[2][NQ];
  float mx[NQ];
  // ---- phase B (runs first): the chunks from dstart to the end of the tile, with the same-block and causal rules
  const int my_blk = q0 / Bs;
  int it = 0;
  for (; it < n_diag; ++it) {
    const int buf = it & 1;
    if (it + 1 < n_iters) gload(ks_fetch);
    const int jc = (dstart >> 6) + it;  // absolute chunk index of the keys
    const int kblk = (jc * 64) / Bs;
    bool active = wave_valid, causal = false;
    if (p.same_block) {
      if (jc > my_chunk) active = false;
      else if (jc == my_chunk) causal = true;
      else active = active && (kblk == my_blk || ((diag_attn >> (kblk - dstart / Bs)) & 1ull));
    } else {
      active = active && jc < my_chunk && kblk < my_blk && ((diag_attn >> (kblk - dstart / Bs)) & 1ull);
    }
    if (active && !NATSL_ABL(p.dbg & 8)) {
      if (causal) scores<DK, NQ, true>(Ks + buf * 64 * KP, QB, s, mx, c, lane, qloc0);
      else scores<DK, NQ, false>(Ks + buf * 64 * KP, QB, s, mx, c, lane, 0);
      if (needs_rescale<NQ>(mx, m_ref)) rescale<DV, NQ>(acc, m_ref, l_run, mx);
      exp_pv<DV, NQ>(Vs + buf * DV * TP, s, acc, m_ref, l_run, c, lane);
    }
    if (it + 1 < n_iters) lstore(buf ^ 1);
    if (it + 2 < n_iters) ks_fetch = next_key_start();
    __syncthreads();
  }

  // ---- phase A: whole attention blocks before the tile; every wave, no masks.  The inner loop is
  // the fast path; an iteration whose maxima outgrow the reference leaves it, rescales, finishes
  // and re-enters.
  if constexpr (NQ == 1) {
    // Software-pipelined in halves of 32 keys, so that each wave feeds the matrix pipe and the vector
    // ALU at the same time:  QK(0) | QK(1) with exp(0) | PV(0) with exp(1) | PV(1).
    // A half whose maximum outgrows the reference leaves the fast loop (pending = 1 or 2), the
    // iteration is finished on the slow path below and the loop is re-entered.
    constexpr int KSTEPS_ = DK / 16;
    while (it < n_iters) {
      int pending = 0;
      bf16x8 PB0[2], PB1[2];
      float rs = 0.f;
      for (; it < n_iters; ++it) {
        const int buf = it & 1;
        const bool more = it + 1 < n_iters;
        const bf16_t* Kb = Ks + buf * 64 * KP;
        const bf16_t* VTb = Vs + buf * DV * TP;
        if (more && !NATSL_ABL(p.dbg & 1)) gload(ks_fetch);
        if (wave_valid && !NATSL_ABL(p.dbg & 2)) {
          qk_half<DK>(Kb, 0, QB[0], s[0][0], lane);
          mx[0] = half_max<false>(s[0][0], 0, c, lane, 0);
          if (__any(mx[0] > m_ref[0] + RESCALE_SLACK)) {
            pending = 1;
            break;
          }
          const float neg = m_ref[0] == -INFINITY ? 0.f : -m_ref[0];
          rs = 0.f;
          // QK(1) with exp(0)
          qk_half<DK>(Kb, 1, QB[0], s[1][0], lane);
          probs_half(s[0][0], c, neg, rs, PB0);
          __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
#pragma unroll
          for (int st = 0; st < KSTEPS_; ++st) {
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
            if (st + 2 < KSTEPS_) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
            __builtin_amdgcn_sched_group_barrier(0x002, 5, 0);
            __builtin_amdgcn_sched_group_barrier(0x400, 2, 0);
          }
          mx[0] = half_max<false>(s[1][0], 1, c, lane, 0);
          if (__any(mx[0] > m_ref[0] + RESCALE_SLACK)) {
            pending = 2;
            break;
          }
          // PV(0) with exp(1)
          pv_half<DV>(VTb, 0, PB0, acc, lane);
          probs_half(s[1][0], c, neg, rs, PB1);
#pragma unroll
          for (int i = 0; i < 2 * VT; ++i) {
            __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
            __builtin_amdgcn_sched_group_barrier(0x002, 5, 0);
            __builtin_amdgcn_sched_group_barrier(0x400, 2, 0);
          }
          pv_half<DV>(VTb, 1, PB1, acc, lane);
          l_run[0] += rs;
        }
        if (more && !NATSL_ABL(p.dbg & 1) && !NATSL_ABL(p.dbg & 32)) lstore(buf ^ 1);
        if (it + 2 < n_iters) ks_fetch = next_key_start();
        __syncthreads();
      }
      if (pending) {
        const int buf = it & 1;
        const bf16_t* Kb = Ks + buf * 64 * KP;
        const bf16_t* VTb = Vs + buf * DV * TP;
        if (pending == 1) {
          rescale<DV, NQ>(acc, m_ref, l_run, mx);
          rs = 0.f;
          qk_half<DK>(Kb, 1, QB[0], s[1][0], lane);
          probs_half(s[0][0], c, -m_ref[0], rs, PB0);
          mx[0] = half_max<false>(s[1][0], 1, c, lane, 0);
        }
        // here: exp(0) is done against the current reference and mx holds the maximum of half 1
        pv_half<DV>(VTb, 0, PB0, acc, lane);
        l_run[0] += rs;
        rs = 0.f;
        if (__any(mx[0] > m_ref[0] + RESCALE_SLACK)) rescale<DV, NQ>(acc, m_ref, l_run, mx);
        probs_half(s[1][0], c, m_ref[0] == -INFINITY ? 0.f : -m_ref[0], rs, PB1);
        pv_half<DV>(VTb, 1, PB1, acc, lane);
        l_run[0] += rs;
        if (it + 1 < n_iters) lstore(buf ^ 1);
        if (it + 2 < n_iters) ks_fetch = next_key_start();
        __syncthreads();
        ++it;
      }
    }
  } else {
  while (it < n_iters) {
    bool pending = false;
    for (; it < n_iters; ++it) {
      const int buf = it & 1;
      const bool more = it + 1 < n_iters;
      if (more && !NATSL_ABL(p.dbg & 1)) gload(ks_fetch);
      if (wave_valid && !NATSL_ABL(p.dbg & 2)) {
        scores<DK, NQ, false>(Ks + buf * 64 * KP, QB, s, mx, c, lane, 0);
        if (needs_rescale<NQ>(mx, m_ref)) {
          pending = true;
          break;
        }
        exp_pv<DV, NQ>(Vs + buf * DV * TP, s, acc, m_ref, l_run, c, lane);
      }
      if (more && !NATSL_ABL(p.dbg & 1)) lstore(buf ^ 1);
      if (it + 2 < n_iters) ks_fetch = next_key_start();
      __syncthreads();
    }
    if (pending) {
      const int buf = it & 1;
      rescale<DV, NQ>(acc, m_ref, l_run, mx);
      exp_pv<DV, NQ>(Vs + buf * DV * TP, s, acc, m_ref, l_run, c, lane);
      if (it + 1 < n_iters) lstore(buf ^ 1);
      if (it + 2 < n_iters) ks_fetch = next_key_start();
      __syncthreads();
      ++it;
    }
  }
  }
  // ---- epilogue: normalise, transpose through LDS, coalesced stores ------------------------
  bf16_t* Os = reinterpret_cast<bf16_t*>(smem) + wave * QW * VP;  // this wave's [QW][VP]
#pragma unroll
  for (int qt = 0; qt < NQ; ++qt) {
    const float l_tot = xhalf_sum(l_run[qt]);
    const bool has = l_tot > 0.f;
    const float inv = has ? 1.f / l_tot : 0.f;
    const int qi = q0 + 32 * qt + l32;
    if (hf == 0 && qi < len)
      p.lse[((size_t)(bos + qi)) * p.HQ + hq] = has ? m_ref[qt] + __builtin_amdgcn_logf(l_tot) : 0.f;
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
  for (int pass = 0; pass < QW / ROWS_PER_PASS; ++pass) {
    const int row = pass * ROWS_PER_PASS + lane / SEGS, seg = lane % SEGS;
    const int qi = q0 + row;
    if (qi < len) {
      const u32x4 w = *reinterpret_cast<const u32x4*>(Os + row * VP + seg * 8);
      *reinterpret_cast<u32x4*>(p.o + ((size_t)(bos + qi) * p.HQ + hq) * DV + seg * 8) = w;
    }
  }
}

template <int DK, int DV, int NQ, int NWAVES>
static int launch_softmax(const SoftmaxParams& p, hipStream_t stream) {
  constexpr int KP = DK + 8, VP = DV + 8, QTILE = 32 * NQ * NWAVES;
  size_t lds = (size_t)2 * (64 * KP + DV * VT_PITCH) * sizeof(bf16_t);
  const size_t epi = (size_t)QTILE * VP * sizeof(bf16_t);
  if (epi > lds) lds = epi;
  auto kern = softmax_sparse_fwd_kernel<DK, DV, NQ, NWAVES>;
  hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
  if (e != hipSuccess) return fail(NATSL_ERR_LAUNCH, "softmax: cannot reserve %zu bytes of LDS: %s", lds, hipGetErrorString(e));
  const long long grid = p.seqs ? (long long)p.total_tiles * (QTILE_TABLE / QTILE) * p.HQ
                                : (long long)8 * ((p.B * p.HQ + 7) / 8) * ((p.T + QTILE - 1) / QTILE);
  if (grid <= 0) return NATSL_OK;
  hipLaunchKernelGGL(kern, dim3((unsigned)grid), dim3(64 * NWAVES), lds, stream, p);
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
  p.nq_tiles = cdiv(T, QTILE_TABLE);
  p.total_tiles = seqs ? total_units : B * p.nq_tiles;
  p.scale_log2 = scale * 1.4426950408889634f;
  p.same_block = same_block_visible ? 1 : 0;
  p.dbg = 0;
  p.variant = 1;
#ifdef NATSL_ABLATE
  if (getenv("NATSL_DBG")) p.dbg = atoi(getenv("NATSL_DBG"));
  if (getenv("NATSL_SOFTMAX_WAVES")) p.variant = atoi(getenv("NATSL_SOFTMAX_WAVES"));
#endif
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
#define NATSL_SM(KK, VV)                                              \
  if (K == KK && V == VV)                                             \
    return p.variant == 4 ? launch_softmax<KK, VV, 2, 4>(p, s) : p.variant == 8 ? launch_softmax<KK, VV, 1, 8>(p, s) : launch_softmax<KK, VV, 1, 4>(p, s);
  NATSL_SM(128, 128)
  NATSL_SM(64, 64)
  NATSL_SM(64, 128)
  NATSL_SM(128, 64)
#undef NATSL_SM
  return fail(NATSL_ERR_UNSUPPORTED, "softmax: head dims K=%d, V=%d not built (supported: 64/128 x 64/128)", K, V);
}
