// Softmax branch: sparse-KV causal flash attention for gfx950.
//
// One workgroup owns a tile of 32 queries per wave (4 waves: 128 queries, 8 waves: 256) of one (sequence, query
// head).  Key/value chunks of 64 tokens stream through LDS (double buffered): first the tile's own chunks with the
// causal / same-block rules, then every earlier block typed "attention" (taken from the sorted block list).
// Scores are computed transposed, S^T = K Q^T, so that a lane owns one query column: the online-softmax
// statistics are per-lane scalars and the probabilities already sit in the B-operand layout of the second
// product O^T = V^T P^T.  V is staged transposed in LDS, so the V^T operand is two 8-byte reads per lane.
#include "natsl_device.h"
#include "natsl_host.h"
#include <type_traits>
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
  int variant;  // 4: 128-query tile on 4 waves, 8: 256-query tile on 8 waves
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

// ---- one 64-key chunk for one wave (32 queries) -------------------------------------------------------------
// The chunk is 32 matrix instructions: S^T = K Q^T for key halves 0 and 1 (2 x DK/16), then O^T += V^T P^T for
// the two halves (2 x 2 x DV/32).  Their LDS operands form one stream (K rows, then V^T rows) that is read
// OPERANDS_AHEAD instructions ahead of its use, across the four phases, so no matrix instruction waits a full
// LDS latency for its operand.  The vector work of a half (exp2, row sums, packing to bf16) runs under the matrix
// instructions of the next phase:   QK(0) | QK(1) with exp(0) | PV(0) with exp(1) | PV(1).
// Accumulator register r of key half kt is key 32kt + 8(r/4) + 4hf + r%4; the same order is used for the k-slots
// of the V^T operand, so the probabilities need no data movement.
// The reference maximum m_ref moves only when a half's maximum outgrows it by more than RESCALE_SLACK; that, and
// the causal mask of the wave's own chunk, live in short side blocks, so there is one main path.
constexpr int OPERANDS_AHEAD = 3;

// hide the keys behind the query (the wave's own chunk): key 32kt + 8(r/4) + 4hf + r%4 against query qloc0 + lane%32
NATSL_DEVICE void mask_half(f32x16& s, const int kt, const int lane, const int qloc0) {
  const int d = qloc0 + (lane & 31) - 32 * kt - 4 * (lane >> 5);  // visible iff 8(r/4) + r%4 <= d
#pragma unroll
  for (int r = 0; r < 16; ++r)
    if (8 * (r >> 2) + (r & 3) > d) s[r] = -INFINITY;
}

// scaled row maximum of one half (both lane halves joined)
NATSL_DEVICE float half_max(const f32x16& s, const float c) {
  float m = -INFINITY;
#pragma unroll
  for (int r = 0; r < 16; ++r) m = fmaxf(m, s[r]);
  return xhalf_max(m) * c;
}

// P = exp2(S*c - m_ref) for one half, packed to bf16 in the B-operand order; adds the row sums
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
NATSL_DEVICE void rescale(f32x16 (&acc)[DV / 32], float& m_ref, float& l_run, const float mx) {
  const float m_new = fmaxf(m_ref, mx);
  const float alpha = __builtin_amdgcn_exp2f(m_ref - (m_new == -INFINITY ? 0.f : m_new));
  m_ref = m_new;
  l_run *= alpha;
#pragma unroll
  for (int vt = 0; vt < DV / 32; ++vt)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[vt][r] *= alpha;
}

template <int DK, int DV>
NATSL_DEVICE void chunk_pipelined(const bf16_t* Kb, const bf16_t* VTb, const bf16x8 (&QB)[DK / 16], f32x16 (&acc)[DV / 32],
                                  float& m_ref, float& l_run, const float c, const int lane, const bool causal,
                                  const int qloc0) {
  constexpr int KP = DK + 8, TP = VT_PITCH, KS = DK / 16, VT = DV / 32;
  constexpr int NK = 2 * KS, NV = 4 * VT, NOPS = NK + NV, A = OPERANDS_AHEAD;
  const int l32 = lane & 31, hf = lane >> 5;
  const bf16_t* krow = Kb + l32 * KP + 8 * hf;
  const bf16_t* vrow = VTb + l32 * TP + 4 * hf;
  // operand j of the chunk: K rows of half j/KS at k-step j%KS, then V^T rows (half, 16-key group ss, value tile vt);
  // the 16-key groups of odd value tiles are stored swapped
  auto ld_op = [&](const int j) __attribute__((always_inline)) -> bf16x8 {
#ifdef NATSL_ABL_NOLDS
    return QB[j % KS];
#endif
    if (j < NK) return ld8(krow + 32 * (j / KS) * KP + 16 * (j % KS));
    const int i = j - NK, half = i / (2 * VT), ss = (i / VT) & 1, vt = i % VT;
    const bf16_t* vr = vrow + 32 * vt * TP + 16 * ((2 * half + ss) ^ (vt & 1));
    const u32x2 lo = *reinterpret_cast<const u32x2*>(vr), hi = *reinterpret_cast<const u32x2*>(vr + 8);
    const u32x4 w = {lo[0], lo[1], hi[0], hi[1]};
    return __builtin_bit_cast(bf16x8, w);
  };
  bf16x8 op[NOPS + A];
#pragma unroll
  for (int j = 0; j < A; ++j) op[j] = ld_op(j);
  f32x16 s0, s1;
#pragma unroll
  for (int r = 0; r < 16; ++r) s0[r] = s1[r] = 0.f;

  // ---- QK(0)
#pragma unroll
  for (int st = 0; st < KS; ++st) {
    op[st + A] = ld_op(st + A);
    s0 = mfma32(op[st], QB[st], s0);
  }
  __builtin_amdgcn_sched_group_barrier(0x100, A, 0);
#pragma unroll
  for (int st = 0; st < KS; ++st) {
    __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
  }
  if (causal) mask_half(s0, 0, lane, qloc0);
  float mx = half_max(s0, c);
#ifndef NATSL_ABL_NOCHECK
  if (__any(mx > m_ref + RESCALE_SLACK)) rescale<DV>(acc, m_ref, l_run, mx);
#endif
  float neg = m_ref == -INFINITY ? 0.f : -m_ref;
  float rs = 0.f;
  bf16x8 PB0[2], PB1[2];

  // ---- QK(1) with exp(0)
#pragma unroll
  for (int st = 0; st < KS; ++st) {
    op[KS + st + A] = ld_op(KS + st + A);
    s1 = mfma32(op[KS + st], QB[st], s1);
  }
  probs_half(s0, c, neg, rs, PB0);
#pragma unroll
  for (int st = 0; st < KS; ++st) {
    __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
    __builtin_amdgcn_sched_group_barrier(0x002, 40 / KS, 0);
    __builtin_amdgcn_sched_group_barrier(0x400, 16 / KS, 0);
  }
  if (causal) mask_half(s1, 1, lane, qloc0);
  mx = half_max(s1, c);
#ifndef NATSL_ABL_NOCHECK
  if (__any(mx > m_ref + RESCALE_SLACK)) {
    // the second half outgrew the reference: move it, and form the first half's probabilities again
    rescale<DV>(acc, m_ref, l_run, mx);
    neg = -m_ref;
    rs = 0.f;
    probs_half(s0, c, neg, rs, PB0);
  }
#endif

  // ---- PV(0) with exp(1)
#pragma unroll
  for (int i = 0; i < 2 * VT; ++i) {
    op[NK + i + A] = ld_op(NK + i + A);
    acc[i % VT] = mfma32(op[NK + i], PB0[i / VT], acc[i % VT]);
  }
  probs_half(s1, c, neg, rs, PB1);
#pragma unroll
  for (int i = 0; i < 2 * VT; ++i) {
    __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
    __builtin_amdgcn_sched_group_barrier(0x002, 40 / (2 * VT), 0);
    __builtin_amdgcn_sched_group_barrier(0x400, 16 / (2 * VT), 0);
  }

  // ---- PV(1)
#pragma unroll
  for (int i = 0; i < 2 * VT; ++i) {
    if (NK + 2 * VT + i + A < NOPS) op[NK + 2 * VT + i + A] = ld_op(NK + 2 * VT + i + A);
    acc[i % VT] = mfma32(op[NK + 2 * VT + i], PB1[i / VT], acc[i % VT]);
  }
#pragma unroll
  for (int i = 0; i < 2 * VT; ++i) {
    if (NK + 2 * VT + i + A < NOPS) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
  }
  l_run += rs;  // partial over this lane's keys; the lane halves are joined in the epilogue
}

// NWAVES waves of 32 queries: the workgroup owns QTILE = 32*NWAVES queries.
template <int DK, int DV, int NWAVES>
__global__ __launch_bounds__(64 * NWAVES, NWAVES == 4 ? 2 : 1) __attribute__((amdgpu_waves_per_eu(2, 2)))
void softmax_sparse_fwd_kernel(const SoftmaxParams p) {
  constexpr int NTHREADS = 64 * NWAVES, QW = 32, QTILE = QW * NWAVES;  // QW = queries per wave
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
  bf16x8 QB[KSTEPS];
  {
    const int qi = min(q0 + l32, len - 1);  // rows past the end are computed on a copy and never stored
    const bf16_t* qr = qp + (size_t)qi * p.HQ * DK + 8 * hf;
#pragma unroll
    for (int s = 0; s < KSTEPS; ++s) QB[s] = ld8(qr + 16 * s);
  }

  if (tile_start >= len) return;  // packed input: a sequence's last 256-row table slot may hold no tile of this size

  f32x16 acc[VT];
#pragma unroll
  for (int vt = 0; vt < VT; ++vt)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[vt][r] = 0.f;
  float m_ref = -INFINITY, l_run = 0.f;

  // ---- global -> register -> LDS staging of one 64-key chunk -----------------------------
  // K: 16-byte segments, whole rows per load instruction, stored row-major.  V: a thread owns 4 keys x 8 value
  // columns; the 4x8 block is transposed in registers and stored as 8 rows of 4 keys.
  // 4 waves: every thread stages K and V, one chunk in flight.  8 waves: a thread stages K or V, never both, so
  // two chunks are in flight per thread (two register sets of 4 loads) at the same register cost.
  static_assert(NTHREADS == 256 || NTHREADS == 512, "staging is written for 4 or 8 waves");
  constexpr bool SPLIT = NTHREADS == 512;
  constexpr int NSETS = SPLIT ? 2 : 1;
  constexpr int KL = DK / 32;
  const int st = SPLIT ? (tid & 255) : tid;
  const bool do_k = !SPLIT || tid < 256, do_v_role = !SPLIT || tid >= 256;
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
  // Every thread issues the same loads on every path (threads without a V role re-read the first keys): loads
  // inside lane- or wave-dependent branches make the compiler wait for ALL outstanding loads at the next use.
  const int v_kg_ld = v_on ? v_kg : 0;
  struct Staged { u32x4 k[SPLIT ? 1 : KL]; u32x4 v[4]; };   // 8 waves: v[] holds the thread's K or V loads
  Staged sreg[NSETS];
  // FULL chunks (wholly inside the sequence, as every prior attention block is): wave-uniform chunk base + a
  // per-thread byte offset that never changes.  8 waves: pointer, token pitch and rows are chosen by the role.
  const char* role_ptr = do_k ? reinterpret_cast<const char*>(kp) : reinterpret_cast<const char*>(vp);
  const size_t role_pitch = (do_k ? krow : vrow) * sizeof(bf16_t);
  const int role_row0 = do_k ? ld_row : 4 * v_kg_ld;
  const unsigned role_seg = (do_k ? 8 * ld_seg : 8 * v_seg) * sizeof(bf16_t);
  auto role_row = [&](const int j) -> int { return role_row0 + (do_k ? KROWS * (j % KL) : j); };  // row of load j in the chunk
  const unsigned k_off = (unsigned)(((size_t)ld_row * krow + ld_seg * 8) * sizeof(bf16_t));
  const size_t k_pass = (size_t)KROWS * krow * sizeof(bf16_t);
  const unsigned v_off = (unsigned)(((size_t)(4 * v_kg_ld) * vrow + 8 * v_seg) * sizeof(bf16_t));
  unsigned role_off[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) role_off[j] = (unsigned)((size_t)role_row(j) * role_pitch) + role_seg;
  auto gload = [&](auto full_c, const int ks, Staged& r) __attribute__((always_inline)) {
    // Not FULL: rows past the end are clamped to the last row: such keys are always hidden by the causal rule
    // (a valid query precedes them), so only finite values are needed there.
    constexpr bool FULL = decltype(full_c)::value;
    if constexpr (SPLIT) {
      const char* cb = role_ptr + (size_t)ks * role_pitch;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        if (FULL) r.v[j] = *reinterpret_cast<const u32x4*>(cb + role_off[j]);
        else r.v[j] = *reinterpret_cast<const u32x4*>(role_ptr + (size_t)min(ks + role_row(j), len - 1) * role_pitch + role_seg);
      }
    } else {
      const char* kb = reinterpret_cast<const char*>(kp + (size_t)ks * krow) + k_off;
      const char* vb = reinterpret_cast<const char*>(vp + (size_t)ks * vrow) + v_off;
#pragma unroll
      for (int i = 0; i < KL; ++i) {
        if (FULL) r.k[i] = *reinterpret_cast<const u32x4*>(kb + i * k_pass);
        else r.k[i] = *reinterpret_cast<const u32x4*>(kp + (size_t)min(ks + ld_row + KROWS * i, len - 1) * krow + 8 * ld_seg);
      }
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        if (FULL) r.v[j] = *reinterpret_cast<const u32x4*>(vb + j * vrow * sizeof(bf16_t));
        else r.v[j] = *reinterpret_cast<const u32x4*>(vp + (size_t)min(ks + 4 * v_kg_ld + j, len - 1) * vrow + 8 * v_seg);
      }
    }
  };
  auto lstore = [&](const int buf, const Staged& r) __attribute__((always_inline)) {
    const u32x4 (&rk)[SPLIT ? 4 : KL] = *reinterpret_cast<const u32x4 (*)[SPLIT ? 4 : KL]>(SPLIT ? r.v : r.k);
    if (do_k) {
      bf16_t* kd = Ks + (buf * 64 + ld_row) * KP + 8 * ld_seg;
#pragma unroll
      for (int i = 0; i < KL; ++i) *reinterpret_cast<u32x4*>(kd + KROWS * i * KP) = rk[i];
    }
    if (v_on) {
      bf16_t* vd = Vs + (buf * DV + 8 * v_seg) * TP + 4 * (v_kg ^ (4 * ((v_seg >> 2) & 1)));
#pragma unroll
      for (int d = 0; d < 4; ++d) {
        // value columns 2d (low halves) and 2d+1 (high halves) of the four keys
        u32x2 lo, hi;
        lo[0] = __builtin_amdgcn_perm(r.v[1][d], r.v[0][d], 0x05040100u);
        lo[1] = __builtin_amdgcn_perm(r.v[3][d], r.v[2][d], 0x05040100u);
        hi[0] = __builtin_amdgcn_perm(r.v[1][d], r.v[0][d], 0x07060302u);
        hi[1] = __builtin_amdgcn_perm(r.v[3][d], r.v[2][d], 0x07060302u);
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
  // Only a sequence's last tile can hold chunks that reach past its end; it takes the plain loop further down.
  const bool ragged_tile = dstart + 64 * n_diag > len;
  if (ragged_tile) {
    gload(std::false_type{}, dstart, sreg[0]);
  } else {
    gload(std::true_type{}, dstart, sreg[0]);
    if (SPLIT && n_diag >= 2) gload(std::true_type{}, dstart + 64, sreg[NSETS - 1]);  // the second chunk too: its address needs no list
  }
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
  lstore(0, sreg[0]);
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

  const float c = p.scale_log2;
  const int my_blk = q0 / Bs;
  // one chunk for this wave: the chunks from dstart on follow the same-block and causal rules, the prior attention
  // blocks are seen whole
  auto compute = [&](const int it, const int buf) __attribute__((always_inline)) {
    bool active = wave_valid, causal = false;
    if (it < n_diag) {
      const int jc = (dstart >> 6) + it;  // absolute chunk index of the keys
      const int kblk = (jc * 64) / Bs;
      if (p.same_block) {
        if (jc > my_chunk) active = false;
        else if (jc == my_chunk) causal = true;
        else active = active && (kblk == my_blk || ((diag_attn >> (kblk - dstart / Bs)) & 1ull));
      } else {
        active = active && jc < my_chunk && kblk < my_blk && ((diag_attn >> (kblk - dstart / Bs)) & 1ull);
      }
    }
    if (active && !NATSL_ABL(p.dbg & 2))
      chunk_pipelined<DK, DV>(Ks + buf * 64 * KP, Vs + buf * DV * TP, QB, acc, m_ref, l_run, c, lane, causal, qloc0);
  };

  if (ragged_tile) {
    // plain loop, one chunk in flight, every row clamped to the sequence
    int ks_fetch = dstart;
    if (n_iters > 1) ks_fetch = next_key_start();
    for (int it = 0; it < n_iters; ++it) {
      const int buf = it & 1;
      if (it + 1 < n_iters) gload(std::false_type{}, ks_fetch, sreg[0]);
      compute(it, buf);
      if (it + 1 < n_iters) lstore(buf ^ 1, sreg[0]);
      if (it + 2 < n_iters) ks_fetch = next_key_start();
      __syncthreads();
    }
  } else if constexpr (SPLIT) {
    // Chunk it+2 is requested while chunk it is computed and chunk it+1 (requested one iteration earlier) is
    // written to LDS: how long a chunk's loads take to come back no longer sets the pace of an iteration.  Every
    // iteration issues its loads unconditionally (past the last chunk it re-reads the last one), so that the wait
    // before the LDS writes counts exactly the loads issued after the ones it needs.
    int ks_next = dstart;                                    // chunk 1 (a repeat of chunk 0 if there is no other)
    if (n_iters > 1) ks_next = next_key_start();
    if (n_diag < 2) gload(std::true_type{}, ks_next, sreg[NSETS - 1]);
    if (n_iters > 2) ks_next = next_key_start();             // chunk 2
    auto step = [&](auto parity, const int it) __attribute__((always_inline)) {
      constexpr int P = decltype(parity)::value;
      if (!NATSL_ABL(p.dbg & 1)) gload(std::true_type{}, ks_next, sreg[P % NSETS]);
      compute(it, P);
      if (it + 1 < n_iters && !NATSL_ABL(p.dbg & 1)) lstore(P ^ 1, sreg[(P ^ 1) % NSETS]);
      if (it + 3 < n_iters) ks_next = next_key_start();
      if (!NATSL_ABL(p.dbg & 4)) __syncthreads();
    };
    int it = 0;
    for (; it + 1 < n_iters; it += 2) {
      step(std::integral_constant<int, 0>{}, it);
      step(std::integral_constant<int, 1>{}, it + 1);
    }
    if (it < n_iters) step(std::integral_constant<int, 0>{}, it);
  } else {
    int ks_fetch = dstart;  // key start of the chunk the next loads bring in (past the last chunk: a repeat)
    if (n_iters > 1) ks_fetch = next_key_start();
    for (int it = 0; it < n_iters; ++it) {
      const int buf = it & 1;
      gload(std::true_type{}, ks_fetch, sreg[0]);
      compute(it, buf);
      if (it + 1 < n_iters) lstore(buf ^ 1, sreg[0]);
      if (it + 2 < n_iters) ks_fetch = next_key_start();
      __syncthreads();
    }
  }

  // ---- epilogue: normalise, transpose through LDS, coalesced stores ------------------------
  bf16_t* Os = reinterpret_cast<bf16_t*>(smem) + wave * QW * VP;  // this wave's [QW][VP]
  {
    const float l_tot = xhalf_sum(l_run);
    const bool has = l_tot > 0.f;
    const float inv = has ? 1.f / l_tot : 0.f;
    const int qi = q0 + l32;
    if (hf == 0 && qi < len)
      p.lse[((size_t)(bos + qi)) * p.HQ + hq] = has ? m_ref + __builtin_amdgcn_logf(l_tot) : 0.f;
#pragma unroll
    for (int vt = 0; vt < VT; ++vt)
#pragma unroll
      for (int rg = 0; rg < 4; ++rg) {
        u32x2 w;
        w[0] = pack_bf16x2(acc[vt][4 * rg] * inv, acc[vt][4 * rg + 1] * inv);
        w[1] = pack_bf16x2(acc[vt][4 * rg + 2] * inv, acc[vt][4 * rg + 3] * inv);
        *reinterpret_cast<u32x2*>(Os + l32 * VP + 32 * vt + 8 * rg + 4 * hf) = w;
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

template <int DK, int DV, int NWAVES>
static int launch_softmax(const SoftmaxParams& p, hipStream_t stream) {
  constexpr int KP = DK + 8, VP = DV + 8, QTILE = 32 * NWAVES;
  size_t lds = (size_t)2 * (64 * KP + DV * VT_PITCH) * sizeof(bf16_t);
  const size_t epi = (size_t)QTILE * VP * sizeof(bf16_t);
  if (epi > lds) lds = epi;
  auto kern = softmax_sparse_fwd_kernel<DK, DV, NWAVES>;
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
  // 256-query tiles on 8 waves (two chunks in flight per thread) once there are enough of them to fill the GPU twice
  p.variant = (long long)B * HQ * cdiv(T, 256) >= 512 ? 8 : 4;
#ifdef NATSL_ABLATE
  if (getenv("NATSL_DBG")) p.dbg = atoi(getenv("NATSL_DBG"));
  if (getenv("NATSL_SOFTMAX_WAVES")) p.variant = atoi(getenv("NATSL_SOFTMAX_WAVES"));
#endif
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
#define NATSL_SM(KK, VV)                                              \
  if (K == KK && V == VV)                                             \
    return p.variant == 8 ? launch_softmax<KK, VV, 8>(p, s) : launch_softmax<KK, VV, 4>(p, s);
  NATSL_SM(128, 128)
  NATSL_SM(64, 64)
  NATSL_SM(64, 128)
  NATSL_SM(128, 64)
#undef NATSL_SM
  return fail(NATSL_ERR_UNSUPPORTED, "softmax: head dims K=%d, V=%d not built (supported: 64/128 x 64/128)", K, V);
}
