// Softmax branch: sparse-KV causal flash attention for gfx950.
//
// One workgroup owns a tile of 32 queries per wave (4 waves: 128 queries, 8 waves: 256) of one (sequence, query
// head).  Key/value chunks of 64 tokens stream through LDS: first the tile's own chunks with the causal / same-block
// rules, then every earlier block typed "attention" (taken from the sorted block list).
// Scores are computed transposed, S^T = K Q^T, so that a lane owns one query column: the online-softmax
// statistics are per-lane scalars and the probabilities already sit in the B-operand layout of the second
// product O^T = V^T P^T.  V is staged transposed in LDS.
// Two ways through a tile: chunk_pipelined() (4 waves, and the ragged last tile of a sequence on 8 waves: K and V
// staged through registers, double buffered, one chunk as one pipelined instruction stream per wave) and, for full
// tiles on 8 waves, the three-phase schedule further down (K and V by LDS-DMA, the two waves of a SIMD half a chunk
// apart).
#include "natsl_device.h"
#include "natsl_host.h"
#include <atomic>
#include <mutex>
#include <type_traits>

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
  int g_kv, g_n;  // query heads per kv head / per selector head
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
  int d = qloc0 + (lane & 31) - 32 * kt - 4 * (lane >> 5);  // visible iff 8(r/4) + r%4 <= d
  // (kept where it is: hoisted out of the chunk loop, the sixteen comparisons below occupy 32 scalar registers for good)
  asm volatile("" : "+v"(d));
#pragma unroll
  for (int r = 0; r < 16; ++r)
    if (8 * (r >> 2) + (r & 3) > d) s[r] = -INFINITY;
}

// max(a, b, c) as ONE instruction.  fmaxf() costs three here: the compiler first quiets possible signalling NaNs of
// each operand (v_mul by 1.0) because it cannot know that matrix-instruction results are canonical.  The scores hold
// no NaNs (masked entries are -inf), so the plain instruction gives the same result.
NATSL_DEVICE float max3_plain(const float a, const float b, const float c) {
  float r;
  asm("v_max3_f32 %0, %1, %2, %3" : "=v"(r) : "v"(a), "v"(b), "v"(c));
  return r;
}

// scaled row maximum of one half (both lane halves joined)
NATSL_DEVICE float half_max(const f32x16& s, const float c) {
  float m0 = -INFINITY, m1 = -INFINITY;
#pragma unroll
  for (int r = 0; r < 16; r += 4) {
    m0 = max3_plain(m0, s[r], s[r + 1]);
    m1 = max3_plain(m1, s[r + 2], s[r + 3]);
  }
  return xhalf_max(max3_plain(m0, m1, m1)) * c;
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
  if (__any(mx > m_ref + RESCALE_SLACK)) rescale<DV>(acc, m_ref, l_run, mx);
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
  if (__any(mx > m_ref + RESCALE_SLACK)) {
    // the second half outgrew the reference: move it, and form the first half's probabilities again
    rescale<DV>(acc, m_ref, l_run, mx);
    neg = -m_ref;
    rs = 0.f;
    probs_half(s0, c, neg, rs, PB0);
  }

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

// ---- the 8-wave schedule: one chunk as three phases ----------------------------------------------------------------
// K chunks go from global memory straight into LDS (global_load_lds_dwordx4: every lane names 16 source bytes, the
// wave's 1 KiB lands contiguously at the LDS address in M0): no staging registers, no LDS store instructions.  The K
// tile is row-major, [64 keys][DK] without padding; bank conflicts are avoided by an XOR swizzle of the 16-byte
// segments of a row, applied on the way in by letting each lane fetch the segment that belongs at its LDS position.
// The operand read is ds_read_b128, 16 lanes = 16 rows = 256 bytes per clock: with DK = 128 (one row = all 64 banks)
// segment s of row r sits at s ^ (r & 15); with DK = 64 (two rows share the banks) at s ^ ((r >> 1) & 7).
// V has to be transposed on the way (the matrix instruction wants 8 consecutive keys per lane, memory has 8
// consecutive value columns), which the DMA cannot do: it passes through registers (4x8 transposes with v_perm_b32).
// The two waves that share a SIMD run half a chunk apart (see the kernel), so a wave's vector phase (softmax_phase)
// meets the other wave's matrix phases (pv_phase, qk_phase).

// one DMA instruction: lane l copies 16 bytes from base + voff to LDS byte address lds + 16 l
NATSL_DEVICE void dma16(const void* base, const unsigned voff, const unsigned lds) {
  asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1" ::"v"(voff), "s"(base), "s"(lds) : "memory", "m0");
}

// S^T = K Q^T - m_ref for both key halves of one chunk: the accumulators start from minus the reference maximum of the
// lane's query, so the scores come out of the matrix pipe already shifted.  The halves alternate so that consecutive
// instructions are independent.  kaddr: LDS byte address of this lane's row (lane%32) in the tile, plus 16*((lane>>5) ^
// swizzle(row)): XOR-ing it with 32*(k-step) gives the swizzled position of the lane's 16 bytes of that k-step.
template <int DK>
NATSL_DEVICE void qk_phase(const unsigned kaddr, const bf16x8 (&QB)[DK / 16], const float m_ref, f32x16& s0, f32x16& s1) {
  constexpr int N = DK / 8, A = OPERANDS_AHEAD;
  typedef __attribute__((address_space(3))) const bf16x8* lds_op;
  unsigned base[DK / 16];  // one register per k-step, opaque to the compiler (see pv_phase)
#pragma unroll
  for (int q = 0; q < DK / 16; ++q) {
    base[q] = kaddr ^ (32u * q);
    asm("" : "+v"(base[q]));
  }
  auto ld_op = [&](const int j) __attribute__((always_inline)) -> bf16x8 {
    const int st = j >> 1, half = j & 1;
    return *reinterpret_cast<lds_op>(base[st] + half * 32u * (2u * DK));
  };
  bf16x8 op[N + A];
#pragma unroll
  for (int j = 0; j < A; ++j) op[j] = ld_op(j);
  f32x16 start;  // short-lived: the first instruction of each chain reads it
#pragma unroll
  for (int r = 0; r < 16; ++r) start[r] = -m_ref;
#pragma unroll
  for (int j = 0; j < N; ++j) {
    if (j + A < N) op[j + A] = ld_op(j + A);
    if (j & 1) s1 = mfma32(op[j], QB[j >> 1], j == 1 ? start : s1);
    else s0 = mfma32(op[j], QB[j >> 1], j == 0 ? start : s0);
  }
  __builtin_amdgcn_sched_group_barrier(0x100, A, 0);
#pragma unroll
  for (int j = 0; j < N; ++j) {
    if (j + A < N) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
  }
}

// sum of the two bf16 halves of w, added to acc in fp32
NATSL_DEVICE float dot2_ones(const unsigned w, const float acc) {
  typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;
  const bf16x2 ones = {(__bf16)1.0f, (__bf16)1.0f};
  return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2, w), ones, acc, false);
}

// O^T += V^T P^T for one chunk: PB[g] holds the probabilities of keys 16 g .. 16 g + 15.  V is staged transposed,
// [DV][VTP] with the keys of a 16-key group stored in the order the probabilities are held (a lane's 8 k-slots are 16
// contiguous bytes), so an operand is ONE ds_read_b128: the LDS pipe takes as long for an 8-byte read instruction as
// for a 16-byte one, and two reads per operand made this phase LDS-bound.  vaddr: LDS byte address of the lane's row
// (lane%32) of the tile plus 16*(lane>>5).  The row sums are taken from the same rounded probabilities, one v_dot2
// under each matrix instruction.
constexpr int VTP = 72;  // elements per row of that tile (64 keys + 8): conflict-free 16-byte reads and 8-byte transposed stores
template <int DV>
NATSL_DEVICE void pv_phase(const unsigned vaddr, const bf16x8 (&PB)[4], f32x16 (&acc)[DV / 32], float& l_run) {
  constexpr int VT = DV / 32, N = 4 * VT, A = OPERANDS_AHEAD, DOTS = 16 / N;  // 16 packed words per lane
  static_assert(16 % N == 0, "row sums ride on the matrix instructions");
  typedef __attribute__((address_space(3))) const bf16x8* lds_op;
  // (opaque to the compiler: it must stay ONE base register with the tile offsets in the instructions' offset fields;
  // re-associated with the ring arithmetic of the caller, half of the offsets came out negative, each read got an
  // address computation of its own and the reads were no longer issued ahead of their use)
  unsigned base = vaddr;
  asm("" : "+v"(base));
  auto ld_op = [&](const int i) __attribute__((always_inline)) -> bf16x8 {
    const int g = i / VT, vt = i % VT;
    return *reinterpret_cast<lds_op>(base + 32u * vt * (2u * VTP) + 32u * g);
  };
  bf16x8 op[N + A];
#pragma unroll
  for (int j = 0; j < A; ++j) op[j] = ld_op(j);
#pragma unroll
  for (int i = 0; i < N; ++i) {
    if (i + A < N) op[i + A] = ld_op(i + A);
    acc[i % VT] = mfma32(op[i], PB[i / VT], acc[i % VT]);
#pragma unroll
    for (int d = 0; d < DOTS; ++d) l_run = dot2_ones(__builtin_bit_cast(u32x4, PB[(i * DOTS + d) / 4])[(i * DOTS + d) % 4], l_run);
  }
  __builtin_amdgcn_sched_group_barrier(0x100, A, 0);
#pragma unroll
  for (int i = 0; i < N; ++i) {
    if (i + A < N) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
  }
}

// Shifted scores of one chunk (s = score - m_ref, straight from the matrix pipe) -> probabilities in the B-operand
// order.  The common path is a maximum (for the check), 32 exp2 and the packing.  The reference moves, in a side
// block, when a score outgrows it by more than `thr`: -inf while the row has seen no key yet (m_ref is then still the
// arbitrary 0 and the first visible score sets the real one), RESCALE_SLACK afterwards.
template <int DV>
NATSL_DEVICE void softmax_phase(f32x16& s0, f32x16& s1, f32x16 (&acc)[DV / 32], float& m_ref, float& l_run, float& thr,
                                const int lane, const bool causal, const int qloc0, bf16x8 (&PB)[4]) {
  if (causal) {
    mask_half(s0, 0, lane, qloc0);
    mask_half(s1, 1, lane, qloc0);
  }
  float m0 = -INFINITY, m1 = -INFINITY;
#pragma unroll
  for (int r = 0; r < 16; r += 2) {
    m0 = max3_plain(m0, s0[r], s0[r + 1]);
    m1 = max3_plain(m1, s1[r], s1[r + 1]);
  }
  const float mx = xhalf_max(max3_plain(m0, m1, m1));
  if (__any(mx > thr)) {
    const bool unset = thr < 0.f;
    float m_new = unset ? m_ref + mx : fmaxf(m_ref, m_ref + mx);
    if (mx == -INFINITY) m_new = m_ref;  // still nothing visible: keep whatever reference there is
    else thr = RESCALE_SLACK;
    const float delta = m_new - m_ref;
    const float alpha = unset ? 1.f : __builtin_amdgcn_exp2f(-delta);  // unset: nothing accumulated yet
    m_ref = m_new;
    l_run *= alpha;
#pragma unroll
    for (int vt = 0; vt < DV / 32; ++vt)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[vt][r] *= alpha;
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      s0[r] -= delta;
      s1[r] -= delta;
    }
  }
#pragma unroll
  for (int g = 0; g < 4; ++g) {
    const f32x16& s = g < 2 ? s0 : s1;
    u32x4 w;
#pragma unroll
    for (int j = 0; j < 4; ++j)
      w[j] = pack_bf16x2(__builtin_amdgcn_exp2f(s[8 * (g & 1) + 2 * j]), __builtin_amdgcn_exp2f(s[8 * (g & 1) + 2 * j + 1]));
    PB[g] = __builtin_bit_cast(bf16x8, w);
  }
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
    // (unsigned arithmetic throughout: a signed division by a run-time value costs a third more scalar instructions,
    // and this preamble is what every tile starts with)
    const unsigned n_pairs = (unsigned)(p.B * p.HQ);
    const unsigned xcd = blockIdx.x & 7u, j = blockIdx.x >> 3;
    const unsigned nq_tiles = ((unsigned)p.T + QTILE - 1) / QTILE;
    const unsigned jq = j / nq_tiles;
    const unsigned pair = jq * 8 + xcd;
    if (pair >= n_pairs) return;
    tile = (int)(nq_tiles - 1 - (j - jq * nq_tiles));
    n = (int)(pair / (unsigned)p.HQ);
    hq = (int)(pair - (unsigned)n * (unsigned)p.HQ);
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
  const int hkv = (int)((unsigned)hq / (unsigned)p.g_kv), hn = (int)((unsigned)hq / (unsigned)p.g_n);
  const int tile_start = tile * QTILE;
  const int q0 = tile_start + wave * QW;      // this wave's first query
  const int my_chunk = q0 >> 6;               // the 64-key chunk of the sequence that holds them
  const int qloc0 = q0 & 63;                  // ... and where in that chunk
  // keys from here on are handled chunk by chunk with the same-block / causal rules: the start of
  // the tile, or of the selector block it falls into when blocks are larger than the tile
  const int dstart = (int)(((unsigned)tile_start / (unsigned)p.block) * (unsigned)p.block);
  const int dblk = (int)((unsigned)dstart / (unsigned)p.block);   // the selector block dstart begins
  const bool wave_valid = q0 < len;

  const bf16_t* qp = p.q + ((size_t)bos * p.HQ + hq) * DK;
  const bf16_t* kp = p.k + ((size_t)bos * p.HKV + hkv) * DK;
  const bf16_t* vp = p.v + ((size_t)bos * p.HKV + hkv) * DV;
  const size_t krow = (size_t)p.HKV * DK, vrow = (size_t)p.HKV * DV;
  const int32_t* list = p.idx + ((size_t)bos_nats * p.HN + hn) * 2;  // element j at list[j*HN*2]
  const size_t list_stride = (size_t)p.HN * 2;
  // (read where it is used: a scalar load from global memory makes the NEXT scalar-memory wait, whatever it is for,
  // last a full memory latency, and this one would sit in front of the tile's first requests)
  const int32_t* n_attn_p = p.nblk + ((size_t)n * p.HN + hn) * 2;

  // ---- Q as the B operand of S^T = K Q^T: lane = query column ----------------------------
  bf16x8 QB[KSTEPS];
  {
    const int qi = min(q0 + l32, len - 1);  // rows past the end are computed on a copy and never stored
    const bf16_t* qr = qp + (size_t)qi * p.HQ * DK + 8 * hf;
    // The queries carry the softmax scale (and log2 e) from here on, rounded to bf16 like the reference's scaled
    // queries: the matrix pipe then delivers the scores in log2 units.
    const float qscale = p.scale_log2;
#pragma unroll
    for (int s = 0; s < KSTEPS; ++s) {
      const u32x4 w = *reinterpret_cast<const u32x4*>(qr + 16 * s);
      u32x4 r;
#pragma unroll
      for (int j = 0; j < 4; ++j)
        r[j] = pack_bf16x2(__uint_as_float(w[j] << 16) * qscale, __uint_as_float(w[j] & 0xffff0000u) * qscale);
      QB[s] = __builtin_bit_cast(bf16x8, r);
    }
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
  constexpr int NSETS = 1;
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

  const int n_diag = (min(len, tile_start + QTILE) - dstart + 63) >> 6;  // chunks from dstart to the end of the tile, >= 1
  // Only a sequence's last tile can hold chunks that reach past its end (or a block so large that there are more such
  // chunks than a lane mask holds): it takes the plain loop further down.
  const bool ragged_tile = dstart + 64 * n_diag > len || n_diag > 63;
  const int my_blk = (int)((unsigned)q0 / (unsigned)Bs);
  bool dma_done = false;
  if constexpr (SPLIT) {
    if (!ragged_tile) {
      // ================= 8 waves, full tile: two wave groups half a chunk apart ===================================
      // Waves w and w+4 share a SIMD.  Every wave runs, per chunk `it`:  softmax(it) | PV(it) | QK(it+1).  Waves 0-3
      // ("early") meet the workgroup barrier at the end of that body, waves 4-7 ("late") in its middle, after softmax:
      // between two barriers one wave of a SIMD does softmax, PV, QK and the other PV, QK, softmax, so the vector work of
      // one meets the matrix work of the other.  Call sync(k) the barrier that ends the early group's body k.  Then
      // keys of chunk c are read in (sync(c-2), sync(c)) and its values in (sync(c-1), sync(c+1)).
      //  * K(c) lives in ring buffer c % 4.  The early waves request K(k+4) by DMA right after sync(k): the buffer it
      //    overwrites, K(k), was last read before sync(k); it must have landed when they arrive at sync(k+2), so their
      //    wait before a barrier leaves exactly the newest request in flight.
      //  * V(c) first lands row-major ("raw", buffer c % 2), also by DMA from the early waves: V(k+3) is requested right
      //    after sync(k), ahead of K(k+4), and must have landed when they arrive at sync(k+1).  The late waves then
      //    transpose it from LDS to LDS into ring buffer c % 3: V(k+2) is stored
      //    after sync(k), into the buffer of V(k-1), last read before sync(k), and is visible from sync(k+1) on.
      constexpr int KRING = 4, KTILE = 64 * DK * 2, VRING = 3, VTILE = DV * VTP * 2, RTILE = 64 * DV * 2;   // bytes
      constexpr int KI = DK / 32, RI = DV / 32;                                          // DMA instructions per early wave and chunk
      constexpr int KROWS_I = 512 / DK, RROWS_I = 512 / DV;                              // tile rows one instruction covers
      // (the swizzled operand addresses are formed with XOR: the ring starts on a 1 KiB boundary)
      const unsigned lds_k = ((unsigned)(size_t)smem + 1023u) & ~1023u, lds_r = lds_k + KRING * KTILE, lds_v = lds_r + 2 * RTILE;
      const bool late = wave >= 4;
      const int gw = wave & 3;  // wave within its group
      // --- early waves: lane l of instruction i fills LDS row KROWS_I*i + l/segs, position l%segs, with the segment that belongs there
      unsigned k_src[KI];
#pragma unroll
      for (int j = 0; j < KI; ++j) {
        const int r = KROWS_I * (KI * gw + j) + lane / (DK / 8), pos = lane % (DK / 8);
        k_src[j] = (unsigned)((size_t)r * krow * sizeof(bf16_t)) + 16u * (pos ^ (DK == 128 ? (r & 15) : ((r >> 1) & 7)));
      }
      // raw V: segment s of row r sits at s ^ ((r >> 2) & 15), so that the 16 lanes of a transposing thread group (16
      // key groups = rows 4 apart, one segment) read 16 different 16-byte slots
      unsigned r_src[RI];
#pragma unroll
      for (int j = 0; j < RI; ++j) {
        const int r = RROWS_I * (RI * gw + j) + lane / (DV / 8), pos = lane % (DV / 8);
        r_src[j] = (unsigned)((size_t)r * vrow * sizeof(bf16_t)) + 16u * (pos ^ ((r >> 2) & (DV / 8 - 1)));
      }
      auto dma_r = [&](const int ks, const int c) __attribute__((always_inline)) {
        const char* g = reinterpret_cast<const char*>(vp + (size_t)ks * vrow);
#pragma unroll
        for (int j = 0; j < RI; ++j) dma16(g, r_src[j], lds_r + (c & 1) * RTILE + (RI * gw + j) * 1024);
      };
      auto dma_k = [&](const int ks, const int c) __attribute__((always_inline)) {
        const char* g = reinterpret_cast<const char*>(kp + (size_t)ks * krow);
#pragma unroll
        for (int j = 0; j < KI; ++j) dma16(g, k_src[j], lds_k + (c & 3) * KTILE + (KI * gw + j) * 1024);
      };
      // --- late waves: a thread owns keys 4 kg .. 4 kg + 3 of one 8-column segment.  16 consecutive lanes take the 16
      // key groups of one segment: their transposed 8-byte stores fill one 128-byte row, the next 16 lanes' row lies
      // 8 rows = 1152 bytes further, on the other half of the banks.
      const int lt = tid & 255;
      const int v_kg = lt & 15, v_sg = lt >> 4;
      const bool v_on = v_sg < DV / 8;   // (DV = 64: half of the late waves have nothing to stage)
      // raw tile: rows 4 kg .. 4 kg + 3, segment sg (swizzled)
      const unsigned v_raw = (unsigned)(4 * v_kg * DV * 2) + 16u * ((v_on ? v_sg : 0) ^ (v_kg & (DV / 8 - 1)));
      // keys 4 kg .. 4 kg + 3 sit at position 4 * slot of their 16-key group, slot = 2 (q & 1) + (q >> 1), q = kg % 4:
      // a lane of half hf then finds its k-slots (keys 4 hf .. +3 and 8 + 4 hf .. +3 of the group) in bytes 16 hf .. 16 hf + 15
      const unsigned v_dst = (unsigned)(8 * v_sg * VTP * 2) + 32u * (v_kg >> 2) + 8u * (2 * (v_kg & 1) + ((v_kg >> 1) & 1));
      auto transpose_v = [&](const int c) __attribute__((always_inline)) {
        if (v_on) {
          typedef __attribute__((address_space(3))) const u32x4* lds_r4;
          typedef __attribute__((address_space(3))) u32x2* lds_w;
          unsigned src = lds_r + (c & 1) * RTILE + v_raw;
          asm("" : "+v"(src));
          u32x4 rv[4];
#pragma unroll
          for (int j = 0; j < 4; ++j) rv[j] = *reinterpret_cast<lds_r4>(src + j * DV * 2);
          const unsigned a = lds_v + (c % VRING) * VTILE + v_dst;
#pragma unroll
          for (int d = 0; d < 4; ++d) {
            // value columns 2d (low halves) and 2d+1 (high halves) of the four keys
            u32x2 lo, hi;
            lo[0] = __builtin_amdgcn_perm(rv[1][d], rv[0][d], 0x05040100u);
            lo[1] = __builtin_amdgcn_perm(rv[3][d], rv[2][d], 0x05040100u);
            hi[0] = __builtin_amdgcn_perm(rv[1][d], rv[0][d], 0x07060302u);
            hi[1] = __builtin_amdgcn_perm(rv[3][d], rv[2][d], 0x07060302u);
            *reinterpret_cast<lds_w>(a + (2 * d) * VTP * 2) = lo;
            *reinterpret_cast<lds_w>(a + (2 * d + 1) * VTP * 2) = hi;
          }
        }
      };
      // operand addresses of this lane inside a tile (see qk_phase / pv_phase)
      const unsigned k_lane = (unsigned)(l32 * DK * 2) + 16u * (hf ^ (DK == 128 ? (l32 & 15) : ((l32 >> 1) & 7)));
      const unsigned v_lane = (unsigned)(l32 * VTP * 2) + 16u * hf;

      // The first four chunks are requested before anything else when their addresses need no block list (the usual
      // case: four or more chunks from dstart on).
      // Request order of the early waves: K(0), V(0), K(1), V(1); K(2) after the first barrier; V(2), K(3) after the second.
      const bool early_request = n_diag >= 4;
      if (early_request && !late) {
        dma_k(dstart, 0);
        dma_r(dstart, 0);
        dma_k(dstart + 64, 1);
        dma_r(dstart + 64, 1);
      }
      // types of the blocks the chunks from dstart on fall into, as a bit mask (bit i = block dstart/Bs + i)
      unsigned long long diag_attn;
      {
        const int blk = dblk + lane;
        const bool in_range = lane < n_diag && (size_t)blk * Bs < (size_t)min(len, tile_start + QTILE);
        diag_attn = __ballot(in_range && type_is_one(p.types, p.types_dtype, ((size_t)(bos_nats + blk) * p.HN + hn) * 2));
      }
      // attention blocks that end at or before dstart: ids into LDS.  The list is sorted and holds distinct block ids
      // (entry j >= j), so only the first dstart/Bs entries can qualify, and those that do form a prefix.
      __shared__ int wave_count[NWAVES];
      {
        const int jmax = min(dblk, p.TN);
        const int n_attn = *n_attn_p;
        int cnt = 0;
        for (int j = tid; j < jmax; j += NTHREADS) {
          const int e = list[j * list_stride];
          const bool ok = j < n_attn && (e + 1) * Bs <= dstart;
          cnt += __popcll(__ballot(ok));
          if (ok && j < MAX_LDS_LIST) lds_list[j] = e;
        }
        if (lane == 0) wave_count[wave] = cnt;
      }
      __syncthreads();
      int n_prior = 0;
#pragma unroll
      for (int w2 = 0; w2 < NWAVES; ++w2) n_prior += wave_count[w2];
      n_prior = __builtin_amdgcn_readfirstlane(n_prior);
      const int n_iters = n_diag + n_prior * per_blk;

      // chunk iterator (wave-uniform): first key of chunk nx_it, then on to the next; past the last chunk it repeats it
      int nx_it = 0, nx_j = 0, nx_sub = 0, ks_cur = dstart;
      // (in the loop the list entry is read from LDS at the top of the body, `ahead`, and used at its end: the
      // iterator only moves in between)
      auto list_ahead = [&]() -> int { return lds_list[min(nx_j, MAX_LDS_LIST - 1)]; };
      auto next_chunk = [&](const int ahead = 0, const bool have_ahead = false) __attribute__((always_inline)) -> int {
        if (nx_it < n_iters) {
          if (nx_it < n_diag) {
            ks_cur = dstart + nx_it * 64;
          } else {
            int e;
            if (nx_j < MAX_LDS_LIST) e = __builtin_amdgcn_readfirstlane(have_ahead ? ahead : lds_list[nx_j]);
            else e = __builtin_amdgcn_readfirstlane(list[nx_j * list_stride]);
            ks_cur = e * Bs + nx_sub * 64;
            if (++nx_sub == per_blk) {
              nx_sub = 0;
              ++nx_j;
            }
          }
        }
        ++nx_it;
        return ks_cur;
      };
      int ks_v = dstart;   // first key of the chunk whose raw V is requested next (one chunk behind the K requests)
      if (!late) {
        if (early_request) {
          nx_it = 2;
        } else {
          int ks = next_chunk();
          dma_k(ks, 0);
          dma_r(ks, 0);
          ks = next_chunk();
          if (1 < n_iters) {
            dma_k(ks, 1);
            dma_r(ks, 1);
          }
        }
        // raw V(0), V(1) (and K(0), K(1)) must have landed for the transposition below
        __builtin_amdgcn_s_waitcnt(0x0f70);
      }
      __syncthreads();
      if (!late) {
        ks_v = next_chunk();                      // chunk 2
        if (2 < n_iters) dma_k(ks_v, 2);
      } else {
        transpose_v(0);
        if (1 < n_iters) transpose_v(1);
      }
      __syncthreads();                            // "sync(-1)"
      if (!late) {
        // raw V(2) only now: its buffer held raw V(0) until the barrier.  Like every later request pair it is followed
        // by the K request that may stay in flight at the next barrier.
        if (2 < n_iters) dma_r(ks_v, 2);
        ks_v = next_chunk();                      // chunk 3
        if (3 < n_iters) dma_k(ks_v, 3);
      }

      // which of the chunks from dstart on this wave takes part in (bit it), and which one is its own, causal chunk:
      // lane i works it out for chunk i, once
      unsigned long long act_mask;
      int causal_it;
      {
        const int jc = (dstart >> 6) + lane;  // absolute chunk index of the keys
        const int kblk = (int)((unsigned)(jc * 64) / (unsigned)Bs);
        const bool typed = (diag_attn >> ((kblk - dblk) & 63)) & 1ull;
        bool a, cz = false;
        if (p.same_block) {
          cz = jc == my_chunk;
          a = cz || (jc < my_chunk && (kblk == my_blk || typed));
        } else {
          a = jc < my_chunk && kblk < my_blk && typed;
        }
        act_mask = __ballot(a && lane < n_diag);
        const unsigned long long cm = __ballot(cz && lane < n_diag);
        causal_it = cm ? __builtin_ctzll(cm) : -1;
      }
      m_ref = 0.f;       // an arbitrary finite reference until the row's first visible key sets the real one
      float thr = -INFINITY;
      f32x16 s0, s1;
      bool cur_active = act_mask & 1ull;
      if (cur_active) qk_phase<DK>(lds_k + k_lane, QB, m_ref, s0, s1);
      auto is_active = [&](const int it) -> bool { return it < n_diag ? (act_mask >> it) & 1ull : it < n_iters; };

      if (!late) {
        for (int it = 0; it < n_iters; ++it) {
          const bool nxt_active = is_active(it + 1);
          const int ahead = list_ahead();
          bf16x8 PB[4];
          if (cur_active) {
            softmax_phase<DV>(s0, s1, acc, m_ref, l_run, thr, lane, it == causal_it, qloc0, PB);
            __builtin_amdgcn_s_setprio(3);
            pv_phase<DV>(lds_v + (it % VRING) * VTILE + v_lane, PB, acc, l_run);
          }
          __builtin_amdgcn_s_setprio(3);
          if (nxt_active) qk_phase<DK>(lds_k + ((it + 1) & 3) * KTILE + k_lane, QB, m_ref, s0, s1);
          __builtin_amdgcn_s_setprio(0);
          // K(it+2) and raw V(it+2) must have landed; the request for K(it+3), the newest, may stay in flight if there is one
          if (it + 3 < n_iters) __builtin_amdgcn_s_waitcnt(0x0f70 | KI);
          else __builtin_amdgcn_s_waitcnt(0x0f70);
          __syncthreads();                                  // sync(it)
          if (it + 3 < n_iters) dma_r(ks_v, it + 3);        // raw V first: it has one interval to land, K has two
          ks_v = next_chunk(ahead, true);
          if (it + 4 < n_iters) dma_k(ks_v, it + 4);
          cur_active = nxt_active;
        }
      } else {
        for (int it = 0; it < n_iters; ++it) {
          const bool nxt_active = is_active(it + 1);
          bf16x8 PB[4];
          if (cur_active) softmax_phase<DV>(s0, s1, acc, m_ref, l_run, thr, lane, it == causal_it, qloc0, PB);
#pragma unroll
          for (int i = 0; i < 4; ++i) asm volatile("" : "+v"(PB[i]));   // the probabilities exist before the barrier
          __syncthreads();                                  // sync(it)
          __builtin_amdgcn_s_setprio(3);
          if (cur_active) pv_phase<DV>(lds_v + (it % VRING) * VTILE + v_lane, PB, acc, l_run);
          if (nxt_active) qk_phase<DK>(lds_k + ((it + 1) & 3) * KTILE + k_lane, QB, m_ref, s0, s1);
          __builtin_amdgcn_s_setprio(0);
          // the matrix phases come first, while the early waves are in their vector phase; the transposition follows
          if (it + 2 < n_iters) transpose_v(it + 2);
          cur_active = nxt_active;
        }
      }
      __builtin_amdgcn_s_waitcnt(0x0f70);
      __syncthreads();  // the late waves finish their last PV after the early ones: the output tile below reuses the rings
      dma_done = true;
    }
  }
  if (!dma_done) {
    // ---- prologue: everything the tile needs first is requested at once -----------------------
    // The chunks from dstart on (same-block / causal rules) come FIRST: their addresses need no
    // routing table, so their loads, the Q loads above and the reads of the block list are all in
    // flight together.  The chunks of the prior attention blocks follow.
    if (ragged_tile) {
      gload(std::false_type{}, dstart, sreg[0]);
    } else {
      gload(std::true_type{}, dstart, sreg[0]);
    }
    if (tid == 0) lds_count = 0;
    __syncthreads();
    {
      // attention blocks that end at or before dstart: ids into LDS, count.  The list is sorted and
      // holds distinct block ids, so entry j >= j: only the first dstart/Bs entries can qualify.
      const int jmax = min(dblk, p.TN);
      const int n_attn = *n_attn_p;
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
      const int blk = dblk + lane;
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

    constexpr float c = 1.f;  // the scale is already in the queries
    // one chunk for this wave: the chunks from dstart on follow the same-block and causal rules, the prior attention
    // blocks are seen whole
    auto compute = [&](const int it, const int buf) __attribute__((always_inline)) {
      bool active = wave_valid, causal = false;
      if (it < n_diag) {
        const int jc = (dstart >> 6) + it;  // absolute chunk index of the keys
        const int kblk = (int)((unsigned)(jc * 64) / (unsigned)Bs);
        if (p.same_block) {
          if (jc > my_chunk) active = false;
          else if (jc == my_chunk) causal = true;
          else active = active && (kblk == my_blk || ((diag_attn >> (kblk - dblk)) & 1ull));
        } else {
          active = active && jc < my_chunk && kblk < my_blk && ((diag_attn >> (kblk - dblk)) & 1ull);
        }
      }
      if (active)
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

// =====================================================================================================================
// The 8-wave schedule as a persistent kernel: one workgroup per CU works through 256-query tiles that it takes from
// work queues, and the K/V rings never drain between two tiles.
//
// What a workgroup of the kernel above pays per tile besides its chunk loop (cycle counters, 19 chunks per tile on
// average): ~5 500 cycles until the CU has been given its next workgroup, ~14 000 of prologue (kernel arguments, index
// arithmetic, the queries, the block types and the block list, the first keys and values: four dependent round trips
// to memory, two barriers, the first transposition) and ~3 800 of epilogue, against ~58 000 in the loop.  Here
//  * the memory side is ONE stream of chunks across tiles.  Chunk c of a tile with n chunks has stream position sp0 + c,
//    the next tile's chunk j has sp0 + n + j, and every ring slot is chosen by stream position.  The rules of the loop
//    (after barrier k: request raw V(k+3), then K(k+4); the late waves transpose V(k+2)) simply run on into the next
//    tile, whose first chunks need no block list: when a tile's loop ends, K(0..3) and V(0..2) of the next tile are on
//    their way or already there, and V(0), V(1) are transposed;
//  * the compute side makes a clean cut between tiles: output straight from the accumulators (no LDS), then one barrier
//    that hands over what the late waves prepared for the new tile while the old one was running (its block types, its
//    list of prior attention blocks in LDS, how many there are, and which tile comes after it), then QK(0);
//  * the queries of the next tile are requested before the output code and used after it;
//  * the kernel starts with a "virtual" tile of four chunks in which no wave has anything to compute: its loop is what
//    fills the rings for the first real tile, so there is no separate prologue.
// Tiles come from eight queues, one per XCD (a workgroup reads which XCD it runs on): queue x lists the tiles of
// (batch, head) pairs x, x+8, ... pair after pair, heaviest tile first, so the tiles that share a pair's K/V run
// together on one L2; a workgroup whose queue is used up takes from the others.  A queue is a ticket counter in device
// memory, zeroed on the launch's stream by a small fill kernel right before the launch (see launch_softmax_stream).
constexpr int STREAM_ROWS = 1088;  // chunk table of a tile: up to 1024 + 32 chunks of its own and four of the next tile (two tiles' tables are resident)
constexpr int STREAM_QUEUES = 8;
constexpr int STREAM_SLOT_WORDS = 16;  // per launch slot: 8 ticket counters (one per XCD), the rest unused padding to a 64-byte line

struct StreamTile {
  int valid, n, hq, tile, hkv, hn, dstart, dblk;  // the tile AFTER the one this record belongs to
  unsigned diag_lo, diag_hi;                      // this tile: which of the blocks from dstart on are typed attention
  int count[4];                                   // this tile: prior attention blocks found by each late wave
  int pad[2];
};

NATSL_DEVICE unsigned xcc_id() {
  unsigned x;
  asm volatile("s_getreg_b32 %0, hwreg(HW_REG_XCC_ID)" : "=s"(x));
  return x & (STREAM_QUEUES - 1);
}

template <int DK, int DV>
__global__ __launch_bounds__(512, 1) __attribute__((amdgpu_waves_per_eu(2, 2)))
void softmax_stream_kernel(const SoftmaxParams p, unsigned* queue) {
  constexpr int QW = 32, QTILE = 256, KSTEPS = DK / 16, VT = DV / 32;
  constexpr int KTILE = 64 * DK * 2, VRING = 3, VTILE = DV * VTP * 2, RTILE = 64 * DV * 2;  // bytes
  constexpr int KI = DK / 32, RI = DV / 32, KROWS_I = 512 / DK, RROWS_I = 512 / DV;
  extern __shared__ __align__(16) unsigned char smem[];
  __shared__ int rows[2][STREAM_ROWS];
  __shared__ __align__(16) StreamTile info[2];

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int l32 = lane & 31, hf = lane >> 5;
  const bool late = wave >= 4;
  const int gw = wave & 3;
  const int Bs = p.block, per_blk = Bs >> 6;
  const unsigned NT = (unsigned)p.T / QTILE;
  const unsigned n_pairs = (unsigned)(p.B * p.HQ);
  const size_t krow = (size_t)p.HKV * DK, vrow = (size_t)p.HKV * DV;
  const size_t list_stride = (size_t)p.HN * 2;
  constexpr int K_SHIFT = DK == 128 ? 8 : 7, V_SHIFT = DV == 128 ? 8 : 7;  // log2 of a K / V row in bytes
  const unsigned lds_k = ((unsigned)(size_t)smem + 1023u) & ~1023u, lds_r = lds_k + 4 * KTILE, lds_v = lds_r + 2 * RTILE;

  // ---- lane constants of the data movement (as in the kernel above) ----------------------------------------------
  // Source offsets of the DMA instructions: lane l of instruction j fills LDS row rows_per_instr * j + l / segs, position
  // l % segs, with the segment that the swizzle puts there.  A chunk is named by the row index of its first key in the
  // [B*T*HKV] row space of K and V, (token * HKV + kv head): its address is the tensor base plus that index shifted.
  unsigned k_src[KI], r_src[RI];
#pragma unroll
  for (int j = 0; j < KI; ++j) {
    const int r = KROWS_I * (KI * gw + j) + lane / (DK / 8), pos = lane % (DK / 8);
    k_src[j] = (unsigned)((size_t)r * krow * sizeof(bf16_t)) + 16u * (pos ^ (DK == 128 ? (r & 15) : ((r >> 1) & 7)));
  }
#pragma unroll
  for (int j = 0; j < RI; ++j) {
    const int r = RROWS_I * (RI * gw + j) + lane / (DV / 8), pos = lane % (DV / 8);
    r_src[j] = (unsigned)((size_t)r * vrow * sizeof(bf16_t)) + 16u * (pos ^ ((r >> 2) & (DV / 8 - 1)));
  }
  auto dma_r = [&](const int row, const unsigned sp) __attribute__((always_inline)) {
    const char* g = reinterpret_cast<const char*>(p.v) + ((size_t)(unsigned)row << V_SHIFT);
    const unsigned l0 = lds_r + (sp & 1) * RTILE + RI * gw * 1024;
#pragma unroll
    for (int j = 0; j < RI; ++j) dma16(g, r_src[j], l0 + j * 1024);
  };
  auto dma_k = [&](const int row, const unsigned sp) __attribute__((always_inline)) {
    const char* g = reinterpret_cast<const char*>(p.k) + ((size_t)(unsigned)row << K_SHIFT);
    const unsigned l0 = lds_k + (sp & 3) * KTILE + KI * gw * 1024;
#pragma unroll
    for (int j = 0; j < KI; ++j) dma16(g, k_src[j], l0 + j * 1024);
  };
  const int lt = tid & 255;
  const int v_kg = lt & 15, v_sg = lt >> 4;
  const bool v_on = v_sg < DV / 8;
  const unsigned v_raw = (unsigned)(4 * v_kg * DV * 2) + 16u * ((v_on ? v_sg : 0) ^ (v_kg & (DV / 8 - 1)));
  const unsigned v_dst = (unsigned)(8 * v_sg * VTP * 2) + 32u * (v_kg >> 2) + 8u * (2 * (v_kg & 1) + ((v_kg >> 1) & 1));
  auto transpose_v = [&](const unsigned sp) __attribute__((always_inline)) {
    if (v_on) {
      typedef __attribute__((address_space(3))) const u32x4* lds_r4;
      typedef __attribute__((address_space(3))) u32x2* lds_w;
      unsigned src = lds_r + (sp & 1) * RTILE + v_raw;
      asm("" : "+v"(src));
      u32x4 rv[4];
#pragma unroll
      for (int j = 0; j < 4; ++j) rv[j] = *reinterpret_cast<lds_r4>(src + j * DV * 2);
      const unsigned a = lds_v + (sp % VRING) * VTILE + v_dst;
#pragma unroll
      for (int d = 0; d < 4; ++d) {
        u32x2 lo, hi;
        lo[0] = __builtin_amdgcn_perm(rv[1][d], rv[0][d], 0x05040100u);
        lo[1] = __builtin_amdgcn_perm(rv[3][d], rv[2][d], 0x05040100u);
        hi[0] = __builtin_amdgcn_perm(rv[1][d], rv[0][d], 0x07060302u);
        hi[1] = __builtin_amdgcn_perm(rv[3][d], rv[2][d], 0x07060302u);
        *reinterpret_cast<lds_w>(a + (2 * d) * VTP * 2) = lo;
        *reinterpret_cast<lds_w>(a + (2 * d + 1) * VTP * 2) = hi;
      }
    }
  };
  const unsigned k_lane = (unsigned)(l32 * DK * 2) + 16u * (hf ^ (DK == 128 ? (l32 & 15) : ((l32 >> 1) & 7)));
  const unsigned v_lane = (unsigned)(l32 * VTP * 2) + 16u * hf;

  // ---- work queues (wave 4 only) -----------------------------------------------------------------------------------
  const unsigned xcc = xcc_id();
  int cq = 0;  // queues used up so far; the queue in use is (xcc + cq) & 7
  unsigned t_ahead = 0;
  auto queue_units = [&](const unsigned qx) -> unsigned { return qx < n_pairs ? ((n_pairs - qx + 7u) / 8u) * NT : 0u; };
  auto take_ticket = [&]() -> unsigned {
    unsigned t = 0;
    if (lane == 0) t = atomicAdd(&queue[(xcc + (unsigned)cq) & 7u], 1u);
    return __builtin_amdgcn_readfirstlane(t);
  };
  // ticket t of the queue in use -> the tile it stands for, written as the "next tile" part of a record; moves on to the
  // other queues (one synchronous ticket each) when the queue in use has no tiles left.  Returns the row index of the
  // tile's first chunk (-1: no tile left).
  auto resolve_ticket = [&](unsigned t, StreamTile* out) -> int {
    bool ok = false;
    unsigned qx = 0;
    while (cq < STREAM_QUEUES) {
      qx = (xcc + (unsigned)cq) & 7u;
      if (t < queue_units(qx)) {
        ok = true;
        break;
      }
      if (++cq < STREAM_QUEUES) t = take_ticket();
    }
    if (!ok) {
      if (lane == 0) out->valid = 0;
      return -1;
    }
    // Order of a queue: first every pair's NT - NL late (long) tiles, pair after pair, latest tile first; then every
    // pair's NL early (short) tiles the same way.  With the pairs' tiles simply one after the other, the last pair's
    // longest tile would start when only that pair's tiles are left, and the other CUs of the XCD idle while it runs.
    const unsigned NL = NT / 3u, NH = NT - NL, heavy = (queue_units(qx) / NT) * NH;
    unsigned pidx, tile;
    if (t < heavy) {
      pidx = t / NH;
      tile = NT - 1u - t % NH;
    } else {
      pidx = (t - heavy) / NL;   // (NL > 0 here: with NL = 0 every ticket is below `heavy`)
      tile = NL - 1u - (t - heavy) % NL;
    }
    const unsigned pair = pidx * 8u + qx;
    const unsigned n = pair / (unsigned)p.HQ, hq = pair - n * (unsigned)p.HQ;
    const unsigned dstart = (tile * QTILE / (unsigned)Bs) * (unsigned)Bs;
    const unsigned hkv = hq / (unsigned)p.g_kv;
    if (lane == 0) {
      out->valid = 1;
      out->n = (int)n;
      out->hq = (int)hq;
      out->tile = (int)tile;
      out->hkv = (int)hkv;
      out->hn = (int)(hq / (unsigned)p.g_n);
      out->dstart = (int)dstart;
      out->dblk = (int)(dstart / (unsigned)Bs);
    }
    return (int)((n * (unsigned)p.T + dstart) * (unsigned)p.HKV + hkv);
  };

  // ---- state of the tile in work; the kernel starts in a virtual tile (four chunks, nothing to compute) ------------
  int a = 0;          // which record / list buffer belongs to the tile in work
  unsigned sp0 = 0;   // stream position of its chunk 0
  bool cur_real = false;
  int c_n = 0, c_hq = 0, c_tile = 0, c_hkv = 0, c_hn = 0, dstart = 0, dblk = 0;
  bool k_req = false;  // the early waves' newest request is a K request that may still be in flight at the next barrier
  int row_v = 0;       // early waves: row index of the chunk whose K was requested last (its V is requested next)
  if (wave == 4) {
    const int r0 = resolve_ticket(take_ticket(), &info[0]);
    if (lane == 0) {
      info[0].diag_lo = info[0].diag_hi = 0u;
      info[0].count[0] = info[0].count[1] = info[0].count[2] = info[0].count[3] = 0;
    }
    if (r0 >= 0 && lane < 4) rows[0][4 + lane] = r0 + 64 * lane * p.HKV;   // the virtual tile has four chunks of its own
  }

  bf16x8 QB[KSTEPS];
#pragma unroll
  for (int s = 0; s < KSTEPS; ++s) QB[s] = bf16x8{};
  f32x16 acc[VT];
  float m_ref, l_run, thr;

  // ---- a tile's output.  A lane holds, of its query, value columns 8 rg + 4 hf .. + 3 of every 32-column tile: stored
  // from there, an instruction would touch 64 separate 16-byte pieces.  The rows go through LDS instead, half of the
  // columns at a time (a wave's 32 rows x DV/2 columns; 16-byte segments XOR-swizzled by the row), and leave as whole
  // lines.  The space is a raw V buffer, a quarter of it per wave.  The early waves use, right after their last chunk,
  // the buffer whose next request (the next tile's chunk 2) they hold back until they are done: a wave's requests go
  // to the same quarter as its rows, so no barrier is needed.  The late waves use the other buffer, whose contents (the
  // next tile's chunk 1) all of them have transposed once the hand-over barrier of the next tile is behind them: they
  // store there, before anything of the new tile touches the accumulators.  row0: flat (token, head) index of the
  // wave's first query.
  auto store_tile = [&](const unsigned stage, const size_t row0) __attribute__((always_inline)) {
    constexpr int PW = DV / 2, RB = PW * 2, NSEG = RB / 16, RPI = 64 / NSEG;   // columns per pass, row bytes, segments, rows per instruction
    typedef __attribute__((address_space(3))) u32x2* lds_w8;
    typedef __attribute__((address_space(3))) const u32x4* lds_r16;
    const float l_tot = xhalf_sum(l_run);
    const bool has = l_tot > 0.f;
    const float inv = has ? 1.f / l_tot : 0.f;
    int ol = lane;
    asm volatile("" : "+v"(ol));   // (the lane's share of the addresses below is not to be kept through the chunk loops)
    const int ol32 = ol & 31, ohf = ol >> 5;
    if (ohf == 0) p.lse[row0 + (size_t)ol32 * p.HQ] = has ? m_ref + __builtin_amdgcn_logf(l_tot) : 0.f;
    const unsigned wbase = stage + (unsigned)(ol32 * RB + 8 * ohf);
    const int rrow = ol / NSEG, rseg = ol % NSEG;
#pragma unroll
    for (int ps = 0; ps < 2; ++ps) {
#pragma unroll
      for (int vl = 0; vl < VT / 2; ++vl) {
        const int vt = ps * (VT / 2) + vl;
#pragma unroll
        for (int rg = 0; rg < 4; ++rg) {
          u32x2 w;
          w[0] = pack_bf16x2(acc[vt][4 * rg] * inv, acc[vt][4 * rg + 1] * inv);
          w[1] = pack_bf16x2(acc[vt][4 * rg + 2] * inv, acc[vt][4 * rg + 3] * inv);
          *reinterpret_cast<lds_w8>(wbase + 16u * ((unsigned)(4 * vl + rg) ^ (unsigned)(ol32 & (NSEG - 1)))) = w;
        }
      }
      __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0): this wave's rows are in LDS
      __builtin_amdgcn_wave_barrier();
#pragma unroll
      for (int i = 0; i < 32 / RPI; ++i) {
        const int row = i * RPI + rrow;
        const u32x4 w = *reinterpret_cast<lds_r16>(stage + (unsigned)(row * RB) + 16u * ((unsigned)rseg ^ (unsigned)(row & (NSEG - 1))));
        *reinterpret_cast<u32x4*>(p.o + (row0 + (size_t)row * p.HQ) * DV + ps * PW + rseg * 8) = w;
      }
      if (ps == 0) {
        __builtin_amdgcn_s_waitcnt(0xc07f);  // the rows have been read before the second half overwrites them
        __builtin_amdgcn_wave_barrier();
      }
    }
  };
  auto scale_next_q = [&]() __attribute__((always_inline)) {
    const float qscale = p.scale_log2;
#pragma unroll
    for (int s = 0; s < KSTEPS; ++s) {
      const u32x4 w = __builtin_bit_cast(u32x4, QB[s]);
      u32x4 r;
#pragma unroll
      for (int j = 0; j < 4; ++j)
        r[j] = pack_bf16x2(__uint_as_float(w[j] << 16) * qscale, __uint_as_float(w[j] & 0xffff0000u) * qscale);
      QB[s] = __builtin_bit_cast(bf16x8, r);
    }
  };
  bool pend_store = false;   // late waves: the previous tile's output is still in the accumulators
  unsigned pend_stage = 0;
  size_t pend_row0 = 0;

  for (;;) {
    // ---- hand-over barrier: the record and the list of the tile in work are complete ------------------------------
    __syncthreads();
    typedef __attribute__((address_space(3))) const int* lds_i;
    const unsigned rec = (unsigned)(size_t)&info[a];
    auto rd = [&](const int i) -> int { return __builtin_amdgcn_readfirstlane(*reinterpret_cast<lds_i>(rec + 4u * i)); };
    // (one 4-byte read per field: a wider uniform read followed by readfirstlane of its elements was folded into
    // element 0 by the compiler)
    const bool n_valid = rd(0) != 0;
    const int n_n = rd(1), n_hq = rd(2), n_tile = rd(3), n_hkv = rd(4), n_hn = rd(5), n_dstart = rd(6), n_dblk = rd(7);
    const unsigned long long diag_attn = (unsigned long long)(unsigned)rd(8) | ((unsigned long long)(unsigned)rd(9) << 32);
    const int n_prior = rd(10) + rd(11) + rd(12) + rd(13);
    const int tile_start = c_tile * QTILE;
    const int n_diag = cur_real ? (tile_start + QTILE - dstart) >> 6 : 4;
    const int n_iters = n_diag + n_prior * per_blk;
    const int bos = c_n * p.T;
    const int q0 = tile_start + wave * QW;
    const int my_chunk = q0 >> 6, qloc0 = q0 & 63;
    const int my_blk = (int)((unsigned)q0 / (unsigned)Bs);
    // the tile after this one
    const int n_bos = n_n * p.T;
    const int n_tile_start = n_tile * QTILE;

    // queries of the next tile: raw into the query registers (issued during this tile's last chunk), scaled in place
    auto load_next_q = [&]() __attribute__((always_inline)) {
      // (lane ids made opaque here and in the output code below: otherwise the lane's share of every such address is
      // computed once per kernel and kept in registers through the chunk loops)
      int ql = lane;
      asm volatile("" : "+v"(ql));
      // (no next tile: this tile's rows are read again, so that the loads and the waits of the scaling below are on
      // every path -- with the loads under a condition the compiler assumes them pending wherever the queries are used)
      const size_t qrow = n_valid ? (size_t)(n_bos + n_tile_start) : (size_t)(bos + tile_start);
      const bf16_t* qr = p.q + ((qrow + wave * QW + (ql & 31)) * p.HQ + (n_valid ? n_hq : c_hq)) * DK + 8 * (ql >> 5);
#pragma unroll
      for (int s = 0; s < KSTEPS; ++s) QB[s] = __builtin_bit_cast(bf16x8, *reinterpret_cast<const u32x4*>(qr + 16 * s));
    };

    if (pend_store) store_tile(pend_stage, pend_row0);
    scale_next_q();   // the queries requested at the end of the previous tile

    // which of the chunks from dstart on this wave takes part in, and which one is its own, causal chunk
    unsigned long long act_mask = 0;
    int causal_it = -1;
    if (cur_real) {
      int al = lane;
      asm volatile("" : "+v"(al));
      const int jc = (dstart >> 6) + al;
      const int kblk = (int)((unsigned)(jc * 64) / (unsigned)Bs);
      const bool typed = (diag_attn >> ((kblk - dblk) & 63)) & 1ull;
      bool act, cz = false;
      if (p.same_block) {
        cz = jc == my_chunk;
        act = cz || (jc < my_chunk && (kblk == my_blk || typed));
      } else {
        act = jc < my_chunk && kblk < my_blk && typed;
      }
      act_mask = __ballot(act && al < n_diag);
      const unsigned long long cm = __ballot(cz && al < n_diag);
      causal_it = cm ? __builtin_ctzll(cm) : -1;
    }
#pragma unroll
    for (int vt = 0; vt < VT; ++vt)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[vt][r] = 0.f;
    m_ref = 0.f;  // an arbitrary finite reference until the row's first visible key sets the real one
    l_run = 0.f;
    thr = -INFINITY;
    f32x16 s0, s1;
    auto is_active = [&](const int it) -> bool { return it < n_diag ? (act_mask >> it) & 1ull : it < n_iters; };
    bool cur_active = act_mask & 1ull;
    if (cur_active) qk_phase<DK>(lds_k + (sp0 & 3) * KTILE + k_lane, QB, m_ref, s0, s1);

    if (!late) {
      // Stream chunks requested during this tile: its own from chunk 4 on (chunks 0..3 were requested while the previous
      // tile ran) and the next tile's first four, all by their entry in this tile's chunk table.
      // (the V request of the last iteration, the next tile's chunk 2, waits until the output code below is done with
      // the buffer it goes to)
      const int rq_lo = cur_real ? 0 : n_iters;
      const unsigned rq_span = (unsigned)((n_valid ? n_iters + 4 : n_iters) - rq_lo);
      const unsigned rv_span = (unsigned)((n_valid ? n_iters + 2 : n_iters) - rq_lo);
      typedef __attribute__((address_space(3))) const int* lds_row;
      const unsigned row_tab = (unsigned)(size_t)&rows[a][4];
      for (int it = 0; it < n_iters; ++it) {
        const bool nxt_active = is_active(it + 1);
        const int row_ahead = *reinterpret_cast<lds_row>(row_tab + 4u * it);   // chunk it + 4, used after the barrier
        bf16x8 PB[4];
        if (cur_active) {
          softmax_phase<DV>(s0, s1, acc, m_ref, l_run, thr, lane, it == causal_it, qloc0, PB);
          __builtin_amdgcn_s_setprio(3);
          pv_phase<DV>(lds_v + ((sp0 + it) % VRING) * VTILE + v_lane, PB, acc, l_run);
        }
        __builtin_amdgcn_s_setprio(3);
        if (nxt_active) qk_phase<DK>(lds_k + ((sp0 + it + 1) & 3) * KTILE + k_lane, QB, m_ref, s0, s1);
        __builtin_amdgcn_s_setprio(0);
        // K(it+2) and raw V(it+2) must have landed; the newest K request, if the last request step made one, may stay
        // in flight
        if (k_req) __builtin_amdgcn_s_waitcnt(0x0f70 | KI);
        else __builtin_amdgcn_s_waitcnt(0x0f70);
        __syncthreads();                                  // sync(it)
        // Requests: V(it+3), whose row index was found when its K was requested, then K(it+4).  (As few instructions
        // as possible: the other wave of the SIMD runs its matrix phases at raised priority meanwhile, and every
        // instruction of this one waits for an issue slot.)
        if ((unsigned)(it + 3 - rq_lo) < rv_span) dma_r(row_v, sp0 + it + 3);
        k_req = (unsigned)(it + 4 - rq_lo) < rq_span;
        if (k_req) {
          row_v = __builtin_amdgcn_readfirstlane(row_ahead);
          dma_k(row_v, sp0 + it + 4);
        }
        cur_active = nxt_active;
      }
    } else {
      // What the late waves prepare for the next tile while this one runs: its chunk table (the rows of its own chunks,
      // then of the prior attention blocks from the sorted list: a thread takes up to four list entries, which covers
      // the 1024 blocks the launcher admits), how many prior blocks there are, and the types of its own blocks.  Loads
      // are issued in the first chunk and used in the second, so that no wave waits for memory.
      const int32_t* n_list = p.idx + ((size_t)(n_n * p.TN) * p.HN + n_hn) * 2;
      const int jmax = min(n_dblk, p.TN);
      const int n_ndiag = (n_tile_start + QTILE - n_dstart) >> 6;
      int pe[4] = {0, 0, 0, 0}, p_nattn = 0;
      float p_type = 0.f;
      int ev_it = n_valid ? 0 : -1;
      // transpositions cover stream chunks tr_lo <= it + 2 < tr_lo + tr_span (this tile's, then the next tile's first two)
      const int tr_lo = cur_real ? 0 : n_iters;
      const unsigned tr_span = (unsigned)((n_valid ? n_iters + 2 : n_iters) - tr_lo);
      for (int it = 0; it < n_iters; ++it) {
        const bool nxt_active = is_active(it + 1);
        const bool last = it == n_iters - 1;
        // Preparation work for the next tile happens in iterations 0, 1, n-2 and n-1 only: `ev_it` is the next of
        // those, so that an ordinary iteration pays one scalar comparison.
        if (it == ev_it) {
          if (it == 0) {
#pragma unroll
            for (int m = 0; m < 4; ++m) {
              const int j = lt + 256 * m;
              pe[m] = j < jmax ? n_list[(size_t)j * list_stride] : 0;
            }
            p_nattn = p.nblk[((size_t)n_n * p.HN + n_hn) * 2];
            if (wave == 4) {
              const int blk = n_dblk + lane;
              const bool in_range = lane < n_ndiag && (size_t)blk * Bs < (size_t)(n_tile_start + QTILE);
              const size_t ti = ((size_t)(n_n * p.TN + (in_range ? blk : n_dblk)) * p.HN + n_hn) * 2;
              p_type = p.types_dtype == NATSL_F32 ? reinterpret_cast<const float*>(p.types)[ti]
                                                  : bf16_to_f32(reinterpret_cast<const bf16_t*>(p.types)[ti]);
            }
          }
          if (it == 1) {
            int cnt = 0;
#pragma unroll
            for (int m = 0; m < 4; ++m) {
              const int j = lt + 256 * m;
              const bool ok = j < jmax && j < p_nattn && (pe[m] + 1) * Bs <= n_dstart;
              cnt += __popcll(__ballot(ok));
              // (the qualifying entries form a prefix of the list: entry j's chunks follow those of the entries before it)
              if (ok)
                for (int sub = 0; sub < per_blk; ++sub)
                  rows[a ^ 1][n_ndiag + j * per_blk + sub] = (n_bos + pe[m] * Bs + 64 * sub) * p.HKV + n_hkv;
            }
            if (lt < n_ndiag) rows[a ^ 1][lt] = (n_bos + n_dstart + 64 * lt) * p.HKV + n_hkv;
            if (lane == 0) info[a ^ 1].count[gw] = cnt;
            if (wave == 4) {
              const int blk = n_dblk + lane;
              const bool in_range = lane < n_ndiag && (size_t)blk * Bs < (size_t)(n_tile_start + QTILE);
              const unsigned long long d = __ballot(in_range && rintf(p_type) == 1.0f);
              if (lane == 0) {
                info[a ^ 1].diag_lo = (unsigned)d;
                info[a ^ 1].diag_hi = (unsigned)(d >> 32);
              }
            }
          }
          if (wave == 4) {
            // the tile after the next: ticket asked for in the last chunk but one, turned into a tile in the last
            if (it == n_iters - 2 && cq < STREAM_QUEUES && lane == 0) t_ahead = atomicAdd(&queue[(xcc + (unsigned)cq) & 7u], 1u);
            if (last) {
              const int r0 = resolve_ticket(__builtin_amdgcn_readfirstlane(t_ahead), &info[a ^ 1]);
              // the next tile's table ends with the first four chunks of the tile after it
              const int nn_iters = n_ndiag + (info[a ^ 1].count[0] + info[a ^ 1].count[1] + info[a ^ 1].count[2] + info[a ^ 1].count[3]) * per_blk;
              if (r0 >= 0 && lane < 4) rows[a ^ 1][nn_iters + lane] = r0 + 64 * lane * p.HKV;
            }
          }
          ev_it = it == 0 ? 1 : (it < n_iters - 2 ? n_iters - 2 : it + 1);
        }
        bf16x8 PB[4];
        if (cur_active) softmax_phase<DV>(s0, s1, acc, m_ref, l_run, thr, lane, it == causal_it, qloc0, PB);
#pragma unroll
        for (int i = 0; i < 4; ++i) asm volatile("" : "+v"(PB[i]));   // the probabilities exist before the barrier
        __syncthreads();                                  // sync(it)
        __builtin_amdgcn_s_setprio(3);
        if (cur_active) pv_phase<DV>(lds_v + ((sp0 + it) % VRING) * VTILE + v_lane, PB, acc, l_run);
        if (nxt_active) qk_phase<DK>(lds_k + ((sp0 + it + 1) & 3) * KTILE + k_lane, QB, m_ref, s0, s1);
        __builtin_amdgcn_s_setprio(0);
        if ((unsigned)(it + 2 - tr_lo) < tr_span) transpose_v(sp0 + it + 2);
        cur_active = nxt_active;
      }
    }

    // ---- end of the tile: output (early waves now, late waves after the next hand-over barrier), the request held back,
    // the next tile's queries
    {
      const size_t row0 = (size_t)(bos + q0) * p.HQ + c_hq;
      const unsigned stage_e = lds_r + ((sp0 + n_iters) & 1) * RTILE + gw * (32 * DV);
      const unsigned stage_l = lds_r + ((sp0 + n_iters + 1) & 1) * RTILE + gw * (32 * DV);
      if (!late) {
        load_next_q();   // (ahead of the stores: what waits for the queries later does not wait for the stores then)
        if (cur_real) store_tile(stage_e, row0);
        __builtin_amdgcn_s_waitcnt(0xc07f);   // the staged rows have been read
        if (!n_valid) break;
        dma_r(__builtin_amdgcn_readfirstlane(rows[a][n_iters + 2]), sp0 + n_iters + 2);
        k_req = false;   // the newest request is now a V request: everything has to land before the next barrier but one
      } else {
        load_next_q();
        if (!n_valid) {
          if (cur_real) store_tile(stage_l, row0);   // (no next tile: nothing was transposed after this tile's own chunks)
          break;
        }
        pend_store = cur_real;
        pend_stage = stage_l;
        pend_row0 = row0;
      }
    }
    c_n = n_n; c_hq = n_hq; c_tile = n_tile; c_hkv = n_hkv; c_hn = n_hn; dstart = n_dstart; dblk = n_dblk;
    cur_real = true;
    sp0 += (unsigned)n_iters;
    a ^= 1;
  }

}

// The LDS reservation of a kernel is an attribute of the function per device: set when a device first runs it.
static int reserve_lds(const void* kern, std::atomic<unsigned long long>& done, size_t lds) {
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return fail(NATSL_ERR_LAUNCH, "softmax: cannot name the current device (%s)", hipGetErrorString(e));
  const unsigned long long bit = 1ull << (dev & 63);
  if (dev < 64 && (done.load(std::memory_order_acquire) & bit)) return NATSL_OK;
  e = hipFuncSetAttribute(kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
  if (e != hipSuccess) return fail(NATSL_ERR_LAUNCH, "softmax: cannot reserve %zu bytes of LDS: %s", lds, hipGetErrorString(e));
  if (dev < 64) done.fetch_or(bit, std::memory_order_release);
  return NATSL_OK;
}

template <int DK, int DV, int NWAVES>
static int launch_softmax(const SoftmaxParams& p, hipStream_t stream) {
  constexpr int KP = DK + 8, VP = DV + 8, QTILE = 32 * NWAVES;
  size_t lds = (size_t)2 * (64 * KP + DV * VT_PITCH) * sizeof(bf16_t);
  const size_t epi = (size_t)QTILE * VP * sizeof(bf16_t);
  if (epi > lds) lds = epi;
  const size_t ring = ((size_t)4 * 64 * DK + (size_t)2 * 64 * DV + (size_t)3 * DV * VTP) * sizeof(bf16_t) + 1024;  // 8 waves: four K tiles, two raw and three transposed V tiles, 1 KiB aligned
  if (NWAVES == 8 && ring > lds) lds = ring;
  auto kern = softmax_sparse_fwd_kernel<DK, DV, NWAVES>;
  static std::atomic<unsigned long long> reserved{0};
  if (const int rc = reserve_lds(reinterpret_cast<const void*>(kern), reserved, lds)) return rc;
  const long long grid = p.seqs ? (long long)p.total_tiles * (QTILE_TABLE / QTILE) * p.HQ
                                : (long long)8 * ((p.B * p.HQ + 7) / 8) * ((p.T + QTILE - 1) / QTILE);
  if (grid <= 0) return NATSL_OK;
  hipLaunchKernelGGL(kern, dim3((unsigned)grid), dim3(64 * NWAVES), lds, stream, p);
  return check_launch("natsl_softmax_sparse_fwd");
}

// Ticket counters of the persistent kernel: library-owned device memory, STREAM_SLOTS slots of counters.  Consecutive
// launches rotate through the slots, and each launch is preceded ON ITS STREAM by a fill kernel that zeroes its slot (a
// kernel, not hipMemsetAsync, so that both can be captured into a HIP graph and replayed).  Nothing is left to set
// back afterwards: a launch that was cut short cannot poison a later one.  Two launches use one slot at the same time
// only if STREAM_SLOTS launches lie between them and both are still running, or if a captured graph (whose slot was
// fixed at capture) is replayed next to an eager launch that drew the same slot; the launches would then share each
// other's tickets and leave tiles uncomputed, so keep fewer than STREAM_SLOTS launches of this entry in flight per GPU
// and replay captured launches on the stream that also carries the eager ones.
constexpr int STREAM_SLOTS = 64;
static __device__ __align__(256) unsigned stream_queues[STREAM_SLOTS * STREAM_SLOT_WORDS];

__global__ void stream_queue_clear_kernel(unsigned* slot) {
  if (threadIdx.x < STREAM_SLOT_WORDS) slot[threadIdx.x] = 0u;
}

struct StreamDevice {
  unsigned* queues = nullptr;
  int cus = 0;
};

static const StreamDevice* stream_device(int* rc) {
  constexpr int MAX_DEVICES = 64;
  static StreamDevice devs[MAX_DEVICES];
  static std::mutex mu;
  *rc = NATSL_OK;
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess || dev < 0 || dev >= MAX_DEVICES) {
    *rc = fail(NATSL_ERR_LAUNCH, "softmax: cannot name the current device (%s)", hipGetErrorString(e));
    return nullptr;
  }
  std::lock_guard<std::mutex> lock(mu);
  if (!devs[dev].queues) {
    void* a = nullptr;
    e = hipGetSymbolAddress(&a, HIP_SYMBOL(stream_queues));  // with device `dev` current: that device's copy
    int cus = 0;
    if (e == hipSuccess) e = hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev);
    if (e != hipSuccess || !a || cus <= 0) {
      *rc = fail(NATSL_ERR_LAUNCH, "softmax: cannot set up the work queues on device %d (%s)", dev, hipGetErrorString(e));
      return nullptr;
    }
    devs[dev].cus = cus;
    devs[dev].queues = static_cast<unsigned*>(a);
  }
  return &devs[dev];
}

template <int DK, int DV>
static int launch_softmax_stream(const SoftmaxParams& p, const StreamDevice* d, hipStream_t stream) {
  static std::atomic<unsigned> launches{0};
  static std::atomic<unsigned long long> reserved{0};
  const size_t lds = ((size_t)4 * 64 * DK + (size_t)2 * 64 * DV + (size_t)3 * DV * VTP) * sizeof(bf16_t) + 1024;
  auto kern = softmax_stream_kernel<DK, DV>;
  if (const int rc = reserve_lds(reinterpret_cast<const void*>(kern), reserved, lds)) return rc;
  unsigned* queue = d->queues + (size_t)(launches.fetch_add(1) % STREAM_SLOTS) * STREAM_SLOT_WORDS;
  hipLaunchKernelGGL(stream_queue_clear_kernel, dim3(1), dim3(64), 0, stream, queue);
  hipLaunchKernelGGL(kern, dim3((unsigned)d->cus), dim3(512), lds, stream, p, queue);
  return check_launch("natsl_softmax_sparse_fwd");
}

// Which kernel natsl_softmax_sparse_fwd runs for a problem: the persistent one for unpacked input of whole 256-query
// tiles, at least two per compute unit (its per-tile saving needs a tile to follow); else one workgroup per tile, of 256
// queries on 8 waves once there is at least one such tile per compute unit (measured: from there on that shape is the
// faster one; below, 128-query tiles fill more compute units).
static int softmax_variant(int B, int T, int HQ, int HKV, int block, bool packed, bool allow_persistent, const StreamDevice** sd, int* rc) {
  *sd = nullptr;
  *rc = NATSL_OK;
  if (allow_persistent && !packed && T % 256 == 0 && T <= 65536 && block <= 2048 && (long long)B * T * HKV < (1ll << 31)) {
    const StreamDevice* d = stream_device(rc);
    if (!d) return -1;
    if ((long long)B * HQ * (T / 256) >= 2ll * d->cus) {
      *sd = d;
      return NATSL_SOFTMAX_PERSISTENT;
    }
  }
  return (long long)B * HQ * cdiv(T, 256) >= 256 ? NATSL_SOFTMAX_TILE_256 : NATSL_SOFTMAX_TILE_128;
}

}  // namespace natsl

using namespace natsl;

static int softmax_fwd(const void* q, const void* k, const void* v, void* o, float* lse, const void* types, int types_dtype,
                       const int32_t* nats_block_indices, const int32_t* n_nats_blocks, int B, int T, int HQ, int HKV, int HN, int K,
                       int V, int TN, int block, float scale, int same_block_visible, int dtype, const natsl_seq_row* seqs,
                       int n_seqs, int total_units, natsl_stream_t stream, bool allow_persistent) {
  if (!q || !k || !v || !o || !lse || !types || !nats_block_indices || !n_nats_blocks)
    return fail(NATSL_ERR_INVALID, "softmax: null pointer argument");
  if (dtype != NATSL_BF16) return fail(NATSL_ERR_UNSUPPORTED, "softmax: only bf16 tensors are supported (got dtype %d)", dtype);
  if (types_dtype != NATSL_BF16 && types_dtype != NATSL_F32) return fail(NATSL_ERR_UNSUPPORTED, "softmax: block types must be f32 or bf16");
  if (B <= 0 || T <= 0 || HQ <= 0 || HKV <= 0 || HN <= 0 || TN <= 0) return fail(NATSL_ERR_INVALID, "softmax: non-positive dimension");
  if (HQ % HKV || HQ % HN) return fail(NATSL_ERR_INVALID, "softmax: HQ=%d must be a multiple of HKV=%d and HN=%d", HQ, HKV, HN);
  if (block < 64 || block % 64) return fail(NATSL_ERR_UNSUPPORTED, "softmax: block size %d must be a multiple of 64", block);
  if (seqs ? (B != 1 || n_seqs <= 0) : (TN != cdiv(T, block)))
    return fail(NATSL_ERR_INVALID, "softmax: TN=%d does not match T=%d, block=%d (or packed input with B != 1)", TN, T, block);
  if (!((K == 64 || K == 128) && (V == 64 || V == 128)))
    return fail(NATSL_ERR_UNSUPPORTED, "softmax: head dims K=%d, V=%d not built (supported: 64/128 x 64/128)", K, V);

  SoftmaxParams p;
  p.q = (const bf16_t*)q; p.k = (const bf16_t*)k; p.v = (const bf16_t*)v; p.o = (bf16_t*)o; p.lse = lse;
  p.types = types; p.types_dtype = types_dtype; p.idx = nats_block_indices; p.nblk = n_nats_blocks;
  p.seqs = reinterpret_cast<const SeqRow*>(seqs); p.n_seqs = seqs ? n_seqs : 0;
  p.B = B; p.T = T; p.HQ = HQ; p.HKV = HKV; p.HN = HN; p.TN = TN; p.block = block;
  p.nq_tiles = cdiv(T, QTILE_TABLE);
  p.total_tiles = seqs ? total_units : B * p.nq_tiles;
  p.scale_log2 = scale * 1.4426950408889634f;
  p.same_block = same_block_visible ? 1 : 0;
  p.g_kv = HQ / HKV;
  p.g_n = HQ / HN;
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  const StreamDevice* sd = nullptr;
  int rc;
  const int variant = softmax_variant(B, T, HQ, HKV, block, seqs != nullptr, allow_persistent, &sd, &rc);
  if (variant < 0) return rc;
  p.variant = variant == NATSL_SOFTMAX_TILE_128 ? 4 : 8;
#define NATSL_SM(KK, VV)                                              \
  if (K == KK && V == VV) {                                           \
    if (sd) return launch_softmax_stream<KK, VV>(p, sd, s);           \
    return p.variant == 8 ? launch_softmax<KK, VV, 8>(p, s) : launch_softmax<KK, VV, 4>(p, s); \
  }
  NATSL_SM(128, 128)
  NATSL_SM(64, 64)
  NATSL_SM(64, 128)
  NATSL_SM(128, 64)
#undef NATSL_SM
  return fail(NATSL_ERR_UNSUPPORTED, "softmax: head dims K=%d, V=%d not built (supported: 64/128 x 64/128)", K, V);
}

extern "C" int natsl_softmax_sparse_fwd(const void* q, const void* k, const void* v, void* o, float* lse,
                                        const void* types, int types_dtype, const int32_t* nats_block_indices,
                                        const int32_t* n_nats_blocks, int B, int T, int HQ, int HKV, int HN, int K,
                                        int V, int TN, int block, float scale, int same_block_visible, int dtype,
                                        const natsl_seq_row* seqs, int n_seqs, int total_units,
                                        natsl_stream_t stream) {
  return softmax_fwd(q, k, v, o, lse, types, types_dtype, nats_block_indices, n_nats_blocks, B, T, HQ, HKV, HN, K, V, TN, block,
                     scale, same_block_visible, dtype, seqs, n_seqs, total_units, stream, true);
}

extern "C" int natsl_softmax_sparse_fwd_per_tile(const void* q, const void* k, const void* v, void* o, float* lse,
                                                 const void* types, int types_dtype, const int32_t* nats_block_indices,
                                                 const int32_t* n_nats_blocks, int B, int T, int HQ, int HKV, int HN, int K,
                                                 int V, int TN, int block, float scale, int same_block_visible, int dtype,
                                                 const natsl_seq_row* seqs, int n_seqs, int total_units,
                                                 natsl_stream_t stream) {
  return softmax_fwd(q, k, v, o, lse, types, types_dtype, nats_block_indices, n_nats_blocks, B, T, HQ, HKV, HN, K, V, TN, block,
                     scale, same_block_visible, dtype, seqs, n_seqs, total_units, stream, false);
}

extern "C" int natsl_softmax_fwd_variant(int B, int T, int HQ, int HKV, int block, int packed) {
  const StreamDevice* sd = nullptr;
  int rc;
  const int variant = softmax_variant(B, T, HQ, HKV, block, packed != 0, true, &sd, &rc);
  return variant < 0 ? rc : variant;
}
