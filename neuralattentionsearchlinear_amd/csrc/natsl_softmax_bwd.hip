// Backward of the softmax branch for gfx950.
//
//   delta_kernel   delta[t] = sum_v dO[t,v] O[t,v]                                  (attns.py:357-372)
//   dq_kernel      one workgroup per tile of 128 queries, the forward's walk over the visible key chunks:
//                  S^T = K Q^T, P = exp2(S c - lse), dP^T = V dO^T, dS = P (dP - delta), dQ^T += K^T dS^T (attns.py:383-708)
//   dkdv_kernel    unit = one 64-key chunk of a kv head, walking the query chunks that see it (the rest of its own
//                  block, and every later chunk when the block is typed attention), for every query head of the group:
//                  S = Q K^T, dP = dO V^T, dV^T += dO^T P, dK^T += Q^T dS, dnats += sum dS over later blocks (attns.py:719-983)
//                  The query tiles (Q, dO, lse, delta) arrive by DMA in a ring of three LDS slots, two steps ahead.
//                  One persistent workgroup per CU takes units from per-XCD work queues.  Eight waves in two roles:
//                  four form S, P and dV, four form dP, dS and dK of the same (32 keys) x (32 queries) quarters; P
//                  passes between the two in fp32 through LDS.  Each wave keeps one stationary operand and one
//                  accumulator, so two waves fit a SIMD.
//
// Layouts follow the forward kernel: the stationary operand of a workgroup (Q, dO there; K, V here) sits in registers
// as the B operand (lane = its row), the streamed tiles are row-major in LDS, the accumulators' own layout is the B
// operand of the second product, and the transposed A operands (K^T, dO^T, Q^T) come out of the row-major tiles with
// the transposing LDS read.
#include "natsl_device.h"
#include "natsl_host.h"

namespace natsl {

struct SoftmaxBwdParams {
  const bf16_t *q, *k, *v, *o, *dout;
  const float* lse;
  bf16_t *dq, *dk, *dv;
  float* dnats;   // [B, TN, HQ], zero on entry
  float* delta;   // [B, T, HQ] workspace
  int* queue;     // [8] workspace: next unit of each XCD's list for the dk/dv kernel, zeroed by the delta kernel
  const void* types;
  int types_dtype;
  const int32_t* idx;
  const int32_t* nblk;
  int B, T, HQ, HKV, HN, TN, block;
  const SeqRow* seqs;   // packed sequences (B = 1): one row per sequence, else null
  int n_seqs, total_tiles, total_chunks;   // packed: 256-query table tiles and 64-token chunks over all sequences
  float scale, scale_log2;
  int same_block;
  int dnats_invalid;   // also give dnats to blocks that are not typed attention (what their keys would contribute, reference attns.py:1318-1325)
};

NATSL_DEVICE bool bwd_type_is_one(const void* types, int dtype, size_t i) {
  float x = dtype == NATSL_F32 ? reinterpret_cast<const float*>(types)[i] : bf16_to_f32(reinterpret_cast<const bf16_t*>(types)[i]);
  return rintf(x) == 1.0f;
}

constexpr int BWD_MAX_LDS_LIST = 2048;

// Position swizzle of the dkdv kernel's query tiles (rows of D bf16, unpadded): 16-byte segment s of row r is stored at
// s ^ bwd_swizzle<D>(r).  A bijection over the 16 rows that one clock of a 16-byte row read serves (conflict-free), and
// two of four consecutive rows never differ by 1, so the 4 rows x 2 segments of a transposing read's 16 lanes
// fall on different banks as well.
template <int D>
NATSL_DEVICE int bwd_swizzle(const int r) {
  if constexpr (D == 128) return ((r & 7) << 1) | ((r >> 3) & 1);
  const int y = (r >> 1) & 7;
  return ((y & 3) << 1) | (y >> 2);
}

// one DMA instruction: lane l copies 16 (4) bytes from base + voff to LDS byte address lds + 16 l (4 l)
NATSL_DEVICE void dma16(const void* base, const unsigned voff, const unsigned lds) {
  asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1" ::"v"(voff), "s"(base), "s"(lds) : "memory", "m0");
}
NATSL_DEVICE void dma4(const void* base, const unsigned voff, const unsigned lds) {
  asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dword %0, %1" ::"v"(voff), "s"(base), "s"(lds) : "memory", "m0");
}
// ... under a wave-uniform condition (non-zero or zero, held in a scalar register): with no lane enabled the instruction
// requests nothing, which lets a request sit in straight-line code between matrix instructions and still be conditional.
NATSL_DEVICE void dma16_if(const void* base, const unsigned voff, const unsigned lds, const unsigned on) {
  unsigned long long saved;
  asm volatile(
      "s_mov_b32 m0, %3\n\ts_mov_b64 %0, exec\n\ts_cmp_lg_u32 %4, 0\n\ts_cselect_b64 exec, exec, 0\n\tglobal_load_lds_dwordx4 %1, %2\n\ts_mov_b64 exec, %0"
      : "=&s"(saved)
      : "v"(voff), "s"(base), "s"(lds), "s"(__builtin_amdgcn_readfirstlane(on))
      : "memory", "m0", "scc");
}
NATSL_DEVICE void dma4_if(const void* base, const unsigned voff, const unsigned lds, const unsigned on) {
  unsigned long long saved;
  asm volatile(
      "s_mov_b32 m0, %3\n\ts_mov_b64 %0, exec\n\ts_cmp_lg_u32 %4, 0\n\ts_cselect_b64 exec, exec, 0\n\tglobal_load_lds_dword %1, %2\n\ts_mov_b64 exec, %0"
      : "=&s"(saved)
      : "v"(voff), "s"(base), "s"(lds), "s"(__builtin_amdgcn_readfirstlane(on))
      : "memory", "m0", "scc");
}

// A operand of a 32x32x16 product taken TRANSPOSED from a row-major LDS tile: A[m = lane%32][k-slot (hf, j)] =
// tile[row_base + 8(j/4) + 4hf + j%4][col_base + m].  ds_read_b64_tr_b16: within each group of 16 lanes, lane i supplies
// the address of a 4-element row R_i and receives { R_{4j + i/4}[i%4] : j < 4 }.
NATSL_DEVICE bf16x8 tr_operand(const bf16_t* tile, const int pitch, const int row_base, const int col_base, const int lane) {
  const int i16 = lane & 15, colsel = 16 * ((lane >> 4) & 1), hf = lane >> 5;
  const bf16_t* p = tile + (row_base + 4 * hf + (i16 >> 2)) * pitch + col_base + colsel + 4 * (i16 & 3);
  return join4(lds_tr4(p), lds_tr4(p + 8 * pitch));
}

NATSL_DEVICE bf16x8 pack8(const f32x16& x, const int ss) {
  u32x4 w;
#pragma unroll
  for (int j = 0; j < 4; ++j) w[j] = pack_bf16x2(x[8 * ss + 2 * j], x[8 * ss + 2 * j + 1]);
  return __builtin_bit_cast(bf16x8, w);
}

// ---------------------------------------------------------------------------------------------
template <int DV>
__global__ __launch_bounds__(256) void delta_kernel(const SoftmaxBwdParams p) {
  constexpr int LPR = DV / 8, RPB = 256 / LPR;   // lanes per row, rows per workgroup
  const long long rows = (long long)p.B * p.T * p.HQ;
  const long long row = (long long)blockIdx.x * RPB + threadIdx.x / LPR;
  const int seg = threadIdx.x % LPR;
  if (blockIdx.x == 0 && threadIdx.x < 8) p.queue[threadIdx.x] = 0;   // the dk/dv kernel's work queues (it runs after this kernel)
  float acc = 0.f;
  if (row < rows) {
    const u32x4 a = *reinterpret_cast<const u32x4*>(p.o + row * DV + 8 * seg);
    const u32x4 b = *reinterpret_cast<const u32x4*>(p.dout + row * DV + 8 * seg);
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      acc += __uint_as_float(a[j] << 16) * __uint_as_float(b[j] << 16);
      acc += __uint_as_float(a[j] & 0xffff0000u) * __uint_as_float(b[j] & 0xffff0000u);
    }
  }
#pragma unroll
  for (int m = LPR / 2; m >= 1; m >>= 1) acc += __shfl_xor(acc, m);
  if (row < rows && seg == 0) p.delta[row] = acc;
}

// ---------------------------------------------------------------------------------------------
// 256 threads stage a [64][D] tile row-major (pitch D+8) from rows tok0.. of a [T][stride] tensor, rows clamped to len-1
template <int D>
struct RowStage {
  static constexpr int SEGS = D / 8, ROWS = 256 / SEGS, PASSES = 64 / ROWS, PITCH = D + 8;
  u32x4 r[PASSES];
  NATSL_DEVICE void load(const bf16_t* base, const size_t row_stride, const int tok0, const int len, const int tid) {
    const int row = tid / SEGS, seg = tid % SEGS;
#pragma unroll
    for (int i = 0; i < PASSES; ++i) {
      const int tok = min(tok0 + row + ROWS * i, len - 1);
      r[i] = *reinterpret_cast<const u32x4*>(base + (size_t)tok * row_stride + 8 * seg);
    }
  }
  NATSL_DEVICE void store(bf16_t* tile, const int tid) const {
    const int row = tid / SEGS, seg = tid % SEGS;
#pragma unroll
    for (int i = 0; i < PASSES; ++i) *reinterpret_cast<u32x4*>(tile + (row + ROWS * i) * PITCH + 8 * seg) = r[i];
  }
};

template <int DK, int DV>
__global__ __launch_bounds__(256, 2) void dq_kernel(const SoftmaxBwdParams p) {
  constexpr int KP = DK + 8, VP = DV + 8, KS = DK / 16, VS = DV / 16, DT = DK / 32, QTILE = 128;
  extern __shared__ __align__(16) unsigned char smem[];
  bf16_t* Ks = reinterpret_cast<bf16_t*>(smem);  // [2][64][KP]
  bf16_t* Vs = Ks + 2 * 64 * KP;                 // [2][64][VP]
  __shared__ int lds_list[BWD_MAX_LDS_LIST];
  __shared__ int lds_count;

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int l32 = lane & 31, hf = lane >> 5;
  int n, hq, tile, len, bos, bos_nats;
  if (p.seqs == nullptr) {
    const int nq_tiles = (p.T + QTILE - 1) / QTILE;
    // every 8th block index lands on the same XCD: an XCD takes the tiles of one (sequence, head) in turn, last tile
    // first, so the workgroups that share an L2 walk the same key blocks
    const int xcd = (int)blockIdx.x & 7, j = (int)blockIdx.x >> 3;
    const int pair = (j / nq_tiles) * 8 + xcd;
    tile = nq_tiles - 1 - j % nq_tiles;
    if (pair >= p.B * p.HQ) return;   // (the grid is rounded up to whole groups of 8 pairs)
    n = pair / p.HQ;
    hq = pair % p.HQ;
    len = p.T;
    bos = n * p.T;
    bos_nats = n * p.TN;
  } else {
    // packed: the table counts 256-query tiles per sequence, two of this kernel's; last tiles first
    const int gt = p.total_tiles * 2 - 1 - (int)blockIdx.x / p.HQ;
    hq = (int)blockIdx.x % p.HQ;
    n = 0;
    for (int i = 1; i < p.n_seqs; ++i)
      if (p.seqs[i].qtile_off * 2 <= gt) n = i;
    tile = gt - p.seqs[n].qtile_off * 2;
    bos = p.seqs[n].bos;
    len = p.seqs[n].eos - bos;
    bos_nats = p.seqs[n].bos_nats;
    if (tile * QTILE >= len) return;   // a sequence's last table slot may hold one tile of this size only
  }
  const int Bs = p.block, per_blk = Bs >> 6;
  const int hkv = hq / (p.HQ / p.HKV), hn = hq / (p.HQ / p.HN);
  const int tile_start = tile * QTILE;
  const int q0 = tile_start + wave * 32;
  const int my_chunk = q0 >> 6, qloc0 = q0 & 63;
  const int dstart = (tile_start / p.block) * p.block;
  const bool wave_valid = q0 < len;

  const bf16_t* kp = p.k + ((size_t)bos * p.HKV + hkv) * DK;
  const bf16_t* vp = p.v + ((size_t)bos * p.HKV + hkv) * DV;
  const size_t krow = (size_t)p.HKV * DK, vrow = (size_t)p.HKV * DV;
  const int32_t* list = p.idx + ((size_t)bos_nats * p.HN + hn) * 2;
  const size_t list_stride = (size_t)p.HN * 2;
  const int n_attn = p.nblk[((size_t)n * p.HN + hn) * 2];

  // Q and dO as B operands (lane = query), lse and delta of the lane's query
  bf16x8 QB[KS], DOB[VS];
  const int qi = min(q0 + l32, len - 1);
  {
    const bf16_t* qr = p.q + ((size_t)(bos + qi) * p.HQ + hq) * DK + 8 * hf;
#pragma unroll
    for (int s = 0; s < KS; ++s) QB[s] = ld8(qr + 16 * s);
    const bf16_t* dr = p.dout + ((size_t)(bos + qi) * p.HQ + hq) * DV + 8 * hf;
#pragma unroll
    for (int s = 0; s < VS; ++s) DOB[s] = ld8(dr + 16 * s);
  }
  const float lse_q = p.lse[(size_t)(bos + qi) * p.HQ + hq], delta_q = p.delta[(size_t)(bos + qi) * p.HQ + hq];

  f32x16 acc[DT];
#pragma unroll
  for (int dt = 0; dt < DT; ++dt)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[dt][r] = 0.f;

  RowStage<DK> sk;
  RowStage<DV> sv;
  const int n_diag = (min(len, tile_start + QTILE) - dstart + 63) >> 6;
  sk.load(kp, krow, dstart, len, tid);
  sv.load(vp, vrow, dstart, len, tid);
  if (tid == 0) lds_count = 0;
  __syncthreads();
  {
    const int jmax = min(dstart / Bs, p.TN);
    int cnt = 0;
    for (int j = tid; j < jmax; j += 256) {
      const int e = list[j * list_stride];
      if (j < n_attn && (e + 1) * Bs <= dstart) {
        ++cnt;
        if (j < BWD_MAX_LDS_LIST) lds_list[j] = e;
      }
    }
    if (cnt) atomicAdd(&lds_count, cnt);
  }
  unsigned long long diag_attn;
  {
    const int blk = dstart / Bs + lane;
    const bool in_range = lane < n_diag && (size_t)blk * Bs < (size_t)min(len, tile_start + QTILE);
    diag_attn = __ballot(in_range && bwd_type_is_one(p.types, p.types_dtype, ((size_t)(bos_nats + blk) * p.HN + hn) * 2));
  }
  sk.store(Ks, tid);
  sv.store(Vs, tid);
  __syncthreads();
  const int n_prior_chunks = __builtin_amdgcn_readfirstlane(lds_count) * per_blk;
  const int n_iters = n_diag + n_prior_chunks;
  int nx_it = 1, nx_j = 0, nx_sub = 0;
  auto next_key_start = [&]() -> int {
    int ks;
    if (nx_it < n_diag) {
      ks = dstart + nx_it * 64;
    } else {
      int e;
      if (nx_j < BWD_MAX_LDS_LIST) e = __builtin_amdgcn_readfirstlane(lds_list[nx_j]);
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
  int ks_fetch = dstart;
  if (n_iters > 1) ks_fetch = next_key_start();
  const float c = p.scale_log2;
  const int my_blk = q0 / Bs;

  for (int it = 0; it < n_iters; ++it) {
    const int buf = it & 1;
    if (it + 1 < n_iters) {
      sk.load(kp, krow, ks_fetch, len, tid);
      sv.load(vp, vrow, ks_fetch, len, tid);
    }
    bool active = wave_valid, causal = false;
    if (it < n_diag) {
      const int jc = (dstart >> 6) + it;
      const int kblk = (jc * 64) / Bs;
      if (p.same_block) {
        if (jc > my_chunk) active = false;
        else if (jc == my_chunk) causal = true;
        else active = active && (kblk == my_blk || ((diag_attn >> (kblk - dstart / Bs)) & 1ull));
      } else {
        active = active && jc < my_chunk && kblk < my_blk && ((diag_attn >> (kblk - dstart / Bs)) & 1ull);
      }
    }
    if (active) {
      const bf16_t* Kb = Ks + buf * 64 * KP;
      const bf16_t* Vb = Vs + buf * 64 * VP;
#pragma unroll
      for (int kt = 0; kt < 2; ++kt) {
        // The LDS operands of the first two products form one stream (K row piece, V row piece, K, V, ...) that is
        // read a few instructions ahead of its use: reading all of them up front needs 64 registers and spills.
        constexpr int NOPS = KS + VS, AHEAD = 4;
        constexpr int NPAIR = KS < VS ? KS : VS;   // the two chains alternate while both last; the longer one ends alone
        auto is_v = [&](const int j) __attribute__((always_inline)) { return j < 2 * NPAIR ? (j & 1) != 0 : VS > KS; };
        auto step_of = [&](const int j) __attribute__((always_inline)) { return j < 2 * NPAIR ? j >> 1 : j - NPAIR; };
        auto ld_op = [&](const int j) __attribute__((always_inline)) -> bf16x8 {
          const int st = step_of(j);
          return is_v(j) ? ld8(Vb + (32 * kt + l32) * VP + 16 * st + 8 * hf) : ld8(Kb + (32 * kt + l32) * KP + 16 * st + 8 * hf);
        };
        bf16x8 op[NOPS + AHEAD];
#pragma unroll
        for (int j = 0; j < AHEAD; ++j) op[j] = ld_op(j);
        f32x16 s, dp;
#pragma unroll
        for (int r = 0; r < 16; ++r) s[r] = dp[r] = 0.f;
#pragma unroll
        for (int j = 0; j < NOPS; ++j) {
          if (j + AHEAD < NOPS) op[j + AHEAD] = ld_op(j + AHEAD);
          if (is_v(j)) dp = mfma32(op[j], DOB[step_of(j)], dp);
          else s = mfma32(op[j], QB[step_of(j)], s);
        }
        __builtin_amdgcn_sched_group_barrier(0x100, AHEAD, 0);
#pragma unroll
        for (int j = 0; j < NOPS; ++j) {
          if (j + AHEAD < NOPS) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
          __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        }
        // dQ^T += K^T dS^T: the transposed K operands are read ahead as well, the first of them before the exponentials
        constexpr int N3 = 2 * DT, A3 = 4 < N3 ? 4 : N3;
        auto tr_op = [&](const int j) __attribute__((always_inline)) -> bf16x8 {
          return tr_operand(Kb, KP, 32 * kt + 16 * (j / DT), 32 * (j % DT), lane);
        };
        bf16x8 at[N3 + A3];
#pragma unroll
        for (int j = 0; j < A3; ++j) at[j] = tr_op(j);
        __builtin_amdgcn_sched_barrier(0);
        f32x16 ds;
        if (!causal) {   // every key of the chunk is visible to every query of the wave: no masks
#pragma unroll
          for (int r = 0; r < 16; ++r) ds[r] = __builtin_amdgcn_exp2f(fmaf(s[r], c, -lse_q)) * (dp[r] - delta_q);
        } else {
#pragma unroll
          for (int r = 0; r < 16; ++r) {
            const int kloc = 32 * kt + 8 * (r >> 2) + 4 * hf + (r & 3);
            const bool vis = kloc <= qloc0 + l32;
            const float pr = vis ? __builtin_amdgcn_exp2f(fmaf(s[r], c, -lse_q)) : 0.f;
            ds[r] = pr * (dp[r] - delta_q);
          }
        }
        bf16x8 PB[2];
#pragma unroll
        for (int ss = 0; ss < 2; ++ss) PB[ss] = pack8(ds, ss);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int j = 0; j < N3; ++j) {
          if (j + A3 < N3) at[j + A3] = tr_op(j + A3);
          acc[j % DT] = mfma32(at[j], PB[j / DT], acc[j % DT]);
        }
#pragma unroll
        for (int j = 0; j < N3; ++j) {
          if (j + A3 < N3) __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
          __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        }
      }
    }
    if (it + 1 < n_iters) {
      sk.store(Ks + (buf ^ 1) * 64 * KP, tid);
      sv.store(Vs + (buf ^ 1) * 64 * VP, tid);
    }
    if (it + 2 < n_iters) ks_fetch = next_key_start();
    __syncthreads();
  }

  // epilogue: dQ = scale * acc, transposed through LDS, coalesced stores
  bf16_t* Os = reinterpret_cast<bf16_t*>(smem) + wave * 32 * KP;
#pragma unroll
  for (int dt = 0; dt < DT; ++dt)
#pragma unroll
    for (int rg = 0; rg < 4; ++rg) {
      u32x2 w;
      w[0] = pack_bf16x2(acc[dt][4 * rg] * p.scale, acc[dt][4 * rg + 1] * p.scale);
      w[1] = pack_bf16x2(acc[dt][4 * rg + 2] * p.scale, acc[dt][4 * rg + 3] * p.scale);
      *reinterpret_cast<u32x2*>(Os + l32 * KP + 32 * dt + 8 * rg + 4 * hf) = w;
    }
  __builtin_amdgcn_s_waitcnt(0xc07f);
  __builtin_amdgcn_wave_barrier();
  constexpr int SEGS = DK / 8, RPP = 64 / SEGS;
#pragma unroll
  for (int pass = 0; pass < 32 / RPP; ++pass) {
    const int row = pass * RPP + lane / SEGS, seg = lane % SEGS;
    const int t = q0 + row;
    if (t < len) {
      const u32x4 w = *reinterpret_cast<const u32x4*>(Os + row * KP + seg * 8);
      *reinterpret_cast<u32x4*>(p.dq + ((size_t)(bos + t) * p.HQ + hq) * DK + seg * 8) = w;
    }
  }
}

// ---------------------------------------------------------------------------------------------
// dk/dv.  Eight waves = 2 roles x 2 key halves x 2 query halves; a wave and its partner of the other role (wave + 4, on
// the same SIMD) work on the same 32 keys x 32 queries of every step:
//   role 0: S = Q K^T, P = exp2(S c - lse) (masks, the clamp for blocks that only give dnats), dV^T += dO^T P
//   role 1: dP = dO V^T, dS = P (dP - delta), dK^T += Q^T dS, dnats
// P goes from role 0 to role 1 in fp32 through LDS (two buffers, written before the step's barrier and read after it).
// Each wave holds one stationary operand (K or V rows) and one accumulator (dV or dK) of its 32 keys: under 256
// registers, so two waves share a SIMD and one's exponentials run under the other's matrix instructions.
struct DkdvShared {
  int unit_pair, unit_jc, unit_seq;
  float red[4];
};

template <int DK, int DV>
struct DkdvLds {
  static constexpr int QROWB = DK * 2, DROWB = DV * 2;
  static constexpr unsigned DOFF = 64 * QROWB, LOFF = DOFF + 64 * DROWB, SLOT = LOFF + 512;   // slot: Q [64][DK], dO [64][DV], lse [64], delta [64]
  static constexpr unsigned XOFF = 3 * SLOT, XBUF = 4 * 4096;   // P exchange: [2][4 wave pairs][4][64 lanes] of 4 floats
  static constexpr unsigned RING = XOFF + 2 * XBUF;
  static constexpr unsigned RED = 2u * (DV / 32 + DK / 32) * 16 * 64 * sizeof(float);   // the unit's end: sums of the query halves
  static constexpr unsigned TOTAL = RING > RED ? RING : RED;
};

template <int DK, int DV, int ROLE>
NATSL_DEVICE void dkdv_role(const SoftmaxBwdParams& p, unsigned char* smem, DkdvShared& sh) {
  typedef DkdvLds<DK, DV> L;
  // the first product contracts over D1 against the rows of tile 1 (Q for role 0, dO for role 1); the second product
  // gives D2 rows from tile 2 transposed (dO for role 0, Q for role 1)
  constexpr int D1 = ROLE == 0 ? DK : DV, D2 = ROLE == 0 ? DV : DK;
  constexpr int S1 = D1 / 16, T2 = D2 / 32, VT = DV / 32, DT = DK / 32;
  constexpr int ROWB1 = D1 * 2, ROWB2 = D2 * 2;
  constexpr unsigned OFF1 = ROLE == 0 ? 0u : L::DOFF, OFF2 = ROLE == 0 ? L::DOFF : 0u;
  constexpr unsigned SLOT = L::SLOT, LOFF = L::LOFF;

  const int tid = threadIdx.x, lane = tid & 63;
  const int quad = __builtin_amdgcn_readfirstlane((tid >> 6) & 3);
  const int l32 = lane & 31, hf = lane >> 5;
  const int kh = quad & 1, qh = quad >> 1;
  const bool packed = p.seqs != nullptr;
  const int n_pairs = p.B * p.HKV;
  // ---- Persistent workgroups (one per CU) take units = (sequence, kv head, key chunk) from work queues: starting a
  // workgroup per unit left the CUs idle a quarter of the time.  Workgroups that run at the same time should stream the
  // same queries, so every XCD (block index mod 8) has a queue of its own with the key chunks of one (sequence, kv
  // head) after the other, earliest (heaviest) chunk first, and every unit walks the later query chunks from the last
  // one down: units started together stay together in L2.  A workgroup whose queue is empty takes from the other
  // XCDs' queues.  Packed sequences: one queue, the units of a sequence (kv head after kv head) after those of the one
  // before.
  const int NT_reg = (p.T + 63) >> 6;
  const bool per_xcd = !packed && n_pairs % 8 == 0;
  const int n_queues = per_xcd ? 8 : 1;
  const int queue_len = packed ? p.total_chunks * p.HKV : (per_xcd ? n_pairs / 8 : n_pairs) * NT_reg;
  int q_probe = 0;   // queues found empty so far (they stay empty)
  for (;;) {
    if (tid == 0) {
      int pr = -1, jj = 0;
      while (q_probe < n_queues) {
        const int x = per_xcd ? ((int)blockIdx.x + q_probe) & 7 : 0;
        const int i = atomicAdd(p.queue + x, 1);
        if (i < queue_len) {
          if (packed) {
            int sn = 0;
            for (int u = 1; u < p.n_seqs; ++u)
              if (p.seqs[u].chunk_off * p.HKV <= i) sn = u;
            const int r = i - p.seqs[sn].chunk_off * p.HKV, ntc = (p.seqs[sn].eos - p.seqs[sn].bos + 63) >> 6;
            pr = r / ntc;   // the kv head
            jj = r % ntc;
            sh.unit_seq = sn;
          } else {
            pr = per_xcd ? (i / NT_reg) * 8 + x : i / NT_reg;
            jj = i % NT_reg;
          }
          break;
        }
        ++q_probe;
      }
      sh.unit_pair = pr;
      sh.unit_jc = jj;
    }
    __syncthreads();
    const int pair = sh.unit_pair, jc = sh.unit_jc, seq = packed ? sh.unit_seq : 0;
    __syncthreads();   // (read before the next round's write)
    if (pair < 0) break;
    const int n = packed ? seq : pair / p.HKV, hkv = packed ? pair : pair % p.HKV;
    const int bos = packed ? p.seqs[n].bos : n * p.T, len = packed ? p.seqs[n].eos - bos : p.T;
    const int bos_nats = packed ? p.seqs[n].bos_nats : n * p.TN;
    const int NTc = (len + 63) >> 6;
    const int Bs = p.block, per_blk = Bs >> 6;
    const int G = p.HQ / p.HKV, GN = p.HQ / p.HN;
    const int kb = (jc * 64) / Bs;
    const int blk_end_chunk = min((kb + 1) * per_blk, NTc);   // one past the last chunk of the key block

    // the stationary operand: K (role 0) or V (role 1) of the wave's 32 keys as B operands (lane = key)
    bf16x8 XB[S1];
    {
      const int ki = min(jc * 64 + 32 * kh + l32, len - 1);
      const bf16_t* xr = (ROLE == 0 ? p.k : p.v) + ((size_t)(bos + ki) * p.HKV + hkv) * D1 + 8 * hf;
#pragma unroll
      for (int s = 0; s < S1; ++s) XB[s] = ld8(xr + 16 * s);
    }
    f32x16 acc[T2];
#pragma unroll
    for (int t = 0; t < T2; ++t)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[t][r] = 0.f;

    const float c = p.scale_log2;

    // ---- the ring of query tiles.  Rows are unpadded and the 16-byte segment s of row r sits at position
    // s ^ bwd_swizzle(r).  Tiles arrive by DMA (global -> LDS, no registers): each instruction fills 1 KiB of a tile, and
    // the swizzle is applied on the global side.  A wave requests its share of its own role's first tile (role 0: Q and
    // lse, role 1: dO and delta).
    constexpr int I1 = D1 / 32;   // 1 KiB DMA instructions per wave and tile
    constexpr int NREQ = I1 + 1;  // requests per wave and tile
    const unsigned lds0 = (unsigned)(size_t)smem;
    unsigned r_row[I1], r_seg[I1];   // per DMA instruction: the lane's tile row and global byte offset in the row
#pragma unroll
    for (int j = 0; j < I1; ++j) {
      const int pos = lane % (D1 / 8), row = (I1 * quad + j) * (1024 / ROWB1) + lane / (D1 / 8);
      r_row[j] = row;
      r_seg[j] = 16u * (pos ^ bwd_swizzle<D1>(row));
    }
    const bf16_t* g_src = ROLE == 0 ? p.q : p.dout;
    const float* l_src = ROLE == 0 ? p.lse : p.delta;
    // request piece r of tile jq of head hq into a slot
    auto piece = [&](const int r, const int hq, const int jq, const int slot, const void*& g, unsigned& voff, unsigned& dst) __attribute__((always_inline)) {
      const unsigned sl = lds0 + slot * SLOT;
      if (r < I1) {
        g = g_src + ((size_t)bos * p.HQ + hq) * D1;
        voff = (unsigned)min(jq * 64 + (int)r_row[r < I1 ? r : 0], len - 1) * ((unsigned)p.HQ * ROWB1) + r_seg[r < I1 ? r : 0];
        dst = sl + OFF1 + (I1 * quad + r) * 1024;
      } else {
        g = l_src + (size_t)bos * p.HQ + hq;
        voff = (unsigned)min(jq * 64 + lane, len - 1) * (unsigned)(p.HQ * 4);
        dst = sl + LOFF + 256 * ROLE;   // (the four waves of a role bring the same 256 bytes)
      }
    };
    auto request = [&](const int hq, const int jq, const int slot) __attribute__((always_inline)) {
#pragma unroll
      for (int r = 0; r < NREQ; ++r) {
        const void* g;
        unsigned voff, dst;
        piece(r, hq, jq, slot, g, voff, dst);
        if (r < I1) dma16(g, voff, dst);
        else dma4(g, voff, dst);
      }
    };
    auto request_piece_if = [&](const int r, const int hq, const int jq, const int slot, const unsigned on) __attribute__((always_inline)) {
      const void* g;
      unsigned voff, dst;
      piece(r, hq, jq, slot, g, voff, dst);
      if (r < I1) dma16_if(g, voff, dst, on);
      else dma4_if(g, voff, dst, on);
    };

    // ---- LDS byte offsets of the lane's operands inside a slot
    typedef __attribute__((address_space(3))) const bf16x8* lds_op;
    typedef __attribute__((address_space(3))) s16x4* lds_tr;
    typedef __attribute__((address_space(3))) f32x4* lds_f4;
    unsigned a1[S1];   // first product: the lane's query row, k-step st
    {
      const int row = 32 * qh + l32;
#pragma unroll
      for (int st = 0; st < S1; ++st) a1[st] = OFF1 + row * ROWB1 + 16u * ((2 * st + hf) ^ bwd_swizzle<D1>(row));
    }
    // second product: transposing reads.  Within 16 lanes, lane i addresses 4 elements of row 4 hf + i/4 (+ 8 for the
    // second read) at column 32 t + 16 (lane/16 % 2) + 4 (i % 4).
    unsigned t2[2][T2][2];
    {
      const int i16 = lane & 15;
#pragma unroll
      for (int ss = 0; ss < 2; ++ss)
#pragma unroll
        for (int rd = 0; rd < 2; ++rd) {
          const int row = 32 * qh + 16 * ss + 8 * rd + 4 * hf + (i16 >> 2);
          const int seg0 = 2 * ((lane >> 4) & 1) + ((i16 >> 1) & 1);
#pragma unroll
          for (int t = 0; t < T2; ++t) t2[ss][t][rd] = OFF2 + row * ROWB2 + 16u * ((4 * t + seg0) ^ bwd_swizzle<D2>(row)) + 8u * (i16 & 1);
        }
    }
    const unsigned xlane = lds0 + L::XOFF + quad * 4096 + 16 * lane;   // the wave pair's exchange area, this lane's 16 bytes of group 0

    for (int g = 0; g < G; ++g) {
      const int hq = hkv * G + g, hn = hq / GN;
      const bool attn = bwd_type_is_one(p.types, p.types_dtype, ((size_t)(bos_nats + kb) * p.HN + hn) * 2);
      const int n_same = p.same_block ? blk_end_chunk - jc : 0;
      // a block that is not typed attention walks the later queries only when its dnats is asked for, and then for nothing else
      const bool walk_later = attn || p.dnats_invalid != 0;
      const int n_later = __builtin_amdgcn_readfirstlane(walk_later ? max(NTc - blk_end_chunk, 0) : 0);   // (the type was read by a vector load)
      const bool attn_u = __builtin_amdgcn_readfirstlane(attn ? 1 : 0) != 0;
      const int n_it = n_same + n_later;
      float dn = 0.f;
      auto chunk_of = [&](const int it) { return it < n_same ? jc + it : NTc - 1 - (it - n_same); };
      if (n_it > 0) {
        __syncthreads();   // the previous head's last reads of the ring are done
        request(hq, chunk_of(0), 0);
        if (n_it > 1) {
          request(hq, chunk_of(1), 1);
          __builtin_amdgcn_s_waitcnt(0x0f70 | NREQ);   // vmcnt: all but the newest tile's requests
        } else {
          __builtin_amdgcn_s_waitcnt(0x0f70);
        }
        __syncthreads();
      }
      int slot = 0;
      for (int it = 0; it < n_it; ++it) {
        const int jq = chunk_of(it);
        const unsigned sb = lds0 + slot * SLOT;
        const unsigned xb = xlane + (it & 1) * L::XBUF;
        const bool own = jq == jc;
        // keys the queries do not see: probabilities against the queries' lse, clamped to 1 as the reference does, enter
        // dnats only (their dV, dK products run on zeros)
        const bool only_dn = !attn_u && it >= n_same;
        // ---- first product, (32 queries) x (32 keys): LDS operands read ahead
        constexpr int AHEAD = 4;
        unsigned c1[S1];
#pragma unroll
        for (int st = 0; st < S1; ++st) { c1[st] = sb + a1[st]; asm("" : "+v"(c1[st])); }
        f32x16 x;
#pragma unroll
        for (int r = 0; r < 16; ++r) x[r] = 0.f;
        {
          bf16x8 op[S1 + AHEAD];
#pragma unroll
          for (int j = 0; j < AHEAD; ++j) op[j] = *reinterpret_cast<lds_op>(c1[j]);
#pragma unroll
          for (int j = 0; j < S1; ++j) {
            if (j + AHEAD < S1) op[j + AHEAD] = *reinterpret_cast<lds_op>(c1[j + AHEAD]);
            x = mfma32(op[j], XB[j], x);
          }
          __builtin_amdgcn_sched_group_barrier(0x100, AHEAD, 0);
#pragma unroll
          for (int j = 0; j < S1; ++j) {
            if (j + AHEAD < S1) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
          }
        }
        // the rows' lse (role 0) or delta (role 1)
        const float* Lb = reinterpret_cast<const float*>(smem + slot * SLOT + LOFF) + 64 * ROLE;
        f32x4 l4[4];
#pragma unroll
        for (int rg = 0; rg < 4; ++rg) l4[rg] = *reinterpret_cast<const f32x4*>(Lb + 32 * qh + 8 * rg + 4 * hf);
        // second product: operand j = (ss = j / T2, tile j % T2), two transposing reads each, read ahead; the first
        // ones are asked for before the barrier (the tile has been complete since the last step)
        constexpr int N2 = 2 * T2, A2 = 4 < N2 ? 4 : N2;
        unsigned ct[N2][2];
#pragma unroll
        for (int j = 0; j < N2; ++j)
#pragma unroll
          for (int rd = 0; rd < 2; ++rd) {
            ct[j][rd] = sb + t2[j / T2][j % T2][rd];
            asm("" : "+v"(ct[j][rd]));
          }
        auto tr_read = [&](const int j, const int rd) __attribute__((always_inline)) -> s16x4 {
          return __builtin_amdgcn_ds_read_tr16_b64_v4i16(reinterpret_cast<lds_tr>(ct[j][rd]));
        };
        s16x4 lo[N2 + A2], hi[N2 + A2];
        bf16x8 PB[2];
        float dsum = 0.f;
        if constexpr (ROLE == 0) {
          f32x16 pr;
          if (!own && jq * 64 + 64 <= len) {   // every (query, key) pair of the tile is visible: no masks
#pragma unroll
            for (int r = 0; r < 16; ++r) {
              float e = __builtin_amdgcn_exp2f(fmaf(x[r], c, -l4[r >> 2][r & 3]));
              if (only_dn) e = fminf(e, 1.f);
              pr[r] = e;
            }
          } else {
#pragma unroll
            for (int rg = 0; rg < 4; ++rg) {
#pragma unroll
              for (int j = 0; j < 4; ++j) {
                const int r = 4 * rg + j;
                const int qloc = 32 * qh + 8 * rg + 4 * hf + j;
                const bool vis = jq * 64 + qloc < len && (!own || 32 * kh + l32 <= qloc);
                float e = vis ? __builtin_amdgcn_exp2f(fmaf(x[r], c, -l4[rg][j])) : 0.f;
                if (only_dn) e = fminf(e, 1.f);
                pr[r] = e;
              }
            }
          }
#pragma unroll
          for (int rg = 0; rg < 4; ++rg)
            *reinterpret_cast<lds_f4>(xb + 1024 * rg) = f32x4{pr[4 * rg], pr[4 * rg + 1], pr[4 * rg + 2], pr[4 * rg + 3]};
#pragma unroll
          for (int ss = 0; ss < 2; ++ss) PB[ss] = only_dn ? bf16x8{} : pack8(pr, ss);
        }
#pragma unroll
        for (int j = 0; j < A2; ++j) {
          lo[j] = tr_read(j, 0);
          hi[j] = tr_read(j, 1);
        }
        // ---- the tile of the next step has been requested a whole step ago: once every wave has seen its own requests
        // land it is complete, and the slot of the previous step is free for the tile two steps ahead
        __builtin_amdgcn_sched_barrier(0);
        __builtin_amdgcn_s_waitcnt(0x0f70);
        __syncthreads();
        const bool ask = it + 2 < n_it;   // the tile two steps ahead goes into the slot of the previous step
        const int ask_jq = ask ? chunk_of(it + 2) : 0, ask_slot = slot == 0 ? 2 : slot - 1;
        // no tile left to ask for: the requests run with no lane enabled (read through a lane so that it sits in scalar registers)
        const unsigned ask_mask = __builtin_amdgcn_readfirstlane(ask ? 1u : 0u);
        if constexpr (ROLE == 1) {
          f32x4 p4[4];
#pragma unroll
          for (int rg = 0; rg < 4; ++rg) p4[rg] = *reinterpret_cast<lds_f4>(xb + 1024 * rg);
          f32x16 ds;
#pragma unroll
          for (int r = 0; r < 16; ++r) {
            ds[r] = p4[r >> 2][r & 3] * (x[r] - l4[r >> 2][r & 3]);
            dsum += ds[r];
          }
          if (it >= n_same && jc * 64 + 32 * kh + l32 < len) dn += dsum;
#pragma unroll
          for (int ss = 0; ss < 2; ++ss) PB[ss] = only_dn ? bf16x8{} : pack8(ds, ss);
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int j = 0; j < N2; ++j) {
          if (j + A2 < N2) {
            lo[j + A2] = tr_read(j + A2, 0);
            hi[j + A2] = tr_read(j + A2, 1);
          }
          acc[j % T2] = mfma32(join4(lo[j], hi[j]), PB[j / T2], acc[j % T2]);
          if (j < NREQ) request_piece_if(j, hq, ask_jq, ask_slot, ask_mask);   // one request under each matrix instruction
        }
#pragma unroll
        for (int j = N2; j < NREQ; ++j) request_piece_if(j, hq, ask_jq, ask_slot, ask_mask);
#pragma unroll
        for (int j = 0; j < N2; ++j) {
          if (j + A2 < N2) __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
          __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        }
        slot = slot == 2 ? 0 : slot + 1;
      }
      // dnats of this (key block, query head): the sums of role 1's four waves
      if (n_later > 0) {
        if constexpr (ROLE == 1) {
#pragma unroll
          for (int m = 32; m >= 1; m >>= 1) dn += __shfl_xor(dn, m);
          if (lane == 0) sh.red[quad] = dn;
        }
        __syncthreads();
        if (ROLE == 1 && quad == 0 && lane == 0)
          atomicAdd(p.dnats + ((size_t)(bos_nats + kb)) * p.HQ + hq, sh.red[0] + sh.red[1] + sh.red[2] + sh.red[3]);
        __syncthreads();
      }
    }

    // ---- the two query halves of a key half are summed through LDS, then the tiles are transposed and stored: role 0
    // its dV tiles, role 1 its dK tiles
    constexpr int TB = ROLE == 0 ? 0 : VT;   // this role's first tile in the order (dV tiles, dK tiles)
    __syncthreads();
    f32x4* Rs = reinterpret_cast<f32x4*>(smem);   // [2 key halves][(VT + DT) * 4 register groups][64 lanes] of 4 floats
    if (qh == 1) {
      f32x4* dst = Rs + (size_t)kh * (VT + DT) * 4 * 64 + lane;
#pragma unroll
      for (int t = 0; t < T2; ++t)
#pragma unroll
        for (int rg = 0; rg < 4; ++rg) dst[((TB + t) * 4 + rg) * 64] = f32x4{acc[t][4 * rg], acc[t][4 * rg + 1], acc[t][4 * rg + 2], acc[t][4 * rg + 3]};
    }
    __syncthreads();
    if (qh == 0) {
      // (all reads first, then the sums)
      const f32x4* src = Rs + (size_t)kh * (VT + DT) * 4 * 64 + lane;
      f32x4 xs[T2 * 4];
#pragma unroll
      for (int i = 0; i < T2 * 4; ++i) xs[i] = src[(TB * 4 + i) * 64];
      const float mul = ROLE == 0 ? 1.f : p.scale;
#pragma unroll
      for (int t = 0; t < T2; ++t)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[t][r] = (acc[t][r] + xs[t * 4 + (r >> 2)][r & 3]) * mul;
    }
    __syncthreads();
    if (qh == 0) {
      // accumulators are [value or dim rows x key columns]: write [key][value|dim] rows to LDS, then coalesced stores
      constexpr int OP = DV + DK + 8, CB = ROLE == 0 ? 0 : DV;
      bf16_t* Os = reinterpret_cast<bf16_t*>(smem) + kh * 32 * OP + CB;
#pragma unroll
      for (int t = 0; t < T2; ++t)
#pragma unroll
        for (int rg = 0; rg < 4; ++rg) {
          u32x2 w;
          w[0] = pack_bf16x2(acc[t][4 * rg], acc[t][4 * rg + 1]);
          w[1] = pack_bf16x2(acc[t][4 * rg + 2], acc[t][4 * rg + 3]);
          *reinterpret_cast<u32x2*>(Os + l32 * OP + 32 * t + 8 * rg + 4 * hf) = w;
        }
      __builtin_amdgcn_s_waitcnt(0xc07f);
      __builtin_amdgcn_wave_barrier();
      // all LDS reads first, then the stores
      constexpr int NS = 32 * (D2 / 8) / 64;
      u32x4 w2[NS];
#pragma unroll
      for (int i = 0; i < NS; ++i) {
        const int e = lane + 64 * i, row = e / (D2 / 8), seg = e % (D2 / 8);
        w2[i] = *reinterpret_cast<const u32x4*>(Os + row * OP + seg * 8);
      }
      const int t_base = jc * 64 + 32 * kh;
      bf16_t* out = ROLE == 0 ? p.dv : p.dk;
#pragma unroll
      for (int i = 0; i < NS; ++i) {
        const int e = lane + 64 * i, row = e / (D2 / 8), seg = e % (D2 / 8);
        if (t_base + row < len) *reinterpret_cast<u32x4*>(out + ((size_t)(bos + t_base + row) * p.HKV + hkv) * D2 + seg * 8) = w2[i];
      }
    }
    __syncthreads();   // the staging area is the next unit's tile ring
  }  // units
}

template <int DK, int DV>
__global__ __launch_bounds__(512, 1) void dkdv_kernel(const SoftmaxBwdParams p) {
  extern __shared__ __align__(16) unsigned char smem[];
  __shared__ DkdvShared sh;
  // (wave-uniform: each role runs the same sequence of workgroup barriers)
  if (__builtin_amdgcn_readfirstlane(threadIdx.x >> 8) == 0) dkdv_role<DK, DV, 0>(p, smem, sh);
  else dkdv_role<DK, DV, 1>(p, smem, sh);
}

// number of CUs of the current device (one persistent dk/dv workgroup each)
static int cu_count() {
  static int cached[64];
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 256;
  if (cached[dev] == 0) {
    int n = 0;
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
    cached[dev] = n;
  }
  return cached[dev];
}

template <int DK, int DV>
static int launch_bwd(const SoftmaxBwdParams& p, hipStream_t stream) {
  constexpr int KP = DK + 8, VP = DV + 8;
  const long long rows = (long long)p.B * p.T * p.HQ;
  constexpr int RPB = 256 / (DV / 8);
  hipLaunchKernelGGL((delta_kernel<DV>), dim3((unsigned)((rows + RPB - 1) / RPB)), dim3(256), 0, stream, p);
  {
    size_t lds = (size_t)2 * 64 * (KP + VP) * sizeof(bf16_t);
    auto kern = dq_kernel<DK, DV>;
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e != hipSuccess) return fail(NATSL_ERR_LAUNCH, "softmax bwd: cannot reserve %zu bytes of LDS: %s", lds, hipGetErrorString(e));
    const long long grid = p.seqs ? (long long)p.total_tiles * 2 * p.HQ : ((long long)p.B * p.HQ + 7) / 8 * 8 * ((p.T + 127) / 128);
    hipLaunchKernelGGL(kern, dim3((unsigned)grid), dim3(256), lds, stream, p);
  }
  {
    const size_t lds = DkdvLds<DK, DV>::TOTAL;   // the ring of three query tiles and the exchange buffers
    auto kern = dkdv_kernel<DK, DV>;
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e != hipSuccess) return fail(NATSL_ERR_LAUNCH, "softmax bwd: cannot reserve %zu bytes of LDS: %s", lds, hipGetErrorString(e));
    const long long units = p.seqs ? (long long)p.total_chunks * p.HKV : (long long)p.B * p.HKV * ((p.T + 63) / 64);
    long long grid = (cu_count() + 7) / 8 * 8;   // whole groups of 8: block index mod 8 names the XCD and its queue
    if (grid > units) grid = units;
    hipLaunchKernelGGL(kern, dim3((unsigned)grid), dim3(512), lds, stream, p);
  }
  return check_launch("natsl_softmax_sparse_bwd");
}

}  // namespace natsl

using namespace natsl;

// delta [B, T, HQ] fp32, then the dk/dv kernel's 8 work-queue counters
static size_t bwd_queue_offset(int B, int T, int HQ) { return ((size_t)B * T * HQ * sizeof(float) + 255) / 256 * 256; }
extern "C" size_t natsl_softmax_bwd_workspace_bytes(int B, int T, int HQ) { return bwd_queue_offset(B, T, HQ) + 256; }

extern "C" int natsl_softmax_sparse_bwd(const void* q, const void* k, const void* v, const void* o, const float* lse,
                                        const void* d_o, void* dq, void* dk, void* dv, float* dnats, const void* types,
                                        int types_dtype, const int32_t* nats_block_indices, const int32_t* n_nats_blocks,
                                        int B, int T, int HQ, int HKV, int HN, int K, int V, int TN, int block, float scale,
                                        int flags, int dtype, void* workspace, size_t workspace_bytes,
                                        const natsl_seq_row* seqs, int n_seqs, int total_tiles, int total_chunks,
                                        natsl_stream_t stream) {
  const char* what = "natsl_softmax_sparse_bwd";
  const int same_block_visible = flags & 1;
  if (!q || !k || !v || !o || !lse || !d_o || !dq || !dk || !dv || !dnats || !types || !nats_block_indices || !n_nats_blocks)
    return fail(NATSL_ERR_INVALID, "%s: null pointer argument", what);
  if (dtype != NATSL_BF16) return fail(NATSL_ERR_UNSUPPORTED, "%s: only bf16 tensors are supported (got dtype %d)", what, dtype);
  if (types_dtype != NATSL_BF16 && types_dtype != NATSL_F32) return fail(NATSL_ERR_UNSUPPORTED, "%s: block types must be f32 or bf16", what);
  if (B <= 0 || T <= 0 || HQ <= 0 || HKV <= 0 || HN <= 0 || TN <= 0) return fail(NATSL_ERR_INVALID, "%s: non-positive dimension", what);
  if (HQ % HKV || HQ % HN) return fail(NATSL_ERR_INVALID, "%s: HQ=%d must be a multiple of HKV=%d and HN=%d", what, HQ, HKV, HN);
  if (block < 64 || block % 64) return fail(NATSL_ERR_UNSUPPORTED, "%s: block size %d must be a multiple of 64", what, block);
  if (seqs ? (B != 1 || n_seqs <= 0 || total_tiles <= 0 || total_chunks <= 0) : (TN != cdiv(T, block)))
    return fail(NATSL_ERR_INVALID, "%s: TN=%d does not match T=%d, block=%d (or bad packed-input arguments)", what, TN, T, block);
  // the dk/dv kernel's DMA requests address the rows of one sequence with 32-bit byte offsets: checked here, before
  // anything is launched
  if ((long long)T * HQ * (K > V ? K : V) * 2 >= (1ll << 32))
    return fail(NATSL_ERR_UNSUPPORTED, "%s: T * HQ * max(K, V) * 2 = %lld bytes per sequence exceed the kernel's 32-bit row offsets",
                what, (long long)T * HQ * (K > V ? K : V) * 2);
  if (!workspace || workspace_bytes < natsl_softmax_bwd_workspace_bytes(B, T, HQ))
    return fail(NATSL_ERR_WORKSPACE, "%s: workspace of %zu bytes needed", what, natsl_softmax_bwd_workspace_bytes(B, T, HQ));
  SoftmaxBwdParams p;
  p.q = (const bf16_t*)q; p.k = (const bf16_t*)k; p.v = (const bf16_t*)v; p.o = (const bf16_t*)o; p.dout = (const bf16_t*)d_o;
  p.lse = lse; p.dq = (bf16_t*)dq; p.dk = (bf16_t*)dk; p.dv = (bf16_t*)dv; p.dnats = dnats; p.delta = (float*)workspace;
  p.queue = reinterpret_cast<int*>(static_cast<char*>(workspace) + bwd_queue_offset(B, T, HQ));
  p.types = types; p.types_dtype = types_dtype; p.idx = nats_block_indices; p.nblk = n_nats_blocks;
  p.B = B; p.T = T; p.HQ = HQ; p.HKV = HKV; p.HN = HN; p.TN = TN; p.block = block;
  p.seqs = reinterpret_cast<const SeqRow*>(seqs); p.n_seqs = seqs ? n_seqs : 0; p.total_tiles = total_tiles; p.total_chunks = total_chunks;
  p.scale = scale; p.scale_log2 = scale * 1.4426950408889634f; p.same_block = same_block_visible ? 1 : 0;
  p.dnats_invalid = (flags & 2) ? 1 : 0;
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
#define NATSL_SB(KK, VV) \
  if (K == KK && V == VV) return launch_bwd<KK, VV>(p, s);
  NATSL_SB(128, 128)
  NATSL_SB(64, 64)
  NATSL_SB(64, 128)
  NATSL_SB(128, 64)
#undef NATSL_SB
  return fail(NATSL_ERR_UNSUPPORTED, "%s: head dims K=%d, V=%d not built (supported: 64/128 x 64/128)", what, K, V);
}

