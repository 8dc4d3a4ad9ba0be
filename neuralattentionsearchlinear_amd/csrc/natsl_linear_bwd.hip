// Backward of the chunked linear-recurrent branches (Gated DeltaNet, Mamba2-style SSD) for gfx950.
// In function it replaces chunk_gated_delta_rule_nats_bwd (src/nats/ops/gated_delta_rule/chunk.py:170-332: dh/dv reverse
// scan chunk_delta_h.py:327+, dq/dk/dw/dg chunk_o.py:217+, the WY backward wy_fast.py) and the Mamba counterpart
// (src/nats/ops/mamba/chunk.py:112-260).
//
// Per 64-token chunk with entering state S (notation of the forward, natsl_linear.hip; q^, k^ = normalised rows):
//     gamma = cumsum g,  G = gamma_last,  L_ij = e^{gamma_i - gamma_j}
//     W = e^{gamma} k^,  Q~ = scale e^{gamma} q^,  K~ = e^{G - gamma} k^,  P = scale tril(q^ k^^T . L)
//     v_new = (1/beta + stril(k^ k^^T . L))^-1 (v - W S) = TmB (v - W S)
//     o = Q~ S + P v_new,   S' = e^G S + K~^T v_new
// Two kernels, run after a forward pass that stored S of every chunk and v_new of every token:
//
//   linear_bwd_scan_kernel   walks the chunks of one (sequence, head) BACKWARDS; a wave owns 16 columns of the state
//                            gradient for all K rows (fp32 accumulators), as the forward scan does for the state:
//                              dv_new = P^T dO + K~ dS',   dX = TmB^T dv_new   (= dv; Mamba: dX = dv_new)
//                              dS = e^G dS' + Q~^T dO - W^T dX
//                            At the end of a block that is not typed linear the forward rolled the state back to the one
//                            that entered the block (times f = e^{sum g} when decay is on): there dS' leaves the chain
//                            and f dS' is added to dS at the block's first chunk.  Stores dS' of every chunk (bf16) and dX.
//
//   linear_bwd_chunk_kernel  one workgroup per (chunk, head), fully parallel: everything else.  With
//                              N = dO v_new^T, M = dX v_new^T (64x64), Gm = scale tril(N . L), Hm = -stril(M . L):
//                              dq^ = Gm k^ + scale e^{gamma} (dO S^T)
//                              dk^ = Gm^T q^ + (Hm + Hm^T) k^ - e^{gamma} (dX S^T) + e^{G-gamma} (v_new dS'^T)
//                              dbeta_i = M_ii / beta_i^2
//                              dgamma_i = <dq^_i, q^_i> - <dk^_i, k^_i> + 2 sum_j Hm_ij (k^_i . k^_j) - 2 <e^{gamma_i} (dX S^T)_i, k^_i>
//                              dG = <e^{G-gamma} (v_new dS'^T), k^> + e^G <dS', S>;   dg_t = sum_{i >= t} dgamma_i + dG
//                            followed by the backward of the row normalisation.  <e^{G-gamma}(v_new dS'^T), k^> is also the
//                            derivative with respect to a gate on the chunk's state update: the selector's straight-through
//                            gradient for the linear operator (src/nats/ops/common/chunk_o.py:438-443, :487-492).
//
// The reverse scan takes a chunk's inputs as the forward scan does: raw q, k rows, and TmB, P and the scale vectors (which
// carry the reciprocal row norms) from the forward's workspace, all by LDS-DMA into a two-stage ring.  The per-chunk kernel
// rebuilds q^, k^ and the decay vectors from q, k, g; its tiles sit in LDS row-major as they lie in memory.  An operand that
// needs the other orientation (k^T, q^T, S, dS', TmB^T, P^T) is fetched with the transposing read ds_read_b64_tr_b16 (within
// 16 lanes, lane i names four consecutive elements R_i and receives element i % 4 of R_{i/4}, R_{4+i/4}, R_{8+i/4},
// R_{12+i/4}): two such reads are the eight contraction slots of a lane.
#include "natsl_device.h"
#include "natsl_host.h"

namespace natsl {

struct LinBwdParams {
  const bf16_t* q;
  const bf16_t* k;
  const bf16_t* vn;       // v_new [tokens][H][V] (Mamba: v)
  const bf16_t* d_o;      // [tokens][H][V]
  const float* g;
  const bf16_t* beta;
  const bf16_t* s_all;    // state entering every chunk, [chunk][H][V][K]
  bf16_t* ds_all;         // gradient of the state behind every chunk, same layout (written by the scan)
  bf16_t* dv;             // dX [tokens][H][V] (written by the scan)
  const float* dht;       // [B][H][K][V] or null
  float* dh0;             // [B][H][K][V] or null
  const float* gsum_blk;  // sum of g over every selector block, [B][TN][H]
  const bf16_t* ws_tm;    // the forward's workspace: TmB of every chunk-head in the forward scan's operand order,
  const bf16_t* ws_p;     // P likewise,
  const float* ws_sc;     // and the four scale vectors
  const void* types;
  int types_dtype;
  bf16_t* dq;
  bf16_t* dk;
  float* dg;              // [tokens][H]
  float* dbeta;           // [tokens][H]
  float* dbeta_parts;     // [tokens][H][V / 16]: <dX, v_new> over each wave's 16 columns (scan -> per-chunk kernel)
  float* gate;            // [chunk][H]: derivative with respect to a gate on the chunk's state update
  float* rb;              // [chunk][H]: f <dS', S_blockstart> behind a rolled-back block's last chunk (the decay's share of dg)
  const SeqRow* seqs;     // packed sequences (B = 1), or null
  int n_seqs, total_chunks;
  int B, T, H, HN, V, TN, block, nt;
  float scale;
  int flags;
};

constexpr int CB = 64;          // tokens per chunk
constexpr int TP = CB + 8;      // row pitch (elements) of the 64-wide bf16 tiles

NATSL_DEVICE bool lin_type_b(const void* types, int dtype, size_t i) {
  float x = dtype == NATSL_F32 ? reinterpret_cast<const float*>(types)[i]
                               : bf16_to_f32(reinterpret_cast<const bf16_t*>(types)[i]);
  return rintf(x) == 1.0f;
}

NATSL_DEVICE void unpack8f(const u32x4 w, float* f) {
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    f[2 * j] = __uint_as_float(w[j] << 16);
    f[2 * j + 1] = __uint_as_float(w[j] & 0xffff0000u);
  }
}

// two 8-byte halves -> one operand: slots 0..3 from lo, 4..7 from hi
NATSL_DEVICE bf16x8 join_u2(const u32x2 lo, const u32x2 hi) {
  u32x4 w = {lo[0], lo[1], hi[0], hi[1]};
  return __builtin_bit_cast(bf16x8, w);
}

// What rounding 8 fp32 to a bf16 operand leaves behind, as a second operand: a product with {pack8(a, b), pack8_rest(a, b)}
// carries the fp32 values to about 16 bits.
NATSL_DEVICE bf16x8 pack8_rest(const f32x4 a, const f32x4 b) {
  f32x4 ra, rb;
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    ra[r] = a[r] - __uint_as_float(__float_as_uint(a[r]) & 0xffff0000u);
    rb[r] = b[r] - __uint_as_float(__float_as_uint(b[r]) & 0xffff0000u);
  }
  return pack8(ra, rb);
}
// (the first operand then has to be the TRUNCATED value, not the rounded one)
NATSL_DEVICE bf16x8 pack8_trunc(const f32x4 a, const f32x4 b) {
  u32x4 w;
  w[0] = (__float_as_uint(a[0]) >> 16) | (__float_as_uint(a[1]) & 0xffff0000u);
  w[1] = (__float_as_uint(a[2]) >> 16) | (__float_as_uint(a[3]) & 0xffff0000u);
  w[2] = (__float_as_uint(b[0]) >> 16) | (__float_as_uint(b[1]) & 0xffff0000u);
  w[3] = (__float_as_uint(b[2]) >> 16) | (__float_as_uint(b[3]) & 0xffff0000u);
  return __builtin_bit_cast(bf16x8, w);
}

// {M[rowA + j][c0 + x] : j < 4} and {M[rowB + j][c0 + x] : j < 4} for lane x of a 16-lane group, M row-major in LDS with
// `pitch` elements per row: the transposed operand of a 16x16x32 matrix instruction (x = the operand's row or column,
// rowA.. and rowB.. = the lane group's eight contraction slots).
NATSL_DEVICE bf16x8 tr_operand(const bf16_t* base, const int pitch, const int rowA, const int rowB, const int c0, const int x16) {
  const int off = (x16 >> 2) * pitch + c0 + 4 * (x16 & 3);
  return join4(lds_tr4(base + rowA * pitch + off), lds_tr4(base + rowB * pitch + off));
}

// q^, k^ rows of a chunk: what a thread fetches (row tid / 4, 16-byte pieces tid % 4 + 4 i) and, normalised, puts into LDS
template <int DK>
struct QkRegs {
  u32x4 a[DK / 32], b[DK / 32];
};

template <int DK>
NATSL_DEVICE void load_qk(const LinBwdParams& p, const int tid, const size_t row0, const int nvalid, const int h, QkRegs<DK>& r) {
  const int row = tid >> 2, sub = tid & 3;
  const bool ok = row < nvalid;
  const size_t off = ((row0 + row) * p.H + h) * DK;
  const u32x4 z = {0u, 0u, 0u, 0u};
#pragma unroll
  for (int i = 0; i < DK / 32; ++i) {
    r.a[i] = ok ? *reinterpret_cast<const u32x4*>(p.q + off + (sub + 4 * i) * 8) : z;
    r.b[i] = ok ? *reinterpret_cast<const u32x4*>(p.k + off + (sub + 4 * i) * 8) : z;
  }
}

// rows past the end of the sequence arrive as zeros
template <int DK>
NATSL_DEVICE void store_qk(const QkRegs<DK>& r, const int tid, const bool l2, bf16_t* Qn, bf16_t* Kn, float* rq, float* rk) {
  constexpr int KP = DK + 8, KL = DK / 32;
  const int row = tid >> 2, sub = tid & 3;
  float sq = 0.f, sk = 0.f;
#pragma unroll
  for (int i = 0; i < KL; ++i) {
    float fa[8], fb[8];
    unpack8f(r.a[i], fa);
    unpack8f(r.b[i], fb);
#pragma unroll
    for (int e = 0; e < 8; ++e) { sq += fa[e] * fa[e]; sk += fb[e] * fb[e]; }
  }
  sq += __shfl_xor(sq, 1); sq += __shfl_xor(sq, 2);
  sk += __shfl_xor(sk, 1); sk += __shfl_xor(sk, 2);
  const float fq = l2 ? rsqrtf(sq + 1e-6f) : 1.f, fk = l2 ? rsqrtf(sk + 1e-6f) : 1.f;
  if (sub == 0) { rq[row] = fq; rk[row] = fk; }
#pragma unroll
  for (int i = 0; i < KL; ++i) {
    const int seg = sub + 4 * i;
    float fa[8], fb[8];
    unpack8f(r.a[i], fa);
    unpack8f(r.b[i], fb);
    u32x4 wa, wb;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      wa[j] = pack_bf16x2(fa[2 * j] * fq, fa[2 * j + 1] * fq);
      wb[j] = pack_bf16x2(fb[2 * j] * fk, fb[2 * j + 1] * fk);
    }
    *reinterpret_cast<u32x4*>(Qn + row * KP + seg * 8) = wa;
    *reinterpret_cast<u32x4*>(Kn + row * KP + seg * 8) = wb;
  }
}

// 64 rows x 64 columns of a token-major [tokens][H][V] tensor: a thread's two 16-byte pieces (rows past the end: zeros)
NATSL_DEVICE void load_tokens64(const bf16_t* src, const int tid, const size_t row0, const int nvalid, const int H, const int V,
                                const int h, const int vcol0, u32x4* w) {
  const u32x4 z = {0u, 0u, 0u, 0u};
#pragma unroll
  for (int it = 0; it < 2; ++it) {
    const int pc = tid + 256 * it, row = pc >> 3, seg = pc & 7;
    w[it] = row < nvalid ? *reinterpret_cast<const u32x4*>(src + ((row0 + row) * H + h) * V + vcol0 + seg * 8) : z;
  }
}
NATSL_DEVICE void store_tokens64(const u32x4* w, const int tid, bf16_t* dst) {
#pragma unroll
  for (int it = 0; it < 2; ++it) {
    const int pc = tid + 256 * it, row = pc >> 3, seg = pc & 7;
    *reinterpret_cast<u32x4*>(dst + row * TP + seg * 8) = w[it];
  }
}

// The chunk's scalars from g (and beta) of the wave's lanes = tokens: gamma (inclusive cumsum of g), e^gamma, e^{G - gamma}
// (Mamba: exponent clamped at 0), scale e^gamma, beta.  Tokens past the end carry g = 0, beta = 0.
template <bool DELTA>
NATSL_DEVICE void store_scalars(const int lane, float x, const float b, const float scale, float* gam, float* eg, float* ek, float* sqv,
                                float* bet) {
#pragma unroll
  for (int d = 1; d < 64; d <<= 1) {
    const float y = __shfl_up(x, d);
    if (lane >= d) x += y;
  }
  const float gl = __shfl(x, 63);
  float dk = gl - x;
  if (!DELTA) dk = fminf(dk, 0.f);
  const float e = __expf(x);
  gam[lane] = x;
  eg[lane] = e;
  ek[lane] = __expf(dk);
  sqv[lane] = scale * e;
  if (DELTA) bet[lane] = b;
}

// =============================================================================================
// reverse scan
// =============================================================================================
// one DMA instruction: lane l copies 16 bytes from base + voff to LDS byte address lds + 16 l
NATSL_DEVICE void dma16(const void* base, const unsigned voff, const unsigned lds) {
  asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1" ::"v"(voff), "s"(base), "s"(lds) : "memory", "m0");
}

// Swizzle of the raw k / q tiles (row-major, unpadded rows of DK bf16; the forward scan's): 16-byte segment s of row r sits at
// s ^ kq_swz(r), so that the row reads (16 lanes = 16 consecutive rows at one segment) and the transposing reads (16 lanes =
// 4 consecutive rows x 4 segments of an aligned group) both fall on 16 different 16-byte slots of the 256-byte bank period.
template <int DK>
NATSL_DEVICE int kq_swz(const int r) {
  if constexpr (DK == 128) return ((r & 3) << 2) | ((r >> 2) & 3);
  return (r >> 1) & 7;
}
// the 64-column dO / v_new tiles (rows of 128 bytes): rows two apart share banks
NATSL_DEVICE int v_swz(const int r) { return 2 * ((r >> 1) & 1); }

typedef __attribute__((address_space(3))) const bf16x8* lds_b128_t;
typedef __attribute__((address_space(3))) const f32x4* lds_f4_t;
typedef __attribute__((address_space(3))) const float* lds_f1_t;
typedef __attribute__((address_space(3))) s16x4* lds_tr_t;
typedef __attribute__((address_space(3))) bf16_t* lds_h_t;
typedef __attribute__((address_space(3))) bf16x8* lds_w128_t;

NATSL_DEVICE s16x4 lds_tr4_at(const unsigned addr) {
  return __builtin_amdgcn_ds_read_tr16_b64_v4i16(reinterpret_cast<lds_tr_t>(addr));
}
// x of another lane of the row, chosen by a data-parallel-primitive control word (row mirror 0x140, half-row mirror 0x141,
// quad permutations 0x00..0xff)
template <int CTRL>
NATSL_DEVICE float lane_mirror(const float x) {
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), CTRL, 0xf, 0xf, true));
}
NATSL_DEVICE float uniform_f(const float x) {
  return __builtin_bit_cast(float, __builtin_amdgcn_readfirstlane(__builtin_bit_cast(int, x)));
}
// index of operand (t, s) of TmB / P among the six that are stored (the two above the diagonal are skipped)
NATSL_DEVICE constexpr int tri_slot(const int t, const int s) { return t < 2 ? t : 2 * t - 2 + s; }

// LDS of the reverse scan: two stages, each one chunk's inputs exactly as they lie in memory (filled by LDS-DMA).
template <int DK, int NW>
struct BwdScanLds {
  static_assert(NW == 4 || (NW == 2 && DK <= 128), "four compute waves, or two where a fifth wave moves the data");
  static constexpr int KROW = DK * 2, VROW = 32 * NW;    // bytes per k / q row, per dO / v_new row (16 NW columns)
  static constexpr int KB = CB * KROW, VB = CB * VROW, TB = 6 * 1024, SCB = 1024;
  static constexpr int OFF_K = 0, OFF_Q = OFF_K + KB, OFF_DO = OFF_Q + KB, OFF_VN = OFF_DO + VB, OFF_T = OFF_VN + VB,
                       OFF_P = OFF_T + TB, OFF_SC = OFF_P + TB;
  static constexpr int STAGE = OFF_SC + SCB;
  // Up to K = 128 a fifth wave does nothing but issue the requests (it shares a SIMD with a compute wave, so every wave has
  // to fit 256 registers: for K = 128 the held-back state gradient of a rolled-back block waits in LDS instead of
  // registers); K = 192 has neither the registers nor the LDS for that, and its compute waves issue the requests themselves.
  static constexpr bool DMAW = DK <= 128, PEND_LDS = DK == 128;
  static constexpr int PEND = (DK / 16) * 4 * 64 * 4;    // bytes per wave
  static constexpr int TOTAL = 2 * STAGE + (PEND_LDS ? NW * PEND : 0);
  static constexpr int THREADS = 64 * (DMAW ? NW + 1 : NW);
};

// The inputs of a chunk are the forward scan's: raw q, k rows (the reciprocal norms ride in the scale vectors), the prep
// kernel's TmB, P and scale vectors {se = e^gamma rk, sq = scale rq e^gamma, sk = rk e^{G-gamma}, {e^G, G, is_linear}} from
// the workspace (Mamba: {gamma log2 e, scale e^gamma, e^{min(G-gamma,0)}, ...}; no TmB, P), plus dO and v_new.  Every wave
// requests its share of chunk c - 1 by LDS-DMA right after the barrier that opens chunk c; nothing is staged in registers.
// The state gradient uses the forward scan's row order: tile m, lane group g, register r hold K row
// 32 (m / 2) + 8 g + 4 (m % 2) + r, so that two tiles side by side are eight consecutive K rows (one 16-byte piece of a k / q
// row as the A operand of K~ dS', one 16-byte store of dS').
template <int DK, bool DELTA, int NW>
__global__ __launch_bounds__((BwdScanLds<DK, NW>::THREADS)) void linear_bwd_scan_kernel(const LinBwdParams p) {
  using L = BwdScanLds<DK, NW>;
  constexpr int KT = DK / 16, KS = DK / 32;
  constexpr bool DMAW = L::DMAW, PEND_LDS = L::PEND_LDS;
  extern __shared__ __align__(1024) unsigned char smem[];
  const unsigned lds0 = (unsigned)(size_t)smem;

  const int tid = threadIdx.x, lane = tid & 63, x16 = lane & 15, g4 = lane >> 4;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  // the column slices of one chain sit on one XCD (workgroup ids go round the eight XCDs): what they share -- q, k, TmB,
  // P -- is then fetched from HBM once
  const int nsplit = p.V / (16 * NW);
  const int n_chains = (p.seqs ? p.n_seqs : p.B) * p.H;
  const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3;
  const int split = slot % nsplit, chain = (slot / nsplit) * 8 + xcd;
  if (chain >= n_chains) return;
  const int n = chain / p.H, h = chain % p.H;
  int bos, len, chunk_off, blk0;   // first token, length, first chunk and first selector block of the sequence
  if (p.seqs == nullptr) {
    bos = n * p.T; len = p.T; chunk_off = n * p.nt; blk0 = n * p.TN;
  } else {
    bos = p.seqs[n].bos; len = p.seqs[n].eos - bos; chunk_off = p.seqs[n].chunk_off; blk0 = p.seqs[n].bos_nats;
  }
  const int NT = (len + CB - 1) / CB;
  const int vcol0 = split * (16 * NW);
  const int col = vcol0 + 16 * wave + x16;
  const int per = p.block / CB;
  const bool decay = (p.flags & NATSL_DECAY_NON_LINEAR) != 0, intra = (p.flags & NATSL_INTRA_CHUNK) != 0;

  auto krow_of = [&](const int m, const int r) { return 32 * (m >> 1) + 8 * g4 + 4 * (m & 1) + r; };
  f32x4 dS[KT], pend[PEND_LDS ? 1 : KT];
  typedef __attribute__((address_space(3))) float* lds_wf_t;
  const unsigned a_pend = lds0 + 2 * L::STAGE + (wave % NW) * L::PEND + 4 * lane;   // value (m, r) of this lane at + 256 (4 m + r)
  if (wave < NW) {
#pragma unroll
    for (int m = 0; m < KT; ++m)
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        dS[m][r] = p.dht ? p.dht[((size_t)chain * DK + krow_of(m, r)) * p.V + col] : 0.f;
        if (!PEND_LDS) pend[m][r] = 0.f;
      }
  }
  if (NT <= 0) return;

  // ---- requests: piece u of a tile covers its LDS bytes [1024 u, 1024 u + 1024); lane l fills byte 1024 u + 16 l, i.e. some
  //      row and 16-byte position of the tile, from the source segment position ^ swizzle(row); wave w moves pieces w, w + 4, ..
  const size_t qk_pitch = (size_t)p.H * DK * 2, v_pitch = (size_t)p.H * p.V * 2;   // bytes per token
  constexpr int KQ_PER = L::KB / 1024 / 4, V_PER = L::VB / 1024 / 4;
  unsigned kq_off[KQ_PER], v_off[V_PER];
  auto set_offsets = [&](const int nvalid) __attribute__((always_inline)) {
    // (rows past the end of the sequence: the last valid row once more; what they produce is never stored and meets zero weights)
#pragma unroll
    for (int j = 0; j < KQ_PER; ++j) {
      const int byte = 1024 * (wave + 4 * j) + 16 * lane, row = byte / L::KROW, pos = (byte % L::KROW) / 16;
      kq_off[j] = (unsigned)((size_t)min(row, nvalid - 1) * qk_pitch) + 16u * (unsigned)(pos ^ kq_swz<DK>(row));
    }
#pragma unroll
    for (int j = 0; j < V_PER; ++j) {
      const int byte = 1024 * (wave + 4 * j) + 16 * lane, row = byte / L::VROW, pos = (byte % L::VROW) / 16;
      v_off[j] = (unsigned)((size_t)min(row, nvalid - 1) * v_pitch) + 16u * (unsigned)(pos ^ v_swz(row));
    }
  };
  if constexpr (DMAW) {
    if (wave == NW) {
      // ======================= the data-movement wave: all requests of chunk c - 1 during step c =======================
      // (the CU's memory pipe takes one 1 KiB request per ~44 cycles, 61 KiB per chunk: a compute wave that issues them
      // waits for the pipe; this wave has nothing else to do)
      constexpr int KQ_ALL = L::KB / 1024, V_ALL = L::VB / 1024;
      unsigned ko[KQ_ALL], vo[V_ALL], wo[6];
      auto offsets = [&](const int nvalid) __attribute__((always_inline)) {
#pragma unroll
        for (int u = 0; u < KQ_ALL; ++u) {
          const int byte = 1024 * u + 16 * lane, row = byte / L::KROW, pos = (byte % L::KROW) / 16;
          ko[u] = (unsigned)((size_t)min(row, nvalid - 1) * qk_pitch) + 16u * (unsigned)(pos ^ kq_swz<DK>(row));
        }
#pragma unroll
        for (int u = 0; u < V_ALL; ++u) {
          const int byte = 1024 * u + 16 * lane, row = byte / L::VROW, pos = (byte % L::VROW) / 16;
          vo[u] = (unsigned)((size_t)min(row, nvalid - 1) * v_pitch) + 16u * (unsigned)(pos ^ v_swz(row));
        }
      };
#pragma unroll
      for (int v = 0; v < 6; ++v) wo[v] = 16u * lane + 1024u * (v < 2 ? 2 * v : v + 2);
      auto request_all = [&](const int cc) __attribute__((always_inline)) {
        const unsigned st = lds0 + (cc & 1) * L::STAGE;
        const size_t tok = ((size_t)bos + (size_t)cc * CB) * p.H + h;
        const size_t unit = (size_t)(chunk_off + cc) * p.H + h;
        // in the order the compute waves need them: scale vectors, k, dO, P, TmB, v_new, q
        dma16(p.ws_sc + unit * (4 * CB), 16u * lane, st + L::OFF_SC);
        const char* kb = reinterpret_cast<const char*>(p.k + tok * DK);
#pragma unroll
        for (int u = 0; u < KQ_ALL; ++u) dma16(kb, ko[u], st + L::OFF_K + 1024 * u);
        const char* dob = reinterpret_cast<const char*>(p.d_o + tok * p.V + vcol0);
#pragma unroll
        for (int u = 0; u < V_ALL; ++u) dma16(dob, vo[u], st + L::OFF_DO + 1024 * u);
        if (DELTA) {
          if (intra) {
            const char* pb = reinterpret_cast<const char*>(p.ws_p + unit * (CB * CB));
#pragma unroll
            for (int v = 0; v < 6; ++v) dma16(pb, wo[v], st + L::OFF_P + 1024 * v);
          }
          const char* tb = reinterpret_cast<const char*>(p.ws_tm + unit * (CB * CB));
#pragma unroll
          for (int v = 0; v < 6; ++v) dma16(tb, wo[v], st + L::OFF_T + 1024 * v);
          const char* vnb = reinterpret_cast<const char*>(p.vn + tok * p.V + vcol0);
#pragma unroll
          for (int u = 0; u < V_ALL; ++u) dma16(vnb, vo[u], st + L::OFF_VN + 1024 * u);
        }
        const char* qb = reinterpret_cast<const char*>(p.q + tok * DK);
#pragma unroll
        for (int u = 0; u < KQ_ALL; ++u) dma16(qb, ko[u], st + L::OFF_Q + 1024 * u);
      };
      const int nlast = min(CB, len - (NT - 1) * CB);
      offsets(nlast);
      request_all(NT - 1);
      if (nlast < CB) offsets(CB);
      for (int c = NT - 1; c >= 0; --c) {
        __builtin_amdgcn_s_waitcnt(0x0f70);   // chunk c has landed
        __syncthreads();                      // .. and every compute wave is done with the other stage
        if (c > 0) request_all(c - 1);
        if (!DELTA && intra) __syncthreads();   // (the compute waves' exchange of P^T)
      }
      return;
    }
  }
  // TmB / P: six 1 KiB operands each (stored at 0, 2, 4..7 of eight), plain copies; wave w moves operands w and w + 4
  const unsigned ws_off0 = 16u * lane + 1024u * (wave < 2 ? 2 * wave : wave + 2), ws_off1 = 16u * lane + 1024u * (wave + 6);
  // The CU's memory pipe takes one such 1 KiB instruction per ~44 cycles (61 KiB per chunk: 2 800 cycles), and a wave that
  // issues its 16 in one go waits for all of them to be accepted; so a chunk's requests are spread over the step in groups
  // (request<G>(cc), G = 0..NGROUPS-1), each small enough to find the pipe free.
  constexpr int NGROUPS = 7;
  const char *rq_k = nullptr, *rq_q = nullptr, *rq_do = nullptr, *rq_vn = nullptr, *rq_t = nullptr, *rq_p = nullptr, *rq_sc = nullptr;
  auto request_bases = [&](const int cc) __attribute__((always_inline)) {
    const size_t tok = ((size_t)bos + (size_t)cc * CB) * p.H + h;
    const size_t unit = (size_t)(chunk_off + cc) * p.H + h;
    rq_k = reinterpret_cast<const char*>(p.k + tok * DK);
    rq_q = reinterpret_cast<const char*>(p.q + tok * DK);
    rq_do = reinterpret_cast<const char*>(p.d_o + tok * p.V + vcol0);
    rq_vn = reinterpret_cast<const char*>(p.vn + tok * p.V + vcol0);
    rq_t = reinterpret_cast<const char*>(p.ws_tm + unit * (CB * CB));
    rq_p = reinterpret_cast<const char*>(p.ws_p + unit * (CB * CB));
    rq_sc = reinterpret_cast<const char*>(p.ws_sc + unit * (4 * CB));
  };
  auto request = [&](const int grp, const int cc) __attribute__((always_inline)) {
    const unsigned st = lds0 + (cc & 1) * L::STAGE;
    constexpr int KH = (KQ_PER + 1) / 2;
    if (grp == 0) {
      if (wave == 3) dma16(rq_sc, 16u * lane, st + L::OFF_SC);
#pragma unroll
      for (int j = 0; j < KH; ++j) dma16(rq_k, kq_off[j], st + L::OFF_K + 1024 * (wave + 4 * j));
    } else if (grp == 1) {
#pragma unroll
      for (int j = KH; j < KQ_PER; ++j) dma16(rq_k, kq_off[j], st + L::OFF_K + 1024 * (wave + 4 * j));
    } else if (grp == 2) {
#pragma unroll
      for (int j = 0; j < V_PER; ++j) dma16(rq_do, v_off[j], st + L::OFF_DO + 1024 * (wave + 4 * j));
    } else if (grp == 3) {
      if (DELTA && intra) {
        dma16(rq_p, ws_off0, st + L::OFF_P + 1024 * wave);
        if (wave < 2) dma16(rq_p, ws_off1, st + L::OFF_P + 1024 * (wave + 4));
      }
    } else if (grp == 4) {
      if (DELTA) {
        dma16(rq_t, ws_off0, st + L::OFF_T + 1024 * wave);
        if (wave < 2) dma16(rq_t, ws_off1, st + L::OFF_T + 1024 * (wave + 4));
      }
    } else if (grp == 5) {
      if (DELTA) {
#pragma unroll
        for (int j = 0; j < V_PER; ++j) dma16(rq_vn, v_off[j], st + L::OFF_VN + 1024 * (wave + 4 * j));
      }
#pragma unroll
      for (int j = 0; j < KH; ++j) dma16(rq_q, kq_off[j], st + L::OFF_Q + 1024 * (wave + 4 * j));
    } else {
#pragma unroll
      for (int j = KH; j < KQ_PER; ++j) dma16(rq_q, kq_off[j], st + L::OFF_Q + 1024 * (wave + 4 * j));
    }
  };

  // ---- per-lane operand addresses inside a stage (the forward scan's) -----------------------------------------------------
  // k / q rows as an operand (token tile t, k-step s): row 16 t + x16, segment 4 s + g4; t goes into the offset
  unsigned a_kq[KS];
#pragma unroll
  for (int s = 0; s < KS; ++s) a_kq[s] = (unsigned)(x16 * L::KROW) + 16u * (unsigned)((4 * s + g4) ^ kq_swz<DK>(x16));
  // q^T / k^T as A operand (state tile m, token k-step s2, read rd): lane x16 names token 32 s2 + 16 rd + 4 g4 + x16 / 4 and
  // the four K rows 32 (m / 2) + 8 (x16 % 4) + 4 (m % 2) ..: segment 4 (m / 2) + x16 % 4, half m % 2
  unsigned a_kt[KT / 2];
  {
    const int tk = 4 * g4 + (x16 >> 2);
#pragma unroll
    for (int mh = 0; mh < KT / 2; ++mh)
      a_kt[mh] = (unsigned)(tk * L::KROW) + 16u * (unsigned)((4 * mh + (x16 & 3)) ^ kq_swz<DK>(tk));
  }
  // dO / v_new through the transposing read (token tile t): lane x16 names token 16 t + 4 g4 + x16 / 4, columns
  // 16 wave + 4 (x16 % 4) ..; it receives tokens 16 t + 4 g4 + 0..3 of column 16 wave + x16 (the accumulator layout)
  unsigned a_v;
  {
    const int tk = 4 * g4 + (x16 >> 2), seg = 2 * wave + ((x16 & 3) >> 1);
    a_v = (unsigned)(tk * L::VROW) + 16u * (unsigned)(seg ^ v_swz(tk)) + 8u * (x16 & 1);
  }
  // TmB^T / P^T as A operand: element (row i, column cc) of the stored matrix sits in operand (i / 16, cc / 32), lane slot
  // 16 ((cc % 16) / 4) + i % 16, element 4 ((cc % 32) / 16) + cc % 4: four consecutive columns are contiguous, so the
  // transposing read applies with "rows" = lane slots; lane x16 names slot 16 (x16 % 4) + 4 g4 + x16 / 4
  const unsigned a_tm = 16u * (unsigned)(16 * (x16 & 3) + 4 * g4 + (x16 >> 2));
  const unsigned a_sc = 16u * g4;    // this lane group's four tokens in a row of the scale vectors

  {
    const int nlast = min(CB, len - (NT - 1) * CB);
    if constexpr (!DMAW) {
      set_offsets(nlast);
      request_bases(NT - 1);
#pragma unroll
      for (int grp = 0; grp < NGROUPS; ++grp) request(grp, NT - 1);
      if (nlast < CB) set_offsets(CB);
    }
  }
  float gs_next = p.gsum_blk[((size_t)blk0 + ((NT - 1) * CB) / p.block) * p.H + h];
  bool have_pend = false;

  for (int c = NT - 1; c >= 0; --c) {
    const unsigned st = lds0 + (c & 1) * L::STAGE;
    const int t0 = c * CB, nvalid = min(CB, len - t0);
    const size_t row0 = (size_t)bos + t0;
    // chunk c has landed (a wave's vector memory operations complete in order) and every wave is done with the other stage
    if constexpr (!DMAW) __builtin_amdgcn_s_waitcnt(0x0f70);
    __syncthreads();
    const float gs_r = gs_next;
    const bool more = !DMAW && c > 0;     // (requests from the compute waves)
    if (more) {
      request_bases(c - 1);
      request(0, c - 1);
    }
    const float dec = uniform_f(*reinterpret_cast<lds_f1_t>(st + L::OFF_SC + 4 * (3 * CB)));
    const bool lin = uniform_f(*reinterpret_cast<lds_f1_t>(st + L::OFF_SC + 4 * (3 * CB + 2))) != 0.f;
    const float f_blk = decay ? __expf(gs_r) : 1.f;
    // dS' of this chunk as it arrived: it goes out at the end of the step (every global store of the compute waves does: right
    // after the barrier the CU's memory pipe is busy with the requests for the next chunk, and a store would wait behind them)
    bf16x8 DSB[KS];
#pragma unroll
    for (int s = 0; s < KS; ++s) DSB[s] = pack8(dS[2 * s], dS[2 * s + 1]);
    // ---- a rolled-back block's dS' leaves the chain here ---------------------------------------------------------------
    const bool last = ((c + 1) % per == 0) || (c == NT - 1);
    // (pend is zero here: it was handed over at the first chunk of the block behind this one)
    if (last && !lin) {
#pragma unroll
      for (int m = 0; m < KT; ++m)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          if constexpr (PEND_LDS) *reinterpret_cast<lds_wf_t>(a_pend + 256 * (4 * m + r)) = dS[m][r] * f_blk;
          else pend[m][r] = dS[m][r] * f_blk;
          dS[m][r] = 0.f;
        }
      have_pend = true;
    }
    if (more) request(1, c - 1);

    // ---- Y1 = K~ dS' ----------------------------------------------------------------------------------------------------
    f32x4 DV[4];
#pragma unroll
    for (int t = 0; t < 4; ++t) DV[t] = (f32x4){0.f, 0.f, 0.f, 0.f};
    if (!(last && !lin)) {   // (behind a rolled-back block dS' is zero)
#pragma unroll
      for (int s = 0; s < KS; ++s)
#pragma unroll
        for (int t = 0; t < 4; ++t)
          DV[t] = mfma16(*reinterpret_cast<lds_b128_t>(st + L::OFF_K + a_kq[s] + t * 16 * L::KROW), DSB[s], DV[t]);
#pragma unroll
      for (int t = 0; t < 4; ++t) {
        const f32x4 e4 = *reinterpret_cast<lds_f4_t>(st + L::OFF_SC + 4 * (2 * CB) + a_sc + 64 * t);
#pragma unroll
        for (int r = 0; r < 4; ++r) DV[t][r] *= e4[r];
      }
    }
    if (more) request(2, c - 1);
    // ---- dO in accumulator layout (lane = column, registers = tokens 16 t + 4 g + r); zero past the end of the sequence ----
    f32x4 DOc[4];
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      const s16x4 w = lds_tr4_at(st + L::OFF_DO + a_v + t * 16 * L::VROW);
#pragma unroll
      for (int r = 0; r < 4; ++r) DOc[t][r] = bf16_to_f32((bf16_t)w[r]);
    }
    if (__builtin_expect(nvalid < CB, 0)) {
      asm volatile("" ::: "memory");   // (keeps this a branch: it runs once per chain)
#pragma unroll
      for (int t = 0; t < 4; ++t)
#pragma unroll
        for (int r = 0; r < 4; ++r)
          if (16 * t + 4 * g4 + r >= nvalid) DOc[t][r] = 0.f;
    }
    if (more) request(3, c - 1);
    // ---- Y2 = P^T dO ----------------------------------------------------------------------------------------------------
    if (intra) {
      const bf16x8 DOB[2] = {pack8(DOc[0], DOc[1]), pack8(DOc[2], DOc[3])};
      if constexpr (DELTA) {
        // P as the prep kernel stored it, read transposed (see a_tm): rows i = 32 s2 + 16 hf + 4 g + j of column 16 tj + x
#pragma unroll
        for (int tj = 0; tj < 4; ++tj)
#pragma unroll
          for (int s2 = 0; s2 < 2; ++s2)
            if (2 * s2 + 1 >= tj) {
              const unsigned lo = st + L::OFF_P + 1024 * tri_slot(2 * s2, tj >> 1) + a_tm + 8 * (tj & 1);
              const unsigned hi = st + L::OFF_P + 1024 * tri_slot(2 * s2 + 1, tj >> 1) + a_tm + 8 * (tj & 1);
              DV[tj] = mfma16(join4(lds_tr4_at(lo), lds_tr4_at(hi)), DOB[s2], DV[tj]);
            }
      } else {
        // P^T formed here, once per workgroup: Z = q k^T leaves lane (x, g) with key 16 tj + x against queries
        // 16 ti + 4 g + r, the four slots this lane holds of operand (tj, ti / 2), half ti % 2.  Operand (tj, s2) at index
        // tj < 2 ? 2 tj + s2 : 2 + tj; waves 0..3 form {(0,0), (1,0)}, {(0,1), (3,1)}, {(1,1)}, {(2,1)}: 3, 3, 2, 2 tiles.
        auto make_operand = [&](const int tj, const int s2) __attribute__((always_inline)) {
          const float gj = *reinterpret_cast<lds_f1_t>(st + L::OFF_SC + 4 * (16 * tj + x16));   // gamma in log2 units
          f32x4 Z[2];
#pragma unroll
          for (int hf = 0; hf < 2; ++hf) {
            const int ti = 2 * s2 + hf;
            Z[hf] = (f32x4){0.f, 0.f, 0.f, 0.f};
            if (ti >= tj) {
#pragma unroll
              for (int s = 0; s < KS; ++s) {
                const bf16x8 a = *reinterpret_cast<lds_b128_t>(st + L::OFF_Q + a_kq[s] + ti * 16 * L::KROW);
                const bf16x8 b = *reinterpret_cast<lds_b128_t>(st + L::OFF_K + a_kq[s] + tj * 16 * L::KROW);
                Z[hf] = mfma16(a, b, Z[hf]);
              }
              const f32x4 gi = *reinterpret_cast<lds_f4_t>(st + L::OFF_SC + a_sc + 64 * ti);
#pragma unroll
              for (int r = 0; r < 4; ++r) {
                const bool vis = ti > tj || 4 * g4 + r >= x16;
                Z[hf][r] = vis ? Z[hf][r] * p.scale * __builtin_amdgcn_exp2f(gi[r] - gj) : 0.f;
              }
            }
          }
          *reinterpret_cast<lds_w128_t>(st + L::OFF_P + 1024 * (tj < 2 ? 2 * tj + s2 : 2 + tj) + 16 * lane) = pack8(Z[0], Z[1]);
        };
        if (wave == 0) { make_operand(0, 0); make_operand(1, 0); }
        else if (wave == 1) { make_operand(0, 1); make_operand(3, 1); }
        if (wave == NW - 2) make_operand(1, 1);
        if (wave == NW - 1) make_operand(2, 1);
        __syncthreads();   // P^T
#pragma unroll
        for (int tj = 0; tj < 4; ++tj)
#pragma unroll
          for (int s2 = 0; s2 < 2; ++s2)
            if (tj < 2 || s2 == 1)
              DV[tj] = mfma16(*reinterpret_cast<lds_b128_t>(st + L::OFF_P + 1024 * (tj < 2 ? 2 * tj + s2 : 2 + tj) + 16 * lane), DOB[s2], DV[tj]);
      }
    }
    if (more) request(4, c - 1);
    // ---- dX = TmB^T dv_new (dv_new as two operands: the truncated value and the remainder) ------------------------------------
    f32x4 DX[4];
    if constexpr (DELTA) {
      const bf16x8 DVB[2] = {pack8_trunc(DV[0], DV[1]), pack8_trunc(DV[2], DV[3])};
      const bf16x8 DVR[2] = {pack8_rest(DV[0], DV[1]), pack8_rest(DV[2], DV[3])};
#pragma unroll
      for (int tj = 0; tj < 4; ++tj) {
        DX[tj] = (f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int s2 = 0; s2 < 2; ++s2)
          if (2 * s2 + 1 >= tj) {
            const unsigned lo = st + L::OFF_T + 1024 * tri_slot(2 * s2, tj >> 1) + a_tm + 8 * (tj & 1);
            const unsigned hi = st + L::OFF_T + 1024 * tri_slot(2 * s2 + 1, tj >> 1) + a_tm + 8 * (tj & 1);
            const bf16x8 a = join4(lds_tr4_at(lo), lds_tr4_at(hi));
            DX[tj] = mfma16(a, DVR[s2], DX[tj]);
            DX[tj] = mfma16(a, DVB[s2], DX[tj]);
          }
      }
    } else {
#pragma unroll
      for (int t = 0; t < 4; ++t) DX[t] = DV[t];
    }
    if (more) request(5, c - 1);
    // ---- dv = dX, through this wave's own 16 columns of the dO tile (read above, by this wave only) so that it leaves as
    //      16-byte pieces; no other wave touches these bytes, so no barrier ----------------------------------------------------
    float dbeta_part = 0.f;
    {
      float pb[16];
      f32x4 VNc[4];
      if constexpr (DELTA) {
#pragma unroll
        for (int t = 0; t < 4; ++t) {
          const s16x4 w = lds_tr4_at(st + L::OFF_VN + a_v + t * 16 * L::VROW);
#pragma unroll
          for (int r = 0; r < 4; ++r) VNc[t][r] = bf16_to_f32((bf16_t)w[r]);
        }
      }
#pragma unroll
      for (int t = 0; t < 4; ++t)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const int tk = 16 * t + 4 * g4 + r;
          *reinterpret_cast<lds_h_t>(st + L::OFF_DO + tk * L::VROW + 16 * ((2 * wave + (x16 >> 3)) ^ v_swz(tk)) + 2 * (x16 & 7)) = f32_to_bf16(DX[t][r]);
          if constexpr (DELTA) pb[4 * t + r] = DX[t][r] * VNc[t][r];
        }
      if constexpr (DELTA) {
        // for dbeta_i = <dX_i, v_new_i> / beta_i^2: this wave's 16 columns of the inner product (dX still in fp32).  Sixteen
        // sums over sixteen lanes as a butterfly: in every step a lane hands half of its values to its partner and adds
        // the partner's other half to the rest; lane x ends up with sum number x.  The partner is the lane's mirror image in
        // its group of 16, 8, 4, 2 lanes (what the cross-lane operand modifiers of the vector ALU offer: no LDS round trip).
        auto step = [&](const int d, auto mirror) __attribute__((always_inline)) {
          const bool up = (x16 & d) != 0;
#pragma unroll
          for (int i = 0; i < 8; ++i)
            if (i < d) {
              const float send = up ? pb[i] : pb[i + d], keep = up ? pb[i + d] : pb[i];
              pb[i] = keep + mirror(send);
            }
        };
        step(8, [](const float x) { return lane_mirror<0x140>(x); });   // lane 15 - x of the row of 16
        step(4, [](const float x) { return lane_mirror<0x141>(x); });   // 7 - x % 8 within each half row
        step(2, [](const float x) { return lane_mirror<0x1b>(x); });    // quad order 3, 2, 1, 0
        step(1, [](const float x) { return lane_mirror<0xb1>(x); });    // quad order 1, 0, 3, 2
        dbeta_part = pb[0];
      }
    }
    if (more) request(6, c - 1);
    // ---- dS = e^G dS' + Q~^T dO - W^T dX ----------------------------------------------------------------------------------------
    {
      f32x4 A1[4], A2[4];
#pragma unroll
      for (int t = 0; t < 4; ++t) {
        const f32x4 s4 = *reinterpret_cast<lds_f4_t>(st + L::OFF_SC + 4 * CB + a_sc + 64 * t);
#pragma unroll
        for (int r = 0; r < 4; ++r) A1[t][r] = DOc[t][r] * s4[r];
        if constexpr (DELTA) {
          const f32x4 e4 = *reinterpret_cast<lds_f4_t>(st + L::OFF_SC + a_sc + 64 * t);
#pragma unroll
          for (int r = 0; r < 4; ++r) A2[t][r] = -DX[t][r] * e4[r];
        }
      }
      const bf16x8 B1[2] = {pack8(A1[0], A1[1]), pack8(A1[2], A1[3])};
      bf16x8 B2[2];
      if constexpr (DELTA) { B2[0] = pack8(A2[0], A2[1]); B2[1] = pack8(A2[2], A2[3]); }
      auto ld_t = [&](const int off, const int m, const int s2) __attribute__((always_inline)) -> bf16x8 {
        const unsigned a = st + off + a_kt[m >> 1] + 8u * (m & 1) + (32 * s2) * L::KROW;
        return join4(lds_tr4_at(a), lds_tr4_at(a + 16 * L::KROW));
      };
#pragma unroll
      for (int m = 0; m < KT; ++m) {
#pragma unroll
        for (int r = 0; r < 4; ++r) dS[m][r] *= dec;
#pragma unroll
        for (int s2 = 0; s2 < 2; ++s2) {
          dS[m] = mfma16(ld_t(L::OFF_Q, m, s2), B1[s2], dS[m]);
          if constexpr (DELTA) dS[m] = mfma16(ld_t(L::OFF_K, m, s2), B2[s2], dS[m]);
        }
      }
    }
    // ---- this step's global stores (and the one scalar the next step needs) -----------------------------------------------
    {
      // eight consecutive K rows of this lane's column per 16-byte store
      bf16_t* dso = p.ds_all + (((size_t)(chunk_off + c) * p.H + h) * p.V + col) * DK + 8 * g4;
#pragma unroll
      for (int s = 0; s < KS; ++s) *reinterpret_cast<bf16x8*>(dso + 32 * s) = DSB[s];
      // (the tile's writes above come first: same wave, and the LDS pipe keeps their order)
#pragma unroll
      for (int it = 0; it < 2; ++it) {
        const int pc = lane + 64 * it, row = pc >> 1, half = pc & 1;
        const bf16x8 w = *reinterpret_cast<lds_b128_t>(st + L::OFF_DO + row * L::VROW + 16 * ((2 * wave + half) ^ v_swz(row)));
        if (row < nvalid) *reinterpret_cast<bf16x8*>(p.dv + ((row0 + row) * p.H + h) * p.V + vcol0 + 16 * wave + 8 * half) = w;
      }
      if constexpr (DELTA) {
        const int tk = 16 * (x16 >> 2) + 4 * g4 + (x16 & 3);
        if (tk < nvalid) p.dbeta_parts[((row0 + tk) * p.H + h) * (p.V / 16) + NW * split + wave] = dbeta_part;
      }
      if (c > 0) gs_next = p.gsum_blk[((size_t)blk0 + ((c - 1) * CB) / p.block) * p.H + h];
    }
    if (c % per == 0 && have_pend) {
#pragma unroll
      for (int m = 0; m < KT; ++m)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          if constexpr (PEND_LDS) dS[m][r] += *reinterpret_cast<lds_f1_t>(a_pend + 256 * (4 * m + r));
          else {
            dS[m][r] += pend[m][r];
            pend[m][r] = 0.f;
          }
        }
      have_pend = false;
    }
  }
  if (p.dh0) {
#pragma unroll
    for (int m = 0; m < KT; ++m)
#pragma unroll
      for (int r = 0; r < 4; ++r) p.dh0[((size_t)chain * DK + krow_of(m, r)) * p.V + col] = dS[m][r];
  }
}

// =============================================================================================
// per-chunk gradients
// =============================================================================================
template <int DK>
struct BwdChunkLds {
  static constexpr int KP = DK + 8;
  // phase 1 (the products that contract over V, one 64-column slice at a time): dO, dX, v_new [64][TP]; S, dS' [64 columns][KP]
  static constexpr int DO = 0, DX = DO + CB * TP, VN = DX + CB * TP, SN = VN + CB * TP, DSN = SN + CB * KP, P1 = DSN + CB * KP;
  // phase 2 (the products that contract over tokens): q^, k^ [64][KP]; the weight tiles Gm, Gm^T, Hm + Hm^T [64][TP]
  static constexpr int QN = 0, KN = QN + CB * KP, GN = KN + CB * KP, GT = GN + CB * TP, HS = GT + CB * TP, P2 = HS + CB * TP;
  static constexpr int ELEMS = P1 > P2 ? P1 : P2;
  static constexpr int FL = ELEMS * 2;
  static constexpr int TOTAL = FL + (8 * CB + 32) * 4;
};

template <int DK, bool DELTA>
__global__ __launch_bounds__(256, DK <= 128 ? 2 : 1) void linear_bwd_chunk_kernel(const LinBwdParams p) {
  using L = BwdChunkLds<DK>;
  constexpr int KP = L::KP, KT16 = DK / 16, KS = DK / 32;
  extern __shared__ __align__(16) unsigned char smem[];
  bf16_t* const sm = reinterpret_cast<bf16_t*>(smem);
  float* const fl = reinterpret_cast<float*>(smem + L::FL);
  float *gam = fl, *eg = fl + CB, *ek = fl + 2 * CB, *bet = fl + 3 * CB, *rq = fl + 4 * CB, *rk = fl + 5 * CB, *dgam = fl + 6 * CB,
        *sqv = fl + 7 * CB;
  // [0..3] <dS', S> and [4..7] <dS', S_blockstart> per wave; [8..23] the gate terms per (wave, lane group): summed in a fixed order
  float* red = fl + 8 * CB;

  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, x16 = lane & 15, g4 = lane >> 4;
  const int gc = blockIdx.x / p.H, h = blockIdx.x % p.H;
  int c, bos, len, blk0, chunk_off;
  if (p.seqs == nullptr) {
    const int n = gc / p.nt;
    c = gc - n * p.nt; bos = n * p.T; len = p.T; blk0 = n * p.TN; chunk_off = n * p.nt;
  } else {
    int n = 0;
    for (int i = 1; i < p.n_seqs; ++i)
      if (p.seqs[i].chunk_off <= gc) n = i;
    chunk_off = p.seqs[n].chunk_off;
    c = gc - chunk_off; bos = p.seqs[n].bos; len = p.seqs[n].eos - bos; blk0 = p.seqs[n].bos_nats;
  }
  const int t0 = c * CB, nvalid = min(CB, len - t0);
  const size_t row0 = (size_t)bos + t0;
  const int per = p.block / CB;
  const bool decay = (p.flags & NATSL_DECAY_NON_LINEAR) != 0, intra = (p.flags & NATSL_INTRA_CHUNK) != 0;
  const bool l2 = DELTA && (p.flags & NATSL_QK_L2NORM) != 0;
  const int hn = h / (p.H / p.HN);
  const int blk = t0 / p.block;
  const bool last = ((c + 1) % per == 0) || (c == (len + CB - 1) / CB - 1);
  const bool lin = lin_type_b(p.types, p.types_dtype, ((size_t)(blk0 + blk) * p.HN + hn) * 2 + 1);
  const bool rolled = last && !lin;
  const bool want_rb = rolled && decay;
  const int c_first = (c / per) * per;

  if (wave == 0) {
    const bool ok = lane < nvalid;
    const size_t gi = (row0 + lane) * p.H + h;
    store_scalars<DELTA>(lane, ok ? p.g[gi] : 0.f, DELTA && ok ? bf16_to_f32(p.beta[gi]) : 0.f, p.scale, gam, eg, ek, sqv, bet);
  }
  // q^, k^ are requested now and put into LDS when phase 1 is done with it
  QkRegs<DK> qk;
  load_qk<DK>(p, tid, row0, nvalid, h, qk);

  // ---- phase 1 -------------------------------------------------------------------------------------------------------
  bf16_t* const DOs = sm + L::DO;
  bf16_t* const DXs = sm + L::DX;
  bf16_t* const VNs = sm + L::VN;
  bf16_t* const Sn = sm + L::SN;
  bf16_t* const DSn = sm + L::DSN;
  f32x4 Nm[4], Mm[4], DQ2[KT16], DW[KT16], DK3[KT16];
#pragma unroll
  for (int t = 0; t < 4; ++t) { Nm[t] = (f32x4){0.f, 0.f, 0.f, 0.f}; Mm[t] = (f32x4){0.f, 0.f, 0.f, 0.f}; }
#pragma unroll
  for (int m = 0; m < KT16; ++m) {
    DQ2[m] = (f32x4){0.f, 0.f, 0.f, 0.f}; DW[m] = (f32x4){0.f, 0.f, 0.f, 0.f}; DK3[m] = (f32x4){0.f, 0.f, 0.f, 0.f};
  }
  float sds = 0.f, srb = 0.f;
  const size_t unit = (size_t)gc * p.H + h;
  const bf16_t* s_src = p.s_all + unit * p.V * DK;
  const bf16_t* ds_src = p.ds_all + unit * p.V * DK;
  const bf16_t* sf_src = p.s_all + ((size_t)(chunk_off + c_first) * p.H + h) * p.V * DK;
  for (int vs = 0; vs < p.V / 64; ++vs) {
    u32x4 w_do[2], w_vn[2], w_dx[2];
    load_tokens64(p.d_o, tid, row0, nvalid, p.H, p.V, h, 64 * vs, w_do);
    load_tokens64(p.vn, tid, row0, nvalid, p.H, p.V, h, 64 * vs, w_vn);
    if (DELTA) load_tokens64(p.dv, tid, row0, nvalid, p.H, p.V, h, 64 * vs, w_dx);
    __syncthreads();   // the previous slice's tiles are dead
    store_tokens64(w_do, tid, DOs);
    store_tokens64(w_vn, tid, VNs);
    if (DELTA) store_tokens64(w_dx, tid, DXs);
    // the state and its gradient as they lie in memory: [64 columns][K]; a thread's pieces are all requested before the
    // first of them is used
    {
      constexpr int NP = 64 * (DK / 8) / 256;
      u32x4 ws[NP], wd[NP];
#pragma unroll
      for (int i = 0; i < NP; ++i) {
        const int pc = tid + 256 * i, v = pc / (DK / 8), seg = pc % (DK / 8);
        const size_t off = (size_t)(64 * vs + v) * DK + seg * 8;
        ws[i] = *reinterpret_cast<const u32x4*>(s_src + off);
        wd[i] = *reinterpret_cast<const u32x4*>(ds_src + off);
      }
#pragma unroll
      for (int i = 0; i < NP; ++i) {
        const int pc = tid + 256 * i, v = pc / (DK / 8), seg = pc % (DK / 8);
        const size_t off = (size_t)(64 * vs + v) * DK + seg * 8;
        *reinterpret_cast<u32x4*>(Sn + v * KP + seg * 8) = ws[i];
        *reinterpret_cast<u32x4*>(DSn + v * KP + seg * 8) = wd[i];
        float fs[8], fd[8];
        unpack8f(ws[i], fs);
        unpack8f(wd[i], fd);
#pragma unroll
        for (int e = 0; e < 8; ++e) sds += fs[e] * fd[e];
        if (want_rb) {
          float ff[8];
          unpack8f(*reinterpret_cast<const u32x4*>(sf_src + off), ff);
#pragma unroll
          for (int e = 0; e < 8; ++e) srb += ff[e] * fd[e];
        }
      }
    }
    __syncthreads();
#pragma unroll
    for (int s = 0; s < 2; ++s) {
      const bf16x8 a_do = *reinterpret_cast<const bf16x8*>(DOs + (16 * wave + x16) * TP + 32 * s + 8 * g4);
      const bf16x8 a_vn = *reinterpret_cast<const bf16x8*>(VNs + (16 * wave + x16) * TP + 32 * s + 8 * g4);
      bf16x8 a_dx = a_vn;
      if (DELTA) a_dx = *reinterpret_cast<const bf16x8*>(DXs + (16 * wave + x16) * TP + 32 * s + 8 * g4);
#pragma unroll
      for (int tj = 0; tj < 4; ++tj) {
        const bf16x8 b = *reinterpret_cast<const bf16x8*>(VNs + (16 * tj + x16) * TP + 32 * s + 8 * g4);
        Nm[tj] = mfma16(a_do, b, Nm[tj]);
        if (DELTA) Mm[tj] = mfma16(a_dx, b, Mm[tj]);
      }
#pragma unroll
      for (int m = 0; m < KT16; ++m) {
        // columns = K index 16 m + x, slots = state columns 32 s + 8 g + j
        const bf16x8 bs = tr_operand(Sn, KP, 32 * s + 8 * g4, 32 * s + 8 * g4 + 4, 16 * m, x16);
        const bf16x8 bd = tr_operand(DSn, KP, 32 * s + 8 * g4, 32 * s + 8 * g4 + 4, 16 * m, x16);
        DQ2[m] = mfma16(a_do, bs, DQ2[m]);
        if (DELTA) DW[m] = mfma16(a_dx, bs, DW[m]);
        DK3[m] = mfma16(a_vn, bd, DK3[m]);
      }
    }
  }
#pragma unroll
  for (int d = 1; d < 64; d <<= 1) { sds += __shfl_xor(sds, d); srb += __shfl_xor(srb, d); }
  if (lane == 0) { red[wave] = sds; red[4 + wave] = srb; }

  // ---- phase 2 -------------------------------------------------------------------------------------------------------
  bf16_t* const Qn = sm + L::QN;
  bf16_t* const Kn = sm + L::KN;
  bf16_t* const Gn = sm + L::GN;
  bf16_t* const GT = sm + L::GT;
  bf16_t* const Hs = sm + L::HS;
  __syncthreads();   // phase 1's tiles are dead
  store_qk<DK>(qk, tid, l2, Qn, Kn, rq, rk);
  if (DELTA)
    for (int i = tid; i < CB * TP / 8; i += 256) *reinterpret_cast<u32x4*>(Hs + 8 * i) = (u32x4){0u, 0u, 0u, 0u};
  __syncthreads();

  // this lane's rows i = 16 wave + 4 g + r; its column in tile tj is 16 tj + x
  const f32x4 gi4 = *reinterpret_cast<const f32x4*>(gam + 16 * wave + 4 * g4);
  f32x4 rsH = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int tj = 0; tj < 4; ++tj) {
    const int j = 16 * tj + x16;
    const float gj = gam[j];
    f32x4 KK = {0.f, 0.f, 0.f, 0.f};
    if (DELTA) {
#pragma unroll
      for (int s = 0; s < KS; ++s) {
        const bf16x8 a = *reinterpret_cast<const bf16x8*>(Kn + (16 * wave + x16) * KP + 32 * s + 8 * g4);
        const bf16x8 b = *reinterpret_cast<const bf16x8*>(Kn + (16 * tj + x16) * KP + 32 * s + 8 * g4);
        KK = mfma16(a, b, KK);
      }
    }
    u32x2 gw;
    float gv[4];
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int i = 16 * wave + 4 * g4 + r;
      const float Lij = i >= j ? __expf(gi4[r] - gj) : 0.f;
      gv[r] = intra ? p.scale * Nm[tj][r] * Lij : 0.f;
      Gn[i * TP + j] = f32_to_bf16(gv[r]);
      if (DELTA) {
        if (i > j) {
          const float hv = -Mm[tj][r] * Lij;
          rsH[r] += hv * KK[r];
          const bf16_t hb = f32_to_bf16(hv);
          Hs[i * TP + j] = hb;
          Hs[j * TP + i] = hb;
        }
      }
    }
    gw[0] = pack_bf16x2(gv[0], gv[1]);
    gw[1] = pack_bf16x2(gv[2], gv[3]);
    *reinterpret_cast<u32x2*>(GT + j * TP + 16 * wave + 4 * g4) = gw;
  }
  if (DELTA) {
#pragma unroll
    for (int r = 0; r < 4; ++r)
#pragma unroll
      for (int d = 1; d < 16; d <<= 1) rsH[r] += __shfl_xor(rsH[r], d);
  }
  __syncthreads();

  // dq^, dk^ of this wave's 16 tokens: lane = K column 16 m + x, registers = tokens 16 wave + 4 g + r
  const f32x4 eg4 = *reinterpret_cast<const f32x4*>(eg + 16 * wave + 4 * g4);
  const f32x4 ek4 = *reinterpret_cast<const f32x4*>(ek + 16 * wave + 4 * g4);
  const float nr = rolled ? 0.f : 1.f;
  f32x4 a_i = {0.f, 0.f, 0.f, 0.f}, b_i = {0.f, 0.f, 0.f, 0.f}, t2_i = {0.f, 0.f, 0.f, 0.f}, t3_i = {0.f, 0.f, 0.f, 0.f};
  bf16x8 ga[2], gta[2], ha[2];
#pragma unroll
  for (int s = 0; s < 2; ++s) {
    ga[s] = *reinterpret_cast<const bf16x8*>(Gn + (16 * wave + x16) * TP + 32 * s + 8 * g4);
    gta[s] = *reinterpret_cast<const bf16x8*>(GT + (16 * wave + x16) * TP + 32 * s + 8 * g4);
    ha[s] = gta[s];
    if (DELTA) ha[s] = *reinterpret_cast<const bf16x8*>(Hs + (16 * wave + x16) * TP + 32 * s + 8 * g4);
  }
  f32x4 DQ[KT16], DKg[KT16];
#pragma unroll
  for (int m = 0; m < KT16; ++m) {
    float qv[4], kv[4];
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      qv[r] = bf16_to_f32(Qn[(16 * wave + 4 * g4 + r) * KP + 16 * m + x16]);
      kv[r] = bf16_to_f32(Kn[(16 * wave + 4 * g4 + r) * KP + 16 * m + x16]);
    }
    f32x4 dq, dk;
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const float w2 = DELTA ? eg4[r] * DW[m][r] : 0.f, w3 = ek4[r] * DK3[m][r];
      dq[r] = p.scale * eg4[r] * DQ2[m][r];
      dk[r] = nr * w3 - w2;
      t2_i[r] += w2 * kv[r];
      t3_i[r] += w3 * kv[r];
    }
#pragma unroll
    for (int s = 0; s < 2; ++s) {
      // columns = K index 16 m + x, slots = tokens 32 s + 8 g + j
      const bf16x8 bk = tr_operand(Kn, KP, 32 * s + 8 * g4, 32 * s + 8 * g4 + 4, 16 * m, x16);
      const bf16x8 bq = tr_operand(Qn, KP, 32 * s + 8 * g4, 32 * s + 8 * g4 + 4, 16 * m, x16);
      dq = mfma16(ga[s], bk, dq);
      dk = mfma16(gta[s], bq, dk);
      if (DELTA) dk = mfma16(ha[s], bk, dk);
    }
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      a_i[r] += dq[r] * qv[r];
      b_i[r] += dk[r] * kv[r];
    }
    DQ[m] = dq;
    DKg[m] = dk;
  }
#pragma unroll
  for (int r = 0; r < 4; ++r)
#pragma unroll
    for (int d = 1; d < 16; d <<= 1) {
      a_i[r] += __shfl_xor(a_i[r], d);
      b_i[r] += __shfl_xor(b_i[r], d);
      t2_i[r] += __shfl_xor(t2_i[r], d);
      t3_i[r] += __shfl_xor(t3_i[r], d);
    }
  if (x16 == 0) {
    float t3s = 0.f;
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      dgam[16 * wave + 4 * g4 + r] = a_i[r] - b_i[r] + 2.f * rsH[r] - 2.f * t2_i[r];
      t3s += t3_i[r];
    }
    red[8 + 4 * wave + g4] = t3s;
  }
  __syncthreads();   // every wave is done with q^, k^ and the weight tiles; dgam and red are complete

  // ---- the row normalisation's backward, then out through LDS (in place of the q^, k^ tiles) ---------------------------
  {
    const f32x4 rq4 = *reinterpret_cast<const f32x4*>(rq + 16 * wave + 4 * g4);
    const f32x4 rk4 = *reinterpret_cast<const f32x4*>(rk + 16 * wave + 4 * g4);
#pragma unroll
    for (int m = 0; m < KT16; ++m)
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int i = 16 * wave + 4 * g4 + r, kc = 16 * m + x16;
        float dq = DQ[m][r], dk = DKg[m][r];
        if (l2) {
          const float qv = bf16_to_f32(Qn[i * KP + kc]), kv = bf16_to_f32(Kn[i * KP + kc]);
          dq = rq4[r] * (dq - qv * a_i[r]);
          dk = rk4[r] * (dk - kv * b_i[r]);
        }
        // (each element is read and then overwritten by the same lane)
        Qn[i * KP + kc] = f32_to_bf16(dq);
        Kn[i * KP + kc] = f32_to_bf16(dk);
      }
  }
  if (DELTA && wave == 1 && lane < nvalid) {
    const float* pp = p.dbeta_parts + ((row0 + lane) * p.H + h) * (p.V / 16);
    float sum = 0.f;
    for (int i = 0; i < p.V / 16; ++i) sum += pp[i];
    p.dbeta[(row0 + lane) * p.H + h] = sum / (bet[lane] * bet[lane]);
  }
  if (wave == 0) {
    // dg_t = sum_{i >= t} dgamma_i + dG
    float gate_sum = 0.f;
    for (int i = 0; i < 16; ++i) gate_sum += red[8 + i];
    const float dG = nr * (gate_sum + __expf(gam[CB - 1]) * (red[0] + red[1] + red[2] + red[3]));
    float x = dgam[lane];
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
      const float y = __shfl_down(x, d);
      if (lane + d < 64) x += y;
    }
    if (lane < nvalid) p.dg[(row0 + lane) * p.H + h] = x + dG;
    if (lane == 0) {
      p.gate[unit] = gate_sum;
      p.rb[unit] = want_rb ? __expf(p.gsum_blk[((size_t)blk0 + blk) * p.H + h]) * (red[4] + red[5] + red[6] + red[7]) : 0.f;
    }
  }
  __syncthreads();
  for (int pc = tid; pc < CB * (DK / 8); pc += 256) {
    const int row = pc / (DK / 8), seg = pc % (DK / 8);
    if (row < nvalid) {
      const size_t off = ((row0 + row) * p.H + h) * DK + seg * 8;
      *reinterpret_cast<u32x4*>(p.dq + off) = *reinterpret_cast<const u32x4*>(Qn + row * KP + seg * 8);
      *reinterpret_cast<u32x4*>(p.dk + off) = *reinterpret_cast<const u32x4*>(Kn + row * KP + seg * 8);
    }
  }
}

static int bwd_cu_count() {
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

template <int DK, bool DELTA, int NW>
static int launch_bwd_scan(const LinBwdParams& p, hipStream_t stream, const char* what) {
  using L = BwdScanLds<DK, NW>;
  auto kern = linear_bwd_scan_kernel<DK, DELTA, NW>;
  hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, L::TOTAL);
  if (e != hipSuccess) return fail(NATSL_ERR_LAUNCH, "%s: cannot reserve %d bytes of LDS: %s", what, L::TOTAL, hipGetErrorString(e));
  const int n_chains = (p.seqs ? p.n_seqs : p.B) * p.H;
  hipLaunchKernelGGL(kern, dim3((unsigned)((n_chains + 7) / 8 * 8 * (p.V / (16 * NW)))), dim3(L::THREADS), L::TOTAL, stream, p);
  return check_launch(what);
}

template <int DK, bool DELTA>
static int launch_bwd(const LinBwdParams& p, hipStream_t stream, const char* what) {
  {
    // one workgroup per CU at most (LDS): 32-column workgroups (two compute waves) when the 64-column ones would leave
    // half of the CUs without work
    const long long wgs64 = (long long)(p.seqs ? p.n_seqs : p.B) * p.H * (p.V / 64);
    int rc;
    if constexpr (DK <= 128) rc = 2 * wgs64 <= bwd_cu_count() ? launch_bwd_scan<DK, DELTA, 2>(p, stream, what) : launch_bwd_scan<DK, DELTA, 4>(p, stream, what);
    else rc = launch_bwd_scan<DK, DELTA, 4>(p, stream, what);
    if (rc != NATSL_OK) return rc;
  }
  {
    using L = BwdChunkLds<DK>;
    auto kern = linear_bwd_chunk_kernel<DK, DELTA>;
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, L::TOTAL);
    if (e != hipSuccess) return fail(NATSL_ERR_LAUNCH, "%s: cannot reserve %d bytes of LDS: %s", what, L::TOTAL, hipGetErrorString(e));
    hipLaunchKernelGGL(kern, dim3((unsigned)(p.total_chunks * p.H)), dim3(256), L::TOTAL, stream, p);
    return check_launch(what);
  }
}

}  // namespace natsl

using namespace natsl;

extern "C" int natsl_linear_chunk_bwd(int delta_rule, const void* q, const void* k, const void* v_new, const float* g, const void* beta,
                                      const void* d_o, const float* dht, const void* chunk_states, const void* types, int types_dtype,
                                      const float* g_block_sums, const void* workspace, void* d_chunk_states, float* dbeta_parts,
                                      void* dq, void* dk, void* dv, float* dg, float* dbeta, float* dh0, float* d_gate, float* d_rollback, int B, int T,
                                      int H, int HN, int K, int V, int TN, int block, float scale, int flags, int dtype,
                                      const natsl_seq_row* seqs, int n_seqs, int total_chunks, natsl_stream_t stream) {
  const char* what = "natsl_linear_chunk_bwd";
  if (!q || !k || !v_new || !g || !d_o || !chunk_states || !types || !g_block_sums || !d_chunk_states || !dq || !dk || !dv || !dg ||
      !d_gate || !d_rollback || !workspace || (delta_rule && (!beta || !dbeta || !dbeta_parts)))
    return fail(NATSL_ERR_INVALID, "%s: null pointer argument", what);
  if (dtype != NATSL_BF16) return fail(NATSL_ERR_UNSUPPORTED, "%s: only bf16 tensors are supported (got dtype %d)", what, dtype);
  if (types_dtype != NATSL_BF16 && types_dtype != NATSL_F32) return fail(NATSL_ERR_UNSUPPORTED, "%s: block types must be f32 or bf16", what);
  if (B <= 0 || T <= 0 || H <= 0 || HN <= 0 || TN <= 0) return fail(NATSL_ERR_INVALID, "%s: non-positive dimension", what);
  if (H % HN) return fail(NATSL_ERR_INVALID, "%s: H=%d must be a multiple of HN=%d", what, H, HN);
  if (block < 64 || block % 64) return fail(NATSL_ERR_UNSUPPORTED, "%s: block size %d must be a multiple of 64", what, block);
  if (V % 64 || V <= 0) return fail(NATSL_ERR_UNSUPPORTED, "%s: V=%d must be a multiple of 64", what, V);
  if (seqs ? (B != 1 || n_seqs <= 0 || total_chunks <= 0) : (TN != cdiv(T, block)))
    return fail(NATSL_ERR_INVALID, "%s: TN=%d does not match T=%d, block=%d (or bad packed-input arguments)", what, TN, T, block);
  LinBwdParams p;
  p.q = (const bf16_t*)q; p.k = (const bf16_t*)k; p.vn = (const bf16_t*)v_new; p.d_o = (const bf16_t*)d_o; p.g = g;
  p.beta = (const bf16_t*)beta; p.s_all = (const bf16_t*)chunk_states; p.ds_all = (bf16_t*)d_chunk_states; p.dv = (bf16_t*)dv;
  p.dht = dht; p.dh0 = dh0; p.gsum_blk = g_block_sums; p.ws_tm = (const bf16_t*)workspace; p.types = types;
  {
    // (the layout natsl_gdn_chunk_fwd / natsl_mamba_chunk_fwd gave the workspace)
    const size_t units = (size_t)(seqs ? total_chunks : B * cdiv(T, CB)) * (size_t)H;
    p.ws_p = p.ws_tm + units * (CB * CB);
    p.ws_sc = reinterpret_cast<const float*>(p.ws_p + units * (CB * CB));
  } p.types_dtype = types_dtype;
  p.dq = (bf16_t*)dq; p.dk = (bf16_t*)dk; p.dg = dg; p.dbeta = dbeta; p.dbeta_parts = dbeta_parts; p.gate = d_gate; p.rb = d_rollback;
  p.B = B; p.T = T; p.H = H; p.HN = HN; p.V = V; p.TN = TN; p.block = block; p.nt = cdiv(T, CB);
  p.seqs = reinterpret_cast<const SeqRow*>(seqs); p.n_seqs = seqs ? n_seqs : 0; p.total_chunks = seqs ? total_chunks : B * p.nt;
  p.scale = scale; p.flags = flags;
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  if (delta_rule) {
    if (K == 128) return launch_bwd<128, true>(p, s, what);
    if (K == 64) return launch_bwd<64, true>(p, s, what);
    if (K == 192) return launch_bwd<192, true>(p, s, what);
  } else {
    p.flags &= ~NATSL_QK_L2NORM;
    if (K == 128) return launch_bwd<128, false>(p, s, what);
    if (K == 64) return launch_bwd<64, false>(p, s, what);
    if (K == 192) return launch_bwd<192, false>(p, s, what);
  }
  return fail(NATSL_ERR_UNSUPPORTED, "%s: key dim K=%d not built (supported: 64, 128, 192)", what, K);
}
