// Linear-recurrent branches (Gated DeltaNet and Mamba2-style SSD), chunked forward for gfx950.
//
// Two kernels per call:
//
//   linear_prep_kernel   one workgroup per (64-token chunk, head), fully parallel.  Everything
//                        that does not depend on the running state: row norms of q and k, the
//                        chunk-local cumulative log-decay gamma, the two 64x64 Gram products
//                        k k^T and q k^T on the matrix cores, the unit-lower-triangular solve
//                        Tm = (I + A)^-1 in LDS, and per-token scale vectors.  It leaves, per
//                        chunk-head, 17 KiB in the workspace:
//                          TmB  bf16 [64][64]   Tm * diag(beta)                      (delta rule only)
//                          P    bf16 [64][64]   scale * tril(q^ k^^T * e^{gamma_i-gamma_j})
//                          sc   f32  [4][64]    se = e^{gamma} rk, sq = scale rq e^{gamma},
//                                               sk = rk e^{gamma_last-gamma}, {e^{gamma_last}, gamma_last, is_linear}
//                        (rq, rk = reciprocal L2 norms, or 1).
//
//   linear_scan_kernel   walks the chunks of one (sequence, head) in order.  A wave owns 16 columns of the state
//                        for ALL K rows, as the fp32 accumulators of 16x16x32 matrix instructions:
//                          R = k S;  X = v - se*R;  v_new = TmB X               (delta rule)
//                          o = sq*(q S) + P v_new
//                          S <- e^{gamma_last} S + k^T (sk*v_new)               (blocks typed linear)
//                        With the columns in the lanes, every product above takes the state, X and v_new as the
//                        B operand STRAIGHT FROM THE ACCUMULATOR REGISTERS (rounded to bf16 in place): an accumulator
//                        tile holds, per lane, four consecutive rows, and two tiles side by side are the eight
//                        contraction slots of a lane -- under a fixed relabelling of the contraction index that the
//                        A operand follows (which K row a state register holds; which token a column of TmB / P
//                        stands for, chosen by the prep kernel).  Nothing state-dependent goes through LDS and the
//                        waves never exchange data: the only barrier of a step hands over the next chunk's inputs.
//                        Those (k, q, v tiles, TmB, P, sc) arrive by LDS-DMA, double buffered, one chunk ahead.
//                        Raw q, k are used: the 1/norm factors are folded into the per-token scale vectors.
//                        A block that is not typed linear leaves S rolled back at its end (times
//                        e^{sum g} when decay is on), which is all the reference's carry logic
//                        (src/nats/ops/utils/cumsum.py:95-133) amounts to.
//
// For a backward the scan can also store the state that enters every chunk (the bf16 B operands it forms anyway, [chunk][H][V][K])
// and the delta rule's v_new of every token; natsl_linear_bwd.hip reads them, and TmB from the workspace.
//
// The Mamba form has no solve: its prep is mamba_scale_kernel (the scale vectors only; q and k are not read), and the
// scan's data-movement waves form P from the k and q tiles of the stage.
//
// The delta rule has a second form of the pair for launches that fill the GPU and need no backward ("PF" below): the prep
// reads k only and leaves no P (two more scale vectors in its place), and the scan forms P from the staged k and q tiles in
// waves that do not hold the state; a second barrier in the middle of a step hands it to the compute waves.
#include "natsl_device.h"
#include "natsl_host.h"

namespace natsl {

struct LinearParams {
  const bf16_t* q;
  const bf16_t* k;
  const bf16_t* v;
  const float* g;
  const bf16_t* beta;
  const float* h0;
  bf16_t* o;
  float* ht;
  float* hs;      // state entering each sequence's last selector block (optional)
  float* gs;      // sum of g over that block, [N,H] (optional)
  bf16_t* s_out;  // the state entering every chunk, transposed: [chunk][H][V][K] bf16 (optional; for the backward)
  bf16_t* vn_out; // v_new of every token, [tokens][H][V] bf16 (optional, delta rule only; for the backward)
  const void* types;
  int types_dtype;
  const SeqRow* seqs;
  int n_seqs;
  int B, T, H, HN, V, TN, block;
  int nt;            // chunks per sequence (regular batch)
  int total_chunks;
  float scale;
  int flags;
  bf16_t* ws_tm;
  bf16_t* ws_p;
  float* ws_sc;
};

constexpr int C = 64;

NATSL_DEVICE bool lin_type(const void* types, int dtype, size_t i) {
  float x = dtype == NATSL_F32 ? reinterpret_cast<const float*>(types)[i]
                               : bf16_to_f32(reinterpret_cast<const bf16_t*>(types)[i]);
  return rintf(x) == 1.0f;
}

// =============================================================================================
// prep
// =============================================================================================
// PF ("P formed by the scan"): the kernel reads k only -- no q tile, no q k^T product, no P -- and leaves TmB and six scale
// vectors; the two extra ones (in the first 512 bytes of the unit's P area) are the exponents the scan needs to form
// P_ij = rq_i (q_i . k_j) exp2(gq_i - gk_j):   gk = gamma log2(e) - log2 rk,   gq = gamma log2(e) + log2 scale,
// and sq comes without its 1/|q| factor (the scan takes the row norms of q from the tile it holds anyway).
template <int DK, bool DELTA, bool PF>
__global__ __launch_bounds__(256, 4) void linear_prep_kernel(const LinearParams p) {
  static_assert(DELTA || !PF, "the Mamba form has its own prep");
  constexpr int KP = DK + 8;   // bf16 row pitch
  constexpr int KL = DK / 32;  // 16-byte loads per thread per tile
  // The 64x64 fp32 matrices of the solve are kept as their ten lower 16x16 blocks, block (i, k) at
  // index i(i+1)/2 + k, rows of BP floats.  A = strictly lower system matrix; X = (I+A)^-1 row-major;
  // Xt = the four DIAGONAL blocks of X transposed (so that such a block serves as an MFMA B operand with one 16-byte read).
  constexpr int BP = 20, BLK = 16 * BP, NBLK = 10;
  constexpr int TILE_BYTES = (PF ? 1 : 2) * C * KP * 2, SOLVE_BYTES = (2 * NBLK + 4) * BLK * 4;
  // LDS: the q, k tiles are dead once the Gram products are done; the solve reuses their space
  constexpr int REGION0 = (DELTA && SOLVE_BYTES > TILE_BYTES) ? SOLVE_BYTES : TILE_BYTES;
  __shared__ __align__(16) unsigned char region0[REGION0];
  __shared__ __align__(16) float gam[C], rq[C], rk[C], bet[C];
  bf16_t* Qs = reinterpret_cast<bf16_t*>(region0);
  bf16_t* Ks = PF ? Qs : Qs + C * KP;   // (no q tile with PF)
  float* Ab = reinterpret_cast<float*>(region0);
  float* Xb = Ab + NBLK * BLK;
  float* Xt = Xb + NBLK * BLK;
  auto bidx = [](int i, int k) { return i * (i + 1) / 2 + k; };

  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int gc = blockIdx.x / p.H, h = blockIdx.x % p.H;
  int bos, len, c, bos_nats;
  if (p.seqs == nullptr) {
    const int n = gc / p.nt;
    c = gc - n * p.nt;
    bos = n * p.T;
    len = p.T;
    bos_nats = n * p.TN;
  } else {
    int n = 0;
    for (int i = 1; i < p.n_seqs; ++i)
      if (p.seqs[i].chunk_off <= gc) n = i;
    c = gc - p.seqs[n].chunk_off;
    bos = p.seqs[n].bos;
    len = p.seqs[n].eos - bos;
    bos_nats = p.seqs[n].bos_nats;
  }
  const int t0 = c * C;
  const bool l2 = (p.flags & NATSL_QK_L2NORM) != 0;

  // ---- load q, k tiles; row sums of squares from the registers just loaded -----------------
  {
    const int row = tid >> 2, seg = tid & 3;
    const bool ok = t0 + row < len;
    const size_t off = ((size_t)(bos + t0 + row) * p.H + h) * DK;
    const u32x4* qr = reinterpret_cast<const u32x4*>(p.q + off);
    const u32x4* kr = reinterpret_cast<const u32x4*>(p.k + off);
    const u32x4 z = {0u, 0u, 0u, 0u};
    float sq = 0.f, sk = 0.f;
    u32x4 qa[KL], kb[KL];
#pragma unroll
    for (int i = 0; i < KL; ++i) {
      qa[i] = (ok && !PF) ? qr[seg + 4 * i] : z;
      kb[i] = ok ? kr[seg + 4 * i] : z;
    }
#pragma unroll
    for (int i = 0; i < KL; ++i) {
      const u32x4 a = qa[i], b = kb[i];
      if (!PF) *reinterpret_cast<u32x4*>(Qs + row * KP + (seg + 4 * i) * 8) = a;
      *reinterpret_cast<u32x4*>(Ks + row * KP + (seg + 4 * i) * 8) = b;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const float a0 = __uint_as_float(a[j] << 16), a1 = __uint_as_float(a[j] & 0xffff0000u);
        const float b0 = __uint_as_float(b[j] << 16), b1 = __uint_as_float(b[j] & 0xffff0000u);
        sq += a0 * a0 + a1 * a1;
        sk += b0 * b0 + b1 * b1;
      }
    }
    sq += __shfl_xor(sq, 1); sq += __shfl_xor(sq, 2);
    sk += __shfl_xor(sk, 1); sk += __shfl_xor(sk, 2);
    if (seg == 0) {
      rq[row] = (l2 && !PF) ? rsqrtf(sq + 1e-6f) : 1.f;
      rk[row] = l2 ? rsqrtf(sk + 1e-6f) : 1.f;
    }
  }
  // ---- gamma = inclusive cumsum of g over the chunk (wave 0), beta -------------------------
  if (wave == 0) {
    const bool ok = t0 + lane < len;
    const size_t gi = (size_t)(bos + t0 + lane) * p.H + h;
    float x = ok ? p.g[gi] : 0.f;
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
      const float y = __shfl_up(x, d);
      if (lane >= d) x += y;
    }
    gam[lane] = x;
    if (DELTA) bet[lane] = ok ? bf16_to_f32(p.beta[gi]) : 0.f;
  }
  __syncthreads();

  const size_t unit = (size_t)gc * p.H + h;
  bf16_t* Pout = p.ws_p + unit * (C * C);
  bf16_t* Tout = p.ws_tm + unit * (C * C);
  float* Sout = p.ws_sc + unit * (4 * C);

  // ---- Gram products on the matrix cores: wave w owns the 32x32 tile (w/2, w%2) ------------
  // P and TmB are stored as the scan kernel's MFMA A operands (16x16x32: 16 rows x 32 contraction tokens), 1 KiB each,
  // operand (t, s) = rows 16t.., tokens 32s.. at index 2t + s; in it, scan-lane (row i%16, group g) finds its 16 bytes
  // at (16 g + i%16) * 16.  The scan feeds the other operand from accumulator registers, where lane group g holds
  // tokens 4g..4g+3 of a 16-token tile, so slot j of group g stands for token 32s + 16(j/4) + 4g + j%4.
  // Operands (0,1) and (1,1) lie above the diagonal: never written, never read.
  {
    const int ti = wave >> 1, tj = wave & 1, l32 = lane & 31, hf = lane >> 5;
    const int i = 32 * ti + l32;  // P row owned by this lane
    bf16_t* prow = Pout + ((size_t)((2 * (i >> 4) + tj) * 64 + (i & 15))) * 8;
    f32x16 gk;
    if (ti >= tj) {
      f32x16 gq;
#pragma unroll
      for (int r = 0; r < 16; ++r) gk[r] = gq[r] = 0.f;
#pragma unroll
      for (int s = 0; s < DK / 16; ++s) {
        const bf16x8 kb = ld8(Ks + (32 * tj + l32) * KP + 16 * s + 8 * hf);
        if (!PF) {
          const bf16x8 qa = ld8(Qs + (32 * ti + l32) * KP + 16 * s + 8 * hf);
          gq = mfma32(kb, qa, gq);  // transposed: lane = query row i, registers = key tokens j
        }
        if (DELTA) {
          const bf16x8 ka = ld8(Ks + (32 * ti + l32) * KP + 16 * s + 8 * hf);
          gk = mfma32(ka, kb, gk);  // lane = column j, registers = rows i
        }
      }
      if (!PF) {
        // this lane's 16 key tokens are four runs of four: 16-byte reads of their gamma and 1/|k|
        const float gi = gam[i], fi = p.scale * rq[i];
        // this lane holds tokens 8 q4 + 4 hf + e of the tile: q4 = 0, 2 are the two halves of group hf's slots,
        // q4 = 1, 3 those of group 2 + hf
        u32x4 w[2];
#pragma unroll
        for (int q4 = 0; q4 < 4; ++q4) {
          const int j0 = 32 * tj + 8 * q4 + 4 * hf;
          const f32x4 gj = *reinterpret_cast<const f32x4*>(gam + j0), rj = *reinterpret_cast<const f32x4*>(rk + j0);
          float pv[4];
#pragma unroll
          for (int e = 0; e < 4; ++e) pv[e] = i >= j0 + e ? fi * rj[e] * gq[4 * q4 + e] * __expf(gi - gj[e]) : 0.f;
          w[q4 & 1][2 * (q4 >> 1)] = pack_bf16x2(pv[0], pv[1]);
          w[q4 & 1][2 * (q4 >> 1) + 1] = pack_bf16x2(pv[2], pv[3]);
        }
        *reinterpret_cast<u32x4*>(prow + hf * 128) = w[0];
        *reinterpret_cast<u32x4*>(prow + (2 + hf) * 128) = w[1];
      }
    }
    if (DELTA) {
      // all waves are done reading the q, k tiles before the A blocks overwrite them
      __syncthreads();
      if (ti >= tj) {
        const int j = 32 * tj + l32;
        const float gj = gam[j], rkj = rk[j];
#pragma unroll
        for (int q4 = 0; q4 < 4; ++q4) {
          const int i0 = 32 * ti + 8 * q4 + 4 * hf;  // rows i0..i0+3, all in one 16-row block
          const f32x4 gi4 = *reinterpret_cast<const f32x4*>(gam + i0), ri4 = *reinterpret_cast<const f32x4*>(rk + i0),
                      bi4 = *reinterpret_cast<const f32x4*>(bet + i0);
          if ((i0 >> 4) >= (j >> 4)) {
            float* dst = Ab + bidx(i0 >> 4, j >> 4) * BLK + (i0 & 15) * BP + (j & 15);
#pragma unroll
            for (int e = 0; e < 4; ++e)
              dst[e * BP] = i0 + e > j ? bi4[e] * ri4[e] * rkj * gk[4 * q4 + e] * __expf(gi4[e] - gj) : 0.f;
          }
        }
      }
    }
  }
  // ---- per-token scale vectors -------------------------------------------------------------
  if (wave == 1) {
    const float gl = gam[C - 1], gt = gam[lane], eg = __expf(gt);
    float dk = gl - gt;
    if (!DELTA) dk = fminf(dk, 0.f);  // src/nats/ops/mamba/chunk_h.py:177
    Sout[lane] = eg * rk[lane];
    Sout[C + lane] = p.scale * rq[lane] * eg;
    Sout[2 * C + lane] = rk[lane] * __expf(dk);
    if (PF) {
      float* Eout = reinterpret_cast<float*>(Pout);
      Eout[lane] = gt * 1.4426950408889634f - __builtin_amdgcn_logf(rk[lane]);
      Eout[C + lane] = gt * 1.4426950408889634f + __builtin_amdgcn_logf(p.scale);
    }
    if (lane == 0) Sout[3 * C] = __expf(gl);
    if (lane == 1) Sout[3 * C + 1] = gl;
    if (lane == 2) {
      // is this chunk's selector block typed linear?  (kept next to the decay so the scan finds it
      // in the cache line it prefetches anyway)
      const int hn = h / (p.H / p.HN);
      Sout[3 * C + 2] = lin_type(p.types, p.types_dtype, ((size_t)(bos_nats + (c * C) / p.block) * p.HN + hn) * 2 + 1) ? 1.f : 0.f;
    }
  }
  if (!DELTA) return;
  __syncthreads();

  // ---- X = (I + A)^-1 in fp32, 4x4 blocks of 16x16 ------------------------------------------
  // diagonal blocks by forward substitution: wave b owns block (b, b), one column per lane
  const int x16 = lane & 15, g4 = lane >> 4;
  if (lane < 16) {
    const float* Ad = Ab + bidx(wave, wave) * BLK;
    f32x4 arow[16][4];
#pragma unroll
    for (int r = 1; r < 16; ++r)
#pragma unroll
      for (int j4 = 0; j4 < (r + 3) / 4; ++j4) arow[r][j4] = *reinterpret_cast<const f32x4*>(Ad + r * BP + 4 * j4);
    float x[16];
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      float acc = r == x16 ? 1.f : 0.f;
#pragma unroll
      for (int j = 0; j < r; ++j) acc -= arow[r][j >> 2][j & 3] * x[j];
      x[r] = acc;
    }
    float* Xd = Xb + bidx(wave, wave) * BLK;
    float* Xtd = Xt + wave * BLK;
#pragma unroll
    for (int r = 0; r < 16; ++r) Xd[r * BP + x16] = x[r];
#pragma unroll
    for (int r4 = 0; r4 < 4; ++r4)
      *reinterpret_cast<f32x4*>(Xtd + x16 * BP + 4 * r4) = (f32x4){x[4 * r4], x[4 * r4 + 1], x[4 * r4 + 2], x[4 * r4 + 3]};
  }
  __syncthreads();
  // off-diagonal blocks on the fp32 matrix cores, wave k down its own block column:
  //   X_ik = -X_ii * sum_{j=k}^{i-1} A_ij X_jk        (i = k+1 .. 3)
  // MFMA 16x16x4: lane (x, g) supplies A[x][kk] and B[kk][x].  With kk = 4g + s in step s, the A operand of all four
  // steps is one 16-byte row read, and an accumulator (lane = column x, registers = rows 4g..4g+3) is already a B
  // operand: the X_jk of the column stay in registers (only the diagonal block comes from LDS), and the inner sum feeds
  // the second product from registers too.  Nothing a wave reads here was written by another wave after the barrier above,
  // so the column needs no barrier of its own.
  {
    const int k = wave;
    f32x4 Xcol[4];
#pragma unroll
    for (int i = 1; i < 4; ++i) {
      Xcol[i] = (f32x4){0.f, 0.f, 0.f, 0.f};
      if (i > k) {
        f32x4 M = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int j = 0; j < i; ++j) {
          if (j >= k) {
            const f32x4 a4 = *reinterpret_cast<const f32x4*>(Ab + bidx(i, j) * BLK + x16 * BP + 4 * g4);
            f32x4 b4 = Xcol[j];
            if (j == k) b4 = *reinterpret_cast<const f32x4*>(Xt + k * BLK + x16 * BP + 4 * g4);
#pragma unroll
            for (int st = 0; st < 4; ++st) M = __builtin_amdgcn_mfma_f32_16x16x4f32(a4[st], b4[st], M, 0, 0, 0);
          }
        }
        const f32x4 d4 = *reinterpret_cast<const f32x4*>(Xb + bidx(i, i) * BLK + x16 * BP + 4 * g4);
        f32x4 Xa = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int st = 0; st < 4; ++st) Xa = __builtin_amdgcn_mfma_f32_16x16x4f32(d4[st], M[st], Xa, 0, 0, 0);
        Xcol[i] = (f32x4){-Xa[0], -Xa[1], -Xa[2], -Xa[3]};
        float* Xo = Xb + bidx(i, k) * BLK;
#pragma unroll
        for (int r = 0; r < 4; ++r) Xo[(4 * g4 + r) * BP + x16] = Xcol[i][r];
      }
    }
  }
  __syncthreads();
  // TmB = Tm * diag(beta), bf16, in the scan kernel's A-operand order (see above): this thread's 16 columns are one
  // half (cb % 2) of the 32 tokens of operand (row / 16, cb / 2); columns 4g..4g+3 of them are the lower (upper) 8 bytes
  // of scan-lane group g.  Blocks above the diagonal are zero; operands (0,1), (1,1) are not stored at all.
  {
    const int row = tid >> 2, cb = tid & 3;
    if (!((row >> 4) < 2 && cb >= 2)) {
      float x[16];
#pragma unroll
      for (int e4 = 0; e4 < 4; ++e4) {
        const f32x4 xv = cb <= (row >> 4) ? *reinterpret_cast<const f32x4*>(Xb + bidx(row >> 4, cb <= (row >> 4) ? cb : 0) * BLK + (row & 15) * BP + 4 * e4)
                                          : (f32x4){0.f, 0.f, 0.f, 0.f};
        const f32x4 bv = *reinterpret_cast<const f32x4*>(bet + 16 * cb + 4 * e4);
#pragma unroll
        for (int e = 0; e < 4; ++e) x[4 * e4 + e] = xv[e] * bv[e];
      }
      bf16_t* trow = Tout + ((size_t)((2 * (row >> 4) + (cb >> 1)) * 64 + (row & 15))) * 8 + 4 * (cb & 1);
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        u32x2 w;
        w[0] = pack_bf16x2(x[4 * g], x[4 * g + 1]);
        w[1] = pack_bf16x2(x[4 * g + 2], x[4 * g + 3]);
        *reinterpret_cast<u32x2*>(trow + g * 128) = w;
      }
    }
  }
}

// The Mamba form needs no Gram products ahead of the scan (its intra-chunk matrix is formed in the scan from the k, q tiles
// that are in LDS anyway): what is left of the prep is the chunk's scale vectors, one wave per chunk-head, nothing read
// but g and the block type:  sc = { gamma log2(e), scale e^{gamma}, e^{min(gamma_last - gamma, 0)}, {e^{gamma_last}, gamma_last, is_linear} }.
__global__ __launch_bounds__(256) void mamba_scale_kernel(const LinearParams p) {
  const int lane = threadIdx.x & 63;
  const long long unit = (long long)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (unit >= (long long)p.total_chunks * p.H) return;
  const int gc = (int)(unit / p.H), h = (int)(unit % p.H);
  int bos, len, c, bos_nats;
  if (p.seqs == nullptr) {
    const int n = gc / p.nt;
    c = gc - n * p.nt;
    bos = n * p.T;
    len = p.T;
    bos_nats = n * p.TN;
  } else {
    int n = 0;
    for (int i = 1; i < p.n_seqs; ++i)
      if (p.seqs[i].chunk_off <= gc) n = i;
    c = gc - p.seqs[n].chunk_off;
    bos = p.seqs[n].bos;
    len = p.seqs[n].eos - bos;
    bos_nats = p.seqs[n].bos_nats;
  }
  const int t0 = c * C;
  float x = t0 + lane < len ? p.g[(size_t)(bos + t0 + lane) * p.H + h] : 0.f;
#pragma unroll
  for (int d = 1; d < 64; d <<= 1) {
    const float y = __shfl_up(x, d);
    if (lane >= d) x += y;
  }
  const float gl = __shfl(x, C - 1);
  float* Sout = p.ws_sc + (size_t)unit * (4 * C);
  Sout[lane] = x * 1.4426950408889634f;   // in log2 units: the scan forms e^{gamma_i - gamma_j} with one exp2 per element
  Sout[C + lane] = p.scale * __expf(x);
  Sout[2 * C + lane] = __expf(fminf(gl - x, 0.f));  // src/nats/ops/mamba/chunk_h.py:177
  if (lane == 0) Sout[3 * C] = __expf(gl);
  if (lane == 1) Sout[3 * C + 1] = gl;
  if (lane == 2) {
    const int hn = h / (p.H / p.HN);
    Sout[3 * C + 2] = lin_type(p.types, p.types_dtype, ((size_t)(bos_nats + (c * C) / p.block) * p.HN + hn) * 2 + 1) ? 1.f : 0.f;
  }
}

// =============================================================================================
// scan
// =============================================================================================
// one DMA instruction: lane l copies 16 bytes from base + voff to LDS byte address lds + 16 l
NATSL_DEVICE void dma16(const void* base, const unsigned voff, const unsigned lds) {
  asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1" ::"v"(voff), "s"(base), "s"(lds) : "memory", "m0");
}

// Swizzle of the k / q tiles in LDS (row-major, unpadded, rows of DK bf16): 16-byte segment s of row r sits at
// s ^ kq_swizzle(r).  The A-operand read of a 16x16x32 instruction (16 lanes = 16 consecutive rows at one segment) and
// the transposing read of k^T (16 lanes = 4 consecutive rows x 4 segments 0..3 of an aligned group) must both fall on
// 16 different 16-byte slots of the 256-byte bank period.
template <int DK>
NATSL_DEVICE int kq_swizzle(const int r) {
  if constexpr (DK == 128) return ((r & 3) << 2) | ((r >> 2) & 3);   // 16 segments per row, a row = one bank period
  return (r >> 1) & 7;                                               // 8 or 24 segments per row: low three bits only
}

typedef __attribute__((address_space(3))) const bf16x8* lds_b128_t;
typedef __attribute__((address_space(3))) const f32x4* lds_f4_t;
typedef __attribute__((address_space(3))) const float* lds_f1_t;
typedef __attribute__((address_space(3))) s16x4* lds_tr_t;
typedef __attribute__((address_space(3))) bf16_t* lds_h_t;
typedef __attribute__((address_space(3))) const u32x4* lds_u4_t;

NATSL_DEVICE s16x4 lds_tr4_at(const unsigned addr) {
  return __builtin_amdgcn_ds_read_tr16_b64_v4i16(reinterpret_cast<lds_tr_t>(addr));
}

// LDS layout of the scan kernel: two or three stages and two output tiles.
template <int DK, int NW, bool PF = false, bool XVEC = false>
struct ScanLds {
  static constexpr int BVW = 16 * NW;                 // state columns of the workgroup
  static constexpr int KROW = DK * 2;                 // bytes per k / q row
  static constexpr int VROW = BVW * 2;                // bytes per v row
  // (with PF, P is formed and used within one step: one area for all stages, behind them; XVEC: two more scale vectors arrive)
  static constexpr int KB = 64 * KROW, VB = 64 * VROW, TB = 6 * 1024, PB = PF ? 0 : 6 * 1024, SCB = XVEC ? 2048 : 1024;
  static constexpr int PSHARED = PF ? 6 * 1024 : 0;
  static constexpr int OFF_K = 0, OFF_Q = OFF_K + KB, OFF_V = OFF_Q + KB, OFF_T = OFF_V + VB, OFF_P = OFF_T + TB, OFF_SC = OFF_P + PB;
  static constexpr int STAGE = OFF_SC + SCB;
  static constexpr int OROW = VROW + 16;              // output tile row pitch (bytes)
  static constexpr int OB = 64 * OROW;
  // Stages: chunk c lives in stage c % NSTAGE.  Three when they fit (narrow workgroups): the requests of chunk c + 2
  // are issued in step c and have a whole step more to land; two otherwise (requests of chunk c + 1 in step c).
  static constexpr int NSTAGE = 3 * STAGE + PSHARED + 2 * OB <= 160 * 1024 ? 3 : 2;
  static constexpr int OFF_PS = NSTAGE * STAGE;          // the shared P area (PF)
  static constexpr int OFF_OUT = OFF_PS + PSHARED;       // the two output tiles
  static constexpr int TOTAL = OFF_OUT + 2 * OB;
};

// index of A operand (t, s) of TmB / P among the six that are stored (the two above the diagonal are skipped)
NATSL_DEVICE constexpr int tri_slot(const int t, const int s) { return t < 2 ? t : 2 * t - 2 + s; }

// Registers per wave: with DK <= 128 the kernel fits 256, so it asks for the two-waves-per-SIMD register budget even though
// LDS admits one workgroup per CU: within that budget the matrix instructions take their accumulators in ordinary vector
// registers and the state can be scaled and rounded in place (with the larger budget the compiler moves accumulators to the
// second register file and every vector operation on the state costs two extra copies).
#define NATSL_SCAN_FITS_256(DK) ((DK) <= 128)
#define NATSL_SCAN_ATTR(DK, NW) \
  __launch_bounds__(64 * ((NW) + 2)) __attribute__((amdgpu_waves_per_eu(NATSL_SCAN_FITS_256(DK) ? 2 : 1, NATSL_SCAN_FITS_256(DK) ? 2 : 1)))

// NW compute waves (16 state columns each) + two data-movement waves.
// PF (the Mamba form always; the delta rule in its four-wave shape when the launch asks for it): P does not come from the
// workspace; the two data-movement waves form it from the stage's k and q tiles while the compute waves work on the state (two
// of the four row tiles each, written to one P area shared by all stages); for the delta rule they also take the q rows'
// reciprocal norms from the operands they read for that and complete sq.  A second barrier in the middle of the step hands it
// over.
// NF = 2 (with four compute waves): two more waves that do nothing but form P (waves NW + 2, NW + 3), so that this work sits on
// the two SIMDs that host no data-movement wave; with NF = 0 the data-movement waves form P themselves (they have a SIMD of
// their own when there are one or two compute waves).
template <int DK, bool DELTA, int NW, bool PF, int NF = 0>
__global__ NATSL_SCAN_ATTR(DK, NW + NF) void linear_scan_kernel(const LinearParams p) {
  static_assert(NF == 0 || (NF == 2 && PF), "the extra waves only form P");
  static_assert(!PF || !DELTA || NW == 4, "the delta rule's P is formed by the data-movement waves only in the four-wave shape");
  static_assert(PF || DELTA, "the Mamba form's P is always formed by the data-movement waves");
  using L = ScanLds<DK, NW, PF, PF && DELTA>;
  constexpr int KS = DK / 32;   // matrix k-steps over the key dimension
  constexpr int KT = DK / 16;   // 16-row state tiles
  extern __shared__ __align__(1024) unsigned char smem[];
  const unsigned lds0 = (unsigned)(size_t)smem;

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int i16 = lane & 15, g4 = lane >> 4;

  // ---- which (sequence, head, column slice): the slices of one chain sit on one XCD --------------
  const int nsplit = p.V / L::BVW;
  const int n_chains = (p.seqs ? p.n_seqs : p.B) * p.H;
  const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3;
  const int split = slot % nsplit;
  const int chain = (slot / nsplit) * 8 + xcd;
  if (chain >= n_chains) return;
  const int n = chain / p.H, h = chain % p.H;
  int bos, len, chunk_off;
  if (p.seqs == nullptr) {
    bos = n * p.T; len = p.T; chunk_off = n * p.nt;
  } else {
    bos = p.seqs[n].bos; len = p.seqs[n].eos - bos; chunk_off = p.seqs[n].chunk_off;
  }
  const int NT = (len + C - 1) / C;
  const int vcol0 = split * L::BVW;           // first column of the workgroup
  constexpr int VSEG = L::VROW / 16;          // 16-byte segments per v row (2, 4 or 8)
  auto v_swz = [](const int r) { return VSEG == 8 ? 2 * ((r >> 1) & 1) : 0; };   // rows 2 apart share banks when a row is 128 bytes
  // Output tile, TRANSPOSED in LDS: [column][64 tokens], rows of OT_ROW bytes: a compute lane writes the four tokens
  // 16 t + 4 g4 .. of its column with one 8-byte store; the data-movement wave reads it back with the transposing read.
  constexpr int OT_ROW = 2 * C + 16;
  static_assert(L::BVW * OT_ROW <= L::OB, "the transposed output tile fits the space of the row-major one");

  if (wave >= NW) {
    // ======================= the two data-movement waves ========================================================
    // Per step c: request chunk c + 1 into stage (c + 1) % 2 by LDS-DMA (wave NW: sc, k, q; wave NW + 1: v, TmB, P),
    // store the output tile of chunk c - 1 (wave NW + 1), wait for the requests, meet the barrier.  The compute waves
    // never touch global memory inside the loop.  (One wave issues about 1 KiB per 36 cycles; two share the 53 KiB.)
    const bool first = wave == NW;
    const bool moves = wave < NW + 2;                          // requests, output stores
    const bool forms = NF == 0 || wave >= NW + 2;              // P (with PF)
    const bool rows30 = ((wave - NW) & 1) == 0;                // which two row tiles of P this wave forms
    // (operand addresses of the k / q tiles and of a row of the scale vectors, as the compute waves use them below)
    unsigned a_kq[KS];
#pragma unroll
    for (int s = 0; s < KS; ++s) a_kq[s] = (unsigned)(i16 * L::KROW) + 16u * (unsigned)((4 * s + g4) ^ kq_swizzle<DK>(i16));
    const unsigned a_sc = 16u * g4;
    const bool l2n = (p.flags & NATSL_QK_L2NORM) != 0;
    const float log2_scale_m = __builtin_amdgcn_logf(p.scale);
    const size_t qk_pitch = (size_t)p.H * DK * 2, v_pitch = (size_t)p.H * p.V * 2;   // bytes per token
    const char* kb = reinterpret_cast<const char*>(p.k + ((size_t)bos * p.H + h) * DK);
    const ptrdiff_t q_minus_k = reinterpret_cast<const char*>(p.q) - reinterpret_cast<const char*>(p.k);
    const char* vb = reinterpret_cast<const char*>(p.v + ((size_t)bos * p.H + h) * p.V + vcol0);
    char* ob_g = reinterpret_cast<char*>(p.o + ((size_t)bos * p.H + h) * p.V + vcol0);
    const size_t unit0 = (size_t)chunk_off * p.H + h;
    const char* tb = reinterpret_cast<const char*>(p.ws_tm + unit0 * (C * C));
    const ptrdiff_t p_minus_t = reinterpret_cast<const char*>(p.ws_p) - reinterpret_cast<const char*>(p.ws_tm);
    const char* sb = reinterpret_cast<const char*>(p.ws_sc + unit0 * (4 * C));
    const size_t ws_step = (size_t)p.H * (C * C) * 2, sc_step = (size_t)p.H * (4 * C) * 4;
    const size_t qk_step = (size_t)C * qk_pitch, v_step = (size_t)C * v_pitch;

    // k, q tiles: piece u covers LDS bytes [1024 u, 1024 u + 1024) of the tile; lane l fills byte 1024 u + 16 l, i.e. row
    // (1024 u + 16 l) / KROW, position pos, with the source segment pos ^ swizzle(row).  v the same with its own geometry.
    constexpr int KQ_PIECES = L::KB / 1024, V_PIECES = L::VB / 1024;
    auto kq_src = [&](const int u, const int nvalid) -> unsigned {
      const int byte = 1024 * u + 16 * lane, row = byte / L::KROW, pos = (byte % L::KROW) / 16;
      return (unsigned)((size_t)min(row, nvalid - 1) * qk_pitch) + 16u * (unsigned)(pos ^ kq_swizzle<DK>(row));
    };
    auto v_src = [&](const int u, const int nvalid) -> unsigned {
      const int byte = 1024 * u + 16 * lane, row = byte / L::VROW, pos = (byte % L::VROW) / 16;
      return (unsigned)((size_t)min(row, nvalid - 1) * v_pitch) + 16u * (unsigned)(pos ^ v_swz(row));
    };
    unsigned kq_off[KQ_PIECES], v_off[V_PIECES];
#pragma unroll
    for (int u = 0; u < KQ_PIECES; ++u) kq_off[u] = kq_src(u, C);
#pragma unroll
    for (int u = 0; u < V_PIECES; ++u) v_off[u] = v_src(u, C);
    // workspace pieces are plain copies: lane l moves bytes [16 l, 16 l + 16) of each; TmB / P keep operands 0, 2, 4..7 of 8
    unsigned ws_off[6];
#pragma unroll
    for (int v = 0; v < 6; ++v) ws_off[v] = 16u * lane + 1024u * (v < 2 ? 2 * v : v + 2);

    auto request = [&](const int cc) __attribute__((always_inline)) {
      const unsigned st = lds0 + (cc % L::NSTAGE) * L::STAGE;
      const int nvalid = min(C, len - cc * C);
      if (nvalid < C) {
        // the sequence's ragged last chunk (at most once per chain): rows past the end are clamped
#pragma unroll
        for (int u = 0; u < KQ_PIECES; ++u) kq_off[u] = kq_src(u, nvalid);
#pragma unroll
        for (int u = 0; u < V_PIECES; ++u) v_off[u] = v_src(u, nvalid);
      }
      const char* qb = kb + q_minus_k;
      const char* pb = tb + p_minus_t;
      if (first) {
        // in the order the compute waves need them: sc, k (R = k S comes first), q
        dma16(sb, 16u * lane, st + L::OFF_SC);
        if (PF && DELTA) dma16(pb, 16u * lane, st + L::OFF_SC + 1024);   // the two exponent vectors (and 512 bytes nobody reads)
#pragma unroll
        for (int u = 0; u < KQ_PIECES; ++u) dma16(kb, kq_off[u], st + L::OFF_K + 1024 * u);
#pragma unroll
        for (int u = 0; u < KQ_PIECES; ++u) dma16(qb, kq_off[u], st + L::OFF_Q + 1024 * u);
      } else {
#pragma unroll
        for (int u = 0; u < V_PIECES; ++u) dma16(vb, v_off[u], st + L::OFF_V + 1024 * u);
        if (DELTA) {
#pragma unroll
          for (int v = 0; v < 6; ++v) dma16(tb, ws_off[v], st + L::OFF_T + 1024 * v);
        }
        if (DELTA && !PF) {
#pragma unroll
          for (int v = 0; v < 6; ++v) dma16(pb, ws_off[v], st + L::OFF_P + 1024 * v);
        }
      }
      kb += qk_step; vb += v_step; tb += ws_step; sb += sc_step;
    };

    // read-back of the output tile.  A 16-lane group covers 4 tokens x 16 or 32 columns: within it lane i'' names the four
    // tokens of one column and lane i receives four adjacent columns of token tok0 + i % 4 -- with 32 columns per group,
    // columns 8 (i / 4) .. + 3 from the first read and the next four from the second (one 16-byte store); with 16
    // columns per group (one-wave workgroups) columns 4 (i / 4) .. + 3 (one 8-byte store).
    constexpr bool WIDE = L::BVW >= 32;
    constexpr int GCOLS = WIDE ? 32 : 16, O_GROUPS = 16 * (L::BVW / GCOLS), O_PASSES = O_GROUPS / 4;
    unsigned o_lds[O_PASSES];
    unsigned o_glb[O_PASSES];
    int o_tok[O_PASSES];
#pragma unroll
    for (int j = 0; j < O_PASSES; ++j) {
      const int grp = 4 * j + g4;
      const int tok0 = 4 * (grp / (L::BVW / GCOLS)), cbase = GCOLS * (grp % (L::BVW / GCOLS));
      const int c_first = WIDE ? cbase + 8 * (i16 & 3) + (i16 >> 2) : cbase + 4 * (i16 & 3) + (i16 >> 2);
      o_lds[j] = (unsigned)(c_first * OT_ROW + 2 * tok0);
      o_tok[j] = tok0 + (i16 & 3);
      o_glb[j] = (unsigned)((size_t)o_tok[j] * v_pitch) + 2u * (unsigned)(cbase + (WIDE ? 8 : 4) * (i16 >> 2));
    }
    auto store_out = [&](const int cc) __attribute__((always_inline)) {
      const unsigned ob = lds0 + L::OFF_OUT + (cc & 1) * L::OB;
      const int nvalid = len - cc * C;
#pragma unroll
      for (int j = 0; j < O_PASSES; ++j) {
        if constexpr (WIDE) {
          const s16x4 lo = lds_tr4_at(ob + o_lds[j]), hi = lds_tr4_at(ob + o_lds[j] + 4 * OT_ROW);
          if (o_tok[j] < nvalid) *reinterpret_cast<bf16x8*>(ob_g + o_glb[j]) = join4(lo, hi);
        } else {
          const s16x4 w = lds_tr4_at(ob + o_lds[j]);
          if (o_tok[j] < nvalid) *reinterpret_cast<s16x4*>(ob_g + o_glb[j]) = w;
        }
      }
      ob_g += v_step;
    };

    // AHEAD = how many chunks the requests run ahead of the compute waves.  With AHEAD = 2 the newest requests (and the
    // stores issued after them) may still be in flight at the barrier: vector memory operations complete in the order
    // they were issued, so allowing as many outstanding as one step issues leaves exactly the older step's complete.
    constexpr int AHEAD = L::NSTAGE - 1;
    constexpr int PER_STEP_FIRST = 1 + (PF && DELTA ? 1 : 0) + 2 * KQ_PIECES, PER_STEP_SECOND = V_PIECES + (DELTA ? (PF ? 6 : 12) : 0) + O_PASSES;
    static_assert(PER_STEP_FIRST <= 63 && PER_STEP_SECOND <= 63, "the wait counter has six bits");
    constexpr int VM_FIRST = (PER_STEP_FIRST & 15) | ((PER_STEP_FIRST >> 4) << 14) | 0x0f70;
    constexpr int VM_SECOND = (PER_STEP_SECOND & 15) | ((PER_STEP_SECOND >> 4) << 14) | 0x0f70;
    if (moves) {
#pragma unroll
      for (int a = 0; a < AHEAD; ++a)
        if (a < NT) request(a);
    }
    __builtin_amdgcn_s_waitcnt(0x0f70);
    __syncthreads();
    if constexpr (PF) {
      // P = scale tril(rq_i rk_j (q_i . k_j) e^{gamma_i - gamma_j}) of chunk c is formed HERE, from the tiles of chunk c's stage,
      // while the compute waves work on the state.  Z^T = k_tile(t2) q_tile(t)^T leaves lane (i16, g4) with query 16 t + i16
      // against keys 16 t2 + 4 g4 .. + 3: the four slots this lane holds of A operand (t, t2 / 2), half t2 % 2.  Each of the two
      // waves forms the operands of two row tiles (five of the ten tiles) and completes sq = scale e^{gamma} / |q| for their
      // rows; |q_i|^2 is the diagonal of q_tile q_tile^T (a lane's 16 bytes are the same slots of its row as A and as B
      // operand), found in lane group i16 / 4, register i16 % 4.
      // Both rows of a wave go through ONE straight piece of code: every operand read first (the k tiles are shared by the two
      // rows), then the matrix instructions of all chains interleaved, then the exponentials, then the stores.  The row norm
      // multiplies at the end, so the exponentials do not wait for it.
      auto form_two_rows = [&](const int ta, const int tb_, const unsigned st) __attribute__((always_inline)) {
        const int tmax = ta > tb_ ? ta : tb_;
        const int tr[2] = {ta, tb_};
        bf16x8 qb[2][KS], ka[4][KS];
#pragma unroll
        for (int w = 0; w < 2; ++w)
#pragma unroll
          for (int s = 0; s < KS; ++s) qb[w][s] = *reinterpret_cast<lds_b128_t>(st + L::OFF_Q + a_kq[s] + tr[w] * 16 * L::KROW);
#pragma unroll
        for (int t2 = 0; t2 < 4; ++t2)
#pragma unroll
          for (int s = 0; s < KS; ++s)
            if (t2 <= tmax) ka[t2][s] = *reinterpret_cast<lds_b128_t>(st + L::OFF_K + a_kq[s] + t2 * 16 * L::KROW);
        // the exponents: two vectors of their own from the delta rule's prep; gamma log2(e) (vector 0) for both in the Mamba form
        constexpr int GK_ROW = DELTA ? 4 : 0, GQ_ROW = DELTA ? 5 : 0;
        f32x4 gj[4];
#pragma unroll
        for (int t2 = 0; t2 < 4; ++t2)
          if (t2 <= tmax) gj[t2] = *reinterpret_cast<lds_f4_t>(st + L::OFF_SC + 4 * (GK_ROW * C) + a_sc + 64 * t2);
        float gq[2], sq0[2];
#pragma unroll
        for (int w = 0; w < 2; ++w) {
          gq[w] = *reinterpret_cast<lds_f1_t>(st + L::OFF_SC + 4 * (GQ_ROW * C + 16 * tr[w] + i16)) + (DELTA ? 0.f : log2_scale_m);
          sq0[w] = DELTA ? *reinterpret_cast<lds_f1_t>(st + L::OFF_SC + 4 * (C + 16 * tr[w] + i16)) : 0.f;
        }
        f32x4 D[2], Z[2][4];
#pragma unroll
        for (int w = 0; w < 2; ++w) {
          D[w] = (f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
          for (int t2 = 0; t2 < 4; ++t2) Z[w][t2] = (f32x4){0.f, 0.f, 0.f, 0.f};
        }
#pragma unroll
        for (int s = 0; s < KS; ++s)
#pragma unroll
          for (int w = 0; w < 2; ++w) {
            if (DELTA) D[w] = mfma16(qb[w][s], qb[w][s], D[w]);
#pragma unroll
            for (int t2 = 0; t2 < 4; ++t2)
              if (t2 <= tr[w]) Z[w][t2] = mfma16(ka[t2][s], qb[w][s], Z[w][t2]);
          }
        const int rsel = i16 & 3;
        float rqi[2];
#pragma unroll
        for (int w = 0; w < 2; ++w) {
          rqi[w] = 1.f;
          if (DELTA) {
            const float dsel = rsel == 0 ? D[w][0] : rsel == 1 ? D[w][1] : rsel == 2 ? D[w][2] : D[w][3];
            const float ss = __shfl(dsel, 16 * (i16 >> 2) + i16);
            rqi[w] = l2n ? rsqrtf(ss + 1e-6f) : 1.f;
          }
        }
#pragma unroll
        for (int w = 0; w < 2; ++w)
#pragma unroll
          for (int t2 = 0; t2 < 4; ++t2)
            if (t2 <= tr[w]) {
#pragma unroll
              for (int r = 0; r < 4; ++r) {
                const float e = Z[w][t2][r] * __builtin_amdgcn_exp2f(gq[w] - gj[t2][r]);
                Z[w][t2][r] = (t2 < tr[w] || i16 >= 4 * g4 + r) ? e * rqi[w] : 0.f;
              }
            }
#pragma unroll
        for (int w = 0; w < 2; ++w) {
#pragma unroll
          for (int sp = 0; sp < 2; ++sp)
            if (2 * sp <= tr[w])
              *reinterpret_cast<__attribute__((address_space(3))) bf16x8*>(lds0 + L::OFF_PS + 1024 * tri_slot(tr[w], sp) + 16 * lane) = pack8(Z[w][2 * sp], Z[w][2 * sp + 1]);
          if (DELTA && g4 == 0) {
            typedef __attribute__((address_space(3))) float* lds_fw_t;
            *reinterpret_cast<lds_fw_t>(st + L::OFF_SC + 4 * (C + 16 * tr[w] + i16)) = sq0[w] * rqi[w];
          }
        }
      };
      for (int c = 0; c < NT; ++c) {
        // requests go into the stage that step c - 1 read: every wave is past the barrier that ended it
        const bool more = c + AHEAD < NT;
        const unsigned st = lds0 + (c % L::NSTAGE) * L::STAGE;
        if (moves) {
          if (more) request(c + AHEAD);
          if (c > 0 && !first) store_out(c - 1);
        }
        if (forms) {
          // five tiles each: rows 48..63 and 0..15 here, rows 32..47 and 16..31 there
          if (rows30) form_two_rows(3, 0, st);
          else form_two_rows(2, 1, st);
        }
        __syncthreads();   // hand-over of P and sq in the middle of the compute waves' step
        if (AHEAD == 2 && more && moves) {
          if (first) __builtin_amdgcn_s_waitcnt(VM_FIRST);
          else __builtin_amdgcn_s_waitcnt(VM_SECOND);
        } else {
          __builtin_amdgcn_s_waitcnt(0x0f70);
        }
        __syncthreads();
      }
    } else {
      for (int c = 0; c < NT; ++c) {
        // into the stage that step c - 1 read: every wave is past the barrier that ended it
        const bool more = c + AHEAD < NT;
        if (more) request(c + AHEAD);
        if (c > 0 && !first) store_out(c - 1);
        if (AHEAD == 2 && more) {
          if (first) __builtin_amdgcn_s_waitcnt(VM_FIRST);
          else __builtin_amdgcn_s_waitcnt(VM_SECOND);
        } else {
          __builtin_amdgcn_s_waitcnt(0x0f70);
        }
        __syncthreads();
      }
    }
    if (NT > 0 && !first && moves) store_out(NT - 1);
    return;
  }

  // ======================= compute waves ===========================================================================
  const int per_blk = p.block / C;
  const bool decay = (p.flags & NATSL_DECAY_NON_LINEAR) != 0;
  const bool intra = (p.flags & NATSL_INTRA_CHUNK) != 0;
  const int col = vcol0 + 16 * wave + i16;    // this lane's state column

  // ---- state: tile m, lane group g4, register r holds K row krow_of(m, r), column `col` -----------------
  // (two tiles 2s, 2s+1 side by side are the eight contraction slots of k-step s: rows 32s + 8 g4 + 0..7, which is what a
  // 16-byte read of a k or q row delivers)
  auto krow_of = [&](const int m, const int r) { return 32 * (m >> 1) + 8 * g4 + 4 * (m & 1) + r; };
  f32x4 S[KT], Ssave[KT];
#pragma unroll
  for (int m = 0; m < KT; ++m)
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      S[m][r] = p.h0 ? p.h0[((size_t)chain * DK + krow_of(m, r)) * p.V + col] : 0.f;
      Ssave[m][r] = 0.f;
    }

  // ---- per-lane operand addresses inside a stage ------------------------------------------------------------------
  // k / q as A operand (token tile t, k-step s): row 16 t + i16, segment 4 s + g4 (swizzled); t goes into the offset field
  unsigned a_kq[KS];
#pragma unroll
  for (int s = 0; s < KS; ++s) a_kq[s] = (unsigned)(i16 * L::KROW) + 16u * (unsigned)((4 * s + g4) ^ kq_swizzle<DK>(i16));
  // k^T as A operand (state tile m, token k-step s2, read rd): lane i16 addresses token 32 s2 + 16 rd + 4 g4 + i16 / 4,
  // the four K rows 32 (m / 2) + 8 (i16 % 4) + 4 (m % 2) ..: segment 4 (m / 2) + i16 % 4, half m % 2
  unsigned a_kt[KT / 2];
  {
    const int tok = 4 * g4 + (i16 >> 2);
#pragma unroll
    for (int mh = 0; mh < KT / 2; ++mh)
      a_kt[mh] = (unsigned)(tok * L::KROW) + 16u * (unsigned)((4 * mh + (i16 & 3)) ^ kq_swizzle<DK>(tok));
  }
  // v through the transposing read (token tile t): lane i16 addresses token 16 t + 4 g4 + i16 / 4, columns 16 wave + 4 (i16 % 4)..
  unsigned a_v;
  {
    const int tok = 4 * g4 + (i16 >> 2), seg = 2 * wave + ((i16 & 3) >> 1);
    a_v = (unsigned)(tok * L::VROW) + 16u * (unsigned)(seg ^ v_swz(tok)) + 8u * (i16 & 1);
  }
  const unsigned a_o = (unsigned)((16 * wave + i16) * OT_ROW + 8 * g4);
  const unsigned a_sc = 16u * g4;    // this lane group's four tokens in a row of sc

  float gsum = 0.f;
  __syncthreads();   // chunk 0 has landed

  for (int c = 0; c < NT; ++c) {
    const unsigned st = lds0 + (c % L::NSTAGE) * L::STAGE;
    // the chunk's scalars (three separate 4-byte reads on purpose: read as one 16-byte vector whose lanes all name the
    // same address, the compiler folded the three elements into the first)
    const float dec_v = *reinterpret_cast<lds_f1_t>(st + L::OFF_SC + 4 * (3 * C));
    const float glast_v = *reinterpret_cast<lds_f1_t>(st + L::OFF_SC + 4 * (3 * C + 1));
    const float linf_v = *reinterpret_cast<lds_f1_t>(st + L::OFF_SC + 4 * (3 * C + 2));
    // (1) the state as B operands
    bf16x8 SB[KS];
#pragma unroll
    for (int s = 0; s < KS; ++s) SB[s] = pack8(S[2 * s], S[2 * s + 1]);
    if (p.s_out) {
      // a B operand is eight consecutive K rows of this lane's column: 16 contiguous bytes of S^T [V][K]
      bf16_t* so = p.s_out + (((size_t)(chunk_off + c) * p.H + h) * p.V + col) * DK + 8 * g4;
#pragma unroll
      for (int s = 0; s < KS; ++s) *reinterpret_cast<bf16x8*>(so + 32 * s) = SB[s];
    }
    const float dec_c = __builtin_bit_cast(float, __builtin_amdgcn_readfirstlane(__builtin_bit_cast(int, dec_v)));
    const float glast_c = __builtin_bit_cast(float, __builtin_amdgcn_readfirstlane(__builtin_bit_cast(int, glast_v)));
    const float linf_c = __builtin_bit_cast(float, __builtin_amdgcn_readfirstlane(__builtin_bit_cast(int, linf_v)));
    const bool last_of_block = ((c + 1) % per_blk == 0) || (c == NT - 1);
    const bool keep = linf_c != 0.f || !last_of_block;
    if (c % per_blk == 0) {
      // The state that enters a block is needed again when the block is rolled back at its end (not typed linear) and
      // for the hand-off output (the sequence's last block).  The type is the same for every chunk of a block.
      if (linf_c == 0.f || c + per_blk >= NT) {
#pragma unroll
        for (int m = 0; m < KT; ++m) Ssave[m] = S[m];
      }
      gsum = 0.f;
    }
    gsum += glast_c;

    // R = k S, then O1 = q S (X below only needs R); operands are read AHEAD instructions before their use.  The state's
    // decay for the update at the end of the step rides along, one multiply under each matrix instruction (a step that
    // ends in a roll-back overwrites the state anyway).
    f32x4 R[4], O1[4];
#pragma unroll
    for (int t = 0; t < 4; ++t) { R[t] = (f32x4){0.f, 0.f, 0.f, 0.f}; O1[t] = (f32x4){0.f, 0.f, 0.f, 0.f}; }
    {
      constexpr int NOP = (DELTA ? 2 : 1) * 4 * KS, AHEAD = 4, NS = 4 * KT, PER = (NS + NOP - 1) / NOP;
      auto ld_op = [&](const int j) __attribute__((always_inline)) -> bf16x8 {
        const int which = DELTA ? j / (4 * KS) : 1, jj = j % (4 * KS), s = jj / 4, t = jj % 4;
        return *reinterpret_cast<lds_b128_t>(st + (which ? L::OFF_Q : L::OFF_K) + a_kq[s] + t * 16 * L::KROW);
      };
      bf16x8 opnd[NOP + AHEAD];
#pragma unroll
      for (int j = 0; j < AHEAD; ++j) opnd[j] = ld_op(j);
#pragma unroll
      for (int j = 0; j < NOP; ++j) {
        if (j + AHEAD < NOP) opnd[j + AHEAD] = ld_op(j + AHEAD);
        const int which = DELTA ? j / (4 * KS) : 1, jj = j % (4 * KS), s = jj / 4, t = jj % 4;
        if (which) O1[t] = mfma16(opnd[j], SB[s], O1[t]);
        else R[t] = mfma16(opnd[j], SB[s], R[t]);
#pragma unroll
        for (int e = PER * j; e < PER * j + PER && e < NS; ++e) S[e >> 2][e & 3] *= dec_c;
      }
    }
    // (2) v in accumulator layout (lane = column, registers = tokens 16 t + 4 g4 + r); zero past the end of the sequence
    f32x4 VN[4];
    const int nvalid = len - c * C;
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      const s16x4 vv = lds_tr4_at(st + L::OFF_V + a_v + t * 16 * L::VROW);
#pragma unroll
      for (int r = 0; r < 4; ++r) VN[t][r] = bf16_to_f32((bf16_t)vv[r]);
    }
    if (__builtin_expect(nvalid < C, 0)) {
      asm volatile("" ::: "memory");   // (keeps this a branch: it runs once per chain)
#pragma unroll
      for (int t = 0; t < 4; ++t)
#pragma unroll
        for (int r = 0; r < 4; ++r)
          if (16 * t + 4 * g4 + r >= nvalid) VN[t][r] = 0.f;
    }
    if (DELTA) {
      // X = v - se * R;  v_new = TmB X
      f32x4 se[4];
      bf16x8 TA[6];
#pragma unroll
      for (int t = 0; t < 4; ++t) se[t] = *reinterpret_cast<lds_f4_t>(st + L::OFF_SC + a_sc + 64 * t);
#pragma unroll
      for (int v = 0; v < 6; ++v) TA[v] = *reinterpret_cast<lds_b128_t>(st + L::OFF_T + 1024 * v + 16 * lane);
#pragma unroll
      for (int t = 0; t < 4; ++t)
#pragma unroll
        for (int r = 0; r < 4; ++r) VN[t][r] -= se[t][r] * R[t][r];
      const bf16x8 XB[2] = {pack8(VN[0], VN[1]), pack8(VN[2], VN[3])};
      const f32x4 zero = {0.f, 0.f, 0.f, 0.f};
      VN[0] = mfma16(TA[tri_slot(0, 0)], XB[0], zero);
      VN[1] = mfma16(TA[tri_slot(1, 0)], XB[0], zero);
      VN[2] = mfma16(TA[tri_slot(2, 0)], XB[0], zero);
      VN[3] = mfma16(TA[tri_slot(3, 0)], XB[0], zero);
      VN[2] = mfma16(TA[tri_slot(2, 1)], XB[1], VN[2]);
      VN[3] = mfma16(TA[tri_slot(3, 1)], XB[1], VN[3]);
    }
    // (3) state update / roll-back (the next step waits for it: before the output)
    const bf16x8 VB[2] = {pack8(VN[0], VN[1]), pack8(VN[2], VN[3])};
    if (DELTA && p.vn_out) {
#pragma unroll
      for (int t = 0; t < 4; ++t)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const int tok = 16 * t + 4 * g4 + r;
          if (tok < nvalid) p.vn_out[((size_t)(bos + c * C + tok) * p.H + h) * p.V + col] = f32_to_bf16(VN[t][r]);
        }
    }
    if (keep) {
      f32x4 W[4];
#pragma unroll
      for (int t = 0; t < 4; ++t) {
        const f32x4 sk = *reinterpret_cast<lds_f4_t>(st + L::OFF_SC + 4 * (2 * C) + a_sc + 64 * t);
#pragma unroll
        for (int r = 0; r < 4; ++r) W[t][r] = VN[t][r] * sk[r];
      }
      const bf16x8 WB[2] = {pack8(W[0], W[1]), pack8(W[2], W[3])};
      constexpr int NOP = 2 * KT, AHEAD = 4;
      auto ld_kt = [&](const int j) __attribute__((always_inline)) -> bf16x8 {
        const int s = j / KT, m = j % KT;
        const unsigned a = st + L::OFF_K + a_kt[m >> 1] + 8u * (m & 1) + (32 * s) * L::KROW;
        return join4(lds_tr4_at(a), lds_tr4_at(a + 16 * L::KROW));
      };
      bf16x8 opnd[NOP + AHEAD];
#pragma unroll
      for (int j = 0; j < AHEAD; ++j) opnd[j] = ld_kt(j);
#pragma unroll
      for (int j = 0; j < NOP; ++j) {
        if (j + AHEAD < NOP) opnd[j + AHEAD] = ld_kt(j + AHEAD);
        S[j % KT] = mfma16(opnd[j], WB[j / KT], S[j % KT]);
      }
    } else {
      const float f = decay ? __expf(gsum) : 1.f;
#pragma unroll
      for (int m = 0; m < KT; ++m)
#pragma unroll
        for (int r = 0; r < 4; ++r) S[m][r] = Ssave[m][r] * f;
    }
    // (4) o = sq * O1 + P v_new, into the (transposed) output tile: the four token tiles side by side
    if constexpr (PF) __syncthreads();   // P and sq of this step are complete
    {
      const unsigned ob = lds0 + L::OFF_OUT + (c & 1) * L::OB;
      f32x4 O[4];
      bf16x8 PA[6];
#pragma unroll
      for (int t = 0; t < 4; ++t) O[t] = *reinterpret_cast<lds_f4_t>(st + L::OFF_SC + 4 * C + a_sc + 64 * t);
      if (intra) {
#pragma unroll
        for (int v = 0; v < 6; ++v) PA[v] = *reinterpret_cast<lds_b128_t>((PF ? lds0 + L::OFF_PS : st + L::OFF_P) + 1024 * v + 16 * lane);
      }
#pragma unroll
      for (int t = 0; t < 4; ++t)
#pragma unroll
        for (int r = 0; r < 4; ++r) O[t][r] *= O1[t][r];
      if (intra) {
        O[0] = mfma16(PA[tri_slot(0, 0)], VB[0], O[0]);
        O[1] = mfma16(PA[tri_slot(1, 0)], VB[0], O[1]);
        O[2] = mfma16(PA[tri_slot(2, 0)], VB[0], O[2]);
        O[3] = mfma16(PA[tri_slot(3, 0)], VB[0], O[3]);
        O[2] = mfma16(PA[tri_slot(2, 1)], VB[1], O[2]);
        O[3] = mfma16(PA[tri_slot(3, 1)], VB[1], O[3]);
      }
#pragma unroll
      for (int t = 0; t < 4; ++t) {
        u32x2 w;
        w[0] = pack_bf16x2(O[t][0], O[t][1]);
        w[1] = pack_bf16x2(O[t][2], O[t][3]);
        *reinterpret_cast<__attribute__((address_space(3))) u32x2*>(ob + a_o + 32 * t) = w;
      }
    }
    // every wave is done with this stage and has written its part of the output tile; the data-movement wave has
    // waited for the next chunk's inputs
    __syncthreads();
  }

  if (p.hs) {
    // Ssave / gsum still belong to the last block: the state that entered it and its total log-decay
#pragma unroll
    for (int m = 0; m < KT; ++m)
#pragma unroll
      for (int r = 0; r < 4; ++r) p.hs[((size_t)chain * DK + krow_of(m, r)) * p.V + col] = Ssave[m][r];
    if (p.gs && split == 0 && tid == 0) p.gs[chain] = gsum;
  }
  if (p.ht) {
#pragma unroll
    for (int m = 0; m < KT; ++m)
#pragma unroll
      for (int r = 0; r < 4; ++r) p.ht[((size_t)chain * DK + krow_of(m, r)) * p.V + col] = S[m][r];
  }
}

constexpr size_t WS_UNIT_BYTES = (size_t)C * C * 2 * 2 + 4 * C * 4;

inline int cu_count_linear() {
  static int n = 0;
  if (n == 0) {
    int dev = 0;
    hipDeviceProp_t prop;
    if (hipGetDevice(&dev) == hipSuccess && hipGetDeviceProperties(&prop, dev) == hipSuccess) n = prop.multiProcessorCount;
    if (n <= 0) n = 256;
  }
  return n;
}

template <int DK, bool DELTA, int NW, bool PF, int NF = 0>
static int launch_scan(const LinearParams& p, hipStream_t stream, const char* what) {
  using L = ScanLds<DK, NW, PF, PF && DELTA>;
  auto kern = linear_scan_kernel<DK, DELTA, NW, PF, NF>;
  hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, L::TOTAL);
  if (e != hipSuccess) return fail(NATSL_ERR_LAUNCH, "%s: cannot reserve %d bytes of LDS: %s", what, L::TOTAL, hipGetErrorString(e));
  const int n_chains = (p.seqs ? p.n_seqs : p.B) * p.H;
  const int grid = 8 * cdiv(n_chains, 8) * (p.V / L::BVW);
  hipLaunchKernelGGL(kern, dim3(grid), dim3(64 * (NW + 2 + NF)), L::TOTAL, stream, p);
  return check_launch(what);
}

template <int DK, bool DELTA>
static int launch_linear(const LinearParams& p, hipStream_t stream, const char* what) {
  const long long units = (long long)p.total_chunks * p.H;
  if (units <= 0) return NATSL_OK;
  // Waves per workgroup (16 state columns each).  A CU holds one workgroup (LDS), so a launch takes
  // ceil(workgroups / CUs) rounds of the chain's length, and a step of a wider workgroup takes longer (measured: 2 700, 3 000,
  // 4 400 cycles for one, two, four waves): the width with the least rounds x step time.  (Wider also means a chunk's inputs
  // are staged once for more columns.)
  const long long n_chains = (long long)(p.seqs ? p.n_seqs : p.B) * p.H;
  const int cus = cu_count_linear();
  auto cost = [&](const int nw, const double step) {
    const long long wgs = n_chains * (p.V / (16 * nw));
    return (double)((wgs + cus - 1) / cus) * step;
  };
  // (K = 192: five waves of that size do not fit the registers of a CU without spilling; three do)
  const bool ok4 = DK <= 128 && p.V % 64 == 0, ok2 = p.V % 32 == 0;
  const double c1 = cost(1, 1.0), c2 = ok2 ? cost(2, 1.1) : 1e30, c4 = ok4 ? cost(4, 1.65) : 1e30;
  const int nw = (c4 <= c2 && c4 <= c1) ? 4 : (c2 <= c1 ? 2 : 1);
  // The delta rule's four-wave scan forms P itself and the prep reads k only, when the launch fills the machine: prep and scan
  // are then bound by their HBM traffic, which this cuts by a fifth (measured at B8 T8192 H16: 0.46 -> 0.43 ms), while a launch
  // that leaves CUs idle is bound by the scan's step and only gets slower from the extra work in it (B8 T4096 H6 V256:
  // 0.152 -> 0.176 ms; the narrower shapes likewise: 1.67 -> 1.90 ms at B1 T65536 H32 with one compute wave).  Not when the
  // caller wants the chunk states for a backward: the backward kernels read P and the complete scale vectors from the workspace.
  constexpr bool CAN_PF = DELTA && DK <= 128;
  const bool pf = CAN_PF && nw == 4 && p.s_out == nullptr && n_chains * (p.V / 64) >= cus;
  if constexpr (DELTA) {
    if (pf) {
      if constexpr (CAN_PF) hipLaunchKernelGGL((linear_prep_kernel<DK, true, true>), dim3((unsigned)units), dim3(256), 0, stream, p);
    } else {
      hipLaunchKernelGGL((linear_prep_kernel<DK, true, false>), dim3((unsigned)units), dim3(256), 0, stream, p);
    }
  } else {
    hipLaunchKernelGGL(mamba_scale_kernel, dim3((unsigned)((units + 3) / 4)), dim3(256), 0, stream, p);
  }
  int rc = check_launch(what);
  if (rc != NATSL_OK) return rc;
  if constexpr (!DELTA) {
    // the Mamba form's P is always formed by the data-movement waves (nothing about it comes from a prep kernel)
    // (four compute waves: two of them share their SIMD with a data-movement wave, so two more waves, on the other two
    // SIMDs, form P -- B8 T4096 H16 d128: 137 -> 132 us; the delta rule at B8 T8192 H16: 428 -> 398 us)
    if (nw == 4) return launch_scan<DK <= 128 ? DK : 128, false, 4, true, 2>(p, stream, what);
    if (nw == 2) return launch_scan<DK, false, 2, true>(p, stream, what);
    return launch_scan<DK, false, 1, true>(p, stream, what);
  } else {
    if (nw == 4) {
      if constexpr (CAN_PF) {
        if (pf) return launch_scan<DK, true, 4, true, 2>(p, stream, what);
      }
      return launch_scan<DK <= 128 ? DK : 128, true, 4, false>(p, stream, what);
    }
    if (nw == 2) return launch_scan<DK, true, 2, false>(p, stream, what);
    return launch_scan<DK, true, 1, false>(p, stream, what);
  }
}

static int linear_fwd(bool delta, const void* q, const void* k, const void* v, const float* g, const void* beta,
                      const float* h0, void* o, float* ht, float* hs, float* gs, void* chunk_states, void* chunk_v_new, const void* types, int types_dtype, int B, int T,
                      int H, int HN, int K, int V, int TN, int block, float scale, int flags, void* workspace, size_t workspace_bytes,
                      int dtype, const natsl_seq_row* seqs, int n_seqs, int total_units, natsl_stream_t stream) {
  const char* what = delta ? "natsl_gdn_chunk_fwd" : "natsl_mamba_chunk_fwd";
  if (!q || !k || !v || !g || !o || !types || (delta && !beta)) return fail(NATSL_ERR_INVALID, "%s: null pointer argument", what);
  if (dtype != NATSL_BF16) return fail(NATSL_ERR_UNSUPPORTED, "%s: only bf16 tensors are supported (got dtype %d)", what, dtype);
  if (types_dtype != NATSL_BF16 && types_dtype != NATSL_F32) return fail(NATSL_ERR_UNSUPPORTED, "%s: block types must be f32 or bf16", what);
  if (B <= 0 || T <= 0 || H <= 0 || HN <= 0 || TN <= 0) return fail(NATSL_ERR_INVALID, "%s: non-positive dimension", what);
  if (H % HN) return fail(NATSL_ERR_INVALID, "%s: H=%d must be a multiple of HN=%d", what, H, HN);
  if (block < 64 || block % 64) return fail(NATSL_ERR_UNSUPPORTED, "%s: block size %d must be a multiple of 64", what, block);
  if (V % 16 || V <= 0) return fail(NATSL_ERR_UNSUPPORTED, "%s: V=%d must be a multiple of 16", what, V);
  if (seqs ? (B != 1 || n_seqs <= 0 || total_units <= 0) : (TN != cdiv(T, block)))
    return fail(NATSL_ERR_INVALID, "%s: TN=%d does not match T=%d, block=%d (or bad packed-input arguments)", what, TN, T, block);
  LinearParams p;
  p.q = (const bf16_t*)q; p.k = (const bf16_t*)k; p.v = (const bf16_t*)v; p.g = g; p.beta = (const bf16_t*)beta;
  p.h0 = h0; p.o = (bf16_t*)o; p.ht = ht; p.hs = hs; p.gs = gs; p.s_out = (bf16_t*)chunk_states; p.vn_out = (bf16_t*)chunk_v_new; p.types = types; p.types_dtype = types_dtype;
  p.seqs = reinterpret_cast<const SeqRow*>(seqs); p.n_seqs = seqs ? n_seqs : 0;
  p.B = B; p.T = T; p.H = H; p.HN = HN; p.V = V; p.TN = TN; p.block = block;
  p.nt = cdiv(T, C);
  p.total_chunks = seqs ? total_units : B * p.nt;
  p.scale = scale; p.flags = flags;
  const size_t units = (size_t)p.total_chunks * H;
  const size_t need = natsl_linear_workspace_bytes(p.total_chunks, H);
  if (!workspace || workspace_bytes < need) return fail(NATSL_ERR_WORKSPACE, "%s: workspace of %zu bytes needed, %zu given", what, need, workspace_bytes);
  if (reinterpret_cast<uintptr_t>(workspace) & 255) return fail(NATSL_ERR_INVALID, "%s: workspace must be 256-byte aligned", what);
  p.ws_tm = reinterpret_cast<bf16_t*>(workspace);
  p.ws_p = p.ws_tm + units * (C * C);
  p.ws_sc = reinterpret_cast<float*>(p.ws_p + units * (C * C));
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  if (delta) {
    if (K == 128) return launch_linear<128, true>(p, s, what);
    if (K == 64) return launch_linear<64, true>(p, s, what);
    if (K == 192) return launch_linear<192, true>(p, s, what);
  } else {
    if (K == 128) return launch_linear<128, false>(p, s, what);
    if (K == 64) return launch_linear<64, false>(p, s, what);
    if (K == 192) return launch_linear<192, false>(p, s, what);
  }
  return fail(NATSL_ERR_UNSUPPORTED, "%s: key dim K=%d not built (supported: 64, 128, 192)", what, K);
}

}  // namespace natsl

using namespace natsl;

extern "C" size_t natsl_linear_workspace_bytes(int64_t total_chunks, int H) {
  if (total_chunks <= 0 || H <= 0) return 0;
  return (size_t)total_chunks * (size_t)H * WS_UNIT_BYTES;
}

extern "C" int natsl_gdn_chunk_fwd(const void* q, const void* k, const void* v, const float* g, const void* beta,
                                   const float* h0, void* o, float* ht, float* h_block_start, float* g_block_sum,
                                   void* chunk_states, void* chunk_v_new, const void* types, int types_dtype, int B, int T,
                                   int H, int HN, int K, int V, int TN, int block, float scale, int flags, void* workspace,
                                   size_t workspace_bytes, int dtype, const natsl_seq_row* seqs, int n_seqs, int total_units,
                                   natsl_stream_t stream) {
  return linear_fwd(true, q, k, v, g, beta, h0, o, ht, h_block_start, g_block_sum, chunk_states, chunk_v_new, types, types_dtype, B, T, H, HN, K, V, TN, block, scale, flags,
                    workspace, workspace_bytes, dtype, seqs, n_seqs, total_units, stream);
}

extern "C" int natsl_mamba_chunk_fwd(const void* q, const void* k, const void* v, const float* g, const float* h0, void* o,
                                     float* ht, float* h_block_start, float* g_block_sum, void* chunk_states, const void* types, int types_dtype, int B, int T, int H, int HN, int K, int V,
                                     int TN, int block, float scale, int flags, void* workspace, size_t workspace_bytes,
                                     int dtype, const natsl_seq_row* seqs, int n_seqs, int total_units,
                                     natsl_stream_t stream) {
  return linear_fwd(false, q, k, v, g, nullptr, h0, o, ht, h_block_start, g_block_sum, chunk_states, nullptr, types, types_dtype, B, T, H, HN, K, V, TN, block, scale,
                    flags & ~NATSL_QK_L2NORM, workspace, workspace_bytes, dtype, seqs, n_seqs, total_units, stream);
}
