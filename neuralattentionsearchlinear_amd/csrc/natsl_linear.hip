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
//   linear_scan_kernel   one workgroup per (sequence, head, 32-wide slice of V) walks the chunks
//                        in order with the state slice S[K][32] in fp32 registers:
//                          R = k S;  X = v - se*R;  v_new = TmB X               (delta rule)
//                          o = sq*(q S) + P v_new
//                          S <- e^{gamma_last} S + (sk*k)^T v_new               (blocks typed linear)
//                        q, k, TmB, P reach the matrix cores straight from global memory in
//                        A-operand layout; only what changes layout goes through LDS (S, X, v_new
//                        written transposed from the accumulator layout, k read back transposed
//                        with the transposing LDS load).  Raw q, k are used: the 1/norm factors
//                        are folded into the per-token scale vectors.
//                        A block that is not typed linear leaves S rolled back at its end (times
//                        e^{sum g} when decay is on), which is all the reference's carry logic
//                        (src/nats/ops/utils/cumsum.py:95-133) amounts to.
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
constexpr int BV = 32;

NATSL_DEVICE bool lin_type(const void* types, int dtype, size_t i) {
  float x = dtype == NATSL_F32 ? reinterpret_cast<const float*>(types)[i]
                               : bf16_to_f32(reinterpret_cast<const bf16_t*>(types)[i]);
  return rintf(x) == 1.0f;
}

// =============================================================================================
// prep
// =============================================================================================
template <int DK, bool DELTA>
__global__ __launch_bounds__(256) void linear_prep_kernel(const LinearParams p) {
  constexpr int KP = DK + 8;   // bf16 row pitch
  constexpr int KL = DK / 32;  // 16-byte loads per thread per tile
  // The 64x64 fp32 matrices of the solve are kept as their ten lower 16x16 blocks, block (i, k) at
  // index i(i+1)/2 + k, rows of BP floats.  A = strictly lower system matrix; X = (I+A)^-1 row-major;
  // Xt = the same blocks transposed (so that a block serves as an MFMA B operand with one 16-byte read).
  constexpr int BP = 20, BLK = 16 * BP, NBLK = 10;
  constexpr int TILE_BYTES = 2 * C * KP * 2, SOLVE_BYTES = 3 * NBLK * BLK * 4;
  // LDS: the q, k tiles are dead once the Gram products are done; the solve reuses their space
  constexpr int REGION0 = (DELTA && SOLVE_BYTES > TILE_BYTES) ? SOLVE_BYTES : TILE_BYTES;
  __shared__ __align__(16) unsigned char region0[REGION0];
  __shared__ __align__(16) float gam[C], rq[C], rk[C], bet[C];
  bf16_t* Qs = reinterpret_cast<bf16_t*>(region0);
  bf16_t* Ks = Qs + C * KP;
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
#pragma unroll
    for (int i = 0; i < KL; ++i) {
      const u32x4 a = ok ? qr[seg + 4 * i] : z, b = ok ? kr[seg + 4 * i] : z;
      *reinterpret_cast<u32x4*>(Qs + row * KP + (seg + 4 * i) * 8) = a;
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
      rq[row] = l2 ? rsqrtf(sq + 1e-6f) : 1.f;
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
  // P and TmB are stored in the order the scan kernel consumes them as MFMA A operands, so that its
  // loads are contiguous: the 16 bytes of scan-lane (row i%16, group g4) of 16-row band i/16 and
  // k-step s sit at ((2(i/16) + s) * 64 + 16 g4 + i%16) * 16 bytes.  Within a k-step the 32
  // contraction tokens are permuted: slot (g4, e) holds token 8(2(g4&1) + e/4) + 4(g4/2) + e%4,
  // which is how one lane of the transposed 32x32 Gram accumulator holds them.
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
        const bf16x8 qa = ld8(Qs + (32 * ti + l32) * KP + 16 * s + 8 * hf);
        gq = mfma32(kb, qa, gq);  // transposed: lane = query row i, registers = key tokens j
        if (DELTA) {
          const bf16x8 ka = ld8(Ks + (32 * ti + l32) * KP + 16 * s + 8 * hf);
          gk = mfma32(ka, kb, gk);  // lane = column j, registers = rows i
        }
      }
      {
        // this lane's 16 key tokens are four runs of four: 16-byte reads of their gamma and 1/|k|
        const float gi = gam[i], fi = p.scale * rq[i];
        u32x4 w[2];
#pragma unroll
        for (int q4 = 0; q4 < 4; ++q4) {
          const int j0 = 32 * tj + 8 * q4 + 4 * hf;
          const f32x4 gj = *reinterpret_cast<const f32x4*>(gam + j0), rj = *reinterpret_cast<const f32x4*>(rk + j0);
          float pv[4];
#pragma unroll
          for (int e = 0; e < 4; ++e) pv[e] = i >= j0 + e ? fi * rj[e] * gq[4 * q4 + e] * __expf(gi - gj[e]) : 0.f;
          w[q4 >> 1][2 * (q4 & 1)] = pack_bf16x2(pv[0], pv[1]);
          w[q4 >> 1][2 * (q4 & 1) + 1] = pack_bf16x2(pv[2], pv[3]);
        }
        *reinterpret_cast<u32x4*>(prow + (2 * hf) * 128) = w[0];
        *reinterpret_cast<u32x4*>(prow + (2 * hf + 1) * 128) = w[1];
      }
    } else {
      // the strictly upper 32x32 tile is zero
      const u32x4 z = {0u, 0u, 0u, 0u};
      *reinterpret_cast<u32x4*>(prow + (2 * hf) * 128) = z;
      *reinterpret_cast<u32x4*>(prow + (2 * hf + 1) * 128) = z;
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
    float* Xtd = Xt + bidx(wave, wave) * BLK;
#pragma unroll
    for (int r = 0; r < 16; ++r) Xd[r * BP + x16] = x[r];
#pragma unroll
    for (int r4 = 0; r4 < 4; ++r4)
      *reinterpret_cast<f32x4*>(Xtd + x16 * BP + 4 * r4) = (f32x4){x[4 * r4], x[4 * r4 + 1], x[4 * r4 + 2], x[4 * r4 + 3]};
  }
  __syncthreads();
  // off-diagonal blocks, one block diagonal at a time, on the fp32 matrix cores:
  //   X_ik = -X_ii * sum_{j=k}^{i-1} A_ij X_jk        (i = k + d; wave k owns block (k+d, k))
  // MFMA 16x16x4: lane (x, g) supplies A[x][kk] and B[kk][x].  With kk = 4g + s in step s, the A
  // operand of all four steps is one 16-byte row read, and an accumulator (lane = column x, registers
  // = rows 4g..4g+3) is already a B operand, so the inner sum feeds the second product from registers.
#pragma unroll
  for (int d = 1; d < 4; ++d) {
    if (wave + d < 4) {
      const int k = wave, i = wave + d;
      f32x4 M = {0.f, 0.f, 0.f, 0.f};
      for (int j = k; j < i; ++j) {
        const f32x4 a4 = *reinterpret_cast<const f32x4*>(Ab + bidx(i, j) * BLK + x16 * BP + 4 * g4);
        const f32x4 b4 = *reinterpret_cast<const f32x4*>(Xt + bidx(j, k) * BLK + x16 * BP + 4 * g4);
#pragma unroll
        for (int st = 0; st < 4; ++st) M = __builtin_amdgcn_mfma_f32_16x16x4f32(a4[st], b4[st], M, 0, 0, 0);
      }
      const f32x4 d4 = *reinterpret_cast<const f32x4*>(Xb + bidx(i, i) * BLK + x16 * BP + 4 * g4);
      f32x4 Xa = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int st = 0; st < 4; ++st) Xa = __builtin_amdgcn_mfma_f32_16x16x4f32(d4[st], M[st], Xa, 0, 0, 0);
      float* Xo = Xb + bidx(i, k) * BLK;
#pragma unroll
      for (int r = 0; r < 4; ++r) Xo[(4 * g4 + r) * BP + x16] = -Xa[r];
      *reinterpret_cast<f32x4*>(Xt + bidx(i, k) * BLK + x16 * BP + 4 * g4) = (f32x4){-Xa[0], -Xa[1], -Xa[2], -Xa[3]};
    }
    __syncthreads();
  }
  // TmB = Tm * diag(beta), bf16, in the scan kernel's A-operand order (see above)
  {
    const int row = tid >> 2, cb = tid & 3;
    float x[16];
#pragma unroll
    for (int e4 = 0; e4 < 4; ++e4) {
      const f32x4 xv = cb <= (row >> 4) ? *reinterpret_cast<const f32x4*>(Xb + bidx(row >> 4, cb <= (row >> 4) ? cb : 0) * BLK + (row & 15) * BP + 4 * e4)
                                        : (f32x4){0.f, 0.f, 0.f, 0.f};
      const f32x4 bv = *reinterpret_cast<const f32x4*>(bet + 16 * cb + 4 * e4);
#pragma unroll
      for (int e = 0; e < 4; ++e) x[4 * e4 + e] = xv[e] * bv[e];
    }
    u32x4 w0, w1;  // tokens {0..3, 8..11} and {4..7, 12..15} of this thread's 16
    w0[0] = pack_bf16x2(x[0], x[1]);  w0[1] = pack_bf16x2(x[2], x[3]);   w0[2] = pack_bf16x2(x[8], x[9]);   w0[3] = pack_bf16x2(x[10], x[11]);
    w1[0] = pack_bf16x2(x[4], x[5]);  w1[1] = pack_bf16x2(x[6], x[7]);   w1[2] = pack_bf16x2(x[12], x[13]); w1[3] = pack_bf16x2(x[14], x[15]);
    bf16_t* trow = Tout + ((size_t)((2 * (row >> 4) + (cb >> 1)) * 64 + (row & 15))) * 8;
    *reinterpret_cast<u32x4*>(trow + (cb & 1) * 128) = w0;
    *reinterpret_cast<u32x4*>(trow + (2 + (cb & 1)) * 128) = w1;
  }
}

// =============================================================================================
// scan
// =============================================================================================
NATSL_DEVICE u32x2 pack4(f32x4 v) {
  u32x2 w;
  w[0] = pack_bf16x2(v[0], v[1]);
  w[1] = pack_bf16x2(v[2], v[3]);
  return w;
}

template <int DK, bool DELTA>
__global__ __launch_bounds__(256, 2) void linear_scan_kernel(const LinearParams p) {
  constexpr int KS = DK / 32;   // MFMA k-steps over the key dimension
  constexpr int MT = DK / 64;   // 16-row state tiles per wave
  constexpr int KP = DK + 8;    // kbuf / ST row pitch (elements)
  constexpr int VP = BV + 8;    // vbuf row pitch
  constexpr int XP = C + 8;     // XT / VNT / VTT row pitch
  __shared__ __align__(16) bf16_t kbuf[2][C * KP];
  __shared__ __align__(16) bf16_t vbuf[2][C * VP];
  __shared__ __align__(16) bf16_t ST[BV * KP];
  __shared__ __align__(16) bf16_t XT[BV * XP];
  __shared__ __align__(16) bf16_t VNT[BV * XP];
  __shared__ __align__(16) bf16_t VTT[BV * XP];
  __shared__ __align__(16) bf16_t Os[C * VP];  // output tile, row-major, for 16-byte stores

  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int i16 = lane & 15, g4 = lane >> 4;

  // ---- which (sequence, head, V slice): the slices of one chain sit on one XCD --------------
  const int nsplit = p.V / BV;
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
  const int per_blk = p.block / C;
  const bool decay = (p.flags & NATSL_DECAY_NON_LINEAR) != 0;
  const bool intra = (p.flags & NATSL_INTRA_CHUNK) != 0;
  const int vcol0 = split * BV;

  const size_t qk_row = (size_t)p.H * DK, v_row = (size_t)p.H * p.V;
  const bf16_t* qp = p.q + ((size_t)bos * p.H + h) * DK;
  const bf16_t* kp = p.k + ((size_t)bos * p.H + h) * DK;
  const bf16_t* vp = p.v + ((size_t)bos * p.H + h) * p.V + vcol0;
  bf16_t* op = p.o + ((size_t)bos * p.H + h) * p.V + vcol0;

  // ---- state slice in accumulator layout: tile (mi, nn) = rows 16(wave*MT+mi).., cols 16nn.. ---
  f32x4 S[MT][2], Ssave[MT][2];
#pragma unroll
  for (int mi = 0; mi < MT; ++mi)
#pragma unroll
    for (int nn = 0; nn < 2; ++nn)
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int kd = 16 * (wave * MT + mi) + 4 * g4 + r, vc = vcol0 + 16 * nn + i16;
        S[mi][nn][r] = p.h0 ? p.h0[((size_t)chain * DK + kd) * p.V + vc] : 0.f;
        Ssave[mi][nn][r] = 0.f;
      }
  auto write_ST = [&]() {
#pragma unroll
    for (int mi = 0; mi < MT; ++mi)
#pragma unroll
      for (int nn = 0; nn < 2; ++nn)
        *reinterpret_cast<u32x2*>(ST + (16 * nn + i16) * KP + 16 * (wave * MT + mi) + 4 * g4) = pack4(S[mi][nn]);
  };

  // ---- operand staging ------------------------------------------------------------------------
  // Two register sets hold the MFMA A operands (q, TmB, P) and the per-token scales of chunks c and
  // c+1.  Each piece of the set in use is reloaded with chunk c+2's data right after its last use,
  // so every one of these loads has two steps to arrive.  k and v go through LDS (double-buffered):
  // they are loaded at the start of step c for chunk c+1 and stored at its end.
  struct Operands {
    bf16x8 qA[KS], TA[2], PA[2];
    f32x4 se, sq, sk;
    float dec, glast, linf;
  };
  struct Staging {
    u32x4 kld[KS], vld;  // row-contiguous k and v pieces on their way to LDS
  };
  const int a_row = 16 * wave + i16;          // this lane's A-operand row (token within the chunk)
  const int v_ld_row = tid >> 2, v_ld_seg = tid & 3;
  const int r0 = 16 * wave + 4 * g4;          // first of this lane's four accumulator rows
  // where those four tokens sit in the contraction order P and TmB were stored in
  const int perm0 = 32 * (wave >> 1) + 8 * (2 * (g4 & 1) + (wave & 1)) + 4 * (g4 >> 1);
  // k staging: one pass of the 256 threads covers KROWS token rows of DK*2 bytes
  constexpr int KSEGS = DK / 8, KROWS = 256 / KSEGS;
  const int k_ld_row = tid / KSEGS, k_ld_seg = tid % KSEGS;
  // rows past the end of the sequence are clamped (beta = 0 there makes their v_new exactly 0, and
  // their outputs are never stored)
  const bf16_t* k_ptr = kp + 8 * k_ld_seg;
  const bf16_t* q_ptr = qp + 8 * g4;
  const bf16_t* v_ptr = vp + 8 * v_ld_seg;
  const size_t unit0 = (size_t)chunk_off * p.H + h;
  const size_t unit_step = (size_t)p.H * (C * C), sc_step = (size_t)p.H * (4 * C);
  // P and TmB come in A-operand order: 16 contiguous bytes per lane, 1 KiB per wave and k-step
  const bf16_t* P_base = p.ws_p + unit0 * (C * C) + (2 * wave * 64 + lane) * 8;
  const bf16_t* T_base = p.ws_tm + unit0 * (C * C) + (2 * wave * 64 + lane) * 8;
  const float* sc_base = p.ws_sc + unit0 * (4 * C);
  // the pieces of an operand set, each loadable on its own (cc = chunk index, must be < NT)
  auto load_q = [&](Operands& A, int cc) {
    const bf16_t* qr = q_ptr + (size_t)min(cc * C + a_row, len - 1) * qk_row;
#pragma unroll
    for (int s = 0; s < KS; ++s) A.qA[s] = ld8(qr + 32 * s);
  };
  auto load_T = [&](Operands& A, int cc) {
    A.TA[0] = ld8(T_base + cc * unit_step);
    A.TA[1] = ld8(T_base + cc * unit_step + 512);
  };
  auto load_P = [&](Operands& A, int cc) {
    A.PA[0] = ld8(P_base + cc * unit_step);
    A.PA[1] = ld8(P_base + cc * unit_step + 512);
  };
  auto load_se = [&](Operands& A, int cc) { A.se = *reinterpret_cast<const f32x4*>(sc_base + cc * sc_step + r0); };
  auto load_sq = [&](Operands& A, int cc) { A.sq = *reinterpret_cast<const f32x4*>(sc_base + cc * sc_step + C + r0); };
  auto load_sk = [&](Operands& A, int cc) { A.sk = *reinterpret_cast<const f32x4*>(sc_base + cc * sc_step + 2 * C + r0); };
  auto load_scalars = [&](Operands& A, int cc) {
    const float* sp = sc_base + cc * sc_step + 3 * C;
    A.dec = sp[0];
    A.glast = sp[1];
    A.linf = sp[2];
  };
  auto load_all = [&](Operands& A, int cc) {
    load_q(A, cc);
    if (DELTA) load_se(A, cc);
    if (DELTA) load_T(A, cc);
    load_sk(A, cc);
    load_P(A, cc);
    load_sq(A, cc);
    load_scalars(A, cc);
  };
  auto gload_kv = [&](Staging& G, int cc) {
#pragma unroll
    for (int s = 0; s < KS; ++s) {
      const int kt = min(cc * C + k_ld_row + KROWS * s, len - 1);
      G.kld[s] = *reinterpret_cast<const u32x4*>(k_ptr + (size_t)kt * qk_row);
    }
    const int vt = cc * C + v_ld_row;
    const u32x4 z = {0u, 0u, 0u, 0u};
    G.vld = vt < len ? *reinterpret_cast<const u32x4*>(v_ptr + (size_t)vt * v_row) : z;  // v must be 0 past the end
  };
  auto lstore = [&](const Staging& G, int buf) {
#pragma unroll
    for (int s = 0; s < KS; ++s) *reinterpret_cast<u32x4*>(&kbuf[buf][(k_ld_row + KROWS * s) * KP + 8 * k_ld_seg]) = G.kld[s];
    *reinterpret_cast<u32x4*>(&vbuf[buf][v_ld_row * VP + 8 * v_ld_seg]) = G.vld;
  };

  float gsum = 0.f;
  // one chunk: CUR holds its operands, kbuf/vbuf[buf] its k and v tiles
  Staging G;
  auto step = [&](const int c, const int buf, Operands& CUR) {
    __syncthreads();  // ST, kbuf[buf], vbuf[buf] are in place
    // Loads are issued unconditionally (chunk indices clamped to the last chunk): a load inside a
    // branch would force the waits below to assume it may not have been issued, i.e. to drain the queue.
    const int c1 = min(c + 1, NT - 1), c2 = min(c + 2, NT - 1);
    const float dec_c = CUR.dec, glast_c = CUR.glast, linf_c = CUR.linf;
    load_scalars(CUR, c2);  // first, so that nothing younger has to be waited for along with them
    gload_kv(G, c1);

    if (c % per_blk == 0) {
#pragma unroll
      for (int mi = 0; mi < MT; ++mi)
#pragma unroll
        for (int nn = 0; nn < 2; ++nn) Ssave[mi][nn] = S[mi][nn];
      gsum = 0.f;
    }

    // (1) R = k S, O1 = q S
    f32x4 R[2], O1[2];
#pragma unroll
    for (int nn = 0; nn < 2; ++nn) { R[nn] = (f32x4){0.f, 0.f, 0.f, 0.f}; O1[nn] = (f32x4){0.f, 0.f, 0.f, 0.f}; }
#pragma unroll
    for (int s = 0; s < KS; ++s) {
      const bf16x8 sb0 = ld8(ST + i16 * KP + 32 * s + 8 * g4);
      const bf16x8 sb1 = ld8(ST + (16 + i16) * KP + 32 * s + 8 * g4);
      if (DELTA) {
        const bf16x8 ka = ld8(&kbuf[buf][a_row * KP + 32 * s + 8 * g4]);
        R[0] = mfma16(ka, sb0, R[0]);
        R[1] = mfma16(ka, sb1, R[1]);
      }
      O1[0] = mfma16(CUR.qA[s], sb0, O1[0]);
      O1[1] = mfma16(CUR.qA[s], sb1, O1[1]);
    }
    load_q(CUR, c2);
    // (2) v in accumulator layout via the transposing read; X = v - se * R
    f32x4 VN[2];
#pragma unroll
    for (int nn = 0; nn < 2; ++nn) {
      const s16x4 vv = lds_tr4(&vbuf[buf][(16 * wave + 4 * g4 + (i16 >> 2)) * VP + 16 * nn + 4 * (i16 & 3)]);
#pragma unroll
      for (int r = 0; r < 4; ++r) VN[nn][r] = bf16_to_f32((bf16_t)vv[r]);
    }
    if (DELTA) {
#pragma unroll
      for (int nn = 0; nn < 2; ++nn) {
        f32x4 X;
#pragma unroll
        for (int r = 0; r < 4; ++r) X[r] = VN[nn][r] - CUR.se[r] * R[nn][r];
        *reinterpret_cast<u32x2*>(XT + (16 * nn + i16) * XP + perm0) = pack4(X);
      }
      load_se(CUR, c2);
      __syncthreads();
      // (3) v_new = TmB X
#pragma unroll
      for (int nn = 0; nn < 2; ++nn) {
        VN[nn] = (f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int s = 0; s < 2; ++s) VN[nn] = mfma16(CUR.TA[s], ld8(XT + (16 * nn + i16) * XP + 32 * s + 8 * g4), VN[nn]);
      }
      load_T(CUR, c2);
    }
    // (4) v_new and sk * v_new, transposed, for the two products that reduce over tokens
#pragma unroll
    for (int nn = 0; nn < 2; ++nn) {
      f32x4 vt;
#pragma unroll
      for (int r = 0; r < 4; ++r) vt[r] = VN[nn][r] * CUR.sk[r];
      *reinterpret_cast<u32x2*>(VNT + (16 * nn + i16) * XP + perm0) = pack4(VN[nn]);
      *reinterpret_cast<u32x2*>(VTT + (16 * nn + i16) * XP + 16 * wave + 4 * g4) = pack4(vt);
    }
    load_sk(CUR, c2);
    __syncthreads();
    // (5) o = sq * O1 + P v_new
#pragma unroll
    for (int nn = 0; nn < 2; ++nn) {
      f32x4 O;
#pragma unroll
      for (int r = 0; r < 4; ++r) O[r] = O1[nn][r] * CUR.sq[r];
      if (intra) {
#pragma unroll
        for (int s = 0; s < 2; ++s) O = mfma16(CUR.PA[s], ld8(VNT + (16 * nn + i16) * XP + 32 * s + 8 * g4), O);
      }
#pragma unroll
      for (int r = 0; r < 4; ++r) Os[(r0 + r) * VP + 16 * nn + i16] = f32_to_bf16(O[r]);
    }
    load_P(CUR, c2);
    load_sq(CUR, c2);
    {
      // each wave stores the 16 rows it owns: 4 lanes x 16 bytes per row
      __builtin_amdgcn_s_waitcnt(0xc07f);
      __builtin_amdgcn_wave_barrier();
      const int row = 16 * wave + (lane >> 2), tok = c * C + row;
      if (tok < len)
        *reinterpret_cast<u32x4*>(op + (size_t)tok * v_row + 8 * (lane & 3)) = *reinterpret_cast<const u32x4*>(Os + row * VP + 8 * (lane & 3));
    }
    // (6) state update / roll-back
    const bool last_of_block = ((c + 1) % per_blk == 0) || (c == NT - 1);
    gsum += glast_c;
    const bool keep = linf_c != 0.f || !last_of_block;
    if (keep) {
#pragma unroll
      for (int mi = 0; mi < MT; ++mi) {
        const int m = wave * MT + mi;
        bf16x8 kt[2];
#pragma unroll
        for (int s = 0; s < 2; ++s) {
          const bf16_t* kb = &kbuf[buf][(32 * s + 8 * g4 + (i16 >> 2)) * KP + 16 * m + 4 * (i16 & 3)];
          kt[s] = join4(lds_tr4(kb), lds_tr4(kb + 4 * KP));
        }
#pragma unroll
        for (int nn = 0; nn < 2; ++nn) {
#pragma unroll
          for (int r = 0; r < 4; ++r) S[mi][nn][r] *= dec_c;
#pragma unroll
          for (int s = 0; s < 2; ++s) S[mi][nn] = mfma16(kt[s], ld8(VTT + (16 * nn + i16) * XP + 32 * s + 8 * g4), S[mi][nn]);
        }
      }
    } else {
      const float f = decay ? __expf(gsum) : 1.f;
#pragma unroll
      for (int mi = 0; mi < MT; ++mi)
#pragma unroll
        for (int nn = 0; nn < 2; ++nn)
#pragma unroll
          for (int r = 0; r < 4; ++r) S[mi][nn][r] = Ssave[mi][nn][r] * f;
    }
    // (7) bf16 copy of the state and the staged k, v tiles for the next step
    write_ST();
    lstore(G, buf ^ 1);
  };

  Operands A0, A1;
  if (NT > 0) {
    gload_kv(G, 0);
    load_all(A0, 0);
    if (NT > 1) load_all(A1, 1);
    lstore(G, 0);
  }
  write_ST();
  for (int c = 0; c < NT; c += 2) {
    step(c, 0, A0);
    if (c + 1 < NT) step(c + 1, 1, A1);
  }

  if (p.hs) {
    // Ssave / gsum still belong to the last block: the state that entered it and its total log-decay
#pragma unroll
    for (int mi = 0; mi < MT; ++mi)
#pragma unroll
      for (int nn = 0; nn < 2; ++nn)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const int kd = 16 * (wave * MT + mi) + 4 * g4 + r, vc = vcol0 + 16 * nn + i16;
          p.hs[((size_t)chain * DK + kd) * p.V + vc] = Ssave[mi][nn][r];
        }
    if (p.gs && split == 0 && tid == 0) p.gs[chain] = gsum;
  }
  if (p.ht) {
#pragma unroll
    for (int mi = 0; mi < MT; ++mi)
#pragma unroll
      for (int nn = 0; nn < 2; ++nn)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const int kd = 16 * (wave * MT + mi) + 4 * g4 + r, vc = vcol0 + 16 * nn + i16;
          p.ht[((size_t)chain * DK + kd) * p.V + vc] = S[mi][nn][r];
        }
  }
}

constexpr size_t WS_UNIT_BYTES = (size_t)C * C * 2 * 2 + 4 * C * 4;

template <int DK, bool DELTA>
static int launch_linear(const LinearParams& p, hipStream_t stream, const char* what) {
  const long long units = (long long)p.total_chunks * p.H;
  if (units <= 0) return NATSL_OK;
  hipLaunchKernelGGL((linear_prep_kernel<DK, DELTA>), dim3((unsigned)units), dim3(256), 0, stream, p);
  int rc = check_launch(what);
  if (rc != NATSL_OK) return rc;
  const int n_chains = (p.seqs ? p.n_seqs : p.B) * p.H;
  const int grid = 8 * cdiv(n_chains, 8) * (p.V / BV);
  hipLaunchKernelGGL((linear_scan_kernel<DK, DELTA>), dim3(grid), dim3(256), 0, stream, p);
  return check_launch(what);
}

static int linear_fwd(bool delta, const void* q, const void* k, const void* v, const float* g, const void* beta,
                      const float* h0, void* o, float* ht, float* hs, float* gs, const void* types, int types_dtype, int B, int T,
                      int H, int HN, int K, int V, int TN, int block, float scale, int flags, void* workspace, size_t workspace_bytes,
                      int dtype, const natsl_seq_row* seqs, int n_seqs, int total_units, natsl_stream_t stream) {
  const char* what = delta ? "natsl_gdn_chunk_fwd" : "natsl_mamba_chunk_fwd";
  if (!q || !k || !v || !g || !o || !types || (delta && !beta)) return fail(NATSL_ERR_INVALID, "%s: null pointer argument", what);
  if (dtype != NATSL_BF16) return fail(NATSL_ERR_UNSUPPORTED, "%s: only bf16 tensors are supported (got dtype %d)", what, dtype);
  if (types_dtype != NATSL_BF16 && types_dtype != NATSL_F32) return fail(NATSL_ERR_UNSUPPORTED, "%s: block types must be f32 or bf16", what);
  if (B <= 0 || T <= 0 || H <= 0 || HN <= 0 || TN <= 0) return fail(NATSL_ERR_INVALID, "%s: non-positive dimension", what);
  if (H % HN) return fail(NATSL_ERR_INVALID, "%s: H=%d must be a multiple of HN=%d", what, H, HN);
  if (block < 64 || block % 64) return fail(NATSL_ERR_UNSUPPORTED, "%s: block size %d must be a multiple of 64", what, block);
  if (V % BV || V <= 0) return fail(NATSL_ERR_UNSUPPORTED, "%s: V=%d must be a multiple of %d", what, V, BV);
  if (seqs ? (B != 1 || n_seqs <= 0 || total_units <= 0) : (TN != cdiv(T, block)))
    return fail(NATSL_ERR_INVALID, "%s: TN=%d does not match T=%d, block=%d (or bad packed-input arguments)", what, TN, T, block);
  LinearParams p;
  p.q = (const bf16_t*)q; p.k = (const bf16_t*)k; p.v = (const bf16_t*)v; p.g = g; p.beta = (const bf16_t*)beta;
  p.h0 = h0; p.o = (bf16_t*)o; p.ht = ht; p.hs = hs; p.gs = gs; p.types = types; p.types_dtype = types_dtype;
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
  } else {
    if (K == 128) return launch_linear<128, false>(p, s, what);
    if (K == 64) return launch_linear<64, false>(p, s, what);
  }
  return fail(NATSL_ERR_UNSUPPORTED, "%s: key dim K=%d not built (supported: 64, 128)", what, K);
}

}  // namespace natsl

using namespace natsl;

extern "C" size_t natsl_linear_workspace_bytes(int64_t total_chunks, int H) {
  if (total_chunks <= 0 || H <= 0) return 0;
  return (size_t)total_chunks * (size_t)H * WS_UNIT_BYTES;
}

extern "C" int natsl_gdn_chunk_fwd(const void* q, const void* k, const void* v, const float* g, const void* beta,
                                   const float* h0, void* o, float* ht, float* h_block_start, float* g_block_sum,
                                   const void* types, int types_dtype, int B, int T,
                                   int H, int HN, int K, int V, int TN, int block, float scale, int flags, void* workspace,
                                   size_t workspace_bytes, int dtype, const natsl_seq_row* seqs, int n_seqs, int total_units,
                                   natsl_stream_t stream) {
  return linear_fwd(true, q, k, v, g, beta, h0, o, ht, h_block_start, g_block_sum, types, types_dtype, B, T, H, HN, K, V, TN, block, scale, flags,
                    workspace, workspace_bytes, dtype, seqs, n_seqs, total_units, stream);
}

extern "C" int natsl_mamba_chunk_fwd(const void* q, const void* k, const void* v, const float* g, const float* h0, void* o,
                                     float* ht, float* h_block_start, float* g_block_sum, const void* types, int types_dtype, int B, int T, int H, int HN, int K, int V,
                                     int TN, int block, float scale, int flags, void* workspace, size_t workspace_bytes,
                                     int dtype, const natsl_seq_row* seqs, int n_seqs, int total_units,
                                     natsl_stream_t stream) {
  return linear_fwd(false, q, k, v, g, nullptr, h0, o, ht, h_block_start, g_block_sum, types, types_dtype, B, T, H, HN, K, V, TN, block, scale,
                    flags & ~NATSL_QK_L2NORM, workspace, workspace_bytes, dtype, seqs, n_seqs, total_units, stream);
}
