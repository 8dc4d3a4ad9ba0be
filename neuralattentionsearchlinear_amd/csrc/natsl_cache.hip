// Compaction of the softmax branch's K/V cache for gfx950.
//
// After a forward pass the selector has typed every completed block of new tokens.  Only blocks typed
// "attention" are ever read again by later queries, and every (sequence, selector head) keeps a different
// subset.  The cache therefore stores, per (sequence, kv head), its attention-typed blocks back to back from
// block 0, and the tokens of the current incomplete block at one block index shared by all heads (the
// largest count of kept blocks), so that one [B, tokens, heads, D] tensor plus a per-block validity flag
// describes the whole cache (src/nats/models/utils.py:509-588 does this with advanced indexing on a clone).
//
// This is byte movement, bound by HBM: a 16-byte lane (token in block, segment of the head row) is owned by
// one thread for all blocks of its (sequence, head), which walks the region in order.  A kept block only
// moves towards the front (its destination is never behind its source), so walking in order makes the move
// safe in place without a second buffer; the kept blocks are moved NATSL_KV_BATCH at a time, all loads of a batch
// ahead of its stores, which stays safe because the stores of a batch only reach positions in front of every
// source not yet loaded.  Which blocks are kept is scanned once per workgroup into a bit mask in LDS.
#include "natsl_device.h"
#include "natsl_host.h"
#include "../../include/natsl.h"

namespace natsl {

#define NATSL_KV_BATCH 8
#define NATSL_KV_SCAN 1024   // blocks typed per scan round (a multiple of 256)

struct KvCompactParams {
  const char* src[2]; char* dst[2];       // K and V: [B, cap, HKV, row] with row bytes below
  int row[2];
  long src_cap, dst_cap;                  // tokens per sequence in the source / destination tensors
  const void* types; int types_dtype;     // [B, NB, HN, 2]; column 0 == 1 marks an attention-typed block
  const int64_t* n_before;                // [B, HN] blocks already kept per (sequence, selector head); may be null
  int B, HKV, HN, block;
  int src_block0;                         // block index of the region's first block in the source
  int NB, n_complete;                     // blocks in the region / how many of them are complete
  int tail_dst, tail_tokens;              // destination block of the incomplete block (-1: none), tokens in it
  int wgs[2];                             // workgroups per (sequence, head) for K and for V
};

NATSL_DEVICE bool kv_is_attn(const KvCompactParams& p, int b, int s, int hn) {
  size_t i = (((size_t)b * p.NB + s) * p.HN + hn) * 2;
  float t = p.types_dtype == NATSL_F32 ? reinterpret_cast<const float*>(p.types)[i]
                                       : bf16_to_f32(reinterpret_cast<const bf16_t*>(p.types)[i]);
  return rintf(t) == 1.0f;   // the predicate of the router and of both branches (mixed_attn_gdn.py:88 rounds the types)
}

__global__ __launch_bounds__(256) void kv_compact_kernel(KvCompactParams p) {
  // which blocks of the region this (sequence, selector head) keeps: one bit per block, NATSL_KV_SCAN blocks at a time
  __shared__ unsigned long long keep[NATSL_KV_SCAN / 64];
  const int bh = blockIdx.y, b = bh / p.HKV, h = bh % p.HKV, hn = h / (p.HKV / p.HN);
  int wg = blockIdx.x;
  const int which = wg >= p.wgs[0] ? 1 : 0;
  if (which) wg -= p.wgs[0];
  const int row = p.row[which], segs = row / 16;
  const int tid = (int)threadIdx.x, lane = wg * 256 + tid;
  const bool active = lane < p.block * segs;            // idle lanes still take part in the scan and its barriers
  const int tok = lane / segs, seg = lane % segs;
  const size_t tok_stride = (size_t)p.HKV * row;
  const char* sbase = p.src[which] + (size_t)b * p.src_cap * tok_stride + (size_t)h * row + seg * 16;
  char* dbase = p.dst[which] + (size_t)b * p.dst_cap * tok_stride + (size_t)h * row + seg * 16;
  auto saddr = [&](long blk) { return reinterpret_cast<const u32x4*>(sbase + ((size_t)blk * p.block + tok) * tok_stride); };
  auto daddr = [&](long blk) { return reinterpret_cast<u32x4*>(dbase + ((size_t)blk * p.block + tok) * tok_stride); };
  const bool in_place = p.src[which] == p.dst[which];

  long dst = p.n_before ? (long)p.n_before[b * p.HN + hn] : 0;
  for (int base = 0; base < p.n_complete; base += NATSL_KV_SCAN) {
    __syncthreads();
#pragma unroll
    for (int r = 0; r < NATSL_KV_SCAN / 256; ++r) {
      const int s = base + r * 256 + tid;
      const unsigned long long m = __ballot(s < p.n_complete && kv_is_attn(p, b, s, hn));
      if ((tid & 63) == 0) keep[r * 4 + (tid >> 6)] = m;
    }
    __syncthreads();
    // walk the kept blocks NATSL_KV_BATCH at a time: all loads of a batch are in flight before its stores
    unsigned long long m = 0;
    int word = -1;
    auto next = [&]() -> int {
      while (m == 0) {
        if (word + 1 >= NATSL_KV_SCAN / 64) return -1;
        m = keep[++word];
      }
      const int bit = __builtin_ctzll(m);
      m &= m - 1;
      return base + word * 64 + bit;
    };
    for (;;) {
      int s[NATSL_KV_BATCH];
#pragma unroll
      for (int j = 0; j < NATSL_KV_BATCH; ++j) s[j] = next();
      if (s[0] < 0) break;
      u32x4 buf[NATSL_KV_BATCH];
#pragma unroll
      for (int j = 0; j < NATSL_KV_BATCH; ++j)
        if (s[j] >= 0 && active) buf[j] = *saddr(p.src_block0 + s[j]);
#pragma unroll
      for (int j = 0; j < NATSL_KV_BATCH; ++j) {
        if (s[j] < 0) continue;
        // the bound only guards against counts the caller did not size the destination for
        if (active && !(in_place && dst == p.src_block0 + s[j]) && (dst + 1) * p.block <= p.dst_cap) *daddr(dst) = buf[j];
        ++dst;
      }
    }
  }
  if (p.tail_dst >= 0 && active) {
    const long sblk = p.src_block0 + p.NB - 1;
    if (!(in_place && sblk == p.tail_dst)) {
      u32x4 x = {0u, 0u, 0u, 0u};
      if (tok < p.tail_tokens) x = *saddr(sblk);
      *daddr(p.tail_dst) = x;
    }
  }
}

}  // namespace natsl

using namespace natsl;

extern "C" int natsl_kv_compact(const void* src_k, const void* src_v, long long src_tokens, int src_block0, void* dst_k,
                                void* dst_v, long long dst_tokens, const void* types, int types_dtype,
                                const int64_t* n_before, int B, int HKV, int HN, int K, int V, int dtype, int block,
                                int NB, int n_complete, int tail_dst, int tail_tokens, natsl_stream_t stream) {
  const char* what = "natsl_kv_compact";
  if (!src_k || !src_v || !dst_k || !dst_v || !types) return fail(NATSL_ERR_INVALID, "%s: null pointer argument", what);
  if (dtype != NATSL_BF16 && dtype != NATSL_F32) return fail(NATSL_ERR_UNSUPPORTED, "%s: tensors must be f32 or bf16", what);
  if (types_dtype != NATSL_BF16 && types_dtype != NATSL_F32) return fail(NATSL_ERR_UNSUPPORTED, "%s: block types must be f32 or bf16", what);
  if (B <= 0 || HKV <= 0 || HN <= 0 || K <= 0 || V <= 0 || block <= 0 || NB <= 0) return fail(NATSL_ERR_INVALID, "%s: non-positive dimension", what);
  if (HKV % HN) return fail(NATSL_ERR_INVALID, "%s: HKV=%d must be a multiple of HN=%d", what, HKV, HN);
  const int esize = dtype == NATSL_BF16 ? 2 : 4;
  if ((K * esize) % 16 || (V * esize) % 16) return fail(NATSL_ERR_UNSUPPORTED, "%s: head rows must be multiples of 16 bytes (K=%d, V=%d)", what, K, V);
  if (n_complete < 0 || n_complete > NB || (tail_dst >= 0 && n_complete != NB - 1) || (tail_dst < 0 && n_complete != NB))
    return fail(NATSL_ERR_INVALID, "%s: n_complete=%d does not fit NB=%d with%s an incomplete block", what, n_complete, NB, tail_dst >= 0 ? "" : "out");
  if (tail_dst >= 0 && (tail_tokens <= 0 || tail_tokens >= block)) return fail(NATSL_ERR_INVALID, "%s: tail_tokens=%d outside (0, %d)", what, tail_tokens, block);
  if (src_block0 < 0) return fail(NATSL_ERR_INVALID, "%s: negative source block", what);
  // the source must hold the region's complete blocks and the tokens of the incomplete one
  const long long src_need = ((long long)src_block0 + n_complete) * block + (tail_dst >= 0 ? tail_tokens : 0);
  if (src_tokens < src_need) return fail(NATSL_ERR_INVALID, "%s: source holds %lld tokens per sequence, the region needs %lld", what, src_tokens, src_need);
  // the destination must hold every block that can be written: at most n_complete more than the largest count the
  // caller has (which it bounds by tail_dst or by dst_tokens itself); the in-place case never moves a block backwards
  if (tail_dst >= 0 && ((long long)tail_dst + 1) * block > dst_tokens) return fail(NATSL_ERR_INVALID, "%s: destination too small for the incomplete block at %d", what, tail_dst);
  if ((src_k == dst_k) != (src_v == dst_v)) return fail(NATSL_ERR_INVALID, "%s: K and V must both be in place or both not", what);
  if (src_k == dst_k && src_tokens != dst_tokens) return fail(NATSL_ERR_INVALID, "%s: in place, source and destination sizes must agree", what);
  if ((long long)B * HKV > 65535) return fail(NATSL_ERR_UNSUPPORTED, "%s: B*HKV=%lld above 65535", what, (long long)B * HKV);
  KvCompactParams p;
  p.src[0] = (const char*)src_k; p.src[1] = (const char*)src_v; p.dst[0] = (char*)dst_k; p.dst[1] = (char*)dst_v;
  p.row[0] = K * esize; p.row[1] = V * esize;
  p.src_cap = (long)src_tokens; p.dst_cap = (long)dst_tokens;
  p.types = types; p.types_dtype = types_dtype; p.n_before = n_before;
  p.B = B; p.HKV = HKV; p.HN = HN; p.block = block; p.src_block0 = src_block0; p.NB = NB; p.n_complete = n_complete;
  p.tail_dst = tail_dst; p.tail_tokens = tail_tokens;
  p.wgs[0] = cdiv(block * (p.row[0] / 16), 256); p.wgs[1] = cdiv(block * (p.row[1] / 16), 256);
  hipLaunchKernelGGL(kv_compact_kernel, dim3(p.wgs[0] + p.wgs[1], B * HKV), dim3(256), 0, (hipStream_t)stream, p);
  return check_launch(what);
}
