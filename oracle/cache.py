"""CPU statement of what the hybrid layers' K/V cache must hold (test infrastructure only, see oracle/__init__.py).

The reference keeps, per (sequence, selector head), the complete blocks typed "attention" and drops the others;
the tokens of the current incomplete block are always kept (src/nats/models/utils.py:34-116 describes the layout,
:509-588 builds it).  Two independent statements of that rule:

whole_sequence     the definition, from all tokens and all block types at once: block j of (b, hn) is kept iff it is
                   complete and types[b, j, hn, 0] == 1.
CacheModel         the same reached incrementally, tokens fed in pieces of any size with the types of the blocks a
                   piece completes -- the way the layers call the cache (update_attn_cache then update).

What pins them: each other on random splits (tests/test_oracle_cache.py), and the checks the reference holds for
its own cache (src/nats/models/utils.py:855-1047: token-index patterns with the reference's sizes T=1078, 1728+45,
1777+195, B=4, H=8, HNAtS=4; a kept block i of a head holds exactly the token indices of that head's i-th attention
block; the incomplete block sits at the largest count; one piece == two pieces == token by token).  Those reference
functions cannot run as written (they call update_attn_cache with one argument, and two of them compare a cache
with itself); their stated invariants are what is checked.
"""
import torch


def whole_sequence(k, v, types, block):
    """k [B,T,HKV,Dk], v [B,T,HKV,Dv], types [B,ceil(T/block),HN,2] -> dict with
       n_attn_blocks int64 [B,HN]; n_max; n_tail (tokens of the incomplete block);
       keys/values: dense [B,(n_max+1)*block,HKV,D] laid out as the cache must be, zero where nothing is kept;
       valid bool [B,n_max+1,HN]."""
    B, T, HKV, _ = k.shape
    HN = types.shape[2]
    G = HKV // HN
    n_complete, n_tail = T // block, T % block
    assert types.shape[1] == -(-T // block)
    is_attn = types[:, :n_complete, :, 0] == 1                                  # [B, n_complete, HN]
    counts = is_attn.sum(1).to(torch.int64)                                     # [B, HN]
    n_max = int(counts.max()) if counts.numel() else 0
    out = {}
    for name, x in (('keys', k), ('values', v)):
        dense = torch.zeros(B, (n_max + 1) * block, HKV, x.shape[-1], dtype=x.dtype)
        for b in range(B):
            for h in range(HKV):
                i = 0
                for j in range(n_complete):
                    if is_attn[b, j, h // G]:
                        dense[b, i * block:(i + 1) * block, h] = x[b, j * block:(j + 1) * block, h]
                        i += 1
        if n_tail:
            dense[:, n_max * block:n_max * block + n_tail] = x[:, n_complete * block:]
        out[name] = dense
    valid = torch.arange(n_max + 1).view(1, -1, 1) < counts.unsqueeze(1)
    if n_tail:
        valid[:, n_max] = True
    out.update(n_attn_blocks=counts, n_max=n_max, n_tail=n_tail, valid=valid)
    return out


def next_query_mask(state, block):
    """Visibility [B,HN,1,n_max*block+n_tail+1] of the cached keys for ONE new token appended to `state`
    (src/nats/models/utils.py:234-244 for the modes whose attention looks into the incomplete block): the kept
    blocks of the head, nothing up to the largest count, then the incomplete block including the new token."""
    counts, n_max, n_tail = state['n_attn_blocks'], state['n_max'], state['n_tail']
    B, HN = counts.shape
    cols = n_max * block + n_tail + 1
    idx = torch.arange(cols).view(1, 1, -1)
    m = (idx < (counts * block).unsqueeze(-1)) | (idx >= n_max * block)
    return m.view(B, HN, 1, cols)


class CacheModel:
    """Incremental form: per (sequence, kv head) a Python list of kept blocks plus the incomplete block's tokens."""

    def __init__(self, block):
        self.block = block
        self.kept = None            # kept[b][h] = list of (k_block, v_block)
        self.tail_k = self.tail_v = None

    def feed(self, k, v, types):
        """k, v: the new tokens [B,n,HKV,D]; types [B,NB,HN,2] for the blocks that the incomplete block plus the new
        tokens make (the type of a still incomplete last block is ignored, src/nats/models/utils.py:516-519)."""
        B, n, HKV, _ = k.shape
        HN = types.shape[2]
        G = HKV // HN
        if self.kept is None:
            self.kept = [[[] for _ in range(HKV)] for _ in range(B)]
            self.tail_k, self.tail_v = k[:, :0], v[:, :0]
        allk, allv = torch.cat([self.tail_k, k], 1), torch.cat([self.tail_v, v], 1)
        total = allk.shape[1]
        n_complete = total // self.block
        if n_complete:
            assert types.shape[1] == -(-total // self.block)
        for j in range(n_complete):
            sl = slice(j * self.block, (j + 1) * self.block)
            for b in range(B):
                for h in range(HKV):
                    if types[b, j, h // G, 0] == 1:
                        self.kept[b][h].append((allk[b, sl, h], allv[b, sl, h]))
        self.tail_k, self.tail_v = allk[:, n_complete * self.block:], allv[:, n_complete * self.block:]

    def state(self):
        B, HKV = len(self.kept), len(self.kept[0])
        block = self.block
        counts_h = torch.tensor([[len(self.kept[b][h]) for h in range(HKV)] for b in range(B)], dtype=torch.int64)
        n_max = int(counts_h.max()) if counts_h.numel() else 0
        n_tail = self.tail_k.shape[1]
        out = {}
        for name, idx, tail in (('keys', 0, self.tail_k), ('values', 1, self.tail_v)):
            dense = torch.zeros(B, (n_max + 1) * block, HKV, tail.shape[-1], dtype=tail.dtype)
            for b in range(B):
                for h in range(HKV):
                    for i, blk in enumerate(self.kept[b][h]):
                        dense[b, i * block:(i + 1) * block, h] = blk[idx]
            if n_tail:
                dense[:, n_max * block:n_max * block + n_tail] = tail
            out[name] = dense
        out.update(n_attn_blocks_per_kv_head=counts_h, n_max=n_max, n_tail=n_tail)
        return out
