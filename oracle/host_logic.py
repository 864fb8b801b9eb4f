"""Integer bookkeeping of the reference, restated in Python (TEST INFRASTRUCTURE ONLY).

Block pool / block tables / slot math follow inference/runtime/gpu_block_pool.go;
batch packing follows inference/scheduler/scheduler.go:245-303 and sequence.go;
candidate trees follow inference/medusa/tree.go; greedy verification and rollback
follow inference/scheduler/medusa_scheduler.go:852,934-977. All results are integers
and are compared bit-exactly.
"""
import math
from dataclasses import dataclass, field
from typing import Dict, List, Optional, Tuple

import numpy as np


# --------------------------------------------------------------------------- block pool
class PoolError(Exception):
    pass


@dataclass
class _SeqState:
    block_tables: List[List[int]]
    seq_len: int = 0


class GPUBlockPool:
    """gpu_block_pool.go:20-123 (integer state only; no K/V data here)."""

    def __init__(self, num_layers, num_kv_heads, head_dim, block_size, max_blocks, use_fp16=True):
        self.num_layers = num_layers
        self.num_kv_heads = num_kv_heads
        self.head_dim = head_dim
        self.block_size = block_size
        self.max_blocks = max_blocks
        self.use_fp16 = use_fp16
        self.bytes_per_element = 2 if use_fp16 else 4
        # gpu_block_pool.go:110-116: free list is [0..max-1]; allocation pops the tail
        self.free_lists = [list(range(max_blocks)) for _ in range(num_layers)]
        self.ref_counts: List[Dict[int, int]] = [dict() for _ in range(num_layers)]
        self.seqs: Dict[int, _SeqState] = {}

    # gpu_block_pool.go:126-135
    def create_sequence(self, seq_id):
        self.seqs[seq_id] = _SeqState(block_tables=[[] for _ in range(self.num_layers)])

    # gpu_block_pool.go:138-157
    def delete_sequence(self, seq_id):
        seq = self.seqs.get(seq_id)
        if seq is None:
            return
        for layer in range(self.num_layers):
            for b in seq.block_tables[layer]:
                self._release(layer, b)
        del self.seqs[seq_id]

    # gpu_block_pool.go:162-190
    def truncate_sequence(self, seq_id, new_len):
        seq = self.seqs.get(seq_id)
        if seq is None or new_len >= seq.seq_len:
            return
        new_blocks = 0
        if new_len > 0:
            new_blocks = (new_len - 1) // self.block_size + 1
        for layer in range(self.num_layers):
            bt = seq.block_tables[layer]
            for i in range(new_blocks, len(bt)):
                self._release(layer, bt[i])
            if new_blocks < len(bt):
                seq.block_tables[layer] = bt[:new_blocks]
        seq.seq_len = new_len

    def has_sequence(self, seq_id):
        return seq_id in self.seqs

    # gpu_block_pool.go:200-209
    def _alloc(self, layer):
        fl = self.free_lists[layer]
        if not fl:
            raise PoolError("no free blocks for layer %d (max=%d)" % (layer, self.max_blocks))
        b = fl.pop()
        self.ref_counts[layer][b] = 1
        return b

    # gpu_block_pool.go:211-219
    def _release(self, layer, b):
        rc = self.ref_counts[layer].get(b, 0)
        if rc <= 1:
            self.ref_counts[layer].pop(b, None)
            self.free_lists[layer].append(b)
        else:
            self.ref_counts[layer][b] = rc - 1

    # gpu_block_pool.go:223-323 (the integer part): returns [(physBlock, offset)] per token
    def store_kv_slots(self, layer, seq_id, start_pos, seq_len) -> List[Tuple[int, int]]:
        seq = self.seqs.get(seq_id)
        if seq is None:
            raise PoolError("sequence %d not found" % seq_id)
        end_pos = start_pos + seq_len
        last_block = (end_pos - 1) // self.block_size
        while len(seq.block_tables[layer]) <= last_block:
            seq.block_tables[layer].append(self._alloc(layer))
        slots = []
        for i in range(seq_len):
            pos = start_pos + i
            slots.append((seq.block_tables[layer][pos // self.block_size], pos % self.block_size))
        if end_pos > seq.seq_len:
            seq.seq_len = end_pos
        return slots

    # gpu_block_pool.go:337-389 (the integer part)
    def attention_args(self, layer, seq_id, kv_len=0):
        """-> (block_table[:numBlocks], numBlocks, tokensInLastBlock)"""
        seq = self.seqs.get(seq_id)
        if seq is None:
            raise PoolError("sequence %d not found" % seq_id)
        bt = seq.block_tables[layer]
        num_blocks = len(bt)
        if num_blocks == 0:
            raise PoolError("no blocks for seq %d layer %d" % (seq_id, layer))
        eff = seq.seq_len
        if kv_len > 0:
            eff = kv_len
        eff_blocks = (eff + self.block_size - 1) // self.block_size
        if eff_blocks < num_blocks:
            num_blocks = eff_blocks
        til = eff - (num_blocks - 1) * self.block_size
        return list(bt), num_blocks, til

    # gpu_block_pool.go:466-515 (the integer part)
    def attention_batched_args(self, layer, seq_ids):
        """-> (block_tables, seq_lens, max_blocks)"""
        tables, lens, mb = [], [], 0
        for sid in seq_ids:
            seq = self.seqs.get(sid)
            if seq is None:
                raise PoolError("sequence %d not found in GPU block pool" % sid)
            bt = seq.block_tables[layer]
            if not bt:
                raise PoolError("no blocks for seq %d layer %d" % (sid, layer))
            tables.append(list(bt))
            lens.append(seq.seq_len)
            mb = max(mb, len(bt))
        return tables, lens, mb

    # gpu_block_pool.go:572-607
    def share_blocks(self, src_id, dst_id, num_tokens):
        src = self.seqs.get(src_id)
        if src is None:
            raise PoolError("source sequence %d not found" % src_id)
        dst = self.seqs.get(dst_id)
        if dst is None:
            raise PoolError("destination sequence %d not found" % dst_id)
        nb = (num_tokens + self.block_size - 1) // self.block_size
        for layer in range(self.num_layers):
            if nb > len(src.block_tables[layer]):
                raise PoolError("source seq %d layer %d has %d blocks, need %d" %
                                (src_id, layer, len(src.block_tables[layer]), nb))
            for i in range(nb):
                b = src.block_tables[layer][i]
                dst.block_tables[layer].append(b)
                self.ref_counts[layer][b] = self.ref_counts[layer].get(b, 0) + 1
        if num_tokens > dst.seq_len:
            dst.seq_len = num_tokens

    # ---- named fragments: kv/fragment.go:18-101 and kv/paged_cache.go:285-343 over this pool's counters
    def cache_content(self, name, seq_id):
        """PagedKVCache.CacheContent: the sequence's blocks, one more reference each; replaces a fragment of that name."""
        seq = self.seqs.get(seq_id)
        if seq is None:
            return None                                       # paged_cache.go:331-333
        frags = self.__dict__.setdefault("fragments", {})
        if name in frags:                                     # fragment.go:41-43
            self._release_fragment(frags.pop(name))
        blocks = [list(bt) for bt in seq.block_tables]
        for layer in range(self.num_layers):
            for b in blocks[layer]:                           # fragment.go:46-50
                self.ref_counts[layer][b] = self.ref_counts[layer].get(b, 0) + 1
        frags[name] = (seq.seq_len, blocks)
        return frags[name]

    def _release_fragment(self, frag):                        # fragment.go:83-89
        for layer, blocks in enumerate(frag[1]):
            for b in blocks:
                self._release(layer, b)

    def delete_fragment(self, name):                          # fragment.go:71-79
        frags = self.__dict__.setdefault("fragments", {})
        if name in frags:
            self._release_fragment(frags.pop(name))

    def fragment(self, name):                                 # fragment.go:63-68
        return self.__dict__.setdefault("fragments", {}).get(name)

    # gpu_block_pool.go:610-624
    def block_stats(self):
        total = self.max_blocks * self.num_layers
        free = sum(len(fl) for fl in self.free_lists)
        shared = sum(1 for rc in self.ref_counts for v in rc.values() if v > 1)
        return total, free, shared

    # gpu_block_pool.go:627-635
    def memory_stats(self):
        total, free, _ = self.block_stats()
        used = total - free
        bpb = 2 * self.block_size * self.num_kv_heads * self.head_dim * self.bytes_per_element
        mb = 1024.0 * 1024.0
        return total * bpb / mb, used * bpb / mb, free * bpb / mb


def int32_le_bytes(values):
    """gpu_block_pool.go:660-670 (block tables are uploaded as int32 little endian)."""
    out = bytearray()
    for v in values:
        u = v & 0xFFFFFFFF
        out += bytes((u & 0xFF, (u >> 8) & 0xFF, (u >> 16) & 0xFF, (u >> 24) & 0xFF))
    return bytes(out)


# --------------------------------------------------------------------------- packing
@dataclass
class Sequence:
    """The fields of scheduler.Sequence that decide what gets packed (sequence.go:116-141,216-219)."""
    kv_seq_id: int
    prompt_tokens: List[int]
    prompt_pos: int = 0
    position: int = 0
    generated: List[int] = field(default_factory=list)

    def next_input_token(self):  # sequence.go:116-133
        if self.prompt_pos < len(self.prompt_tokens):
            return self.prompt_tokens[self.prompt_pos], self.prompt_pos, True
        if self.generated:
            return self.generated[-1], self.position, True
        return 0, 0, False

    def advance_position(self):  # sequence.go:136-141
        if self.prompt_pos < len(self.prompt_tokens):
            self.prompt_pos += 1
        self.position += 1

    def set_prefill_complete(self, num_tokens):  # sequence.go:216-219
        self.prompt_pos = len(self.prompt_tokens)
        self.position = num_tokens


def pack_decode_inputs(seqs: List[Sequence]):
    """scheduler.go:290-303: tokens[i], positions[i], seqIDs[i] for the decode batch.
    The reference takes the batch in Go map order; callers pass sequences ordered by id."""
    tokens, positions, seq_ids = [], [], []
    for s in seqs:
        tok, pos, more = s.next_input_token()
        if not more:
            tok, pos = 1, 0  # BOS fallback, scheduler.go:296-299
        tokens.append(tok)
        positions.append(pos)
        seq_ids.append(s.kv_seq_id)
    return tokens, positions, seq_ids


def pack_batch(pool: GPUBlockPool, layer, seq_ids, positions, q_lens=None):
    """What a batched step needs from the pool, derived from per-sequence StoreKV /
    Attention calls in batch order (block.go:866-874 runs StoreKV then Attention for each
    sequence; decode.go:642-650 runs the sequences in batch order).

    q_lens[i] new tokens of sequence i start at positions[i] (1 for decode).
    Returns dict with:
      cu_seqlens  [B+1]  prefix sum of q_lens
      slot_mapping[T]    physBlock*blockSize + offset for every new token
      token_pos   [T]    RoPE position of every new token
      kv_lens     [B]    context length after the store (positions[i]+q_lens[i])
      block_tables[B][maxBlocks] padded with -1, max_blocks
    """
    if q_lens is None:
        q_lens = [1] * len(seq_ids)
    cu = [0]
    slot_mapping, token_pos, kv_lens, tables = [], [], [], []
    for sid, pos, ql in zip(seq_ids, positions, q_lens):
        slots = pool.store_kv_slots(layer, sid, pos, ql)
        for i, (blk, off) in enumerate(slots):
            slot_mapping.append(blk * pool.block_size + off)
            token_pos.append(pos + i)
        cu.append(cu[-1] + ql)
        kv_lens.append(pos + ql)
    mb = 0
    for sid in seq_ids:
        bt = pool.seqs[sid].block_tables[layer]
        tables.append(list(bt))
        mb = max(mb, len(bt))
    padded = [bt + [-1] * (mb - len(bt)) for bt in tables]
    return dict(cu_seqlens=cu, slot_mapping=slot_mapping, token_pos=token_pos, kv_lens=kv_lens,
                block_tables=padded, max_blocks=mb)


# --------------------------------------------------------------------------- candidate trees
@dataclass
class _Node:
    token: int
    conf: float
    head: int
    depth: int
    parent: Optional["_Node"]
    children: List["_Node"] = field(default_factory=list)


class CandidateTree:
    """tree.go:25-28"""

    def __init__(self):
        self.root = _Node(-1, 0.0, -1, -1, None)
        self.num_nodes = 0

    # tree.go:104-135 (stable sort by confidence descending is what sort.Slice gives for
    # distinct confidences; ties are not ordered by the reference)
    def paths(self):
        out = []

        def dfs(node, toks, conf):
            if not node.children:
                out.append((list(toks), conf))
                return
            for c in node.children:
                dfs(c, toks + [c.token], conf + c.conf)

        dfs(self.root, [], 0.0)
        out.sort(key=lambda p: -p[1])
        return out

    # tree.go:144-178
    def linearize(self):
        queue = [(c, -1) for c in self.root.children]
        tokens, parent_idx = [], []
        head = 0
        while head < len(queue):
            node, ppos = queue[head]
            my = head
            head += 1
            tokens.append(node.token)
            parent_idx.append(ppos)
            for c in node.children:
                queue.append((c, my))
        return tokens, parent_idx


def build_candidate_tree_from_topk(head_topk_tokens, head_topk_vals, max_nodes):
    """tree.go:46-99 after the top-k selection (tree.go:59-67): head_topk_tokens[h] is the
    list of candidate ids of head h in descending-logit order."""
    if not head_topk_tokens:
        return None
    tree = CandidateTree()
    level = [tree.root]
    for h, (toks, vals) in enumerate(zip(head_topk_tokens, head_topk_vals)):
        nxt = []
        done = False
        for parent in level:
            for j in range(len(toks)):
                if tree.num_nodes >= max_nodes:
                    done = True
                    break
                child = _Node(toks[j], vals[j], h, h, parent)
                parent.children.append(child)
                nxt.append(child)
                tree.num_nodes += 1
            if done:
                break
        if done:
            break
        level = nxt
    return tree


def medusa_top_k(values, k):
    """heads.go:146-171 (topK): k rounds, each taking the first strictly largest value not yet used, starting from
    -MaxFloat32; a round that finds nothing yields -1."""
    k = min(k, len(values))
    used, out = [False] * len(values), []
    for _ in range(k):
        best_idx, best_val = -1, -3.4028234663852886e38
        for j, v in enumerate(values):
            if not used[j] and v > best_val:
                best_val, best_idx = v, j
        out.append(best_idx)
        if best_idx >= 0:
            used[best_idx] = True
    return out


def top_k_with_values(values, k):
    """tree.go:242-271 for inputs without ties among the top k."""
    k = min(k, len(values))
    idx = sorted(range(len(values)), key=lambda i: -values[i])[:k]
    return idx, [values[i] for i in idx]


def build_candidate_tree(head_logits, top_k, max_nodes):
    """tree.go:46-99"""
    if not head_logits:
        return None
    toks, vals = [], []
    for lg in head_logits:
        if len(lg) == 0:
            return None
        t, v = top_k_with_values(list(lg), top_k)
        toks.append(t)
        vals.append(v)
    return build_candidate_tree_from_topk(toks, vals, max_nodes)


def build_tree_attention_mask(n, parent_idx):
    """tree.go:186-202: mask[i*n+j] = node i attends to node j (self + ancestors)."""
    mask = [False] * (n * n)
    for i in range(n):
        mask[i * n + i] = True
        j = parent_idx[i]
        while j >= 0:
            mask[i * n + j] = True
            j = parent_idx[j]
    return mask


def tree_depths(parent_idx):
    d = []
    for i, p in enumerate(parent_idx):
        d.append(0 if p < 0 else d[p] + 1)
    return d


def argmax_list(values):
    """tree.go:274-287 / sampler.go:80-91"""
    if len(values) == 0:
        return 0
    mi, mv = 0, -3.4028234663852886e+38
    for i, v in enumerate(values):
        if v > mv:
            mv, mi = v, i
    return mi


def verify_tree_path(path_tokens, target_argmax):
    """tree.go:211-238 with targetLogits reduced to their argmax per position.
    Returns (accepted, finalToken)."""
    if not path_tokens:
        return 0, 0
    accepted, final = 0, 0
    for i, draft in enumerate(path_tokens):
        if i >= len(target_argmax):
            break
        t = target_argmax[i]
        if draft == t:
            accepted += 1
        else:
            return accepted, t
    if accepted == len(path_tokens) and len(target_argmax) > len(path_tokens):
        final = target_argmax[len(path_tokens)]
    elif 0 < accepted <= len(target_argmax):
        final = target_argmax[accepted - 1]
    return accepted, final


def select_best_tree_path(path0_tokens, verify_argmax):
    """medusa_scheduler.go:934-977 with verifyLogits reduced to per-position argmax.
    Returns (bestIdx=0, accepted, finalToken)."""
    if len(verify_argmax) == 0:
        return 0, 0, 0
    npos = len(verify_argmax)
    acc, final = 0, 0
    if path0_tokens:
        for i, draft in enumerate(path0_tokens):
            if i >= npos:
                break
            t = verify_argmax[i]
            if draft == t:
                acc += 1
            else:
                final = t
                break
        if acc == len(path0_tokens) and acc < npos:
            final = verify_argmax[acc]
    if acc == 0 and npos > 0 and final == 0:
        final = verify_argmax[0]
    return 0, acc, final


def cache_len_after_verify(start_pos, num_accepted):
    """medusa_scheduler.go:852"""
    return start_pos + 1 + num_accepted


def greedy_tree_accept(tokens, parent_idx, root_argmax, node_argmax):
    """Greedy acceptance over a whole candidate tree verified in one pass with the
    ancestor mask (the batched form of tree.go:211-238 applied to every root-to-leaf
    path at once): starting from the model's own next token root_argmax (the argmax of
    the logits at the input token), descend into the child whose token equals the
    current argmax; node_argmax[i] is the argmax of the logits computed at node i.
    Returns (accepted node indices in path order, final token)."""
    children: Dict[int, List[int]] = {}
    for i, p in enumerate(parent_idx):
        children.setdefault(p, []).append(i)
    accepted = []
    cur, want = -1, root_argmax
    while True:
        nxt = None
        for c in children.get(cur, []):
            if tokens[c] == want:
                nxt = c
                break
        if nxt is None:
            return accepted, want
        accepted.append(nxt)
        cur, want = nxt, node_argmax[nxt]


# --------------------------------------------------------------------------- sampler and scheduler step
def sampler_argmax(logits):
    """sampler.go:80-91: first index of the strict maximum, starting from -MaxFloat32."""
    best, idx = -np.finfo(np.float32).max, 0
    for i, v in enumerate(np.asarray(logits, dtype=np.float32)):
        if v > best:
            best, idx = v, i
    return idx


def sampler_sample(logits, temperature, top_k, top_p, r):
    """Sampler.Sample (sampler.go:48-77, 94-203) in float32, the uniform draw r given. Ties at the nucleus cutoff keep
    the lower index (the reference's sort.Slice is unstable: its order among equal probabilities is unspecified)."""
    f32 = np.float32
    logits = np.asarray(logits, dtype=f32)
    if temperature == 0:
        return sampler_argmax(logits)
    scaled = logits / f32(temperature)
    mx = -np.finfo(f32).max
    for v in scaled:
        if v > mx:
            mx = v
    probs = np.empty_like(scaled)
    s = f32(0)
    for i, v in enumerate(scaled):
        probs[i] = f32(math.exp(float(f32(v - mx))))
        s = f32(s + probs[i])
    probs = probs / s
    n = len(probs)
    if 0 < top_k < n:
        threshold = np.sort(probs)[::-1][top_k - 1]
        s = f32(0)
        for i in range(n):
            if probs[i] < threshold:
                probs[i] = 0
            else:
                s = f32(s + probs[i])
        if s > 0:
            probs = probs / s
    if 0 < top_p < 1.0:
        order = sorted(range(n), key=lambda i: (-float(probs[i]), i))
        cum, cutoff = f32(0), n
        for j, i in enumerate(order):
            cum = f32(cum + probs[i])
            if cum > f32(top_p):
                cutoff = j + 1
                break
        keep = set(order[:cutoff])
        s = f32(0)
        for i in range(n):
            if i not in keep:
                probs[i] = 0
            else:
                s = f32(s + probs[i])
        if s > 0:
            probs = probs / s
    cum = f32(0)
    for i in range(n):
        cum = f32(cum + probs[i])
        if f32(r) < cum:
            return i
    return n - 1


def splitmix_uniform(state):
    """The uniform stream of sampled requests: SplitMix64, top 24 bits. Returns (r, new state)."""
    mask = (1 << 64) - 1
    state = (state + 0x9E3779B97F4A7C15) & mask
    z = state
    z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & mask
    z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & mask
    z ^= z >> 31
    return float(np.float32(z >> 40) * np.float32(1.0 / 16777216.0)), state


PENDING, PREFILL, DECODING, FINISHED = range(4)  # sequence.go:15-20


class SchedSeq:
    def __init__(self, prompt, max_tokens=0):
        self.prompt, self.generated = list(prompt), []
        self.prompt_pos = self.position = 0
        self.state, self.max_tokens = PENDING, max_tokens
        self.sampling = None   # (temperature, top_k, top_p, rng state)

    def prefill_complete(self):  # sequence.go:205-207
        return self.prompt_pos >= len(self.prompt)

    def reached_max(self, global_max):  # sequence.go:196-202
        limit = self.max_tokens if self.max_tokens > 0 else global_max
        return limit > 0 and len(self.generated) >= limit


class Scheduler:
    """Scheduler.step (scheduler.go:166-483) over any model with prefill_with_paged_kv / decode_batched, sequences
    taken in ascending id; prefill_chunk > 0 feeds prompts in pieces, one per step."""

    def __init__(self, model, max_batch_size, max_tokens, eos_token, prefill_chunk=0):
        self.model, self.max_batch_size, self.max_tokens = model, max_batch_size, max_tokens
        self.eos, self.chunk = eos_token, prefill_chunk
        self.seqs: Dict[int, SchedSeq] = {}

    def add_sequence(self, seq_id, prompt, max_tokens=0):
        self.model.pool.create_sequence(seq_id)
        self.seqs[seq_id] = SchedSeq(prompt, max_tokens)

    def remove_sequence(self, seq_id):
        if seq_id in self.seqs:
            del self.seqs[seq_id]
            if self.model.pool.has_sequence(seq_id):
                self.model.pool.delete_sequence(seq_id)

    def _pick(self, q, logits):
        if q.sampling is None or q.sampling[0] == 0:
            return sampler_argmax(logits)
        t, k, p, st = q.sampling
        r, st = splitmix_uniform(st)
        q.sampling = (t, k, p, st)
        cap = getattr(getattr(self.model, "cfg", None), "final_softcap", 0.0)
        if cap > 0:                      # scheduler.go:772-773 -> model.go:336-350, sampled requests only
            from . import numerics as nx
            logits = nx.logit_softcap(logits, cap)
        return sampler_sample(logits, t, k, p, r)

    def step(self):
        batch = [i for i in sorted(self.seqs) if self.seqs[i].state in (PENDING, PREFILL, DECODING)][:self.max_batch_size]
        if not batch:
            for i in [i for i, q in self.seqs.items() if q.state == FINISHED]:
                self.remove_sequence(i)   # the reference only forgets it here; its KV blocks would leak
            return 0
        produced = 0
        for i in batch:
            q = self.seqs[i]
            if q.state not in (PENDING, PREFILL) or not q.prompt or q.prefill_complete():
                continue
            left = len(q.prompt) - q.prompt_pos
            n = min(left, self.chunk) if self.chunk > 0 else left
            logits = self.model.prefill_with_paged_kv(q.prompt[q.prompt_pos:q.prompt_pos + n], i, q.prompt_pos)
            q.prompt_pos += n
            q.position = q.prompt_pos
            if not q.prefill_complete():
                q.state = PREFILL
                continue
            tok = self._pick(q, logits)
            q.generated.append(tok)
            produced += 1
            q.state = FINISHED if tok == self.eos else DECODING
        dec = [i for i in batch if self.seqs[i].state == DECODING or
               (self.seqs[i].state == PENDING and self.seqs[i].prefill_complete())]
        if dec:
            toks, pos = [], []
            for i in dec:
                q = self.seqs[i]
                toks.append(q.generated[-1] if q.generated else 1)
                pos.append(q.position if q.generated else 0)
            logits = self.model.decode_batched(toks, dec, pos)
            for row, i in enumerate(dec):
                q = self.seqs[i]
                q.position += 1
                if q.state == PENDING:
                    q.state = DECODING
                tok = self._pick(q, logits[row])
                q.generated.append(tok)
                produced += 1
                if tok == self.eos or q.reached_max(self.max_tokens):
                    q.state = FINISHED
        return produced
