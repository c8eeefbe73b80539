"""Which rank's CA server attends which part of which document.

Each rank holds tokens for its linear layers.  Causal attention over a document of L tokens costs
L(L+1)/2 query-key pairs, so ranks whose batches hold long documents have far more attention work
than the others.  The planner moves attention work, not tokens: it cuts documents into shards and
names for every shard the rank whose CA server computes it (`ShardInfo.rid` = the rank of the linear
layers, `dispatch_rid` = the server).  The result is the plan
`compute_metadata.from_planner_output` turns into all-to-all metadata.

The surface is the reference's (distca/planner/planner.py): an `Item` is one rank's part of one
document, given as one `{'q', 'kv'}` dict (the whole document) or two (a span near the start and a
span near the end: `q` tokens that end a prefix of `kv` tokens), `batch_to_items_general` and
`batch_to_items_with_dummy` place a batch of documents onto ranks (:58-271), `Planner.plan_items`
balances the pairs per server (:627-732), `postprocess_items` and `items_into_shardinfos` turn the
result into the plan (:742-756, runtime/shard_info.py:115-141).  Same objective and cost unit as the
reference (:366-378 cost of an item, :394-402 bytes moved per unit of work as the order of
preference); the bodies are this file's own.

How work is cut: an item is peeled from its inner edges outwards in layers.  A layer of m tokens at
the end of the head span [.., h) and m tokens at the start of the tail span [t, ..) costs
m (h + t + 1) pairs, linear in m, so any amount can be cut off exactly (for a span pair that is
symmetric about the middle of a document of L tokens, h + t = L: the reference's L + 1 per token
pair, :446).  What remains with the server is the outer pair: the first tokens, which are cheap, and
the last, which are dear.
"""
from __future__ import annotations

import copy
from collections import defaultdict
from dataclasses import dataclass
from types import SimpleNamespace
from typing import Any, Dict, List, Optional, Sequence, Tuple

from .compute_metadata import ShardInfo


def causal_cost(q: int, kv: int) -> int:
    """Query-key pairs of q query tokens that end a prefix of kv tokens (planner.py:366-378)."""
    q, kv = int(q), int(kv)
    return q * kv - q * (q - 1) // 2


def get_flops(q=None, kv=None, **_):
    """Pairs of one `{'q', 'kv'}` dict; further keys are ignored (planner.py:832-834)."""
    if q is None or kv is None:
        raise ValueError("q and kv must be provided")
    return causal_cost(q, kv)


class Item:
    """One rank's part of one document (planner.py:334-516).

    `Item(model_config, seq_len, seqid, gpuid, src_gpuid, d)` holds the span d of document `seqid`
    (of `seq_len` tokens) whose tokens live on rank `src_gpuid` and whose attention runs on rank
    `gpuid`; with two dicts the item is a head span and a tail span.  `is_original` says that the
    attention still runs where the tokens are."""

    def __init__(self, model_config, seq_len, seqid, gpuid, src_gpuid, *item_dicts, is_original=True):
        if len(item_dicts) not in (1, 2):
            raise AssertionError("item_dicts must contain exactly 1 or 2 items")
        for d in item_dicts:
            if "q" not in d or "kv" not in d:
                raise AssertionError("Each item must have 'q' and 'kv' keys")
            if not 0 <= int(d["q"]) <= int(d["kv"]) <= int(seq_len):
                raise ValueError(f"span {d} does not lie in a document of {seq_len} tokens")
        self.model_config = model_config
        self.seq_len = int(seq_len)
        self.seqid = seqid
        self.gpuid = gpuid
        self.src_gpuid = src_gpuid
        self.is_original = is_original
        self.shard_id = None
        self.items: List[Dict[str, int]] = [{"q": int(d["q"]), "kv": int(d["kv"])} for d in item_dicts]
        self.total_flops = self.get_flops()

    # --- the reference's attribute names ------------------------------------------------------
    @property
    def complete(self) -> bool:
        return len(self.items) == 1

    @property
    def complete_item(self) -> Optional[Dict[str, int]]:
        return self.items[0] if self.complete else None

    @property
    def head(self) -> Dict[str, int]:
        if self.complete:
            raise AttributeError("a complete item has no head")
        return self.items[0]

    @property
    def tail(self) -> Dict[str, int]:
        if self.complete:
            raise AttributeError("a complete item has no tail")
        return self.items[1]

    def get_flops(self) -> int:
        return sum(causal_cost(d["q"], d["kv"]) for d in self.items)

    # --- cutting ------------------------------------------------------------------------------
    def _spans(self) -> Tuple[int, int, int, int]:
        """(h0, h1, t0, t1): head tokens [h0, h1), tail tokens [t0, t1).  A complete item counts as
        two halves that meet in its middle, the head the longer one."""
        if self.complete:
            d = self.items[0]
            lo, hi = d["kv"] - d["q"], d["kv"]
            mid = lo + (d["q"] + 1) // 2
            return lo, mid, mid, hi
        h, t = self.items
        return h["kv"] - h["q"], h["kv"], t["kv"] - t["q"], t["kv"]

    def layer_unit(self) -> int:
        """Pairs per token pair of the next layer: a layer of m tokens per side costs m * unit."""
        _, h1, t0, _ = self._spans()
        return h1 + t0 + 1

    def max_layer(self) -> int:
        h0, h1, t0, t1 = self._spans()
        return min(h1 - h0, t1 - t0)

    def peel(self, m: int, remote_gpuid) -> "Item":
        """Cut the innermost m tokens off either span into a new item served by `remote_gpuid`."""
        h0, h1, t0, t1 = self._spans()
        if not 0 < m <= min(h1 - h0, t1 - t0):
            raise ValueError(f"cannot peel {m} tokens per side off {self!r}")
        before = self.total_flops
        self.items = [{"q": h1 - m - h0, "kv": h1 - m}, {"q": t1 - t0 - m, "kv": t1}]
        self.total_flops = self.get_flops()
        new = Item(self.model_config, self.seq_len, self.seqid, remote_gpuid, self.src_gpuid,
                   {"q": m, "kv": h1}, {"q": m, "kv": t0 + m}, is_original=False)
        assert new.total_flops + self.total_flops == before
        return new

    def split_item(self, flops, remote_gpuid, verbose=False):
        """Move up to `flops` pairs of this item to rank `remote_gpuid` (planner.py:404-494).
        Returns (new item, pairs moved): the whole item changes server when `flops` covers it
        (then there is no new item), else the inner layers worth at most `flops` become a new item
        and this one shrinks; (None, 0) when not even one token pair fits."""
        if self.total_flops <= 0:
            return None, 0
        if flops >= self.total_flops:
            self.gpuid = remote_gpuid
            self.is_original = False
            return None, self.total_flops
        m = min(int(flops // self.layer_unit()), self.max_layer())
        if m <= 0:
            return None, 0
        new = self.peel(m, remote_gpuid)
        return new, new.total_flops

    def to_dicts(self) -> List[Dict[str, Any]]:
        """One dict per non-empty span (planner.py:499-515)."""
        return [{"q": d["q"], "kv": d["kv"], "gpuid": self.gpuid, "seqid": self.seqid, "src_gpuid": self.src_gpuid,
                 "is_original": self.is_original, "shard_id": self.shard_id} for d in self.items if d["q"] > 0]

    def __repr__(self):
        where = f"<Item seqid={self.seqid} src_gpuid = {self.src_gpuid} gpuid={self.gpuid} "
        if self.complete:
            d = self.items[0]
            return where + f"complete=q={d['q']} kv={d['kv']}>"
        h, t = self.items
        return where + f"split=head(q={h['q']}, kv={h['kv']}) tail(q={t['q']}, kv={t['kv']})>"


# ---------------------------------------------------------------------------------------------
# placing a batch onto ranks
# ---------------------------------------------------------------------------------------------
def _place(groups: Sequence[Sequence[int]], budget: int, ranks: int, model_config, dummies: bool) -> List[Item]:
    """Fill ranks in order with `budget` tokens each.  A document that fits what is left of the
    current rank becomes one complete item; one that does not is consumed from both ends at once,
    each rank taking half of its share from the front and half from the back, so that every rank's
    share costs about the same.  With `dummies`, a group of one document shorter than the budget is
    a placeholder that takes a rank of its own."""
    items: List[Item] = []
    room = [int(budget)] * ranks
    rank = 0
    seqid = 0

    def next_rank_with_room():
        nonlocal rank
        while rank < ranks and room[rank] == 0:
            rank += 1
        if rank >= ranks:
            raise ValueError(f"Not enough space to allocate document. seqid={seqid}: {ranks} ranks of {budget} tokens "
                             f"hold {ranks * budget}, the batch has {sum(sum(g) for g in groups)}")

    for group in groups:
        if dummies and len(group) == 1 and group[0] < budget:
            next_rank_with_room()
            if room[rank] != budget:
                raise AssertionError("dummy doc should put on a empty rank")
            n = int(group[0])
            items.append(Item(model_config, n, seqid, rank, rank, {"q": n, "kv": n}))
            rank += 1
            seqid += 1
            continue
        for n in group:
            n = int(n)
            front, back, left = 0, n, n
            first = True
            while left > 0:
                next_rank_with_room()
                take = min(left, room[rank])
                if first and take == n:
                    items.append(Item(model_config, n, seqid, rank, rank, {"q": n, "kv": n}))
                else:
                    a = take // 2
                    b = take - a
                    items.append(Item(model_config, n, seqid, rank, rank, {"q": a, "kv": front + a}, {"q": b, "kv": back},
                                      is_original=first))
                    front += a
                    back -= b
                room[rank] -= take
                left -= take
                first = False
            seqid += 1
    return items


def batch_to_items_general(batches: Sequence[Sequence[int]], num_tokens_per_rank: int, DP_degree: int, model_config) -> List[Item]:
    """Documents (lengths, in groups that only give the order) onto `DP_degree` ranks of
    `num_tokens_per_rank` tokens (planner.py:190-271)."""
    return _place(batches, num_tokens_per_rank, DP_degree, model_config, dummies=False)


def batch_to_items_with_dummy(batches: Sequence[Sequence[int]], num_tokens_per_rank: int, as_world_size: int, model_config) -> List[Item]:
    """As `batch_to_items_general`, where a group of one short document is an idle rank's
    placeholder and keeps that rank to itself (planner.py:58-131)."""
    return _place(batches, num_tokens_per_rank, as_world_size, model_config, dummies=True)


def cp_list_to_mlp_list(cp_rank_doc_lens: Sequence[Sequence[int]], as_world_size: int, num_token_per_rank: int) -> List[List[int]]:
    """Document lengths per context-parallel group -> piece lengths per rank of the linear layers
    (planner.py:276-327).  Every group starts on a fresh rank; a document that overflows a rank is
    cut the way `_place` cuts it and each rank lists its front piece and its back piece."""
    ranks: List[List[int]] = []
    for group in cp_rank_doc_lens:
        current: List[int] = []
        for n in group:
            left, cut = int(n), False
            while True:
                room = num_token_per_rank - sum(current)
                if room == 0:
                    ranks.append(current)
                    current, room = [], num_token_per_rank
                take = min(left, room)
                if take == left and not cut:
                    current.append(left)
                else:
                    current.extend([take // 2, take - take // 2])
                left -= take
                if left == 0:
                    break
                cut = True
        if current:
            ranks.append(current)
    ranks += [[] for _ in range(as_world_size - len(ranks))]
    return ranks[:as_world_size]


# ---------------------------------------------------------------------------------------------
# balancing
# ---------------------------------------------------------------------------------------------
@dataclass
class PlannerConfig:
    q_token_bytes: int = 8192 + 8192   # a query token out and its attention output back
    kv_token_bytes: int = 2 * 2048     # a key and a value token
    tolerance: float = 0.05            # stop when every rank is within this fraction of the mean


def _balance(items: List[Item], world: int, config: PlannerConfig) -> Tuple[List[Item], List[int]]:
    """Greedy relocation.  The least loaded server takes work, one move at a time, from whichever
    item of an overloaded server costs the fewest transported bytes per pair moved: the query tokens
    (and their outputs back) unless the recipient holds them anyway, plus the part of the K/V prefix
    the recipient does not get already.  A move is the whole item or some of its inner layers.
    Layers that have moved stay where they went.  Returns (all items, pairs per server)."""
    load = [0] * world
    for it in items:
        if not 0 <= it.gpuid < world or not 0 <= it.src_gpuid < world:
            raise ValueError(f"{it!r} names a rank outside 0..{world - 1}")
        load[it.gpuid] += it.total_flops
    mean = sum(load) / world if world else 0.0
    slack = mean * config.tolerance
    kv_on: Dict[Any, Dict[int, int]] = defaultdict(dict)   # document -> server -> K/V prefix it gets already
    for it in items:
        if it.gpuid != it.src_gpuid:
            kv_on[it.seqid][it.gpuid] = max(kv_on[it.seqid].get(it.gpuid, 0), max(d["kv"] for d in it.items))
    movable = list(items)
    moved_layers: List[Item] = []

    for _ in range(64 * max(1, len(items))):   # every step moves work or ends the loop
        recipient = min(range(world), key=lambda r: load[r])
        need = mean - load[recipient]
        if need <= 0 or (need <= slack and max(load) - mean <= slack):
            break
        best = None
        for i, it in enumerate(movable):
            donor = it.gpuid
            surplus = load[donor] - mean
            if donor == recipient or surplus <= 0 or it.total_flops <= 0:
                continue
            amount = min(need, surplus, it.total_flops)
            whole = amount >= it.total_flops
            m = 0 if whole else min(int(amount // it.layer_unit()), it.max_layer())
            if m <= 0 and not whole:
                continue
            h0, h1, t0, t1 = it._spans()
            cost = it.total_flops if whole else m * it.layer_unit()
            prefix = t1 if whole else t0 + m
            tokens = (h1 - h0) + (t1 - t0) if whole else 2 * m
            away = it.src_gpuid != recipient
            new_kv = max(0, prefix - kv_on[it.seqid].get(recipient, 0)) if away else 0
            bytes_moved = tokens * config.q_token_bytes * away + new_kv * config.kv_token_bytes
            key = (bytes_moved / cost, -cost)
            if best is None or key < best[0]:
                best = (key, i, whole, m, cost, prefix)
        if best is None:
            break
        _, i, whole, m, cost, prefix = best
        it = movable[i]
        load[it.gpuid] -= cost
        load[recipient] += cost
        if whole:
            it.gpuid = recipient
            it.is_original = False
        else:
            moved_layers.append(it.peel(m, recipient))
        if it.src_gpuid != recipient:
            kv_on[it.seqid][recipient] = max(kv_on[it.seqid].get(recipient, 0), prefix)
    return [it for it in movable + moved_layers if it.total_flops > 0], load


def postprocess_items(items: Sequence[Item]) -> List[Dict[str, Any]]:
    """Items -> one dict per span, numbered by position within the document (planner.py:742-756)."""
    dicts = [d for it in items for d in it.to_dicts()]
    by_doc: Dict[Any, List[Dict[str, Any]]] = defaultdict(list)
    for d in dicts:
        by_doc[d["seqid"]].append(d)
    for spans in by_doc.values():
        spans.sort(key=lambda d: d["kv"])
        at = 0
        for i, d in enumerate(spans):
            if d["kv"] - d["q"] != at:
                raise ValueError(f"document {d['seqid']}: spans leave a gap or overlap at token {at}")
            at = d["kv"]
            d["shard_id"] = i
    return dicts


def items_into_shardinfos(item_dicts: Sequence[Dict[str, Any]]) -> List[List[ShardInfo]]:
    """Span dicts -> the plan: one list per document in order of first appearance, shards in
    position order (runtime/shard_info.py:115-141)."""
    by_doc: Dict[Any, List[Dict[str, Any]]] = {}
    for d in item_dicts:
        by_doc.setdefault(d["seqid"], []).append(d)
    return [[ShardInfo(d["src_gpuid"], d["gpuid"], d["shard_id"], d["q"]) for d in sorted(spans, key=lambda d: d["shard_id"])]
            for spans in by_doc.values()]


class Planner:
    """planner.py:550-829.  `world_size` counts all ranks; the CA servers are one per tensor-parallel
    group, `attention_server_world_size` of them."""

    def __init__(self, world_size: int, parallel_config, tolerance_factor: float = 0.1, model_config=None, dtype=None):
        self.model_config = model_config
        self.world_size = world_size
        self.parallel_config = parallel_config
        tp = parallel_config.tensor_model_parallel_size
        pp = parallel_config.pipeline_model_parallel_size
        self.data_parallel = world_size // (pp * tp)
        self.attention_server_world_size = self.data_parallel * pp
        self.tolerance_factor = tolerance_factor
        if dtype is None:
            import torch
            dtype = torch.bfloat16
        self.dtype = dtype

    @classmethod
    def from_individual_params(cls, tp_size: int, pp_size: int, dp_size: int, world_size: int, hidden_size_q: int, hidden_size_k: int):
        """A planner from per-rank hidden sizes instead of a model config (planner.py:806-829).  The
        stand-in model has one key/value head per hidden_size_q / hidden_size_k query heads, so that
        the sizes derived from it are the ones given."""
        return cls(world_size=world_size,
                   parallel_config=SimpleNamespace(tensor_model_parallel_size=tp_size, pipeline_model_parallel_size=pp_size),
                   model_config=SimpleNamespace(hidden_size=hidden_size_q * tp_size, num_attention_heads=hidden_size_q // hidden_size_k,
                                                num_key_value_heads=1, num_hidden_layers=1))

    def _hidden_sizes(self) -> Tuple[int, int]:
        """(query, key) elements per token on one rank of a tensor-parallel group."""
        mc, tp = self.model_config, self.parallel_config.tensor_model_parallel_size
        hq = mc.hidden_size
        hk = hq * getattr(mc, "num_key_value_heads", mc.num_attention_heads) // mc.num_attention_heads
        return hq // tp, hk // tp

    def _config(self) -> PlannerConfig:
        if self.model_config is None:
            return PlannerConfig(tolerance=self.tolerance_factor)
        hq, hk = self._hidden_sizes()
        size = self.dtype.itemsize
        return PlannerConfig(q_token_bytes=2 * hq * size, kv_token_bytes=2 * hk * size, tolerance=self.tolerance_factor)

    def plan_items(self, items_: Sequence[Item], verbose=False, plot=False) -> List[Item]:
        """The balanced items; the input is left as it is (planner.py:627-732)."""
        items, load = _balance(copy.deepcopy(list(items_)), self.attention_server_world_size, self._config())
        if verbose:
            print(f"pairs per server after planning: {load}")
        return items

    def postprocess_items(self, items: Sequence[Item]) -> List[Dict[str, Any]]:
        return postprocess_items(items)

    def items_into_shardinfos(self, item_dicts):
        return items_into_shardinfos(item_dicts)

    def items_to_shardinfo(self, items_: Sequence[Item], verbose=False) -> List[List[ShardInfo]]:
        """planner.py:735-739."""
        return items_into_shardinfos(postprocess_items(self.plan_items(items_, verbose)))

    def items_to_mlp_doc_len(self, items: Sequence[Item], device: str = "cuda"):
        """Per rank of the linear layers: the lengths of the spans it holds, and their [start, end)
        within their documents, in order of (rank, document) (planner.py:758-801)."""
        import torch
        lens: List[List[int]] = [[] for _ in range(self.attention_server_world_size)]
        ranges: List[List[List[int]]] = [[] for _ in range(self.attention_server_world_size)]
        for it in sorted(items, key=lambda it: (it.src_gpuid, it.seqid)):   # stable: ties keep the order given
            for d in it.items:
                lens[it.src_gpuid].append(d["q"])
                ranges[it.src_gpuid].append([d["kv"] - d["q"], d["kv"]])
        return ([torch.tensor(x, dtype=torch.int32, device=device) for x in lens],
                [torch.tensor(x, dtype=torch.int32, device=device) for x in ranges])

    def plan(self, items_: Sequence[Item], verbose=False, plot=False, is_resend_qkv: bool = False, device: str = "cuda"):
        """Items -> (the four all-to-all metadata, attention cu_seqlens per rank, span lengths per
        rank, span ranges per rank) (planner.py:567-608)."""
        from .compute_metadata import from_planner_output
        import torch
        if self.parallel_config.pipeline_model_parallel_size != 1:
            raise NotImplementedError("a pipelined step is planned tick by tick, not here")
        mlp_shard_len, shard_logical_range = self.items_to_mlp_doc_len(items_, device=device)
        plan = self.items_to_shardinfo(items_, verbose)
        hq, hk = self._hidden_sizes()
        size = self.dtype.itemsize
        lse_size = self.model_config.num_attention_heads // self.parallel_config.tensor_model_parallel_size
        if getattr(self.model_config, "attention_softmax_in_fp32", True):
            lse_size *= torch.float32.itemsize // size
        qkv_fwd, qkv_rev, out_fwd, out_rev, attn = from_planner_output(
            self.attention_server_world_size, plan, hq, hk, lse_size, size, is_pipeline_tick=False, is_resend_qkv=is_resend_qkv)
        return (qkv_fwd, qkv_rev, out_fwd, out_rev), attn, mlp_shard_len, shard_logical_range


# ---------------------------------------------------------------------------------------------
# whole documents in, plan out
# ---------------------------------------------------------------------------------------------
def plan_documents(docs_per_rank: Sequence[Sequence[int]], config: PlannerConfig = PlannerConfig()):
    """docs_per_rank[r] = lengths of the documents rank r holds.  Returns (plan, load): the plan as
    one list of ShardInfo per document (documents in rank order, shards in position order,
    neighbours on one server merged) and the pairs each rank's CA server ends up with."""
    items: List[Item] = []
    for r, lens in enumerate(docs_per_rank):
        for n in lens:
            if n <= 0:
                raise ValueError("document lengths must be positive")
            items.append(Item(None, int(n), len(items), r, r, {"q": int(n), "kv": int(n)}))
    planned, load = _balance(items, len(docs_per_rank), config)
    plan = []
    for doc in items_into_shardinfos(postprocess_items(planned)):
        merged: List[ShardInfo] = []
        for s in doc:
            if merged and merged[-1].dispatch_rid == s.dispatch_rid and merged[-1].rid == s.rid:
                merged[-1] = ShardInfo(s.rid, s.dispatch_rid, merged[-1].logical_sid, merged[-1].shard_len + s.shard_len)
            else:
                merged.append(ShardInfo(s.rid, s.dispatch_rid, len(merged), s.shard_len))
        plan.append(merged)
    return plan, load


def plan_cost_per_rank(plan: Sequence[Sequence[ShardInfo]], world_size: int) -> List[int]:
    """Pairs per server rank, counted from the plan itself."""
    load = [0] * world_size
    for doc in plan:
        end = 0
        for s in doc:
            end += s.shard_len
            load[s.dispatch_rid] += causal_cost(s.shard_len, end)
    return load
