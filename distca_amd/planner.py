"""Which rank's CA server attends which part of which document.

Each rank holds whole documents for its linear layers.  Causal attention over a document of L
tokens costs L(L+1)/2 query-key pairs, so ranks whose batches hold long documents have far more
attention work than the others.  The planner moves attention work, not tokens: it cuts documents
into shards and names for every shard the rank whose CA server computes it (`ShardInfo.rid` = the
owner, `dispatch_rid` = the server).  The result is the plan `compute_metadata.from_planner_output`
turns into all-to-all metadata.

Same objective and cost unit as the reference (distca/planner/planner.py:366-378 cost of an item,
:627-732 greedy relocation, :394-402 bytes moved per unit of work as the order of preference); the
data structure is this file's own.  A document is peeled from its middle outwards in symmetric
layers: a layer of m tokens left of the middle and m tokens right of it costs m (L + 1) pairs
wherever it is taken (m (L + 2) for odd L), so the cost moved is linear in m and any amount can be
cut off exactly.  What remains with the owner is the outer pair (the first tokens, which are cheap,
and the last, which are dear).
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import List, Sequence, Tuple

from .compute_metadata import ShardInfo


def causal_cost(q: int, kv: int) -> int:
    """Query-key pairs of q query tokens that end a prefix of kv tokens (planner.py:366-378)."""
    return q * kv - q * (q - 1) // 2


@dataclass
class _Doc:
    owner: int
    length: int
    head: int                      # unpeeled tokens [0, head)
    tail: int                      # unpeeled tokens [length - tail, length)
    layers: List[Tuple[int, int]] = field(default_factory=list)   # (tokens per side, server rank) in the order peeled: innermost first
    server: int = -1               # server of the unpeeled pair

    def remaining_cost(self) -> int:
        return causal_cost(self.head, self.head) + causal_cost(self.tail, self.length)

    def layer_cost(self, m: int) -> int:
        """Cost of the next layer of m tokens per side."""
        lo = self.length - self.tail
        return causal_cost(m, self.head) + causal_cost(m, lo + m)

    def unit(self) -> int:
        """Cost per token-pair of a layer: layer_cost(m) == m * unit()."""
        return self.head + (self.length - self.tail) + 1


@dataclass
class PlannerConfig:
    q_token_bytes: int = 8192 + 8192   # a query token out and its attention output back
    kv_token_bytes: int = 2 * 2048     # a key and a value token
    tolerance: float = 0.05            # stop when every rank is within this fraction of the mean


def plan_documents(docs_per_rank: Sequence[Sequence[int]], config: PlannerConfig = PlannerConfig()):
    """docs_per_rank[r] = lengths of the documents rank r holds.  Returns (plan, load): the plan as
    one list of ShardInfo per document (documents in rank order, shards in position order) and the
    pairs each rank's CA server ends up with."""
    world = len(docs_per_rank)
    docs: List[_Doc] = []
    for r, lens in enumerate(docs_per_rank):
        for n in lens:
            if n <= 0:
                raise ValueError("document lengths must be positive")
            docs.append(_Doc(r, int(n), (int(n) + 1) // 2, int(n) // 2, server=r))
    load = [0] * world
    for d in docs:
        load[d.owner] += d.remaining_cost()
    mean = sum(load) / world if world else 0.0
    slack = mean * config.tolerance
    kv_on = [dict() for _ in docs]   # per document: server rank -> prefix length whose K/V it already gets

    for _ in range(64 * max(1, len(docs))):   # every step moves work or ends the loop
        recipient = min(range(world), key=lambda r: load[r])
        need = mean - load[recipient]
        if need <= slack:
            break
        best = None
        for i, d in enumerate(docs):
            donor = d.server
            surplus = load[donor] - mean
            if donor == recipient or surplus <= 0 or d.head + d.tail == 0:
                continue
            amount = min(need, surplus, d.remaining_cost())
            whole = amount >= d.remaining_cost()
            m = min(d.head, d.tail) if whole else int(amount // d.unit())
            if m <= 0 and not whole:
                continue
            moved = d.remaining_cost() if whole else d.layer_cost(m)
            prefix = d.length if whole else d.length - d.tail + m
            new_kv = max(0, prefix - kv_on[i].get(recipient, 0)) if d.owner != recipient else 0
            tokens = d.head + d.tail if whole else 2 * m
            bytes_moved = tokens * config.q_token_bytes * (d.owner != recipient) + new_kv * config.kv_token_bytes
            key = (bytes_moved / moved, -moved)
            if best is None or key < best[0]:
                best = (key, i, whole, m, moved, prefix)
        if best is None:
            break
        _, i, whole, m, moved, prefix = best
        d = docs[i]
        load[d.server] -= moved
        load[recipient] += moved
        if whole:
            d.server = recipient          # the unpeeled pair changes hands; peeled layers stay where they went
        else:
            d.layers.append((m, recipient))
            d.head -= m
            d.tail -= m
        kv_on[i][recipient] = max(kv_on[i].get(recipient, 0), prefix)

    plan = [_shards(d) for d in docs]
    return plan, load


def _shards(d: _Doc) -> List[ShardInfo]:
    """The document's pieces in position order, neighbours on the same server merged."""
    # the first layer peeled lies next to the middle, the last one next to the unpeeled pair
    left: List[Tuple[int, int]] = ([(d.head, d.server)] if d.head else []) + list(reversed(d.layers))
    right: List[Tuple[int, int]] = list(d.layers) + ([(d.tail, d.server)] if d.tail else [])
    pieces: List[List[int]] = []
    for n, server in left + right:
        if pieces and pieces[-1][1] == server:
            pieces[-1][0] += n
        else:
            pieces.append([n, server])
    assert sum(p[0] for p in pieces) == d.length
    return [ShardInfo(d.owner, server, i, n) for i, (n, server) in enumerate(pieces)]


def plan_cost_per_rank(plan: Sequence[Sequence[ShardInfo]], world_size: int) -> List[int]:
    """Pairs per server rank, counted from the plan itself."""
    load = [0] * world_size
    for doc in plan:
        end = 0
        for s in doc:
            end += s.shard_len
            load[s.dispatch_rid] += causal_cost(s.shard_len, end)
    return load
