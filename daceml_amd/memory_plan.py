"""Launch order and placement of an SDFG's transients for a small memory footprint.

The reference leaves transients to DaCe, which allocates each one for the lifetime of the SDFG. Here the executor may
instead (``CompiledSDFG(reuse_transients=True)``) place them in one arena, by lifetime: a buffer that no later kernel
touches hands its bytes to the next buffer that is born. For a training step this is what decides whether the step's
working set fits the 256 MB last-level cache of the GPU: stored activations die one by one during the backward pass, and
the gradients of the same shapes can live where they were.

Both functions work on the graph only (no device), so the plan can be checked on any machine.
"""
from typing import Dict, List, Tuple

import torch

from .sdfg import SDFG, AccessNode, Array

_ITEM = {torch.float16: 2, torch.float32: 4, torch.float64: 8, torch.int64: 8, torch.int32: 4, torch.bool: 1}


def nbytes(desc: Array) -> int:
    n = _ITEM[desc.dtype]
    for d in desc.shape:
        n *= int(d)
    return n


def _root(sdfg: SDFG, name: str) -> str:
    while sdfg.arrays[name].view_of is not None:
        name = sdfg.arrays[name].view_of
    return name


def _placed(sdfg: SDFG, name: str) -> bool:
    return sdfg.arrays[name].transient and name not in sdfg.constants


def launch_order(sdfg: SDFG, small_peak: bool = False) -> List[Tuple[object, object]]:
    """[(state, node)]: the states in order, each state's nodes (access nodes left out) in topological order. With
    ``small_peak`` a state's order is chosen for a small peak of live transients: of the nodes that are ready, the one
    that adds the fewest bytes goes next (a weight-gradient contraction that is the last reader of a stored activation
    runs before the input-gradient contraction that needs a new buffer of that size). Two nodes that touch the same
    array, at least one of them writing it, keep the order the topological sort gave them."""
    topo = [(state, [n for n in state.topological_sort() if not isinstance(n, AccessNode)]) for state in sdfg.states()]
    if not small_peak:
        return [(state, n) for state, nodes in topo for n in nodes]
    touch = {}       # id(node) -> (roots read, roots written)
    users: Dict[str, int] = {}
    for state, nodes in topo:
        for n in nodes:
            rd = {_root(sdfg, e.data.data) for e in state.in_edges(n)}
            wr = {_root(sdfg, e.data.data) for e in state.out_edges(n)}
            touch[id(n)] = (rd, wr)
            for a in rd | wr:
                users[a] = users.get(a, 0) + 1
    seen = set()
    order = []
    for state, nodes in topo:
        before = {id(n): set() for n in nodes}
        for j, b in enumerate(nodes):
            rb, wb = touch[id(b)]
            for a in nodes[:j]:
                ra, wa = touch[id(a)]
                if (wa & (rb | wb)) or (wb & ra):
                    before[id(b)].add(id(a))
        left = list(nodes)
        done = set()
        while left:
            best, best_cost = None, None
            for n in left:
                if not before[id(n)] <= done:
                    continue
                both = touch[id(n)][0] | touch[id(n)][1]
                cost = sum(nbytes(sdfg.arrays[a]) for a in both if _placed(sdfg, a) and a not in seen) \
                    - sum(nbytes(sdfg.arrays[a]) for a in both if _placed(sdfg, a) and users[a] == 1)
                if best is None or cost < best_cost:
                    best, best_cost = n, cost
            left.remove(best)
            done.add(id(best))
            for a in touch[id(best)][0] | touch[id(best)][1]:
                seen.add(a)
                users[a] -= 1
            order.append((state, best))
    return order


def lifetimes(sdfg: SDFG, order) -> Tuple[Dict[str, int], Dict[str, int]]:
    """(first, last): for every transient that some node touches (views count for the array they live in), the
    positions in ``order`` of the first and the last node that does."""
    first: Dict[str, int] = {}
    last: Dict[str, int] = {}
    for pos, (state, node) in enumerate(order):
        for e in list(state.in_edges(node)) + list(state.out_edges(node)):
            r = _root(sdfg, e.data.data)
            if _placed(sdfg, r):
                first.setdefault(r, pos)
                last[r] = pos
    return first, last


def place_transients(sdfg: SDFG, order, align: int = 256, leave_out=()) -> Dict[str, int]:
    """Byte offsets in one arena for the transients, from their lifetimes in ``order``. A node's outputs are placed
    before its inputs are released, so no kernel reads and writes the same bytes under two names - unless the node says
    it may (``in_place``: {output connector: input connector}): then an output born at the node takes over the bytes of
    that input if the input dies there, has the same size and is connected to the node once. Among the free blocks that
    fit, the one released last is taken: its lines are the ones most likely to be in cache still. Arrays that no node
    touches, and those named in ``leave_out``, get no place (the caller gives them a buffer of their own)."""
    first, last = lifetimes(sdfg, order)
    for n in leave_out:
        first.pop(n, None)
        last.pop(n, None)
    size = {n: max((nbytes(sdfg.arrays[n]) + align - 1) // align * align, align) for n in first}
    free: List[List[int]] = []      # [offset, bytes, position of the release]
    end = 0
    plan: Dict[str, int] = {}
    for p, (state, node) in enumerate(order):
        heirs = {}      # output born here -> input that dies here and whose bytes it takes over
        names_in = {e.dst_conn: e.data.data for e in state.in_edges(node)}
        names_out = {e.src_conn: e.data.data for e in state.out_edges(node)}
        connected = [_root(sdfg, a) for a in list(names_in.values()) + list(names_out.values())]
        for oc, ic in getattr(node, "in_place", {}).items():
            o, i = names_out.get(oc), names_in.get(ic)
            if o in first and i in first and first[o] == p and last[i] == p and first[i] < p and size[o] == size[i] \
                    and i not in heirs.values() and connected.count(i) == 1:
                heirs[o] = i
        for o, i in heirs.items():
            plan[o] = plan[i]
        for n in sorted((n for n in first if first[n] == p and n not in heirs), key=lambda n: -size[n]):
            fits = [b for b in free if b[1] >= size[n]]
            if fits:
                b = max(fits, key=lambda b: (b[2], -b[1]))
                plan[n] = b[0]
                b[0] += size[n]
                b[1] -= size[n]
                if b[1] == 0:
                    free.remove(b)
            else:
                tail = [b for b in free if b[0] + b[1] == end]
                if tail:                 # grow the free block at the end of the arena
                    plan[n] = tail[0][0]
                    free.remove(tail[0])
                else:
                    plan[n] = end
                end = plan[n] + size[n]
        for n in (n for n in last if last[n] == p and n not in heirs.values()):
            block = [plan[n], size[n], p]
            for b in list(free):         # merge with free neighbours
                if b[0] + b[1] == block[0]:
                    block[0], block[1] = b[0], b[1] + block[1]
                    free.remove(b)
                elif block[0] + block[1] == b[0]:
                    block[1] += b[1]
                    free.remove(b)
            free.append(block)
    return plan
