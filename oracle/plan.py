"""CPU restatement of the reference's plan generation — TEST INFRASTRUCTURE ONLY (never imported by the product).

Follows helium/src/backend/plan_generation.rs (generate_plan = make_instr_graph + do_fusions +
generate_plan_from_graph + delay_computations + analyze_tensor_lifetimes), helium/src/cuda.rs:33-60
(make_instr_for_op), helium/src/cuda/instr/pointwise.rs:121-186 (supports_subgraph),
helium/src/cuda/instr/permute_dims.rs:95-142 (can_fuse_with / enumerate_swaps),
helium/src/cuda/instr/cudnn_graph.rs:319-321 (matmul instructions never fuse) and
helium-ir/src/opgraph/subgraph.rs:27-69 (inputs / leafs of a node set).

The instruction graph lives in a slotmap (slotmap 1.0.7, Cargo.lock; not vendored). Two documented properties of
that crate fix the greedy order and are restated here: keys order by slot index first, and freed slots are reused
last-in-first-out, so the instruction made by fusing `a` into `b` (remove a, remove b, insert) takes b's slot.

Pinned by: hand-derived plans for small graphs in tests/test_plan_cpu.py (the orders and release lists there are
worked out from the reference text by hand, not produced by this file) and by the invariants the reference asserts
under debug_assertions (plan_generation.rs:418-445). The exact grouping the reference would choose for a LARGE graph
can only be confirmed by running it, which this container cannot: parity unpinned beyond those checks.
"""
from . import helium_ir as hir

POINTWISE, PERMUTE, GEMM = "pointwise", "permute", "gemm"


class Graph:
    """Edges and descriptors of a helium-ir node list (the plain-data form helium_amd.ir.OpGraph.nodes records)."""

    def __init__(self, nodes):
        self.nodes = {n["id"]: n for n in nodes}
        self.order = [n["id"] for n in nodes]
        self.desc = {}
        self.inbound, self.outbound = {}, {i: [] for i in self.order}
        for n in nodes:
            i = n["id"]
            if n["node"] == "input":
                self.desc[i] = (list(n["shape"]), n["dtype"])
                self.inbound[i] = []
            elif n["node"] == "output":
                self.desc[i] = self.desc[n["from"]]
                self.inbound[i] = [n["from"]]
            else:
                self.desc[i] = hir.infer(n, self.desc)
                self.inbound[i] = list(n["inputs"])
            for p in self.inbound[i]:
                self.outbound[p].append(i)

    def numel(self, i):
        r = 1
        for d in self.desc[i][0]:
            r *= d
        return r

    def feeds_output(self, i):
        return any(self.nodes[o]["node"] == "output" for o in self.outbound[i])


class Instr:
    def __init__(self, graph, kind, nodes):
        self.g, self.kind, self.nodes = graph, kind, sorted(set(nodes))
        inside = set(self.nodes)
        ins = []
        for n in self.nodes:
            for p in graph.inbound[n]:
                if p not in inside and p not in ins:
                    ins.append(p)
        self.inputs = sorted(ins)
        self.outputs = [n for n in self.nodes if any(o not in inside for o in graph.outbound[n])]

    def merged(self, other):
        kind = GEMM if GEMM in (self.kind, other.kind) else self.kind
        return Instr(self.g, kind, self.nodes + other.nodes)

    def can_fuse_with(self, nxt, gemm_epilogue=None):
        if gemm_epilogue is not None and {self.kind, nxt.kind} == {GEMM, POINTWISE}:
            return bool(gemm_epilogue(self.merged(nxt)))
        if self.kind != nxt.kind:
            return False
        if self.kind == GEMM:
            return False
        m = self.merged(nxt)
        return supports_subgraph(m) if self.kind == POINTWISE else enumerate_swaps(m) is not None


def supports_subgraph(instr):
    g = instr.g
    output_size, reduction_shape, x = None, None, 0
    for node in instr.nodes:
        n = g.nodes[node]
        check = n["inputs"][0] if n["op"] == "reduce" else node
        if node in instr.outputs:
            if output_size is None:
                output_size = g.numel(check)
            elif output_size != g.numel(check):
                return False
        op = n["op"]
        if op in ("select", "reshape", "compare", "unary", "binary", "change_dtype"):
            continue
        if op == "broadcast":
            x += 1
        elif op == "swap_dims":
            x += 1
            if x > 1:
                return False
        elif op == "reduce":
            if node not in instr.outputs:
                return False
            # (not in the reference's text, which asks for a leaf only: a reduction that another member reads cannot
            # be computed by that member's threads, so such a merge is refused as well)
            if any(o in instr.nodes for o in g.outbound[node]):
                return False
            key = (list(g.desc[n["inputs"][0]][0]), n["depth"])
            if reduction_shape is None:
                reduction_shape = key
            elif reduction_shape != key:
                return False
        else:
            return False
    return True


def enumerate_swaps(instr):
    g = instr.g
    if len(instr.inputs) > 1:
        return None
    inside = set(instr.nodes)
    current = next(o for o in g.outbound[instr.inputs[0]] if o in inside)
    visited, swaps = [current], []
    while True:
        n = g.nodes[current]
        if n.get("op") != "swap_dims":
            return None
        swaps.append((n["axis_a"], n["axis_b"]))
        nxt = g.outbound[current]
        if len(nxt) == 1 and nxt[0] in inside:
            current = nxt[0]
            visited.append(current)
        else:
            break
    if any(n not in visited for n in instr.nodes):
        return None
    return swaps


def make_instr_for_op(g, node):
    op = g.nodes[node]["op"]
    if op == "swap_dims" and g.numel(node) > 1_000_000:
        return Instr(g, PERMUTE, [node])
    if op == "matmul":
        return Instr(g, GEMM, [node])
    return Instr(g, POINTWISE, [node])


class _InstrGraph:
    def __init__(self):
        self.instrs, self.next_slot = {}, 1
        self.producers, self.consumers = {}, {}
        self.dependencies, self.dependents = {}, {}

    def insert(self, instr, slot=None):
        if slot is None:
            slot, self.next_slot = self.next_slot, self.next_slot + 1
        self.instrs[slot] = instr
        for i in instr.inputs:
            self.consumers.setdefault(i, set()).add(slot)
            if i in self.producers:
                self.dependents[self.producers[i]].add(slot)
        for o in instr.outputs:
            assert o not in self.producers
            self.producers[o] = slot
            for c in self.consumers.get(o, ()):
                self.dependencies[c].add(slot)
        self.dependents[slot] = {c for o in instr.outputs for c in self.consumers.get(o, ())}
        self.dependencies[slot] = {self.producers[i] for i in instr.inputs if i in self.producers}
        return slot

    def remove(self, slot):
        instr = self.instrs.pop(slot)
        for i in instr.inputs:
            self.consumers[i].discard(slot)
            if i in self.producers:
                self.dependents[self.producers[i]].discard(slot)
        for o in instr.outputs:
            del self.producers[o]
            for c in self.consumers.get(o, ()):
                self.dependencies[c].discard(slot)
        del self.dependencies[slot], self.dependents[slot]
        return instr

    def exist_multiple_paths(self, a, b):
        stack = [d for d in sorted(self.dependents[a]) if d != b]
        visited = set(stack)
        while stack:
            cur = stack.pop()
            if cur == b:
                return True
            for n in sorted(self.dependents[cur]):
                if n not in visited:
                    visited.add(n)
                    stack.append(n)
        return False


def generate_plan(nodes, gemm_epilogue=None):
    """Returns [(instrs, tensors_to_release)], instrs = [(kind, [node ids])] in the reference's order.

    `gemm_epilogue`: None for the reference's rule (a matmul instruction never fuses). The backend's extension lets
    a matmul instruction and a pointwise one merge when the ops can run as the fused GEMM's epilogue; a test passes
    the predicate (merged Instr -> bool) that states which merges it expects to be admitted."""
    g = Graph(nodes)
    ig = _InstrGraph()
    for i in g.order:
        if g.nodes[i]["node"] == "op":
            ig.insert(make_instr_for_op(g, i))

    work = set(ig.instrs)
    while work:
        cur = min(work)
        work.discard(cur)
        for nxt in sorted(ig.dependents[cur]):
            if ig.instrs[cur].can_fuse_with(ig.instrs[nxt], gemm_epilogue) and not ig.exist_multiple_paths(cur, nxt):
                a, b = ig.remove(cur), ig.remove(nxt)
                new = ig.insert(a.merged(b), slot=nxt)
                work.discard(nxt)
                work.add(new)
                break

    if gemm_epilogue is not None:
        # the backend's second look: every product is offered its finished pointwise dependents again (a SwapDims
        # alone is no epilogue, SwapDims + Reduce is a column reduction), until nothing merges
        changed = True
        while changed:
            changed = False
            for cur in sorted(ig.instrs):
                if ig.instrs[cur].kind != "gemm":
                    continue
                for nxt in sorted(ig.dependents[cur]):
                    if (ig.instrs[nxt].kind == "pointwise" and ig.instrs[cur].can_fuse_with(ig.instrs[nxt], gemm_epilogue)
                            and not ig.exist_multiple_paths(cur, nxt)):
                        a, b = ig.remove(cur), ig.remove(nxt)
                        ig.insert(a.merged(b), slot=nxt)
                        changed = True
                        break
                if changed:
                    break

    total = len(ig.instrs)
    indeg, stack = {}, []
    for s in sorted(ig.instrs):
        indeg[s] = len(ig.dependencies[s])
        if indeg[s] == 0:
            stack.append(s)
    steps = []
    while stack:
        step, stack = stack, []
        for s in step:
            for nxt in sorted(ig.dependents[s]):
                indeg[nxt] -= 1
                assert indeg[nxt] >= 0
                if indeg[nxt] == 0:
                    stack.append(nxt)
        steps.append([ig.instrs[s] for s in step])
    assert sum(len(s) for s in steps) == total, "cycle detected in instruction graph?"

    for i in reversed(range(len(steps))):
        kept = []
        for instr in steps[i]:
            target = None
            for j in range(i + 1, len(steps)):
                if any(set(o.inputs) & set(instr.outputs) for o in steps[j]):
                    target = j - 1
                    break
            if target is not None and target != i:
                steps[target].append(instr)
            else:
                kept.append(instr)
        steps[i] = kept

    releases = [[]]
    for i, step in enumerate(steps):
        used = sorted({t for instr in step for t in instr.inputs})
        rel = []
        for t in used:
            if g.feeds_output(t):
                continue
            if not any(t in o.inputs for later in steps[i + 1:] for o in later):
                rel.append(t)
        releases.append(rel)
    steps.append([])
    return [([(x.kind, x.nodes) for x in step], rel) for step, rel in zip(steps, releases)]
