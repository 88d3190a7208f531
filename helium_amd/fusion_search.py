"""Fusion search over a whole fusion-IR graph — host-side mirror of helium-playground/src/fused_graph.rs,
cost_model.rs and subdivision.rs through the C ABI."""
import ctypes as C

from . import _ffi
from ._ffi import check, lib

MAXIMAL, MIN_NAIVE_COST, MIN_ANALYTICAL_COST, MIN_MI355X_COST = 0, 1, 2, 3
COST_TERMS = ["launches", "mma_flops", "mainloop_l2_bytes", "mainloop_ops", "hbm_bytes", "epilogue_ops", "aux_ops"]
ROLES = ["mainloop", "epilogue", "anchor", "aux"]
PORTIONS = ["mainloop", "epilogue", "full"]

_ffi._sig("he_fusion_search", C.c_void_p, C.c_int, C.POINTER(C.c_void_p))
_ffi._sig("he_fusion_search_subdivided", C.c_void_p, C.c_int, C.POINTER(C.c_void_p))
_ffi._sig("he_fusion_plan_num_fusions", C.c_void_p, C.POINTER(C.c_int))
_ffi._sig("he_fusion_plan_fusion_info", C.c_void_p, C.c_int, C.POINTER(C.c_int32), C.POINTER(C.c_uint64), C.POINTER(C.c_uint64),
          C.POINTER(C.c_int32), C.c_int, C.POINTER(C.c_int))
_ffi._sig("he_fusion_plan_describe", C.c_void_p, restype=C.c_char_p)
_ffi._sig("he_fusion_plan_cost", C.c_void_p, C.c_int, C.c_int, C.POINTER(C.c_double), C.POINTER(C.c_uint64))
_ffi._sig("he_fusion_plan_cost_terms", C.c_void_p, C.POINTER(C.c_double), C.c_int, C.POINTER(C.c_int))
_ffi._sig("he_fusion_plan_precompile", C.c_void_p)
_ffi._sig("he_fusion_plan_execute", C.c_void_p, C.POINTER(C.c_uint64), C.POINTER(C.c_void_p), C.c_int, C.POINTER(C.c_uint64),
          C.POINTER(C.c_void_p), C.c_int, C.c_void_p)
_ffi._sig("he_fusion_plan_destroy", C.c_void_p)
_ffi._sig("he_fgraph_subdivide", C.c_void_p, C.POINTER(C.c_uint64), C.POINTER(C.c_int32), C.POINTER(C.c_int32), C.c_int,
          C.POINTER(C.c_int))


class FusionPlan:
    """minimize_cost_function / produce_maximal_fusions for `graph`. `fusions` lists the kernels in execution
    order: {"core": bool, "anchor": id, "mainloop": [...], "epilogue": [...], "aux": [...]}."""

    def __init__(self, graph, objective=MAXIMAL, subdivided=False):
        """subdivided: minimize_cost_function_with_subdivision (cost_model.rs:241-259) — every subdivision is
        searched on its own and the results are merged (fused_graph.rs:910-1058)."""
        self.graph = graph
        self.handle = C.c_void_p()
        search = lib.he_fusion_search_subdivided if subdivided else lib.he_fusion_search
        check(search(graph.handle, objective, C.byref(self.handle)))
        n = C.c_int()
        check(lib.he_fusion_plan_num_fusions(self.handle, C.byref(n)))
        self.fusions = []
        cap = len(graph.nodes) + 1
        for i in range(n.value):
            core, anchor, count = C.c_int32(), C.c_uint64(), C.c_int()
            nodes, roles = (C.c_uint64 * cap)(), (C.c_int32 * cap)()
            check(lib.he_fusion_plan_fusion_info(self.handle, i, C.byref(core), C.byref(anchor), nodes, roles, cap, C.byref(count)))
            f = {"core": bool(core.value), "anchor": anchor.value if core.value else None, "mainloop": [], "epilogue": [], "aux": []}
            for k in range(count.value):
                if ROLES[roles[k]] != "anchor":
                    f[ROLES[roles[k]]].append(nodes[k])
            self.fusions.append(f)
        self.text = lib.he_fusion_plan_describe(self.handle).decode()

    def cost(self, objective=MIN_NAIVE_COST, reference_constants=False):
        c, states = C.c_double(), C.c_uint64()
        check(lib.he_fusion_plan_cost(self.handle, objective, int(reference_constants), C.byref(c), C.byref(states)))
        return c.value

    def cost_terms(self):
        """The terms of the MI355X cost model for this plan, by name (the model is their weighted sum)."""
        v, n = (C.c_double * 16)(), C.c_int()
        check(lib.he_fusion_plan_cost_terms(self.handle, v, 16, C.byref(n)))
        return dict(zip(COST_TERMS, v[: n.value]))

    def precompile(self):
        check(lib.he_fusion_plan_precompile(self.handle))

    def execute(self, producers, consumers, stream=None):
        """producers / consumers: {node id: DeviceBuffer}."""
        pn = _ffi.arr(C.c_uint64, list(producers.keys()))
        pp = (C.c_void_p * max(1, len(producers)))(*[b.ptr for b in producers.values()])
        cn = _ffi.arr(C.c_uint64, list(consumers.keys()))
        cp = (C.c_void_p * max(1, len(consumers)))(*[b.ptr for b in consumers.values()])
        check(lib.he_fusion_plan_execute(self.handle, pn, pp, len(producers), cn, cp, len(consumers),
                                         stream.handle if stream is not None else None))

    def __del__(self):
        try:
            if self.handle:
                lib.he_fusion_plan_destroy(self.handle)
                self.handle = C.c_void_p()
        except Exception:
            pass


def subdivide(graph):
    """subdivide (subdivision.rs:24-113): a list of sets of (node, portion)."""
    cap = 2 * len(graph.nodes) + 2
    nodes, portions, subs, count = (C.c_uint64 * cap)(), (C.c_int32 * cap)(), (C.c_int32 * cap)(), C.c_int()
    check(lib.he_fgraph_subdivide(graph.handle, nodes, portions, subs, cap, C.byref(count)))
    out = {}
    for k in range(count.value):
        out.setdefault(subs[k], set()).add((nodes[k], PORTIONS[portions[k]]))
    return [out[i] for i in sorted(out)]
