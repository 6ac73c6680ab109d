"""The apply / touch / fill nodes of one LLaMA decoder layer, in the merged forms the
reference's graph builder produces, and a sequential runner over the C-ABI kernel manager.

Derived from transformer_block_t::forward (llama/modules.cc:477-485), rms_norm_t (:126-195),
attention_t::forward (:282-356), feedforward_t::forward (:410-431) and
graph_writer_t::matmul / softmax_v1 / to_dtype (src/einsummable/gwriter.cc:763-855): virtual
transposes are folded into the einsummables' mode lists, a formation (here: a 1-D touch copy)
follows every contraction and reduction, the causal mask is a lower-triangular fill and the
attention scale 1/sqrt(head_dim) is computed but not applied (modules.cc:323-344).

Buffers are named byte ranges; a node reads and writes them under its own dtype (the
"complexer" view of an f32 tensor as c64 is the same bytes under another name).
"""
import math

from .km import C64, F16, F32, Einsummable, Touch

DT_NAME = {F16: "f16", F32: "f32", C64: "c64"}
DT_SIZE = {F16: 2, F32: 4, C64: 8}


def _g6(v):
    """Scalars reach a scalarop as 6-significant-digit text (write_with_ss,
    src/base/setup.h:621-626)."""
    return "%g" % v


class LayerGraph:
    def __init__(self, dim=4096, n_heads=32, ffn=11008, seq=2048, eps=1e-6):
        assert dim % n_heads == 0 and (dim // n_heads) % 2 == 0
        self.dim, self.n_heads, self.ffn, self.seq, self.eps = dim, n_heads, ffn, seq, eps
        self.hd = dim // n_heads
        self.buffers = {}   # name -> bytes
        self.nodes = []     # dicts
        self.inputs = {}    # name -> (dtype, shape)
        self._build()

    # ---- construction helpers
    def buf(self, name, dtype, nelem):
        nbytes = DT_SIZE[dtype] * nelem
        assert self.buffers.get(name, nbytes) == nbytes
        self.buffers[name] = nbytes
        return name

    def inp(self, name, dtype, shape):
        self.inputs[name] = (dtype, shape)
        return self.buf(name, dtype, math.prod(shape))

    def es(self, label, e, out, inns, flops=0):
        self.nodes.append({"kind": "einsummable", "label": label, "e": e, "out": out,
                           "inns": inns, "flops": flops})
        return out

    def formation(self, label, src, dtype, nelem):
        """formation node -> partialize with one input -> one 1-D copy touch
        (gwriter.cc:481, 503; taskgraph.cc:3047-3061)."""
        dst = self.buf(src + ".f", dtype, nelem)
        t = Touch([(nelem, nelem, 0, 0, nelem)], None, dtype)
        self.nodes.append({"kind": "touch", "label": label + " formation", "t": t, "out": dst,
                           "inn": src})
        return dst

    def unary(self, label, join, src, dt_in, dt_out, n, out=None):
        out = out or self.buf(label, dt_out, n)
        return self.es(label, Einsummable([n], [[0]], 1, join), out, [src])

    def rms_norm(self, p, x, w):
        s, d = self.seq, self.dim
        n = s * d
        xf = self.unary(p + "to_f32", "to_f32[hole|f16@0]", x, F16, F32, n)
        sq = self.unary(p + "square", "power{2}[hole|f32@0]", xf, F32, F32, n)
        ms = self.es(p + "sumsq", Einsummable([s, d], [[0, 1]], 1, "hole|f32@0", "+"),
                     self.buf(p + "sumsq", F32, s), [sq])
        ms = self.formation(p + "sumsq", ms, F32, s)
        scale_eps = "+[*[constant{f32|%s},hole|f32@0],constant{f32|%s}]" % (_g6(1.0 / d),
                                                                          _g6(self.eps))
        ms2 = self.unary(p + "mean_eps", scale_eps, ms, F32, F32, s)
        rs = self.unary(p + "rsqrt", "power{-0.5}[hole|f32@0]", ms2, F32, F32, s)
        xn = self.es(p + "x_rstd", Einsummable([s, d], [[0, 1], [0]], 2,
                                               "*[hole|f32@0,hole|f32@1]"),
                     self.buf(p + "x_rstd", F32, n), [xf, rs])
        xh = self.unary(p + "to_f16", "to_f16[hole|f32@0]", xn, F32, F16, n)
        return self.es(p + "weight", Einsummable([s, d], [[0, 1], [1]], 2,
                                                 "*[hole|f16@0,hole|f16@1]"),
                       self.buf(p + "weight", F16, n), [xh, w])

    def linear(self, label, x, w, n_in, n_out):
        s = self.seq
        e = Einsummable.from_str("ij,kj->ik", dict(i=s, j=n_in, k=n_out),
                                 "*[hole|f16@0,hole|f16@1]", "+")
        y = self.es(label, e, self.buf(label + ".mm", F16, s * n_out), [x, w],
                    flops=2 * s * n_in * n_out)
        return self.formation(label, y, F16, s * n_out)

    def rotary(self, p, x, freqs):
        s, h, hd = self.seq, self.n_heads, self.hd
        n = s * h * hd
        xf = self.unary(p + "to_f32", "to_f32[hole|f16@0]", x, F16, F32, n)
        # complexer view: [1, s, h, hd] f32 -> [1, s, h, hd/2] c64, same bytes
        e = Einsummable([1, s, h, hd // 2], [[0, 1, 2, 3], [1, 3]], 4, "*[hole|c64@0,hole|c64@1]")
        rot = self.es(p + "rotate", e, self.buf(p + "rotate", C64, n // 2), [xf, freqs])
        return self.unary(p + "to_f16", "to_f16[hole|f32@0]", rot, F32, F16, n)

    def _build(self):
        s, d, h, hd, f = self.seq, self.dim, self.n_heads, self.hd, self.ffn
        x = self.inp("x", F16, (1, s, d))
        w_an = self.inp("attention_norm.weight", F16, (d,))
        wq, wk, wv, wo = (self.inp("w" + c, F16, (d, d)) for c in "qkvo")
        w_fn = self.inp("ffn_norm.weight", F16, (d,))
        w1 = self.inp("w1", F16, (f, d))
        w2 = self.inp("w2", F16, (d, f))
        w3 = self.inp("w3", F16, (f, d))
        full_freqs = self.inp("full_freqs_cis", C64, (2 * s, hd // 2))

        # constants: causal mask (modules.cc:628-635), freqs_cis = full_freqs_cis[0:s]
        # (modules.cc:637-652; the subset simplifies to a 1-D touch)
        mask = self.buf("mask", F16, s * s)
        self.nodes.append({"kind": "lowertri", "label": "mask", "dtype": F16, "lower": 0.0,
                           "upper": -math.inf, "nrow": s, "ncol": s, "start": 0, "out": mask})
        nfr = s * (hd // 2)
        freqs = self.buf("freqs_cis", C64, nfr)
        self.nodes.append({"kind": "touch", "label": "freqs_cis subset",
                           "t": Touch([(2 * s, s, 0, 0, s), (hd // 2, hd // 2, 0, 0, hd // 2)],
                                      None, C64),
                           "out": freqs, "inn": full_freqs})

        # attention
        xa = self.rms_norm("an.", x, w_an)
        q = self.linear("wq", xa, wq, d, d)
        k = self.linear("wk", xa, wk, d, d)
        v = self.linear("wv", xa, wv, d, d)
        q = self.rotary("rq.", q, freqs)
        k = self.rotary("rk.", k, freqs)
        mul = "*[hole|f16@0,hole|f16@1]"
        e_scores = Einsummable.from_str("acbe,adbe->abcd", dict(a=1, b=h, c=s, d=s, e=hd), mul, "+")
        sc = self.es("scores", e_scores, self.buf("scores", F16, h * s * s), [q, k],
                     flops=2 * h * s * s * hd)
        sc = self.formation("scores", sc, F16, h * s * s)
        sc = self.es("scores+mask", Einsummable([h, s * s], [[0, 1], [1]], 2,
                                                "+[hole|f16@0,hole|f16@1]"),
                     self.buf("scores+mask", F16, h * s * s), [sc, mask])
        n_sc = h * s * s
        scf = self.unary("sm.to_f32", "to_f32[hole|f16@0]", sc, F16, F32, n_sc)
        mx = self.es("sm.rowmax", Einsummable([h * s, s], [[0, 1]], 1, "hole|f32@0", "^"),
                     self.buf("sm.rowmax", F32, h * s), [scf])
        mx = self.formation("sm.rowmax", mx, F32, h * s)
        sub = self.es("sm.sub", Einsummable([h * s, s], [[0, 1], [0]], 2,
                                            "+[hole|f32@0,*[constant{f32|-1},hole|f32@1]]"),
                      self.buf("sm.sub", F32, n_sc), [scf, mx])
        ex = self.unary("sm.exp", "exp[hole|f32@0]", sub, F32, F32, n_sc)
        sm = self.es("sm.rowsum", Einsummable([h * s, s], [[0, 1]], 1, "hole|f32@0", "+"),
                     self.buf("sm.rowsum", F32, h * s), [ex])
        sm = self.formation("sm.rowsum", sm, F32, h * s)
        pr = self.es("sm.div", Einsummable([h * s, s], [[0, 1], [0]], 2,
                                           "*[hole|f32@0,power{-1}[hole|f32@1]]"),
                     self.buf("sm.div", F32, n_sc), [ex, sm])
        prh = self.unary("sm.to_f16", "to_f16[hole|f32@0]", pr, F32, F16, n_sc)
        e_pv = Einsummable.from_str("abce,aebd->abcd", dict(a=1, b=h, c=s, e=s, d=hd), mul, "+")
        at = self.es("values", e_pv, self.buf("values", F16, s * d), [prh, v],
                     flops=2 * h * s * s * hd)
        at = self.formation("values", at, F16, s * d)
        e_o = Einsummable.from_str("adbe,cde->abc", dict(a=1, d=h, b=s, e=hd, c=d), mul, "+")
        ao = self.es("wo", e_o, self.buf("wo.mm", F16, s * d), [at, wo], flops=2 * s * d * d)
        ao = self.formation("wo", ao, F16, s * d)
        add = "+[hole|f16@0,hole|f16@1]"
        h1 = self.es("residual1", Einsummable([s * d], [[0], [0]], 1, add),
                     self.buf("residual1", F16, s * d), [x, ao])

        # feed forward: w2(silu(w1 x) * w3 x)
        xf = self.rms_norm("fn.", h1, w_fn)
        a1 = self.linear("w1", xf, w1, d, f)
        a3 = self.linear("w3", xf, w3, d, f)
        silu = "*[hole|f16@0,power{-1}[+[constant{f16|1},exp[*[constant{f16|-1},hole|f16@0]]]]]"
        g = self.unary("silu", silu, a1, F16, F16, s * f)
        g = self.es("gate", Einsummable([s * f], [[0], [0]], 1, mul), self.buf("gate", F16, s * f),
                    [g, a3])
        y = self.linear("w2", g, w2, f, d)
        self.output = self.es("residual2", Einsummable([s * d], [[0], [0]], 1, add),
                              self.buf("residual2", F16, s * d), [h1, y])

    def contraction_flops(self):
        return sum(n.get("flops", 0) for n in self.nodes)


def freqs_cis_table(n_pos, half_dim, theta=10000.0):
    """precompute_freqs_cis (llama/modules.cc:578-605): exp(i * t * theta^(-2j/dim)),
    as (real, imag) float pairs of shape [n_pos, half_dim, 2]."""
    import numpy as np

    dim = 2 * half_dim
    freqs = 1.0 / (theta ** (np.arange(0, dim, 2)[:half_dim].astype(np.float64) / dim))
    ang = np.outer(np.arange(n_pos, dtype=np.float64), freqs)
    return np.stack([np.cos(ang), np.sin(ang)], axis=-1).astype(np.float32)


class DeviceRunner:
    """Owns one device buffer per named range (a stand-in for the engine's arena) and runs the
    node list in order on one stream.  Every node goes through the C ABI."""

    def __init__(self, km, graph):
        import torch

        self.km, self.g, self.torch = km, graph, torch
        self.mem = {name: torch.empty(nbytes, dtype=torch.uint8, device="cuda")
                    for name, nbytes in graph.buffers.items()}
        need = 0
        for n in graph.nodes:
            if n["kind"] == "einsummable":
                ws = km.build(n["e"])
                assert ws is not None, "no kernel for node " + n["label"]
                n["ws"] = ws
                need = max(need, ws)
        # one scratch buffer serves every node: they run one after the other on one stream
        self.workspace = torch.empty(max(need, 1), dtype=torch.uint8, device="cuda")

    def set_input(self, name, array):
        import numpy as np

        t = self.torch.from_numpy(np.ascontiguousarray(array).view(np.uint8).reshape(-1))
        assert t.numel() == self.mem[name].numel(), name
        self.mem[name].copy_(t)

    def get(self, name, np_dtype):
        return self.mem[name].cpu().numpy().view(np_dtype)

    def run(self, stream=None, timers=None):
        import struct

        km = self.km
        stream = stream if stream is not None else self.torch.cuda.current_stream().cuda_stream
        for i, n in enumerate(self.g.nodes):
            def launch(n=n):
                if n["kind"] == "einsummable":
                    km(n["e"], stream, self.mem[n["out"]].data_ptr(),
                       [self.mem[b].data_ptr() for b in n["inns"]],
                       (self.workspace.data_ptr(), n["ws"]) if n["ws"] else None)
                elif n["kind"] == "touch":
                    km.touch(n["t"], stream, self.mem[n["out"]].data_ptr(),
                             self.mem[n["inn"]].data_ptr())
                else:
                    assert n["dtype"] == F16
                    lo = struct.unpack("<H", struct.pack("<e", n["lower"]))[0]
                    up = struct.unpack("<H", struct.pack("<e", n["upper"]))[0]
                    km.lowerTri_fill(n["dtype"], lo, up, n["nrow"], n["ncol"], n["start"], stream,
                                     self.mem[n["out"]].data_ptr())
            if timers is not None:
                timers[i].record(launch)
            else:
                launch()

    def capture(self):
        """Records the whole node list into a HIP graph (every node is a plain kernel launch
        on the given stream, so stream capture sees all of it) and returns the graph; replay
        removes the host's per-node launch cost."""
        torch = self.torch
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            self.run(stream=side.cuda_stream)      # everything compiled and loaded
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            self.run(stream=torch.cuda.current_stream().cuda_stream)
        return graph


class ArenaRunner:
    """The same node list through the exec-node layer: every buffer is a range of ONE device
    arena (as in the engine: `arena + mems[i].offset`, src/engine/gpu/exec_graph.cc:295-301),
    the dependencies follow from the ranges, the nodes are placed on `n_streams` streams at
    construction and run() enqueues the whole layer with no host synchronisation."""

    ALIGN = 256

    def __init__(self, km, graph, n_streams=4, optimize=False):
        """`optimize`: every range that is neither an input nor the layer's output gets the
        del node a memgraph holds for it (a dummy behind its last reader), and the exec graph
        may then absorb whole-range copies and single-reader elementwise nodes into their
        neighbours; what stays in memory keeps every bit."""
        import struct

        import torch

        from .km import ApplyGraph

        self.km, self.g, self.torch = km, graph, torch
        self.ranges, off = {}, 0
        for name, nbytes in graph.buffers.items():
            self.ranges[name] = (off, nbytes)
            off += (nbytes + self.ALIGN - 1) // self.ALIGN * self.ALIGN
        self.arena = torch.empty(max(off, 1), dtype=torch.uint8, device="cuda")
        ag = ApplyGraph(km)
        self.ids = []
        for n in graph.nodes:
            if n["kind"] == "einsummable":
                i = ag.add_einsummable(n["e"], [self.ranges[n["out"]]] +
                                       [self.ranges[b] for b in n["inns"]])
            elif n["kind"] == "touch":
                i = ag.add_touch(n["t"], -1, [self.ranges[n["out"]], self.ranges[n["inn"]]])
            else:
                assert n["dtype"] == F16
                lo = struct.unpack("<H", struct.pack("<e", n["lower"]))[0]
                up = struct.unpack("<H", struct.pack("<e", n["upper"]))[0]
                i = ag.add_lowertri_fill(n["dtype"], lo, up, n["nrow"], n["ncol"], n["start"],
                                         self.ranges[n["out"]])
            self.ids.append(i)
        self.absorbed = 0
        if optimize:
            last_reader = {}
            for i, n in zip(self.ids, graph.nodes):
                for b in n.get("inns", [n["inn"]] if "inn" in n else []):
                    last_reader[b] = i
            for name, i in last_reader.items():
                if name not in graph.inputs and name != graph.output:
                    ag.add_dummy(self.ranges[name], [i])
        ag.add_memory_dependencies()
        if optimize:
            self.absorbed = ag.optimize()
        ag.finalize(n_streams)
        self.graph = ag
        self.n_streams = n_streams

    def view(self, name):
        off, nbytes = self.ranges[name]
        return self.arena[off:off + nbytes]

    def set_input(self, name, array):
        import numpy as np

        t = self.torch.from_numpy(np.ascontiguousarray(array).view(np.uint8).reshape(-1))
        assert t.numel() == self.view(name).numel(), name
        self.view(name).copy_(t)

    def get(self, name, np_dtype):
        return self.view(name).cpu().numpy().view(np_dtype)

    def run(self, stream=None):
        stream = stream if stream is not None else self.torch.cuda.current_stream().cuda_stream
        self.graph.run(stream, self.arena.data_ptr())

    def capture(self):
        """The burst captured into one HIP graph.  Only for a single-stream placement:
        capturing a run whose pool streams fork from and join the capturing stream crashed
        inside the HIP runtime on ROCm 7.2 (host-side segmentation fault during capture),
        so that combination is refused here."""
        if self.n_streams != 1:
            raise NotImplementedError("HIP graph capture of a multi-stream exec graph is "
                                      "switched off (the runtime crashed during capture)")
        torch = self.torch
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            self.run(stream=side.cuda_stream)
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            self.run(stream=torch.cuda.current_stream().cuda_stream)
        return graph
