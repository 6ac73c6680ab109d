"""An independent encoder for serialized memgraphs, for the tests of the wire reader.

The schema below restates the messages of the reference's src/proto/einsummable.proto that a
MemGraph is made of (MemGraph :233-238, MemGraphNode :216-231, MGApply :156-165, the other MG*
:137-214, Einsummable :9-15, Touch :17-33, Fill :35-51) as data: field name, number, type,
label.  The message classes are built from it at run time by the protobuf library that ships
with Python, so the bytes the tests feed to the C++ reader come from Google's encoder, not
from code that shares anything with the reader.

A memgraph is described by plain dicts (`node(...)` below); `to_wire` serialises one and
`describe` gives the text es_km_memgraph_describe must produce for it.
"""
from google.protobuf import descriptor_pb2, descriptor_pool, message_factory

_F = descriptor_pb2.FieldDescriptorProto
_TYPES = {"int32": _F.TYPE_INT32, "uint64": _F.TYPE_UINT64, "int64": _F.TYPE_INT64,
          "string": _F.TYPE_STRING, "bool": _F.TYPE_BOOL}
_LABELS = {"req": _F.LABEL_REQUIRED, "opt": _F.LABEL_OPTIONAL, "rep": _F.LABEL_REPEATED}

_LOS = [("loc", 1, "int32", "req"), ("offset", 2, "uint64", "req"), ("size", 3, "uint64", "req")]
_STO = [("storage_loc", 1, "int32", "req"), ("storage_id", 2, "int32", "req"),
        ("loc", 3, "int32", "req"), ("offset", 4, "uint64", "req"), ("size", 5, "uint64", "req")]

# (name, number, type, label[, oneof])
SCHEMA = {
    "EsInn": [("idxs", 1, "int32", "rep")],
    "Einsummable": [("join_shape", 1, "uint64", "rep"), ("inns", 2, "EsInn", "rep"),
                    ("out_rank", 3, "int32", "req"), ("join", 4, "string", "req"),
                    ("castable", 5, "string", "opt")],
    "TouchDim": [("d_inn", 1, "uint64", "req"), ("d_out", 2, "uint64", "req"),
                 ("offset_inn", 3, "uint64", "req"), ("offset_out", 4, "uint64", "req"),
                 ("size", 5, "uint64", "req")],
    "Touch": [("selection", 1, "TouchDim", "rep"), ("castable", 2, "string", "opt"),
              ("dtype", 3, "string", "req")],
    "Constant": [("value", 1, "string", "req"), ("shape", 2, "uint64", "rep")],
    "Lowertri": [("lower", 1, "string", "req"), ("upper", 2, "string", "req"),
                 ("ncol", 3, "uint64", "req"), ("nrow", 4, "uint64", "req"),
                 ("start", 5, "int64", "req")],
    "Fill": [("constant", 1, "Constant", "opt", "op"), ("lowertri", 2, "Lowertri", "opt", "op")],
    "MGInputMem": _LOS,
    "MGInputSto": [("storage_loc", 1, "int32", "req"), ("storage_id", 2, "int32", "req"),
                   ("size", 3, "uint64", "req")],
    "MGConstant": [("loc", 1, "int32", "req"), ("offset", 2, "uint64", "req"),
                   ("fill", 3, "Fill", "req")],
    "MGApply": [("loc", 1, "int32", "req"), ("mems_offset", 2, "uint64", "rep"),
                ("mems_size", 3, "uint64", "rep"), ("einsummable", 4, "Einsummable", "opt", "op"),
                ("touch", 5, "Touch", "opt", "op"), ("group", 6, "int32", "req")],
    "MGMove": [("src_loc", 1, "int32", "req"), ("src_offset", 2, "uint64", "req"),
               ("dst_loc", 3, "int32", "req"), ("dst_offset", 4, "uint64", "req"),
               ("size", 5, "uint64", "req")],
    "MGCopy": [("loc", 1, "int32", "req"), ("size", 2, "uint64", "req"),
               ("src_offset", 3, "uint64", "req"), ("dst_offset", 4, "uint64", "req")],
    "MGEvict": _STO,
    "MGLoad": _STO,
    "MGPartialize": _LOS,
    "MGAlloc": _LOS,
    "MGDel": _LOS,
    "MemGraphNode": [("inputmem", 1, "MGInputMem", "opt", "node"),
                     ("inputsto", 2, "MGInputSto", "opt", "node"),
                     ("constant", 3, "MGConstant", "opt", "node"),
                     ("apply", 4, "MGApply", "opt", "node"),
                     ("move", 5, "MGMove", "opt", "node"),
                     ("copy", 100, "MGCopy", "opt", "node"),
                     ("evict", 6, "MGEvict", "opt", "node"),
                     ("load", 7, "MGLoad", "opt", "node"),
                     ("partialize", 8, "MGPartialize", "opt", "node"),
                     ("alloc", 9, "MGAlloc", "opt", "node"),
                     ("del", 10, "MGDel", "opt", "node"),
                     ("inns", 11, "int32", "rep")],
    "MemGraph": [("num_compute_locs", 1, "int32", "req"), ("num_storage_locs", 2, "int32", "req"),
                 ("storage_locs", 3, "int32", "rep"), ("nodes", 4, "MemGraphNode", "rep")],
}

KIND_NUMBER = {"inputmem": 1, "inputsto": 2, "constant": 3, "apply": 4, "move": 5, "evict": 6,
               "load": 7, "partialize": 8, "alloc": 9, "del": 10, "copy": 100}


def _build(package, packed):
    fd = descriptor_pb2.FileDescriptorProto()
    fd.name = package + ".proto"
    fd.package = package
    fd.syntax = "proto2"
    for mname, fields in SCHEMA.items():
        m = fd.message_type.add()
        m.name = mname
        oneofs = []
        for f in fields:
            name, number, typ, label = f[:4]
            fld = m.field.add()
            fld.name = name
            fld.number = number
            fld.label = _LABELS[label]
            if typ in _TYPES:
                fld.type = _TYPES[typ]
                if packed and label == "rep":
                    fld.options.packed = True
            else:
                fld.type = _F.TYPE_MESSAGE
                fld.type_name = "." + package + "." + typ
            if len(f) == 5:
                if f[4] not in oneofs:
                    oneofs.append(f[4])
                    m.oneof_decl.add().name = f[4]
                fld.oneof_index = oneofs.index(f[4])
    pool = descriptor_pool.DescriptorPool()
    pool.Add(fd)
    return {n: message_factory.GetMessageClass(pool.FindMessageTypeByName(package + "." + n))
            for n in SCHEMA}


_CLASSES = {}


def classes(packed=False):
    """Message classes; packed=True encodes repeated scalars in the packed form (one
    length-delimited run), which every protobuf reader accepts for the same schema."""
    if packed not in _CLASSES:
        _CLASSES[packed] = _build("es_proto_packed" if packed else "es_proto", packed)
    return _CLASSES[packed]


def node(kind, inns=(), **fields):
    d = dict(kind=kind, inns=sorted(set(inns)))
    d.update(fields)
    return d


def _fill_einsummable(msg, e):
    msg.join_shape.extend(e["join_shape"])
    for inn in e["inns"]:
        msg.inns.add().idxs.extend(inn)
    msg.out_rank = e["out_rank"]
    msg.join = e["join"]
    if e.get("castable"):
        msg.castable = e["castable"]


def _fill_touch(msg, t):
    for d in t["selection"]:
        td = msg.selection.add()
        td.d_inn, td.d_out, td.offset_inn, td.offset_out, td.size = d
    if t.get("castable"):
        msg.castable = t["castable"]
    msg.dtype = t["dtype"]


def to_message(mg, packed=False):
    """mg: dict(num_compute_locs, num_storage_locs, storage_locs, nodes=[node(...)])."""
    C = classes(packed)
    out = C["MemGraph"]()
    out.num_compute_locs = mg["num_compute_locs"]
    out.num_storage_locs = mg["num_storage_locs"]
    out.storage_locs.extend(mg.get("storage_locs", []))
    for n in mg["nodes"]:
        pn = out.nodes.add()
        k = n["kind"]
        if k in ("inputmem", "partialize", "alloc", "del"):
            m = getattr(pn, k)
            m.loc, m.offset, m.size = n["loc"], n["offset"], n["size"]
        elif k == "inputsto":
            m = pn.inputsto
            m.storage_loc, m.storage_id, m.size = n["storage_loc"], n["storage_id"], n["size"]
        elif k == "constant":
            m = pn.constant
            m.loc, m.offset = n["loc"], n["offset"]
            f = n["fill"]
            if "lower" in f:
                lt = m.fill.lowertri
                lt.lower, lt.upper = f["lower"], f["upper"]
                lt.nrow, lt.ncol, lt.start = f["nrow"], f["ncol"], f["start"]
            else:
                m.fill.constant.value = f["value"]
                m.fill.constant.shape.extend(f["shape"])
        elif k == "apply":
            m = pn.apply
            m.loc = n["loc"]
            m.mems_offset.extend(o for o, _ in n["mems"])
            m.mems_size.extend(s for _, s in n["mems"])
            if "einsummable" in n:
                _fill_einsummable(m.einsummable, n["einsummable"])
            else:
                _fill_touch(m.touch, n["touch"])
            m.group = n["group"]
        elif k == "move":
            m = pn.move
            m.src_loc, m.src_offset = n["src_loc"], n["src_offset"]
            m.dst_loc, m.dst_offset, m.size = n["loc"], n["offset"], n["size"]
        elif k == "copy":
            m = pn.copy
            m.loc, m.size = n["loc"], n["size"]
            m.src_offset, m.dst_offset = n["src_offset"], n["offset"]
        elif k in ("evict", "load"):
            m = getattr(pn, k)
            m.storage_loc, m.storage_id = n["storage_loc"], n["storage_id"]
            m.loc, m.offset, m.size = n["loc"], n["offset"], n["size"]
        else:
            raise ValueError(k)
        pn.inns.extend(n["inns"])
    return out


def to_wire(mg, packed=False):
    return to_message(mg, packed).SerializeToString()


DTYPE_SIZE = {"f16": 2, "f32": 4, "f64": 8, "c64": 8}


def _list(xs):
    return "[" + ",".join(str(int(x)) for x in xs) + "]"


def describe(mg):
    """The text es_km_memgraph_describe gives for `mg`, written from the dicts."""
    lines = ["memgraph compute_locs=%d storage_locs=%d map=%s nodes=%d" % (
        mg["num_compute_locs"], mg["num_storage_locs"], _list(mg.get("storage_locs", [])),
        len(mg["nodes"]))]
    for i, n in enumerate(mg["nodes"]):
        k = n["kind"]
        loc = n.get("loc", 0)
        src_loc = n.get("src_loc", loc if k == "copy" else 0)
        offset, size = n.get("offset", 0), n.get("size", 0)
        mems = n.get("mems", [])
        if k == "apply" and mems:
            offset, size = mems[0]
        tail = ""
        if k == "constant":
            f = n["fill"]
            if "lower" in f:
                # the reader keeps the message's ncol as nrow and its nrow as ncol
                nrow, ncol = f["ncol"], f["nrow"]
                size = nrow * ncol * DTYPE_SIZE[f["lower"].split("|")[0]]
                tail = " lowertri{%s;%s;%d;%d;%d}" % (f["lower"], f["upper"], nrow, ncol,
                                                      f["start"])
            else:
                nelem = 1
                for d in f["shape"]:
                    nelem *= d
                size = nelem * DTYPE_SIZE[f["value"].split("|")[0]]
                tail = " constant{%s;%s}" % (f["value"], _list(f["shape"]))
        if "einsummable" in n:
            e = n["einsummable"]
            tail = " einsummable{%s;%s;%d;%s;%s}" % (
                _list(e["join_shape"]), "".join(_list(x) for x in e["inns"]), e["out_rank"],
                e["join"], e.get("castable") or "")
        if "touch" in n:
            t = n["touch"]
            tail = " touch{%s;%s;%s}" % (t["dtype"], t.get("castable") or "",
                                         "".join(_list(d) for d in t["selection"]))
        lines.append("%d kind=%d loc=%d src_loc=%d offset=%d size=%d src_offset=%d "
                     "storage=%d:%d group=%d inns=%s mems=[%s]%s" % (
                         i, KIND_NUMBER[k], loc, src_loc, offset, size, n.get("src_offset", 0),
                         n.get("storage_loc", 0), n.get("storage_id", 0), n.get("group", -1),
                         _list(n["inns"]),
                         ",".join("%d:%d" % (o, s) for o, s in mems), tail))
    return "\n".join(lines) + "\n"


def layer_node(n, deps, out, inns):
    """One node of einsummable_amd.llama_layer.LayerGraph (einsummable, touch or the mask's
    lowertri fill) as a memgraph node dict over the given ranges."""
    import numpy as np

    import einsummable_amd as ea

    if n["kind"] == "einsummable":
        e = n["e"]
        return node("apply", deps, loc=0, mems=[out] + inns, group=-1,
                    einsummable=dict(join_shape=e.join_shape, inns=e.inns, out_rank=e.out_rank,
                                     join=e.join, castable=e.castable or ""))
    if n["kind"] == "touch":
        t = n["t"]
        return node("apply", deps, loc=0, mems=[out] + inns, group=-1,
                    touch=dict(selection=t.selection, castable=t.castable or "",
                               dtype=["f16", "f32", "f64", "c64"][t.dtype]))
    assert n["dtype"] == ea.F16 and n["lower"] == 0.0 and n["upper"] == -np.inf
    # written as the reference's to_proto writes it; its reader exchanges the two (the mask
    # is square here, so the exchange does not show)
    assert n["nrow"] == n["ncol"]
    return node("constant", deps, loc=0, offset=out[0],
                fill=dict(lower="f16|0", upper="f16|NINF", nrow=n["nrow"], ncol=n["ncol"],
                          start=n["start"]))


def layer_memgraph_reusing(graph, align=256):
    """The decoder layer as the reference's memgraph compiler lays it out: an inputmem per
    layer input; every other buffer is allocated right before its first writer, deleted right
    behind its last user (the del depends on every user) and its range handed to later allocs
    (first fit), which depend on the dels that freed what they cover.  Apply nodes depend on
    the producers of what they read and on the alloc of what they write -- nothing is derived
    from the ranges.  Returns (memgraph dict, {input name: range}, output range, arena bytes)."""
    def names_in(n):
        if n["kind"] == "einsummable":
            return list(n["inns"])
        return [n["inn"]] if n["kind"] == "touch" else []

    written = {n["out"] for n in graph.nodes}
    last_use = {}
    for i, n in enumerate(graph.nodes):
        for b in names_in(n) + [n["out"]]:
            last_use[b] = i
    nodes, where, top = [], {}, 0
    users = {}        # buffer -> ids of the nodes that read or wrote it
    producer = {}     # buffer -> id of the inputmem / last writer
    input_ranges = {}
    for name, nbytes in graph.buffers.items():
        if name in written:
            continue
        where[name] = (top, nbytes)
        input_ranges[name] = where[name]
        producer[name] = len(nodes)
        nodes.append(node("inputmem", loc=0, offset=top, size=nbytes))
        top += (nbytes + align - 1) // align * align
    free = []         # (offset, size, id of the del that freed it)
    for i, n in enumerate(graph.nodes):
        out = n["out"]
        deps = set()
        if out not in where:
            nbytes = graph.buffers[out]
            need = (nbytes + align - 1) // align * align
            hit = next((f for f in free if f[1] >= need), None)
            if hit is None:
                off, freed_by = top, []
                top += need
            else:
                free.remove(hit)
                off, freed_by = hit[0], [hit[2]]
                if hit[1] > need:
                    free.append((hit[0] + need, hit[1] - need, hit[2]))
                    free.sort()
            where[out] = (off, nbytes)
            deps.add(len(nodes))
            nodes.append(node("alloc", freed_by, loc=0, offset=off, size=nbytes))
        else:
            deps.update(users.get(out, ()))
        ins = names_in(n)
        for b in ins:
            deps.add(producer[b])
        me = len(nodes)
        nodes.append(layer_node(n, deps, where[out], [where[b] for b in ins]))
        producer[out] = me
        for b in ins + [out]:
            users.setdefault(b, set()).add(me)
        for b in dict.fromkeys(ins + [out]):
            if last_use[b] == i and b in written and b != graph.output:
                off, nbytes = where[b]
                d = len(nodes)
                nodes.append(node("del", users[b], loc=0, offset=off, size=nbytes))
                free.append((off, (nbytes + align - 1) // align * align, d))
                free.sort()
    mg = dict(num_compute_locs=1, num_storage_locs=0, nodes=nodes)
    return mg, input_ranges, where[graph.output], top


def unordered_conflicts(g):
    """Pairs (i, j), i < j, of launching nodes of an einsummable_amd.ApplyGraph where j writes
    what i reads or writes, or reads what i writes, without depending on i (through any
    chain of dependencies)."""
    n = g.num_nodes()
    kinds, mems, deps = [], [], []
    for i in range(n):
        k, m = g.node_mems(i)
        kinds.append(k)
        mems.append(m)
        deps.append(g.node_info(i)[2])
    reach = []
    for i in range(n):
        r = set()
        for d in deps[i]:
            r.add(d)
            r |= reach[d]
        reach.append(r)

    def overlap(x, y):
        return x[1] and y[1] and x[0] < y[0] + y[1] and y[0] < x[0] + x[1]

    def split(i):
        if kinds[i] == "dummy":
            return [], []
        if kinds[i] == "evict":
            return [], mems[i]
        return mems[i][:1], mems[i][1:]

    bad = []
    for j in range(n):
        wj, rj = split(j)
        for i in range(j):
            wi, ri = split(i)
            clash = any(overlap(a, b) for a in wj for b in wi + ri) or \
                any(overlap(a, b) for a in rj for b in wi)
            if clash and i not in reach[j]:
                bad.append((i, j))
    return bad
