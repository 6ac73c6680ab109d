#include "memgraph_wire.h"

#include <algorithm>

namespace es
{
namespace
{

[[noreturn]] void bad(std::string const& what)
{
    throw ir_error("could not parse memgraph: " + what);
}

// Cursor over one protocol-buffers message.
struct reader_t {
    uint8_t const* p;
    uint8_t const* end;

    bool done() const { return p == end; }

    uint64_t varint()
    {
        uint64_t v = 0;
        for (int shift = 0; shift < 70; shift += 7) {
            if (p == end) bad("truncated varint");
            uint8_t const b = *p++;
            if (shift < 64) v |= uint64_t(b & 0x7f) << shift;
            if (!(b & 0x80)) return v;
        }
        bad("varint longer than ten bytes");
    }

    // reads a tag; field numbers are positive and below 2^29
    void tag(uint32_t& field, int& wire_type)
    {
        uint64_t const t = varint();
        field = uint32_t(t >> 3);
        wire_type = int(t & 7);
        if (field == 0 || (t >> 32) != 0) bad("bad field number");
    }

    reader_t sub()
    {
        uint64_t const n = varint();
        if (n > uint64_t(end - p)) bad("length past the end of the message");
        reader_t r{p, p + n};
        p += n;
        return r;
    }

    std::string str()
    {
        reader_t r = sub();
        return std::string(reinterpret_cast<char const*>(r.p), size_t(r.end - r.p));
    }

    void skip(int wire_type)
    {
        switch (wire_type) {
            case 0:
                (void)varint();
                break;
            case 1:
                if (end - p < 8) bad("truncated fixed64");
                p += 8;
                break;
            case 2:
                (void)sub();
                break;
            case 5:
                if (end - p < 4) bad("truncated fixed32");
                p += 4;
                break;
            default:
                bad("unsupported wire type " + std::to_string(wire_type));
        }
    }

    // a varint-typed singular field
    uint64_t scalar(int wire_type)
    {
        if (wire_type != 0) bad("expected a varint field");
        return varint();
    }

    // a varint-typed repeated field: one element, or a packed run of them
    template <typename T>
    void repeated(int wire_type, std::vector<T>& out)
    {
        if (wire_type == 0) {
            out.push_back(T(varint()));
        } else if (wire_type == 2) {
            reader_t r = sub();
            while (!r.done()) out.push_back(T(r.varint()));
        } else {
            bad("expected a repeated varint field");
        }
    }

    reader_t message(int wire_type)
    {
        if (wire_type != 2) bad("expected a length-delimited field");
        return sub();
    }
};

// int32 fields carry negative values sign-extended to 64 bits (ten bytes on the wire)
int as_int32(uint64_t v) { return int(int32_t(uint32_t(v))); }

// tracks which required fields of a message were seen
struct required_t {
    uint32_t    seen = 0;
    void        mark(uint32_t field) { if (field < 32) seen |= 1u << field; }
    void        need(std::initializer_list<uint32_t> fields, const char* message) const
    {
        for (uint32_t f : fields) {
            if (!(seen & (1u << f))) {
                bad(std::string(message) + " lacks required field " + std::to_string(f));
            }
        }
    }
};

// messages of the shape {int32 loc = 1; uint64 offset = 2; uint64 size = 3}
void read_loc_offset_size(reader_t r, mg_node_t& n, const char* message)
{
    required_t req;
    while (!r.done()) {
        uint32_t f;
        int      wt;
        r.tag(f, wt);
        req.mark(f);
        if (f == 1) n.loc = as_int32(r.scalar(wt));
        else if (f == 2) n.offset = r.scalar(wt);
        else if (f == 3) n.size = r.scalar(wt);
        else r.skip(wt);
    }
    req.need({1, 2, 3}, message);
}

mg_einsummable_t read_einsummable(reader_t r)
{
    mg_einsummable_t e;
    required_t       req;
    while (!r.done()) {
        uint32_t f;
        int      wt;
        r.tag(f, wt);
        req.mark(f);
        if (f == 1) {
            r.repeated(wt, e.join_shape);
        } else if (f == 2) {
            reader_t inn = r.message(wt);
            e.inns.emplace_back();
            while (!inn.done()) {
                uint32_t g;
                int      gwt;
                inn.tag(g, gwt);
                if (g == 1) {
                    std::vector<uint64_t> raw;
                    inn.repeated(gwt, raw);
                    for (uint64_t v : raw) e.inns.back().push_back(as_int32(v));
                } else {
                    inn.skip(gwt);
                }
            }
        } else if (f == 3) {
            e.out_rank = as_int32(r.scalar(wt));
        } else if (f == 4) {
            if (wt != 2) bad("Einsummable.join is a string");
            e.join = r.str();
        } else if (f == 5) {
            if (wt != 2) bad("Einsummable.castable is a string");
            e.castable = r.str();
        } else {
            r.skip(wt);
        }
    }
    req.need({3, 4}, "Einsummable");
    return e;
}

std::optional<castable_t> read_castable(std::string const& text)
{
    if (text.empty()) return std::nullopt;
    std::optional<castable_t> c = text.size() == 1 ? castable_from_char(text[0]) : std::nullopt;
    if (!c) bad("castable '" + text + "'");
    return c;
}

touch_t read_touch(reader_t r)
{
    touch_t     t;
    std::string castable, dtype;
    required_t  req;
    while (!r.done()) {
        uint32_t f;
        int      wt;
        r.tag(f, wt);
        req.mark(f);
        if (f == 1) {
            reader_t   d = r.message(wt);
            touchdim_t td{0, 0, 0, 0, 0};
            required_t dreq;
            while (!d.done()) {
                uint32_t g;
                int      gwt;
                d.tag(g, gwt);
                dreq.mark(g);
                if (g == 1) td.d_inn = d.scalar(gwt);
                else if (g == 2) td.d_out = d.scalar(gwt);
                else if (g == 3) td.offset_inn = d.scalar(gwt);
                else if (g == 4) td.offset_out = d.scalar(gwt);
                else if (g == 5) td.size = d.scalar(gwt);
                else d.skip(gwt);
            }
            dreq.need({1, 2, 3, 4, 5}, "TouchDim");
            t.selection.push_back(td);
        } else if (f == 2) {
            if (wt != 2) bad("Touch.castable is a string");
            castable = r.str();
        } else if (f == 3) {
            if (wt != 2) bad("Touch.dtype is a string");
            dtype = r.str();
        } else {
            r.skip(wt);
        }
    }
    req.need({3}, "Touch");
    t.castable = read_castable(castable);
    std::optional<dtype_t> d = dtype_from_name(dtype);
    if (!d) bad("dtype '" + dtype + "'");
    t.dtype = *d;
    return t;
}

mg_fill_t read_fill(reader_t r)
{
    mg_fill_t fill;
    bool      any = false;
    while (!r.done()) {
        uint32_t f;
        int      wt;
        r.tag(f, wt);
        if (f == 1) {
            reader_t   c = r.message(wt);
            required_t req;
            fill = mg_fill_t{};
            while (!c.done()) {
                uint32_t g;
                int      gwt;
                c.tag(g, gwt);
                req.mark(g);
                if (g == 1) {
                    if (gwt != 2) bad("Constant.value is a string");
                    fill.value = c.str();
                } else if (g == 2) {
                    c.repeated(gwt, fill.shape);
                } else {
                    c.skip(gwt);
                }
            }
            req.need({1}, "Constant");
            any = true;
        } else if (f == 2) {
            reader_t   c = r.message(wt);
            required_t req;
            fill = mg_fill_t{};
            fill.is_lowertri = true;
            while (!c.done()) {
                uint32_t g;
                int      gwt;
                c.tag(g, gwt);
                req.mark(g);
                if (g == 1) {
                    if (gwt != 2) bad("Lowertri.lower is a string");
                    fill.lower = c.str();
                } else if (g == 2) {
                    if (gwt != 2) bad("Lowertri.upper is a string");
                    fill.upper = c.str();
                } else if (g == 3) {
                    fill.nrow = c.scalar(gwt);  // the message's ncol: see mg_fill_t
                } else if (g == 4) {
                    fill.ncol = c.scalar(gwt);  // the message's nrow
                } else if (g == 5) {
                    fill.start = int64_t(c.scalar(gwt));
                } else {
                    c.skip(gwt);
                }
            }
            req.need({1, 2, 3, 4, 5}, "Lowertri");
            any = true;
        } else {
            r.skip(wt);
        }
    }
    if (!any) bad("Fill holds neither a constant nor a lowertri");
    return fill;
}

uint64_t fill_bytes(mg_fill_t const& f)
{
    if (f.is_lowertri) return f.nrow * f.ncol * dtype_size(parse_scalar(f.lower).dtype);
    uint64_t n = 1;
    for (uint64_t d : f.shape) n *= d;
    return n * dtype_size(parse_scalar(f.value).dtype);
}

void read_apply(reader_t r, mg_node_t& n)
{
    std::vector<uint64_t> offsets, sizes;
    required_t            req;
    while (!r.done()) {
        uint32_t f;
        int      wt;
        r.tag(f, wt);
        req.mark(f);
        if (f == 1) {
            n.loc = as_int32(r.scalar(wt));
        } else if (f == 2) {
            r.repeated(wt, offsets);
        } else if (f == 3) {
            r.repeated(wt, sizes);
        } else if (f == 4) {
            n.einsummable = read_einsummable(r.message(wt));
            n.touch.reset();  // members of a oneof: the last one on the wire stays
        } else if (f == 5) {
            n.touch = read_touch(r.message(wt));
            n.einsummable.reset();
        } else if (f == 6) {
            n.group = as_int32(r.scalar(wt));
        } else {
            r.skip(wt);
        }
    }
    req.need({1, 6}, "MGApply");
    if (offsets.size() != sizes.size()) bad("invalid apply_t: mems len must match");
    if (!n.einsummable && !n.touch) bad("apply op holds neither an einsummable nor a touch");
    for (size_t i = 0; i != offsets.size(); ++i) n.mems.push_back(mem_t{offsets[i], sizes[i]});
    if (!n.mems.empty()) {
        n.offset = n.mems[0].offset;
        n.size = n.mems[0].size;
    }
}

void read_storage_move(reader_t r, mg_node_t& n, const char* message)
{
    required_t req;
    while (!r.done()) {
        uint32_t f;
        int      wt;
        r.tag(f, wt);
        req.mark(f);
        if (f == 1) n.storage_loc = as_int32(r.scalar(wt));
        else if (f == 2) n.storage_id = as_int32(r.scalar(wt));
        else if (f == 3) n.loc = as_int32(r.scalar(wt));
        else if (f == 4) n.offset = r.scalar(wt);
        else if (f == 5) n.size = r.scalar(wt);
        else r.skip(wt);
    }
    req.need({1, 2, 3, 4, 5}, message);
}

mg_node_t read_node(reader_t r)
{
    mg_node_t n;
    bool      any = false;
    std::vector<uint64_t> inns;
    while (!r.done()) {
        uint32_t f;
        int      wt;
        r.tag(f, wt);
        if (f == 11) {
            r.repeated(wt, inns);
            continue;
        }
        bool const is_op = (f >= 1 && f <= 10) || f == 100;
        if (!is_op) {
            r.skip(wt);
            continue;
        }
        reader_t m = r.message(wt);
        n = mg_node_t{};
        n.kind = mg_kind(int(f));
        any = true;
        switch (n.kind) {
            case mg_kind::inputmem:
                read_loc_offset_size(m, n, "MGInputMem");
                break;
            case mg_kind::partialize:
                read_loc_offset_size(m, n, "MGPartialize");
                break;
            case mg_kind::alloc:
                read_loc_offset_size(m, n, "MGAlloc");
                break;
            case mg_kind::del:
                read_loc_offset_size(m, n, "MGDel");
                break;
            case mg_kind::inputsto: {
                required_t req;
                while (!m.done()) {
                    uint32_t g;
                    int      gwt;
                    m.tag(g, gwt);
                    req.mark(g);
                    if (g == 1) n.storage_loc = as_int32(m.scalar(gwt));
                    else if (g == 2) n.storage_id = as_int32(m.scalar(gwt));
                    else if (g == 3) n.size = m.scalar(gwt);
                    else m.skip(gwt);
                }
                req.need({1, 2, 3}, "MGInputSto");
                break;
            }
            case mg_kind::constant: {
                required_t req;
                while (!m.done()) {
                    uint32_t g;
                    int      gwt;
                    m.tag(g, gwt);
                    req.mark(g);
                    if (g == 1) n.loc = as_int32(m.scalar(gwt));
                    else if (g == 2) n.offset = m.scalar(gwt);
                    else if (g == 3) n.fill = read_fill(m.message(gwt));
                    else m.skip(gwt);
                }
                req.need({1, 2, 3}, "MGConstant");
                n.size = fill_bytes(n.fill);
                break;
            }
            case mg_kind::apply:
                read_apply(m, n);
                break;
            case mg_kind::move: {
                required_t req;
                while (!m.done()) {
                    uint32_t g;
                    int      gwt;
                    m.tag(g, gwt);
                    req.mark(g);
                    if (g == 1) n.src_loc = as_int32(m.scalar(gwt));
                    else if (g == 2) n.src_offset = m.scalar(gwt);
                    else if (g == 3) n.loc = as_int32(m.scalar(gwt));
                    else if (g == 4) n.offset = m.scalar(gwt);
                    else if (g == 5) n.size = m.scalar(gwt);
                    else m.skip(gwt);
                }
                req.need({1, 2, 3, 4, 5}, "MGMove");
                break;
            }
            case mg_kind::copy: {
                required_t req;
                while (!m.done()) {
                    uint32_t g;
                    int      gwt;
                    m.tag(g, gwt);
                    req.mark(g);
                    if (g == 1) n.loc = as_int32(m.scalar(gwt));
                    else if (g == 2) n.size = m.scalar(gwt);
                    else if (g == 3) n.src_offset = m.scalar(gwt);
                    else if (g == 4) n.offset = m.scalar(gwt);
                    else m.skip(gwt);
                }
                req.need({1, 2, 3, 4}, "MGCopy");
                n.src_loc = n.loc;
                break;
            }
            case mg_kind::evict:
                read_storage_move(m, n, "MGEvict");
                break;
            case mg_kind::load:
                read_storage_move(m, n, "MGLoad");
                break;
        }
    }
    if (!any) bad("proto node op contains something unexpected");
    // the reference collects these into a set (memgraph.cc:470-473)
    for (uint64_t v : inns) n.inns.push_back(as_int32(v));
    std::sort(n.inns.begin(), n.inns.end());
    n.inns.erase(std::unique(n.inns.begin(), n.inns.end()), n.inns.end());
    return n;
}

}  // namespace

memgraph_t decode_memgraph(void const* bytes, uint64_t size)
{
    if (!bytes && size) bad("null buffer");
    auto const* b = static_cast<uint8_t const*>(bytes);
    reader_t    r{b, b + size};
    memgraph_t  mg;
    required_t  req;
    while (!r.done()) {
        uint32_t f;
        int      wt;
        r.tag(f, wt);
        req.mark(f);
        if (f == 1) {
            mg.num_compute_locs = as_int32(r.scalar(wt));
        } else if (f == 2) {
            mg.num_storage_locs = as_int32(r.scalar(wt));
        } else if (f == 3) {
            std::vector<uint64_t> raw;
            r.repeated(wt, raw);
            for (uint64_t v : raw) mg.storage_locs.push_back(as_int32(v));
        } else if (f == 4) {
            mg_node_t n = read_node(r.message(wt));
            int const id = int(mg.nodes.size());
            for (int d : n.inns) {
                if (d < 0 || d >= id) {
                    bad("node " + std::to_string(id) + " waits for node " + std::to_string(d) +
                        ", which does not precede it");
                }
            }
            mg.nodes.push_back(std::move(n));
        } else {
            r.skip(wt);
        }
    }
    req.need({1, 2}, "MemGraph");
    return mg;
}

void memgraph_t::populate(apply_graph_t& g, int loc,
                          std::vector<std::pair<std::string, double>> const& vars) const
{
    if (g.n_nodes() != 0) throw ir_error("memgraph: the apply graph must be empty");
    // an inputsto has no location of its own: it is here if one of its readers is
    // (memgraph_t::is_local_to, memgraph.cc:793-809)
    auto here = [&](mg_node_t const& n) {
        if (n.kind == mg_kind::move) return n.loc == loc || n.src_loc == loc;
        return n.loc == loc;
    };
    std::vector<char> sto_here(nodes.size(), 0);
    for (size_t id = 0; id != nodes.size(); ++id) {
        if (nodes[id].kind == mg_kind::inputsto || !here(nodes[id])) continue;
        for (int d : nodes[id].inns) {
            if (nodes[size_t(d)].kind == mg_kind::inputsto) sto_here[size_t(d)] = 1;
        }
    }
    for (size_t id = 0; id != nodes.size(); ++id) {
        mg_node_t const& n = nodes[id];
        auto where = [&](std::string const& what) {
            return "memgraph node " + std::to_string(id) + ": " + what;
        };
        mem_t const range{n.offset, n.size};
        if (n.kind == mg_kind::inputsto) {
            if (sto_here[id]) g.declare_storage(n.storage_id, n.size);
            g.add_dummy(mem_t{0, 0}, n.inns);
            continue;
        }
        if (!here(n)) {
            g.add_dummy(mem_t{0, 0}, n.inns);
            continue;
        }
        switch (n.kind) {
            case mg_kind::inputmem:
            case mg_kind::partialize:
            case mg_kind::alloc:
                g.add_dummy(range, n.inns, false);
                break;
            case mg_kind::del:
                g.add_dummy(range, n.inns, true);
                break;
            case mg_kind::inputsto:
                break;
            case mg_kind::constant: {
                if (n.fill.is_lowertri) {
                    scalar_bits_t lo = parse_scalar(n.fill.lower);
                    scalar_bits_t up = parse_scalar(n.fill.upper);
                    if (lo.dtype != up.dtype) throw ir_error(where("lowertri of two dtypes"));
                    g.add_lowertri_fill(lo.dtype, lo.bits, up.bits, n.fill.nrow, n.fill.ncol,
                                        n.fill.start, range, n.inns);
                } else {
                    scalar_bits_t v = parse_scalar(n.fill.value);
                    g.add_constant_fill(v.dtype, v.bits, n.size / dtype_size(v.dtype), range,
                                        n.inns);
                }
                break;
            }
            case mg_kind::apply: {
                if (n.einsummable) {
                    if (n.group >= 0) {
                        throw ir_error(where("only allowing touches to have a group"));
                    }
                    mg_einsummable_t const& m = *n.einsummable;
                    // as einsummable_t::replace_scalar_variables does (einsummable.cc:220-233):
                    // the new join is a scalarop_t built from a node, i.e. simplified
                    scalarop_t join = scalarop_t::parse(m.join);
                    if (join.has_variables()) join = join.replace_variables(vars).simplify();
                    einsummable_t e = einsummable_t::make(m.join_shape, m.inns, m.out_rank, join,
                                                          read_castable(m.castable));
                    g.add_einsummable(e, n.mems, n.inns);
                } else {
                    g.add_touch(*n.touch, n.group, n.mems, n.inns);
                }
                break;
            }
            case mg_kind::move:
                if (n.loc != n.src_loc) {
                    throw ir_error(where("a move between locations " + std::to_string(n.src_loc) +
                                         " and " + std::to_string(n.loc) +
                                         " needs both devices; this graph runs on one"));
                }
                g.add_copy(range, mem_t{n.src_offset, n.size}, n.inns);
                break;
            case mg_kind::copy:
                g.add_copy(range, mem_t{n.src_offset, n.size}, n.inns);
                break;
            case mg_kind::evict:
                g.add_evict(range, n.storage_id, n.inns);
                break;
            case mg_kind::load:
                g.add_load(n.storage_id, range, n.inns);
                break;
        }
    }
}

}  // namespace es
