#include "ir.h"

#include <algorithm>
#include <cmath>
#include <complex>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <map>
#include <set>

namespace es
{

uint64_t dtype_size(dtype_t d)
{
    switch (d) {
        case dtype_t::f16:
            return 2;
        case dtype_t::f32:
            return 4;
        case dtype_t::f64:
        case dtype_t::c64:
            return 8;
    }
    throw ir_error("bad dtype");
}

const char* dtype_name(dtype_t d)
{
    switch (d) {
        case dtype_t::f16:
            return "f16";
        case dtype_t::f32:
            return "f32";
        case dtype_t::f64:
            return "f64";
        case dtype_t::c64:
            return "c64";
    }
    throw ir_error("bad dtype");
}

std::optional<castable_t> castable_from_char(char c)
{
    switch (c) {
        case 0:
        case ':':
            return std::nullopt;
        case '+':
            return castable_t::add;
        case 'x':
            return castable_t::mul;
        case 'v':
            return castable_t::min;
        case '^':
            return castable_t::max;
    }
    throw ir_error(std::string("bad castable character '") + c + "'");
}

char castable_to_char(std::optional<castable_t> const& c)
{
    if (!c) return ':';
    switch (c.value()) {
        case castable_t::add:
            return '+';
        case castable_t::mul:
            return 'x';
        case castable_t::min:
            return 'v';
        case castable_t::max:
            return '^';
    }
    return ':';
}

// ---------------------------------------------------------------- scalarop text

namespace
{

struct cursor_t {
    std::string const& s;
    size_t             p = 0;

    bool starts(const char* lit) const { return s.compare(p, std::strlen(lit), lit) == 0; }
    bool eat(const char* lit)
    {
        if (!starts(lit)) return false;
        p += std::strlen(lit);
        return true;
    }
    void need(const char* lit)
    {
        if (!eat(lit)) {
            throw ir_error("scalarop parse: expected '" + std::string(lit) + "' at offset " +
                           std::to_string(p) + " of '" + s + "'");
        }
    }
    double number(bool as_float)
    {
        const char* b = s.c_str() + p;
        char*       e = nullptr;
        double      v = as_float ? double(std::strtof(b, &e)) : std::strtod(b, &e);
        if (e == b) throw ir_error("scalarop parse: number expected at offset " + std::to_string(p));
        p += size_t(e - b);
        return v;
    }
};

dtype_t parse_dtype(cursor_t& c)
{
    if (c.eat("f16")) return dtype_t::f16;
    if (c.eat("f32")) return dtype_t::f32;
    if (c.eat("f64")) return dtype_t::f64;
    if (c.eat("c64")) return dtype_t::c64;
    throw ir_error("scalarop parse: dtype expected at offset " + std::to_string(c.p));
}

// Value of a decimal string once stored in `d`: the reference extracts f32 with the float
// stream operator, f64 as double and f16 as a double rounded to binary16
// (scalarop.cc:2808-2820, half.hpp:2708-2718).
double round_to_dtype(dtype_t d, double v)
{
    switch (d) {
        case dtype_t::f16:
            return double(_Float16(v));
        case dtype_t::f32:
            return double(float(v));
        default:
            return v;
    }
}

std::optional<dtype_t> result_type(node_t const& n)
{
    auto dt = [&](int i) { return n.children[i].dtype; };
    switch (n.kind) {
        case op_kind::add:
        case op_kind::mul:
            if (dt(0) != dt(1)) return std::nullopt;
            return dt(0);
        case op_kind::exp:
        case op_kind::log:
        case op_kind::power:
            if (dt(0) == dtype_t::c64) return std::nullopt;
            return dt(0);
        case op_kind::ite:
            if (dt(0) != dt(1) || dt(0) == dtype_t::c64 || dt(2) != dt(3)) return std::nullopt;
            return dt(2);
        case op_kind::convert:
            if (dt(0) == dtype_t::c64 || n.dtype == dtype_t::c64 || dt(0) == n.dtype) {
                return std::nullopt;
            }
            return n.dtype;
        case op_kind::conj:
            if (dt(0) != dtype_t::c64) return std::nullopt;
            return dtype_t::c64;
        case op_kind::real:
        case op_kind::imag:
            if (dt(0) != dtype_t::c64) return std::nullopt;
            return dtype_t::f32;
        case op_kind::cplex:
            if (dt(0) != dt(1) || dt(0) != dtype_t::f32) return std::nullopt;
            return dtype_t::c64;
        default:
            return n.dtype;
    }
}

int arity(op_kind k)
{
    switch (k) {
        case op_kind::constant:
        case op_kind::hole:
        case op_kind::variable:
            return 0;
        case op_kind::add:
        case op_kind::mul:
        case op_kind::cplex:
            return 2;
        case op_kind::ite:
            return 4;
        default:
            return 1;
    }
}

node_t parse_node(cursor_t& c, int depth)
{
    if (depth > 200) throw ir_error("scalarop parse: expression too deep");
    node_t n;
    n.dtype = dtype_t::f32;
    if (c.eat("constant{")) {
        n.kind = op_kind::constant;
        n.dtype = parse_dtype(c);
        c.need("|");
        if (n.dtype == dtype_t::c64) {
            c.need("(");
            n.re = c.number(true);
            c.need(",");
            n.im = c.number(true);
            c.need(")");
        } else if (c.eat("INF")) {
            n.re = INFINITY;
        } else if (c.eat("NINF")) {
            n.re = -INFINITY;
        } else if (c.eat("NAN")) {
            n.re = NAN;
        } else {
            n.re = round_to_dtype(n.dtype, c.number(n.dtype == dtype_t::f32));
        }
        c.need("}");
    } else if (c.eat("conj")) {
        n.kind = op_kind::conj;
    } else if (c.eat("complex")) {
        n.kind = op_kind::cplex;
    } else if (c.eat("variable{")) {
        n.kind = op_kind::variable;
        while (c.p < c.s.size() && (std::isalnum((unsigned char)c.s[c.p]) || c.s[c.p] == '_')) {
            n.name.push_back(c.s[c.p++]);
        }
        c.need("|");
        n.dtype = parse_dtype(c);
        c.need("}");
    } else if (c.eat("hole|")) {
        n.kind = op_kind::hole;
        n.dtype = parse_dtype(c);
        c.need("@");
        const char* b = c.s.c_str() + c.p;
        char*       e = nullptr;
        long        v = std::strtol(b, &e, 10);
        if (e == b || v < 0 || v > 63) throw ir_error("scalarop parse: bad hole index");
        c.p += size_t(e - b);
        n.arg = int(v);
    } else if (c.eat("+")) {
        n.kind = op_kind::add;
    } else if (c.eat("*")) {
        n.kind = op_kind::mul;
    } else if (c.eat("exp")) {
        n.kind = op_kind::exp;
    } else if (c.eat("log")) {
        n.kind = op_kind::log;
    } else if (c.eat("power{")) {
        n.kind = op_kind::power;
        n.power = c.number(false);
        c.need("}");
    } else if (c.eat("ite_")) {
        n.kind = op_kind::ite;
        if (c.eat("<=")) {
            n.compare = compare_t::le;
        } else if (c.eat(">=")) {
            n.compare = compare_t::ge;
        } else if (c.eat("==")) {
            n.compare = compare_t::eq;
        } else if (c.eat("<")) {
            n.compare = compare_t::lt;
        } else if (c.eat(">")) {
            n.compare = compare_t::gt;
        } else {
            throw ir_error("scalarop parse: bad comparison");
        }
    } else if (c.eat("imag")) {
        n.kind = op_kind::imag;
    } else if (c.eat("to_")) {
        n.kind = op_kind::convert;
        n.dtype = parse_dtype(c);
    } else if (c.eat("real")) {
        n.kind = op_kind::real;
    } else {
        throw ir_error("scalarop parse: unknown op at offset " + std::to_string(c.p) + " of '" +
                       c.s + "'");
    }

    int k = arity(n.kind);
    if (k == 0) return n;
    c.need("[");
    for (int i = 0; i != k; ++i) {
        if (i) c.need(",");
        n.children.push_back(parse_node(c, depth + 1));
    }
    c.need("]");
    auto t = result_type(n);
    if (!t) throw ir_error("scalarop parse: type failure in '" + c.s + "'");
    n.dtype = t.value();
    return n;
}

void format_number(std::string& out, double v)
{
    if (std::isinf(v)) {
        out += v > 0 ? "INF" : "NINF";
    } else if (std::isnan(v)) {
        out += "NAN";
    } else {
        char buf[64];
        std::snprintf(buf, sizeof(buf), "%g", v);  // default ostream formatting
        out += buf;
    }
}

void print_node(std::string& out, node_t const& n)
{
    static const char* cmp[] = {"<", ">", "==", "<=", ">="};
    char               buf[96];
    switch (n.kind) {
        case op_kind::constant:
            out += "constant{";
            out += dtype_name(n.dtype);
            out += "|";
            if (n.dtype == dtype_t::c64) {
                std::snprintf(buf, sizeof(buf), "(%g,%g)", n.re, n.im);
                out += buf;
            } else {
                format_number(out, n.re);
            }
            out += "}";
            break;
        case op_kind::hole:
            out += "hole|";
            out += dtype_name(n.dtype);
            out += "@" + std::to_string(n.arg);
            break;
        case op_kind::variable:
            out += "variable{" + n.name + "|" + dtype_name(n.dtype) + "}";
            break;
        case op_kind::add:
            out += "+";
            break;
        case op_kind::mul:
            out += "*";
            break;
        case op_kind::exp:
            out += "exp";
            break;
        case op_kind::log:
            out += "log";
            break;
        case op_kind::power:
            std::snprintf(buf, sizeof(buf), "power{%g}", n.power);
            out += buf;
            break;
        case op_kind::ite:
            out += "ite_";
            out += cmp[int(n.compare)];
            break;
        case op_kind::convert:
            out += "to_";
            out += dtype_name(n.dtype);
            break;
        case op_kind::conj:
            out += "conj";
            break;
        case op_kind::real:
            out += "real";
            break;
        case op_kind::imag:
            out += "imag";
            break;
        case op_kind::cplex:
            out += "complex";
            break;
    }
    if (!n.children.empty()) {
        out += "[";
        for (size_t i = 0; i != n.children.size(); ++i) {
            if (i) out += ",";
            print_node(out, n.children[i]);
        }
        out += "]";
    }
}

void gather_holes(node_t const& n, std::vector<std::optional<dtype_t>>& holes)
{
    if (n.kind == op_kind::hole) {
        if (int(holes.size()) <= n.arg) holes.resize(size_t(n.arg) + 1);
        if (holes[n.arg] && holes[n.arg].value() != n.dtype) {
            throw ir_error("scalarop: hole " + std::to_string(n.arg) + " used with two dtypes");
        }
        holes[n.arg] = n.dtype;
    }
    for (auto const& c : n.children) gather_holes(c, holes);
}

bool node_has_variable(node_t const& n)
{
    if (n.kind == op_kind::variable) return true;
    for (auto const& c : n.children) {
        if (node_has_variable(c)) return true;
    }
    return false;
}

bool is_hole(node_t const& n, int arg) { return n.kind == op_kind::hole && n.arg == arg; }

}  // namespace

scalarop_t scalarop_t::parse(std::string const& text)
{
    cursor_t   c{text};
    scalarop_t ret;
    ret.root = parse_node(c, 0);
    if (c.p != text.size()) {
        throw ir_error("scalarop parse: trailing text at offset " + std::to_string(c.p));
    }
    gather_holes(ret.root, ret.hole_dtypes);
    return ret;
}

std::string scalarop_t::str() const
{
    std::string out;
    print_node(out, root);
    return out;
}

bool scalarop_t::has_variables() const { return node_has_variable(root); }

namespace
{
void replace_in(node_t& n, std::vector<std::pair<std::string, double>> const& values)
{
    if (n.kind == op_kind::variable) {
        for (auto const& nv : values) {
            if (nv.first != n.name) continue;
            if (n.dtype == dtype_t::c64) throw ir_error("replace_variables: complex variable");
            n.kind = op_kind::constant;
            n.re = round_to_dtype(n.dtype, nv.second);
            n.im = 0.0;
            n.name.clear();
            break;
        }
    }
    for (node_t& c : n.children) replace_in(c, values);
}
}  // namespace

scalarop_t scalarop_t::replace_variables(
    std::vector<std::pair<std::string, double>> const& values) const
{
    scalarop_t ret = *this;
    replace_in(ret.root, values);
    return ret;
}

namespace
{
// node_t's operator== in the reference compares the printed texts (scalarop.cc:2648-2651): two
// constants that print alike are equal, and a NaN equals a NaN
bool same_node(node_t const& a, node_t const& b)
{
    std::string x, y;
    print_node(x, a);
    print_node(y, b);
    return x == y;
}

int max_hole(node_t const& n)
{
    if (n.kind == op_kind::hole) return n.arg;
    int r = -1;
    for (node_t const& c : n.children) r = std::max(r, max_hole(c));
    return r;
}

bool has_hole(node_t const& n) { return max_hole(n) >= 0; }

struct value_t {
    double re = 0.0, im = 0.0;  // held in the node's dtype (f16 / f32 values are exact in double)
};

// op_t::eval (scalarop.cc:554-780) on constants: every operation in its dtype
value_t eval_constant(node_t const& n)
{
    if (n.kind == op_kind::constant) return value_t{n.re, n.im};
    std::vector<value_t> x;
    for (node_t const& c : n.children) x.push_back(eval_constant(c));
    dtype_t const in = n.children.empty() ? n.dtype : n.children[0].dtype;
    auto          rnd = [&](dtype_t d, double v) { return round_to_dtype(d, v); };
    switch (n.kind) {
        case op_kind::add:
            if (in == dtype_t::c64) {
                return value_t{double(float(x[0].re) + float(x[1].re)),
                               double(float(x[0].im) + float(x[1].im))};
            }
            // the sum of two f16 or two f32 values is exact in double: one rounding
            return value_t{rnd(in, x[0].re + x[1].re), 0.0};
        case op_kind::mul:
            if (in == dtype_t::c64) {
                std::complex<float> const r = std::complex<float>(float(x[0].re), float(x[0].im)) *
                                              std::complex<float>(float(x[1].re), float(x[1].im));
                return value_t{double(r.real()), double(r.imag())};
            }
            if (in == dtype_t::f32) return value_t{double(float(x[0].re) * float(x[1].re)), 0.0};
            return value_t{rnd(in, x[0].re * x[1].re), 0.0};
        case op_kind::exp:
            if (in == dtype_t::f32) return value_t{double(std::exp(float(x[0].re))), 0.0};
            return value_t{rnd(in, std::exp(x[0].re)), 0.0};
        case op_kind::log:
            if (in == dtype_t::f32) return value_t{double(std::log(float(x[0].re))), 0.0};
            return value_t{rnd(in, std::log(x[0].re)), 0.0};
        case op_kind::power:
            if (in == dtype_t::f32) {
                return value_t{double(std::pow(float(x[0].re), float(n.power))), 0.0};
            }
            if (in == dtype_t::f16) {
                return value_t{rnd(in, std::pow(x[0].re, rnd(dtype_t::f16, n.power))), 0.0};
            }
            return value_t{std::pow(x[0].re, n.power), 0.0};
        case op_kind::ite: {
            bool c = false;
            switch (n.compare) {
                case compare_t::lt: c = x[0].re < x[1].re; break;
                case compare_t::gt: c = x[0].re > x[1].re; break;
                case compare_t::eq: c = x[0].re == x[1].re; break;
                case compare_t::le: c = x[0].re <= x[1].re; break;
                case compare_t::ge: c = x[0].re >= x[1].re; break;
            }
            return c ? x[2] : x[3];
        }
        case op_kind::convert:
            return value_t{rnd(n.dtype, x[0].re), 0.0};
        case op_kind::conj:
            return value_t{x[0].re, -x[0].im};
        case op_kind::real:
            return value_t{x[0].re, 0.0};
        case op_kind::imag:
            return value_t{x[0].im, 0.0};
        case op_kind::cplex:
            return value_t{x[0].re, x[1].re};
        default:
            throw ir_error("simplify: cannot evaluate a hole or a variable");
    }
}

// "constant{" + write_with_ss(value) + "}" read back (scalarop.cc:1258-1260): the value
// passes through six significant digits
node_t constant_through_text(dtype_t dt, value_t v)
{
    node_t c;
    c.kind = op_kind::constant;
    c.dtype = dt;
    c.re = v.re;
    c.im = v.im;
    std::string text;
    print_node(text, c);
    cursor_t cur{text};
    return parse_node(cur, 0);
}

node_t make_const(dtype_t dt, double re, double im = 0.0)
{
    node_t c;
    c.kind = op_kind::constant;
    c.dtype = dt;
    c.re = re;
    c.im = im;
    return c;
}

bool is_const(node_t const& n, double re, double im = 0.0)
{
    return n.kind == op_kind::constant && n.re == re && n.im == im;
}

compare_t compare_flip(compare_t c)
{
    switch (c) {
        case compare_t::lt: return compare_t::ge;
        case compare_t::gt: return compare_t::le;
        case compare_t::eq: return compare_t::eq;
        case compare_t::le: return compare_t::gt;
        default: return compare_t::lt;
    }
}

node_t simplify_node(node_t const& n);

node_t simplify_once(node_t const& n)
{
    if (n.kind == op_kind::hole || n.kind == op_kind::constant || n.kind == op_kind::variable) {
        return n;
    }
    if (!has_hole(n) && !node_has_variable(n)) {
        return constant_through_text(n.dtype, eval_constant(n));
    }
    node_t self = n;
    for (node_t& c : self.children) c = simplify_node(c);
    std::vector<node_t>& ch = self.children;

    // normalize_order: the operand with the smaller highest hole comes first (a constant has
    // none: -1); equal highest holes are left as they stand
    auto unordered = [](node_t const& l, node_t const& r) { return max_hole(r) < max_hole(l); };
    if (n.kind == op_kind::add || n.kind == op_kind::mul) {
        if (unordered(ch[0], ch[1])) {
            std::swap(ch[0], ch[1]);
            return self;
        }
    } else if (n.kind == op_kind::ite) {
        bool const fix_co = unordered(ch[0], ch[1]);
        bool const fix_tt = unordered(ch[2], ch[3]);
        if (fix_co) {
            self.compare = compare_flip(self.compare);
            std::swap(ch[0], ch[1]);
        }
        if (fix_tt) std::swap(ch[2], ch[3]);
        if (fix_co || fix_tt) return self;
    }

    dtype_t const dt = n.dtype;
    bool const    cx = dt == dtype_t::c64;
    if (n.kind == op_kind::add) {
        if (is_const(ch[0], 0.0)) return ch[1];
        if (is_const(ch[1], 0.0)) return ch[0];
        if (!cx) {
            for (int i = 0; i != 2; ++i) {
                if (ch[i].kind == op_kind::constant && std::isinf(ch[i].re)) return ch[i];
            }
        }
    }
    if (n.kind == op_kind::mul) {
        if (is_const(ch[0], 0.0) || is_const(ch[1], 0.0)) return make_const(dt, 0.0);
        auto fold_pair = [&]() -> std::optional<node_t> {
            // c0 * (c1 * hole)
            if (ch[0].kind == op_kind::constant && ch[1].kind == op_kind::mul &&
                ch[1].children[0].kind == op_kind::constant &&
                ch[1].children[1].kind == op_kind::hole) {
                node_t prod;
                prod.kind = op_kind::mul;
                prod.dtype = ch[0].dtype;
                prod.children = {ch[0], ch[1].children[0]};
                value_t const v = eval_constant(prod);
                node_t        r;
                r.kind = op_kind::mul;
                r.dtype = ch[0].dtype;
                r.children = {make_const(ch[0].dtype, v.re, v.im), ch[1].children[1]};
                return r;
            }
            return std::nullopt;
        };
        if (auto r = fold_pair()) return r.value();
        if (is_const(ch[0], 1.0)) return ch[1];
        if (is_const(ch[1], 1.0)) return ch[0];
    }
    if (n.kind == op_kind::power) {
        if (n.power == 0.0) return make_const(dt, 1.0);
        if (n.power == 1.0) return ch[0];
    }
    if (n.kind == op_kind::ite) {
        if (same_node(ch[0], ch[1]) && self.compare == compare_t::eq) return ch[2];
        if (same_node(ch[2], ch[3])) return ch[2];
    }
    if (n.kind == op_kind::conj && ch[0].kind == op_kind::conj) return ch[0].children[0];
    return self;
}

node_t simplify_node(node_t const& n)
{
    node_t r0 = simplify_once(n);
    if (same_node(r0, n)) return r0;
    for (int guard = 0; guard != 1000; ++guard) {
        node_t r1 = simplify_once(r0);
        if (same_node(r0, r1)) return r1;
        r0 = std::move(r1);
    }
    throw ir_error("simplify: no fixed point");
}
}  // namespace

scalarop_t scalarop_t::simplify() const
{
    scalarop_t ret;
    ret.root = simplify_node(root);
    // a hole that folded away keeps its dtype: the einsummable still has that input
    ret.hole_dtypes = hole_dtypes;
    return ret;
}

namespace
{
void compose_in(node_t& n, int k, int n_inner, node_t const& inner)
{
    if (n.kind == op_kind::hole) {
        if (n.arg == k) {
            node_t c;
            c.kind = op_kind::convert;
            c.dtype = inner.dtype;
            c.children.push_back(inner);
            n = std::move(c);
        } else {
            n.arg = n_inner + (n.arg < k ? n.arg : n.arg - 1);
        }
        return;
    }
    for (node_t& c : n.children) compose_in(c, k, n_inner, inner);
}
}  // namespace

scalarop_t scalarop_t::compose(scalarop_t const& outer, int k, scalarop_t const& inner)
{
    if (k < 0 || k >= outer.num_inputs() || !outer.hole_dtypes[size_t(k)]) {
        throw ir_error("compose: the outer expression has no hole " + std::to_string(k));
    }
    if (outer.hole_dtypes[size_t(k)].value() != inner.out_dtype()) {
        throw ir_error("compose: hole and inner expression differ in dtype");
    }
    scalarop_t ret;
    ret.root = outer.root;
    compose_in(ret.root, k, inner.num_inputs(), inner.root);
    ret.hole_dtypes = inner.hole_dtypes;
    for (int i = 0; i != outer.num_inputs(); ++i) {
        if (i != k) ret.hole_dtypes.push_back(outer.hole_dtypes[size_t(i)]);
    }
    return ret;
}

scalar_bits_t parse_scalar(std::string const& text)
{
    scalarop_t op = scalarop_t::parse("constant{" + text + "}");
    node_t const& n = op.root;
    scalar_bits_t ret{n.dtype, 0};
    switch (n.dtype) {
        case dtype_t::f16: {
            _Float16 v = _Float16(n.re);
            uint16_t b;
            std::memcpy(&b, &v, 2);
            ret.bits = b;
            break;
        }
        case dtype_t::f32: {
            float    v = float(n.re);
            uint32_t b;
            std::memcpy(&b, &v, 4);
            ret.bits = b;
            break;
        }
        case dtype_t::f64:
            std::memcpy(&ret.bits, &n.re, 8);
            break;
        case dtype_t::c64: {
            float    v[2] = {float(n.re), float(n.im)};
            std::memcpy(&ret.bits, v, 8);
            break;
        }
    }
    return ret;
}

std::optional<dtype_t> dtype_from_name(std::string const& name)
{
    for (dtype_t d : {dtype_t::f16, dtype_t::f32, dtype_t::f64, dtype_t::c64}) {
        if (name == dtype_name(d)) return d;
    }
    return std::nullopt;
}

bool scalarop_t::is_identity() const { return is_hole(root, 0); }

bool scalarop_t::is_mul() const
{
    return root.kind == op_kind::mul && is_hole(root.children[0], 0) &&
           is_hole(root.children[1], 1);
}

bool scalarop_t::is_scaled_mul(double& scale) const
{
    auto product = [](node_t const& n) {
        return n.kind == op_kind::mul &&
               ((is_hole(n.children[0], 0) && is_hole(n.children[1], 1)) ||
                (is_hole(n.children[0], 1) && is_hole(n.children[1], 0)));
    };
    scale = 1.0;
    if (product(root)) return true;
    if (root.kind != op_kind::mul) return false;
    for (int c = 0; c != 2; ++c) {
        node_t const& k = root.children[c];
        if (k.kind == op_kind::constant && k.dtype != dtype_t::c64 && product(root.children[1 - c])) {
            scale = k.re;
            return true;
        }
    }
    return false;
}

bool scalarop_t::is_add() const
{
    return root.kind == op_kind::add && is_hole(root.children[0], 0) &&
           is_hole(root.children[1], 1);
}

// ------------------------------------------------------------------ einsummable

einsummable_t einsummable_t::make(std::vector<uint64_t> join_shape,
                                  std::vector<std::vector<int>> inns, int out_rank,
                                  scalarop_t join, std::optional<castable_t> castable)
{
    if (out_rank < 1) throw ir_error("einsummable: invalid inns, out rank");
    if (inns.empty()) throw ir_error("einsummable: no inputs");
    if (out_rank < int(join_shape.size()) && !castable) {
        throw ir_error("Must have castable when aggregating.");
    }
    if (join.num_inputs() != int(inns.size())) {
        throw ir_error("einsummable inns size not same as scalarop join");
    }
    for (auto const& h : join.hole_dtypes) {
        if (!h) throw ir_error("einsummable does not use all of its inputs!");
    }
    // aggregated modes are numbered in order of first appearance
    {
        int                next = out_rank;
        std::map<int, int> renamed;
        for (auto& inn : inns) {
            if (inn.empty()) throw ir_error("compute_join_rank: empty inn given");
            for (int& m : inn) {
                if (m < 0) throw ir_error("einsummable: negative mode");
                if (m >= out_rank) {
                    auto it = renamed.find(m);
                    if (it == renamed.end()) it = renamed.emplace(m, next++).first;
                    m = it->second;
                }
            }
        }
    }
    int top = 0;
    for (auto const& inn : inns) top = std::max(top, *std::max_element(inn.begin(), inn.end()));
    int join_rank = std::max(top + 1, out_rank);
    if (join_rank != int(join_shape.size())) throw ir_error("invalid join shape size");
    // every element count and byte size derived from the shape must fit 64 bits
    uint64_t total = 1;
    for (uint64_t d : join_shape) {
        if (d == 0) throw ir_error("einsummable: cannot have zero join size");
        if (d >= (1ull << 58) / total) throw ir_error("einsummable: join shape too large");
        total *= d;
    }
    for (auto const& inn : inns) {
        std::set<int> uniq(inn.begin(), inn.end());
        if (uniq.size() != inn.size()) throw ir_error("einsummable: invalid inns, out rank");
    }
    einsummable_t e;
    e.join_shape = std::move(join_shape);
    e.inns = std::move(inns);
    e.out_rank = out_rank;
    e.join = std::move(join);
    e.castable = castable;
    return e;
}

einsummable_t einsummable_t::merge_adjacent_dims() const
{
    int const R = int(join_shape.size());
    // terms: every input and the output
    std::vector<std::vector<int>> terms = inns;
    {
        std::vector<int> o(out_rank);
        for (int i = 0; i != out_rank; ++i) o[i] = i;
        terms.push_back(o);
    }
    // mode m+1 can be glued to mode m when every term either holds neither of them or
    // holds them next to each other in that order
    auto glued = [&](int m) {
        for (auto const& t : terms) {
            auto a = std::find(t.begin(), t.end(), m);
            auto b = std::find(t.begin(), t.end(), m + 1);
            bool has_a = a != t.end(), has_b = b != t.end();
            if (has_a != has_b) return false;
            if (has_a && (a + 1) != b) return false;
        }
        return true;
    };
    std::vector<int> group_of(R);
    int              n_groups = 0;
    for (int m = 0; m != R; ++m) {
        if (m > 0 && glued(m - 1)) {
            group_of[m] = n_groups - 1;
        } else {
            group_of[m] = n_groups++;
        }
    }
    if (n_groups == R) return *this;

    std::vector<uint64_t> shape(n_groups, 1);
    for (int m = 0; m != R; ++m) shape[group_of[m]] *= join_shape[m];
    auto squash = [&](std::vector<int> const& t) {
        std::vector<int> r;
        for (int m : t) {
            int g = group_of[m];
            if (r.empty() || r.back() != g) r.push_back(g);
        }
        return r;
    };
    std::vector<std::vector<int>> new_inns;
    for (auto const& inn : inns) new_inns.push_back(squash(inn));
    int new_out_rank = int(squash(terms.back()).size());
    einsummable_t r = make(shape, new_inns, new_out_rank, join, castable);
    r.half_complex = half_complex;
    return r;
}

std::string einsummable_t::str() const
{
    std::string s;
    for (size_t k = 0; k != inns.size(); ++k) {
        if (k) s += ",";
        for (int m : inns[k]) s.push_back(char('a' + m));
    }
    s += "->";
    for (int i = 0; i != out_rank; ++i) s.push_back(char('a' + i));
    return s;
}

std::string einsummable_t::key() const
{
    std::string s = "[";
    for (size_t i = 0; i != join_shape.size(); ++i) {
        if (i) s += ",";
        s += std::to_string(join_shape[i]);
    }
    s += "]";
    s.push_back(castable_to_char(castable));
    s += " ";
    for (size_t k = 0; k != inns.size(); ++k) {
        if (k) s += ",";
        for (int m : inns[k]) s += std::to_string(m) + ".";
    }
    s += "->" + std::to_string(out_rank) + " | " + join.str();
    if (any_half_pairs()) {
        s += " | f16 pairs:";
        for (size_t i = 0; i != half_complex.size(); ++i) {
            if (half_complex[i]) s += i ? " in" + std::to_string(i - 1) : " out";
        }
    }
    return s;
}

bool einsummable_t::has_broadcast() const
{
    std::set<int> seen;
    for (auto const& inn : inns) {
        for (int m : inn) {
            if (m < out_rank) seen.insert(m);
        }
    }
    return int(seen.size()) != out_rank;
}

bool einsummable_t::is_straight_elementwise() const
{
    if (has_aggregation()) return false;
    for (auto const& inn : inns) {
        if (inn.size() != join_shape.size()) return false;
        for (size_t i = 0; i != inn.size(); ++i) {
            if (inn[i] != int(i)) return false;
        }
    }
    return true;
}

bool einsummable_t::is_permutation() const
{
    return inns.size() == 1 && !has_aggregation() && !has_broadcast() && join.is_identity();
}

bool einsummable_t::is_contraction() const
{
    return inns.size() == 2 && has_aggregation() && !has_broadcast() && castable &&
           castable.value() == castable_t::add && join.is_mul();
}

bool einsummable_t::is_scaled_contraction(double& scale) const
{
    return inns.size() == 2 && has_aggregation() && !has_broadcast() && castable &&
           castable.value() == castable_t::add && join.is_scaled_mul(scale);
}

uint64_t einsummable_t::out_nelem() const
{
    uint64_t n = 1;
    for (int i = 0; i != out_rank; ++i) n *= join_shape[i];
    return n;
}

uint64_t einsummable_t::inn_nelem(int k) const
{
    uint64_t n = 1;
    for (int m : inns[k]) n *= join_shape[m];
    return n;
}

// ------------------------------------------------------------------------ touch

touch_t touch_t::simplify() const
{
    touch_t r;
    r.castable = castable;
    r.dtype = dtype;
    for (auto const& d : selection) {
        bool whole = d.d_inn == d.d_out && d.offset_inn == 0 && d.offset_out == 0 &&
                     d.d_inn == d.size;
        if (!r.selection.empty() && whole) {
            auto& b = r.selection.back();
            b.d_inn *= d.d_inn;
            b.d_out *= d.d_inn;
            b.offset_inn *= d.d_inn;
            b.offset_out *= d.d_inn;
            b.size *= d.d_inn;
        } else {
            r.selection.push_back(d);
        }
    }
    return r;
}

void touch_t::validate() const
{
    if (selection.empty()) throw ir_error("touch: empty selection");
    for (auto const& d : selection) {
        if (d.size == 0) throw ir_error("touch: zero-sized dimension");
        if (d.offset_inn + d.size > d.d_inn || d.offset_out + d.size > d.d_out) {
            throw ir_error("touch: window leaves its tensor");
        }
    }
    if (dtype == dtype_t::c64 && castable &&
        (castable.value() == castable_t::min || castable.value() == castable_t::max)) {
        throw ir_error("touch: min/max of complex values");
    }
}

}  // namespace es
