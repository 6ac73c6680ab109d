#include "codegen.h"

#include "kernel_manager.h"

#include <hip/hip_runtime.h>
#include <hip/hiprtc.h>

#include <algorithm>
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <future>
#include <set>
#include <map>
#include <mutex>
#include <sstream>

#include <sys/stat.h>
#include <unistd.h>

namespace es
{

namespace
{

// ---------------------------------------------------------------- expression emission

// Arithmetic type a node is evaluated in: f16 and f32 nodes in float (f16 results are rounded
// once, when stored or at an explicit to_f16), f64 in double, c64 as a pair of floats.
const char* compute_type(dtype_t d)
{
    switch (d) {
        case dtype_t::f16:
        case dtype_t::f32:
            return "float";
        case dtype_t::f64:
            return "double";
        case dtype_t::c64:
            return "c64";
    }
    return "float";
}

const char* storage_type(dtype_t d)
{
    switch (d) {
        case dtype_t::f16:
            return "f16";
        case dtype_t::f32:
            return "float";
        case dtype_t::f64:
            return "double";
        case dtype_t::c64:
            return "c64";
    }
    return "float";
}

bool is_double(dtype_t d) { return d == dtype_t::f64; }

std::string literal(dtype_t d, double v)
{
    char buf[96];
    bool dbl = is_double(d);
    if (std::isnan(v)) return dbl ? "__builtin_nan(\"\")" : "__builtin_nanf(\"\")";
    if (std::isinf(v)) {
        std::string s = dbl ? "__builtin_huge_val()" : "__builtin_huge_valf()";
        return v < 0 ? "(-" + s + ")" : s;
    }
    std::snprintf(buf, sizeof(buf), dbl ? "(%a)" : "(%af)", v);
    return buf;
}

struct emitter_t {
    std::ostringstream body;
    int                next = 0;

    std::string fresh() { return "t" + std::to_string(next++); }

    std::string define(dtype_t d, std::string const& rhs)
    {
        std::string v = fresh();
        body << "    const " << compute_type(d) << " " << v << " = " << rhs << ";\n";
        return v;
    }

    std::string emit(node_t const& n)
    {
        std::vector<std::string> c;
        for (auto const& ch : n.children) c.push_back(emit(ch));
        bool const dbl = is_double(n.dtype);
        switch (n.kind) {
            case op_kind::constant:
                if (n.dtype == dtype_t::c64) {
                    return define(n.dtype, "c64{" + literal(dtype_t::f32, n.re) + ", " +
                                               literal(dtype_t::f32, n.im) + "}");
                }
                return define(n.dtype, literal(n.dtype, n.re));
            case op_kind::hole:
                return "x" + std::to_string(n.arg);
            case op_kind::variable:
                throw ir_error("scalarop with variables cannot be compiled");
            case op_kind::add:
                if (n.dtype == dtype_t::c64) return define(n.dtype, "c_add(" + c[0] + ", " + c[1] + ")");
                return define(n.dtype, c[0] + " + " + c[1]);
            case op_kind::mul:
                if (n.dtype == dtype_t::c64) return define(n.dtype, "c_mul(" + c[0] + ", " + c[1] + ")");
                return define(n.dtype, c[0] + " * " + c[1]);
            case op_kind::exp:
                // f16 / f32: v_exp_f32 on x * log2(e); relative error ~ (2 + |x|) * 2^-24, well
                // inside the 1e-4 contract on the whole finite range of expf
                return define(n.dtype, std::string(dbl ? "exp(" : "__expf(") + c[0] + ")");
            case op_kind::log:
                return define(n.dtype, std::string(dbl ? "log(" : "logf(") + c[0] + ")");
            case op_kind::power: {
                // The exponent is used at the precision the reference gives it
                // (scalarop.cc:711-726): rounded to f16 / f32 for those dtypes.
                double p = n.power;
                if (n.dtype == dtype_t::f16) p = double(_Float16(p));
                if (n.dtype == dtype_t::f32) p = double(float(p));
                std::string const& x = c[0];
                std::string one = dbl ? "1.0" : "1.0f";
                if (p == 1.0) return define(n.dtype, x);
                if (p == 2.0) return define(n.dtype, x + " * " + x);
                if (p == 3.0) return define(n.dtype, x + " * " + x + " * " + x);
                if (p == -1.0) return define(n.dtype, one + " / " + x);
                if (p == -2.0) return define(n.dtype, one + " / (" + x + " * " + x + ")");
                if (p == 0.5) return define(n.dtype, std::string(dbl ? "sqrt(" : "sqrtf(") + x + ")");
                if (p == -0.5) {
                    return define(n.dtype, one + " / " + (dbl ? "sqrt(" : "sqrtf(") + x + ")");
                }
                return define(n.dtype, std::string(dbl ? "pow(" : "powf(") + x + ", " +
                                           literal(n.dtype, p) + ")");
            }
            case op_kind::ite: {
                static const char* cmp[] = {"<", ">", "==", "<=", ">="};
                return define(n.dtype, "(" + c[0] + " " + cmp[int(n.compare)] + " " + c[1] +
                                           ") ? " + c[2] + " : " + c[3]);
            }
            case op_kind::convert: {
                dtype_t from = n.children[0].dtype;
                // A conversion to the dtype the value already has stands where two
                // expressions were joined into one (scalarop_t::compose): the value is what a
                // kernel would have stored and the next one loaded.  For f16 that is the
                // rounding below; for the others the value is unchanged, but the compiler
                // must not contract a product on one side with a sum on the other into one
                // fused multiply-add, which rounds differently.
                if (from == n.dtype && n.dtype != dtype_t::f16) {
                    return define(n.dtype, "keep_apart(" + c[0] + ")");
                }
                if (n.dtype == dtype_t::f16) return define(n.dtype, "(float)(f16)(" + c[0] + ")");
                if (n.dtype == dtype_t::f32) {
                    return define(n.dtype, from == dtype_t::f64 ? "(float)(" + c[0] + ")" : c[0]);
                }
                return define(n.dtype, "(double)(" + c[0] + ")");
            }
            case op_kind::conj:
                return define(n.dtype, "c64{" + c[0] + ".re, -" + c[0] + ".im}");
            case op_kind::real:
                return define(n.dtype, c[0] + ".re");
            case op_kind::imag:
                return define(n.dtype, c[0] + ".im");
            case op_kind::cplex:
                return define(n.dtype, "c64{" + c[0] + ", " + c[1] + "}");
        }
        throw ir_error("emit: bad node");
    }
};

const char* PRELUDE = R"(
typedef _Float16 f16;
struct c64 { float re, im; };
__device__ __forceinline__ c64 c_add(c64 a, c64 b) { return c64{a.re + b.re, a.im + b.im}; }
__device__ __forceinline__ c64 c_mul(c64 a, c64 b)
{
    return c64{a.re * b.re - a.im * b.im, a.re * b.im + a.im * b.re};
}
__device__ __forceinline__ float keep_apart(float v)
{
    asm("" : "+v"(v));
    return v;
}
__device__ __forceinline__ double keep_apart(double v)
{
    asm("" : "+v"(v));
    return v;
}
__device__ __forceinline__ c64 keep_apart(c64 v) { return c64{keep_apart(v.re), keep_apart(v.im)}; }
// (at most 16 bytes of alignment: a wider vector moves as 16-byte pieces)
template <typename T, int N>
struct __attribute__((aligned(sizeof(T) * N < 16 ? sizeof(T) * N : 16))) vec_t { T v[N]; };
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
struct u32x8 { u32x4 lo, hi; };
// vector load / store; NT != 0 marks the access non-temporal (streamed once, no reuse)
template <int NT, typename VT>
__device__ __forceinline__ VT ldv(const VT* p)
{
    if constexpr (NT && sizeof(VT) == 16) {
        return __builtin_bit_cast(VT, __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(p)));
    } else if constexpr (NT && sizeof(VT) == 32) {
        const u32x4* q = reinterpret_cast<const u32x4*>(p);
        return __builtin_bit_cast(VT, u32x8{__builtin_nontemporal_load(q),
                                            __builtin_nontemporal_load(q + 1)});
    } else {
        return *p;
    }
}
template <int NT, typename VT>
__device__ __forceinline__ void stv(VT* p, VT v)
{
    if constexpr (NT && sizeof(VT) == 16) {
        __builtin_nontemporal_store(__builtin_bit_cast(u32x4, v), reinterpret_cast<u32x4*>(p));
    } else if constexpr (NT && sizeof(VT) == 32) {
        u32x8 w = __builtin_bit_cast(u32x8, v);
        __builtin_nontemporal_store(w.lo, reinterpret_cast<u32x4*>(p));
        __builtin_nontemporal_store(w.hi, reinterpret_cast<u32x4*>(p) + 1);
    } else {
        *p = v;
    }
}
__device__ __forceinline__ float  cvt_in(f16 v) { return (float)v; }
__device__ __forceinline__ float  cvt_in(float v) { return v; }
__device__ __forceinline__ double cvt_in(double v) { return v; }
__device__ __forceinline__ c64    cvt_in(c64 v) { return v; }
// a complex number kept as two f16
struct h2 { f16 re, im; };
__device__ __forceinline__ c64 cvt_in(h2 v) { return c64{(float)v.re, (float)v.im}; }
__device__ __forceinline__ h2  narrow_c64(c64 v) { return h2{(f16)v.re, (f16)v.im}; }
__device__ __forceinline__ float  lane_xor(float v, int m) { return __shfl_xor(v, m); }
__device__ __forceinline__ double lane_xor(double v, int m) { return __shfl_xor(v, m); }
__device__ __forceinline__ c64    lane_xor(c64 v, int m)
{
    return c64{__shfl_xor(v.re, m), __shfl_xor(v.im, m)};
}
)";

// how one input sees the vectorised mode
enum class access_t { straight, vec, bcast, gather };

struct layout_t {
    int                                R = 0;  // join rank
    int                                O = 0;  // out rank
    int                                NI = 0;
    std::vector<uint64_t>              shape;
    std::vector<std::vector<uint64_t>> stride;  // [input][join mode], 0 when absent
};

layout_t make_layout(einsummable_t const& e)
{
    layout_t L;
    L.R = int(e.join_shape.size());
    L.O = e.out_rank;
    L.NI = int(e.inns.size());
    L.shape = e.join_shape;
    L.stride.assign(size_t(L.NI), std::vector<uint64_t>(size_t(L.R), 0));
    for (int k = 0; k != L.NI; ++k) {
        uint64_t s = 1;
        for (int i = int(e.inns[k].size()) - 1; i >= 0; --i) {
            L.stride[k][e.inns[k][i]] = s;
            s *= e.join_shape[e.inns[k][i]];
        }
    }
    return L;
}

access_t classify(einsummable_t const& e, int k, int vmode, bool allow_straight)
{
    auto const& inn = e.inns[k];
    if (allow_straight && int(inn.size()) == e.out_rank) {
        bool straight = true;
        for (size_t i = 0; i != inn.size(); ++i) straight = straight && inn[i] == int(i);
        if (straight) return access_t::straight;
    }
    auto it = std::find(inn.begin(), inn.end(), vmode);
    if (it == inn.end()) return access_t::bcast;
    if (it + 1 == inn.end()) return access_t::vec;
    return access_t::gather;
}

int pow2_divisor(uint64_t n, int cap)
{
    int v = 1;
    while (v * 2 <= cap && n % uint64_t(v * 2) == 0) v *= 2;
    return v;
}

std::string identity_of(castable_t c, dtype_t d)
{
    bool dbl = is_double(d);
    if (d == dtype_t::c64) return c == castable_t::add ? "c64{0.0f, 0.0f}" : "c64{1.0f, 0.0f}";
    switch (c) {
        case castable_t::add:
            return dbl ? "0.0" : "0.0f";
        case castable_t::mul:
            return dbl ? "1.0" : "1.0f";
        case castable_t::min:
            return dbl ? "__builtin_huge_val()" : "__builtin_huge_valf()";
        case castable_t::max:
            return dbl ? "(-__builtin_huge_val())" : "(-__builtin_huge_valf())";
    }
    return "0";
}

// acc <- castable(acc, v); min/max follow make_min / make_max (scalarop.cc:2267-2280)
std::string combine_expr(castable_t c, dtype_t d, std::string const& a, std::string const& v)
{
    if (d == dtype_t::c64) {
        return c == castable_t::add ? "c_add(" + a + ", " + v + ")" : "c_mul(" + a + ", " + v + ")";
    }
    switch (c) {
        case castable_t::add:
            return a + " + " + v;
        case castable_t::mul:
            return a + " * " + v;
        // one v_min / v_max instead of compare + select; identical to make_min / make_max
        // (scalarop.cc:2267-2280) for every pair of non-NaN values up to the sign of a zero
        case castable_t::min:
            return std::string(is_double(d) ? "__builtin_fmin(" : "__builtin_fminf(") + a + ", " +
                   v + ")";
        case castable_t::max:
            return std::string(is_double(d) ? "__builtin_fmax(" : "__builtin_fmaxf(") + a + ", " +
                   v + ")";
    }
    return a;
}

struct gen_t {
    einsummable_t const& e;
    layout_t             L;
    std::ostringstream   src;
    cg_kernel_t          k;
    int                  n_params = 0;

    explicit gen_t(einsummable_t const& e_) : e(e_), L(make_layout(e_)) {}

    int param(uint64_t v)
    {
        k.params.push_back(v);
        return n_params++;
    }

    std::string P(int i) const { return "a.p[" + std::to_string(i) + "]"; }

    // how operand `op` (0 the output, 1 + k input k) lies in memory
    std::string storage(int op) const
    {
        if (e.stored_as_half_pairs(op)) return "h2";
        return storage_type(op == 0 ? e.out_dtype() : e.inn_dtype(op - 1));
    }
    int storage_size(int op) const
    {
        if (e.stored_as_half_pairs(op)) return 4;
        return int(dtype_size(op == 0 ? e.out_dtype() : e.inn_dtype(op - 1)));
    }

    void header()
    {
        src << PRELUDE;
        src << "typedef " << (k.idx64 ? "unsigned long long" : "unsigned int") << " idx_t;\n";
        // the join as a function of the (converted) inputs
        emitter_t em;
        std::string r = em.emit(e.join.root);
        src << "__device__ __forceinline__ " << compute_type(e.out_dtype()) << " join_fn(";
        for (int i = 0; i != L.NI; ++i) {
            src << (i ? ", " : "") << compute_type(e.inn_dtype(i)) << " x" << i;
        }
        src << ")\n{\n" << em.body.str() << "    return " << r << ";\n}\n";
    }

    // `with_ws`: a pointer to partial results (in the accumulator type) follows the inputs
    void args_struct(bool with_ws = false)
    {
        src << "struct args_t {\n    " << storage(0) << "* out;\n";
        for (int i = 0; i != L.NI; ++i) {
            src << "    const " << storage(1 + i) << "* in" << i << ";\n";
        }
        if (with_ws) src << "    " << compute_type(e.out_dtype()) << "* ws;\n";
        src << "    idx_t p[" << std::max(n_params, 1) << "];\n};\n";
    }

    std::string store_cast(std::string const& v) const
    {
        if (e.stored_as_half_pairs(0)) return "narrow_c64(" + v + ")";
        if (e.out_dtype() == dtype_t::f16) return "(f16)(" + v + ")";
        return v;
    }
};

// Entry point name that identifies the kernel in profiles: kind, einsummable string, output
// dtype and a hash of the join text, e.g. es_ew__ab_a__ab__f16_1a2b3c4d.
std::string entry_name(einsummable_t const& e, const char* kind)
{
    std::string s = std::string("es_") + kind + "__";
    for (char c : e.str()) {
        if (c == ',') {
            s += '_';
        } else if (c == '-') {
            s += "__";
        } else if (c != '>') {
            s += c;
        }
    }
    s += std::string("__") + dtype_name(e.out_dtype());
    if (e.castable) {
        static const char* names[] = {"add", "mul", "min", "max"};
        s += std::string("_") + names[int(e.castable.value())];
    }
    uint32_t h = 2166136261u;
    for (char c : e.join.str()) h = (h ^ uint8_t(c)) * 16777619u;
    for (char c : e.half_complex) h = (h ^ uint8_t(c + 1)) * 16777619u;
    char buf[16];
    std::snprintf(buf, sizeof(buf), "_%08x", h);
    return s + buf + (e.any_half_pairs() ? "_h2" : "");
}

// Tuning aids: ES_KM_EW_UNROLL (vectors per thread of the elementwise kernels) and
// ES_KM_RED_UNROLL / ES_KM_RED_TEAM (row reductions) override the generators' defaults.
int env_int(const char* name, int fallback)
{
    const char* v = std::getenv(name);
    if (!v || !*v) return fallback;
    int x = std::atoi(v);
    return x > 0 ? x : fallback;
}

bool fits32(einsummable_t const& e)
{
    uint64_t const lim = (1ull << 32) - 1;
    if (e.out_nelem() >= lim) return false;
    for (int k = 0; k != int(e.inns.size()); ++k) {
        if (e.inn_nelem(k) >= lim) return false;
    }
    uint64_t join = 1;
    for (uint64_t d : e.join_shape) {
        join *= d;
        if (join >= (1ull << 62)) return false;
    }
    return true;
}

bool is_pow2(uint64_t v) { return v != 0 && (v & (v - 1)) == 0; }

int log2_of(uint64_t v)
{
    int n = 0;
    while ((1ull << n) < v) ++n;
    return n;
}

int min_elem_size(einsummable_t const& e)
{
    int m = int(dtype_size(e.out_dtype()));
    for (int k = 0; k != int(e.inns.size()); ++k) m = std::min(m, int(dtype_size(e.inn_dtype(k))));
    return m;
}

// ------------------------------------------------------------------------ elementwise
//
// One thread produces V consecutive elements of the innermost output mode; U such vectors
// per thread, 256 lanes apart, all loads issued before the first store (so an output that
// aliases a same-index input is safe).
cg_kernel_t gen_elementwise(einsummable_t const& e, int max_vec)
{
    gen_t g(e);
    auto& L = g.L;
    int const R = L.R;
    g.k.kind = cg_kind::elementwise;
    g.k.n_inns = L.NI;
    g.k.idx64 = !fits32(e);
    g.k.entry = entry_name(e, "ew");

    std::vector<access_t> acc(L.NI);
    bool all_straight = true;
    for (int k = 0; k != L.NI; ++k) {
        acc[k] = classify(e, k, R - 1, true);
        all_straight = all_straight && acc[k] == access_t::straight;
    }
    uint64_t const inner = L.shape[R - 1];
    uint64_t const n_out = e.out_nelem();
    // 16 bytes per lane for the widest type involved.  With 16 bytes for the narrowest (say
    // eight f16 in, eight f32 out) a lane moves 32 bytes of the wide tensor as two 16-byte
    // accesses 32 bytes apart, so every instruction touches half of each line: a 2^27-element
    // f16 -> f32 conversion ran at 3.1 TB/s that way and runs at 5.0 TB/s this way, the
    // reverse went from 4.4 to 5.0.
    // (An input without the innermost mode is one scalar per vector and has no say in this.)
    int widest = g.storage_size(0);
    for (int k = 0; k != int(e.inns.size()); ++k) {
        if (acc[k] == access_t::bcast) continue;
        // (a small input that every row reads again comes from the caches whatever its
        // access width: the rotary product's frequencies beside its f16 pairs)
        if (e.any_half_pairs() && e.inn_nelem(k) * 8 <= n_out) continue;
        widest = std::max(widest, g.storage_size(1 + k));
    }
    int const vcap = std::min(max_vec, 16 / widest);
    int V;
    uint64_t tail = 0;
    if (all_straight) {
        // the whole tensor is one row: full vectors plus a scalar tail
        V = (n_out >= uint64_t(vcap)) ? vcap : 1;
        tail = n_out % uint64_t(V);
    } else {
        V = pow2_divisor(inner, vcap);
    }
    int U = env_int("ES_KM_EW_UNROLL", 1);
    // A large permutation that keeps the innermost mode moves rows: the workgroup's 256
    // consecutive output vectors are whole rows that lie next to each other in the output,
    // while in the input each stands alone (C3a: 256-byte rows, 8 KiB apart).  When the mode
    // that follows the innermost one in the INPUT has an even extent, a thread takes the same
    // vector of two neighbours along it: the reads then come in runs of two rows as well
    // (abcd->acbd over 32 x 2048 x 32 x 128 f16, stand-alone: 0.77 -> 0.80 of HBM; more
    // than two neighbours per thread gain no more).
    int      pair_mode = -1;
    uint64_t pair_inner = 0;  // output vectors per index of that mode
    int const pair_rule = env_int("ES_KM_EW_PAIR", 1);  // tuning and tests: 0 never, 2 at any size
    if (U == 1 && !all_straight && L.NI == 1 && acc[0] == access_t::vec && R >= 3 &&
        (pair_rule == 2 || (pair_rule == 1 && n_out * dtype_size(e.out_dtype()) >= (32ull << 20)))) {
        int next = -1;
        for (int m = 0; m + 1 < R; ++m) {
            if (L.stride[0][m] == 0) continue;
            if (next < 0 || L.stride[0][m] < L.stride[0][next]) next = m;
        }
        if (next >= 0 && next != R - 2 && L.shape[next] % 2 == 0) {
            pair_mode = next;
            g.k.row_pairs = true;
            pair_inner = inner / uint64_t(V);
            for (int m = next + 1; m + 1 < R; ++m) pair_inner *= L.shape[m];
            U = 2;
        }
    }
    // Outputs far larger than the last-level cache are written non-temporally: they would
    // only evict inputs that later nodes still read (measured on 8192^2 f16: +20% on the
    // producing kernel).  ES_KM_EW_NT: 1 loads and stores, 2 loads only, 3 stores only, 4 none.
    // A node whose operands and result together fit the 256 MiB memory-side cache leaves its
    // result there for the node that reads it next (C2: the row sum after exp(x - m) reads at
    // 6.0 instead of 5.4 TB/s, the producer is as fast either way); beyond that the cache
    // holds nothing useful at the end and plain stores only cost bandwidth.
    uint64_t const out_bytes = n_out * uint64_t(g.storage_size(0));
    uint64_t footprint = out_bytes;
    for (int k = 0; k != int(e.inns.size()); ++k) {
        footprint += e.inn_nelem(k) * uint64_t(g.storage_size(1 + k));
    }
    bool const stream_out = out_bytes >= (64ull << 20) && footprint > (288ull << 20);
    // With a result beyond the cache's size such a node reads non-temporally too.  A line
    // that was read normally is still in the memory-side cache when its result is stored, the
    // store hits it there, and the dirty line is written back during the NEXT node: the row
    // max behind a 1 GiB in-place scale read at 5.1 TB/s, behind the same node with
    // streaming loads at 6.2 (C4: row max 0.206 -> 0.173 ms, row sum 0.205 -> 0.168, P.V
    // 0.275 -> 0.215, chain 1.92 -> 1.77 ms).
    // A result that itself fits the cache (C2's 128 MiB product, read by the row max next)
    // is better off with plain loads: row max 22.7 against 25.0 us.
    bool const stream_in = stream_out && out_bytes >= (256ull << 20);
    int const nt_mode = env_int("ES_KM_EW_NT", stream_in ? 1 : (stream_out ? 3 : 4));
    int const NT_LD = (nt_mode == 1 || nt_mode == 2) ? 1 : 0;
    int const NT_ST = (nt_mode == 1 || nt_mode == 3) ? 1 : 0;
    uint64_t const n_vec = n_out / uint64_t(V);
    g.k.vec = V;

    int p_nvec = g.param(n_vec);
    uint64_t const vpr = all_straight ? n_vec : inner / uint64_t(V);
    int p_vpr = g.param(vpr);
    std::vector<int> p_shape(R);
    for (int m = 0; m != R; ++m) p_shape[m] = g.param(L.shape[m]);
    std::vector<std::vector<int>> p_str(L.NI, std::vector<int>(R, -1));
    for (int k = 0; k != L.NI; ++k) {
        if (acc[k] == access_t::straight) continue;
        for (int m = 0; m != R; ++m) {
            if (L.stride[k][m]) p_str[k][m] = g.param(L.stride[k][m]);
        }
    }
    // Every thread takes its vector's index apart.  A division by a run-time value is some
    // twenty vector instructions, two of them as many as the arithmetic of eight elements of
    // a softmax; by a power of two (the shift is a parameter, so all such shapes share the
    // code) it is two.
    int p_pair = pair_mode >= 0 ? g.param(pair_inner) : -1;
    int p_pair_sh = (pair_mode >= 0 && is_pow2(pair_inner)) ? g.param(uint64_t(log2_of(pair_inner))) : -1;
    int p_vpr_sh = (!all_straight && is_pow2(vpr)) ? g.param(uint64_t(log2_of(vpr))) : -1;
    std::vector<int> p_shape_sh(R, -1);
    for (int m = 1; m + 1 < R; ++m) {
        if (!all_straight && is_pow2(L.shape[m])) p_shape_sh[m] = g.param(uint64_t(log2_of(L.shape[m])));
    }

    g.header();
    g.args_struct();
    auto& s = g.src;
    s << "#define V " << V << "\n#define U " << U << "\n";
    s << "extern \"C\" __global__ __launch_bounds__(256) void " << g.k.entry << "(args_t a)\n{\n";
    s << "    const idx_t n_vec = " << g.P(p_nvec) << ";\n";
    for (int k = 0; k != L.NI; ++k) {
        std::string T = g.storage(1 + k);
        if (acc[k] == access_t::bcast) {
            s << "    " << T << " s" << k << "[U];\n";
        } else {
            s << "    vec_t<" << T << ", V> r" << k << "[U];\n";
        }
    }
    s << "    idx_t vid[U];\n    bool live[U];\n";
    if (pair_mode >= 0) {
        // work item w stands for the vectors (.., 2 q, ..) and (.., 2 q + 1, ..) of the paired
        // mode: with t = w / inner (all outer indices and q), the first is w + t * inner
        s << "    const idx_t w = ((idx_t)blockIdx.y * gridDim.x + blockIdx.x) * 256 + threadIdx.x;\n";
        if (p_pair_sh >= 0) {
            s << "    const idx_t wt = w >> " << g.P(p_pair_sh) << ";\n";
        } else {
            s << "    const idx_t wt = w / " << g.P(p_pair) << ";\n";
        }
    }
    s << "#pragma unroll\n    for (int u = 0; u != U; ++u) {\n";
    if (pair_mode >= 0) {
        s << "        vid[u] = w + (wt + (idx_t)u) * " << g.P(p_pair) << ";\n";
        s << "        live[u] = w < n_vec / 2;\n";
    } else {
        s << "        vid[u] = (((idx_t)blockIdx.y * gridDim.x + blockIdx.x) * U + u) * 256 + threadIdx.x;\n";
        s << "        live[u] = vid[u] < n_vec;\n";
    }
    s << "        if (live[u]) {\n";
    if (!all_straight) {
        // name = rem mod divisor; rem = rem / divisor
        auto split = [&](std::string const& name, int p_div, int p_sh, const char* scale) {
            if (p_sh >= 0) {
                s << "            const idx_t " << name << " = (rem & (" << g.P(p_div) << " - 1))"
                  << scale << ";\n";
                s << "            rem >>= " << g.P(p_sh) << ";\n";
            } else {
                s << "            const idx_t " << name << " = (rem % " << g.P(p_div) << ")" << scale
                  << ";\n";
                s << "            rem /= " << g.P(p_div) << ";\n";
            }
        };
        s << "            idx_t rem = vid[u];\n";
        split("c", p_vpr, p_vpr_sh, " * V");
        for (int m = R - 2; m >= 1; --m) split("d" + std::to_string(m), p_shape[m], p_shape_sh[m], "");
        if (R >= 2) s << "            const idx_t d0 = rem;\n";
    }
    for (int k = 0; k != L.NI; ++k) {
        std::string T = g.storage(1 + k);
        if (acc[k] == access_t::straight) {
            s << "            r" << k << "[u] = ldv<" << NT_LD << ">(reinterpret_cast<const vec_t<" << T
              << ", V>*>(a.in" << k << " + vid[u] * V));\n";
            continue;
        }
        std::string off = "0";
        for (int m = 0; m != R - 1; ++m) {
            if (p_str[k][m] >= 0) off += " + d" + std::to_string(m) + " * " + g.P(p_str[k][m]);
        }
        if (acc[k] == access_t::vec) {
            // an input that lacks an outer mode is read again for every index of that mode:
            // it is not streamed, whatever the node's size
            int const nt = e.inn_nelem(k) == n_out ? NT_LD : 0;
            s << "            r" << k << "[u] = ldv<" << nt << ">(reinterpret_cast<const vec_t<" << T
              << ", V>*>(a.in" << k << " + (" << off << " + c)));\n";
        } else if (acc[k] == access_t::bcast) {
            s << "            s" << k << "[u] = a.in" << k << "[" << off << "];\n";
        } else {
            s << "            {\n                const idx_t o = " << off << " + c * "
              << g.P(p_str[k][R - 1]) << ";\n";
            s << "#pragma unroll\n                for (int j = 0; j != V; ++j) r" << k
              << "[u].v[j] = a.in" << k << "[o + j * " << g.P(p_str[k][R - 1]) << "];\n";
            s << "            }\n";
        }
    }
    s << "        }\n    }\n";
    s << "#pragma unroll\n    for (int u = 0; u != U; ++u) {\n        if (live[u]) {\n";
    s << "            vec_t<" << g.storage(0) << ", V> res;\n";
    s << "#pragma unroll\n            for (int j = 0; j != V; ++j) {\n";
    s << "                res.v[j] = " << g.store_cast([&] {
        std::string call = "join_fn(";
        for (int k = 0; k != L.NI; ++k) {
            call += (k ? ", " : "");
            if (acc[k] == access_t::bcast) {
                call += "cvt_in(s" + std::to_string(k) + "[u])";
            } else {
                call += "cvt_in(r" + std::to_string(k) + "[u].v[j])";
            }
        }
        return call + ")";
    }()) << ";\n";
    s << "            }\n";
    s << "            stv<" << NT_ST << ">(reinterpret_cast<vec_t<" << g.storage(0)
      << ", V>*>(a.out + vid[u] * V), res);\n";
    s << "        }\n    }\n";
    if (tail) {
        s << "    if (blockIdx.x == 0 && blockIdx.y == 0 && threadIdx.x < " << tail << ") {\n";
        s << "        const idx_t i = n_vec * V + threadIdx.x;\n";
        s << "        a.out[i] = " << g.store_cast([&] {
            std::string call = "join_fn(";
            for (int k = 0; k != L.NI; ++k) {
                call += std::string(k ? ", " : "") + "cvt_in(a.in" + std::to_string(k) + "[i])";
            }
            return call + ")";
        }()) << ";\n    }\n";
    }
    s << "}\n";

    g.k.source = s.str();
    uint64_t per_block = 256ull * uint64_t(U);
    g.k.grid = std::max<uint64_t>(1, (n_vec + per_block - 1) / per_block);
    g.k.block = 256;
    g.k.out_inn_align.push_back(V * g.storage_size(0));
    for (int k = 0; k != L.NI; ++k) {
        bool wide = acc[k] == access_t::straight || acc[k] == access_t::vec;
        g.k.out_inn_align.push_back((wide ? V : 1) * g.storage_size(1 + k));
    }
    return std::move(g.k);
}

}  // namespace

// Elements of a row that one lane takes per step of a row reduction.  It fixes how a row is
// dealt to the lanes, i.e. the order of a sum: the same for 2- and 4-byte elements (16 bytes
// of the former, two 16-byte pieces of the latter), so that a reduction keeps its order when
// its input arrives in another of those types.
int row_reduction_lane_elems(int smallest_elem_bytes)
{
    return smallest_elem_bytes <= 4 ? 8 : std::max(1, 16 / smallest_elem_bytes);
}

namespace
{
// --------------------------------------------------------------- reduce, aggregated modes
// innermost: a team of TEAM lanes (one wavefront, or a 256-thread workgroup for long rows)
// owns one output element, strides over the flattened aggregated index space in V-element
// vectors, accumulates in float / double, then reduces across lanes with DPP shuffles and
// across wavefronts through LDS.
cg_kernel_t gen_reduce_row(einsummable_t const& e, int max_vec)
{
    gen_t g(e);
    auto& L = g.L;
    int const R = L.R, O = L.O;
    g.k.kind = cg_kind::reduce_row;
    g.k.n_inns = L.NI;
    g.k.idx64 = !fits32(e);
    g.k.entry = entry_name(e, "redrow");
    castable_t const cast = e.castable.value();
    dtype_t const od = e.out_dtype();

    std::vector<access_t> acc(L.NI);
    for (int k = 0; k != L.NI; ++k) acc[k] = classify(e, k, R - 1, false);
    uint64_t nA = 1;
    for (int m = O; m != R; ++m) nA *= L.shape[m];
    uint64_t const n_out = e.out_nelem();
    int const vcap = std::min(max_vec, row_reduction_lane_elems(min_elem_size(e)));
    int const V = pow2_divisor(L.shape[R - 1], vcap);
    uint64_t const nvecA = nA / uint64_t(V);
    int const TEAM = env_int("ES_KM_RED_TEAM", (nvecA >= 512) ? 256 : 64) == 256 ? 256 : 64;
    int const BLOCK = 256;
    int const U = env_int("ES_KM_RED_UNROLL",
                          (nvecA >= uint64_t(TEAM) * 4) ? 4 : ((nvecA >= uint64_t(TEAM) * 2) ? 2 : 1));
    g.k.vec = V;
    // A handful of very long rows: one team per row leaves the device idle.  Each row is
    // then cut into slices on grid z; a second kernel folds the slices' partial results in
    // order (needs a workspace of slices x rows accumulators).
    uint64_t S = 1, chunk = nvecA;
    if (TEAM == 256 && n_out < 1024 && nvecA >= uint64_t(TEAM) * U * 16) {
        S = std::min<uint64_t>({(2048 + n_out - 1) / n_out, nvecA / (uint64_t(TEAM) * U * 8), 4096});
        S = uint64_t(std::max(1, env_int("ES_KM_RED_SPLITS", int(S))));
        uint64_t const step = uint64_t(TEAM) * U;
        chunk = ((nvecA + S - 1) / S + step - 1) / step * step;
        S = (nvecA + chunk - 1) / chunk;
    }
    bool const split = S > 1;
    g.k.splits = int(S);
    g.k.ws_bytes = split ? S * n_out * dtype_size(od == dtype_t::f16 ? dtype_t::f32 : od) : 0;

    int p_nout = g.param(n_out);
    int p_nvec = g.param(nvecA);
    int p_chunk = g.param(chunk);
    std::vector<int> p_shape(R);
    for (int m = 0; m != R; ++m) p_shape[m] = g.param(L.shape[m]);
    std::vector<std::vector<int>> p_str(L.NI, std::vector<int>(R, -1));
    for (int k = 0; k != L.NI; ++k) {
        for (int m = 0; m != R; ++m) {
            if (L.stride[k][m]) p_str[k][m] = g.param(L.stride[k][m]);
        }
    }

    g.header();
    g.args_struct(split);
    auto& s = g.src;
    std::string ACC = compute_type(od);
    s << "#define V " << V << "\n#define U " << U << "\n#define TEAM " << TEAM << "\n";
    s << "__device__ __forceinline__ " << ACC << " comb(" << ACC << " x, " << ACC
      << " y) { return " << combine_expr(cast, od, "x", "y") << "; }\n";
    if (split) {
        // Second pass: one wavefront per output row.  Lane l adds slices l, l + 64, ... and
        // the 64 sums meet in a fixed butterfly, so the result does not depend on timing (a
        // thread of its own per row waits for one load after the other: 38 us for the 2048
        // slices of a single row, as long as the first pass).
        g.k.entry2 = g.k.entry + "_fold";
        g.k.grid2 = (n_out + 3) / 4;
        s << "extern \"C\" __global__ __launch_bounds__(" << BLOCK << ") void " << g.k.entry2
          << "(args_t a)\n{\n";
        s << "    const idx_t row = ((idx_t)blockIdx.y * gridDim.x + blockIdx.x) * 4 + threadIdx.x / 64;\n";
        s << "    if (row >= " << g.P(p_nout) << ") return;\n";
        s << "    " << ACC << " acc = " << identity_of(cast, od) << ";\n";
        s << "#pragma unroll 4\n";
        s << "    for (unsigned z = threadIdx.x % 64; z < " << S << "u; z += 64) acc = comb(acc, a.ws[(size_t)z * "
          << g.P(p_nout) << " + row]);\n";
        s << "#pragma unroll\n    for (int m = 32; m >= 1; m >>= 1) acc = comb(acc, lane_xor(acc, m));\n";
        s << "    if (threadIdx.x % 64 == 0) a.out[row] = " << g.store_cast("acc") << ";\n}\n";
    }
    s << "extern \"C\" __global__ __launch_bounds__(" << BLOCK << ") void " << g.k.entry << "(args_t a)\n{\n";
    s << "    const idx_t n_out = " << g.P(p_nout) << ";\n";
    if (split) {
        s << "    const idx_t v_lo = (idx_t)blockIdx.z * " << g.P(p_chunk) << ";\n";
        s << "    const idx_t nvec = v_lo + " << g.P(p_chunk) << " < " << g.P(p_nvec) << " ? v_lo + "
          << g.P(p_chunk) << " : " << g.P(p_nvec) << ";  // end of this slice\n";
    } else {
        s << "    const idx_t v_lo = 0;\n";
        s << "    const idx_t nvec = " << g.P(p_nvec) << ";\n";
    }
    s << "    const unsigned lane = threadIdx.x % TEAM;\n";
    // An input larger than the 256 MiB memory-side cache is walked from its last row to its
    // first.  The node that produced it wrote it front to back, so its tail is what the
    // cache still holds; and the node that follows (an elementwise pass, front to back) finds
    // the head, which this kernel read last.  C4's row max and row sum gain 3-4 %, the
    // elementwise node after them 2 %, the LLaMA layer 1.2 %; below that size it is a wash.
    uint64_t in_bytes = 0;
    for (int k = 0; k != L.NI; ++k) in_bytes += e.inn_nelem(k) * dtype_size(e.inn_dtype(k));
    bool const reverse = env_int("ES_KM_RED_REVERSE", in_bytes >= (256ull << 20) ? 1 : 0) != 0;
    s << "    const idx_t row_fwd = ((idx_t)blockIdx.y * gridDim.x + blockIdx.x) * (" << BLOCK
      << " / TEAM) + threadIdx.x / TEAM;\n";
    if (reverse) {
        s << "    const idx_t row = row_fwd < n_out ? n_out - 1 - row_fwd : row_fwd;\n";
    } else {
        s << "    const idx_t row = row_fwd;\n";
    }
    // min / max of f16 values is exact in f16: keep V packed half accumulators per lane
    // (v_pk_max_f16 / v_pk_min_f16, no conversions) and widen once after the loop
    bool const half_minmax = od == dtype_t::f16 && L.NI == 1 && e.join.is_identity() &&
                             acc[0] == access_t::vec &&
                             (cast == castable_t::min || cast == castable_t::max);
    s << "    " << ACC << " acc = " << identity_of(cast, od) << ";\n";
    if (half_minmax) {
        s << "    vec_t<f16, V> accv;\n#pragma unroll\n    for (int j = 0; j != V; ++j) accv.v[j] = "
             "(f16)("
          << identity_of(cast, od) << ");\n";
    }
    s << "    if (row < n_out) {\n";
    s << "        idx_t rem = row;\n";
    for (int m = O - 1; m >= 1; --m) {
        s << "        const idx_t d" << m << " = rem % " << g.P(p_shape[m]) << ";\n";
        s << "        rem /= " << g.P(p_shape[m]) << ";\n";
    }
    s << "        const idx_t d0 = rem;\n";
    for (int k = 0; k != L.NI; ++k) {
        std::string off = "0";
        for (int m = 0; m != O; ++m) {
            if (p_str[k][m] >= 0) off += " + d" + std::to_string(m) + " * " + g.P(p_str[k][m]);
        }
        s << "        const idx_t b" << k << " = " << off << ";\n";
    }
    // inputs without any aggregated mode are loaded once per row
    std::vector<bool> row_const(L.NI, true);
    for (int k = 0; k != L.NI; ++k) {
        for (int m = O; m != R; ++m) row_const[k] = row_const[k] && p_str[k][m] < 0;
        if (row_const[k]) {
            s << "        const " << compute_type(e.inn_dtype(k)) << " c" << k << " = cvt_in(a.in"
              << k << "[b" << k << "]);\n";
        }
    }
    s << "        for (idx_t v0 = v_lo + lane; v0 < nvec; v0 += (idx_t)TEAM * U) {\n";
    for (int k = 0; k != L.NI; ++k) {
        if (row_const[k]) continue;
        std::string T = storage_type(e.inn_dtype(k));
        if (acc[k] == access_t::bcast) {
            s << "            " << T << " s" << k << "[U];\n";
        } else {
            s << "            vec_t<" << T << ", V> r" << k << "[U];\n";
        }
    }
    s << "#pragma unroll\n            for (int u = 0; u != U; ++u) {\n";
    s << "                const idx_t vv = v0 + (idx_t)u * TEAM;\n";
    s << "                if (vv < nvec) {\n";
    s << "                    idx_t ar = vv * V;\n";
    if (R - 1 > O) {
        s << "                    const idx_t g" << (R - 1) << " = ar % " << g.P(p_shape[R - 1]) << ";\n";
        s << "                    ar /= " << g.P(p_shape[R - 1]) << ";\n";
    } else {
        // a single aggregated mode: the flat index is the mode's index
        s << "                    const idx_t g" << (R - 1) << " = ar;\n";
    }
    for (int m = R - 2; m > O; --m) {
        s << "                    const idx_t g" << m << " = ar % " << g.P(p_shape[m]) << ";\n";
        s << "                    ar /= " << g.P(p_shape[m]) << ";\n";
    }
    if (R - 1 > O) s << "                    const idx_t g" << O << " = ar;\n";
    for (int k = 0; k != L.NI; ++k) {
        if (row_const[k]) continue;
        std::string T = storage_type(e.inn_dtype(k));
        std::string off = "b" + std::to_string(k);
        for (int m = O; m != R - 1; ++m) {
            if (p_str[k][m] >= 0) off += " + g" + std::to_string(m) + " * " + g.P(p_str[k][m]);
        }
        if (acc[k] == access_t::vec) {
            s << "                    r" << k << "[u] = *reinterpret_cast<const vec_t<" << T
              << ", V>*>(a.in" << k << " + (" << off << " + g" << (R - 1) << "));\n";
        } else if (acc[k] == access_t::bcast) {
            s << "                    s" << k << "[u] = a.in" << k << "[" << off << "];\n";
        } else {
            s << "#pragma unroll\n                    for (int j = 0; j != V; ++j) r" << k
              << "[u].v[j] = a.in" << k << "[" << off << " + (g" << (R - 1) << " + j) * "
              << g.P(p_str[k][R - 1]) << "];\n";
        }
    }
    s << "                }\n            }\n";
    s << "#pragma unroll\n            for (int u = 0; u != U; ++u) {\n";
    s << "                if (v0 + (idx_t)u * TEAM < nvec) {\n";
    s << "#pragma unroll\n                    for (int j = 0; j != V; ++j) {\n";
    if (half_minmax) {
        s << "                        accv.v[j] = "
          << (cast == castable_t::max ? "__builtin_fmaxf16" : "__builtin_fminf16")
          << "(accv.v[j], r0[u].v[j]);\n                    }\n                }\n            }\n";
        s << "        }\n    }\n";
        s << "#pragma unroll\n    for (int j = 0; j != V; ++j) acc = comb(acc, (float)accv.v[j]);\n";
    } else {
        s << "                        acc = comb(acc, join_fn(";
        for (int k = 0; k != L.NI; ++k) {
            s << (k ? ", " : "");
            if (row_const[k]) {
                s << "c" << k;
            } else if (acc[k] == access_t::bcast) {
                s << "cvt_in(s" << k << "[u])";
            } else {
                s << "cvt_in(r" << k << "[u].v[j])";
            }
        }
        s << "));\n                    }\n                }\n            }\n";
        s << "        }\n    }\n";
    }
    s << "#pragma unroll\n    for (int m = 32; m >= 1; m >>= 1) acc = comb(acc, lane_xor(acc, m));\n";
    if (TEAM == 256) {
        s << "    __shared__ " << ACC << " part[4];\n";
        s << "    if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = acc;\n";
        s << "    __syncthreads();\n";
        s << "    if (threadIdx.x == 0 && row < n_out) {\n";
        s << "        acc = comb(comb(part[0], part[1]), comb(part[2], part[3]));\n";
        if (split) {
            s << "        a.ws[(size_t)blockIdx.z * n_out + row] = acc;\n    }\n";
        } else {
            s << "        a.out[row] = " << g.store_cast("acc") << ";\n    }\n";
        }
    } else {
        s << "    if (lane == 0 && row < n_out) a.out[row] = " << g.store_cast("acc") << ";\n";
    }
    s << "}\n";

    g.k.source = s.str();
    uint64_t rows_per_block = uint64_t(BLOCK / TEAM);
    g.k.grid = (n_out + rows_per_block - 1) / rows_per_block;
    g.k.block = unsigned(BLOCK);
    g.k.out_inn_align.push_back(int(dtype_size(od)));
    for (int k = 0; k != L.NI; ++k) {
        bool wide = acc[k] == access_t::vec && !row_const[k];
        g.k.out_inn_align.push_back(std::min(16, (wide ? V : 1) * int(dtype_size(e.inn_dtype(k)))));
    }
    return std::move(g.k);
}

// ------------------------------------------------------------- reduce, any other layout:
// one thread owns V consecutive elements of the innermost output mode and walks the
// aggregated modes serially (nested loops, one per aggregated mode).  Lanes stay coalesced
// along the output's innermost mode.
cg_kernel_t gen_reduce_col(einsummable_t const& e, int max_vec)
{
    gen_t g(e);
    auto& L = g.L;
    int const R = L.R, O = L.O;
    g.k.kind = cg_kind::reduce_col;
    g.k.n_inns = L.NI;
    g.k.idx64 = !fits32(e);
    g.k.entry = entry_name(e, "redcol");
    castable_t const cast = e.castable.value();
    dtype_t const od = e.out_dtype();

    std::vector<access_t> acc(L.NI);
    bool any_vec = false;
    for (int k = 0; k != L.NI; ++k) {
        acc[k] = classify(e, k, O - 1, false);
        any_vec = any_vec || acc[k] == access_t::vec;
    }
    uint64_t const n_out = e.out_nelem();
    int const vcap = std::min(max_vec, 16 / min_elem_size(e));
    // vectors only pay when some input is contiguous along the output's inner mode
    int const V = any_vec ? pow2_divisor(L.shape[O - 1], vcap) : 1;
    uint64_t const n_vec = n_out / uint64_t(V);
    g.k.vec = V;
    // Few outputs and a long aggregation: one thread per output vector leaves the device
    // idle.  The outermost aggregated mode is then cut into slices that run side by side
    // (grid z), each leaving partial results in the workspace; a second kernel folds the
    // slices in order, so the result does not depend on scheduling.  (One launch, in which
    // the slices raise flags in the workspace and the last one folds, was measured on 8192 x
    // 8192 f16: the fences that make partial results and flags visible across the device's
    // L2 caches cost 23 us in all, the second launch costs 4.)
    uint64_t const outer = L.shape[O];
    // measured with the slice-parallel fold below: 128 K threads with 4 rows in flight each
    // (8192 x 8192 f16: 4.2 TB/s with 64 K, 4.6 with 128 K, 4.9 with 256 K, where 2048 x 4096
    // f32 and 64 x 2048 x 1024 f16 lose 6-9 %); eight rows in flight are 3 % faster than four
    uint64_t const want_threads = 1ull << 17;
    uint64_t       S = 1;
    if (n_vec * 2 <= want_threads && outer >= 16) {
        S = std::min<uint64_t>({(want_threads + n_vec - 1) / n_vec, outer / 8, 1024});
        S = uint64_t(std::max(1, env_int("ES_KM_RED_SPLITS", int(S))));
        S = std::min<uint64_t>(S, outer);
    }
    uint64_t const chunk = (outer + S - 1) / S;
    S = (outer + chunk - 1) / chunk;  // no empty slice
    bool const split = S > 1;
    g.k.splits = int(S);
    g.k.ws_bytes = split ? S * n_out * dtype_size(od == dtype_t::f16 ? dtype_t::f32 : od) : 0;

    int p_nvec = g.param(n_vec);
    int p_nout = g.param(n_out);
    int p_chunk = g.param(chunk);
    int p_vpr = g.param(L.shape[O - 1] / uint64_t(V));
    std::vector<int> p_shape(R);
    for (int m = 0; m != R; ++m) p_shape[m] = g.param(L.shape[m]);
    std::vector<std::vector<int>> p_str(L.NI, std::vector<int>(R, -1));
    for (int k = 0; k != L.NI; ++k) {
        for (int m = 0; m != R; ++m) {
            if (L.stride[k][m]) p_str[k][m] = g.param(L.stride[k][m]);
        }
    }

    g.header();
    g.args_struct(split);
    auto& s = g.src;
    std::string ACC = compute_type(od);
    s << "#define V " << V << "\n";
    s << "__device__ __forceinline__ " << ACC << " comb(" << ACC << " x, " << ACC
      << " y) { return " << combine_expr(cast, od, "x", "y") << "; }\n";
    if (split) {
        // Second pass: fold the slices' partial results.  A workgroup owns 16 output vectors;
        // its 16 groups of lanes each add every 16th slice (a thread of its own per output
        // would wait for one load after the other: 23 us for 256 slices of 1024 floats), then
        // group 0 adds the 16 sums in group order, so the result does not depend on timing.
        g.k.entry2 = g.k.entry + "_fold";
        g.k.grid2 = (n_vec + 15) / 16;
        s << "extern \"C\" __global__ __launch_bounds__(256) void " << g.k.entry2
          << "(args_t a)\n{\n";
        s << "    __shared__ " << ACC << " sh[256 * V];\n";
        s << "    const unsigned vl = threadIdx.x % 16, zl = threadIdx.x / 16;\n";
        s << "    const idx_t vid = ((idx_t)blockIdx.y * gridDim.x + blockIdx.x) * 16 + vl;\n";
        s << "    const bool live = vid < " << g.P(p_nvec) << ";\n";
        s << "    " << ACC << " acc[V];\n";
        s << "#pragma unroll\n    for (int j = 0; j != V; ++j) acc[j] = "
          << identity_of(cast, od) << ";\n";
        s << "    if (live) {\n";
        s << "#pragma unroll 4\n        for (unsigned z = zl; z < " << S << "u; z += 16) {\n";
        s << "            const " << ACC << "* part = a.ws + (size_t)z * " << g.P(p_nout)
          << " + (size_t)vid * V;\n";
        s << "#pragma unroll\n            for (int j = 0; j != V; ++j) acc[j] = comb(acc[j], part[j]);\n";
        s << "        }\n    }\n";
        s << "#pragma unroll\n    for (int j = 0; j != V; ++j) sh[threadIdx.x * V + j] = acc[j];\n";
        s << "    __syncthreads();\n";
        s << "    if (zl != 0 || !live) return;\n";
        s << "    for (unsigned z = 1; z != 16; ++z) {\n";
        s << "#pragma unroll\n        for (int j = 0; j != V; ++j) acc[j] = comb(acc[j], sh[(z * 16 + vl) * V + j]);\n";
        s << "    }\n";
        s << "    vec_t<" << storage_type(od) << ", V> res;\n";
        s << "#pragma unroll\n    for (int j = 0; j != V; ++j) res.v[j] = "
          << g.store_cast("acc[j]") << ";\n";
        s << "    *reinterpret_cast<vec_t<" << storage_type(od)
          << ", V>*>(a.out + vid * V) = res;\n}\n";
    }
    s << "extern \"C\" __global__ __launch_bounds__(256) void " << g.k.entry << "(args_t a)\n{\n";
    s << "    const idx_t vid = ((idx_t)blockIdx.y * gridDim.x + blockIdx.x) * 256 + threadIdx.x;\n";
    s << "    if (vid >= " << g.P(p_nvec) << ") return;\n";
    s << "    idx_t rem = vid;\n";
    s << "    const idx_t c = (rem % " << g.P(p_vpr) << ") * V;\n";
    s << "    rem /= " << g.P(p_vpr) << ";\n";
    for (int m = O - 2; m >= 1; --m) {
        s << "    const idx_t d" << m << " = rem % " << g.P(p_shape[m]) << ";\n";
        s << "    rem /= " << g.P(p_shape[m]) << ";\n";
    }
    if (O >= 2) s << "    const idx_t d0 = rem;\n";
    for (int k = 0; k != L.NI; ++k) {
        std::string off = "0";
        for (int m = 0; m != O - 1; ++m) {
            if (p_str[k][m] >= 0) off += " + d" + std::to_string(m) + " * " + g.P(p_str[k][m]);
        }
        if (p_str[k][O - 1] >= 0) off += " + c * " + g.P(p_str[k][O - 1]);
        s << "    const idx_t b" << k << " = " << off << ";\n";
    }
    s << "    " << ACC << " acc[V];\n";
    s << "#pragma unroll\n    for (int j = 0; j != V; ++j) acc[j] = " << identity_of(cast, od)
      << ";\n";
    std::string indent = "    ";
    for (int m = O; m != R; ++m) {
        if (m == O && split) {
            s << indent << "const idx_t lo" << m << " = (idx_t)blockIdx.z * " << g.P(p_chunk) << ";\n";
            s << indent << "const idx_t hi" << m << " = lo" << m << " + " << g.P(p_chunk) << " < "
              << g.P(p_shape[m]) << " ? lo" << m << " + " << g.P(p_chunk) << " : "
              << g.P(p_shape[m]) << ";\n";
            if (m == R - 1) s << "#pragma unroll 8\n";  // several rows' loads in flight
            s << indent << "for (idx_t g" << m << " = lo" << m << "; g" << m << " < hi" << m
              << "; ++g" << m << ") {\n";
        } else {
            if (m == R - 1) s << "#pragma unroll 8\n";
            s << indent << "for (idx_t g" << m << " = 0; g" << m << " != " << g.P(p_shape[m])
              << "; ++g" << m << ") {\n";
        }
        indent += "    ";
    }
    for (int k = 0; k != L.NI; ++k) {
        std::string T = storage_type(e.inn_dtype(k));
        std::string off = "b" + std::to_string(k);
        for (int m = O; m != R; ++m) {
            if (p_str[k][m] >= 0) off += " + g" + std::to_string(m) + " * " + g.P(p_str[k][m]);
        }
        if (acc[k] == access_t::vec) {
            s << indent << "const vec_t<" << T << ", V> r" << k
              << " = *reinterpret_cast<const vec_t<" << T << ", V>*>(a.in" << k << " + (" << off
              << "));\n";
        } else if (acc[k] == access_t::bcast) {
            s << indent << "const " << T << " s" << k << " = a.in" << k << "[" << off << "];\n";
        } else {
            s << indent << "vec_t<" << T << ", V> r" << k << ";\n";
            s << "#pragma unroll\n" << indent << "for (int j = 0; j != V; ++j) r" << k
              << ".v[j] = a.in" << k << "[" << off << " + j * " << g.P(p_str[k][O - 1]) << "];\n";
        }
    }
    s << "#pragma unroll\n" << indent << "for (int j = 0; j != V; ++j) acc[j] = comb(acc[j], join_fn(";
    for (int k = 0; k != L.NI; ++k) {
        s << (k ? ", " : "");
        if (acc[k] == access_t::bcast) {
            s << "cvt_in(s" << k << ")";
        } else {
            s << "cvt_in(r" << k << ".v[j])";
        }
    }
    s << "));\n";
    for (int m = O; m != R; ++m) {
        indent.resize(indent.size() - 4);
        s << indent << "}\n";
    }
    if (split) {
        s << "    " << ACC << "* part = a.ws + (size_t)blockIdx.z * " << g.P(p_nout)
          << " + (size_t)vid * V;\n";
        s << "#pragma unroll\n    for (int j = 0; j != V; ++j) part[j] = acc[j];\n";
    } else {
        s << "    vec_t<" << storage_type(od) << ", V> res;\n";
        s << "#pragma unroll\n    for (int j = 0; j != V; ++j) res.v[j] = "
          << g.store_cast("acc[j]") << ";\n";
        s << "    *reinterpret_cast<vec_t<" << storage_type(od)
          << ", V>*>(a.out + vid * V) = res;\n";
    }
    s << "}\n";

    g.k.source = s.str();
    g.k.grid = std::max<uint64_t>(1, (n_vec + 255) / 256);
    g.k.block = 256;
    // (a vector wider than 16 bytes moves as 16-byte pieces: vec_t asks for no more)
    g.k.out_inn_align.push_back(std::min(16, V * int(dtype_size(od))));
    for (int k = 0; k != L.NI; ++k) {
        bool wide = acc[k] == access_t::vec;
        g.k.out_inn_align.push_back(std::min(16, (wide ? V : 1) * int(dtype_size(e.inn_dtype(k)))));
    }
    return std::move(g.k);
}

}  // namespace

// ------------------------------------------------------------------- chains over rows
//
// One team of lanes per row, as in gen_reduce_row (the same team size, vector width and
// order of accumulation: a sum comes out with the bits the reduction kernel gives it), but
// the row's vectors stay in registers from the first stage to the last.
cg_kernel_t gen_row_chain(cg_chain_t const& c, int max_vec)
{
    int const R = int(c.shape.size());
    int const NE = int(c.exts.size());
    int const NS = int(c.stages.size());
    if (R < 1 || NS < 2 || NE < 1) throw ir_error("row chain: nothing to chain");
    int const O = R - 1;
    uint64_t const n = c.shape[size_t(R - 1)];
    uint64_t n_rows = 1;
    for (int m = 0; m != O; ++m) n_rows *= c.shape[size_t(m)];

    // what every stage yields, and which inputs are whole rows
    std::vector<dtype_t> result(static_cast<size_t>(NS));
    std::vector<bool>    is_vec(static_cast<size_t>(NE));
    for (int k = 0; k != NE; ++k) {
        auto const& modes = c.exts[size_t(k)].modes;
        for (size_t i = 1; i < modes.size(); ++i) {
            if (modes[i] <= modes[i - 1]) throw ir_error("row chain: an input is permuted");
        }
        is_vec[size_t(k)] = !modes.empty() && modes.back() == R - 1;
        if (c.exts[size_t(k)].dtype == dtype_t::c64) throw ir_error("row chain: complex input");
    }
    int vcap = max_vec;
    bool any_vec = false;
    for (int t = 0; t != NS; ++t) {
        auto const& st = c.stages[size_t(t)];
        result[size_t(t)] = st.join.out_dtype();
        if (result[size_t(t)] == dtype_t::c64) throw ir_error("row chain: complex stage");
        if (int(st.args.size()) != st.join.num_inputs()) throw ir_error("row chain: argument count");
        bool const last = t + 1 == NS;
        if (last && st.castable) throw ir_error("row chain: the last stage writes the tensor");
        int smallest = int(dtype_size(result[size_t(t)]));
        for (size_t h = 0; h != st.args.size(); ++h) {
            int const a = st.args[h];
            if (a >= NE || a < -t) throw ir_error("row chain: argument out of range");
            if (!st.join.hole_dtypes[h]) throw ir_error("row chain: unused argument");
            dtype_t const d = a >= 0 ? c.exts[size_t(a)].dtype : result[size_t(-1 - a)];
            if (d != st.join.hole_dtypes[h].value()) throw ir_error("row chain: argument dtype");
            if (a >= 0 && is_vec[size_t(a)]) {
                if (!st.castable && !last) throw ir_error("row chain: a per-row step reads a whole row");
                any_vec = true;
            }
            smallest = std::min(smallest, int(dtype_size(d)));
        }
        // the width the stage's own kernel would use (gen_reduce_row); stages that add must
        // agree in it, the others do not care
        if (st.castable) vcap = std::min(vcap, row_reduction_lane_elems(smallest));
    }
    if (!any_vec) throw ir_error("row chain: no stage reads a row");
    for (int k = 0; k != NE; ++k) {
        if (is_vec[size_t(k)] && dtype_size(c.exts[size_t(k)].dtype) == 8) vcap = std::min(vcap, 2);
    }
    int const V = pow2_divisor(n, std::max(1, vcap));
    for (int t = 0; t != NS; ++t) {
        auto const& st = c.stages[size_t(t)];
        if (!st.castable) continue;
        int smallest = int(dtype_size(result[size_t(t)]));
        for (int a : st.args) {
            smallest = std::min(smallest, int(dtype_size(a >= 0 ? c.exts[size_t(a)].dtype
                                                                  : result[size_t(-1 - a)])));
        }
        if (pow2_divisor(n, std::min(max_vec, row_reduction_lane_elems(smallest))) != V) {
            throw ir_error("row chain: stages deal a row to the lanes differently");
        }
    }
    uint64_t const nvec = n / uint64_t(V);
    int const      TEAM = env_int("ES_KM_RED_TEAM", (nvec >= 512) ? 256 : 64) == 256 ? 256 : 64;
    int const      BLOCK = 256;
    uint64_t const vpl = (nvec + uint64_t(TEAM) - 1) / uint64_t(TEAM);
    if (vpl > 8) throw ir_error("row chain: the row does not fit the team's registers");
    int const VPL = int(vpl);
    uint64_t regs = 0;
    for (int k = 0; k != NE; ++k) {
        if (is_vec[size_t(k)]) regs += uint64_t(VPL) * uint64_t(V) * dtype_size(c.exts[size_t(k)].dtype) / 4;
    }
    if (regs > 128) throw ir_error("row chain: the row does not fit the team's registers");
    // (a row reduction with fewer than 1024 rows of 16 steps and more is cut into slices)
    if (TEAM == 256 && n_rows < 1024 && nvec >= uint64_t(TEAM) * 4 * 16) {
        throw ir_error("row chain: the reduction would be split");
    }

    cg_kernel_t k;
    k.kind = cg_kind::row_chain;
    k.n_inns = NE;
    k.vec = V;
    uint64_t biggest = n_rows * n;
    for (int e = 0; e != NE; ++e) {
        uint64_t ne = 1;
        for (int m : c.exts[size_t(e)].modes) ne *= c.shape[size_t(m)];
        biggest = std::max(biggest, ne);
    }
    k.idx64 = biggest >= (1ull << 32) - 1;
    auto param = [&](uint64_t v) {
        k.params.push_back(v);
        return "a.p[" + std::to_string(k.params.size() - 1) + "]";
    };
    std::string const p_rows = param(n_rows), p_nvec = param(nvec), p_n = param(n);
    std::vector<std::string> p_shape(static_cast<size_t>(R));
    for (int m = 0; m != R; ++m) p_shape[size_t(m)] = param(c.shape[size_t(m)]);
    std::vector<std::vector<std::string>> p_str(static_cast<size_t>(NE));
    for (int e = 0; e != NE; ++e) {
        auto const& modes = c.exts[size_t(e)].modes;
        p_str[size_t(e)].assign(size_t(R), "");
        uint64_t stride = 1;
        for (int i = int(modes.size()) - 1; i >= 0; --i) {
            p_str[size_t(e)][size_t(modes[size_t(i)])] = param(stride);
            stride *= c.shape[size_t(modes[size_t(i)])];
        }
    }

    // the name: the stages' joins and castables, the shape's rank and the dtypes
    {
        uint32_t h = 2166136261u;
        auto mix = [&](std::string const& text) {
            for (char ch : text) h = (h ^ uint8_t(ch)) * 16777619u;
        };
        for (auto const& st : c.stages) {
            mix(st.join.str());
            mix(std::string(1, castable_to_char(st.castable)));
            for (int a : st.args) mix(std::to_string(a) + ",");
        }
        for (auto const& e : c.exts) {
            mix(dtype_name(e.dtype));
            for (int m : e.modes) mix(std::to_string(m) + ".");
        }
        char buf[96];
        std::snprintf(buf, sizeof(buf), "es_rowchain__%dstages_%dinputs__%s_%08x", NS, NE,
                      dtype_name(result[size_t(NS - 1)]), h);
        k.entry = buf;
    }

    std::ostringstream s;
    s << PRELUDE;
    s << "typedef " << (k.idx64 ? "unsigned long long" : "unsigned int") << " idx_t;\n";
    for (int t = 0; t != NS; ++t) {
        auto const& st = c.stages[size_t(t)];
        emitter_t   em;
        std::string r = em.emit(st.join.root);
        s << "__device__ __forceinline__ " << compute_type(result[size_t(t)]) << " join_fn" << t << "(";
        for (int i = 0; i != st.join.num_inputs(); ++i) {
            s << (i ? ", " : "") << compute_type(st.join.hole_dtypes[size_t(i)].value()) << " x" << i;
        }
        s << ")\n{\n" << em.body.str() << "    return " << r << ";\n}\n";
        if (st.castable) {
            std::string const ACC = compute_type(result[size_t(t)]);
            s << "__device__ __forceinline__ " << ACC << " comb" << t << "(" << ACC << " x, " << ACC
              << " y) { return " << combine_expr(st.castable.value(), result[size_t(t)], "x", "y")
              << "; }\n";
        }
    }
    dtype_t const od = result[size_t(NS - 1)];
    s << "struct args_t {\n    " << storage_type(od) << "* out;\n";
    for (int e = 0; e != NE; ++e) {
        s << "    const " << storage_type(c.exts[size_t(e)].dtype) << "* in" << e << ";\n";
    }
    s << "    idx_t p[" << k.params.size() << "];\n};\n";
    s << "#define V " << V << "\n#define TEAM " << TEAM << "\n#define VPL " << VPL << "\n";
    s << "extern \"C\" __global__ __launch_bounds__(" << BLOCK << ") void " << k.entry << "(args_t a)\n{\n";
    s << "    const unsigned lane = threadIdx.x % TEAM;\n";
    s << "    const idx_t row = ((idx_t)blockIdx.y * gridDim.x + blockIdx.x) * (" << BLOCK
      << " / TEAM) + threadIdx.x / TEAM;\n";
    // (with a team of 256 the workgroup holds one row: all of it leaves, or none)
    s << "    if (row >= " << p_rows << ") return;\n";
    s << "    const idx_t nvec = " << p_nvec << ";\n";
    s << "    idx_t rem = row;\n";
    for (int m = O - 1; m >= 1; --m) {
        s << "    const idx_t d" << m << " = rem % " << p_shape[size_t(m)] << ";\n";
        s << "    rem /= " << p_shape[size_t(m)] << ";\n";
    }
    if (O >= 1) s << "    const idx_t d0 = rem;\n";
    for (int e = 0; e != NE; ++e) {
        std::string off = "0";
        for (int m = 0; m != O; ++m) {
            if (!p_str[size_t(e)][size_t(m)].empty()) {
                off += " + d" + std::to_string(m) + " * " + p_str[size_t(e)][size_t(m)];
            }
        }
        s << "    const idx_t b" << e << " = " << off << ";\n";
        std::string const T = storage_type(c.exts[size_t(e)].dtype);
        if (is_vec[size_t(e)]) {
            s << "    vec_t<" << T << ", V> r" << e << "[VPL];\n";
        } else {
            s << "    const " << compute_type(c.exts[size_t(e)].dtype) << " c" << e << " = cvt_in(a.in"
              << e << "[b" << e << "]);\n";
        }
    }
    // Streaming loads and stores.  A tensor of the 256 MiB memory-side cache's size or more
    // is read past the caches (its lines would still be there when the result is stored, and
    // their write-back would fall into the next node: gen_elementwise); the result is stored
    // past them only if it is larger than that cache -- one that fits is what the next node
    // reads (the LLaMA layer's 256 MiB of probabilities: the product behind the softmax 71
    // against 98 us).  An input the rows share (a mask) always takes the caches.
    // ES_KM_CHAIN_NT: 1 loads and stores, 2 loads only, 3 stores only, 4 none.
    uint64_t const out_bytes = n_rows * n * dtype_size(od);
    std::vector<bool> whole(static_cast<size_t>(NE), false);
    for (int e = 0; e != NE; ++e) {
        uint64_t ne = 1;
        for (int m : c.exts[size_t(e)].modes) ne *= c.shape[size_t(m)];
        whole[size_t(e)] = ne == n_rows * n;
    }
    bool const stream_in = out_bytes >= (256ull << 20);
    bool const stream_out = out_bytes > (256ull << 20);
    int const  nt_mode = env_int("ES_KM_CHAIN_NT", stream_out ? 1 : (stream_in ? 2 : 4));
    int const  NT_LD = (nt_mode == 1 || nt_mode == 2) ? 1 : 0;
    int const  NT_ST = (nt_mode == 1 || nt_mode == 3) ? 1 : 0;
    // every load of the row before anything is stored: the output may lie on an input
    // Rows that fill every lane's vectors need no tests: the stages are then one straight
    // piece of code, and what two of them compute alike (softmax: exp(x - max), for the sum
    // and again for the quotient) the compiler computes once.
    bool const        full_rows = nvec == uint64_t(TEAM) * uint64_t(VPL);
    std::string const in_row = full_rows ? "true" : "vv < nvec";
    s << "#pragma unroll\n    for (int i = 0; i != VPL; ++i) {\n";
    s << "        const idx_t vv = lane + (idx_t)i * TEAM;\n";
    s << "        if (" << in_row << ") {\n";
    for (int e = 0; e != NE; ++e) {
        if (!is_vec[size_t(e)]) continue;
        std::string const T = storage_type(c.exts[size_t(e)].dtype);
        s << "            r" << e << "[i] = ldv<" << (whole[size_t(e)] ? NT_LD : 0)
          << ">(reinterpret_cast<const vec_t<" << T << ", V>*>(a.in" << e << " + (b" << e
          << " + vv * V)));\n";
    }
    s << "        }\n    }\n";
    auto call = [&](int t, std::string const& i, std::string const& j) {
        auto const& st = c.stages[size_t(t)];
        std::string x = "join_fn" + std::to_string(t) + "(";
        for (size_t h = 0; h != st.args.size(); ++h) {
            int const a = st.args[h];
            x += h ? ", " : "";
            if (a < 0) {
                x += "s" + std::to_string(-1 - a);
            } else if (is_vec[size_t(a)]) {
                x += "cvt_in(r" + std::to_string(a) + "[" + i + "].v[" + j + "])";
            } else {
                x += "c" + std::to_string(a);
            }
        }
        return x + ")";
    };
    auto rounded = [&](dtype_t d, std::string const& v) {
        // through the dtype a kernel of its own would have stored it in
        return d == dtype_t::f16 ? "(float)(f16)(" + v + ")" : v;
    };
    if (TEAM == 256) s << "    __shared__ double part[" << NS << "][4];\n";
    for (int t = 0; t + 1 != NS; ++t) {
        auto const&       st = c.stages[size_t(t)];
        std::string const ACC = compute_type(result[size_t(t)]);
        std::string const T = std::to_string(t);
        if (!st.castable) {
            s << "    const " << ACC << " s" << T << " = " << rounded(result[size_t(t)], call(t, "0", "0"))
              << ";\n";
            continue;
        }
        s << "    " << ACC << " acc" << T << " = " << identity_of(st.castable.value(), result[size_t(t)])
          << ";\n";
        s << "#pragma unroll\n    for (int i = 0; i != VPL; ++i) {\n";
        s << "        const idx_t vv = lane + (idx_t)i * TEAM;\n";
        s << "        if (" << in_row << ") {\n";
        s << "#pragma unroll\n            for (int j = 0; j != V; ++j) acc" << T << " = comb" << T << "(acc"
          << T << ", " << call(t, "i", "j") << ");\n";
        s << "        }\n    }\n";
        s << "#pragma unroll\n    for (int m = 32; m >= 1; m >>= 1) acc" << T << " = comb" << T << "(acc" << T
          << ", lane_xor(acc" << T << ", m));\n";
        if (TEAM == 256) {
            s << "    if ((threadIdx.x & 63) == 0) part[" << T << "][threadIdx.x >> 6] = acc" << T << ";\n";
            s << "    __syncthreads();\n";
            s << "    acc" << T << " = comb" << T << "(comb" << T << "((" << ACC << ")part[" << T << "][0], ("
              << ACC << ")part[" << T << "][1]), comb" << T << "((" << ACC << ")part[" << T << "][2], ("
              << ACC << ")part[" << T << "][3]));\n";
        }
        s << "    const " << ACC << " s" << T << " = " << rounded(result[size_t(t)], "acc" + T) << ";\n";
    }
    s << "#pragma unroll\n    for (int i = 0; i != VPL; ++i) {\n";
    s << "        const idx_t vv = lane + (idx_t)i * TEAM;\n";
    s << "        if (" << in_row << ") {\n";
    s << "            vec_t<" << storage_type(od) << ", V> o;\n";
    s << "#pragma unroll\n            for (int j = 0; j != V; ++j) o.v[j] = "
      << (od == dtype_t::f16 ? "(f16)(" : "(") << call(NS - 1, "i", "j") << ");\n";
    s << "            stv<" << NT_ST << ">(reinterpret_cast<vec_t<" << storage_type(od)
      << ", V>*>(a.out + (row * " << p_n << " + vv * V)), o);\n";
    s << "        }\n    }\n}\n";

    k.source = s.str();
    uint64_t const rows_per_block = uint64_t(BLOCK / TEAM);
    k.grid = (n_rows + rows_per_block - 1) / rows_per_block;
    k.block = unsigned(BLOCK);
    k.out_inn_align.push_back(std::min(16, V * int(dtype_size(od))));
    for (int e = 0; e != NE; ++e) {
        k.out_inn_align.push_back(
            std::min(16, (is_vec[size_t(e)] ? V : 1) * int(dtype_size(c.exts[size_t(e)].dtype))));
    }
    return k;
}

cg_kernel_t generate_kernel(einsummable_t const& e, int max_vec)
{
    if (e.join_shape.size() > 12 || e.inns.size() > 8) {
        throw ir_error("generate_kernel: too many modes or inputs");
    }
    for (int op = 0; op <= int(e.inns.size()); ++op) {
        if (e.stored_as_half_pairs(op) &&
            (op == 0 ? e.out_dtype() : e.inn_dtype(op - 1)) != dtype_t::c64) {
            throw ir_error("generate_kernel: only complex tensors are kept as f16 pairs");
        }
    }
    if (!e.has_aggregation()) return gen_elementwise(e, max_vec);
    if (e.any_half_pairs()) throw ir_error("generate_kernel: f16 pairs in a reduction");
    if (e.out_dtype() == dtype_t::c64 &&
        (e.castable.value() == castable_t::min || e.castable.value() == castable_t::max)) {
        throw ir_error("generate_kernel: min/max aggregation of complex values");
    }
    return is_row_reduction(e) ? gen_reduce_row(e, max_vec) : gen_reduce_col(e, max_vec);
}

cg_kernel_t generate_row_chain(cg_chain_t const& c, int max_vec) { return gen_row_chain(c, max_vec); }

bool is_row_reduction(einsummable_t const& e)
{
    if (!e.has_aggregation()) return false;
    int const R = int(e.join_shape.size());
    for (int k = 0; k != int(e.inns.size()); ++k) {
        if (!e.inns[k].empty() && e.inns[k].back() == R - 1) return true;
    }
    return false;
}

// The options every generated kernel is compiled with; the on-disk cache keys on this very
// list.
std::vector<std::string> compile_options(std::string const& arch)
{
    return {"--offload-arch=" + arch, "-O3",     "-std=c++17",       "-Xclang",
            "-target-feature",        "-Xclang", "-packed-fp32-ops", "-ffp-contract=off"};
}

std::vector<char> compile_hip_source(std::string const& source, std::string const& name,
                                     std::string const& arch)
{
    hiprtcProgram prog;
    if (hiprtcCreateProgram(&prog, source.c_str(), name.c_str(), 0, nullptr, nullptr) !=
        HIPRTC_SUCCESS) {
        throw km_error(km_status::device, "hiprtcCreateProgram failed");
    }
    // packed-fp32 instruction selection is switched off for all device code of this library.
    // No contraction of a product and a sum into a fused multiply-add: every node of a join
    // rounds by itself, as the reference's interpreter does, and -- what matters when the
    // exec graph merges two einsummables into one kernel -- the same expression gives the same
    // bits in whatever kernel it ends up (left to the compiler, 1.7 * x + y became an FMA in
    // a kernel of its own and a product and a sum inside a larger join).
    std::vector<std::string> const options = compile_options(arch);
    std::vector<const char*>       opts;
    for (std::string const& o : options) opts.push_back(o.c_str());
    int const n_opts = int(opts.size());
    hiprtcResult rc = hiprtcCompileProgram(prog, n_opts, opts.data());
    if (rc != HIPRTC_SUCCESS) {
        size_t n = 0;
        hiprtcGetProgramLogSize(prog, &n);
        std::string log(n, 0);
        if (n) hiprtcGetProgramLog(prog, &log[0]);
        hiprtcDestroyProgram(&prog);
        throw km_error(km_status::device, "runtime compile of " + name + " failed:\n" + log +
                                              "\n---- source ----\n" + source);
    }
    size_t n = 0;
    hiprtcGetCodeSize(prog, &n);
    std::vector<char> code(n);
    hiprtcGetCode(prog, code.data());
    hiprtcDestroyProgram(&prog);
    return code;
}

// ---------------------------------------------------------------------------- the plan

namespace
{

// ---- code objects on disk.  A runtime compile costs a good part of a second per kernel, and
// a server process builds the same einsummables every time it starts.  The code object of a
// source is kept in a file named by a 128-bit hash of (runtime-compiler version, options,
// source); the file holds that whole text in front of the code object and a hit is one whose
// text is the same, byte for byte.  ES_KM_CACHE_DIR names the directory ("off" or "" switches the cache off);
// by default it is $XDG_CACHE_HOME/es_km or $HOME/.cache/es_km.  Files are written under a
// temporary name and renamed, so concurrent processes never see half a file.

std::string cache_dir()
{
    const char* env = std::getenv("ES_KM_CACHE_DIR");
    if (env) {
        std::string d = env;
        if (d.empty() || d == "off" || d == "0") return "";
        return d;
    }
    if (const char* x = std::getenv("XDG_CACHE_HOME")) {
        if (*x) return std::string(x) + "/es_km";
    }
    if (const char* h = std::getenv("HOME")) {
        if (*h) return std::string(h) + "/.cache/es_km";
    }
    return "";
}

uint64_t fnv1a(std::string const& text, uint64_t h)
{
    for (unsigned char c : text) {
        h ^= c;
        h *= 1099511628211ull;
    }
    return h;
}

std::string cache_text(std::string const& source)
{
    // the compiler that would compile it: its version as the library reports it, the
    // runtime's full version number (patch level included) and the build the headers of this
    // library came from
    int major = 0, minor = 0, runtime = 0;
    hiprtcVersion(&major, &minor);
    (void)hipRuntimeGetVersion(&runtime);
    std::string text = "hiprtc " + std::to_string(major) + "." + std::to_string(minor) +
                       " runtime " + std::to_string(runtime) + " headers " +
                       std::to_string(HIP_VERSION) + " " + HIP_VERSION_GITHASH + "\n";
    for (std::string const& o : compile_options("gfx950")) text += o + " ";
    return text + "\n" + source;
}

std::string cache_file(std::string const& dir, std::string const& text)
{
    char name[64];
    std::snprintf(name, sizeof(name), "%016llx%016llx.co",
                  (unsigned long long)fnv1a(text, 14695981039346656037ull),
                  (unsigned long long)fnv1a(text, 0x9e3779b97f4a7c15ull));
    return dir + "/" + name;
}

struct cache_header_t {
    char     magic[8];  // "ESKMCO2\0"
    uint64_t text_bytes;
    uint64_t code_bytes;
};

bool read_cached(std::string const& path, std::string const& text, std::vector<char>& code)
{
    std::FILE* f = std::fopen(path.c_str(), "rb");
    if (!f) return false;
    cache_header_t h;
    bool           ok = std::fread(&h, sizeof(h), 1, f) == 1 &&
              std::memcmp(h.magic, "ESKMCO2", 8) == 0 && h.text_bytes == text.size() &&
              h.code_bytes > 0 && h.code_bytes < (1ull << 30);
    if (ok) {
        // two texts with one hash would share a file name: the text itself decides
        std::string stored(text.size(), 0);
        ok = std::fread(&stored[0], 1, stored.size(), f) == stored.size() && stored == text;
    }
    if (ok) {
        code.resize(size_t(h.code_bytes));
        ok = std::fread(code.data(), 1, code.size(), f) == code.size() && std::fgetc(f) == EOF;
    }
    std::fclose(f);
    return ok;
}

void write_cached(std::string const& dir, std::string const& path, std::string const& text,
                  std::vector<char> const& code)
{
    // failures only mean that the next process compiles again
    for (size_t at = dir.find('/', 1); at != std::string::npos; at = dir.find('/', at + 1)) {
        ::mkdir(dir.substr(0, at).c_str(), 0755);
    }
    ::mkdir(dir.c_str(), 0755);
    std::string tmp = path + ".tmp" + std::to_string(long(::getpid()));
    std::FILE*  f = std::fopen(tmp.c_str(), "wb");
    if (!f) return;
    cache_header_t h;
    std::memcpy(h.magic, "ESKMCO2", 8);
    h.text_bytes = text.size();
    h.code_bytes = code.size();
    bool ok = std::fwrite(&h, sizeof(h), 1, f) == 1 &&
              std::fwrite(text.data(), 1, text.size(), f) == text.size() &&
              std::fwrite(code.data(), 1, code.size(), f) == code.size();
    ok = (std::fclose(f) == 0) && ok;
    if (!ok || std::rename(tmp.c_str(), path.c_str()) != 0) std::remove(tmp.c_str());
}

}  // namespace

std::vector<char> code_object_for(std::string const& source, bool* from_disk)
{
    if (from_disk) *from_disk = false;
    std::string const dir = cache_dir();
    if (dir.empty()) return compile_hip_source(source, "es_generated.hip", "gfx950");
    std::string const text = cache_text(source);
    std::string const path = cache_file(dir, text);
    std::vector<char> code;
    if (read_cached(path, text, code)) {
        if (from_disk) *from_disk = true;
        return code;
    }
    code = compile_hip_source(source, "es_generated.hip", "gfx950");
    write_cached(dir, path, text, code);
    return code;
}

namespace
{

// Loaded modules of this process, one per (device, source): a module belongs to the device
// that was current when it was loaded.
struct loaded_t {
    hipModule_t mod;
    std::string suffix;  // appended to the source's entry points (programs compiled together)
};
struct module_cache_t {
    std::mutex                                      mu;
    std::map<std::pair<int, std::string>, loaded_t> by_source;
};

module_cache_t& module_cache()
{
    static module_cache_t c;
    return c;
}

struct variant_t {
    cg_kernel_t   k;
    hipFunction_t fn = nullptr;
    hipFunction_t fn2 = nullptr;  // second pass of a split reduction
};

bool module_loaded(int device, std::string const& source)
{
    auto&                       cache = module_cache();
    std::lock_guard<std::mutex> lock(cache.mu);
    return cache.by_source.count({device, source}) != 0;
}

// Loads the variant's module on `device` (once per distinct source; `code` may be empty when
// the module is known to be loaded, otherwise it is the source's code object) and resolves
// the entry points.
void load_kernel(variant_t& v, int device, std::vector<char> const& code)
{
    auto&                       cache = module_cache();
    std::lock_guard<std::mutex> lock(cache.mu);
    hipModule_t                 mod;
    std::string                 suffix;
    auto                        it = cache.by_source.find({device, v.k.source});
    if (it != cache.by_source.end()) {
        mod = it->second.mod;
        suffix = it->second.suffix;
    } else {
        std::vector<char> compiled;
        if (code.empty()) compiled = code_object_for(v.k.source, nullptr);
        hipError_t err = hipModuleLoadData(&mod, code.empty() ? compiled.data() : code.data());
        if (err != hipSuccess) {
            throw km_error(km_status::device,
                           std::string("hipModuleLoadData: ") + hipGetErrorString(err));
        }
        cache.by_source.emplace(std::make_pair(device, v.k.source), loaded_t{mod, ""});
    }
    auto get = [&](std::string const& base) {
        std::string const name = base + suffix;
        hipFunction_t fn;
        hipError_t    err = hipModuleGetFunction(&fn, mod, name.c_str());
        if (err != hipSuccess) {
            throw km_error(km_status::device,
                           std::string("hipModuleGetFunction: ") + hipGetErrorString(err));
        }
        return fn;
    };
    v.fn = get(v.k.entry);
    if (v.k.splits > 1) v.fn2 = get(v.k.entry2);
}

struct codegen_plan_t : plan_t {
    einsummable_t     e;
    variant_t         wide;
    variant_t         narrow;  // scalar accesses: for buffers that are not 16-byte aligned

    explicit codegen_plan_t(einsummable_t const& e_) : e(e_) {}
    codegen_plan_t() = default;  // a chain of einsummables
    std::string source() const override { return wide.k.source; }
    bool has_narrow = true;
    bool waiting = false;  // the variants' kernels are not loaded yet
    void deferred(std::vector<plan_t*>& out) override
    {
        if (waiting) out.push_back(this);
    }

    static void launch(variant_t const& v, hipStream_t stream, void* out, void const* const* inns,
                       void* workspace)
    {
        // argument block: out pointer, input pointers, (partial results,) idx_t parameters
        unsigned char buf[1024];
        size_t        n = 0;
        std::memcpy(buf + n, &out, 8);
        n += 8;
        for (int i = 0; i != v.k.n_inns; ++i) {
            std::memcpy(buf + n, &inns[i], 8);
            n += 8;
        }
        if (v.k.splits > 1) {
            std::memcpy(buf + n, &workspace, 8);
            n += 8;
        }
        if (v.k.idx64) {
            for (uint64_t p : v.k.params) {
                std::memcpy(buf + n, &p, 8);
                n += 8;
            }
        } else {
            for (uint64_t p : v.k.params) {
                uint32_t q = uint32_t(p);
                std::memcpy(buf + n, &q, 4);
                n += 4;
            }
            n = (n + 7) & ~size_t(7);
        }
        void* config[] = {HIP_LAUNCH_PARAM_BUFFER_POINTER, buf, HIP_LAUNCH_PARAM_BUFFER_SIZE, &n,
                          HIP_LAUNCH_PARAM_END};
        // a grid dimension times the block size must stay below 2^32: fold large grids
        // into two dimensions (the kernels linearise blockIdx.y * gridDim.x + blockIdx.x)
        uint64_t const gx_max = 1ull << 22;
        unsigned gx = unsigned(std::min<uint64_t>(v.k.grid, gx_max));
        unsigned gy = unsigned((v.k.grid + gx - 1) / gx);
        hipError_t err = hipModuleLaunchKernel(v.fn, gx, gy, unsigned(v.k.splits), v.k.block, 1, 1,
                                               0, stream, nullptr, config);
        if (err == hipSuccess && v.k.splits > 1) {
            if (v.k.grid2) {
                gx = unsigned(std::min<uint64_t>(v.k.grid2, gx_max));
                gy = unsigned((v.k.grid2 + gx - 1) / gx);
            }
            err = hipModuleLaunchKernel(v.fn2, gx, gy, 1, v.k.block, 1, 1, 0, stream, nullptr,
                                        config);
        }
        if (err != hipSuccess) {
            throw km_error(km_status::device,
                           std::string("hipModuleLaunchKernel: ") + hipGetErrorString(err));
        }
    }

    static bool aligned(variant_t const& v, void* out, void const* const* inns)
    {
        if (reinterpret_cast<uintptr_t>(out) % uintptr_t(std::min(v.k.out_inn_align[0], 16))) {
            return false;
        }
        for (int i = 0; i != v.k.n_inns; ++i) {
            if (reinterpret_cast<uintptr_t>(inns[i]) %
                uintptr_t(std::min(v.k.out_inn_align[1 + i], 16))) {
                return false;
            }
        }
        return true;
    }

    void run(hipStream_t stream, void* out, void const* const* inns, void* workspace,
             uint64_t) const override
    {
        if (aligned(wide, out, inns)) {
            launch(wide, stream, out, inns, workspace);
            return;
        }
        if (!has_narrow) {
            throw km_error(km_status::invalid,
                           "this kernel needs its buffers aligned to 16 bytes");
        }
        launch(narrow, stream, out, inns, workspace);
    }
};

}  // namespace

std::shared_ptr<plan_t> plan_codegen(einsummable_t const& e, int device, bool defer)
{
    cg_kernel_t k;
    try {
        k = generate_kernel(e);
    } catch (ir_error const&) {
        return nullptr;
    }
    if (k.grid >= (1ull << 36)) return nullptr;
    if (8 * (1 + k.n_inns) + 8 * k.params.size() > 1000) return nullptr;
    auto p = std::make_shared<codegen_plan_t>(e);
    p->wide.k = std::move(k);
    p->narrow.k = generate_kernel(e, 1);
    // Both variants are compiled and loaded at build time -- here, or with the other
    // kernels of the caller's list (finish_codegen_plans): run() only ever launches.
    if (defer) {
        p->waiting = true;
    } else {
        load_kernel(p->wide, device, {});
        load_kernel(p->narrow, device, {});
    }
    switch (p->wide.k.kind) {
        case cg_kind::elementwise:
            p->description = "elementwise";
            break;
        case cg_kind::reduce_row:
            p->description = "reduce_row";
            break;
        case cg_kind::reduce_col:
            p->description = "reduce_col";
            break;
    }
    p->description += " vec=" + std::to_string(p->wide.k.vec);
    if (p->wide.k.idx64) p->description += " idx64";
    if (p->wide.k.row_pairs) p->description += " row_pairs";
    if (p->wide.k.splits > 1) p->description += " splits=" + std::to_string(p->wide.k.splits);
    p->workspace_bytes = std::max(p->wide.k.ws_bytes, p->narrow.k.ws_bytes);
    return p;
}

std::shared_ptr<plan_t> plan_row_chain(cg_chain_t const& c, int device, bool defer)
{
    auto p = std::make_shared<codegen_plan_t>();
    p->wide.k = generate_row_chain(c);  // throws ir_error when the chain has no kernel
    if (p->wide.k.grid >= (1ull << 36) ||
        8 * (1 + p->wide.k.n_inns) + 8 * p->wide.k.params.size() > 1000) {
        throw ir_error("row chain: too large");
    }
    try {
        p->narrow.k = generate_row_chain(c, 1);
    } catch (ir_error const&) {
        p->has_narrow = false;  // rows too long for one element per lane and step
    }
    p->n_inns = p->wide.k.n_inns;
    if (device >= 0 && defer) {
        p->waiting = true;
    } else if (device >= 0) {
        load_kernel(p->wide, device, {});
        if (p->has_narrow) load_kernel(p->narrow, device, {});
    }
    p->description = "row_chain stages=" + std::to_string(c.stages.size()) +
                     " vec=" + std::to_string(p->wide.k.vec);
    if (p->wide.k.idx64) p->description += " idx64";
    return p;
}

void finish_codegen_plans(std::vector<plan_t*> const& plans, int device)
{
    std::vector<codegen_plan_t*> ps;
    for (plan_t* p : plans) {
        if (auto* c = dynamic_cast<codegen_plan_t*>(p)) ps.push_back(c);
    }
    if (ps.empty()) return;
    // the distinct sources that no module of this device holds yet, in order of appearance
    std::vector<variant_t*> fresh;
    {
        std::set<std::string> seen;
        for (codegen_plan_t* p : ps) {
            for (variant_t* v : {&p->wide, &p->narrow}) {
                if (v == &p->narrow && !p->has_narrow) continue;
                if (seen.count(v->k.source) || module_loaded(device, v->k.source)) continue;
                seen.insert(v->k.source);
                fresh.push_back(v);
            }
        }
    }
    if (fresh.size() > 1) {
        // One program: the prelude once, every kernel's own text (its join function, argument
        // block and entry points share their names with the others') in a namespace of its
        // own, the entry points, which have C linkage, told apart by a suffix.
        size_t const pre = std::strlen(PRELUDE);
        std::string  text = PRELUDE;
        for (size_t i = 0; i != fresh.size(); ++i) {
            cg_kernel_t const& k = fresh[i]->k;
            if (k.source.compare(0, pre, PRELUDE) != 0) {
                throw km_error(km_status::invalid, "generated source without its prelude");
            }
            std::string       body = k.source.substr(pre);
            std::string const suffix = "_u" + std::to_string(i);
            for (std::string const& name : {k.entry, k.splits > 1 ? k.entry2 : std::string()}) {
                if (name.empty()) continue;
                std::string const from = name + "(";
                size_t            hits = 0;
                for (size_t at = body.find(from); at != std::string::npos;
                     at = body.find(from, at + from.size() + suffix.size())) {
                    body.insert(at + name.size(), suffix);
                    ++hits;
                }
                if (hits == 0) throw km_error(km_status::invalid, "entry point not found: " + name);
            }
            text += "namespace es_unit_" + std::to_string(i) + "\n{\n" + body + "\n}\n";
        }
        std::vector<char> const code = code_object_for(text, nullptr);
        hipModule_t             mod;
        hipError_t              err = hipModuleLoadData(&mod, code.data());
        if (err != hipSuccess) {
            throw km_error(km_status::device,
                           std::string("hipModuleLoadData: ") + hipGetErrorString(err));
        }
        auto&                       cache = module_cache();
        std::lock_guard<std::mutex> lock(cache.mu);
        for (size_t i = 0; i != fresh.size(); ++i) {
            cache.by_source.emplace(std::make_pair(device, fresh[i]->k.source),
                                    loaded_t{mod, "_u" + std::to_string(i)});
        }
    }
    for (codegen_plan_t* p : ps) {
        load_kernel(p->wide, device, {});
        if (p->has_narrow) load_kernel(p->narrow, device, {});
        p->waiting = false;
    }
}

}  // namespace es
