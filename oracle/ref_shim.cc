// extern "C" driver over the reference's own scalarop_t and permute_t, compiled from the
// sources where they lie in the reference tree (see Makefile, target _ref/libes_ref.so).
// TEST INFRASTRUCTURE ONLY: it pins the C oracle's scalarop parser / printer / per-op
// arithmetic and permute semantics against the real reference implementation.  Nothing in
// this file restates reference logic; it only marshals arguments.
#include "src/base/permute.h"
#include "src/einsummable/scalarop.h"

#include <cstring>
#include <sstream>

static thread_local std::string g_err;

static int copy_out(std::string const& s, char* out, size_t cap)
{
    if (s.size() + 1 > cap) {
        g_err = "buffer too small";
        return -1;
    }
    std::memcpy(out, s.c_str(), s.size() + 1);
    return 0;
}

static scalar_t scalar_from_bits(dtype_t d, uint64_t bits)
{
    scalar_t s;
    s.dtype = d;
    std::memcpy(s.data, &bits, 8);
    return s;
}

extern "C" {

const char* es_ref_last_error() { return g_err.c_str(); }

// parse then print
int es_ref_scalarop_roundtrip(const char* text, char* out, size_t cap)
{
    try {
        scalarop_t op = parse_with_ss<scalarop_t>(text);
        return copy_out(write_with_ss(op), out, cap);
    } catch (std::exception const& e) {
        g_err = e.what();
        return -1;
    }
}

// parse, simplify, print
int es_ref_scalarop_simplify(const char* text, char* out, size_t cap)
{
    try {
        scalarop_t op = parse_with_ss<scalarop_t>(text);
        return copy_out(write_with_ss(op.simplify()), out, cap);
    } catch (std::exception const& e) {
        g_err = e.what();
        return -1;
    }
}

// evaluate at one point; values travel as raw bit patterns in a uint64_t
int es_ref_scalarop_eval(const char* text, int n_inputs, const uint64_t* input_bits,
                         uint64_t* out_bits, int* out_dtype)
{
    try {
        scalarop_t       op = parse_with_ss<scalarop_t>(text);
        vector<scalar_t> inputs;
        for (int i = 0; i != n_inputs; ++i) {
            auto maybe = op.inn_dtype(i);
            dtype_t d = maybe ? maybe.value() : dtype_t::f32;
            inputs.push_back(scalar_from_bits(d, input_bits[i]));
        }
        scalar_t r = op.eval(inputs);
        *out_bits = 0;
        std::memcpy(out_bits, r.data, dtype_size(r.dtype));
        *out_dtype = int(r.dtype);
        return 0;
    } catch (std::exception const& e) {
        g_err = e.what();
        return -1;
    }
}

// evaluate a unary op over n f16 inputs given as bit patterns (for exhaustive sweeps)
int es_ref_scalarop_map_f16_unary(const char* text, const uint16_t* x, uint64_t n, uint16_t* out)
{
    try {
        scalarop_t op = parse_with_ss<scalarop_t>(text);
        for (uint64_t i = 0; i != n; ++i) {
            scalar_t r = op.eval({scalar_from_bits(dtype_t::f16, x[i])});
            std::memcpy(out + i, r.data, 2);
        }
        return 0;
    } catch (std::exception const& e) {
        g_err = e.what();
        return -1;
    }
}

// binary op over n f16 pairs
int es_ref_scalarop_map_f16_binary(const char* text, const uint16_t* x, const uint16_t* y,
                                   uint64_t n, uint16_t* out)
{
    try {
        scalarop_t op = parse_with_ss<scalarop_t>(text);
        for (uint64_t i = 0; i != n; ++i) {
            scalar_t r = op.eval(
                {scalar_from_bits(dtype_t::f16, x[i]), scalar_from_bits(dtype_t::f16, y[i])});
            std::memcpy(out + i, r.data, 2);
        }
        return 0;
    } catch (std::exception const& e) {
        g_err = e.what();
        return -1;
    }
}

// the make_* constructors whose canonical text the configs rely on
int es_ref_scalarop_make(const char* which, int dtype, char* out, size_t cap)
{
    try {
        dtype_t     d = dtype_t(dtype);
        std::string w(which);
        scalarop_t  op;
        if (w == "relu") {
            op = scalarop_t::make_relu(d);
        } else if (w == "silu") {
            op = scalarop_t::make_silu(d);
        } else if (w == "sub") {
            op = scalarop_t::make_sub(d);
        } else if (w == "div") {
            op = scalarop_t::make_div(d);
        } else if (w == "max") {
            op = scalarop_t::make_max(d);
        } else if (w == "min") {
            op = scalarop_t::make_min(d);
        } else if (w == "exp") {
            op = scalarop_t::make_exp(d);
        } else if (w == "square") {
            op = scalarop_t::make_square(d);
        } else if (w == "inverse_sqrt") {
            op = scalarop_t::make_inverse_sqrt(d);
        } else if (w == "sigmoid") {
            op = scalarop_t::make_sigmoid(d);
        } else if (w == "neg") {
            op = scalarop_t::make_neg(d);
        } else if (w == "relu_mul") {
            op = scalarop_t::combine(scalarop_t::make_mul(d),
                                     {scalarop_t::make_relu(d), scalarop_t::make_identity(d)});
        } else if (w == "exp_sub") {
            op = scalarop_t::combine(scalarop_t::make_exp(d), {scalarop_t::make_sub(d)});
        } else {
            g_err = "unknown constructor";
            return -1;
        }
        return copy_out(write_with_ss(op), out, cap);
    } catch (std::exception const& e) {
        g_err = e.what();
        return -1;
    }
}

// make_scale / make_increment through the 6-significant-digit text path
int es_ref_scalarop_make_scale(int dtype, double value, int increment, char* out, size_t cap)
{
    try {
        dtype_t  d = dtype_t(dtype);
        scalar_t v = scalar_t(d, write_with_ss(value));
        scalarop_t op = increment ? scalarop_t::make_increment(v) : scalarop_t::make_scale(v);
        return copy_out(write_with_ss(op), out, cap);
    } catch (std::exception const& e) {
        g_err = e.what();
        return -1;
    }
}

// permute_t: out_perm = {2,0,1} means ijk->kij.  elem_size in {2,4,8}.
int es_ref_permute(const uint64_t* inn_dims, int rank, const int* out_perm, int elem_size,
                   void* out, const void* inn)
{
    try {
        vector<uint64_t> dims(inn_dims, inn_dims + rank);
        vector<int>      perm(out_perm, out_perm + rank);
        permute_t        p(1024);
        if (elem_size == 2) {
            p(dims, perm, (uint16_t*)out, (uint16_t const*)inn);
        } else if (elem_size == 4) {
            p(dims, perm, (uint32_t*)out, (uint32_t const*)inn);
        } else if (elem_size == 8) {
            p(dims, perm, (uint64_t*)out, (uint64_t const*)inn);
        } else {
            g_err = "bad elem size";
            return -1;
        }
        return 0;
    } catch (std::exception const& e) {
        g_err = e.what();
        return -1;
    }
}
}
