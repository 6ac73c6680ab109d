// Host-side IR of the apply-node path: dtype / castable / scalarop expression trees,
// einsummable descriptors and touch selections.  Mirrors the data model of
// dcbdan/einsummable (src/einsummable/scalarop.h:4-521, einsummable.h:8-288, touch.h:8-46)
// at the level the kernel manager needs: parse the reference's text forms, type-check,
// normalise (aggregation renumbering, merge_adjacent_dims, touch simplify) and classify.
#pragma once
#include <cstdint>
#include <memory>
#include <optional>
#include <stdexcept>
#include <string>
#include <utility>
#include <vector>

namespace es
{

enum class dtype_t : int { f16 = 0, f32 = 1, f64 = 2, c64 = 3 };
enum class castable_t : int { add = 0, mul = 1, min = 2, max = 3 };
enum class compare_t : int { lt = 0, gt = 1, eq = 2, le = 3, ge = 4 };

uint64_t    dtype_size(dtype_t);
const char* dtype_name(dtype_t);
// '+' 'x' 'v' '^' (scalarop.cc:3078-3093); 0 means "no castable"
std::optional<castable_t> castable_from_char(char c);
char                      castable_to_char(std::optional<castable_t> const&);

// A scalar in the reference's text form, "f32|1.5", "f16|NINF", "c64|(1,2)"
// (scalarop.cc:2720-2830): its dtype and its bytes in the low bytes of a uint64.
struct scalar_bits_t {
    dtype_t  dtype;
    uint64_t bits;
};
scalar_bits_t parse_scalar(std::string const& text);
std::optional<dtype_t> dtype_from_name(std::string const& name);

struct ir_error : std::runtime_error {
    using std::runtime_error::runtime_error;
};

enum class op_kind {
    constant,
    hole,
    variable,
    add,
    mul,
    exp,
    log,
    power,
    ite,
    convert,
    conj,
    real,
    imag,
    cplex
};

// One node of a scalarop expression tree (scalar_ns::node_t, scalarop.h:227-276).
struct node_t {
    op_kind             kind;
    dtype_t             dtype;     // result dtype of this node
    double              re = 0.0;  // constant value, already rounded to `dtype`
    double              im = 0.0;
    int                 arg = -1;  // hole index
    double              power = 0.0;
    compare_t           compare = compare_t::lt;
    std::string         name;  // variable name
    std::vector<node_t> children;
};

struct scalarop_t {
    node_t root;
    // dtype of hole k; nullopt when the expression does not use hole k
    std::vector<std::optional<dtype_t>> hole_dtypes;

    // Parses the reference's operator<< text, e.g.
    //   *[hole|f16@0,power{-1}[+[constant{f16|1},exp[*[constant{f16|-1},hole|f16@0]]]]]
    // (grammar: scalarop.cc:2881-3011).  Throws ir_error on malformed or ill-typed text.
    static scalarop_t parse(std::string const& text);

    // Every variable named in `values` becomes a constant of the variable's dtype
    // (scalarop_t::replace_variables, scalarop.cc; einsummable_t::replace_scalar_variables,
    // einsummable.cc:221-233).  Variables not named stay.
    scalarop_t replace_variables(std::vector<std::pair<std::string, double>> const& values) const;

    // The reference's canonical form (node_t::simplify, scalarop.cc:1233-1416, which every
    // scalarop_t constructor applies, :1942-1948): a subtree without holes and variables
    // becomes one constant -- evaluated in its dtype, printed with six significant digits and
    // read back, as the reference does -- commutative operands and comparisons are ordered by
    // the highest hole they use (normalize_order, :1442-1493, with its habit of turning
    // ite_>[x,c,x,c] into ite_<=[c,x,c,x]), and 0 + x, 0 * x, 1 * x, c0 * (c1 * hole),
    // x ^ 0, x ^ 1, ite with equal arms and conj(conj(x)) fold.  Repeated until nothing
    // changes.  Texts the reference wrote are fixed points; what is not is a join whose
    // variables have just been replaced by constants.
    scalarop_t simplify() const;

    // `outer` with hole k replaced by the whole of `inner`, whose value passes through a
    // conversion to inner's own output dtype first (what a store by one kernel and a load by
    // the next do to it: a rounding for f16, nothing for the other dtypes, where the node
    // still keeps the two expressions apart).  inner's holes keep their numbers; outer's other
    // holes follow them in their old order.  Throws ir_error when the dtypes do not meet.
    static scalarop_t compose(scalarop_t const& outer, int k, scalarop_t const& inner);

    std::string str() const;
    dtype_t     out_dtype() const { return root.dtype; }
    int         num_inputs() const { return int(hole_dtypes.size()); }
    bool        has_variables() const;
    bool        is_identity() const;  // exactly hole@0
    bool        is_mul() const;       // exactly *[hole@0,hole@1]
    // *[hole@0,hole@1], or that product times one real constant on either side (holes in
    // either order); `scale` is the constant, 1 for the plain product
    bool        is_scaled_mul(double& scale) const;
    bool        is_add() const;       // exactly +[hole@0,hole@1]
};

// einsummable_t (einsummable.h:8-288): out modes are 0..out_rank-1, aggregated modes follow.
struct einsummable_t {
    std::vector<uint64_t>         join_shape;
    std::vector<std::vector<int>> inns;
    int                           out_rank = 0;
    scalarop_t                    join;
    std::optional<castable_t>     castable;
    // Not part of the reference's einsummable: [0] the output, [1 + k] input k -- a c64 tensor
    // that lies in memory as pairs of f16 (real, imaginary) and is widened on the load or
    // rounded on the store.  Empty: none.  Set by the exec graph's optimisation pass where a
    // conversion node stood between an f16 tensor and its view as complex numbers (rotary
    // embeddings: to_f32, the c64 product on the reinterpreted buffer, to_f16); only the
    // generated elementwise kernels take such an einsummable.
    std::vector<char>             half_complex;
    bool stored_as_half_pairs(int operand) const
    {
        return size_t(operand) < half_complex.size() && half_complex[size_t(operand)] != 0;
    }
    bool any_half_pairs() const
    {
        for (char c : half_complex) {
            if (c) return true;
        }
        return false;
    }

    // Runs the checks and the aggregation-mode renumbering of the reference constructor
    // (einsummable.cc:32-93).  Throws ir_error when invalid.
    static einsummable_t make(std::vector<uint64_t> join_shape, std::vector<std::vector<int>> inns,
                              int out_rank, scalarop_t join, std::optional<castable_t> castable);

    // Fuse modes that are adjacent in every term (einsummable.cc:166-218).
    einsummable_t merge_adjacent_dims() const;

    std::string str() const;  // "ab,bc->ac"
    // canonical lookup key: shape, modes, join text and castable
    std::string key() const;

    bool     has_aggregation() const { return out_rank < int(join_shape.size()); }
    bool     has_broadcast() const;
    bool     is_straight_elementwise() const;
    bool     is_permutation() const;
    bool     is_contraction() const;
    // is_contraction() with is_scaled_mul() in place of is_mul(): a product whose result is
    // multiplied by a constant once, after the sum (the reference has no such form: it runs
    // the scale as a node of its own, or passes it as cuTENSOR's alpha,
    // gpu_kernel_manager.cc:1577-1609)
    bool     is_scaled_contraction(double& scale) const;
    dtype_t  out_dtype() const { return join.out_dtype(); }
    dtype_t  inn_dtype(int k) const { return join.hole_dtypes[k].value(); }
    uint64_t out_nelem() const;
    uint64_t inn_nelem(int k) const;
};

struct touchdim_t {
    uint64_t d_inn, d_out, offset_inn, offset_out, size;
};

struct touch_t {
    std::vector<touchdim_t>   selection;
    std::optional<castable_t> castable;
    dtype_t                   dtype;

    // Merge trailing dimensions that are copied in full into their predecessor
    // (touch.cc:3-28).
    touch_t simplify() const;
    // throws ir_error if a window leaves its tensor or the selection is empty
    void validate() const;
};

}  // namespace es
