// Index-expression front end: parser, validator, C emitter and affine
// classifier for the strings that reindex / reindex_reduce take.
//
// The language is "C integer expressions" (reference:
// python/jittor/src/ops/reindex_op.h:58-68 for the names,
// python/jittor/src/opt/expr.cc:16-52 for the operator table,
// python/jittor/src/op_compiler.cc:665-699 for @eK(...)).
#pragma once
#include <memory>
#include <string>
#include <vector>
#include <cstdint>

namespace mjt {

struct Expr {
    enum Kind { CONST_INT, CONST_FLOAT, VAR, UNARY, BINARY, TERNARY, EXTRA, CAST } kind;
    int64_t ival = 0;          // CONST_INT
    std::string text;          // CONST_FLOAT literal, VAR name, operator, CAST type
    int extra = -1;            // EXTRA: K of @eK
    std::vector<std::unique_ptr<Expr>> kids;
};

// Throws mjt::Error (MJT_ERR_INVALID) on a syntax error.
std::unique_ptr<Expr> parse_expr(const std::string& s);

struct ExprEnv {
    int n_loop = 0;                 // i0..i{n_loop-1} are defined
    int xdim = 0, ydim = 0;         // XDIM / YDIM, xshapeK / yshapeK ...
    std::vector<int> extra_rank;    // rank of extras[K]
};
// Checks every identifier and @eK arity against the environment.
void validate_expr(const Expr& e, const ExprEnv& env);

// C source for the expression.  Names are emitted as they are (the kernel
// defines i0.., xshapeK, yshapeK, xstrideK, ystrideK, XDIM, YDIM); @eK(a,b)
// becomes eKp[(a)*eKstride0+(b)*eKstride1].
std::string emit_c(const Expr& e);

// True when the expression contains no @eK load.
bool is_pure(const Expr& e);

// Affine analysis: value == c0 + sum coef[k] * i_k for all coordinates.
// xshape/yshape give the values of xshapeK / yshapeK (strides are derived).
struct Affine {
    int64_t c0 = 0;
    int64_t coef[10] = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
};
bool affine_of(const Expr& e, const std::vector<int64_t>& xshape, const std::vector<int64_t>& yshape, Affine* out);

}  // namespace mjt
