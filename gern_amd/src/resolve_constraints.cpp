// resolve::solve for an equation linear in one variable (see the header; the
// reference's src/resolve_constraints/resolve_constraints.cpp:172-192 hands the
// same job to GiNaC::lsolve).
#include "resolve_constraints/resolve_constraints.h"

#include "utils/error.h"

namespace gern {
namespace resolve {

namespace {

bool isLiteral(const Expr &e, double value) {
    if (!e.defined() || e.ptr->kind != ExprKind::Literal) {
        return false;
    }
    auto n = static_cast<const LiteralNode *>(e.ptr);
    return n->isFloating() ? n->f == value : n->i == (int64_t)value && (double)(int64_t)value == value;
}

bool bothLiterals(const Expr &a, const Expr &b) {
    return a.ptr->kind == ExprKind::Literal && b.ptr->kind == ExprKind::Literal;
}

// a (op) b on two literals: in integers while both are integers and the result is one
Expr fold(ExprKind op, const Expr &a, const Expr &b) {
    auto x = static_cast<const LiteralNode *>(a.ptr), y = static_cast<const LiteralNode *>(b.ptr);
    const bool whole = !x->isFloating() && !y->isFloating();
    switch (op) {
    case ExprKind::Add:
        return whole ? Expr(x->i + y->i) : Expr(x->f + y->f);
    case ExprKind::Sub:
        return whole ? Expr(x->i - y->i) : Expr(x->f - y->f);
    case ExprKind::Mul:
        return whole ? Expr(x->i * y->i) : Expr(x->f * y->f);
    default:  // Div
        if (whole && y->i != 0 && x->i % y->i == 0) {
            return Expr(x->i / y->i);
        }
        return Expr(x->f / y->f);
    }
}

Expr negated(const Expr &literal) {
    auto n = static_cast<const LiteralNode *>(literal.ptr);
    return n->isFloating() ? Expr(-n->f) : Expr(-n->i);
}

bool isNegativeLiteral(const Expr &e) {
    if (e.ptr->kind != ExprKind::Literal) {
        return false;
    }
    auto n = static_cast<const LiteralNode *>(e.ptr);
    return n->isFloating() ? n->f < 0 : n->i < 0;
}

Expr add(const Expr &a, const Expr &b) {
    if (isLiteral(a, 0)) {
        return b;
    }
    if (isLiteral(b, 0)) {
        return a;
    }
    if (bothLiterals(a, b)) {
        return fold(ExprKind::Add, a, b);
    }
    if (isNegativeLiteral(b)) {
        return Expr(a - negated(b));
    }
    return Expr(a + b);
}

Expr sub(const Expr &a, const Expr &b) {
    if (isLiteral(b, 0)) {
        return a;
    }
    if (bothLiterals(a, b)) {
        return fold(ExprKind::Sub, a, b);
    }
    if (isNegativeLiteral(b)) {
        return add(a, negated(b));
    }
    return Expr(a - b);
}

Expr mul(const Expr &a, const Expr &b) {
    if (isLiteral(a, 0) || isLiteral(b, 0)) {
        return Expr((int64_t)0);
    }
    if (isLiteral(a, 1)) {
        return b;
    }
    if (isLiteral(b, 1)) {
        return a;
    }
    if (bothLiterals(a, b)) {
        return fold(ExprKind::Mul, a, b);
    }
    return Expr(a * b);
}

Expr div(const Expr &a, const Expr &b) {
    if (isLiteral(b, 0)) {
        throw error::UserError("resolve::solve: division by zero");
    }
    if (isLiteral(b, 1) || isLiteral(a, 0)) {
        return a;
    }
    if (bothLiterals(a, b)) {
        return fold(ExprKind::Div, a, b);
    }
    return Expr(a / b);
}

// e = coefficient * v + rest, both free of v
struct Linear {
    Expr coefficient;
    Expr rest;
};

Linear decompose(const Expr &e, const Variable &v) {
    const Expr zero((int64_t)0), one((int64_t)1);
    if (!e.defined()) {
        throw error::UserError("resolve::solve: undefined expression");
    }
    switch (e.ptr->kind) {
    case ExprKind::Variable:
        if (static_cast<const VariableNode *>(e.ptr)->name == v.getName()) {
            return {one, zero};
        }
        return {zero, e};
    case ExprKind::Literal:
    case ExprKind::ADTMember:
    case ExprKind::GridDim:
        return {zero, e};
    default:
        break;
    }
    auto n = static_cast<const BinaryExprNode *>(e.ptr);
    const Linear a = decompose(n->a, v), b = decompose(n->b, v);
    const bool in_a = !isLiteral(a.coefficient, 0), in_b = !isLiteral(b.coefficient, 0);
    switch (e.ptr->kind) {
    case ExprKind::Add:
        return {add(a.coefficient, b.coefficient), add(a.rest, b.rest)};
    case ExprKind::Sub:
        return {sub(a.coefficient, b.coefficient), sub(a.rest, b.rest)};
    case ExprKind::Mul:
        if (in_a && in_b) {
            throw error::UserError("resolve::solve: " + e.str() + " is not linear in " + v.getName());
        }
        if (in_a) {
            return {mul(a.coefficient, b.rest), mul(a.rest, b.rest)};
        }
        return {mul(a.rest, b.coefficient), mul(a.rest, b.rest)};
    case ExprKind::Div:
        if (in_b) {
            throw error::UserError("resolve::solve: " + e.str() + " divides by " + v.getName());
        }
        return {div(a.coefficient, b.rest), div(a.rest, b.rest)};
    default:  // Mod
        if (in_a || in_b) {
            throw error::UserError("resolve::solve: " + e.str() + " takes " + v.getName() + " modulo something");
        }
        return {zero, e};
    }
}

}  // namespace

Expr solve(Eq eq, Variable v) {
    if (!eq.defined()) {
        throw error::UserError("resolve::solve: undefined equation");
    }
    const Linear lhs = decompose(eq.getA(), v), rhs = decompose(eq.getB(), v);
    // lhs.c v + lhs.r = rhs.c v + rhs.r
    const Expr coefficient = sub(lhs.coefficient, rhs.coefficient);
    if (isLiteral(coefficient, 0)) {
        throw error::UserError("resolve::solve: " + eq.str() + " does not determine " + v.getName());
    }
    if (isNegativeLiteral(coefficient)) {  // -k v = r  is  k v = -r
        return div(sub(lhs.rest, rhs.rest), negated(coefficient));
    }
    return div(sub(rhs.rest, lhs.rest), coefficient);
}

}  // namespace resolve
}  // namespace gern
