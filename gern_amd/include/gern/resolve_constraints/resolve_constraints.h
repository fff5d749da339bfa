// Solving one equation for one variable: the interface of the reference's
// include/gern/resolve_constraints/resolve_constraints.h:8-25 (there a thin
// layer over GiNaC::lsolve that no part of the library calls; the grid mapping
// and the bounds of tiles are resolved by substitution in the lowering).
// This implementation needs no algebra library: it handles what the interface
// promises, an equation that is LINEAR in the variable asked for, and the
// solution is an expression over the same nodes as the equation.
#pragma once

#include "annotations/data_dependency_language.h"

namespace gern {
namespace resolve {

// The v that satisfies eq, as an expression free of v.  eq must be linear in
// v (v may be added, subtracted, multiplied by and divided by expressions that
// do not contain it); anything else, and an equation that does not contain v
// or leaves its coefficient zero, is a UserError.  Literals are folded,
// additions of zero and multiplications by one are dropped; a coefficient
// that is not one ends up as a division, which is exact over the rationals
// and the caller's to interpret over integers.
Expr solve(Eq eq, Variable v);

}  // namespace resolve
}  // namespace gern
