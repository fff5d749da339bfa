// Lowering: from a composed program to a flat, ordered statement tree
// (allocate / query / compute / insert / free inside loops) with every subset
// extent resolved to an expression over user-provided variables, loop indices
// and data-structure members.
//
// Three steps, as in the reference (src/codegen/concretize.cpp,
// src/codegen/finalizer.cpp):
//   concretize  - walk the composition, chase variable definitions to size
//                 every intermediate (this is where halos are inferred);
//   hoist       - move each statement out of every unmapped loop it does not
//                 depend on;
//   reuse+free  - merge temporaries with disjoint live ranges and identical
//                 allocation calls, then place frees and deferred inserts at
//                 scope exits.
#pragma once

#include "gern/core/composable.h"

#include <memory>

namespace gern {
namespace lower {

enum class NodeKind {
    Block,
    Allocate,  // call.output = the new data structure
    Free,      // method
    Insert,    // method (last argument = the child)
    Query,     // method, parent -> child
    Compute,   // call
    Interval,  // loop or grid-mapped range
    Assert,
    GridDecl,   // explicit launch dimension
    SmemDecl,   // dynamic LDS size
    Opaque,     // a call emitted verbatim (LDS allocator init)
    Blank,
};

struct Node;
using NodePtr = std::shared_ptr<const Node>;

struct Node {
    NodeKind kind = NodeKind::Blank;

    // Block
    std::vector<NodePtr> children;

    // Allocate / Compute / Opaque
    FunctionCall call;
    std::vector<std::string> headers;
    AbstractDataTypePtr adt;  // Compute: the (current name of the) output

    // Free / Insert / Query
    MethodCall method;
    AbstractDataTypePtr parent;
    AbstractDataTypePtr child;
    std::vector<Expr> fields;
    bool insert = false;      // Query: the child must be written back
    NodePtr insert_node;      // Query: the Insert to emit at scope exit

    // Interval
    Assign start = Assign(Expr(), Expr());
    Expr end;
    Expr step;
    NodePtr body;
    Grid::Unit unit = Grid::Unit::UNDEFINED;

    // Assert
    Constraint constraint;

    // GridDecl / SmemDecl
    Grid::Dim dim = Grid::Dim::NULL_DIM;
    Variable var;

    bool isMappedToGrid() const {
        return kind == NodeKind::Interval && isLegalUnit(unit);
    }
    Variable intervalVariable() const {
        return to<Variable>(start.getA());
    }
};

// A placeholder data structure for the result of a query: same functions as
// the structure it was cut from, its own name, type `auto`.
AbstractDataTypePtr makeQueried(const std::string &name, const std::string &type, AbstractDataTypePtr from);

// Runs all three steps.
NodePtr lowerProgram(Composable program);

// Step 1 only (exposed for tests).
NodePtr concretize(Composable program);

std::ostream &operator<<(std::ostream &, const NodePtr &);

}  // namespace lower
}  // namespace gern
