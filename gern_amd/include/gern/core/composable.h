// Composition: function calls chained into pipelines, tiled / reduced over a
// loop (optionally distributed over a grid unit), staged through an
// intermediate view, and wrapped for a device launch.
//
// Same user surface as the reference (include/gern/compose/composable.h:18-174,
// compose/compose.h:87-127, compose/composable_node.h).
#pragma once

#include "gern/core/function.h"

namespace gern {

enum class ComposableKind { Call, Computation, Tiled, Stage, Global };

class ComposableNode : public util::Manageable<ComposableNode>, public util::Uncopyable {
public:
    explicit ComposableNode(ComposableKind kind)
        : kind(kind) {
    }
    virtual ~ComposableNode() = default;
    virtual Annotation getAnnotation() const = 0;
    const ComposableKind kind;
};

class Composable : public util::IntrusivePtr<const ComposableNode> {
public:
    Composable()
        : util::IntrusivePtr<const ComposableNode>(nullptr) {
    }
    // Checks that the composition is legal (no intermediate written and never
    // read, no structure written twice or written while read); throws
    // UserError otherwise.
    Composable(const ComposableNode *n);
    Composable(std::vector<Composable> composed);
    Annotation getAnnotation() const;
    bool isDeviceLaunch() const;
};

std::ostream &operator<<(std::ostream &, const Composable &);

// One call of a user function, with the annotation specialised to this call
// site (fresh variable names, concrete data structures).
class ComputeFunctionCall : public ComposableNode {
public:
    ComputeFunctionCall(FunctionCall call, Annotation annotation, std::vector<std::string> header)
        : ComposableNode(ComposableKind::Call), call(call), annotation(annotation), header(header) {
    }
    FunctionCall getCall() const {
        return call;
    }
    Annotation getAnnotation() const override {
        return annotation;
    }
    std::vector<std::string> getHeader() const {
        return header;
    }
    static bool classof(const ComposableNode *n) {
        return n->kind == ComposableKind::Call;
    }

private:
    FunctionCall call;
    Annotation annotation;
    std::vector<std::string> header;
};

using ComputeFunctionCallPtr = const ComputeFunctionCall *;
std::ostream &operator<<(std::ostream &, const ComputeFunctionCall &);

// A chain of composables; the output of the last one is the output of the
// chain.  Its annotation is synthesised: it produces what the last stage
// produces and consumes, of each true input, what the stages need once every
// intermediate's producer fields are equated with its consumer's requirement.
class Computation : public ComposableNode {
public:
    Computation(std::vector<Composable> composed);
    Annotation getAnnotation() const override {
        return _annotation;
    }
    static bool classof(const ComposableNode *n) {
        return n->kind == ComposableKind::Computation;
    }

    std::vector<Composable> composed;
    // producer field := consumer requirement, for every intermediate
    std::vector<Assign> declarations;
    std::map<Variable, Expr> declarations_map;
    std::map<AbstractDataTypePtr, std::vector<Composable>> consumer_functions;
    Annotation _annotation;

private:
    void init_annotation();
    void infer_relationships(AbstractDataTypePtr output, std::vector<Variable> output_fields);
};

// body executed once per `v`-sized step of the loop whose bound is `to_tile`.
class TiledComputation : public ComposableNode {
public:
    TiledComputation(Expr to_tile, Variable v, Composable body, Grid::Unit unit, bool reduce);
    Annotation getAnnotation() const override {
        return _annotation;
    }
    static bool classof(const ComposableNode *n) {
        return n->kind == ComposableKind::Tiled;
    }

    Expr to_tile;
    Variable v;
    Composable tiled;
    Variable captured;    // the loop index in the body's annotation
    Variable loop_index;  // its fresh name in this node's annotation
    Expr start;
    Expr parameter;
    Variable step;
    Annotation _annotation;
    std::map<Variable, Variable> old_to_new;
    Grid::Unit unit{Grid::Unit::UNDEFINED};
    bool reduce = false;
};

// body executed against a subset of `adt` obtained once, outside the body,
// with query_f (and written back with insert_f when it is the body's output).
class StageNode : public ComposableNode {
public:
    StageNode(AbstractDataTypePtr adt, FunctionSignature query_f, FunctionSignature insert_f,
              Composable body, bool insert);
    Annotation getAnnotation() const override {
        return _annotation;
    }
    static bool classof(const ComposableNode *n) {
        return n->kind == ComposableKind::Stage;
    }

    Annotation _annotation;
    AbstractDataTypePtr adt;
    FunctionSignature query_f;
    FunctionSignature insert_f;
    Composable body;
    bool insert;
    SubsetObj staged_subset;
    std::map<Variable, Variable> old_to_new;
};

// Marks the program as one device kernel.  launch_args fixes launch
// dimensions explicitly; smem_size is the dynamic LDS size in bytes.
class GlobalNode : public ComposableNode {
public:
    GlobalNode(Composable program, std::map<Grid::Dim, Variable> launch_args, Variable smem_size,
               grid::SharedMemoryManager smem_manager);
    Annotation getAnnotation() const override {
        return program.getAnnotation();
    }
    static bool classof(const ComposableNode *n) {
        return n->kind == ComposableKind::Global;
    }

    Composable program;
    std::map<Grid::Dim, Variable> launch_args;
    Variable smem_size;
    grid::SharedMemoryManager smem_manager;
};

Composable Global(Composable program, std::map<Grid::Dim, Variable> launch_args = {},
                  Variable smem_size = Variable(), grid::SharedMemoryManager smem_manager = {});

Composable Stage(AbstractDataTypePtr adt, FunctionSignature query_f, FunctionSignature insert_f,
                 Composable body, bool insert);
Composable Stage(AbstractDataTypePtr adt, FunctionSignature query_f, FunctionSignature insert_f,
                 Composable body);
Composable Stage(AbstractDataTypePtr adt, FunctionSignature query_f, Composable body);
Composable Stage(AbstractDataTypePtr adt, Composable body);

// Tile(bound, v)(body...) and Reduce(bound, v)(body...), optionally
// `|| Grid::Unit` to distribute the loop over the launch grid.
struct TileDummy {
    TileDummy(Expr to_tile, Variable v, bool reduce)
        : to_tile(to_tile), v(v), reduce(reduce) {
    }
    Composable operator()(Composable c);
    template<typename First, typename Second, typename... ToCompose>
    Composable operator()(First first, Second second, ToCompose... c) {
        static_assert(std::is_same_v<First, Composable> && std::is_same_v<Second, Composable> &&
                          (std::is_same_v<ToCompose, Composable> && ...),
                      "All arguments must be of type Composable");
        std::vector<Composable> to_compose{first, second, c...};
        return operator()(Composable(new const Computation(to_compose)));
    }
    TileDummy operator||(Grid::Unit p);

    Expr to_tile;
    Variable v;
    bool reduce;
    Grid::Unit unit{Grid::Unit::UNDEFINED};
};

TileDummy Tile(Expr tileable, Variable v);
TileDummy Reduce(Expr tileable, Variable v);

template<typename E>
inline bool isa(const ComposableNode *e) {
    return e != nullptr && E::classof(e);
}
template<typename E>
inline const E *to(const ComposableNode *e) {
    assert(isa<E>(e));
    return static_cast<const E *>(e);
}

}  // namespace gern
