// Composition nodes: annotation synthesis for chains, tiling, staging, and the
// legality check every Composable runs when it is built (reference behaviour:
// src/compose/composable.cpp, src/compose/composable_visitor.cpp:62-135).
#include "gern/core/composable.h"

#include <sstream>

namespace gern {

namespace {

std::set<std::string> adtNames(const std::vector<SubsetObj> &subsets) {
    std::set<std::string> names;
    for (const auto &s : subsets) {
        names.insert(s.getDS().getName());
    }
    return names;
}

// Collects reads and writes of data structures over a composition and rejects
// the illegal ones.
struct LegalityCheck {
    std::set<std::string> reads;
    std::set<std::string> writes;
    std::vector<std::set<std::string>> scopes{{}};

    bool inScope(const std::string &n) const {
        for (const auto &s : scopes) {
            if (s.count(n)) {
                return true;
            }
        }
        return false;
    }

    void call(const ComputeFunctionCall *node) {
        Pattern p = node->getAnnotation().getPattern();
        for (const auto &in : adtNames(p.getInputs())) {
            reads.insert(in);
        }
        const std::string out = p.getOutput().getDS().getName();
        if (reads.count(out)) {
            throw error::UserError("Cannot assign to " + out + " that is being used as input");
        }
        if (writes.count(out)) {
            throw error::UserError("Cannot assign to " + out + " twice ");
        }
        writes.insert(out);
    }

    void visit(const Composable &c) {
        if (!c.defined()) {
            return;
        }
        switch (c.ptr->kind) {
        case ComposableKind::Call:
            call(static_cast<const ComputeFunctionCall *>(c.ptr));
            break;
        case ComposableKind::Computation:
            for (const auto &child : static_cast<const Computation *>(c.ptr)->composed) {
                visit(child);
                scopes.back().insert(child.getAnnotation().getPattern().getOutput().getDS().getName());
            }
            break;
        case ComposableKind::Tiled: {
            auto node = static_cast<const TiledComputation *>(c.ptr);
            scopes.push_back({});
            visit(node->tiled);
            Pattern p = node->getAnnotation().getPattern();
            for (const auto &in : adtNames(p.getInputs())) {
                if (writes.count(in) && !inScope(in)) {
                    throw error::UserError("Nested pipeline is writing to input " + in + " from nested pipeline");
                }
            }
            scopes.pop_back();
            scopes.back().insert(p.getOutput().getDS().getName());
            break;
        }
        case ComposableKind::Stage:
            visit(static_cast<const StageNode *>(c.ptr)->body);
            break;
        case ComposableKind::Global:
            visit(static_cast<const GlobalNode *>(c.ptr)->program);
            break;
        }
    }

    void run(const Composable &c) {
        visit(c);
        const std::string out = c.getAnnotation().getPattern().getOutput().getDS().getName();
        for (const auto &w : writes) {
            if (!reads.count(w) && w != out) {
                throw error::UserError(" Wrote to intermediate " + w + ", but never read it");
            }
        }
    }
};

// Rebuilds `consumes` inside the same nest of reducible loops that `like` has.
Consumes wrapLikeConsumes(const Stmt &like, ConsumeMany consumes) {
    if (!like.defined()) {
        return consumes;
    }
    switch (like.ptr->kind) {
    case StmtKind::ConsumesFor: {
        auto n = static_cast<const ConsumesForNode *>(like.ptr);
        ConsumeMany inner(wrapLikeConsumes(n->body, consumes).ptr);
        return Reducible(n->start, n->parameter, n->step, inner);
    }
    case StmtKind::ComputesFor:
        return wrapLikeConsumes(static_cast<const ComputesForNode *>(like.ptr)->body, consumes);
    case StmtKind::Computes:
        return wrapLikeConsumes(static_cast<const ComputesNode *>(like.ptr)->c, consumes);
    default:
        return consumes;
    }
}

// Rebuilds `computes` inside the same nest of tileable loops that `like` has.
Pattern wrapLikeComputes(const Stmt &like, Pattern computes) {
    if (like.defined() && like.ptr->kind == StmtKind::ComputesFor) {
        auto n = static_cast<const ComputesForNode *>(like.ptr);
        return Tileable(n->start, n->parameter, n->step, wrapLikeComputes(n->body, computes));
    }
    return computes;
}

void printComposable(std::ostream &os, const Composable &c, int indent) {
    auto pad = [&](int n) {
        for (int i = 0; i < n; i++) {
            os << "  ";
        }
    };
    if (!c.defined()) {
        return;
    }
    switch (c.ptr->kind) {
    case ComposableKind::Call:
        pad(indent);
        os << *static_cast<const ComputeFunctionCall *>(c.ptr);
        break;
    case ComposableKind::Computation: {
        auto node = static_cast<const Computation *>(c.ptr);
        for (size_t i = 0; i < node->composed.size(); i++) {
            printComposable(os, node->composed[i], indent);
            os << (i + 1 != node->composed.size() ? "\n" : "");
        }
        break;
    }
    case ComposableKind::Tiled: {
        auto node = static_cast<const TiledComputation *>(c.ptr);
        pad(indent);
        os << (node->reduce ? "Reduce " : "For ") << node->to_tile << " with " << node->v;
        if (isLegalUnit(node->unit)) {
            os << " over " << node->unit;
        }
        os << " {\n";
        printComposable(os, node->tiled, indent + 1);
        os << "\n";
        pad(indent);
        os << "}";
        break;
    }
    case ComposableKind::Stage: {
        auto node = static_cast<const StageNode *>(c.ptr);
        pad(indent);
        os << "Stage " << node->adt.getName() << " {\n";
        printComposable(os, node->body, indent + 1);
        os << "\n";
        pad(indent);
        os << "}";
        break;
    }
    case ComposableKind::Global: {
        auto node = static_cast<const GlobalNode *>(c.ptr);
        pad(indent);
        os << "Global {\n";
        printComposable(os, node->program, indent + 1);
        os << "\n";
        pad(indent);
        os << "}";
        break;
    }
    }
}

}  // namespace

// ---------------------------------------------------------------------------
Composable::Composable(const ComposableNode *n)
    : util::IntrusivePtr<const ComposableNode>(n) {
    LegalityCheck check;
    check.run(*this);
}

Composable::Composable(std::vector<Composable> composed)
    : Composable(new const Computation(composed)) {
}

Annotation Composable::getAnnotation() const {
    return defined() ? ptr->getAnnotation() : Annotation();
}

bool Composable::isDeviceLaunch() const {
    return defined() && ptr->kind == ComposableKind::Global;
}

std::ostream &operator<<(std::ostream &os, const Composable &c) {
    printComposable(os, c, 0);
    return os;
}

std::ostream &operator<<(std::ostream &os, const ComputeFunctionCall &f) {
    return os << f.getCall();
}

// ---------------------------------------------------------------------------
Computation::Computation(std::vector<Composable> composed)
    : ComposableNode(ComposableKind::Computation), composed(composed) {
    if (composed.empty()) {
        return;
    }
    for (const auto &c : composed) {
        for (const auto &input : c.getAnnotation().getPattern().getInputs()) {
            consumer_functions[input.getDS()].push_back(c);
        }
    }
    init_annotation();
}

void Computation::infer_relationships(AbstractDataTypePtr output, std::vector<Variable> output_fields) {
    auto it = consumer_functions.find(output);
    if (it == consumer_functions.end() || it->second.empty()) {
        return;
    }
    if (it->second.size() != 1) {
        // A structure read by several later stages: every reader is assumed to
        // need the same subset, and the first reader (in program order)
        // defines it.
        std::cerr << "WARNING::FORKS ARE NOT IMPL, ASSUMING EQUAL CONSUMPTION!" << std::endl;
    }
    const Composable &consumer = it->second.front();
    std::vector<Expr> needed = consumer.getAnnotation().getPattern().getRequirement(output);
    for (size_t i = 0; i < needed.size() && i < output_fields.size(); i++) {
        declarations.push_back(output_fields[i] = needed[i]);
        declarations_map[output_fields[i]] = needed[i];
    }
}

void Computation::init_annotation() {
    Pattern last = composed.back().getAnnotation().getPattern();
    Produces produces = Produces::Subset(last.getOutput().getDS(), last.getProducesField());

    // Walk the chain backwards: each stage's produced fields are defined by
    // what its consumer needs.
    std::set<std::string> intermediates;
    for (auto it = composed.rbegin(); it != composed.rend(); ++it) {
        Pattern p = it->getAnnotation().getPattern();
        AbstractDataTypePtr produced = p.getOutput().getDS();
        infer_relationships(produced, p.getProducesField());
        intermediates.insert(produced.getName());
    }

    Substitution defs;
    for (const auto &kv : declarations_map) {
        defs.variables[kv.first.getName()] = kv.second;
    }

    std::set<Grid::Unit> occupied;
    std::vector<Constraint> constraints;
    std::vector<SubsetObj> true_inputs;
    for (const auto &c : composed) {
        Annotation a = c.getAnnotation();
        auto units = a.getOccupiedUnits();
        occupied.insert(units.begin(), units.end());
        auto cs = a.getConstraints();
        constraints.insert(constraints.begin(), cs.begin(), cs.end());
        for (const auto &input : a.getPattern().getInputs()) {
            if (intermediates.count(input.getDS().getName())) {
                continue;
            }
            // One substitution per stage between this input and the output: the fields end up over the
            // variables of the LAST stage, which are the ones a tile or a stage around the chain renames.
            std::vector<Expr> fields;
            for (const auto &f : input.getFields()) {
                Expr over_output = f;
                for (size_t stage = 0; stage < composed.size(); stage++) {
                    over_output = substitute(over_output, defs);
                }
                fields.push_back(over_output);
            }
            true_inputs.push_back(SubsetObj(input.getDS(), fields));
        }
    }

    Consumes consumes = wrapLikeConsumes(last, SubsetObjMany(true_inputs));
    Pattern pattern = wrapLikeComputes(last, Computes(produces, consumes));
    _annotation = Annotation(pattern, occupied, constraints);
}

// ---------------------------------------------------------------------------
TiledComputation::TiledComputation(Expr to_tile, Variable v, Composable body, Grid::Unit unit, bool reduce)
    : ComposableNode(ComposableKind::Tiled), to_tile(to_tile), v(v), tiled(body), unit(unit), reduce(reduce) {
    Annotation annotation = body.getAnnotation();
    auto units = annotation.getOccupiedUnits();
    units.insert(unit);
    _annotation = resetUnit(annotation, units);

    Pattern pattern = _annotation.getPattern();
    auto loops = reduce ? pattern.getReducableFields() : pattern.getTileableFields();
    auto found = loops.find(to_tile);
    if (found == loops.end()) {
        throw error::UserError("Cannot tile " + to_tile.str());
    }
    captured = std::get<0>(found->second);
    start = std::get<1>(found->second);
    parameter = to_tile;
    step = std::get<2>(found->second);

    // This node's view of the body: every variable renamed, so that the same
    // body can be tiled again from outside without name clashes.
    _annotation = refreshVariables(_annotation, old_to_new);
    loop_index = old_to_new.at(captured);
    // `step` deliberately keeps its name from the body's annotation: lowering
    // defines body-step := v after it has recorded body-name -> fresh-name.
}

TileDummy Tile(Expr tileable, Variable v) {
    return TileDummy(tileable, v, false);
}

TileDummy Reduce(Expr tileable, Variable v) {
    return TileDummy(tileable, v, true);
}

TileDummy TileDummy::operator||(Grid::Unit p) {
    unit = p;
    return *this;
}

Composable TileDummy::operator()(Composable c) {
    Composable nested = c;
    if (isa<ComputeFunctionCall>(c.ptr)) {
        nested = new const Computation({c});
    }
    if (isLegalUnit(unit) && !reduce) {
        std::set<Grid::Unit> occupied = c.getAnnotation().getOccupiedUnits();
        if (occupied.empty()) {
            throw error::UserError("The function does not have a legal unit for the current GPU");
        }
        if (!legalToDistribute(occupied, unit)) {
            std::stringstream ss;
            ss << "Trying to distribute " << getLevel(occupied) << " over unit " << unit;
            throw error::UserError(ss.str());
        }
    }
    return new const TiledComputation(to_tile, v, nested, unit, reduce);
}

// ---------------------------------------------------------------------------
StageNode::StageNode(AbstractDataTypePtr adt, FunctionSignature query_f, FunctionSignature insert_f,
                     Composable body, bool insert)
    : ComposableNode(ComposableKind::Stage), adt(adt), query_f(query_f), insert_f(insert_f), body(body),
      insert(insert) {
    _annotation = refreshVariables(body.getAnnotation(), old_to_new);
    staged_subset = _annotation.getPattern().getCorrespondingSubset(adt);
}

Composable Stage(AbstractDataTypePtr adt, FunctionSignature query_f, FunctionSignature insert_f,
                 Composable body, bool insert) {
    if (isa<ComputeFunctionCall>(body.ptr)) {
        body = new const Computation({body});
    }
    for (const auto &in_scope : body.getAnnotation().getPattern().getAllADTs()) {
        if (in_scope.getDS() == adt) {
            return new const StageNode(adt, query_f, insert_f, body, insert);
        }
    }
    throw error::UserError("Stage must have " + adt.getName() + " as an input or output of the body in scope.");
}

Composable Stage(AbstractDataTypePtr adt, FunctionSignature query_f, FunctionSignature insert_f, Composable body) {
    return Stage(adt, query_f, insert_f, body, true);
}

Composable Stage(AbstractDataTypePtr adt, FunctionSignature query_f, Composable body) {
    return Stage(adt, query_f, adt.getInsertFunction(), body, false);
}

Composable Stage(AbstractDataTypePtr adt, Composable body) {
    return Stage(adt, adt.getQueryFunction(), adt.getInsertFunction(), body, adt.insertQuery());
}

// ---------------------------------------------------------------------------
GlobalNode::GlobalNode(Composable program, std::map<Grid::Dim, Variable> launch_args, Variable smem_size,
                       grid::SharedMemoryManager smem_manager)
    : ComposableNode(ComposableKind::Global), program(program), launch_args(launch_args), smem_size(smem_size),
      smem_manager(smem_manager) {
    auto legal = getDims(program.getAnnotation().getOccupiedUnits());
    for (const auto &arg : launch_args) {
        if (!isDimInScope(arg.first, legal)) {
            std::stringstream ss;
            ss << "Cannot specify the size of " << arg.first << ".";
            throw error::UserError(ss.str());
        }
    }
}

Composable Global(Composable program, std::map<Grid::Dim, Variable> launch_args, Variable smem_size,
                  grid::SharedMemoryManager smem_manager) {
    return new const GlobalNode(program, launch_args, smem_size, smem_manager);
}

}  // namespace gern
