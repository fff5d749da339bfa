// Lowering of a composed program to an ordered statement tree; see
// gern/lower/lower.h for the three steps.  The rules each step applies are the
// reference's (src/codegen/concretize.cpp, src/codegen/finalizer.cpp); the
// data structures and code are this project's.
#include "gern/lower/lower.h"

#include <algorithm>
#include <sstream>

namespace gern {
namespace lower {

namespace {

// ---------------------------------------------------------------------------
// A data structure that stands for the result of a query (or for a renamed
// temporary): it answers like the structure it was derived from.
// ---------------------------------------------------------------------------
class DerivedADT : public AbstractDataType {
public:
    DerivedADT(const std::string &name, const std::string &type, AbstractDataTypePtr from)
        : name(name), type(type), from(from) {
    }
    std::string getName() const override {
        return name;
    }
    std::string getType() const override {
        return type;
    }
    std::vector<Variable> getFields() const override {
        return from.getFields();
    }
    FunctionSignature getAllocateFunction() const override {
        return from.getAllocateFunction();
    }
    FunctionSignature getFreeFunction() const override {
        return from.getFreeFunction();
    }
    FunctionSignature getInsertFunction() const override {
        return from.getInsertFunction();
    }
    FunctionSignature getQueryFunction() const override {
        return from.getQueryFunction();
    }
    bool freeQuery() const override {
        return from.freeQuery();
    }
    bool insertQuery() const override {
        return from.insertQuery();
    }
    bool freeAlloc() const override {
        return from.freeAlloc();
    }

private:
    std::string name;
    std::string type;
    AbstractDataTypePtr from;
};

NodePtr make(Node n) {
    return std::make_shared<const Node>(std::move(n));
}

NodePtr blank() {
    return make(Node{});
}

NodePtr block(std::vector<NodePtr> children) {
    Node n;
    n.kind = NodeKind::Block;
    n.children = std::move(children);
    return make(std::move(n));
}

// Innermost-first stack of maps.
template<typename K, typename V, typename Cmp = std::less<K>>
class Scoped {
public:
    Scoped() {
        push();
    }
    void push() {
        scopes.emplace_back();
    }
    void pop() {
        scopes.pop_back();
    }
    void put(const K &k, const V &v) {
        scopes.back()[k] = v;
    }
    bool hasHere(const K &k) const {
        return scopes.back().count(k) > 0;
    }
    bool has(const K &k) const {
        for (auto it = scopes.rbegin(); it != scopes.rend(); ++it) {
            if (it->count(k)) {
                return true;
            }
        }
        return false;
    }
    const V &at(const K &k) const {
        for (auto it = scopes.rbegin(); it != scopes.rend(); ++it) {
            auto f = it->find(k);
            if (f != it->end()) {
                return f->second;
            }
        }
        throw error::InternalError("scoped lookup failed");
    }

private:
    std::vector<std::map<K, V, Cmp>> scopes;
};

using NameSet = std::set<std::string>;

// ---------------------------------------------------------------------------
// Step 1: concretize
// ---------------------------------------------------------------------------
class Concretizer {
public:
    NodePtr run(Composable program) {
        Pattern pattern = program.getAnnotation().getPattern();
        // What the caller passes in is in scope from the start.
        auto out = pattern.getOutput().getDS();
        adt_staged_at.put(out.getName(), {});
        current.put(out.getName(), SubsetObj(out, {}));
        for (const auto &in : pattern.getInputs()) {
            adt_staged_at.put(in.getDS().getName(), {});
            current.put(in.getDS().getName(), SubsetObj(in.getDS(), {}));
        }
        return visit(program);
    }

private:
    // variable name -> the expression that defines it
    std::map<std::string, Expr> relations;
    // variables whose value the user provides (arguments, tile sizes)
    std::vector<NameSet> defined{{}};
    // loop indices of the loops being lowered
    NameSet loop_indices;
    // data structure -> loop indices in scope when it was staged
    Scoped<std::string, NameSet> adt_staged_at;
    // data structure -> its current (queried / allocated) name and subset
    Scoped<std::string, SubsetObj> current;
    // loop bound -> tile size variable of the enclosing loop over that bound
    Scoped<Expr, Variable> tiled_bounds;

    bool isDefined(const std::string &v) const {
        for (const auto &s : defined) {
            if (s.count(v)) {
                return true;
            }
        }
        return false;
    }

    void define(const Variable &var, const Expr &e) {
        if (var.isBound() || isDefined(var.getName())) {
            return;
        }
        relations[var.getName()] = e;
    }

    // Rewrites e over "base" quantities only: user-provided variables, loop
    // indices in scope, members and literals.  A loop index that itself has a
    // definition contributes index + definition (its offset inside the
    // enclosing tile).  Variables in stop_at, and variables nobody defines,
    // contribute 0.
    Expr base(const Expr &e, const NameSet &stop_at) const {
        if (!e.defined()) {
            return e;
        }
        switch (e.ptr->kind) {
        case ExprKind::Variable: {
            auto v = static_cast<const VariableNode *>(e.ptr);
            auto rel = relations.find(v->name);
            if (rel != relations.end() && !stop_at.count(v->name)) {
                Expr rest = base(rel->second, stop_at);
                return loop_indices.count(v->name) ? Expr(e + rest) : rest;
            }
            if (stop_at.count(v->name)) {
                return Expr(0);
            }
            if (!isDefined(v->name) && !loop_indices.count(v->name) && !v->bound) {
                return Expr(0);
            }
            return e;
        }
        case ExprKind::Add:
        case ExprKind::Sub:
        case ExprKind::Mul:
        case ExprKind::Div:
        case ExprKind::Mod: {
            auto n = static_cast<const BinaryExprNode *>(e.ptr);
            return Expr(new const BinaryExprNode(n->kind, base(n->a, stop_at), base(n->b, stop_at)));
        }
        default:
            return e;
        }
    }

    Constraint base(const Constraint &c) const {
        auto n = static_cast<const BinaryConstraintNode *>(c.ptr);
        return Constraint(new const BinaryConstraintNode(n->kind, base(n->a, {}), base(n->b, {})));
    }

    void declareLoop(const Expr &bound, const Variable &step) {
        Expr s = base(step, {});
        // A step nobody has fixed covers the whole range.
        define(step, isa<Literal>(s) ? bound : s);
        if (isa<Variable>(bound)) {
            defined.back().insert(to<Variable>(bound).getName());
        }
    }

    void declareLoops(const Annotation &a, const Variable *skip_index) {
        Pattern p = a.getPattern();
        for (const auto &f : p.getTileableFields()) {
            if (skip_index && std::get<0>(f.second).getName() == skip_index->getName()) {
                continue;
            }
            declareLoop(f.first, std::get<2>(f.second));
        }
        for (const auto &f : p.getReducableFields()) {
            if (skip_index && std::get<0>(f.second).getName() == skip_index->getName()) {
                continue;
            }
            declareLoop(f.first, std::get<2>(f.second));
        }
    }

    // Builds a call of signature f on a structure whose abstract fields are
    // ref_fields, given the actual value of every field.
    static FunctionCall bindCall(const FunctionSignature &f, const std::vector<Variable> &ref_fields,
                                 const std::vector<Expr> &values) {
        if (ref_fields.size() != values.size()) {
            throw error::InternalError("Incorrect number of fields passed!");
        }
        std::map<std::string, Expr> by_name;
        for (size_t i = 0; i < ref_fields.size(); i++) {
            by_name[ref_fields[i].getName()] = values[i];
        }
        auto value_of = [&](const Variable &v) -> Expr {
            auto it = by_name.find(v.getName());
            if (it == by_name.end()) {
                throw error::UserError("function " + f.name + " uses " + v.getName() +
                                       ", which is not a field of its data structure");
            }
            return it->second;
        };
        FunctionCall call = f.constructCall();
        call.args.clear();
        call.template_args.clear();
        for (const auto &a : f.args) {
            call.args.push_back(Argument(value_of(a.getVar())));
        }
        for (const auto &t : f.template_args) {
            call.template_args.push_back(Argument(value_of(t)));
        }
        call.grid = LaunchArguments();
        call.block = LaunchArguments();
        return call;
    }

    // Makes `subset` available in the current scope: nothing if it already
    // is; a query from the enclosing scope's version if the structure exists
    // outside; an allocation if it is a temporary nobody has made yet.
    NodePtr prepare(const SubsetObj &subset, const FunctionSignature &query_f, const FunctionSignature &insert_f,
                    bool write_back) {
        AbstractDataTypePtr adt = subset.getDS();
        const std::string name = adt.getName();
        if (adt_staged_at.hasHere(name)) {
            return blank();
        }
        if (adt_staged_at.has(name)) {
            const NameSet staged_at = adt_staged_at.at(name);
            std::vector<Expr> fields;
            for (const auto &f : subset.getFields()) {
                fields.push_back(base(f, staged_at));
            }
            adt_staged_at.put(name, loop_indices);

            AbstractDataTypePtr parent = current.at(name).getDS();
            FunctionCall call = bindCall(query_f, parent.getFields(), fields);
            AbstractDataTypePtr queried = makeQueried(getUniqueName("_query_" + name), "auto", adt);
            call.output = Parameter(queried);
            current.put(name, SubsetObj(queried, fields));

            Node q;
            q.kind = NodeKind::Query;
            q.parent = adt;
            q.child = queried;
            q.fields = fields;
            q.method = MethodCall{parent, call};
            q.insert = write_back;
            q.insert_node = blank();
            if (write_back) {
                FunctionCall ins = bindCall(insert_f, parent.getFields(), fields);
                ins.args.push_back(Argument(queried));
                Node i;
                i.kind = NodeKind::Insert;
                i.method = MethodCall{parent, ins};
                q.insert_node = make(std::move(i));
            }
            return make(std::move(q));
        }
        std::vector<Expr> fields;
        for (const auto &f : subset.getFields()) {
            fields.push_back(base(f, {}));
        }
        adt_staged_at.put(name, loop_indices);
        FunctionCall call = bindCall(adt.getAllocateFunction(), adt.getFields(), fields);
        call.output = Parameter(adt);
        current.put(name, SubsetObj(adt, fields));
        Node a;
        a.kind = NodeKind::Allocate;
        a.call = call;
        return make(std::move(a));
    }

    NodePtr prepare(const SubsetObj &subset, bool write_back) {
        AbstractDataTypePtr adt = subset.getDS();
        return prepare(subset, adt.getQueryFunction(), adt.getInsertFunction(), adt.insertQuery() && write_back);
    }

    std::vector<Argument> concreteArguments(const std::vector<Argument> &args) {
        std::vector<Argument> out;
        for (const auto &a : args) {
            if (a.isData() && current.has(a.getADTPtr().getName())) {
                out.push_back(Argument(current.at(a.getADTPtr().getName()).getDS()));
            } else if (a.isExpr()) {
                // Whatever a call passes by value must come from the user.
                for (const auto &v : getVariables(a.getExpr())) {
                    defined.back().insert(v.getName());
                }
                out.push_back(Argument(base(a.getExpr(), {})));
            } else {
                throw error::InternalError("Unknown argument type: " + a.str());
            }
        }
        return out;
    }

    NodePtr visit(const Composable &c) {
        switch (c.ptr->kind) {
        case ComposableKind::Call:
            return visitCall(static_cast<const ComputeFunctionCall *>(c.ptr));
        case ComposableKind::Computation:
            return visitChain(static_cast<const Computation *>(c.ptr));
        case ComposableKind::Tiled:
            return visitTiled(static_cast<const TiledComputation *>(c.ptr));
        case ComposableKind::Stage:
            return visitStage(static_cast<const StageNode *>(c.ptr));
        case ComposableKind::Global:
            return visitGlobal(static_cast<const GlobalNode *>(c.ptr));
        }
        throw error::InternalError("unknown composable");
    }

    NodePtr visitChain(const Computation *node) {
        declareLoops(node->getAnnotation(), nullptr);
        for (const auto &d : node->declarations) {
            define(to<Variable>(d.getA()), d.getB());
        }
        std::vector<NodePtr> out;
        out.push_back(prepare(node->getAnnotation().getPattern().getOutput(), true));
        for (const auto &c : node->composed) {
            out.push_back(prepare(c.getAnnotation().getPattern().getOutput(), true));
            out.push_back(visit(c));
        }
        return block(out);
    }

    NodePtr visitTiled(const TiledComputation *node) {
        std::vector<NodePtr> out;
        for (const auto &rel : node->old_to_new) {
            define(rel.first, rel.second);
        }
        // The tiled loop advances by the variable the user gave.
        define(node->step, node->v);
        defined.back().insert(node->v.getName());

        declareLoops(node->getAnnotation(), &node->loop_index);

        SubsetObj output = node->getAnnotation().getPattern().getOutput();
        if (node->reduce) {
            // A reduction accumulates into one output subset: stage it before
            // the loop.
            out.push_back(prepare(output, true));
        }

        adt_staged_at.push();
        defined.emplace_back();
        tiled_bounds.push();
        current.push();
        loop_indices.insert(node->loop_index.getName());
        tiled_bounds.put(node->parameter, node->v);
        if (isa<Variable>(node->parameter)) {
            Variable p = to<Variable>(node->parameter);
            defined.back().insert(p.getName());
            relations[p.getName()] = node->v;
        }
        if (node->reduce) {
            const std::string name = output.getDS().getName();
            adt_staged_at.put(name, adt_staged_at.at(name));
            current.put(name, current.at(name));
        }

        NodePtr body = visit(node->tiled);

        adt_staged_at.pop();
        loop_indices.erase(node->loop_index.getName());
        defined.pop_back();
        tiled_bounds.pop();
        current.pop();

        // Nested inside another loop over the same bound, this loop walks the
        // enclosing tile, from 0 to that tile's size.
        const bool nested = tiled_bounds.has(node->parameter);
        Node loop;
        loop.kind = NodeKind::Interval;
        loop.start = nested ? (node->loop_index = Expr(0)) : (node->loop_index = node->start);
        loop.end = nested ? Expr(tiled_bounds.at(node->parameter)) : node->parameter;
        loop.step = node->v;
        loop.body = body;
        loop.unit = node->unit;
        out.push_back(make(std::move(loop)));
        return block(out);
    }

    NodePtr visitCall(const ComputeFunctionCall *node) {
        std::vector<NodePtr> out;
        Annotation annotation = node->getAnnotation();
        declareLoops(annotation, nullptr);
        for (const auto &c : annotation.getConstraints()) {
            Node a;
            a.kind = NodeKind::Assert;
            a.constraint = base(c);
            out.push_back(make(std::move(a)));
        }
        Pattern pattern = annotation.getPattern();
        for (const auto &in : pattern.getInputs()) {
            out.push_back(prepare(in, false));
        }
        out.push_back(prepare(pattern.getOutput(), true));

        FunctionCall call = node->getCall();
        call.args = concreteArguments(call.args);
        call.template_args = concreteArguments(call.template_args);
        Node c;
        c.kind = NodeKind::Compute;
        c.call = call;
        c.headers = node->getHeader();
        c.adt = current.at(pattern.getOutput().getDS().getName()).getDS();
        out.push_back(make(std::move(c)));
        return block(out);
    }

    NodePtr visitGlobal(const GlobalNode *node) {
        std::vector<NodePtr> out;
        for (const auto &def : node->launch_args) {
            Node g;
            g.kind = NodeKind::GridDecl;
            g.dim = def.first;
            g.var = def.second;
            out.push_back(make(std::move(g)));
        }
        Node s;
        s.kind = NodeKind::SmemDecl;
        s.var = node->smem_size;
        out.push_back(make(std::move(s)));
        if (node->smem_manager.isInitialized()) {
            Node o;
            o.kind = NodeKind::Opaque;
            o.call = node->smem_manager.getInit();
            o.headers = node->smem_manager.getHeaders();
            out.push_back(make(std::move(o)));
        }
        out.push_back(visit(node->program));
        return block(out);
    }

    NodePtr visitStage(const StageNode *node) {
        for (const auto &rel : node->old_to_new) {
            define(rel.first, rel.second);
        }
        declareLoops(node->getAnnotation(), nullptr);
        const std::string name = node->adt.getName();
        if (!adt_staged_at.has(name)) {
            throw error::UserError("Cannot stage " + name + " because it is not in scope.");
        }
        if (adt_staged_at.hasHere(name)) {
            throw error::UserError("Cannot stage " + name + " because it is already in the current scope.");
        }
        const bool is_output = node->staged_subset.getDS() == node->body.getAnnotation().getPattern().getOutput().getDS();
        std::vector<NodePtr> out;
        out.push_back(prepare(node->staged_subset, node->query_f, node->insert_f, node->insert && is_output));
        out.push_back(visit(node->body));
        return block(out);
    }
};

// ---------------------------------------------------------------------------
// Step 2: hoist statements out of unmapped loops they do not depend on
// ---------------------------------------------------------------------------
class Hoister {
public:
    NodePtr run(const NodePtr &ir) {
        visit(ir);
        return block(at_depth[depth]);
    }

private:
    int depth = 0;  // number of enclosing unmapped loops
    std::map<std::string, int> adt_depth;
    std::map<std::string, int> var_depth;
    std::map<int, std::vector<NodePtr>> at_depth;

    int depthOf(const Expr &e) const {
        int d = 0;
        for (const auto &v : getVariables(e)) {
            auto it = var_depth.find(v.getName());
            d = std::max(d, it == var_depth.end() ? 0 : it->second);
        }
        collectMembers(e, d);
        if (!getDims(e).empty()) {
            d = std::max(d, depth);
        }
        return d;
    }

    void collectMembers(const Expr &e, int &d) const {
        if (!e.defined()) {
            return;
        }
        if (e.ptr->kind == ExprKind::ADTMember) {
            auto it = adt_depth.find(static_cast<const ADTMemberNode *>(e.ptr)->ds.getName());
            d = std::max(d, it == adt_depth.end() ? 0 : it->second);
        } else if (e.ptr->kind >= ExprKind::Add) {
            auto n = static_cast<const BinaryExprNode *>(e.ptr);
            collectMembers(n->a, d);
            collectMembers(n->b, d);
        }
    }

    int depthOf(const std::vector<Argument> &args) const {
        int d = 0;
        for (const auto &a : args) {
            if (a.isData()) {
                auto it = adt_depth.find(a.getADTPtr().getName());
                d = std::max(d, it == adt_depth.end() ? 0 : it->second);
            } else if (a.isExpr()) {
                d = std::max(d, depthOf(a.getExpr()));
            }
        }
        return std::min(d, depth);
    }

    void visit(const NodePtr &n) {
        switch (n->kind) {
        case NodeKind::Block:
            for (const auto &c : n->children) {
                visit(c);
            }
            break;
        case NodeKind::Allocate: {
            const std::string out = n->call.output.getADTPtr().getName();
            adt_depth[out] = depthOf(n->call.args);
            at_depth[adt_depth[out]].push_back(n);
            break;
        }
        case NodeKind::Free:
            throw error::InternalError("No Frees at this point!");
        case NodeKind::Insert: {
            const std::string data = n->method.data.getName();
            adt_depth[data] = depthOf(n->method.call.args);
            at_depth[adt_depth[data]].push_back(n);
            break;
        }
        case NodeKind::Query: {
            std::vector<Argument> by = n->method.call.args;
            by.push_back(Argument(n->method.data));
            const std::string child = n->child.getName();
            adt_depth[child] = depthOf(by);
            auto &level = at_depth[adt_depth[child]];
            // A data structure that a statement of this scope defines (allocates, computes or queries) is not
            // a parameter of the kernel: a query of it must stay behind that statement.
            const std::string parent = n->method.data.getName();
            bool parent_is_parameter = true;
            for (const auto &earlier : level) {
                if ((earlier->kind == NodeKind::Allocate && earlier->call.output.getADTPtr().getName() == parent) ||
                    (earlier->kind == NodeKind::Compute && earlier->adt.getName() == parent) ||
                    (earlier->kind == NodeKind::Query && earlier->child.getName() == parent)) {
                    parent_is_parameter = false;
                }
            }
            if (adt_depth[child] == 0 && n->method.call.args.empty() && n->method.call.template_args.empty() &&
                !n->insert && parent_is_parameter) {
                // A query that takes nothing (it opens a session on a parameter: a
                // load whose result is needed much later) goes first, behind the
                // launch declarations, so that its latency hides behind what follows.
                auto at = level.begin();
                while (at != level.end() && ((*at)->kind == NodeKind::GridDecl || (*at)->kind == NodeKind::SmemDecl ||
                                             (*at)->kind == NodeKind::Opaque || (*at)->kind == NodeKind::Assert)) {
                    ++at;
                }
                level.insert(at, n);
            } else {
                level.push_back(n);
            }
            break;
        }
        case NodeKind::Compute: {
            const std::string out = n->adt.getName();
            adt_depth[out] = depthOf(n->call.args);
            at_depth[adt_depth[out]].push_back(n);
            break;
        }
        case NodeKind::Interval: {
            const bool mapped = n->isMappedToGrid();
            if (!mapped) {
                depth++;
            }
            const int mine = mapped ? 0 : depth;
            var_depth[n->intervalVariable().getName()] = mine;
            if (mapped && depth > 0) {
                // A grid-mapped range inside an unmapped loop: its index does not depend
                // on the loop, and neither may some of its statements.  Those stay where
                // they are, in the scope around the loop (a copy made there is written
                // back when THAT scope ends, after the loop); the range itself only
                // defines its index, ahead of them.
                const size_t at = at_depth[0].size();
                visit(n->body);
                Node range = *n;
                range.body = block({});
                at_depth[0].insert(at_depth[0].begin() + (std::ptrdiff_t)at, make(std::move(range)));
                break;
            }
            visit(n->body);
            std::vector<NodePtr> body = at_depth[mine];
            at_depth.erase(mine);
            if (!mapped) {
                depth--;
            }
            Node loop = *n;
            loop.body = block(body);
            at_depth[mapped ? 0 : depth].push_back(make(std::move(loop)));
            break;
        }
        case NodeKind::Assert:
            at_depth[std::max(depthOf(n->constraint.getA()), depthOf(n->constraint.getB()))].push_back(n);
            break;
        case NodeKind::GridDecl:
        case NodeKind::SmemDecl:
        case NodeKind::Opaque:
            at_depth[depth].push_back(n);
            break;
        case NodeKind::Blank:
            break;
        }
    }
};

// ---------------------------------------------------------------------------
// Step 3a: reuse temporaries
// ---------------------------------------------------------------------------
class Reuser {
public:
    NodePtr run(const NodePtr &ir) {
        scan(ir);
        // head of a reuse group -> members
        std::map<std::string, std::vector<std::string>> groups;
        for (const auto &entry : alloc_calls) {
            const std::string &cur = entry.first;
            bool placed = false;
            for (auto &g : groups) {
                std::vector<std::string> members = g.second;
                members.push_back(g.first);
                bool ok = true;
                for (const auto &m : members) {
                    if (range.at(m).second > range.at(cur).first ||
                        !isSameFunctionCall(entry.second, alloc_calls.at(m))) {
                        ok = false;
                        break;
                    }
                }
                if (ok) {
                    g.second.push_back(cur);
                    placed = true;
                    break;
                }
            }
            if (!placed) {
                groups[cur] = {};
            }
        }
        for (const auto &g : groups) {
            for (const auto &m : g.second) {
                rewrites[adts.at(m)] = adts.at(g.first);
            }
        }
        return rewrites.empty() ? ir : rewrite(ir);
    }

private:
    int line = 0;
    std::map<std::string, std::pair<int, int>> range;  // first, last use
    std::map<std::string, FunctionCall> alloc_calls;
    std::map<std::string, AbstractDataTypePtr> adts;
    std::map<AbstractDataTypePtr, AbstractDataTypePtr> rewrites;

    void touch(const AbstractDataTypePtr &adt) {
        if (!adt.defined()) {
            return;
        }
        const std::string n = adt.getName();
        adts[n] = adt;
        auto it = range.find(n);
        if (it == range.end()) {
            range[n] = {line, line};
        } else {
            it->second.second = line;
        }
    }

    void touchArgs(const std::vector<Argument> &args) {
        for (const auto &a : args) {
            if (a.isData()) {
                touch(a.getADTPtr());
            }
        }
    }

    void scan(const NodePtr &n) {
        switch (n->kind) {
        case NodeKind::Block:
            for (const auto &c : n->children) {
                scan(c);
            }
            break;
        case NodeKind::Allocate:
            line++;
            touch(n->call.output.getADTPtr());
            alloc_calls[n->call.output.getADTPtr().getName()] = n->call;
            break;
        case NodeKind::Free:
            line++;
            touch(n->method.data);
            break;
        case NodeKind::Insert:
            line++;
            touch(n->method.data);
            touchArgs(n->method.call.args);
            break;
        case NodeKind::Query:
            line++;
            touch(n->parent);
            touch(n->method.data);
            touch(n->child);
            break;
        case NodeKind::Compute:
            line++;
            touch(n->adt);
            touchArgs(n->call.args);
            break;
        case NodeKind::Interval:
            line++;
            scan(n->body);
            break;
        case NodeKind::GridDecl:
            line++;
            break;
        case NodeKind::Opaque:
            touchArgs(n->call.args);
            break;
        default:
            break;
        }
    }

    AbstractDataTypePtr renamed(const AbstractDataTypePtr &adt) const {
        if (!adt.defined()) {
            return adt;
        }
        auto it = rewrites.find(adt);
        return it == rewrites.end() ? adt : it->second;
    }

    NodePtr rewrite(const NodePtr &n) const {
        Node out = *n;
        switch (n->kind) {
        case NodeKind::Block:
            for (auto &c : out.children) {
                c = rewrite(c);
            }
            break;
        case NodeKind::Allocate:
            if (rewrites.count(n->call.output.getADTPtr())) {
                return blank();
            }
            break;
        case NodeKind::Insert:
            out.method.call = n->method.call.replaceAllDS(rewrites);
            break;
        case NodeKind::Query:
            out.method = MethodCall{renamed(n->method.data), n->method.call.replaceAllDS(rewrites)};
            out.parent = renamed(n->parent);
            out.child = renamed(n->child);
            break;
        case NodeKind::Compute:
            out.call = n->call.replaceAllDS(rewrites);
            out.adt = renamed(n->adt);
            break;
        case NodeKind::Interval:
            out.body = rewrite(n->body);
            break;
        case NodeKind::Opaque:
            out.call = n->call.replaceAllDS(rewrites);
            break;
        default:
            break;
        }
        return make(std::move(out));
    }
};

// ---------------------------------------------------------------------------
// Step 3b: frees and deferred inserts at scope exits
// ---------------------------------------------------------------------------
class Closer {
public:
    NodePtr run(const NodePtr &ir) {
        open();
        std::vector<NodePtr> out{visit(ir)};
        close(out);
        return block(out);
    }

private:
    struct Pending {
        std::map<std::string, AbstractDataTypePtr> to_free;
        std::vector<NodePtr> to_insert;
    };
    std::vector<Pending> pending;

    void open() {
        pending.emplace_back();
    }

    void close(std::vector<NodePtr> &out) {
        Pending p = std::move(pending.back());
        pending.pop_back();
        for (const auto &f : p.to_free) {
            Node n;
            n.kind = NodeKind::Free;
            FunctionCall call;
            call.name = f.second.getFreeFunction().name;
            call.access = HOST;
            n.method = MethodCall{f.second, call};
            out.push_back(make(std::move(n)));
        }
        // innermost query first
        for (auto it = p.to_insert.rbegin(); it != p.to_insert.rend(); ++it) {
            out.push_back(*it);
        }
    }

    NodePtr visit(const NodePtr &n) {
        switch (n->kind) {
        case NodeKind::Block: {
            Node out = *n;
            for (auto &c : out.children) {
                c = visit(c);
            }
            return make(std::move(out));
        }
        case NodeKind::Allocate: {
            AbstractDataTypePtr adt = n->call.output.getADTPtr();
            if (adt.freeAlloc()) {
                pending.back().to_free[adt.getName()] = adt;
            }
            return n;
        }
        case NodeKind::Query:
            if (n->child.freeQuery()) {
                pending.back().to_free[n->child.getName()] = n->child;
            }
            if (n->insert && n->parent.insertQuery()) {
                pending.back().to_insert.push_back(n->insert_node);
            }
            return n;
        case NodeKind::Interval: {
            open();
            std::vector<NodePtr> body{visit(n->body)};
            close(body);
            Node out = *n;
            out.body = block(body);
            return make(std::move(out));
        }
        default:
            return n;
        }
    }
};

const char *kindName(NodeKind k) {
    switch (k) {
    case NodeKind::Block:
        return "block";
    case NodeKind::Allocate:
        return "allocate";
    case NodeKind::Free:
        return "free";
    case NodeKind::Insert:
        return "insert";
    case NodeKind::Query:
        return "query";
    case NodeKind::Compute:
        return "compute";
    case NodeKind::Interval:
        return "interval";
    case NodeKind::Assert:
        return "assert";
    case NodeKind::GridDecl:
        return "grid";
    case NodeKind::SmemDecl:
        return "smem";
    case NodeKind::Opaque:
        return "opaque";
    case NodeKind::Blank:
        return "blank";
    }
    return "?";
}

void print(std::ostream &os, const NodePtr &n, int indent) {
    auto pad = [&]() {
        for (int i = 0; i < indent; i++) {
            os << "  ";
        }
    };
    switch (n->kind) {
    case NodeKind::Block:
        for (const auto &c : n->children) {
            print(os, c, indent);
        }
        break;
    case NodeKind::Blank:
        break;
    case NodeKind::Interval:
        pad();
        os << "interval " << Stmt(n->start) << " < " << n->end << " step " << n->step;
        if (n->isMappedToGrid()) {
            os << " over " << n->unit;
        }
        os << " {\n";
        print(os, n->body, indent + 1);
        pad();
        os << "}\n";
        break;
    case NodeKind::Allocate:
    case NodeKind::Compute:
    case NodeKind::Opaque:
        pad();
        os << kindName(n->kind) << " " << n->call << "\n";
        break;
    case NodeKind::Free:
    case NodeKind::Insert:
    case NodeKind::Query:
        pad();
        os << kindName(n->kind) << " " << n->method << "\n";
        break;
    case NodeKind::Assert:
        pad();
        os << "assert " << n->constraint << "\n";
        break;
    case NodeKind::GridDecl:
        pad();
        os << "grid " << n->dim << " = " << n->var << "\n";
        break;
    case NodeKind::SmemDecl:
        if (n->var.defined()) {
            pad();
            os << "smem " << n->var << "\n";
        }
        break;
    }
}

}  // namespace

AbstractDataTypePtr makeQueried(const std::string &name, const std::string &type, AbstractDataTypePtr from) {
    return AbstractDataTypePtr(new const DerivedADT(name, type, from));
}

NodePtr concretize(Composable program) {
    Concretizer c;
    return c.run(program);
}

NodePtr lowerProgram(Composable program) {
    NodePtr ir = concretize(program);
    ir = Hoister().run(ir);
    ir = Reuser().run(ir);
    ir = Closer().run(ir);
    return ir;
}

std::ostream &operator<<(std::ostream &os, const NodePtr &n) {
    if (n) {
        print(os, n, 0);
    }
    return os;
}

}  // namespace lower
}  // namespace gern
