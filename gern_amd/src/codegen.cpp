// Source-text emission for the two targets (HIP kernel for gfx950, host C++);
// see gern/codegen/codegen.h.
#include "gern/codegen/codegen.h"

#include <algorithm>
#include <optional>
#include <sstream>

namespace gern {
namespace codegen {

// ---------------------------------------------------------------------------
// Host-side evaluation
// ---------------------------------------------------------------------------
bool evaluate(const Expr &e, const EvalEnv &env, int64_t &value) {
    if (!e.defined()) {
        return false;
    }
    switch (e.ptr->kind) {
    case ExprKind::Literal:
        value = static_cast<const LiteralNode *>(e.ptr)->i;
        return true;
    case ExprKind::Variable: {
        auto v = static_cast<const VariableNode *>(e.ptr);
        if (v->bound) {
            value = v->val;
            return true;
        }
        return env.variable && env.variable(v->name, value);
    }
    case ExprKind::ADTMember: {
        auto m = static_cast<const ADTMemberNode *>(e.ptr);
        return env.member && env.member(m->ds, m->member, value);
    }
    case ExprKind::GridDim:
        return false;
    default: {
        auto n = static_cast<const BinaryExprNode *>(e.ptr);
        int64_t a, b;
        if (!evaluate(n->a, env, a) || !evaluate(n->b, env, b)) {
            return false;
        }
        switch (n->kind) {
        case ExprKind::Add:
            value = a + b;
            return true;
        case ExprKind::Sub:
            value = a - b;
            return true;
        case ExprKind::Mul:
            value = a * b;
            return true;
        case ExprKind::Div:
            if (b == 0) {
                return false;
            }
            value = a / b;
            return true;
        case ExprKind::Mod:
            if (b == 0) {
                return false;
            }
            value = a % b;
            return true;
        default:
            return false;
        }
    }
    }
}

bool evaluate(const Constraint &c, const EvalEnv &env, bool &value) {
    if (!c.defined()) {
        return false;
    }
    int64_t a, b;
    if (!evaluate(c.getA(), env, a) || !evaluate(c.getB(), env, b)) {
        return false;
    }
    switch (c.ptr->kind) {
    case ConstraintKind::Eq:
        value = a == b;
        break;
    case ConstraintKind::Neq:
        value = a != b;
        break;
    case ConstraintKind::Leq:
        value = a <= b;
        break;
    case ConstraintKind::Geq:
        value = a >= b;
        break;
    case ConstraintKind::Less:
        value = a < b;
        break;
    case ConstraintKind::Greater:
        value = a > b;
        break;
    case ConstraintKind::And:
        value = a && b;
        break;
    case ConstraintKind::Or:
        value = a || b;
        break;
    }
    return true;
}

namespace {

using lower::Node;
using lower::NodeKind;
using lower::NodePtr;

const char *op(ExprKind k) {
    switch (k) {
    case ExprKind::Add:
        return "+";
    case ExprKind::Sub:
        return "-";
    case ExprKind::Mul:
        return "*";
    case ExprKind::Div:
        return "/";
    default:
        return "%";
    }
}

const char *op(ConstraintKind k) {
    switch (k) {
    case ConstraintKind::Eq:
        return "==";
    case ConstraintKind::Neq:
        return "!=";
    case ConstraintKind::Leq:
        return "<=";
    case ConstraintKind::Geq:
        return ">=";
    case ConstraintKind::Less:
        return "<";
    case ConstraintKind::Greater:
        return ">";
    case ConstraintKind::And:
        return "&&";
    default:
        return "||";
    }
}

class Emitter {
public:
    Emitter(bool device, const GeneratorOptions &options)
        : device(device), options(options) {
        for (Grid::Dim d : {Grid::GRID_DIM_X, Grid::GRID_DIM_Y, Grid::GRID_DIM_Z, Grid::BLOCK_DIM_X,
                            Grid::BLOCK_DIM_Y, Grid::BLOCK_DIM_Z}) {
            dims[d] = {{Expr(1)}, {}};
        }
        for (Grid::Dim d : {Grid::WARP_DIM_X, Grid::WARP_DIM_Y, Grid::WARP_DIM_Z}) {
            dims[d] = {{Expr(Grid::kWavefrontSize)}, {}};
        }
    }

    const bool device;
    bool device_function = false;
    const GeneratorOptions options;
    std::ostringstream body;
    std::set<std::string> headers;
    std::set<std::string> declared_vars, declared_adts;
    std::map<std::string, Variable> used_vars;
    std::map<std::string, AbstractDataTypePtr> used_adts;
    // per launch dimension: a stack (outermost first) of the extents claimed
    // at each nesting level
    std::map<Grid::Dim, std::vector<std::vector<Expr>>> dims;
    std::map<Grid::Dim, Variable> explicit_dims;
    Variable smem_size;
    std::vector<Constraint> host_asserts;
    bool uses_block_units = false;

    Expr currentDim(Grid::Dim d) {
        auto ex = explicit_dims.find(d);
        if (ex != explicit_dims.end()) {
            return ex->second;
        }
        const auto &innermost = dims[d].back();
        if (innermost.empty()) {
            return getLevel(d) == Grid::Level::THREADS_WARPS ? Expr(Grid::kWavefrontSize) : Expr(1);
        }
        return innermost.front();
    }

    std::string gen(const Expr &e) {
        if (!e.defined()) {
            return "";
        }
        switch (e.ptr->kind) {
        case ExprKind::Literal: {
            auto n = static_cast<const LiteralNode *>(e.ptr);
            std::ostringstream os;
            if (n->isFloating()) {
                os << n->f;
            } else {
                os << n->i;
            }
            return os.str();
        }
        case ExprKind::Variable: {
            Variable v = to<Variable>(e);
            used_vars.emplace(v.getName(), v);
            return v.getName();
        }
        case ExprKind::ADTMember: {
            auto n = static_cast<const ADTMemberNode *>(e.ptr);
            return gen(n->ds) + "." + n->member;
        }
        case ExprKind::GridDim:
            return gen(currentDim(static_cast<const GridDimNode *>(e.ptr)->dim));
        default: {
            auto n = static_cast<const BinaryExprNode *>(e.ptr);
            return "(" + gen(n->a) + " " + op(n->kind) + " " + gen(n->b) + ")";
        }
        }
    }

    std::string gen(const Constraint &c) {
        return "(" + gen(c.getA()) + " " + op(c.ptr->kind) + " " + gen(c.getB()) + ")";
    }

    std::string gen(const AbstractDataTypePtr &ds) {
        used_adts.emplace(ds.getName(), ds);
        return ds.getName();
    }

    std::string gen(const Argument &a) {
        return a.isData() ? gen(a.getADTPtr()) : gen(a.getExpr());
    }

    std::string genCall(const FunctionCall &f, const std::string &prefix = "") {
        std::ostringstream os;
        os << prefix << f.name;
        if (!f.template_args.empty()) {
            os << "<";
            for (size_t i = 0; i < f.template_args.size(); i++) {
                // A template argument is a compile-time value: every variable
                // in it must have been bound (reference: the same complaint is
                // raised for the generated function's own template
                // parameters, src/codegen/codegen.cpp:179-183).
                const Argument &targ = f.template_args[i];
                for (const auto &v : targ.isExpr() ? getVariables(targ.getExpr()) : std::set<Variable>{}) {
                    if (!v.isConstExpr()) {
                        throw error::UserError(v.getName() + " must be bound to an int64_t, it is a template argument of " +
                                               f.name);
                    }
                }
                os << (i ? ", " : "") << gen(f.template_args[i]);
            }
            os << ">";
        }
        os << "(";
        for (size_t i = 0; i < f.args.size(); i++) {
            os << (i ? ", " : "") << gen(f.args[i]);
        }
        os << ")";
        return os.str();
    }

    void line(int indent, const std::string &text) {
        for (int i = 0; i < indent; i++) {
            body << "    ";
        }
        body << text << "\n";
    }

    void callStatement(int indent, const FunctionCall &f, const std::string &prefix = "") {
        std::string call = genCall(f, prefix);
        if (f.output.defined()) {
            std::string type = f.output.getType();
            std::string name = f.output.isData() ? f.output.getADTPtr().getName() : f.output.getVar().getName();
            if (f.output.isData()) {
                declared_adts.insert(name);
                used_adts.emplace(name, f.output.getADTPtr());
            } else {
                declared_vars.insert(name);
            }
            line(indent, type + " " + name + " = " + call + ";");
        } else {
            line(indent, call + ";");
        }
    }

    std::string unitIndex(Grid::Unit u) {
        if (!device) {
            throw error::UserError("a loop is distributed over a grid unit, but the program is not wrapped in Global()");
        }
        const std::string w = std::to_string(Grid::kWavefrontSize);
        switch (u) {
        case Grid::BLOCK_X:
            uses_block_units = true;
            return (options.xcd_remap || options.xcd_tile_blocks) ? "gern_block_x" : "blockIdx.x";
        case Grid::BLOCK_Y:
            uses_block_units = true;
            return (options.xcd_remap || options.xcd_tile_blocks) ? "gern_block_y" : "blockIdx.y";
        case Grid::BLOCK_Z:
            uses_block_units = true;
            return (options.xcd_remap || options.xcd_tile_blocks) ? "gern_block_z" : "blockIdx.z";
        case Grid::THREAD_X:
            return "threadIdx.x";
        case Grid::THREAD_Y:
            return "threadIdx.y";
        case Grid::THREAD_Z:
            return "threadIdx.z";
        case Grid::WARP_X:
            return "(threadIdx.x / " + w + ")";
        case Grid::WARP_Y:
            return "(threadIdx.y / " + w + ")";
        case Grid::WARP_Z:
            return "(threadIdx.z / " + w + ")";
        case Grid::THREAD_X_IN_WRAPS:
            return "(threadIdx.x % " + w + ")";
        case Grid::THREAD_Y_IN_WRAPS:
            return "(threadIdx.y % " + w + ")";
        case Grid::THREAD_Z_IN_WRAPS:
            return "(threadIdx.z % " + w + ")";
        default:
            throw error::InternalError("Undefined Grid unit Passed!");
        }
    }

    void emit(const NodePtr &n, int indent) {
        switch (n->kind) {
        case NodeKind::Block:
            for (const auto &c : n->children) {
                emit(c, indent);
            }
            break;
        case NodeKind::Blank:
            break;
        case NodeKind::Allocate:
            callStatement(indent, n->call);
            break;
        case NodeKind::Free:
            if (!declared_adts.count(n->method.data.getName())) {
                throw error::InternalError("Freeing a data-structure that hasn't been allocated??");
            }
            callStatement(indent, n->method.call, gen(n->method.data) + ".");
            break;
        case NodeKind::Insert:
        case NodeKind::Query:
            callStatement(indent, n->method.call, gen(n->method.data) + ".");
            if (n->kind == NodeKind::Query) {
                gen(n->parent);
            }
            break;
        case NodeKind::Compute:
            callStatement(indent, n->call);
            headers.insert(n->headers.begin(), n->headers.end());
            break;
        case NodeKind::Opaque:
            callStatement(indent, n->call);
            headers.insert(n->headers.begin(), n->headers.end());
            break;
        case NodeKind::Interval:
            emitInterval(n, indent);
            break;
        case NodeKind::Assert:
            emitAssert(n, indent);
            break;
        case NodeKind::GridDecl:
            gen(Expr(n->var));
            explicit_dims[n->dim] = n->var;
            break;
        case NodeKind::SmemDecl:
            smem_size = n->var;
            break;
        }
    }

    static constexpr int64_t kUnrollTrips = 32;
    int loop_depth = 0;  // loops (not grid-mapped ranges) around the statement being emitted

    // The value of an index expression when every variable in it is bound to a number.
    static std::optional<int64_t> constantValue(const Expr &e) {
        if (e.ptr == nullptr) {
            return std::nullopt;
        }
        const ExprNode *n = e.ptr;
        switch (n->kind) {
        case ExprKind::Literal:
            return static_cast<const LiteralNode *>(n)->i;
        case ExprKind::Variable: {
            const Variable v = to<Variable>(e);
            return v.isBound() ? std::optional<int64_t>(v.getInt64Val()) : std::nullopt;
        }
        case ExprKind::ADTMember:
        case ExprKind::GridDim:
            return std::nullopt;
        default:
            break;
        }
        const auto *b = static_cast<const BinaryExprNode *>(n);
        const auto x = constantValue(b->a), y = constantValue(b->b);
        if (!x || !y) {
            return std::nullopt;
        }
        switch (n->kind) {
        case ExprKind::Add:
            return *x + *y;
        case ExprKind::Sub:
            return *x - *y;
        case ExprKind::Mul:
            return *x * *y;
        case ExprKind::Div:
            return *y == 0 ? std::nullopt : std::optional<int64_t>(*x / *y);
        case ExprKind::Mod:
            return *y == 0 ? std::nullopt : std::optional<int64_t>(*x % *y);
        default:
            return std::nullopt;
        }
    }

    // True if a loop (not a grid-mapped range) lies anywhere below n.
    static bool containsLoop(const NodePtr &n) {
        if (!n) {
            return false;
        }
        if (n->kind == NodeKind::Interval) {
            return !n->isMappedToGrid() || containsLoop(n->body);
        }
        for (const auto &c : n->children) {
            if (containsLoop(c)) {
                return true;
            }
        }
        return false;
    }

    void emitInterval(const NodePtr &n, int indent) {
        const Variable index = n->intervalVariable();
        const Expr extent = n->end - n->start.getB();
        Expr ceil = (n->step + extent - 1) / n->step;

        if (!n->isMappedToGrid()) {
            declared_vars.insert(index.getName());
            std::string i = index.getName();
            // An innermost loop of a few steps, inside another loop, whose bounds are all bound at generation
            // time is unrolled: per-thread register tiles indexed by the loop variable (RegTile::get_view) then
            // have constant indices; indexed by a variable they live in scratch memory.  (The outermost loop
            // of a kernel is the one that stages tiles and meets at barriers: that one stays a loop.)
            const auto trips = constantValue(ceil);
            if (loop_depth > 0 && trips && *trips > 1 && *trips <= kUnrollTrips && !containsLoop(n->body)) {
                line(indent, "#pragma unroll");
            }
            loop_depth++;
            line(indent, "for (int64_t " + i + " = " + gen(n->start.getB()) + "; " + i + " < " + gen(n->end) + "; " +
                             i + " = " + i + " + " + gen(n->step) + ") {");
            emit(n->body, indent + 1);
            line(indent, "}");
            loop_depth--;
            return;
        }

        const Grid::Dim dim = getDim(n->unit);
        // The body is emitted first (into a side buffer) because loops nested
        // inside it and mapped to the same dimension claim the low part of the
        // unit index, and this loop must divide by what they claimed.
        dims[dim].emplace_back();
        std::ostringstream saved;
        saved.swap(body);
        emit(n->body, indent);
        std::string body_text = body.str();
        body.swap(saved);
        std::vector<Expr> claimed = dims[dim].back();
        dims[dim].pop_back();

        Expr inner = claimed.empty() ? Expr(1) : claimed.front();
        Expr span = ceil;
        if (getLevel(n->unit) == Grid::Level::WARPS) {
            span = ceil * Expr(Grid::kWavefrontSize);
        }
        dims[dim].back().insert(dims[dim].back().begin(), inner * span);

        declared_vars.insert(index.getName());
        line(indent, "int64_t " + index.getName() + " = (((" + unitIndex(n->unit) + " / " + gen(inner) + ") % " +
                         gen(ceil) + ") * " + gen(n->step) + ") + " + gen(n->start.getB()) + ";");
        body << body_text;
    }

    void emitAssert(const NodePtr &n, int indent) {
        Substitution s;
        for (const auto &d : dims) {
            s.dims[d.first] = currentDim(d.first);
        }
        Constraint c = substitute(n->constraint, s);
        if (isConstExpr(c)) {
            line(indent, "static_assert(" + gen(c) + ");");
        } else if (device_function) {
            // Nobody checks a precondition of a device function that is not a
            // launch; it is recorded for the reader only.
            line(indent, "// assumes " + gen(c));
        } else if (!device) {
            line(indent, "assert(" + gen(c) + ");");
        } else {
            // Device code never traps; the Runner checks this before launch
            // and refuses the launch when it does not hold.  The kernel may
            // therefore rely on it: the compiler is told, which lets it, for
            // one, see that a loop over a single tile runs once.
            line(indent, "__builtin_assume(" + gen(c) + ");");
            host_asserts.push_back(c);
        }
    }
};

}  // namespace

std::string CodeGenerator::generate_code(Composable c) {
    const bool device = c.isDeviceLaunch();
    // A program made of device gernels (its calls occupy grid units) that is
    // not wrapped in Global() is not launched: it becomes a __device__ function
    // that another generated kernel calls (FunctionPtr).  The reference only
    // ever exercised FunctionPtr on the host (test/test-function-ptr.cpp).
    const bool device_function =
        !device && c.defined() && getLevel(c.getAnnotation().getOccupiedUnits()) >= Grid::Level::SCALAR;
    NodePtr ir = lower::lowerProgram(c);

    Emitter em(device, options);
    em.device_function = device_function;
    em.emit(ir, 1);

    plan = LaunchPlan();
    plan.device = device;
    plan.device_function = device_function;
    plan.function_name = getUniqueName("function");

    plan.grid[0] = em.currentDim(Grid::GRID_DIM_X);
    plan.grid[1] = em.currentDim(Grid::GRID_DIM_Y);
    plan.grid[2] = em.currentDim(Grid::GRID_DIM_Z);
    plan.block[0] = em.currentDim(Grid::BLOCK_DIM_X);
    plan.block[1] = em.currentDim(Grid::BLOCK_DIM_Y);
    plan.block[2] = em.currentDim(Grid::BLOCK_DIM_Z);
    plan.lds_bytes = em.smem_size;
    plan.host_asserts = em.host_asserts;
    // Launch dimensions are evaluated by the caller, so whatever they mention
    // is an input of the generated function too.
    for (int i = 0; i < 3; i++) {
        em.gen(plan.grid[i]);
        em.gen(plan.block[i]);
    }
    em.gen(Expr(plan.lds_bytes));

    // Data structures that are used but never produced inside are the true
    // inputs and outputs; variables that are used but never declared are
    // either template parameters (compile-time, must be bound) or run-time
    // parameters.  Both lists are ordered by name.
    std::vector<Parameter> parameters;
    for (const auto &a : em.used_adts) {
        if (!em.declared_adts.count(a.first)) {
            parameters.push_back(Parameter(a.second));
        }
    }
    std::vector<Variable> template_args;
    for (const auto &v : em.used_vars) {
        if (em.declared_vars.count(v.first)) {
            continue;
        }
        if (v.second.isConstExpr()) {
            if (!v.second.isBound()) {
                throw error::UserError(v.first + " must be bound to an int64_t, it is a template parameter");
            }
            template_args.push_back(v.second);
        } else {
            parameters.push_back(Parameter(v.second));
        }
    }
    if (ordered_parameters.has_value()) {
        if (!same_parameters(ordered_parameters.value(), parameters)) {
            throw error::UserError("provided ordered arguments dont match the parameters needed for the function");
        }
        parameters = ordered_parameters.value();
    }
    argument_order = get_parameter_names(parameters);
    plan.parameters = parameters;
    plan.template_args = template_args;
    headers = em.headers;

    signature = FunctionSignature();
    signature.name = plan.function_name;
    signature.args = parameters;
    signature.template_args = template_args;
    signature.device = device || device_function;
    signature.access = device ? GLOBAL : (device_function ? DEVICE : HOST);
    signature.grid = LaunchArguments{plan.grid[0], plan.grid[1], plan.grid[2]};
    signature.block = LaunchArguments{plan.block[0], plan.block[1], plan.block[2]};
    signature.smem_size = em.smem_size;

    std::ostringstream name_expr;
    name_expr << plan.function_name;
    if (!template_args.empty()) {
        name_expr << "<";
        for (size_t i = 0; i < template_args.size(); i++) {
            name_expr << (i ? ", " : "") << template_args[i].getInt64Val();
        }
        name_expr << ">";
    }
    plan.name_expression = name_expr.str();

    // ---- assemble the file -------------------------------------------------
    std::ostringstream out;
    if (device || device_function) {
        out << "// HIP device code for gfx950, generated by Gern.\n"
               "#if defined(__HIPCC_RTC__)\n"
               "using __hip_internal::int32_t;\n"
               "using __hip_internal::int64_t;\n"
               "using __hip_internal::uint32_t;\n"
               "using __hip_internal::uint64_t;\n"
               "#else\n"
               "#include <cstdint>\n"
               "#include <hip/hip_runtime.h>\n"
               "#endif\n";
    } else {
        out << "#include <cassert>\n#include <cstdint>\n";
    }
    for (const auto &h : em.headers) {
        out << "#include \"" << h << "\"\n";
    }
    out << "\n";
    if (!template_args.empty()) {
        out << "template<";
        for (size_t i = 0; i < template_args.size(); i++) {
            out << (i ? ", " : "") << "int64_t " << template_args[i].getName();
        }
        out << ">\n";
    }
    if (device) {
        out << "__global__ void ";
        // The block shape is usually fixed by bound tile sizes; telling the
        // compiler lifts its default 1024-thread register budget.
        EvalEnv none;
        int64_t bx, by, bz;
        if (evaluate(plan.block[0], none, bx) && evaluate(plan.block[1], none, by) &&
            evaluate(plan.block[2], none, bz) && bx * by * bz > 0 && bx * by * bz <= 1024) {
            out << "__launch_bounds__(" << (bx * by * bz);
            if (options.min_waves_per_simd > 0) {
                out << ", " << options.min_waves_per_simd;
            }
            out << ") ";
        }
    } else if (device_function) {
        out << "__device__ __forceinline__ void ";
    } else {
        out << "void ";
    }
    out << plan.function_name << "(";
    for (size_t i = 0; i < parameters.size(); i++) {
        const Parameter &p = parameters[i];
        std::string name = p.isData() ? p.getADTPtr().getName() : p.getVar().getName();
        // Host functions take data structures by reference (the callee's
        // insert must reach the caller's object); variables go by value, so
        // that a caller may pass a compile-time constant.
        out << (i ? ", " : "") << p.getType() << ((device || !p.isData()) ? " " : " &") << name;
    }
    out << ") {\n";
    if (device && em.uses_block_units && options.xcd_tile_blocks) {
        // Workgroups are handed to the 8 XCDs round-robin in launch order, so
        // the l-th workgroup of XCD x has launch number 8 l + x.  The 32 that
        // an XCD runs at a time (one per CU) take a block of 4 x 8 tiles:
        // block number (l / 32) * 8 + x, tile l % 32 inside it.
        out << "    const unsigned gern_nbx = gridDim.x, gern_nby = gridDim.y;\n"
               "    unsigned gern_bx = blockIdx.x, gern_by = blockIdx.y;\n"
               "    if (gern_nbx % 4u == 0u && gern_nby % 8u == 0u && (gern_nbx * gern_nby) % 256u == 0u) {\n"
               "        const unsigned gern_wg = blockIdx.x + gern_nbx * blockIdx.y;\n"
               "        const unsigned gern_l = gern_wg / 8u;\n"
               "        const unsigned gern_sb = (gern_l / 32u) * 8u + gern_wg % 8u;\n"
               "        gern_bx = (gern_sb % (gern_nbx / 4u)) * 4u + gern_l % 4u;\n"
               "        gern_by = (gern_sb / (gern_nbx / 4u)) * 8u + (gern_l % 32u) / 4u;\n"
               "    }\n"
               "    const int64_t gern_block_x = gern_bx;\n"
               "    const int64_t gern_block_y = gern_by;\n"
               "    const int64_t gern_block_z = blockIdx.z;\n"
               "    (void)gern_block_x; (void)gern_block_y; (void)gern_block_z;\n";
    } else if (device && em.uses_block_units && options.xcd_remap && options.xcd_band_rows > 0) {
        // The same idea with shorter runs: XCD x takes bands x, x + 8, x + 16, ... of `xcd_band_rows` rows of
        // tiles each (a row = gridDim.x tiles), so that at any time the eight XCDs work side by side in one
        // window of the data instead of in eight places an eighth of the data apart.  Launch numbers past the
        // last whole group of eight bands keep their tiles.
        out << "    const unsigned gern_nbx = gridDim.x, gern_nby = gridDim.y;\n"
               "    unsigned gern_wg = blockIdx.x + gern_nbx * (blockIdx.y + gern_nby * blockIdx.z);\n"
               "    {\n"
               "        const unsigned gern_band = " << options.xcd_band_rows << "u * gern_nbx;\n"
               "        const unsigned gern_whole = ((gern_nbx * gern_nby * gridDim.z) / (8u * gern_band)) * (8u * gern_band);\n"
               "        if (gern_wg < gern_whole) {\n"
               "            const unsigned gern_l = gern_wg / 8u;\n"
               "            gern_wg = ((gern_l / gern_band) * 8u + gern_wg % 8u) * gern_band + gern_l % gern_band;\n"
               "        }\n"
               "    }\n"
               "    const int64_t gern_block_x = gern_wg % gern_nbx;\n"
               "    const int64_t gern_block_y = (gern_wg / gern_nbx) % gern_nby;\n"
               "    const int64_t gern_block_z = gern_wg / (gern_nbx * gern_nby);\n"
               "    (void)gern_block_x; (void)gern_block_y; (void)gern_block_z;\n";
    } else if (device && em.uses_block_units && options.xcd_remap) {
        // Workgroups are handed to the 8 XCDs round-robin in launch order.
        // Renumbering them so that each XCD walks a contiguous run of tiles
        // keeps halo and shared-line traffic inside one XCD's L2.
        out << "    const unsigned gern_nbx = gridDim.x, gern_nby = gridDim.y;\n"
               "    unsigned gern_wg = blockIdx.x + gern_nbx * (blockIdx.y + gern_nby * blockIdx.z);\n"
               "    const unsigned gern_per_xcd = (gern_nbx * gern_nby * gridDim.z) / 8u;\n"
               "    if (gern_wg < gern_per_xcd * 8u) {\n"
               "        gern_wg = (gern_wg % 8u) * gern_per_xcd + gern_wg / 8u;\n"
               "    }\n"
               "    const int64_t gern_block_x = gern_wg % gern_nbx;\n"
               "    const int64_t gern_block_y = (gern_wg / gern_nbx) % gern_nby;\n"
               "    const int64_t gern_block_z = gern_wg / (gern_nbx * gern_nby);\n"
               "    (void)gern_block_x; (void)gern_block_y; (void)gern_block_z;\n";
    }
    out << em.body.str();
    out << "}\n";

    if (!device && !device_function) {
        out << "\nextern \"C\" {\nvoid hook_" << plan.function_name << "(void **args) {\n";
        for (const auto &t : template_args) {
            out << "    constexpr int64_t " << t.getName() << " = " << t.getInt64Val() << ";\n";
        }
        for (size_t i = 0; i < parameters.size(); i++) {
            const Parameter &p = parameters[i];
            std::string name = p.isData() ? p.getADTPtr().getName() : p.getVar().getName();
            out << "    " << p.getType() << " &" << name << " = *((" << p.getType() << " *)args[" << i << "]);\n";
        }
        out << "    " << plan.function_name;
        if (!template_args.empty()) {
            out << "<";
            for (size_t i = 0; i < template_args.size(); i++) {
                out << (i ? ", " : "") << template_args[i].getName();
            }
            out << ">";
        }
        out << "(";
        for (size_t i = 0; i < parameters.size(); i++) {
            const Parameter &p = parameters[i];
            out << (i ? ", " : "") << (p.isData() ? p.getADTPtr().getName() : p.getVar().getName());
        }
        out << ");\n}\n}\n";
    }
    return out.str();
}

}  // namespace codegen
}  // namespace gern
