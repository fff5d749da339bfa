// Expressions, constraints and annotation statements: construction, printing,
// structural queries and substitution.
#include "gern/core/function.h"
#include "gern/core/lang.h"

#include <sstream>

namespace gern {

// ---------------------------------------------------------------------------
// unique names
// ---------------------------------------------------------------------------
static std::atomic<int> name_counter{0};

std::string getUniqueName(const std::string &prefix) {
    int n = ++name_counter;
    return prefix + "_" + std::to_string(n);
}

// ---------------------------------------------------------------------------
// Datatype
// ---------------------------------------------------------------------------
int Datatype::getNumBits() const {
    switch (kind) {
    case Bool:
    case UInt8:
    case Int8:
        return 8;
    case UInt16:
    case Int16:
        return 16;
    case UInt32:
    case Int32:
    case Float32:
        return 32;
    case UInt64:
    case Int64:
    case Float64:
    case Complex64:
        return 64;
    case Complex128:
        return 128;
    default:
        return 0;
    }
}

std::string Datatype::str() const {
    switch (kind) {
    case Bool:
        return "bool";
    case UInt8:
        return "uint8_t";
    case UInt16:
        return "uint16_t";
    case UInt32:
        return "uint32_t";
    case UInt64:
        return "uint64_t";
    case Int8:
        return "int8_t";
    case Int16:
        return "int16_t";
    case Int32:
        return "int32_t";
    case Int64:
        return "int64_t";
    case Float32:
        return "float";
    case Float64:
        return "double";
    case Complex64:
        return "float complex";
    case Complex128:
        return "double complex";
    default:
        return "Undefined";
    }
}

std::ostream &operator<<(std::ostream &os, const Datatype &t) {
    return os << t.str();
}

// ---------------------------------------------------------------------------
// Expr construction
// ---------------------------------------------------------------------------
Expr::Expr(uint32_t v)
    : Expr(new const LiteralNode(v)) {
}
Expr::Expr(uint64_t v)
    : Expr(new const LiteralNode(v)) {
}
Expr::Expr(int32_t v)
    : Expr(new const LiteralNode(v)) {
}
Expr::Expr(int64_t v)
    : Expr(new const LiteralNode(v)) {
}
Expr::Expr(double v)
    : Expr(new const LiteralNode(v)) {
}
Expr::Expr(Grid::Dim dim)
    : Expr(new const GridDimNode(dim)) {
}

Datatype Expr::getType() const {
    // The type of the last variable met in a left-to-right walk; a lone
    // variable, the only case the code generator asks about, gives its own.
    Datatype t;
    for (const auto &v : getVariables(*this)) {
        t = v.getDatatype();
    }
    return t;
}

Expr Constraint::getA() const {
    if (!defined()) {
        return Expr();
    }
    return static_cast<const BinaryConstraintNode *>(ptr)->a;
}

Expr Constraint::getB() const {
    if (!defined()) {
        return Expr();
    }
    return static_cast<const BinaryConstraintNode *>(ptr)->b;
}

Add operator+(const Expr &a, const Expr &b) {
    return Add(a, b);
}
Sub operator-(const Expr &a, const Expr &b) {
    return Sub(a, b);
}
Mul operator*(const Expr &a, const Expr &b) {
    return Mul(a, b);
}
Div operator/(const Expr &a, const Expr &b) {
    return Div(a, b);
}
Mod operator%(const Expr &a, const Expr &b) {
    return Mod(a, b);
}
Eq operator==(const Expr &a, const Expr &b) {
    return Eq(a, b);
}
Neq operator!=(const Expr &a, const Expr &b) {
    return Neq(a, b);
}
Leq operator<=(const Expr &a, const Expr &b) {
    return Leq(a, b);
}
Geq operator>=(const Expr &a, const Expr &b) {
    return Geq(a, b);
}
Less operator<(const Expr &a, const Expr &b) {
    return Less(a, b);
}
Greater operator>(const Expr &a, const Expr &b) {
    return Greater(a, b);
}
And operator&&(const Expr &a, const Expr &b) {
    return And(a, b);
}
Or operator||(const Expr &a, const Expr &b) {
    return Or(a, b);
}

// ---------------------------------------------------------------------------
// Variable
// ---------------------------------------------------------------------------
static const VariableNode *vnode(const Variable &v) {
    if (!v.defined()) {
        throw error::InternalError("use of an undefined Variable");
    }
    return static_cast<const VariableNode *>(v.ptr);
}

Variable::Variable(const std::string &name, Datatype type, bool const_expr)
    : Expr(new const VariableNode(name, Grid::Unit::UNDEFINED, type, const_expr, false, 0)) {
}

Variable Variable::bind(int64_t val) const {
    return Variable(new const VariableNode(getName(), getBoundUnit(), Datatype::Int64, true, true, val));
}
bool Variable::isConstExpr() const {
    return vnode(*this)->const_expr;
}
bool Variable::isBound() const {
    return vnode(*this)->bound;
}
int64_t Variable::getInt64Val() const {
    return vnode(*this)->val;
}
Grid::Unit Variable::getBoundUnit() const {
    return vnode(*this)->unit;
}
Datatype Variable::getDatatype() const {
    return vnode(*this)->type;
}
Datatype Variable::getType() const {
    return vnode(*this)->type;
}
std::string Variable::getName() const {
    return vnode(*this)->name;
}
Assign Variable::operator=(const Expr &e) const {
    return Assign(*this, e);
}
Assign Variable::operator+=(const Expr &e) const {
    return Assign(*this, *this + e);
}

// ---------------------------------------------------------------------------
// Abstract data types
// ---------------------------------------------------------------------------
const AbstractDataType *AbstractDataTypePtr::checked() const {
    if (!defined()) {
        throw error::InternalError("Deref null!");
    }
    return ptr;
}
std::string AbstractDataTypePtr::getName() const {
    return checked()->getName();
}
std::string AbstractDataTypePtr::getType() const {
    return checked()->getType();
}
FunctionSignature AbstractDataTypePtr::getAllocateFunction() const {
    return checked()->getAllocateFunction();
}
FunctionSignature AbstractDataTypePtr::getQueryFunction() const {
    return checked()->getQueryFunction();
}
FunctionSignature AbstractDataTypePtr::getInsertFunction() const {
    return checked()->getInsertFunction();
}
FunctionSignature AbstractDataTypePtr::getFreeFunction() const {
    return checked()->getFreeFunction();
}
std::vector<Variable> AbstractDataTypePtr::getFields() const {
    return checked()->getFields();
}
bool AbstractDataTypePtr::freeQuery() const {
    return checked()->freeQuery();
}
bool AbstractDataTypePtr::insertQuery() const {
    return checked()->insertQuery();
}
bool AbstractDataTypePtr::freeAlloc() const {
    return checked()->freeAlloc();
}
bool AbstractDataTypePtr::readMember(const void *object, const std::string &member, int64_t &value) const {
    return checked()->readMember(object, member, value);
}
std::string AbstractDataTypePtr::str() const {
    std::stringstream ss;
    ss << *this;
    return ss.str();
}
ADTMember AbstractDataTypePtr::operator[](std::string member) const {
    return ADTMember(*this, member, false);
}
bool AbstractDataTypePtr::operator==(const AbstractDataTypePtr &other) const {
    return getName() == other.getName();
}
std::ostream &operator<<(std::ostream &os, const AbstractDataTypePtr &ds) {
    if (ds.defined()) {
        os << ds.ptr->getName();
    }
    return os;
}

ADTMember::ADTMember(AbstractDataTypePtr ds, const std::string &member, bool const_expr)
    : Expr(new const ADTMemberNode(ds, member, const_expr)) {
}
AbstractDataTypePtr ADTMember::getDS() const {
    return static_cast<const ADTMemberNode *>(ptr)->ds;
}
std::string ADTMember::getMember() const {
    return static_cast<const ADTMemberNode *>(ptr)->member;
}
bool ADTMember::isConstExpr() const {
    return static_cast<const ADTMemberNode *>(ptr)->const_expr;
}

// ---------------------------------------------------------------------------
// Printing
// ---------------------------------------------------------------------------
namespace {

const char *exprOp(ExprKind k) {
    switch (k) {
    case ExprKind::Add:
        return "+";
    case ExprKind::Sub:
        return "-";
    case ExprKind::Mul:
        return "*";
    case ExprKind::Div:
        return "/";
    case ExprKind::Mod:
        return "%";
    default:
        return "?";
    }
}

const char *constraintOp(ConstraintKind k) {
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
    case ConstraintKind::Or:
        return "||";
    }
    return "?";
}

void pad(std::ostream &os, int indent) {
    for (int i = 0; i < indent; i++) {
        os << "  ";
    }
}

void printExpr(std::ostream &os, const Expr &e) {
    if (!e.defined()) {
        return;
    }
    switch (e.ptr->kind) {
    case ExprKind::Literal: {
        auto n = static_cast<const LiteralNode *>(e.ptr);
        if (n->isFloating()) {
            os << n->f;
        } else if (n->getDatatype().isUInt()) {
            os << (uint64_t)n->i;
        } else {
            os << n->i;
        }
        break;
    }
    case ExprKind::Variable: {
        auto n = static_cast<const VariableNode *>(e.ptr);
        os << n->name;
        if (isLegalUnit(n->unit)) {
            os << n->unit;
        }
        break;
    }
    case ExprKind::ADTMember: {
        auto n = static_cast<const ADTMemberNode *>(e.ptr);
        os << n->ds << "." << n->member;
        break;
    }
    case ExprKind::GridDim:
        os << static_cast<const GridDimNode *>(e.ptr)->dim;
        break;
    default: {
        auto n = static_cast<const BinaryExprNode *>(e.ptr);
        os << "(";
        printExpr(os, n->a);
        os << " " << exprOp(n->kind) << " ";
        printExpr(os, n->b);
        os << ")";
    }
    }
}

void printStmt(std::ostream &os, const Stmt &s, int indent);

void printSubset(std::ostream &os, const SubsetNode *n, int indent) {
    pad(os, indent);
    os << n->data << " {\n";
    for (size_t i = 0; i < n->mdFields.size(); i++) {
        pad(os, indent + 1);
        printExpr(os, n->mdFields[i]);
        os << (i + 1 != n->mdFields.size() ? "," : "") << "\n";
    }
    pad(os, indent);
    os << "}";
}

void printStmt(std::ostream &os, const Stmt &s, int indent) {
    if (!s.defined()) {
        return;
    }
    switch (s.ptr->kind) {
    case StmtKind::Assign: {
        auto n = static_cast<const AssignNode *>(s.ptr);
        os << "(";
        printExpr(os, n->a);
        os << " = ";
        printExpr(os, n->b);
        os << ")";
        break;
    }
    case StmtKind::Subset:
        printSubset(os, static_cast<const SubsetNode *>(s.ptr), indent);
        break;
    case StmtKind::SubsetMany: {
        auto n = static_cast<const SubsetObjManyNode *>(s.ptr);
        for (size_t i = 0; i < n->subsets.size(); i++) {
            printStmt(os, n->subsets[i], indent);
            os << (i + 1 != n->subsets.size() ? ",\n" : "");
        }
        break;
    }
    case StmtKind::Produces: {
        auto n = static_cast<const ProducesNode *>(s.ptr);
        pad(os, indent);
        os << "produces {\n";
        printStmt(os, n->output, indent + 1);
        os << "\n";
        pad(os, indent);
        os << "}";
        break;
    }
    case StmtKind::ConsumesFor: {
        auto n = static_cast<const ConsumesForNode *>(s.ptr);
        pad(os, indent);
        os << "for ( ";
        printStmt(os, n->start, 0);
        os << " ; ";
        printExpr(os, n->parameter);
        os << " ; ";
        printExpr(os, n->step);
        os << " ) {\n";
        printStmt(os, n->body, indent + 1);
        os << "\n";
        pad(os, indent);
        os << "}";
        break;
    }
    case StmtKind::Allocates: {
        auto n = static_cast<const AllocatesNode *>(s.ptr);
        pad(os, indent);
        os << "allocates { register : ";
        printExpr(os, n->reg);
        os << " , smem : ";
        printExpr(os, n->smem);
        os << "}";
        break;
    }
    case StmtKind::ComputesFor: {
        auto n = static_cast<const ComputesForNode *>(s.ptr);
        pad(os, indent);
        os << "for ( ";
        printStmt(os, n->start, 0);
        os << " ; ";
        printExpr(os, n->parameter);
        os << " ; ";
        printExpr(os, n->step);
        os << " ) {\n";
        printStmt(os, n->body, indent + 1);
        os << "\n";
        pad(os, indent);
        os << "}";
        break;
    }
    case StmtKind::Computes: {
        auto n = static_cast<const ComputesNode *>(s.ptr);
        pad(os, indent);
        os << "computes {\n";
        printStmt(os, n->p, indent + 1);
        os << "\n";
        pad(os, indent + 1);
        os << "when consumes {\n";
        printStmt(os, n->c, indent + 2);
        os << "\n";
        pad(os, indent + 1);
        os << "}\n";
        if (n->a.defined()) {
            printStmt(os, n->a, indent + 1);
            os << "\n";
        }
        pad(os, indent);
        os << "}";
        break;
    }
    case StmtKind::Annotation: {
        auto n = static_cast<const AnnotationNode *>(s.ptr);
        printStmt(os, n->p, indent);
        os << "\n";
        pad(os, indent);
        os << "@ {";
        bool first = true;
        for (const auto &u : n->occupied) {
            os << (first ? "" : ", ") << u;
            first = false;
        }
        os << "}";
        if (!n->constraints.empty()) {
            os << " assumes {";
            for (size_t i = 0; i < n->constraints.size(); i++) {
                os << (i ? ", " : "") << n->constraints[i];
            }
            os << "}";
        }
        break;
    }
    }
}

}  // namespace

std::ostream &operator<<(std::ostream &os, const Expr &e) {
    printExpr(os, e);
    return os;
}

std::ostream &operator<<(std::ostream &os, const Constraint &c) {
    if (c.defined()) {
        auto n = static_cast<const BinaryConstraintNode *>(c.ptr);
        os << "(" << n->a << " " << constraintOp(n->kind) << " " << n->b << ")";
    }
    return os;
}

std::ostream &operator<<(std::ostream &os, const Stmt &s) {
    printStmt(os, s, 0);
    return os;
}

std::string Expr::str() const {
    std::stringstream ss;
    ss << *this;
    return ss.str();
}
std::string Constraint::str() const {
    std::stringstream ss;
    ss << *this;
    return ss.str();
}
std::string Stmt::str() const {
    std::stringstream ss;
    ss << *this;
    return ss.str();
}

// ---------------------------------------------------------------------------
// Structural equality
// ---------------------------------------------------------------------------
bool isSameExpr(const Expr &a, const Expr &b) {
    if (!a.defined() || !b.defined()) {
        return !a.defined() && !b.defined();
    }
    if (a.ptr->kind != b.ptr->kind) {
        return false;
    }
    switch (a.ptr->kind) {
    case ExprKind::Literal: {
        auto x = static_cast<const LiteralNode *>(a.ptr), y = static_cast<const LiteralNode *>(b.ptr);
        if (x->getDatatype() != y->getDatatype()) {
            return false;
        }
        return x->isFloating() ? x->f == y->f : x->i == y->i;
    }
    case ExprKind::Variable:
        return static_cast<const VariableNode *>(a.ptr)->name == static_cast<const VariableNode *>(b.ptr)->name;
    case ExprKind::ADTMember: {
        auto x = static_cast<const ADTMemberNode *>(a.ptr), y = static_cast<const ADTMemberNode *>(b.ptr);
        return x->ds == y->ds && x->member == y->member;
    }
    case ExprKind::GridDim:
        return static_cast<const GridDimNode *>(a.ptr)->dim == static_cast<const GridDimNode *>(b.ptr)->dim;
    default: {
        auto x = static_cast<const BinaryExprNode *>(a.ptr), y = static_cast<const BinaryExprNode *>(b.ptr);
        return isSameExpr(x->a, y->a) && isSameExpr(x->b, y->b);
    }
    }
}

// ---------------------------------------------------------------------------
// Walks
// ---------------------------------------------------------------------------
namespace {

using ExprFn = std::function<void(const ExprNode *)>;
using StmtFn = std::function<void(const StmtNode *)>;

void walkExpr(const Expr &e, const ExprFn &fn) {
    if (!e.defined()) {
        return;
    }
    fn(e.ptr);
    switch (e.ptr->kind) {
    case ExprKind::Add:
    case ExprKind::Sub:
    case ExprKind::Mul:
    case ExprKind::Div:
    case ExprKind::Mod: {
        auto n = static_cast<const BinaryExprNode *>(e.ptr);
        walkExpr(n->a, fn);
        walkExpr(n->b, fn);
        break;
    }
    default:
        break;
    }
}

void walkConstraint(const Constraint &c, const ExprFn &fn) {
    if (!c.defined()) {
        return;
    }
    auto n = static_cast<const BinaryConstraintNode *>(c.ptr);
    walkExpr(n->a, fn);
    walkExpr(n->b, fn);
}

// Pre-order over statements; every expression met is handed to efn.
void walkStmt(const Stmt &s, const StmtFn &sfn, const ExprFn &efn) {
    if (!s.defined()) {
        return;
    }
    sfn(s.ptr);
    switch (s.ptr->kind) {
    case StmtKind::Assign: {
        auto n = static_cast<const AssignNode *>(s.ptr);
        walkExpr(n->a, efn);
        walkExpr(n->b, efn);
        break;
    }
    case StmtKind::Subset:
        for (const auto &f : static_cast<const SubsetNode *>(s.ptr)->mdFields) {
            walkExpr(f, efn);
        }
        break;
    case StmtKind::SubsetMany:
        for (const auto &sub : static_cast<const SubsetObjManyNode *>(s.ptr)->subsets) {
            walkStmt(sub, sfn, efn);
        }
        break;
    case StmtKind::Produces:
        walkStmt(static_cast<const ProducesNode *>(s.ptr)->output, sfn, efn);
        break;
    case StmtKind::ConsumesFor: {
        auto n = static_cast<const ConsumesForNode *>(s.ptr);
        walkStmt(n->start, sfn, efn);
        walkExpr(n->parameter, efn);
        walkExpr(n->step, efn);
        walkStmt(n->body, sfn, efn);
        break;
    }
    case StmtKind::Allocates: {
        auto n = static_cast<const AllocatesNode *>(s.ptr);
        walkExpr(n->reg, efn);
        walkExpr(n->smem, efn);
        break;
    }
    case StmtKind::ComputesFor: {
        auto n = static_cast<const ComputesForNode *>(s.ptr);
        walkStmt(n->start, sfn, efn);
        walkExpr(n->parameter, efn);
        walkExpr(n->step, efn);
        walkStmt(n->body, sfn, efn);
        break;
    }
    case StmtKind::Computes: {
        auto n = static_cast<const ComputesNode *>(s.ptr);
        walkStmt(n->p, sfn, efn);
        walkStmt(n->c, sfn, efn);
        walkStmt(n->a, sfn, efn);
        break;
    }
    case StmtKind::Annotation: {
        auto n = static_cast<const AnnotationNode *>(s.ptr);
        walkStmt(n->p, sfn, efn);
        for (const auto &c : n->constraints) {
            walkConstraint(c, efn);
        }
        break;
    }
    }
}

const StmtFn noStmt = [](const StmtNode *) {};
const ExprFn noExpr = [](const ExprNode *) {};

}  // namespace

std::set<Variable> getVariables(const Expr &e) {
    std::set<Variable> vars;
    walkExpr(e, [&](const ExprNode *n) {
        if (n->kind == ExprKind::Variable) {
            vars.insert(Variable(static_cast<const VariableNode *>(n)));
        }
    });
    return vars;
}

std::set<Variable> getVariables(const Constraint &c) {
    std::set<Variable> vars;
    walkConstraint(c, [&](const ExprNode *n) {
        if (n->kind == ExprKind::Variable) {
            vars.insert(Variable(static_cast<const VariableNode *>(n)));
        }
    });
    return vars;
}

std::set<Variable> getVariables(const Stmt &s) {
    std::set<Variable> vars;
    walkStmt(s, noStmt, [&](const ExprNode *n) {
        if (n->kind == ExprKind::Variable) {
            vars.insert(Variable(static_cast<const VariableNode *>(n)));
        }
    });
    return vars;
}

std::set<Grid::Dim> getDims(const Expr &e) {
    std::set<Grid::Dim> dims;
    walkExpr(e, [&](const ExprNode *n) {
        if (n->kind == ExprKind::GridDim) {
            dims.insert(static_cast<const GridDimNode *>(n)->dim);
        }
    });
    return dims;
}

std::set<Grid::Dim> getDims(const Constraint &c) {
    std::set<Grid::Dim> dims;
    walkConstraint(c, [&](const ExprNode *n) {
        if (n->kind == ExprKind::GridDim) {
            dims.insert(static_cast<const GridDimNode *>(n)->dim);
        }
    });
    return dims;
}

bool isConstExpr(const Expr &e) {
    bool ok = true;
    walkExpr(e, [&](const ExprNode *n) {
        if (n->kind == ExprKind::Variable && !static_cast<const VariableNode *>(n)->const_expr) {
            ok = false;
        }
        if (n->kind == ExprKind::ADTMember && !static_cast<const ADTMemberNode *>(n)->const_expr) {
            ok = false;
        }
        if (n->kind == ExprKind::GridDim) {
            ok = false;
        }
    });
    return ok;
}

bool isConstExpr(const Constraint &c) {
    return isConstExpr(c.getA()) && isConstExpr(c.getB());
}

// ---------------------------------------------------------------------------
// Stmt queries
// ---------------------------------------------------------------------------
std::set<Variable> Stmt::getDefinedVariables() const {
    std::set<Variable> vars;
    walkStmt(*this, [&](const StmtNode *n) {
        if (n->kind == StmtKind::Assign) {
            vars.insert(to<Variable>(static_cast<const AssignNode *>(n)->a));
        } }, noExpr);
    return vars;
}

std::set<Variable> Stmt::getIntervalVariables() const {
    std::set<Variable> vars;
    walkStmt(*this, [&](const StmtNode *n) {
        if (n->kind == StmtKind::ConsumesFor) {
            vars.insert(to<Variable>(static_cast<const ConsumesForNode *>(n)->start.getA()));
        } else if (n->kind == StmtKind::ComputesFor) {
            vars.insert(to<Variable>(static_cast<const ComputesForNode *>(n)->start.getA()));
        } }, noExpr);
    return vars;
}

std::map<Variable, Variable> Stmt::getConsumesIntervalAndStepVars() const {
    std::map<Variable, Variable> vars;
    walkStmt(*this, [&](const StmtNode *n) {
        if (n->kind == StmtKind::ConsumesFor) {
            auto f = static_cast<const ConsumesForNode *>(n);
            vars[to<Variable>(f->start.getA())] = f->step;
        } }, noExpr);
    return vars;
}

std::map<Variable, Variable> Stmt::getComputesIntervalAndStepVars() const {
    std::map<Variable, Variable> vars;
    walkStmt(*this, [&](const StmtNode *n) {
        if (n->kind == StmtKind::ComputesFor) {
            auto f = static_cast<const ComputesForNode *>(n);
            vars[to<Variable>(f->start.getA())] = f->step;
        } }, noExpr);
    return vars;
}

std::map<Expr, std::tuple<Variable, Expr, Variable>> Stmt::getTileableFields() const {
    std::map<Expr, std::tuple<Variable, Expr, Variable>> fields;
    walkStmt(*this, [&](const StmtNode *n) {
        if (n->kind == StmtKind::ComputesFor) {
            auto f = static_cast<const ComputesForNode *>(n);
            fields[f->parameter] = std::make_tuple(to<Variable>(f->start.getA()), f->start.getB(), f->step);
        } }, noExpr);
    return fields;
}

std::map<Expr, std::tuple<Variable, Expr, Variable>> Stmt::getReducableFields() const {
    std::map<Expr, std::tuple<Variable, Expr, Variable>> fields;
    walkStmt(*this, [&](const StmtNode *n) {
        if (n->kind == StmtKind::ConsumesFor) {
            auto f = static_cast<const ConsumesForNode *>(n);
            fields[f->parameter] = std::make_tuple(to<Variable>(f->start.getA()), f->start.getB(), f->step);
        } }, noExpr);
    return fields;
}

std::vector<Expr> SubsetObj::getFields() const {
    return static_cast<const SubsetNode *>(ptr)->mdFields;
}
AbstractDataTypePtr SubsetObj::getDS() const {
    return static_cast<const SubsetNode *>(ptr)->data;
}

Produces Produces::Subset(AbstractDataTypePtr ds, std::vector<Variable> v) {
    return Produces(new const ProducesNode(ds, v));
}
SubsetObj Produces::getSubset() const {
    return static_cast<const ProducesNode *>(ptr)->output;
}
std::vector<Variable> Produces::getFieldsAsVars() const {
    std::vector<Variable> vars;
    for (const auto &e : getSubset().getFields()) {
        vars.push_back(to<Variable>(e));
    }
    return vars;
}

Consumes::Consumes(SubsetObj s)
    : Stmt(new const SubsetObjManyNode({s})) {
}
Consumes Consumes::Subset(AbstractDataTypePtr ds, std::vector<Expr> fields) {
    return Consumes(SubsetObj(ds, fields));
}
Consumes Consumes::Subsets(ConsumeMany many) {
    return Consumes(many.ptr);
}

ConsumeMany Reducible(Assign start, Expr parameter, Variable step, ConsumeMany body, bool parallel) {
    return ConsumeMany(new const ConsumesForNode(start, parameter, step, body, parallel));
}
ConsumeMany Reducible(Assign start, Expr parameter, Variable step, std::vector<SubsetObj> body, bool parallel) {
    return Reducible(start, parameter, step, SubsetObjMany(body), parallel);
}
ConsumeMany Reducible(Assign start, Expr parameter, Variable step, SubsetObj body, bool parallel) {
    return Reducible(start, parameter, step, std::vector<SubsetObj>{body}, parallel);
}

Pattern Tileable(Assign start, Expr parameter, Variable step, Pattern body, bool parallel) {
    return Pattern(new const ComputesForNode(start, parameter, step, body, parallel));
}
Pattern Tileable(Assign start, Expr parameter, Variable step, Produces produces, Consumes consumes,
                 bool parallel) {
    return Tileable(start, parameter, step, Computes(produces, consumes), parallel);
}

Annotation Pattern::occupies(std::set<Grid::Unit> occupied) const {
    return Annotation(*this, occupied, {});
}
Annotation Pattern::assumes(std::vector<Constraint> constraints) const {
    return annotate(*this).assumes(constraints);
}

std::vector<SubsetObj> Pattern::getInputs() const {
    std::vector<SubsetObj> inputs;
    walkStmt(*this, [&](const StmtNode *n) {
        if (n->kind == StmtKind::SubsetMany) {
            inputs = static_cast<const SubsetObjManyNode *>(n)->subsets;
        } }, noExpr);
    return inputs;
}

std::vector<SubsetObj> Pattern::getAllADTs() const {
    std::vector<SubsetObj> all = getInputs();
    all.push_back(getOutput());
    return all;
}

SubsetObj Pattern::getOutput() const {
    SubsetObj out;
    walkStmt(*this, [&](const StmtNode *n) {
        if (n->kind == StmtKind::Produces) {
            out = static_cast<const ProducesNode *>(n)->output;
        } }, noExpr);
    return out;
}

std::vector<Variable> Pattern::getProducesField() const {
    std::vector<Variable> fields;
    SubsetObj out = getOutput();
    if (out.defined()) {
        for (const auto &e : out.getFields()) {
            fields.push_back(to<Variable>(e));
        }
    }
    return fields;
}

SubsetObj Pattern::getCorrespondingSubset(AbstractDataTypePtr d) const {
    SubsetObj found;
    walkStmt(*this, [&](const StmtNode *n) {
        if (n->kind == StmtKind::Subset && static_cast<const SubsetNode *>(n)->data == d) {
            found = SubsetObj(static_cast<const SubsetNode *>(n));
        } }, noExpr);
    return found;
}

std::vector<Expr> Pattern::getRequirement(AbstractDataTypePtr d) const {
    SubsetObj s = getCorrespondingSubset(d);
    return s.defined() ? s.getFields() : std::vector<Expr>{};
}

Annotation::Annotation(Pattern p, std::set<Grid::Unit> occupied, std::vector<Constraint> constraints)
    : Stmt(new const AnnotationNode(p, occupied, constraints)) {
}
Pattern Annotation::getPattern() const {
    return static_cast<const AnnotationNode *>(ptr)->p;
}
std::vector<Constraint> Annotation::getConstraints() const {
    return static_cast<const AnnotationNode *>(ptr)->constraints;
}
std::set<Grid::Unit> Annotation::getOccupiedUnits() const {
    return static_cast<const AnnotationNode *>(ptr)->occupied;
}

Annotation annotate(Pattern p) {
    return Annotation(p, {}, {});
}
Annotation resetUnit(Annotation a, std::set<Grid::Unit> occupied) {
    return Annotation(a.getPattern(), occupied, a.getConstraints());
}

Annotation Annotation::assumes(std::vector<Constraint> constraints) const {
    std::set<std::string> known;
    for (const auto &v : getVariables(getPattern())) {
        known.insert(v.getName());
    }
    const auto legal_dims = gern::getDims(getOccupiedUnits());
    const auto level = getLevel(getOccupiedUnits());
    for (const auto &c : constraints) {
        for (const auto &v : getVariables(c)) {
            if (!known.count(v.getName())) {
                throw error::UserError("Putting constraints on variables that are not "
                                       "present in statement's scope");
            }
        }
        for (const auto &dim : gern::getDims(c)) {
            if (!isDimInScope(dim, legal_dims)) {
                std::stringstream ss;
                ss << " Cannot constrain " << dim << " at " << level;
                throw error::UserError(ss.str());
            }
        }
    }
    return Annotation(getPattern(), getOccupiedUnits(), constraints);
}

// ---------------------------------------------------------------------------
// Substitution
// ---------------------------------------------------------------------------
Expr substitute(const Expr &e, const Substitution &s) {
    if (!e.defined() || s.empty()) {
        return e;
    }
    switch (e.ptr->kind) {
    case ExprKind::Literal:
        return e;
    case ExprKind::Variable: {
        auto it = s.variables.find(static_cast<const VariableNode *>(e.ptr)->name);
        return it == s.variables.end() ? e : it->second;
    }
    case ExprKind::ADTMember: {
        auto n = static_cast<const ADTMemberNode *>(e.ptr);
        auto it = s.structures.find(n->ds.getName());
        return it == s.structures.end() ? e : Expr(ADTMember(it->second, n->member, n->const_expr));
    }
    case ExprKind::GridDim: {
        auto it = s.dims.find(static_cast<const GridDimNode *>(e.ptr)->dim);
        return it == s.dims.end() ? e : it->second;
    }
    default: {
        auto n = static_cast<const BinaryExprNode *>(e.ptr);
        return Expr(new const BinaryExprNode(n->kind, substitute(n->a, s), substitute(n->b, s)));
    }
    }
}

Constraint substitute(const Constraint &c, const Substitution &s) {
    if (!c.defined() || s.empty()) {
        return c;
    }
    auto n = static_cast<const BinaryConstraintNode *>(c.ptr);
    return Constraint(new const BinaryConstraintNode(n->kind, substitute(n->a, s), substitute(n->b, s)));
}

static Variable substituteVar(const Variable &v, const Substitution &s) {
    Expr e = substitute(Expr(v), s);
    if (!isa<Variable>(e)) {
        throw error::InternalError("a loop or field variable was replaced by a non-variable: " + e.str());
    }
    return to<Variable>(e);
}

Stmt substitute(const Stmt &st, const Substitution &s) {
    if (!st.defined() || s.empty()) {
        return st;
    }
    switch (st.ptr->kind) {
    case StmtKind::Assign: {
        auto n = static_cast<const AssignNode *>(st.ptr);
        return Assign(substitute(n->a, s), substitute(n->b, s));
    }
    case StmtKind::Subset: {
        auto n = static_cast<const SubsetNode *>(st.ptr);
        std::vector<Expr> fields;
        for (const auto &f : n->mdFields) {
            fields.push_back(substitute(f, s));
        }
        auto it = s.structures.find(n->data.getName());
        return SubsetObj(it == s.structures.end() ? n->data : it->second, fields);
    }
    case StmtKind::SubsetMany: {
        auto n = static_cast<const SubsetObjManyNode *>(st.ptr);
        std::vector<SubsetObj> subs;
        for (const auto &sub : n->subsets) {
            subs.push_back(to<SubsetObj>(substitute(Stmt(sub), s)));
        }
        return SubsetObjMany(subs);
    }
    case StmtKind::Produces: {
        auto n = static_cast<const ProducesNode *>(st.ptr);
        SubsetObj out = to<SubsetObj>(substitute(Stmt(n->output), s));
        std::vector<Variable> vars;
        for (const auto &f : out.getFields()) {
            if (!isa<Variable>(f)) {
                throw error::InternalError("a produced field was replaced by a non-variable: " + f.str());
            }
            vars.push_back(to<Variable>(f));
        }
        return Produces::Subset(out.getDS(), vars);
    }
    case StmtKind::ConsumesFor: {
        auto n = static_cast<const ConsumesForNode *>(st.ptr);
        return Reducible(to<Assign>(substitute(Stmt(n->start), s)), substitute(n->parameter, s),
                         substituteVar(n->step, s),
                         ConsumeMany(substitute(Stmt(n->body), s).ptr), n->parallel);
    }
    case StmtKind::Allocates: {
        auto n = static_cast<const AllocatesNode *>(st.ptr);
        return Allocates(substitute(n->reg, s), substitute(n->smem, s));
    }
    case StmtKind::ComputesFor: {
        auto n = static_cast<const ComputesForNode *>(st.ptr);
        return Tileable(to<Assign>(substitute(Stmt(n->start), s)), substitute(n->parameter, s),
                        substituteVar(n->step, s), Pattern(substitute(Stmt(n->body), s).ptr), n->parallel);
    }
    case StmtKind::Computes: {
        auto n = static_cast<const ComputesNode *>(st.ptr);
        Stmt a = substitute(Stmt(n->a), s);
        return Computes(to<Produces>(substitute(Stmt(n->p), s)), Consumes(substitute(Stmt(n->c), s).ptr),
                        a.defined() ? to<Allocates>(a) : Allocates());
    }
    case StmtKind::Annotation: {
        auto n = static_cast<const AnnotationNode *>(st.ptr);
        std::vector<Constraint> cs;
        for (const auto &c : n->constraints) {
            cs.push_back(substitute(c, s));
        }
        return Annotation(Pattern(substitute(Stmt(n->p), s).ptr), n->occupied, cs);
    }
    }
    return st;
}

Annotation substitute(const Annotation &a, const Substitution &s) {
    return to<Annotation>(substitute(Stmt(a), s));
}

Pattern substitute(const Pattern &p, const Substitution &s) {
    return Pattern(substitute(Stmt(p), s).ptr);
}

Annotation refreshVariables(Annotation annot, std::map<Variable, Variable> &new_vars) {
    // Loop bounds that are plain variables (e.g. a reduction extent `k`) keep
    // their names: they are what the user tiles by.
    std::set<std::string> keep;
    walkStmt(annot, [&](const StmtNode *n) {
        Expr parameter;
        if (n->kind == StmtKind::ConsumesFor) {
            parameter = static_cast<const ConsumesForNode *>(n)->parameter;
        } else if (n->kind == StmtKind::ComputesFor) {
            parameter = static_cast<const ComputesForNode *>(n)->parameter;
        }
        if (parameter.defined() && isa<Variable>(parameter)) {
            keep.insert(to<Variable>(parameter).getName());
        } }, noExpr);

    Substitution s;
    for (const auto &v : getVariables(annot)) {
        // So does a variable the user has bound to a value: it is a constant wherever it appears, and the
        // footprint of a tile or a stage around the body may need it (a halo of stride - 1 elements).
        if (keep.count(v.getName()) || v.isBound()) {
            continue;
        }
        Variable fresh(getUniqueName(v.getName()), v.getDatatype(), v.isConstExpr());
        new_vars[v] = fresh;
        s.variables[v.getName()] = fresh;
    }
    return substitute(annot, s);
}

}  // namespace gern
