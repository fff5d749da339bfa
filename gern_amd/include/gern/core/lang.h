// The data-dependency annotation language: integer expressions, constraints,
// abstract data types, and the statements (subsets, produces / consumes,
// tileable / reducible loops) that describe what part of its inputs a function
// needs to produce a given part of its output.
//
// The user-visible classes, constructors and free functions are those of the
// reference (include/gern/annotations/expr.h:37-274, stmt.h:31-199,
// abstract_nodes.h, std_less_specialization.h).  Internally every node carries
// a kind tag and the passes are plain recursive functions over those tags.
#pragma once

#include "gern/core/datatype.h"
#include "gern/core/grid.h"
#include "gern/core/support.h"

#include <cassert>
#include <functional>
#include <map>
#include <set>
#include <string>
#include <tuple>
#include <vector>

namespace gern {

class Expr;
class Constraint;
class Stmt;
class Variable;
class ADTMember;
class Assign;
class Annotation;
class Pattern;
struct FunctionSignature;

// ---------------------------------------------------------------------------
// Nodes
// ---------------------------------------------------------------------------
enum class ExprKind { Literal, Variable, ADTMember, GridDim, Add, Sub, Mul, Div, Mod };
enum class ConstraintKind { Eq, Neq, Leq, Geq, Less, Greater, And, Or };
enum class StmtKind { Assign, Subset, SubsetMany, Produces, ConsumesFor, Allocates, ComputesFor, Computes, Annotation };

class ExprNode : public util::Manageable<ExprNode>, public util::Uncopyable {
public:
    ExprNode(ExprKind kind, Datatype type)
        : kind(kind), datatype(type) {
    }
    virtual ~ExprNode() = default;
    Datatype getDatatype() const {
        return datatype;
    }
    const ExprKind kind;

private:
    Datatype datatype;
};

class ConstraintNode : public util::Manageable<ConstraintNode>, public util::Uncopyable {
public:
    explicit ConstraintNode(ConstraintKind kind)
        : kind(kind) {
    }
    virtual ~ConstraintNode() = default;
    const ConstraintKind kind;
};

class StmtNode : public util::Manageable<StmtNode>, public util::Uncopyable {
public:
    explicit StmtNode(StmtKind kind)
        : kind(kind) {
    }
    virtual ~StmtNode() = default;
    const StmtKind kind;
};

// ---------------------------------------------------------------------------
// Expr
// ---------------------------------------------------------------------------
class Expr : public util::IntrusivePtr<const ExprNode> {
public:
    Expr()
        : util::IntrusivePtr<const ExprNode>(nullptr) {
    }
    Expr(const ExprNode *n)
        : util::IntrusivePtr<const ExprNode>(n) {
    }
    Expr(uint32_t);
    Expr(uint64_t);
    Expr(int32_t);
    Expr(int64_t);
    Expr(double);
    Expr(Grid::Dim);

    std::string str() const;
    // The declared type of a variable; Undefined for anything else.
    Datatype getType() const;
};

std::ostream &operator<<(std::ostream &, const Expr &);

// Structural equality: same shape, variables equal by name, data structures
// equal by name, literals equal by value.
bool isSameExpr(const Expr &a, const Expr &b);

class Constraint : public util::IntrusivePtr<const ConstraintNode> {
public:
    Constraint()
        : util::IntrusivePtr<const ConstraintNode>(nullptr) {
    }
    Constraint(const ConstraintNode *n)
        : util::IntrusivePtr<const ConstraintNode>(n) {
    }
    virtual Expr getA() const;
    virtual Expr getB() const;
    std::string str() const;
};

std::ostream &operator<<(std::ostream &, const Constraint &);

struct LiteralNode : public ExprNode {
    template<typename T>
    explicit LiteralNode(T v)
        : ExprNode(ExprKind::Literal, type<T>()) {
        if constexpr (std::is_floating_point_v<T>) {
            f = (double)v;
            i = (int64_t)v;
        } else {
            i = (int64_t)v;
            f = (double)v;
        }
    }
    bool isFloating() const {
        return getDatatype().isFloat();
    }
    int64_t i = 0;
    double f = 0;
};

class Literal : public Expr {
public:
    Literal(const LiteralNode *n)
        : Expr(n) {
    }
    int64_t getInt() const {
        return static_cast<const LiteralNode *>(ptr)->i;
    }
    typedef LiteralNode Node;
    static bool classof(const ExprNode *n) {
        return n->kind == ExprKind::Literal;
    }
};

struct BinaryExprNode : public ExprNode {
    BinaryExprNode(ExprKind kind, Expr a, Expr b)
        : ExprNode(kind, Datatype::Int64), a(a), b(b) {
    }
    Expr a;
    Expr b;
};

struct BinaryConstraintNode : public ConstraintNode {
    BinaryConstraintNode(ConstraintKind kind, Expr a, Expr b)
        : ConstraintNode(kind), a(a), b(b) {
    }
    Expr a;
    Expr b;
};

#define GERN_BINARY_EXPR(NAME)                                                   \
    class NAME : public Expr {                                                   \
    public:                                                                      \
        explicit NAME(const BinaryExprNode *n)                                   \
            : Expr(n) {                                                          \
        }                                                                        \
        NAME(Expr a, Expr b)                                                     \
            : Expr(new const BinaryExprNode(ExprKind::NAME, a, b)) {             \
        }                                                                        \
        Expr getA() const {                                                      \
            return static_cast<const BinaryExprNode *>(ptr)->a;                  \
        }                                                                        \
        Expr getB() const {                                                      \
            return static_cast<const BinaryExprNode *>(ptr)->b;                  \
        }                                                                        \
        typedef BinaryExprNode Node;                                             \
        static bool classof(const ExprNode *n) {                                 \
            return n->kind == ExprKind::NAME;                                    \
        }                                                                        \
    };

GERN_BINARY_EXPR(Add)
GERN_BINARY_EXPR(Sub)
GERN_BINARY_EXPR(Mul)
GERN_BINARY_EXPR(Div)
GERN_BINARY_EXPR(Mod)
#undef GERN_BINARY_EXPR

#define GERN_BINARY_CONSTRAINT(NAME)                                                     \
    class NAME : public Constraint {                                                     \
    public:                                                                              \
        explicit NAME(const BinaryConstraintNode *n)                                     \
            : Constraint(n) {                                                            \
        }                                                                                \
        NAME(Expr a, Expr b)                                                             \
            : Constraint(new const BinaryConstraintNode(ConstraintKind::NAME, a, b)) {   \
        }                                                                                \
        Expr getA() const override {                                                     \
            return static_cast<const BinaryConstraintNode *>(ptr)->a;                    \
        }                                                                                \
        Expr getB() const override {                                                     \
            return static_cast<const BinaryConstraintNode *>(ptr)->b;                    \
        }                                                                                \
        typedef BinaryConstraintNode Node;                                               \
        static bool classof(const ConstraintNode *n) {                                   \
            return n->kind == ConstraintKind::NAME;                                      \
        }                                                                                \
    };

GERN_BINARY_CONSTRAINT(Eq)
GERN_BINARY_CONSTRAINT(Neq)
GERN_BINARY_CONSTRAINT(Leq)
GERN_BINARY_CONSTRAINT(Geq)
GERN_BINARY_CONSTRAINT(Less)
GERN_BINARY_CONSTRAINT(Greater)
GERN_BINARY_CONSTRAINT(And)
GERN_BINARY_CONSTRAINT(Or)
#undef GERN_BINARY_CONSTRAINT

Add operator+(const Expr &, const Expr &);
Sub operator-(const Expr &, const Expr &);
Mul operator*(const Expr &, const Expr &);
Div operator/(const Expr &, const Expr &);
Mod operator%(const Expr &, const Expr &);
Eq operator==(const Expr &, const Expr &);
Neq operator!=(const Expr &, const Expr &);
Leq operator<=(const Expr &, const Expr &);
Geq operator>=(const Expr &, const Expr &);
Less operator<(const Expr &, const Expr &);
Greater operator>(const Expr &, const Expr &);
And operator&&(const Expr &, const Expr &);
Or operator||(const Expr &, const Expr &);

// ---------------------------------------------------------------------------
// Variable
// ---------------------------------------------------------------------------
struct VariableNode : public ExprNode {
    VariableNode(const std::string &name, Grid::Unit unit, Datatype type, bool const_expr,
                 bool bound, int64_t val)
        : ExprNode(ExprKind::Variable, Datatype::Int64), name(name), unit(unit), type(type),
          const_expr(const_expr), bound(bound), val(val) {
    }
    std::string name;
    Grid::Unit unit;
    Datatype type;
    bool const_expr;
    bool bound;
    int64_t val;
};

// A named integer (or float, for pass-through scalar arguments) unknown.
// Identity is the NAME: two Variable objects with the same name are the same
// variable everywhere in the system.
class Variable : public Expr {
public:
    Variable() = default;
    Variable(const std::string &name, Datatype type = Datatype::Int64, bool const_expr = false);
    Variable(const VariableNode *n)
        : Expr(n) {
    }

    // The same variable fixed to a value; it becomes a compile-time constant
    // (a template argument of the generated function).
    Variable bind(int64_t) const;
    bool isConstExpr() const;
    bool isBound() const;
    int64_t getInt64Val() const;
    Grid::Unit getBoundUnit() const;
    Datatype getDatatype() const;
    Datatype getType() const;
    std::string getName() const;

    Assign operator=(const Expr &) const;
    Assign operator+=(const Expr &) const;

    typedef VariableNode Node;
    static bool classof(const ExprNode *n) {
        return n->kind == ExprKind::Variable;
    }
};

// ---------------------------------------------------------------------------
// Abstract data types
// ---------------------------------------------------------------------------
// What the code generator needs to know about a user data structure: its name
// and C++ type in generated code, the metadata fields that identify a subset
// of it, and the four functions (allocate / free / insert / query) whose names
// are pasted into generated code.
class AbstractDataType : public util::Manageable<AbstractDataType> {
public:
    AbstractDataType() = default;
    virtual ~AbstractDataType() = default;
    AbstractDataType(const std::string &name, const std::string &type)
        : name(name), type(type) {
    }

    virtual std::string getName() const {
        return name;
    }
    virtual std::string getType() const {
        return type;
    }
    virtual std::vector<Variable> getFields() const = 0;
    virtual FunctionSignature getAllocateFunction() const = 0;
    virtual FunctionSignature getFreeFunction() const = 0;
    virtual FunctionSignature getInsertFunction() const = 0;
    virtual FunctionSignature getQueryFunction() const = 0;

    // A queried subset owns storage that must be released.
    virtual bool freeQuery() const {
        return false;
    }
    // A queried subset is a copy that must be written back.
    virtual bool insertQuery() const {
        return false;
    }
    // An allocated temporary must be released.
    virtual bool freeAlloc() const {
        return true;
    }

    // Host-side access to a member (e.g. "row") of the concrete object the
    // caller hands to Runner::evaluate under this data structure's name.  A
    // device launch sizes its grid on the host, where the generated device
    // code cannot be asked; a data structure whose members appear in launch
    // dimensions overrides this.  The reference reads such members in the
    // host hook that nvcc compiles together with the kernel
    // (src/codegen/codegen.cpp:153-171); hiprtc compiles device code only.
    virtual bool readMember(const void *object, const std::string &member, int64_t &value) const {
        (void)object;
        (void)member;
        (void)value;
        return false;
    }

private:
    std::string name;
    std::string type;
};

class AbstractDataTypePtr : public util::IntrusivePtr<const AbstractDataType> {
public:
    AbstractDataTypePtr()
        : util::IntrusivePtr<const AbstractDataType>(nullptr) {
    }
    explicit AbstractDataTypePtr(const AbstractDataType *p)
        : util::IntrusivePtr<const AbstractDataType>(p) {
    }
    template<typename T, std::enable_if_t<std::is_base_of_v<AbstractDataType, T>, int> = 0>
    AbstractDataTypePtr(const T obj)
        : util::IntrusivePtr<const AbstractDataType>(new T(obj)) {
    }

    std::string getName() const;
    std::string getType() const;
    FunctionSignature getAllocateFunction() const;
    FunctionSignature getQueryFunction() const;
    FunctionSignature getInsertFunction() const;
    FunctionSignature getFreeFunction() const;
    std::vector<Variable> getFields() const;
    bool freeQuery() const;
    bool insertQuery() const;
    bool freeAlloc() const;
    bool readMember(const void *object, const std::string &member, int64_t &value) const;
    std::string str() const;
    // adt["member"]: a run-time member of the concrete object.
    ADTMember operator[](std::string) const;
    // Data structures are identified by name.
    bool operator==(const AbstractDataTypePtr &other) const;
    bool operator!=(const AbstractDataTypePtr &other) const {
        return !(*this == other);
    }

private:
    const AbstractDataType *checked() const;
};

std::ostream &operator<<(std::ostream &, const AbstractDataTypePtr &);

struct ADTMemberNode : public ExprNode {
    ADTMemberNode(AbstractDataTypePtr ds, const std::string &member, bool const_expr)
        : ExprNode(ExprKind::ADTMember, Datatype::Int64), ds(ds), member(member), const_expr(const_expr) {
    }
    AbstractDataTypePtr ds;
    std::string member;
    bool const_expr;
};

class ADTMember : public Expr {
public:
    ADTMember() = default;
    ADTMember(const ADTMemberNode *n)
        : Expr(n) {
    }
    ADTMember(AbstractDataTypePtr ds, const std::string &member, bool const_expr);
    AbstractDataTypePtr getDS() const;
    std::string getMember() const;
    bool isConstExpr() const;
    typedef ADTMemberNode Node;
    static bool classof(const ExprNode *n) {
        return n->kind == ExprKind::ADTMember;
    }
};

struct GridDimNode : public ExprNode {
    explicit GridDimNode(Grid::Dim dim)
        : ExprNode(ExprKind::GridDim, Datatype::Int64), dim(dim) {
    }
    Grid::Dim dim;
};

// A launch dimension used as a value inside a constraint.
class GridDim : public Expr {
public:
    GridDim(const GridDimNode *n)
        : Expr(n) {
    }
    GridDim(const Grid::Dim &dim)
        : Expr(new const GridDimNode(dim)) {
    }
    Grid::Dim getDim() const {
        return static_cast<const GridDimNode *>(ptr)->dim;
    }
    typedef GridDimNode Node;
    static bool classof(const ExprNode *n) {
        return n->kind == ExprKind::GridDim;
    }
};

template<typename E, typename T>
inline bool isa(const T &e) {
    return e.ptr != nullptr && E::classof(e.ptr);
}

template<typename E, typename T>
inline const E to(const T &e) {
    if constexpr (std::is_same_v<E, T>) {
        return e;
    } else {
        assert(isa<E>(e));
        return E(static_cast<const typename E::Node *>(e.ptr));
    }
}

}  // namespace gern

// Ordering used by every std::map / std::set keyed on these handles: variables
// and data structures by name, members by (structure, member), other
// expressions by node identity.
namespace std {
template<>
struct less<gern::Variable> {
    bool operator()(const gern::Variable &a, const gern::Variable &b) const {
        return a.getName() < b.getName();
    }
};
template<>
struct less<gern::AbstractDataTypePtr> {
    bool operator()(const gern::AbstractDataTypePtr &a, const gern::AbstractDataTypePtr &b) const {
        return a.getName() < b.getName();
    }
};
template<>
struct less<gern::ADTMember> {
    bool operator()(const gern::ADTMember &a, const gern::ADTMember &b) const {
        const std::string an = a.getDS().getName(), bn = b.getDS().getName();
        if (an != bn) {
            return an < bn;
        }
        return a.getMember() < b.getMember();
    }
};
template<>
struct less<gern::Expr> {
    // Variables order by name and members by (structure, member), so that a
    // loop bound is found no matter which handle of it the user passes; every
    // other expression orders by node identity.
    bool operator()(const gern::Expr &a, const gern::Expr &b) const {
        auto rank = [](const gern::Expr &e) {
            return gern::isa<gern::Variable>(e) ? 0 : gern::isa<gern::ADTMember>(e) ? 1 : 2;
        };
        const int ra = rank(a), rb = rank(b);
        if (ra != rb) {
            return ra < rb;
        }
        if (ra == 0) {
            return std::less<gern::Variable>()(gern::to<gern::Variable>(a), gern::to<gern::Variable>(b));
        }
        if (ra == 1) {
            return std::less<gern::ADTMember>()(gern::to<gern::ADTMember>(a), gern::to<gern::ADTMember>(b));
        }
        return a.ptr < b.ptr;
    }
};
}  // namespace std

namespace gern {

// ---------------------------------------------------------------------------
// Statements
// ---------------------------------------------------------------------------
class Stmt : public util::IntrusivePtr<const StmtNode> {
public:
    Stmt()
        : util::IntrusivePtr<const StmtNode>(nullptr) {
    }
    Stmt(const StmtNode *n)
        : util::IntrusivePtr<const StmtNode>(n) {
    }

    std::set<Variable> getDefinedVariables() const;
    std::set<Variable> getIntervalVariables() const;
    std::map<Variable, Variable> getConsumesIntervalAndStepVars() const;
    std::map<Variable, Variable> getComputesIntervalAndStepVars() const;
    // loop bound -> (index variable, start, step variable), for the loops on
    // the output side (tileable) and on the input side (reducible).
    std::map<Expr, std::tuple<Variable, Expr, Variable>> getTileableFields() const;
    std::map<Expr, std::tuple<Variable, Expr, Variable>> getReducableFields() const;
    std::string str() const;
};

std::ostream &operator<<(std::ostream &, const Stmt &);

struct AssignNode : public StmtNode {
    AssignNode(Expr a, Expr b)
        : StmtNode(StmtKind::Assign), a(a), b(b) {
    }
    Expr a;
    Expr b;
};

class Assign : public Stmt {
public:
    explicit Assign(const AssignNode *n)
        : Stmt(n) {
    }
    Assign(Expr a, Expr b)
        : Stmt(new const AssignNode(a, b)) {
    }
    Expr getA() const {
        return static_cast<const AssignNode *>(ptr)->a;
    }
    Expr getB() const {
        return static_cast<const AssignNode *>(ptr)->b;
    }
    typedef AssignNode Node;
    static bool classof(const StmtNode *n) {
        return n->kind == StmtKind::Assign;
    }
};

struct SubsetNode : public StmtNode {
    SubsetNode(AbstractDataTypePtr data, std::vector<Expr> fields)
        : StmtNode(StmtKind::Subset), data(data), mdFields(std::move(fields)) {
    }
    AbstractDataTypePtr data;
    std::vector<Expr> mdFields;
};

// A subset of a data structure, identified by values for its metadata fields.
class SubsetObj : public Stmt {
public:
    SubsetObj() = default;
    SubsetObj(const SubsetNode *n)
        : Stmt(n) {
    }
    SubsetObj(AbstractDataTypePtr data, std::vector<Expr> mdFields)
        : Stmt(new const SubsetNode(data, std::move(mdFields))) {
    }
    std::vector<Expr> getFields() const;
    AbstractDataTypePtr getDS() const;
    typedef SubsetNode Node;
    static bool classof(const StmtNode *n) {
        return n->kind == StmtKind::Subset;
    }
};

struct ProducesNode : public StmtNode {
    ProducesNode(AbstractDataTypePtr ds, const std::vector<Variable> &v)
        : StmtNode(StmtKind::Produces), output(ds, std::vector<Expr>(v.begin(), v.end())) {
    }
    SubsetObj output;
};

class Produces : public Stmt {
public:
    explicit Produces(const ProducesNode *n)
        : Stmt(n) {
    }
    static Produces Subset(AbstractDataTypePtr, std::vector<Variable>);
    SubsetObj getSubset() const;
    std::vector<Variable> getFieldsAsVars() const;
    typedef ProducesNode Node;
    static bool classof(const StmtNode *n) {
        return n->kind == StmtKind::Produces;
    }
};

class ConsumeMany;

// Either a list of input subsets or a reducible loop around one.
class Consumes : public Stmt {
public:
    explicit Consumes(const StmtNode *n)
        : Stmt(n) {
    }
    Consumes(SubsetObj s);
    static Consumes Subset(AbstractDataTypePtr, std::vector<Expr>);
    static Consumes Subsets(ConsumeMany);
    typedef StmtNode Node;
    static bool classof(const StmtNode *n) {
        return n->kind == StmtKind::SubsetMany || n->kind == StmtKind::ConsumesFor;
    }
};

class ConsumeMany : public Consumes {
public:
    ConsumeMany(const StmtNode *n)
        : Consumes(n) {
    }
};

struct SubsetObjManyNode : public StmtNode {
    explicit SubsetObjManyNode(std::vector<SubsetObj> subsets)
        : StmtNode(StmtKind::SubsetMany), subsets(std::move(subsets)) {
    }
    std::vector<SubsetObj> subsets;
};

class SubsetObjMany : public ConsumeMany {
public:
    SubsetObjMany(const SubsetObjManyNode *n)
        : ConsumeMany(n) {
    }
    SubsetObjMany(const std::vector<SubsetObj> &subsets)
        : ConsumeMany(new const SubsetObjManyNode(subsets)) {
    }
    SubsetObjMany(std::initializer_list<SubsetObj> subsets)
        : SubsetObjMany(std::vector<SubsetObj>(subsets)) {
    }
    SubsetObjMany(SubsetObj s)
        : SubsetObjMany(std::vector<SubsetObj>{s}) {
    }
    typedef SubsetObjManyNode Node;
    static bool classof(const StmtNode *n) {
        return n->kind == StmtKind::SubsetMany;
    }
};

// for (start; < parameter; += step) over the INPUT side: the function reduces
// over this range, `step` of it at a time.
struct ConsumesForNode : public StmtNode {
    ConsumesForNode(Assign start, Expr parameter, Variable step, ConsumeMany body, bool parallel)
        : StmtNode(StmtKind::ConsumesFor), start(start), parameter(parameter), step(step), body(body),
          parallel(parallel) {
    }
    Assign start;
    Expr parameter;
    Variable step;
    ConsumeMany body;
    bool parallel;
};

ConsumeMany Reducible(Assign start, Expr parameter, Variable step, ConsumeMany body, bool parallel = false);
ConsumeMany Reducible(Assign start, Expr parameter, Variable step, std::vector<SubsetObj> body,
                      bool parallel = false);
ConsumeMany Reducible(Assign start, Expr parameter, Variable step, SubsetObj body, bool parallel = false);

struct AllocatesNode : public StmtNode {
    AllocatesNode(Expr reg, Expr smem)
        : StmtNode(StmtKind::Allocates), reg(reg), smem(smem) {
    }
    Expr reg;
    Expr smem;
};

class Allocates : public Stmt {
public:
    Allocates()
        : Stmt() {
    }
    explicit Allocates(const AllocatesNode *n)
        : Stmt(n) {
    }
    Allocates(Expr reg, Expr smem = Expr())
        : Stmt(new const AllocatesNode(reg, smem)) {
    }
    typedef AllocatesNode Node;
    static bool classof(const StmtNode *n) {
        return n->kind == StmtKind::Allocates;
    }
};

// Either a tileable loop around a pattern, or the innermost
// (produces, consumes) pair.
class Pattern : public Stmt {
public:
    Pattern()
        : Stmt() {
    }
    explicit Pattern(const StmtNode *n)
        : Stmt(n) {
    }
    Annotation occupies(std::set<Grid::Unit>) const;
    Annotation assumes(std::vector<Constraint>) const;
    template<typename First, typename... Remaining>
    Annotation assumes(First first, Remaining... remaining) const;

    std::vector<SubsetObj> getInputs() const;
    std::vector<SubsetObj> getAllADTs() const;
    std::vector<Variable> getProducesField() const;
    // The subset fields this pattern requires of data structure d (as an input
    // or as the output).
    std::vector<Expr> getRequirement(AbstractDataTypePtr d) const;
    SubsetObj getOutput() const;
    SubsetObj getCorrespondingSubset(AbstractDataTypePtr d) const;
    typedef StmtNode Node;
    static bool classof(const StmtNode *n) {
        return n->kind == StmtKind::ComputesFor || n->kind == StmtKind::Computes;
    }
};

struct ComputesNode : public StmtNode {
    ComputesNode(Produces p, Consumes c, Allocates a)
        : StmtNode(StmtKind::Computes), p(p), c(c), a(a) {
    }
    Produces p;
    Consumes c;
    Allocates a;
};

class Computes : public Pattern {
public:
    explicit Computes(const ComputesNode *n)
        : Pattern(n) {
    }
    Computes(Produces p, Consumes c, Allocates a = Allocates())
        : Pattern(new const ComputesNode(p, c, a)) {
    }
    typedef ComputesNode Node;
    static bool classof(const StmtNode *n) {
        return n->kind == StmtKind::Computes;
    }
};

// for (start; < parameter; += step) over the OUTPUT side: the output can be
// produced `step` of this range at a time.
struct ComputesForNode : public StmtNode {
    ComputesForNode(Assign start, Expr parameter, Variable step, Pattern body, bool parallel)
        : StmtNode(StmtKind::ComputesFor), start(start), parameter(parameter), step(step), body(body),
          parallel(parallel) {
    }
    Assign start;
    Expr parameter;
    Variable step;
    Pattern body;
    bool parallel;
};

Pattern Tileable(Assign start, Expr parameter, Variable step, Pattern body, bool parallel = false);
Pattern Tileable(Assign start, Expr parameter, Variable step, Produces produces, Consumes consumes,
                 bool parallel = false);

struct AnnotationNode : public StmtNode {
    AnnotationNode(Pattern p, std::set<Grid::Unit> occupied, std::vector<Constraint> constraints)
        : StmtNode(StmtKind::Annotation), p(p), occupied(std::move(occupied)),
          constraints(std::move(constraints)) {
    }
    Pattern p;
    std::set<Grid::Unit> occupied;
    std::vector<Constraint> constraints;
};

// A pattern plus the grid units the function occupies when it runs and the
// constraints it assumes of its variables and of the launch dimensions.
class Annotation : public Stmt {
public:
    Annotation() = default;
    Annotation(const AnnotationNode *n)
        : Stmt(n) {
    }
    Annotation(Pattern, std::set<Grid::Unit>, std::vector<Constraint>);
    Pattern getPattern() const;
    std::vector<Constraint> getConstraints() const;
    std::set<Grid::Unit> getOccupiedUnits() const;

    // Throws UserError when a constraint mentions a variable that is not in
    // the pattern, or a launch dimension the occupied units do not control.
    Annotation assumes(std::vector<Constraint>) const;
    template<typename First, typename... Remaining>
    Annotation assumes(First first, Remaining... remaining) const {
        static_assert(std::is_base_of_v<Constraint, First> && (std::is_base_of_v<Constraint, Remaining> && ...),
                      "All arguments must be children of Constraint");
        return this->assumes(std::vector<Constraint>{first, remaining...});
    }
    typedef AnnotationNode Node;
    static bool classof(const StmtNode *n) {
        return n->kind == StmtKind::Annotation;
    }
};

template<typename First, typename... Remaining>
Annotation Pattern::assumes(First first, Remaining... remaining) const {
    static_assert(std::is_base_of_v<Constraint, First> && (std::is_base_of_v<Constraint, Remaining> && ...),
                  "All arguments must be children of Constraint");
    return this->assumes(std::vector<Constraint>{first, remaining...});
}

Annotation annotate(Pattern);
Annotation resetUnit(Annotation, std::set<Grid::Unit>);

// ---------------------------------------------------------------------------
// Queries and rewrites used by composition and lowering
// ---------------------------------------------------------------------------
struct Substitution {
    std::map<std::string, Expr> variables;                 // by variable name
    std::map<std::string, AbstractDataTypePtr> structures;  // by data-structure name
    std::map<Grid::Dim, Expr> dims;
    bool empty() const {
        return variables.empty() && structures.empty() && dims.empty();
    }
};

Expr substitute(const Expr &, const Substitution &);
Constraint substitute(const Constraint &, const Substitution &);
Stmt substitute(const Stmt &, const Substitution &);

std::set<Variable> getVariables(const Expr &);
std::set<Variable> getVariables(const Constraint &);
std::set<Variable> getVariables(const Stmt &);
std::set<Grid::Dim> getDims(const Constraint &);
std::set<Grid::Dim> getDims(const Expr &);

Annotation substitute(const Annotation &, const Substitution &);
Pattern substitute(const Pattern &, const Substitution &);

// True when every leaf is a compile-time constant (literal, const-expr
// variable, const-expr member).
bool isConstExpr(const Expr &);
bool isConstExpr(const Constraint &);

// Gives every variable of the annotation a fresh unique name, except those
// that are loop bounds; records old -> new.
Annotation refreshVariables(Annotation annot, std::map<Variable, Variable> &new_vars);

}  // namespace gern
