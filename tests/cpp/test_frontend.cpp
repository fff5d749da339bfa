// Front-end behaviour that needs no code generation: expression nodes and
// their printed form, structural equality, call-site checks, pipeline
// legality, grid constraints and unit mapping.
//
// Each case states the behaviour that the reference's own tests specify:
// test/test-nodes.cpp, test-same-expr.cpp, test-functions.cpp,
// test-pipeline.cpp, test-grid-constraints.cpp, test-map-grid.cpp,
// test-set-unit.cpp.
#include "resolve_constraints/resolve_constraints.h"
#include "annotations/data_dependency_language.h"
#include "annotations/visitor.h"
#include "compose/composable.h"
#include "compose/compose.h"
#include "utils/error.h"

#include "check.h"
#include "library/array_annot.h"
#include "library/array_device_annot.h"

#include <algorithm>
#include <set>

using namespace gern;
using check::stripped;

template<typename T>
static bool disjoint(const std::set<T> &a, const std::set<T> &b) {
    for (const auto &v : a) {
        if (b.count(v)) {
            return false;
        }
    }
    return true;
}

// ---- test-nodes.cpp -----------------------------------------------------------

CASE("nodes.literal_datatypes") {  // test-nodes.cpp:11-23
    REQUIRE(Expr((uint64_t)4).ptr->getDatatype().getKind() == Datatype::Kind::UInt64);
    REQUIRE(Expr((uint32_t)4).ptr->getDatatype().getKind() == Datatype::Kind::UInt32);
    REQUIRE(Expr((double)4).ptr->getDatatype().getKind() == Datatype::Kind::Float64);
}

CASE("nodes.binary_printing") {  // test-nodes.cpp:25-33
    Variable v{"v"};
    REQUIRE_EQ(stripped((v + 4) / (v * 4)), std::string("((v+4)/(v*4))"));
    REQUIRE_EQ(stripped(v + 4 && v * 4), std::string("((v+4)&&(v*4))"));
    REQUIRE_EQ(stripped(v % 4 >= v * 4), std::string("((v%4)>=(v*4))"));
    REQUIRE_EQ(stripped(Argument(v + v)), std::string("(v+v)"));
}

CASE("nodes.constraint_printing") {  // test-nodes.cpp:35-52
    Variable v("v_");
    Expr e = 1 - v;
    REQUIRE_EQ(stripped(e == e), std::string("((1-v_)==(1-v_))"));
    REQUIRE_EQ(stripped(e <= e), std::string("((1-v_)<=(1-v_))"));
    REQUIRE_EQ(stripped(e != e), std::string("((1-v_)!=(1-v_))"));
    REQUIRE_EQ(stripped(e < e), std::string("((1-v_)<(1-v_))"));
    REQUIRE_EQ(stripped(e > e), std::string("((1-v_)>(1-v_))"));
    REQUIRE_EQ(stripped(e && e), std::string("((1-v_)&&(1-v_))"));
    REQUIRE_EQ(stripped(e || e), std::string("((1-v_)||(1-v_))"));
    auto ds = AbstractDataTypePtr(new const annot::ArrayCPU());
    SubsetObj subset{ds, {1 - v, v * 2}};
    REQUIRE_EQ(stripped(subset), std::string("test{(1-v_),(v_*2)}"));
}

CASE("nodes.assumes_only_known_variables") {  // test-nodes.cpp:54-72
    Variable v("v"), v1("v1");
    auto ds = AbstractDataTypePtr(new const annot::ArrayCPU());
    SubsetObj s{ds, {1 - v, v * 2}};
    REQUIRE_NOTHROW(Tileable(v = Expr(0), ds["dummy"], v,
                             Computes(Produces::Subset(ds, {v, v}), Consumes(SubsetObjMany(s))))
                        .assumes(Constraint(v == 1)));
    REQUIRE_THROWS_AS(Tileable(v = Expr(0), ds["dummy"], v,
                               Computes(Produces::Subset(ds, {v, v}), Consumes(SubsetObjMany(s))))
                          .assumes(Constraint(v1 == 1)),
                      error::UserError);
}

CASE("nodes.null_handles") {  // test-nodes.cpp:74-90
    Expr().str();
    Stmt().str();
    Constraint().str();
    AbstractDataTypePtr().str();
    Argument().str();
    REQUIRE_THROWS_AS(AbstractDataTypePtr().getInsertFunction(), error::InternalError);
    REQUIRE_THROWS_AS(AbstractDataTypePtr().getQueryFunction(), error::InternalError);
    REQUIRE_THROWS_AS(AbstractDataTypePtr().getName(), error::InternalError);
    REQUIRE_THROWS_AS(AbstractDataTypePtr().getType(), error::InternalError);
    REQUIRE_THROWS_AS(AbstractDataTypePtr().getFields(), error::InternalError);
    REQUIRE_THROWS_AS(AbstractDataTypePtr().getAllocateFunction(), error::InternalError);
    REQUIRE_THROWS_AS(AbstractDataTypePtr().freeQuery(), error::InternalError);
    REQUIRE_THROWS_AS(AbstractDataTypePtr().insertQuery(), error::InternalError);
    REQUIRE_THROWS_AS(AbstractDataTypePtr().freeAlloc(), error::InternalError);
}

// ---- test-same-expr.cpp -------------------------------------------------------

CASE("same_expr.variables_members_dims") {  // test-same-expr.cpp:9-41
    Variable a("a"), b("b");
    REQUIRE(isSameExpr(a, a));
    REQUIRE(!isSameExpr(a, b));
    REQUIRE(!isSameExpr(a, 0));
    REQUIRE(!isSameExpr(a, Expr()));
    REQUIRE(!isSameExpr(Expr(), a));
    REQUIRE(isSameExpr(Expr(), Expr()));
    AbstractDataTypePtr da = annot::ArrayCPU("a");
    AbstractDataTypePtr db = annot::ArrayCPU("b");
    REQUIRE(isSameExpr(da["a"], da["a"]));
    REQUIRE(!isSameExpr(da["a"], db["a"]));
    REQUIRE(!isSameExpr(da["a"], da["b"]));
    Grid::Dim x(Grid::Dim::BLOCK_DIM_X), x2(Grid::Dim::BLOCK_DIM_X), y(Grid::Dim::BLOCK_DIM_Y);
    REQUIRE(isSameExpr(x, x));
    REQUIRE(isSameExpr(x, x2));
    REQUIRE(!isSameExpr(x, y));
}

CASE("same_expr.compound") {  // test-same-expr.cpp:43-67
    Variable a("a"), b("b"), c("c");
    REQUIRE(isSameExpr(a + b, a + b));
    REQUIRE(isSameExpr(a - b, a - b));
    REQUIRE(isSameExpr(a * b, a * b));
    REQUIRE(isSameExpr(a / b, a / b));
    REQUIRE(isSameExpr(a % b, a % b));
    REQUIRE(!isSameExpr(a + b, a + c));
    REQUIRE(!isSameExpr(a, a + c));
    REQUIRE(!isSameExpr(a + b, a));
    REQUIRE(!isSameExpr(a + b, a - b));
    REQUIRE(isSameExpr(a + b * c, a + b * c));
    REQUIRE(isSameExpr(a % b / c, a % b / c));
    REQUIRE(!isSameExpr(a + b * c, a - b * c));
    REQUIRE(!isSameExpr(a + b * c, a - b));
    REQUIRE(!isSameExpr(a + b * c, a));
}

// ---- test-resolve-constraints.cpp ------------------------------------------------
// The reference's cases (its solver is GiNaC, whose answers come out over the rationals: y*0.25; here the
// solution stays over the nodes of the equation: y / 4), and what the interface excludes.

CASE("resolve.one_variable_on_either_side") {  // test-resolve-constraints.cpp:8-22
    Variable x("x"), y("y");
    Expr sol = resolve::solve(x == y, x);
    REQUIRE(sol.ptr == y.ptr);  // the variable itself, as the reference asserts
    REQUIRE_EQ(resolve::solve((x - 1) == y, x).str(), std::string("(y + 1)"));
    REQUIRE_EQ(resolve::solve(x == y - 1, x).str(), std::string("(y - 1)"));
    REQUIRE_EQ(resolve::solve(y == x + 3, x).str(), std::string("(y - 3)"));
    REQUIRE_EQ(resolve::solve(Expr(7) == x, x).str(), std::string("7"));
}

CASE("resolve.coefficients") {  // test-resolve-constraints.cpp:24-36
    Variable x("x"), y("y"), z("z");
    REQUIRE_EQ(resolve::solve((x * 4) == y, x).str(), std::string("(y / 4)"));
    REQUIRE(isSameExpr(resolve::solve(x * z == y, x), y / z));
    REQUIRE(isSameExpr(resolve::solve(z * x == y, x), y / z));
    REQUIRE_EQ(resolve::solve(x / 2 == y, x).str(), std::string("(y / 0.5)"));  // 1 / 2 is not a whole number: folded as a fraction
    // literals fold: 2 x + 3 x = 10
    REQUIRE_EQ(resolve::solve(x * 2 + x * 3 == Expr(10), x).str(), std::string("2"));
}

CASE("resolve.coefficients_and_sums") {  // test-resolve-constraints.cpp:38-47
    Variable x("x"), y("y"), z("z");
    REQUIRE_EQ(resolve::solve((x * 4) + z == y, x).str(), std::string("((y - z) / 4)"));
    // the variable on both sides: 3 x + y = x + z
    REQUIRE_EQ(resolve::solve(x * 3 + y == x + z, x).str(), std::string("((z - y) / 2)"));
    // a tile's extent from its consumer's: l + stride - 1 = n
    Variable l("l"), stride("stride"), n("n");
    REQUIRE_EQ(resolve::solve(l + stride - 1 == n, l).str(), std::string("(n - (stride - 1))"));
}

CASE("resolve.what_is_not_linear_is_refused") {
    Variable x("x"), y("y");
    REQUIRE_THROWS_AS(resolve::solve(x * x == y, x), error::UserError);
    REQUIRE_THROWS_AS(resolve::solve(y / x == Expr(2), x), error::UserError);
    REQUIRE_THROWS_AS(resolve::solve(x % 4 == y, x), error::UserError);
    REQUIRE_THROWS_AS(resolve::solve(y == Expr(3), x), error::UserError);   // x does not occur
    REQUIRE_THROWS_AS(resolve::solve(x + y == x + 1, x), error::UserError);  // its coefficient cancels
}

// ---- test-functions.cpp -------------------------------------------------------

CASE("functions.argument_types") {  // test-functions.cpp:13-18
    Variable x("x"), y("y");
    REQUIRE(Argument(x + y).isSameTypeAs(x));
    REQUIRE(Argument(x + y).isSameTypeAs(Argument(x + y)));
}

CASE("functions.call_site_checks") {  // test-functions.cpp:20-41
    annot::add_1 add_1;
    AbstractDataTypePtr in(new const annot::ArrayCPU("input_con"));
    AbstractDataTypePtr out(new const annot::ArrayCPU("output_con"));
    REQUIRE_THROWS_AS(add_1(), error::UserError);
    REQUIRE_THROWS_AS(add_1(in), error::UserError);
    REQUIRE_THROWS_AS(add_1(in, in, out), error::UserError);
    REQUIRE_THROWS_AS(add_1(Argument(), Argument()), error::UserError);
    REQUIRE_THROWS_AS(add_1(in, in), error::UserError);  // would overwrite its input
    annot::addWithSize with_size;
    REQUIRE_THROWS_AS(with_size(in, Variable{"x"}, out), error::UserError);
    REQUIRE_NOTHROW(with_size(in, out, Variable{"x"}));
}

CASE("functions.fresh_variables_per_call") {  // test-functions.cpp:43-72
    AbstractDataTypePtr in(new const annot::ArrayCPU("input_con"));
    AbstractDataTypePtr out(new const annot::ArrayCPU("output_con"));
    AbstractDataTypePtr out2(new const annot::ArrayCPU("output_con_2"));
    annot::add_1 add_1;
    Composable c1 = add_1(in, out);
    Composable c2 = add_1(out, out2);
    std::set<Variable> abstract_vars = getVariables(add_1.getAnnotation().getPattern());
    std::set<Variable> vars1 = getVariables(c1.getAnnotation().getPattern());
    std::set<Variable> vars2 = getVariables(c2.getAnnotation().getPattern());
    REQUIRE(disjoint(vars1, abstract_vars));
    REQUIRE(disjoint(vars2, abstract_vars));
    REQUIRE(disjoint(vars2, vars1));
    REQUIRE(c1.getAnnotation().getPattern().getOutput().getDS() == out);
    REQUIRE(c2.getAnnotation().getPattern().getOutput().getDS() == out2);
    std::vector<SubsetObj> in1 = c1.getAnnotation().getPattern().getInputs();
    REQUIRE(in1.size() == 1 && in1.begin()->getDS() == in);
    std::vector<SubsetObj> in2 = c2.getAnnotation().getPattern().getInputs();
    REQUIRE(in2.size() == 1 && in2.begin()->getDS() == out);
}

// ---- test-pipeline.cpp --------------------------------------------------------

CASE("pipeline.outputs_are_assigned_once") {  // test-pipeline.cpp:13-72
    AbstractDataTypePtr in(new const annot::ArrayCPU("input_con"));
    AbstractDataTypePtr out(new const annot::ArrayCPU("output_con_val"));
    AbstractDataTypePtr temp(new const annot::ArrayCPU("tempDS"));
    annot::add_1 add_1;
    Variable v("v"), v1("v1");
    REQUIRE_NOTHROW(Composable());
    REQUIRE_NOTHROW(Composable({add_1(in, temp), add_1(temp, out)}));
    REQUIRE_THROWS_AS(Composable({add_1(in, out), Tile(out["size"], v)(add_1(in, out))}), error::UserError);
    REQUIRE_THROWS_AS(Tile(out["size"], v)(Tile(out["size"], v1)(add_1(out, out)), add_1(in, out)), error::UserError);
    // writes an output the nested stage has read
    REQUIRE_THROWS_AS(Tile(out["size"], v)(Tile(out["size"], v1)(add_1(in, out)), add_1(out, in)), error::UserError);
    // writes an input the enclosing stage has read
    REQUIRE_THROWS_AS(Tile(out["size"], v)(add_1(in, out), Tile(out["size"], v1)(add_1(out, in))), error::UserError);
}

CASE("pipeline.chained_outputs_are_fine") {  // test-pipeline.cpp:74-93
    AbstractDataTypePtr in(new const annot::ArrayCPU("input_con"));
    AbstractDataTypePtr out(new const annot::ArrayCPU("output_con"));
    AbstractDataTypePtr out_new(new const annot::ArrayCPU("output_con_new"));
    annot::add_1 add_1;
    Variable v("v"), v1("v1");
    REQUIRE_NOTHROW(Composable({add_1(in, out), add_1(out, out_new)}));
    REQUIRE_NOTHROW(Tile(out_new["size"], v)(add_1(in, out), Tile(out_new["size"], v1)(add_1(out, out_new))));
}

CASE("pipeline.intermediates_stay_private") {  // test-pipeline.cpp:95-133
    AbstractDataTypePtr in(new const annot::ArrayCPU("input_con"));
    AbstractDataTypePtr out(new const annot::ArrayCPU("output_con"));
    AbstractDataTypePtr out_vis(new const annot::ArrayCPU("output_con_vis"));
    AbstractDataTypePtr out_new(new const annot::ArrayCPU("output_con_new"));
    annot::add_1 add_1;
    Variable v("v");
    REQUIRE_THROWS_AS(Composable({Tile(out_new["size"], v)(add_1(in, out), add_1(out, out_new)), add_1(out, out_vis)}),
                      error::UserError);
    REQUIRE_THROWS_AS(Composable({Tile(out_new["size"], v)(add_1(in, out), add_1(out, out_new)), add_1(out_new, out)}),
                      error::UserError);
    REQUIRE_NOTHROW(Composable({Composable({add_1(in, out), add_1(out, out_new)}), add_1(out_new, out_vis)}));
}

CASE("pipeline.no_unused_outputs") {  // test-pipeline.cpp:135-164
    AbstractDataTypePtr in(new const annot::ArrayCPU("input_con"));
    AbstractDataTypePtr out(new const annot::ArrayCPU("output_con"));
    AbstractDataTypePtr out_new(new const annot::ArrayCPU("output_con_new"));
    annot::add_1 add_1;
    Variable v("v"), v1("v1");
    REQUIRE_THROWS_AS(Composable({add_1(in, out), add_1(in, out_new)}), error::UserError);
    REQUIRE_THROWS_AS(Composable({add_1(in, out), Tile(out_new["size"], v)(add_1(in, out_new))}), error::UserError);
    REQUIRE_THROWS_AS(Composable({Tile(out_new["size"], v)(add_1(in, out_new)), add_1(in, out)}), error::UserError);
    REQUIRE_THROWS_AS(Composable({Tile(out_new["size"], v)(Tile(out_new["size"], v)(Tile(out_new["size"], v1)(add_1(in, out_new)))),
                                  add_1(in, out)}),
                      error::UserError);
}

// ---- test-grid-constraints.cpp -----------------------------------------------

CASE("grid.constrainable_dimensions") {  // test-grid-constraints.cpp:12-76
    Variable v("v");
    auto ds = AbstractDataTypePtr(new const annot::ArrayCPU());
    SubsetObj s{ds, {1 - v, v * 2}};
    auto pattern = [&]() {
        return Tileable(v = Expr(0), ds["dummy"], v, Computes(Produces::Subset(ds, {v, v}), Consumes(SubsetObjMany(s))));
    };
    // a dimension the function does not occupy
    REQUIRE_THROWS_AS(pattern().assumes(Grid::Dim::BLOCK_DIM_X == v), error::UserError);
    // a different dimension of the same level
    REQUIRE_THROWS_AS(pattern().occupies({Grid::Unit::THREAD_X}).assumes(Grid::Dim::BLOCK_DIM_Y == v), error::UserError);
    // a parent level
    REQUIRE_THROWS_AS(pattern().occupies({Grid::Unit::THREAD_X, Grid::Unit::THREAD_Y}).assumes(Grid::Dim::GRID_DIM_X == v),
                      error::UserError);
    REQUIRE_NOTHROW(pattern().occupies({Grid::Unit::THREAD_X}).assumes(Grid::Dim::BLOCK_DIM_X == v));
    REQUIRE_NOTHROW(pattern().occupies({Grid::Unit::THREAD_X, Grid::Unit::THREAD_Y}).assumes(Grid::Dim::BLOCK_DIM_Y == v));
    // a child level of an occupied unit
    REQUIRE_NOTHROW(pattern().occupies({Grid::Unit::BLOCK_X, Grid::Unit::THREAD_Y}).assumes(Grid::Dim::BLOCK_DIM_Y == v));
}

// ---- test-map-grid.cpp ----------------------------------------------------------

CASE("grid.mapping_respects_hierarchy") {  // test-map-grid.cpp:12-58
    auto in = AbstractDataTypePtr(new const annot::ArrayStaticGPU("input_con"));
    auto temp = AbstractDataTypePtr(new const annot::ArrayStaticGPU("temp", true));
    auto out = AbstractDataTypePtr(new const annot::ArrayStaticGPU("output_con"));
    annot::Add1GPUTemplate add_1;
    Variable step("step"), blk("blk");
    REQUIRE_THROWS_AS((Tile(out["size"], blk) || Grid::Unit::THREAD_X)(
                          (Tile(out["size"], step) || Grid::Unit::BLOCK_X)(add_1(in, temp), add_1(temp, out))),
                      error::UserError);
    REQUIRE_THROWS_AS((Tile(out["size"], blk) || Grid::Unit::THREAD_X)(Tile(out["size"], blk)(
                          (Tile(out["size"], step) || Grid::Unit::BLOCK_X)(add_1(in, temp), add_1(temp, out)))),
                      error::UserError);
    REQUIRE_NOTHROW((Tile(out["size"], blk) || Grid::Unit::THREAD_X)(Tile(out["size"], blk)(
        (Tile(out["size"], step) || Grid::Unit::THREAD_Y)(add_1(in, temp), add_1(temp, out)))));
    REQUIRE_NOTHROW(Composable({
        (Tile(temp["size"], blk) || Grid::Unit::BLOCK_X)(add_1(in, temp)),
        (Tile(out["size"], step) || Grid::Unit::THREAD_X)(add_1(temp, out)),
    }));
}

// ---- test-set-unit.cpp ----------------------------------------------------------

CASE("grid.occupied_level_without_mapping") {  // test-set-unit.cpp:12-47
    auto in = AbstractDataTypePtr(new const annot::ArrayStaticGPU("input_con"));
    auto temp = AbstractDataTypePtr(new const annot::ArrayStaticGPU("temp", true));
    auto out = AbstractDataTypePtr(new const annot::ArrayStaticGPU("output_con"));
    annot::Add1GPUTemplate add_1;
    Variable step("step"), blk("blk");
    Composable program = add_1(temp, out);
    REQUIRE(getLevel(program.getAnnotation().getOccupiedUnits()) == Grid::Level::SCALAR);
    program = Tile(out["size"], step)(add_1(temp, out));
    REQUIRE(getLevel(program.getAnnotation().getOccupiedUnits()) == Grid::Level::SCALAR);
    program = Tile(out["size"], blk)(Tile(out["size"], step)(add_1(temp, out)));
    REQUIRE(getLevel(program.getAnnotation().getOccupiedUnits()) == Grid::Level::SCALAR);
    program = Tile(out["size"], blk)(Tile(out["size"], step)(add_1(in, temp), add_1(temp, out)));
    REQUIRE(getLevel(program.getAnnotation().getOccupiedUnits()) == Grid::Level::SCALAR);
}

CASE("grid.occupied_level_with_mapping") {  // test-set-unit.cpp:49-90
    auto in = AbstractDataTypePtr(new const annot::ArrayStaticGPU("input_con"));
    auto temp = AbstractDataTypePtr(new const annot::ArrayStaticGPU("temp", true));
    auto out = AbstractDataTypePtr(new const annot::ArrayStaticGPU("output_con"));
    annot::Add1GPUTemplate add_1;
    Variable step("step"), blk("blk");
    Composable program = (Tile(out["size"], step) || Grid::Unit::THREAD_X)(add_1(temp, out));
    REQUIRE(getLevel(program.getAnnotation().getOccupiedUnits()) == Grid::Level::THREADS);
    program = (Tile(out["size"], step) || Grid::Unit::BLOCK_X)(add_1(temp, out));
    REQUIRE(getLevel(program.getAnnotation().getOccupiedUnits()) == Grid::Level::BLOCK);
    program = (Tile(out["size"], blk) || Grid::Unit::BLOCK_X)((Tile(out["size"], step) || Grid::Unit::THREAD_X)(add_1(temp, out)));
    REQUIRE(getLevel(program.getAnnotation().getOccupiedUnits()) == Grid::Level::BLOCK);
    program = Composable({(Tile(temp["size"], blk) || Grid::Unit::BLOCK_X)(add_1(in, temp)),
                          (Tile(out["size"], step) || Grid::Unit::THREAD_X)(add_1(temp, out))});
    REQUIRE(getLevel(program.getAnnotation().getOccupiedUnits()) == Grid::Level::BLOCK);
    program = Composable({(Tile(temp["size"], blk) || Grid::Unit::BLOCK_X)(add_1(in, temp)),
                          Tile(out["size"], step)(add_1(temp, out))});
    REQUIRE(getLevel(program.getAnnotation().getOccupiedUnits()) == Grid::Level::BLOCK);
}

// ---- wave64: what this backend changes in the unit model -------------------------

CASE("grid.wavefront_is_64_lanes") {
    // The reference's users assume 32 (include/gern/annotations/grid.h:8-58);
    // on gfx950 a WARP unit is a 64-lane wavefront.
    REQUIRE_EQ(Grid::kWavefrontSize, 64);
    REQUIRE_EQ(stripped(Grid::Unit::WARP_Z), std::string("WARP_Z"));
}

CHECK_MAIN()
