// Lowering to host code and running it: every case composes a small program,
// lets the Runner generate C++, compile it with the host compiler, load it and
// run it, and compares the result with a closed form.
//
// The cases follow the reference's host lowering tests: test/test-cpu-array.cpp,
// test-cpu-reduction.cpp, test-composable.cpp, test-stage.cpp,
// test-temp-reuse.cpp, test-ordered-parameters.cpp, test-cpu-static-store.cpp,
// test-function-ptr.cpp, test-cpu-matrix.cpp, test-cpu-mm.cpp.
#include "annotations/abstract_function.h"
#include "compose/composable.h"
#include "compose/compose.h"
#include "compose/runner.h"
#include "utils/error.h"

#include "check.h"
#include "library/array_annot.h"
#include "library/array_host.h"
#include "library/array_static_annot.h"
#include "library/array_static_host.h"
#include "library/matrix_annot.h"
#include "library/matrix_host.h"

#include <cmath>
#include <cstdlib>

using namespace gern;

static Runner::Options hostOptions() {
    Runner::Options o;
    const char *lib = std::getenv("GERN_TEST_LIBRARY");
    const char *tmp = std::getenv("GERN_TEST_TMP");
    o.filename = "gern_test_host.cpp";
    o.prefix = tmp ? tmp : "/tmp";
    o.include = std::string(" -I ") + (lib ? lib : "tests/cpp/library");
    o.cpp_std = "c++17";
    return o;
}

static AbstractDataTypePtr arrayDS(const std::string &name) {
    return AbstractDataTypePtr(new const annot::ArrayCPU(name));
}

struct Arrays {
    impl::ArrayCPU a, b;
    explicit Arrays(int64_t n)
        : a(n), b(n) {
        a.ascending();
        b.fill(0.0f);
    }
    ~Arrays() {
        a.destroy();
        b.destroy();
    }
    void expect_offset(float off) const {
        for (int64_t i = 0; i < a.size; i++) {
            REQUIRE_EQ(b.data[i], a.data[i] + off);
        }
    }
    void expect_constant(float v) const {
        for (int64_t i = 0; i < b.size; i++) {
            REQUIRE_EQ(b.data[i], v);
        }
    }
};

// ---- test-cpu-array.cpp ---------------------------------------------------------

CASE("array.single_function_and_argument_errors") {  // test-cpu-array.cpp:13-57
    auto in = arrayDS("input_con"), out = arrayDS("output_con");
    annot::add_1 add_1;
    Runner run(Composable(add_1(in, out)));
    run.compile(hostOptions());
    Arrays t(10);
    REQUIRE_NOTHROW(run.evaluate({{in.getName(), &t.a}, {out.getName(), &t.b}}));
    t.expect_offset(1);
    REQUIRE_THROWS_AS(run.evaluate({{in.getName(), &t.a}}), error::UserError);
    auto dummy = arrayDS("dummy_ds");
    REQUIRE_THROWS_AS(run.evaluate({{in.getName(), &t.a}, {dummy.getName(), &t.b}}), error::UserError);
}

CASE("array.two_fused_functions_temp_is_internal") {  // test-cpu-array.cpp:59-94
    auto in = arrayDS("input_con"), out = arrayDS("output_con"), temp = arrayDS("temp");
    annot::add_1 add_1;
    Variable step("step");
    Runner run(Composable(Tile(out["size"], step)(add_1(in, temp), add_1(temp, out))));
    REQUIRE_NOTHROW(run.compile(hostOptions()));
    Arrays t(10);
    int64_t step_val = 2;
    REQUIRE_NOTHROW(run.evaluate({{in.getName(), &t.a}, {out.getName(), &t.b}, {step.getName(), &step_val}}));
    t.expect_offset(2);
}

CASE("array.template_argument_must_be_bound") {  // test-cpu-array.cpp:96-150
    auto in = arrayDS("input_con"), out = arrayDS("output_con");
    annot::add1Template add_1;
    Variable step("step");
    Runner unbound(Composable(Tile(out["size"], step)(add_1(in, out))));
    REQUIRE_THROWS_AS(unbound.compile(hostOptions()), error::UserError);

    Runner run(Composable(Tile(out["size"], step.bind(5))(add_1(in, out))));
    REQUIRE_NOTHROW(run.compile(hostOptions()));
    Arrays t(10);
    int64_t step_val = 1;
    // a bound variable cannot be passed at run time
    REQUIRE_THROWS_AS(run.evaluate({{in.getName(), &t.a}, {out.getName(), &t.b}, {step.getName(), &step_val}}), error::UserError);
    REQUIRE_NOTHROW(run.evaluate({{in.getName(), &t.a}, {out.getName(), &t.b}}));
    t.expect_offset(1);
}

CASE("array.two_templated_functions") {  // test-cpu-array.cpp:152-187
    auto in = arrayDS("input_con"), out = arrayDS("output_con"), temp = arrayDS("temp");
    annot::add1Template add_1;
    Variable step("step");
    Runner run(Composable(Tile(out["size"], step.bind(5))(add_1(in, temp), add_1(temp, out))));
    REQUIRE_NOTHROW(run.compile(hostOptions()));
    Arrays t(10);
    REQUIRE_NOTHROW(run.evaluate({{in.getName(), &t.a}, {out.getName(), &t.b}}));
    t.expect_offset(2);
}

CASE("array.float_parameter") {  // test-cpu-array.cpp:212-253
    auto in = arrayDS("input_con"), out = arrayDS("output_con"), temp = arrayDS("temp");
    annot::add_1_float add;
    Variable v("v", Datatype::Float32), step("step");
    Runner run(Composable(Tile(out["size"], step.bind(5))(add(in, temp, v), add(temp, out, v))));
    REQUIRE_NOTHROW(run.compile(hostOptions()));
    Arrays t(10);
    float v_val = 1.0f;
    REQUIRE_NOTHROW(run.evaluate({{in.getName(), &t.a}, {out.getName(), &t.b}, {v.getName(), &v_val}}));
    t.expect_offset(2);
}

// ---- test-composable.cpp ----------------------------------------------------------

CASE("compose.unfused_sequence") {  // test-composable.cpp:15-49
    AbstractDataTypePtr in = annot::ArrayCPU("input_con"), out = annot::ArrayCPU("output_con"), temp = annot::ArrayCPU("temp");
    annot::add_1 add_1;
    Arrays t(10);
    evaluate(Composable({add_1(in, temp), add_1(temp, out)}), {{in.getName(), &t.a}, {out.getName(), &t.b}}, hostOptions());
    t.expect_offset(2);
}

CASE("compose.nested_tiles") {  // test-composable.cpp:51-88
    AbstractDataTypePtr in = annot::ArrayCPU("input_con"), out = annot::ArrayCPU("output_con"), temp = annot::ArrayCPU("temp");
    annot::add_1 add_1;
    Variable v("x"), v1("y");
    Arrays t(10);
    int64_t s1 = 5, s2 = 1;
    evaluate(Tile(out["size"], v)(Tile(out["size"], v1)(add_1(in, temp), add_1(temp, out))),
             {{in.getName(), &t.a}, {out.getName(), &t.b}, {v.getName(), &s1}, {v1.getName(), &s2}}, hostOptions());
    t.expect_offset(2);
}

CASE("compose.two_tiles_in_one_scope") {  // test-composable.cpp:90-123
    AbstractDataTypePtr in = annot::ArrayCPU("input_con"), out = annot::ArrayCPU("output_con"), temp = annot::ArrayCPU("temp");
    annot::add_1 add_1;
    Variable v("v"), v1("v1");
    Arrays t(10);
    int64_t s1 = 5, s2 = 1;
    evaluate(Composable({Tile(temp["size"], v)(add_1(in, temp)), Tile(out["size"], v1)(add_1(temp, out))}),
             {{in.getName(), &t.a}, {out.getName(), &t.b}, {v.getName(), &s1}, {v1.getName(), &s2}}, hostOptions());
    t.expect_offset(2);
}

// ---- test-cpu-reduction.cpp ---------------------------------------------------------

static void run_reduction(Composable program, std::map<std::string, int64_t> vars, float expected) {
    Runner run(program);
    run.compile(hostOptions());
    Arrays t(10);
    std::map<std::string, void *> args = {{"input_con", &t.a}, {"output_con", &t.b}};
    for (auto &kv : vars) {
        args[kv.first] = &kv.second;
    }
    REQUIRE_NOTHROW(run.evaluate(args));
    t.expect_constant(expected);
}

CASE("reduction.untiled") {  // test-cpu-reduction.cpp:13-43
    auto in = arrayDS("input_con"), out = arrayDS("output_con");
    annot::reduction reduction;
    Variable r_dim("r_dim");
    run_reduction(Composable(reduction(in, out, r_dim)), {{"r_dim", 10}}, 45);
}

CASE("reduction.outer_tile") {  // test-cpu-reduction.cpp:45-84
    auto in = arrayDS("input_con"), out = arrayDS("output_con");
    annot::reduction reduction;
    Variable v("v"), r_dim("r_dim");
    run_reduction(Tile(out["size"], v)(reduction(in, out, r_dim)), {{"r_dim", 10}, {"v", 1}}, 45);
}

CASE("reduction.inner_reduce") {  // test-cpu-reduction.cpp:86-127
    auto in = arrayDS("input_con"), out = arrayDS("output_con");
    annot::reduction reduction;
    Variable v("v"), r_dim("r_dim");
    run_reduction(Tile(out["size"], v)(Reduce(r_dim, v)(reduction(in, out, r_dim))), {{"r_dim", 10}, {"v", 1}}, 45);
}

CASE("reduction.tiles_and_reduces_nested") {  // test-cpu-reduction.cpp:129-175
    auto in = arrayDS("input_con"), out = arrayDS("output_con");
    annot::reduction reduction;
    Variable v("v"), v1("v1"), r_dim("r_dim");
    run_reduction(Tile(out["size"], v)(Tile(out["size"], v1)(Reduce(r_dim, v)(Reduce(r_dim, v1)(reduction(in, out, r_dim))))),
                  {{"r_dim", 10}, {"v", 5}, {"v1", 5}}, 45);
}

CASE("reduction.mixed_with_elementwise") {  // test-cpu-reduction.cpp:177-248
    auto in = arrayDS("input_con"), out = arrayDS("output_con"), temp = arrayDS("temp");
    annot::reduction reduction;
    annot::add_1 add_1;
    Variable v("v"), v1("v1"), r_dim("r_dim");
    // n(n-1)/2 + n
    run_reduction(Tile(out["size"], v)(Tile(out["size"], v1)(
                      Reduce(r_dim, v)(Reduce(r_dim, v1)(add_1(in, temp), reduction(temp, out, r_dim))))),
                  {{"r_dim", 10}, {"v", 5}, {"v1", 5}}, 55);
    run_reduction(Tile(out["size"], v)(Tile(out["size"], v1)(
                      add_1(in, temp), Reduce(r_dim, v)(Reduce(r_dim, v1)(reduction(temp, out, r_dim))))),
                  {{"r_dim", 10}, {"v", 5}, {"v1", 5}}, 55);
}

// ---- test-stage.cpp --------------------------------------------------------------------

CASE("stage.rejects_data_structure_not_in_scope") {  // test-stage.cpp:12-23
    auto in = arrayDS("input_con"), out = arrayDS("output_con"), temp = arrayDS("temp");
    annot::add_1 add_1;
    REQUIRE_THROWS_AS(Stage(temp, add_1(in, out)), error::UserError);
}

static void run_stage(Composable call, int64_t n, std::map<std::string, int64_t> vars, bool constant, float expected) {
    Runner run(call);
    run.compile(hostOptions());
    Arrays t(n);
    std::map<std::string, void *> args = {{"input_con", &t.a}, {"output_con", &t.b}};
    for (auto &kv : vars) {
        args[kv.first] = &kv.second;
    }
    run.evaluate(args);
    if (constant) {
        t.expect_constant(expected);
    } else {
        t.expect_offset(expected);
    }
}

CASE("stage.input_above_inner_tile") {  // test-stage.cpp:25-62
    auto in = arrayDS("input_con"), out = arrayDS("output_con");
    annot::add_1 add_1;
    Variable v("v");
    run_stage(Tile(out["size"], v)(Stage(in, Tile(out["size"], v)(add_1(in, out)))), 8, {{"v", 2}}, false, 1);
}

CASE("stage.input_above_two_inner_tiles") {  // test-stage.cpp:64-101
    auto in = arrayDS("input_con"), out = arrayDS("output_con");
    annot::add_1 add_1;
    Variable v("v");
    run_stage(Tile(out["size"], v)(Stage(in, Tile(out["size"], v)(Tile(out["size"], v)(add_1(in, out))))), 8, {{"v", 2}}, false, 1);
}

CASE("stage.twice") {  // test-stage.cpp:103-142
    auto in = arrayDS("input_con"), out = arrayDS("output_con");
    annot::add_1 add_1;
    Variable v("v");
    run_stage(Tile(out["size"], v)(Stage(in, Tile(out["size"], v)(Stage(in, Tile(out["size"], v)(Tile(out["size"], v)(add_1(in, out))))))),
              16, {{"v", 2}}, false, 1);
}

CASE("stage.around_a_reduction") {  // test-stage.cpp:144-182
    auto in = arrayDS("input_con"), out = arrayDS("output_con");
    annot::reduction reduction;
    Variable v("v"), v1("v1");
    run_stage(Tile(out["size"], v)(Stage(out, Reduce(v1, v)(Stage(in, reduction(in, out, v1))))), 16, {{"v", 2}, {"v1", 16}}, true,
              8 * 15);
}

CASE("stage.custom_stage_and_insert_functions") {  // test-stage.cpp:184-224
    auto in = arrayDS("input_con"), out = arrayDS("output_con");
    annot::ArrayCPU stage("stage_con");
    annot::add_1 add_1;
    Variable v("v");
    Composable call = Tile(out["size"], v)(
        Stage(out, stage.newStageFunction(), stage.getNewInsertFunction(),
              Tile(out["size"], v)(Tile(out["size"], v)(
                  Stage(in, stage.newStageFunction(),
                        Stage(out, stage.newStageFunction(), stage.getNewInsertFunction(), add_1(in, out)))))));
    Runner run(call);
    run.compile(hostOptions());
    REQUIRE(run.getSource().find("new_stage") != std::string::npos);
    // The write-back call is only emitted for data structures whose queries are
    // copies (insertQuery(), src/codegen/finalizer.cpp:73-76); ArrayCPU's are views.
    REQUIRE(run.getSource().find("new_insert") == std::string::npos);
    Arrays t(8);
    int64_t v_val = 2;
    run.evaluate({{"input_con", &t.a}, {"output_con", &t.b}, {"v", &v_val}});
    t.expect_offset(1);
}

// ---- test-temp-reuse.cpp ------------------------------------------------------------------

static void chain_of(int n) {
    annot::add_1 add_1;
    std::vector<AbstractDataTypePtr> ds;
    ds.push_back(annot::ArrayCPU("input_con"));
    for (int i = 1; i < n; i++) {
        ds.push_back(annot::ArrayCPU("temp" + std::to_string(i) + "_con"));
    }
    ds.push_back(annot::ArrayCPU("output_con"));
    std::vector<Composable> calls;
    for (int i = 0; i < n; i++) {
        calls.push_back(add_1(ds[i], ds[i + 1]));
    }
    Runner run{Composable(calls)};
    run.compile(hostOptions());
    Arrays t(10);
    run.evaluate({{"input_con", &t.a}, {"output_con", &t.b}});
    t.expect_offset((float)n);
}

CASE("temp_reuse.chains_of_4_5_6") {  // test-temp-reuse.cpp:31-98
    chain_of(4);
    chain_of(5);
    chain_of(6);
}

// ---- test-ordered-parameters.cpp --------------------------------------------------------------

CASE("runner.ordered_parameters") {  // test-ordered-parameters.cpp:13-69
    auto in = arrayDS("input_con"), out = arrayDS("output_con"), bad = arrayDS("bad");
    annot::add_1 add_1;
    Composable program(add_1(in, out));
    auto bad_init = [&] {
        Runner r(program, std::vector<Parameter>{Parameter{out}, Parameter{bad}});
        r.compile(hostOptions());
    };
    REQUIRE_THROWS_AS(bad_init(), error::UserError);
    Runner run(program, std::vector<Parameter>{Parameter{out}, Parameter{in}});
    run.compile(hostOptions());
    std::vector<std::string> order = run.getArgumentOrder();
    REQUIRE(order.size() == 2 && order[0] == "output_con" && order[1] == "input_con");
    Arrays t(10);
    REQUIRE_NOTHROW(run.evaluate({{in.getName(), &t.a}, {out.getName(), &t.b}}));
    t.expect_offset(1);
    REQUIRE_THROWS_AS(run.evaluate({{in.getName(), &t.a}}), error::UserError);
    auto dummy = arrayDS("dummy_ds");
    REQUIRE_THROWS_AS(run.evaluate({{in.getName(), &t.a}, {dummy.getName(), &t.b}}), error::UserError);
}

CASE("runner.default_parameter_order_is_by_name") {  // src/codegen/codegen.cpp:137-198
    auto in = arrayDS("zz_input"), out = arrayDS("aa_output");
    annot::add_1 add_1;
    Variable step("step");
    Runner run(Composable(Tile(out["size"], step)(add_1(in, out))));
    run.compile(hostOptions());
    std::vector<std::string> order = run.getArgumentOrder();
    REQUIRE(order.size() == 3 && order[0] == "aa_output" && order[1] == "zz_input" && order[2] == "step");
}

// ---- test-runner.cpp -----------------------------------------------------------------------------

CASE("runner.compile_failure_is_a_user_error") {  // test-runner.cpp:13-28
    auto in = arrayDS("input_con"), out = arrayDS("output_con");
    annot::add_1 add_1;
    Runner run(Composable(add_1(in, out)));
    Runner::Options no_include;
    no_include.filename = "gern_test_fail.cpp";
    no_include.prefix = hostOptions().prefix;
    REQUIRE_THROWS_AS(run.compile(no_include), error::UserError);  // the header is not on the include path
    REQUIRE_NOTHROW(run.compile(hostOptions()));
}

// ---- test-cpu-static-store.cpp ---------------------------------------------------------------------

CASE("static_store.single_and_fused") {  // test-cpu-static-store.cpp:13-75
    auto in = AbstractDataTypePtr(new const annot::ArrayCPUTemplate<10>("input_con"));
    auto temp = AbstractDataTypePtr(new const annot::ArrayCPUTemplate<10>("temp", true));
    auto out = AbstractDataTypePtr(new const annot::ArrayCPUTemplate<10>("output_con"));
    annot::addStaticStore add_1;
    Variable step("step");
    {
        Runner run(Composable(Tile(out["size"], step.bind(5))(add_1(in, out))));
        REQUIRE_NOTHROW(run.compile(hostOptions()));
        impl::ArrayCPUTemplate<10> a, b;
        a.ascending();
        REQUIRE_NOTHROW(run.evaluate({{in.getName(), &a}, {out.getName(), &b}}));
        for (int i = 0; i < 10; i++) {
            REQUIRE_EQ(b.data[i], a.data[i] + 1);
        }
    }
    {
        Runner run(Composable(Tile(out["size"], step.bind(5))(add_1(in, temp), add_1(temp, out))));
        REQUIRE_NOTHROW(run.compile(hostOptions()));
        impl::ArrayCPUTemplate<10> a, b;
        a.ascending();
        REQUIRE_NOTHROW(run.evaluate({{in.getName(), &a}, {out.getName(), &b}}));
        for (int i = 0; i < 10; i++) {
            REQUIRE_EQ(b.data[i], a.data[i] + 2);
        }
    }
}

// ---- test-function-ptr.cpp ---------------------------------------------------------------------------

CASE("function_ptr.basic") {  // test-function-ptr.cpp:13-42
    annot::add_1 add_1;
    auto in = arrayDS("input_con"), out = arrayDS("output_con");
    Runner::Options inner = hostOptions();
    inner.filename = "gern_test_inner.cpp";
    FunctionPtr fn(Composable(add_1(in, out)), inner);
    Runner run(Composable(fn(in, out)));
    run.compile(hostOptions());
    Arrays t(10);
    run.evaluate({{"input_con", &t.a}, {"output_con", &t.b}});
    t.expect_offset(1);
}

CASE("function_ptr.fused_inside") {  // test-function-ptr.cpp:44-86
    annot::add_1 add_1;
    auto in = arrayDS("input_con"), out = arrayDS("output_con"), temp = arrayDS("temp_con");
    Variable size("size");
    Runner::Options inner = hostOptions();
    inner.filename = "gern_test_inner.cpp";
    FunctionPtr fn(Tile(out["size"], size)(add_1(in, temp), add_1(temp, out)), inner);
    Runner run(Composable(fn(in, out, size)));
    run.compile(hostOptions());
    Arrays t(10);
    int64_t size_val = 5;
    run.evaluate({{in.getName(), &t.a}, {out.getName(), &t.b}, {size.getName(), &size_val}});
    t.expect_offset(2);
}

CASE("function_ptr.fused_inside_and_outside") {  // test-function-ptr.cpp:88-137
    annot::add_1 add_1;
    auto in = arrayDS("input_con"), out = arrayDS("output_con"), temp = arrayDS("temp_con");
    Variable size("size");
    Runner::Options inner = hostOptions();
    inner.filename = "gern_test_inner.cpp";
    FunctionPtr fn(Tile(out["size"], size)(add_1(in, temp), add_1(temp, out)), inner);
    Runner run(Composable(Tile(out["size"], size)(fn(in, temp, size), fn(temp, out, size))));
    run.compile(hostOptions());
    Arrays t(10);
    int64_t size_val = 5;
    run.evaluate({{in.getName(), &t.a}, {out.getName(), &t.b}, {size.getName(), &size_val}});
    t.expect_offset(4);
}

// ---- test-cpu-matrix.cpp -------------------------------------------------------------------------------

static AbstractDataTypePtr matrixDS(const std::string &name) {
    return AbstractDataTypePtr(new const annot::MatrixCPU(name));
}

CASE("matrix.tiled_add_runs_twice_with_new_tiles") {  // test-cpu-matrix.cpp:13-64
    auto in = matrixDS("input_con"), out = matrixDS("output_con");
    annot::MatrixAddCPU add;
    Variable l_x("l_x"), l_y("l_y");
    Runner run(Composable(Tile(out["row"], l_x)(Tile(out["col"], l_y)(add(in, out)))));
    run.compile(hostOptions());
    impl::MatrixCPU a(10, 20, 20), b(10, 20, 20);
    a.fill(2.0f);
    b.fill(0.0f);
    int64_t lx = 5, ly = 5;
    REQUIRE_NOTHROW(run.evaluate({{in.getName(), &a}, {out.getName(), &b}, {l_x.getName(), &lx}, {l_y.getName(), &ly}}));
    for (int i = 0; i < 200; i++) {
        REQUIRE_EQ(b.data[i], 3.0f);
    }
    a.fill(7.0f);
    ly = 2;
    REQUIRE_NOTHROW(run.evaluate({{in.getName(), &a}, {out.getName(), &b}, {l_x.getName(), &lx}, {l_y.getName(), &ly}}));
    for (int i = 0; i < 200; i++) {
        REQUIRE_EQ(b.data[i], 8.0f);
    }
    a.destroy();
    b.destroy();
}

// ---- test-cpu-mm.cpp -------------------------------------------------------------------------------------

CASE("mm.two_level_tiling_matches_direct_product") {  // test-cpu-mm.cpp:13-83
    auto A = matrixDS("A"), B = matrixDS("B"), C = matrixDS("C");
    annot::MatrixMultiplyCPU mm;
    Variable ti("ti"), ti_2("ti_2"), tj("tj"), tj_2("tj_2"), k("k"), k_2("k_2"), k_dim("k_dim");
    Runner run(Composable(Tile(C["row"], ti)(Tile(C["col"], tj)(Reduce(k_dim, k)(
        Tile(C["row"], ti_2)(Tile(C["col"], tj_2)(Reduce(k_dim, k_2)(mm(A, B, C, k_dim)))))))));
    run.compile(hostOptions());
    const int64_t n = 10;
    impl::MatrixCPU a(n, n, n), b(n, n, n), c(n, n, n), ref(n, n, n);
    a.ascending();
    b.ascending();
    c.fill(0.0f);
    ref.fill(0.0f);
    int64_t v5 = 5, v1 = 1, kd = n;
    run.evaluate({{"A", &a}, {"B", &b}, {"C", &c}, {"ti", &v5}, {"ti_2", &v1}, {"tj", &v5}, {"tj_2", &v1}, {"k", &v5},
                  {"k_2", &v1}, {"k_dim", &kd}});
    // One k per innermost call: the partial sums are added in the same order
    // as the direct product adds its terms, so the results are bit-identical.
    impl::MatrixCPU ref1(n, n, n);
    ref1.fill(0.0f);
    for (int64_t kk = 0; kk < n; kk++) {
        impl::matrix_multiply(a.query(0, kk, n, 1), b.query(kk, 0, 1, n), ref1, 1);
    }
    impl::matrix_multiply(a, b, ref, n);
    for (int i = 0; i < n * n; i++) {
        REQUIRE_EQ(c.data[i], ref1.data[i]);
        REQUIRE(c.data[i] == ref.data[i] || std::abs(c.data[i] - ref.data[i]) <= 1e-6f * std::abs(ref.data[i]));
    }
    a.destroy();
    b.destroy();
    c.destroy();
    ref.destroy();
    ref1.destroy();
}

static void double_mm(bool hoist) {  // test-cpu-mm.cpp:266-407
    auto A = matrixDS("A"), B = matrixDS("B"), D = matrixDS("D"), E = matrixDS("E");
    auto C = AbstractDataTypePtr(new const annot::MatrixCPUZero("C"));
    annot::MatrixMultiplyCPU mm;
    Variable k2("k2"), ti("ti"), tj("tj"), tk("tk");
    Composable program = hoist ? Composable({Tile(E["row"], ti)(mm(A, B, C, k2), Tile(E["col"], tj)(Reduce(k2, tk)(mm(C, D, E, k2))))}) :
                                 Composable({Tile(E["row"], ti)(Tile(E["col"], tj)(mm(A, B, C, k2), Reduce(k2, tk)(mm(C, D, E, k2))))});
    Runner run(program);
    run.compile(hostOptions());
    int64_t n = 4, t2 = 2;
    impl::MatrixCPU a(n, n, n), b(n, n, n), c(n, n, n), d(n, n, n), e(n, n, n), ref(n, n, n);
    a.ascending();
    b.ascending();
    d.ascending();
    c.fill(0.0f);
    e.fill(0.0f);
    ref.fill(0.0f);
    run.evaluate({{"A", &a}, {"B", &b}, {"D", &d}, {"E", &e}, {"k2", &n}, {"ti", &t2}, {"tj", &t2}, {"tk", &n}});
    impl::matrix_multiply(a, b, c, n);
    impl::matrix_multiply(c, d, ref, n);
    for (int i = 0; i < n * n; i++) {
        REQUIRE_EQ(e.data[i], ref.data[i]);
    }
    for (auto *m : {&a, &b, &c, &d, &e, &ref}) {
        m->destroy();
    }
}

CASE("mm.two_products_intermediate_per_tile") {
    double_mm(false);
}

CASE("mm.two_products_intermediate_hoisted") {
    double_mm(true);
}

CASE("mm.function_ptr_with_bound_tiles") {  // test-cpu-mm.cpp:189-264
    auto A = matrixDS("A"), B = matrixDS("B"), C = matrixDS("C");
    annot::MatrixMultiplyCPU mm;
    Variable ti("ti"), tj("tj"), tk("tk"), k_dim("k_dim"), ti_g("ti_g"), tj_g("tj_g");
    Runner::Options inner = hostOptions();
    inner.filename = "gern_test_inner_mm.cpp";
    Composable inner_program = Tile(C["row"], ti.bind(2))(Tile(C["col"], tj.bind(2))(mm(A, B, C, k_dim)));
    FunctionPtr inner_mm(inner_program, inner);
    // The inner function's template parameters are bound again at the call
    // site (bindings hold for the next call only).
    auto &bound_mm = inner_mm[{{"ti", ti.bind(2)}, {"tj", tj.bind(2)}}];
    Runner run(Composable(Tile(C["row"], ti_g.bind(4))(Tile(C["col"], tj_g.bind(4))(Reduce(k_dim, tk.bind(4))(bound_mm(A, B, C, k_dim))))));
    run.compile(hostOptions());
    const int64_t n = 8;
    impl::MatrixCPU a(n, n, n), b(n, n, n), c(n, n, n), ref(n, n, n);
    for (int64_t i = 0; i < n * n; i++) {
        a.data[i] = (float)(i % 10);
        b.data[i] = (float)((i * 7) % 10);
    }
    c.fill(0.0f);
    ref.fill(0.0f);
    int64_t kd = n;
    run.evaluate({{"A", &a}, {"B", &b}, {"C", &c}, {"k_dim", &kd}});
    impl::matrix_multiply(a, b, ref, n);
    for (int i = 0; i < n * n; i++) {
        REQUIRE_EQ(c.data[i], ref.data[i]);  // small integers: exact in any order
    }
    for (auto *m : {&a, &b, &c, &ref}) {
        m->destroy();
    }
}

// A query that takes nothing is moved to the top of the generated function when it opens a PARAMETER (its
// latency then hides behind what follows); a data structure that the program itself allocates and computes
// must be opened behind the statements that define it.
CASE("array.fieldless_query_of_an_intermediate_stays_behind_its_definition") {
    auto in = arrayDS("input_con"), out = arrayDS("output_con");
    auto s = AbstractDataTypePtr(new const annot::ScalarCPU("first"));
    annot::first_element first_element;
    annot::add_scalar add_scalar;
    Variable step("step");
    Runner run(Composable({first_element(in, s), Tile(out["size"], step)(add_scalar(in, s, out))}));
    REQUIRE_NOTHROW(run.compile(hostOptions()));
    const std::string src = run.getSource();
    const size_t allocated = src.find("ScalarCPU::allocate"), computed = src.find("first_element("), opened = src.find(".open(");
    REQUIRE(allocated != std::string::npos);
    REQUIRE(computed != std::string::npos);
    REQUIRE(opened != std::string::npos);
    REQUIRE(allocated < computed);
    REQUIRE(computed < opened);
    Arrays t(10);
    for (int64_t i = 0; i < t.a.size; i++) {
        t.a.data[i] = (float)(i + 5);
    }
    int64_t step_val = 5;
    REQUIRE_NOTHROW(run.evaluate({{in.getName(), &t.a}, {out.getName(), &t.b}, {step.getName(), &step_val}}));
    t.expect_offset(5);  // every element grew by the first one
}

CHECK_MAIN()
