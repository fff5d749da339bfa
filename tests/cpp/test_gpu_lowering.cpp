// Lowering to ONE HIP kernel for gfx950 and running it: unmapped loops,
// loops mapped to blocks / threads / wavefronts, repeated units, explicit
// launch dimensions, dynamic LDS with an allocator, LDS-staged tiles.
//
// The cases follow the reference's device lowering tests: test/test-gpu-array.cu,
// test-set-grid.cu, test-dynamic-shared.cu, test-gpu-matrix.cu, and the two
// reduction programs gernels/cccl/global_reduce.cu and rdom_mimic.cu.
//
// With GERN_TEST_COMPILE_ONLY=1 every program is generated and compiled for
// gfx950 with hiprtc but not loaded or run (no GPU needed).
#include "annotations/abstract_function.h"
#include "codegen/codegen.h"
#include "compose/composable.h"
#include "compose/compose.h"
#include "compose/runner.h"
#include "utils/error.h"

#include "check.h"
#include "library/array_device_annot.h"
#include "library/device_host.h"
#include "library/matrix_device_annot.h"

#include "annot/blur.h"
#include "annot/lds_matrix.h"
#include "annot/reduce.h"

#include <cstdlib>
#include <iostream>
#include <map>

using namespace gern;

static std::string libraryDir() {
    const char *lib = std::getenv("GERN_TEST_LIBRARY");
    return lib ? lib : "tests/cpp/library";
}

static std::string packageDir() {
    const char *pkg = std::getenv("GERN_TEST_PACKAGE");
    return pkg ? pkg : "gern_amd";
}

static bool compileOnly() {
    const char *v = std::getenv("GERN_TEST_COMPILE_ONLY");
    return v && v[0] == '1';
}

static std::string last_source;

// Compiles the program; returns false when it was only compiled (no GPU run).
static bool build(Runner &run, Composable program) {
    if (compileOnly()) {
        codegen::CodeGenerator cg;
        last_source = cg.generate_code(program);
        const std::string name = cg.getLaunchPlan().name_expression;
        const std::string i1 = "-I" + libraryDir(), i2 = "-I" + packageDir();
        const char *names[1] = {name.c_str()};
        const char *opts[2] = {i1.c_str(), i2.c_str()};
        size_t size = 0;
        if (std::getenv("GERN_TEST_PRINT_SOURCE") != nullptr) {
            const auto plan = cg.getLaunchPlan();
            std::cerr << last_source << "\n// launch: " << name << "  grid (" << plan.grid[0] << ", " << plan.grid[1] << ", " << plan.grid[2]
                      << ")  block (" << plan.block[0] << ", " << plan.block[1] << ", " << plan.block[2] << ")\n";
        }
        if (gern_hip_compile_only(last_source.c_str(), names, 1, opts, 2, "gfx950", &size) != 0) {
            impl::hipCheck(1);
        }
        REQUIRE(size > 0);
        return false;
    }
    Runner::Options o;
    o.filename = "";
    o.include = " -I " + libraryDir() + " -I " + packageDir();
    run.compile(o);
    last_source = run.getSource();
    return true;
}

static AbstractDataTypePtr arrayDS(const std::string &name) {
    return AbstractDataTypePtr(new const annot::ArrayGPU(name));
}

static void expect_offset(impl::ArrayGPU &a, impl::ArrayGPU &b, float off, int64_t n) {
    std::vector<float> in = a.get(), out = b.get();
    for (int64_t i = 0; i < n; i++) {
        REQUIRE_EQ(out[i], in[i] + off);
    }
}

// ---- test-gpu-array.cu ------------------------------------------------------------

CASE("array.unmapped_runs_on_one_thread") {  // test-gpu-array.cu:16-76
    auto in = arrayDS("input_con"), out = arrayDS("output_con");
    annot::Add1GPU add_1;
    Variable step("step");
    Composable program = Global(Tile(out["size"], step)(add_1(in, out)));
    Runner run(program);
    if (!build(run, program)) {
        return;
    }
    impl::ArrayGPU a(10), b(10);
    a.ascending();
    int64_t step_val = 10;
    REQUIRE_NOTHROW(run.evaluate({{in.getName(), &a}, {out.getName(), &b}, {step.getName(), &step_val}}));
    expect_offset(a, b, 1, 10);
    REQUIRE_THROWS_AS(run.evaluate({{in.getName(), &a}, {out.getName(), &b}}), error::UserError);
    auto dummy = arrayDS("dummy_ds");
    REQUIRE_THROWS_AS(run.evaluate({{in.getName(), &a}, {dummy.getName(), &b}}), error::UserError);
    a.destroy();
    b.destroy();
}

CASE("array.tile_mapped_to_blocks") {  // test-gpu-array.cu:78-120
    auto in = arrayDS("input_con"), out = arrayDS("output_con");
    annot::Add1GPU add_1;
    Variable step("step");
    Composable program = Global((Tile(out["size"], step) || Grid::Unit::BLOCK_X)(add_1(in, out)));
    Runner run(program);
    if (!build(run, program)) {
        return;
    }
    impl::ArrayGPU a(10), b(10);
    a.ascending();
    int64_t step_val = 1;
    REQUIRE_NOTHROW(run.evaluate({{in.getName(), &a}, {out.getName(), &b}, {step.getName(), &step_val}}));
    expect_offset(a, b, 1, 10);
    a.destroy();
    b.destroy();
}

CASE("array.tiles_mapped_to_blocks_and_threads") {  // test-gpu-array.cu:122-168
    auto in = arrayDS("input_con"), out = arrayDS("output_con");
    annot::Add1GPU add_1;
    Variable step("step"), blk("blk");
    Composable program =
        Global((Tile(out["size"], blk) || Grid::Unit::BLOCK_X)((Tile(out["size"], step) || Grid::Unit::THREAD_X)(add_1(in, out))));
    Runner run(program);
    if (!build(run, program)) {
        return;
    }
    impl::ArrayGPU a(10), b(10);
    a.ascending();
    int64_t step_val = 1, blk_val = 1;
    REQUIRE_NOTHROW(run.evaluate({{in.getName(), &a}, {out.getName(), &b}, {step.getName(), &step_val}, {blk.getName(), &blk_val}}));
    expect_offset(a, b, 1, 10);
    // a block of 5 elements, one thread each
    blk_val = 5;
    REQUIRE_NOTHROW(run.evaluate({{in.getName(), &a}, {out.getName(), &b}, {step.getName(), &step_val}, {blk.getName(), &blk_val}}));
    expect_offset(a, b, 1, 10);
    a.destroy();
    b.destroy();
}

CASE("array.register_arrays_fused") {  // test-gpu-array.cu:170-210
    auto in = AbstractDataTypePtr(new const annot::ArrayStaticGPU("input_con"));
    auto temp = AbstractDataTypePtr(new const annot::ArrayStaticGPU("temp", true));
    auto out = AbstractDataTypePtr(new const annot::ArrayStaticGPU("output_con"));
    annot::Add1GPUTemplate add_1;
    Variable step("step"), blk("blk");
    Composable program = Global((Tile(out["size"], blk) || Grid::Unit::BLOCK_X)(
        (Tile(out["size"], step.bind(1)) || Grid::Unit::THREAD_X)(add_1(in, temp), add_1(temp, out))));
    Runner run(program);
    if (!build(run, program)) {
        return;
    }
    impl::ArrayGPU a(10), b(10);
    a.ascending();
    int64_t blk_val = 5;
    REQUIRE_NOTHROW(run.evaluate({{in.getName(), &a}, {out.getName(), &b}, {blk.getName(), &blk_val}}));
    expect_offset(a, b, 2, 10);
    a.destroy();
    b.destroy();
}

CASE("array.repeated_units") {  // test-gpu-array.cu:212-254
    auto in = AbstractDataTypePtr(new const annot::ArrayStaticGPU("input_con"));
    auto temp = AbstractDataTypePtr(new const annot::ArrayStaticGPU("temp", true));
    auto out = AbstractDataTypePtr(new const annot::ArrayStaticGPU("output_con"));
    annot::Add1GPUTemplate add_1;
    Variable step("step"), step2("step2"), step3("step3"), blk("blk");
    Composable program = Global((Tile(out["size"], blk.bind(8)) || Grid::Unit::BLOCK_X)(
        (Tile(out["size"], step.bind(4)) || Grid::Unit::BLOCK_X)((Tile(out["size"], step2.bind(2)) || Grid::Unit::THREAD_X)(
            (Tile(out["size"], step3.bind(1)) || Grid::Unit::THREAD_Y)(
                (Tile(out["size"], step3.bind(1)) || Grid::Unit::THREAD_X)(add_1(in, temp), add_1(temp, out)))))));
    Runner run(program);
    if (!build(run, program)) {
        return;
    }
    impl::ArrayGPU a(16), b(16);
    a.ascending();
    REQUIRE_NOTHROW(run.evaluate({{in.getName(), &a}, {out.getName(), &b}}));
    expect_offset(a, b, 2, 16);
    a.destroy();
    b.destroy();
}

CASE("array.reduction_hoisted_out_of_mapped_loops") {  // test-gpu-array.cu:256-297
    auto in = arrayDS("input_con"), out = arrayDS("output_con");
    annot::reductionGPU reduce;
    Variable step("step"), blk("blk"), k("k"), k2("k2");
    Composable program = Global(Tile(out["size"], k2.bind(10))(Reduce(k, step.bind(5))(
        (Tile(out["size"], step.bind(5)) || Grid::Unit::BLOCK_X)(
            (Tile(out["size"], blk.bind(1)) || Grid::Unit::THREAD_X)(Reduce(k, blk.bind(1))(reduce(in, out, k)))))));
    Runner run(program);
    if (!build(run, program)) {
        return;
    }
    impl::ArrayGPU a(10), b(10);
    a.ascending();
    int64_t k_val = 10;
    REQUIRE_NOTHROW(run.evaluate({{in.getName(), &a}, {out.getName(), &b}, {k.getName(), &k_val}}));
    std::vector<float> r = b.get();
    for (int i = 0; i < 10; i++) {
        REQUIRE_EQ(r[i], 45.0f);
    }
    a.destroy();
    b.destroy();
}

CASE("array.tile_mapped_to_wavefronts") {
    // Specific to this backend: a WARP unit is a 64-lane wavefront, so the
    // index expression divides threadIdx.x by 64 and the block grows by 64
    // threads per tile.  All 64 lanes of a wavefront compute the same tile.
    auto in = arrayDS("input_con"), out = arrayDS("output_con");
    annot::Add1GPU add_1;
    Variable step("step"), blk("blk");
    Composable program =
        Global((Tile(out["size"], blk) || Grid::Unit::BLOCK_X)((Tile(out["size"], step) || Grid::Unit::WARP_X)(add_1(in, out))));
    Runner run(program);
    const bool ran = build(run, program);
    REQUIRE(last_source.find("/ 64") != std::string::npos);
    REQUIRE(last_source.find("/ 32") == std::string::npos);
    if (!ran) {
        return;
    }
    impl::ArrayGPU a(12), b(12);
    a.ascending();
    int64_t step_val = 2, blk_val = 6;  // 2 blocks x 3 wavefronts
    REQUIRE_NOTHROW(run.evaluate({{in.getName(), &a}, {out.getName(), &b}, {step.getName(), &step_val}, {blk.getName(), &blk_val}}));
    expect_offset(a, b, 1, 12);
    a.destroy();
    b.destroy();
}

CASE("array.tile_mapped_to_lanes_inside_wavefronts") {
    // WARP_X over THREAD_X_IN_WRAPS: the outer tile picks the wavefront
    // (threadIdx.x / 64), the inner one the lane inside it (threadIdx.x % 64),
    // and the block has 64 threads per wavefront however few lanes work.
    auto in = arrayDS("input_con"), out = arrayDS("output_con");
    annot::Add1GPU add_1;
    Variable per_wave("per_wave"), step("step");
    Composable program = Global(
        (Tile(out["size"], per_wave) || Grid::Unit::WARP_X)((Tile(out["size"], step) || Grid::Unit::THREAD_X_IN_WRAPS)(add_1(in, out))));
    Runner run(program);
    const bool ran = build(run, program);
    REQUIRE(last_source.find("(threadIdx.x / 64)") != std::string::npos);
    REQUIRE(last_source.find("(threadIdx.x % 64)") != std::string::npos);
    if (!ran) {
        return;
    }
    impl::ArrayGPU a(96), b(96);
    a.ascending();
    int64_t per_wave_val = 32, step_val = 2;  // 3 wavefronts x 16 working lanes x 2 elements
    REQUIRE_NOTHROW(run.evaluate({{in.getName(), &a}, {out.getName(), &b}, {per_wave.getName(), &per_wave_val}, {step.getName(), &step_val}}));
    expect_offset(a, b, 1, 96);
    a.destroy();
    b.destroy();
}

// ---- test-set-grid.cu -----------------------------------------------------------------

CASE("set_grid.only_dimensions_in_scope") {  // test-set-grid.cu:15-44
    auto in = arrayDS("input_con"), out = arrayDS("output_con");
    annot::AddArrayThreads add_1;
    Variable step("step");
    REQUIRE_NOTHROW(Global(Tile(out["size"], step)(add_1(in, out))));
    REQUIRE_NOTHROW(Global(Tile(out["size"], step)(add_1(in, out)), {{Grid::Dim::BLOCK_DIM_X, step}}));
    REQUIRE_THROWS_AS(Global(Tile(out["size"], step)(add_1(in, out)), {{Grid::Dim::BLOCK_DIM_Y, step}}), error::UserError);
}

static void set_grid_run(bool separate_variable) {  // test-set-grid.cu:46-136
    auto in = arrayDS("input_con"), out = arrayDS("output_con");
    annot::AddArrayThreads add_1;
    Variable step("step"), num_threads("num_threads");
    Composable program =
        Global(Tile(out["size"], step)(add_1(in, out)), {{Grid::Dim::BLOCK_DIM_X, separate_variable ? num_threads : step}});
    Runner run(program);
    if (!build(run, program)) {
        return;
    }
    impl::ArrayGPU a(10), b(10);
    a.ascending();
    int64_t step_val = 5, threads_val = 5;
    std::map<std::string, void *> args = {{in.getName(), &a}, {out.getName(), &b}, {step.getName(), &step_val}};
    if (separate_variable) {
        args[num_threads.getName()] = &threads_val;
    }
    REQUIRE_NOTHROW(run.evaluate(args));
    expect_offset(a, b, 1, 10);
    if (separate_variable) {
        // the function assumes blockDim.x >= step: the launch is refused on the host
        threads_val = 2;
        REQUIRE_THROWS_AS(run.evaluate(args), error::UserError);
    }
    a.destroy();
    b.destroy();
}

CASE("set_grid.block_size_from_tile_variable") {
    set_grid_run(false);
}

CASE("set_grid.block_size_from_own_variable_and_assumption") {
    set_grid_run(true);
}

// A kernel is compiled to rely on its launch assumptions, so one that the host cannot check
// (the data structure does not say how to read the member it names) refuses the launch.
namespace {
class ArrayWithoutHostMembers : public annot::ArrayGPU {
public:
    using annot::ArrayGPU::ArrayGPU;
    bool readMember(const void *, const std::string &, int64_t &) const override {
        return false;
    }
};
struct AddAssumingSize : annot::Add1GPU {
    Annotation getAnnotation() override {
        return resetUnit(annot::Add1GPU::getAnnotation(), {Grid::Unit::SCALAR_UNIT}).assumes(Constraint(output["size"] >= step));
    }
};
}  // namespace

CASE("set_grid.assumption_the_host_cannot_check_refuses_the_launch") {
    for (bool readable : {true, false}) {
        auto in = readable ? arrayDS("input_con") : AbstractDataTypePtr(new const ArrayWithoutHostMembers("input_con"));
        auto out = readable ? arrayDS("output_con") : AbstractDataTypePtr(new const ArrayWithoutHostMembers("output_con"));
        AddAssumingSize add_1;
        Variable step("step");
        Composable program = Global(Tile(out["size"], step)(add_1(in, out)));
        Runner run(program);
        if (!build(run, program)) {
            return;
        }
        REQUIRE(last_source.find("__builtin_assume") != std::string::npos);
        impl::ArrayGPU a(10), b(10);
        a.ascending();
        int64_t step_val = 5;
        std::map<std::string, void *> args = {{in.getName(), &a}, {out.getName(), &b}, {step.getName(), &step_val}};
        if (readable) {
            REQUIRE_NOTHROW(run.evaluate(args));
            expect_offset(a, b, 1, 10);
            step_val = 20;  // violated
            REQUIRE_THROWS_AS(run.evaluate(args), error::UserError);
        } else {
            REQUIRE_THROWS_AS(run.evaluate(args), error::UserError);
        }
        a.destroy();
        b.destroy();
    }
}

// ---- test-dynamic-shared.cu ----------------------------------------------------------------

using annot::LdsManager;

static void dynamic_lds_run(bool with_manager) {  // test-dynamic-shared.cu:15-105
    auto in = arrayDS("input_con"), out = arrayDS("output_con");
    annot::Add1GPU add_1;
    Variable step("step"), smem_size("smem_size");
    Composable program = with_manager ? Global(Tile(out["size"], step)(add_1(in, out)), {}, smem_size, LdsManager(smem_size)) :
                                        Global(Tile(out["size"], step)(add_1(in, out)), {}, smem_size);
    Runner run(program);
    if (!build(run, program)) {
        return;
    }
    impl::ArrayGPU a(10), b(10);
    a.ascending();
    int64_t step_val = 10, smem_val = 1024;
    REQUIRE_NOTHROW(run.evaluate({{in.getName(), &a}, {out.getName(), &b}, {step.getName(), &step_val}, {smem_size.getName(), &smem_val}}));
    expect_offset(a, b, 1, 10);
    // more LDS than a gfx950 workgroup can have (160 KB) is refused on the host
    smem_val = 200 * 1024;
    REQUIRE_THROWS_AS(run.evaluate({{in.getName(), &a}, {out.getName(), &b}, {step.getName(), &step_val}, {smem_size.getName(), &smem_val}}),
                      error::UserError);
    a.destroy();
    b.destroy();
}

CASE("dynamic_lds.size_only") {
    dynamic_lds_run(false);
}

CASE("dynamic_lds.with_allocator_init") {
    dynamic_lds_run(true);
}

CASE("dynamic_lds.tiles_staged_into_lds") {  // test-dynamic-shared.cu:107-175
    auto in = AbstractDataTypePtr(new const annot::MatrixGPUStageSmem("input_con"));
    auto out = AbstractDataTypePtr(new const annot::MatrixGPUStageSmem("output_con"));
    annot::MatrixAddGPUBlocks add_blocks;
    Variable l_x("l_x"), l_y("l_y"), smem_size("smem_size"), thread_x("thread_x"), thread_y("thread_y");
    Composable program =
        Global((Tile(out["row"], l_x) || Grid::Unit::BLOCK_X)((Tile(out["col"], l_y) || Grid::Unit::BLOCK_Y)(add_blocks(in, out))),
               {{Grid::Dim::BLOCK_DIM_X, thread_x}, {Grid::Dim::BLOCK_DIM_Y, thread_y}}, smem_size, LdsManager(smem_size));
    Runner run(program);
    if (!build(run, program)) {
        return;
    }
    const int64_t rows = 4, cols = 8;
    impl::MatrixGPU a(rows, cols, cols), b(rows, cols, cols);
    a.ascending();
    int64_t lx = 4, ly = 2, tx = 1, ty = 2, smem = 1024;
    REQUIRE_NOTHROW(run.evaluate({{in.getName(), &a}, {out.getName(), &b}, {l_x.getName(), &lx}, {l_y.getName(), &ly},
                                  {smem_size.getName(), &smem}, {thread_x.getName(), &tx}, {thread_y.getName(), &ty}}));
    std::vector<float> r = b.get(), src = a.get();
    for (int64_t i = 0; i < rows * cols; i++) {
        REQUIRE_EQ(r[i], src[i] + 1.0f);
    }
    a.destroy();
    b.destroy();
}

// ---- test-gpu-matrix.cu ----------------------------------------------------------------------

static void matrix_add(int mapped) {  // test-gpu-matrix.cu:15-190
    auto in = AbstractDataTypePtr(new const annot::MatrixGPU("input_con"));
    auto out = AbstractDataTypePtr(new const annot::MatrixGPU("output_con"));
    annot::MatrixAddGPU add;
    Variable l_x("l_x"), l_y("l_y");
    Composable program;
    if (mapped == 0) {
        program = Global(Tile(out["row"], l_x)(Tile(out["col"], l_y)(add(in, out))));
    } else if (mapped == 1) {
        program = Global((Tile(out["row"], l_x) || Grid::Unit::BLOCK_X)(Tile(out["col"], l_y)(add(in, out))));
    } else {
        program = Global((Tile(out["row"], l_x) || Grid::Unit::BLOCK_X)((Tile(out["col"], l_y) || Grid::Unit::BLOCK_Y)(add(in, out))));
    }
    Runner run(program);
    if (!build(run, program)) {
        return;
    }
    impl::MatrixGPU a(10, 10, 10), b(10, 10, 10);
    a.fill(2.0f);
    int64_t lx = 5, ly = 5;
    REQUIRE_NOTHROW(run.evaluate({{in.getName(), &a}, {out.getName(), &b}, {l_x.getName(), &lx}, {l_y.getName(), &ly}}));
    for (float v : b.get()) {
        REQUIRE_EQ(v, 3.0f);
    }
    a.fill(7.0f);
    ly = 2;
    REQUIRE_NOTHROW(run.evaluate({{in.getName(), &a}, {out.getName(), &b}, {l_x.getName(), &lx}, {l_y.getName(), &ly}}));
    for (float v : b.get()) {
        REQUIRE_EQ(v, 8.0f);
    }
    a.destroy();
    b.destroy();
}

CASE("matrix.add_unmapped") {
    matrix_add(0);
}

CASE("matrix.add_rows_on_blocks") {
    matrix_add(1);
}

CASE("matrix.add_rows_and_columns_on_blocks") {
    matrix_add(2);
}

// Workgroup order in which an XCD takes blocks of 4 x 8 tiles (Runner::Options::xcd_tile_blocks): whatever the
// grid, every tile is visited exactly once; grids that are not whole blocks keep the plain order.
CASE("matrix.add_on_blocks_in_xcd_tile_block_order") {
    auto in = AbstractDataTypePtr(new const annot::MatrixGPU("input_con"));
    auto out = AbstractDataTypePtr(new const annot::MatrixGPU("output_con"));
    annot::MatrixAddGPU add;
    Variable l_x("l_x"), l_y("l_y");
    Composable program = Global((Tile(out["row"], l_x) || Grid::Unit::BLOCK_X)((Tile(out["col"], l_y) || Grid::Unit::BLOCK_Y)(add(in, out))));
    if (compileOnly()) {
        codegen::GeneratorOptions go;
        go.xcd_tile_blocks = true;
        codegen::CodeGenerator cg(std::nullopt, go);
        const std::string text = cg.generate_code(program);
        REQUIRE(text.find("gern_sb") != std::string::npos);
        return;
    }
    Runner run(program);
    Runner::Options o;
    o.filename = "";
    o.include = " -I " + libraryDir() + " -I " + packageDir();
    o.xcd_tile_blocks = true;
    run.compile(o);
    REQUIRE(run.getSource().find("gern_sb") != std::string::npos);
    const int64_t shapes[][2] = {{16, 16}, {32, 8}, {8, 32}, {64, 16}, {12, 8}, {4, 8}, {40, 24}};  // tiles along x, along y
    for (const auto &shape : shapes) {
        const int64_t rows = 2 * shape[0], cols = 3 * shape[1];
        impl::MatrixGPU a(rows, cols, cols), b(rows, cols, cols);
        a.fill(2.0f);
        b.fill(-5.0f);
        int64_t lx = 2, ly = 3;
        REQUIRE_NOTHROW(run.evaluate({{in.getName(), &a}, {out.getName(), &b}, {l_x.getName(), &lx}, {l_y.getName(), &ly}}));
        for (float v : b.get()) {
            REQUIRE_EQ(v, 3.0f);
        }
        a.destroy();
        b.destroy();
    }
}

// Bands of rows of tiles dealt to the XCDs in turn (Runner::Options::xcd_band_rows): every tile is visited
// exactly once, also when the grid is not a whole number of groups of eight bands.
CASE("matrix.add_on_blocks_in_xcd_band_order") {
    auto in = AbstractDataTypePtr(new const annot::MatrixGPU("input_con"));
    auto out = AbstractDataTypePtr(new const annot::MatrixGPU("output_con"));
    annot::MatrixAddGPU add;
    Variable l_x("l_x"), l_y("l_y");
    // columns on BLOCK_X, rows on BLOCK_Y: a row of tiles is gridDim.x tiles, as in the blur
    Composable program = Global((Tile(out["row"], l_x) || Grid::Unit::BLOCK_Y)((Tile(out["col"], l_y) || Grid::Unit::BLOCK_X)(add(in, out))));
    for (int band_rows : {1, 3, 16}) {
        if (compileOnly()) {
            codegen::GeneratorOptions go;
            go.xcd_band_rows = band_rows;
            codegen::CodeGenerator cg(std::nullopt, go);
            REQUIRE(cg.generate_code(program).find("gern_band") != std::string::npos);
            continue;
        }
        Runner run(program);
        Runner::Options o;
        o.filename = "";
        o.include = " -I " + libraryDir() + " -I " + packageDir();
        o.xcd_band_rows = band_rows;
        run.compile(o);
        REQUIRE(run.getSource().find("gern_band") != std::string::npos);
        const int64_t shapes[][2] = {{128, 5}, {24, 7}, {49, 3}, {8, 1}, {7, 2}, {300, 4}};  // rows of tiles, tiles per row
        for (const auto &shape : shapes) {
            const int64_t rows = 2 * shape[0], cols = 3 * shape[1];
            impl::MatrixGPU a(rows, cols, cols), b(rows, cols, cols);
            a.fill(2.0f);
            b.fill(-5.0f);
            int64_t lx = 2, ly = 3;
            REQUIRE_NOTHROW(run.evaluate({{in.getName(), &a}, {out.getName(), &b}, {l_x.getName(), &lx}, {l_y.getName(), &ly}}));
            for (float v : b.get()) {
                REQUIRE_EQ(v, 3.0f);
            }
            a.destroy();
            b.destroy();
        }
        run.release();
    }
}

// ---- user-written GEMM schedule staged through LDS -----------------------------------------------

CASE("schedule.gemm_staged_through_lds") {  // gernels/mm/kernel_3.cu:13-118 of the reference
    constexpr int64_t m = 128, n = 128, k = 128;
    using AType = annot::MatrixGlobalToShared<m, k>;
    using BType = annot::MatrixGlobalToShared<k, n>;
    using CType = annot::MatrixGlobalToGlobal<m, n>;
    auto A = AbstractDataTypePtr(new const AType("A", false));
    auto B = AbstractDataTypePtr(new const BType("B", false));
    auto C = AbstractDataTypePtr(new const CType("C", false));
    AType view_of("A_vec", false);
    Variable k_dim("k_dim"), k_tiled("k_tiled"), block_x("block_x"), block_y("block_y"), thread_x("thread_x"),
        thread_y("thread_y"), smem_size("smem_size"), one_val("one_val");
    block_x = block_x.bind(16);
    block_y = block_y.bind(8);
    thread_x = thread_x.bind(4);
    thread_y = thread_y.bind(4);
    k_dim = k_dim.bind(k);
    k_tiled = k_tiled.bind(8);
    one_val = one_val.bind(8);
    annot::MatrixMultiplyScalar mm(A, B, C);
    auto &mm_sp = mm[{{"k_dim", k_dim}}];
    Composable program = Global(
        (Tile(C["row"], block_x) || Grid::Unit::BLOCK_X)((Tile(C["col"], block_y) || Grid::Unit::BLOCK_Y)(Reduce(k_dim, k_tiled)(
            Stage(A, Stage(B, (Tile(C["row"], thread_x) || Grid::Unit::THREAD_Y)((Tile(C["col"], thread_y) || Grid::Unit::THREAD_X)(
                                  Reduce(k_dim, one_val)(Stage(A, view_of.getView(), Stage(B, view_of.getView(), mm_sp(A, B, C))))))))))),
        {}, smem_size, LdsManager(smem_size));
    Runner run(program);
    const bool ran = build(run, program);
    REQUIRE(last_source.find("stage_into_smem") != std::string::npos);
    REQUIRE(last_source.find("get_view") != std::string::npos);
    REQUIRE(last_source.find("free_smem") != std::string::npos);
    if (!ran) {
        return;
    }
    impl::MatrixGPU a(m, k, k), b(k, n, n), c(m, n, n);
    std::vector<float> ha(m * k), hb(k * n);
    for (int64_t e = 0; e < m * k; e++) {
        ha[e] = (float)(e % 10);  // the reference's ascending(): i % 10
    }
    for (int64_t e = 0; e < k * n; e++) {
        hb[e] = (float)((e * 7) % 10);
    }
    impl::hipCheck(gern_hip_memcpy_h2d(a.data, ha.data(), sizeof(float) * ha.size()));
    impl::hipCheck(gern_hip_memcpy_h2d(b.data, hb.data(), sizeof(float) * hb.size()));
    hip::GlobalMatrixF32 pa{a.data}, pb{b.data}, pc{c.data};
    int64_t smem = 16 * 1024;
    run.evaluate({{A.getName(), &pa}, {B.getName(), &pb}, {C.getName(), &pc}, {smem_size.getName(), &smem}});
    std::vector<float> got = c.get();
    for (int64_t i = 0; i < m; i++) {
        for (int64_t j = 0; j < n; j++) {
            float want = 0.0f;
            for (int64_t kk = 0; kk < k; kk++) {
                want += ha[i * k + kk] * hb[kk * n + j];
            }
            REQUIRE_EQ(got[i * n + j], want);  // small integers: exact in any order
        }
    }
    // a second launch accumulates again: nothing leaked from the LDS allocator
    run.evaluate({{A.getName(), &pa}, {B.getName(), &pb}, {C.getName(), &pc}, {smem_size.getName(), &smem}});
    got = c.get();
    float want00 = 0.0f;
    for (int64_t kk = 0; kk < k; kk++) {
        want00 += ha[kk] * hb[kk * n];
    }
    REQUIRE_EQ(got[0], 2 * want00);
    REQUIRE_EQ(run.ldsOverflows(), 0);
    // Too little dynamic LDS for both staged tiles (16 x 8 and 8 x 8 floats after the allocator's
    // 128-byte table): the kernel still ends, and the host can tell that its results are void.
    smem = 128 + 16 * 8 * 4 + 64;
    run.evaluate({{A.getName(), &pa}, {B.getName(), &pb}, {C.getName(), &pc}, {smem_size.getName(), &smem}});
    REQUIRE(run.ldsOverflows() > 0);
    a.destroy();
    b.destroy();
    c.destroy();
}

// Fills A with the reference's ascending() pattern (i % 10) and B with another small-integer
// pattern, runs C += A B through `run` and compares with the host product (exact in any order).
template<int64_t m, int64_t n, int64_t k>
static void check_schedule_product(Runner &run, const std::map<std::string, void *> &extra = {}) {
    impl::MatrixGPU a(m, k, k), b(k, n, n), c(m, n, n);
    std::vector<float> ha(m * k), hb(k * n);
    for (int64_t e = 0; e < m * k; e++) {
        ha[e] = (float)(e % 10);
    }
    for (int64_t e = 0; e < k * n; e++) {
        hb[e] = (float)((e * 7) % 10);
    }
    impl::hipCheck(gern_hip_memcpy_h2d(a.data, ha.data(), sizeof(float) * ha.size()));
    impl::hipCheck(gern_hip_memcpy_h2d(b.data, hb.data(), sizeof(float) * hb.size()));
    hip::GlobalMatrixF32 pa{a.data}, pb{b.data}, pc{c.data};
    std::map<std::string, void *> args{{"A", &pa}, {"B", &pb}, {"C", &pc}};
    args.insert(extra.begin(), extra.end());
    run.evaluate(args);
    std::vector<float> got = c.get();
    for (int64_t i = 0; i < m; i++) {
        for (int64_t j = 0; j < n; j++) {
            float want = 0.0f;
            for (int64_t kk = 0; kk < k; kk++) {
                want += ha[i * k + kk] * hb[kk * n + j];
            }
            REQUIRE_EQ(got[i * n + j], want);
        }
    }
    a.destroy();
    b.destroy();
    c.destroy();
}

CASE("schedule.gemm_staged_16_bytes_per_lane") {  // gernels/mm/kernel_6.cu:13-112 of the reference
    constexpr int64_t m = 128, n = 128, k = 128;
    using AType = annot::MatrixGlobalToSharedVec<m, k>;
    using BType = annot::MatrixGlobalToSharedVec<k, n>;
    using CType = annot::MatrixGlobalToGlobal<m, n>;
    auto A = AbstractDataTypePtr(new const AType("A", false));
    auto B = AbstractDataTypePtr(new const BType("B", false));
    auto C = AbstractDataTypePtr(new const CType("C", false));
    AType view_of("A_vec", false);
    Variable k_dim("k_dim"), k_tiled("k_tiled"), block_x("block_x"), block_y("block_y"), thread_x("thread_x"),
        thread_y("thread_y"), smem_size("smem_size");
    block_x = block_x.bind(8);
    block_y = block_y.bind(8);
    thread_x = thread_x.bind(4);
    thread_y = thread_y.bind(4);
    k_dim = k_dim.bind(k);
    k_tiled = k_tiled.bind(4);
    annot::MatrixMultiplyScalar mm(A, B, C);
    auto &mm_sp = mm[{{"k_dim", k_dim}}];
    Composable program = Global(
        (Tile(C["row"], block_x) || Grid::Unit::BLOCK_X)((Tile(C["col"], block_y) || Grid::Unit::BLOCK_Y)(Reduce(k_dim, k_tiled)(
            Stage(A, Stage(B, (Tile(C["row"], thread_x) || Grid::Unit::THREAD_Y)((Tile(C["col"], thread_y) || Grid::Unit::THREAD_X)(
                                  Stage(A, view_of.getViewVec(), Stage(B, view_of.getViewVec(), mm_sp(A, B, C)))))))))),
        {}, smem_size, LdsManager(smem_size));
    Runner run(program);
    const bool ran = build(run, program);
    REQUIRE(last_source.find("stage_into_smem_vec") != std::string::npos);
    REQUIRE(last_source.find("get_view_vec") != std::string::npos);
    if (!ran) {
        return;
    }
    int64_t smem = 32 * 32 * 8 * 2 + 1000;  // the reference's figure
    check_schedule_product<m, n, k>(run, {{smem_size.getName(), &smem}});
}

CASE("schedule.gemm_blocks_wavefronts_lanes") {  // gernels/mm/kernel_10.cu:13-172 of the reference
    // Block tile -> "warp" tile (WARP_Y x WARP_X) -> one output per lane
    // (THREAD_X_IN_WRAPS x THREAD_Y_IN_WRAPS), A and B staged into LDS by loads that
    // write it directly, a register copy of C, A and B per lane, and an inner
    // reduction over windows of those copies.  The reference's constants are for
    // 32-lane warps (a 32 x 32 patch of threads per "warp"); here a wavefront unit
    // is 64 wide, and 64 x 16 lanes make the 1024 threads of the workgroup.
    constexpr int64_t m = 128, n = 128, k = 128;
    using AType = annot::MatrixGlobalToSharedFlat<m, k>;
    using BType = annot::MatrixGlobalToSharedFlat<k, n>;
    // The lane's register copy of C must be written back.  A staged copy is written back only if
    // the data structure says its queries are copies (insertQuery(), src/codegen/finalizer.cpp:73-76
    // of the reference; its own MatrixGlobalToGlobal says "just a view", so kernel_10.cu as written
    // drops the copy, while the kernel generated from it earlier, gernels/mm/bench.cu:41, inserts it).
    struct CType : annot::MatrixGlobalToGlobal<m, n> {
        using annot::MatrixGlobalToGlobal<m, n>::MatrixGlobalToGlobal;
        bool insertQuery() const override {
            return true;
        }
    };
    using RegType = annot::MatrixQueryRegNoVector<m, n>;
    auto A = AbstractDataTypePtr(new const AType("A", false));
    auto B = AbstractDataTypePtr(new const BType("B", false));
    auto C = AbstractDataTypePtr(new const CType("C", false));
    AType view_of("A_vec", false);
    RegType in_registers("C_reg", false);
    Variable k_dim("k_dim"), k_tiled("k_tiled"), block_x("block_x"), block_y("block_y"), warp_x("warp_x"), warp_y("warp_y"),
        thread_x("thread_x"), thread_y("thread_y"), thread_k("thread_k"), smem_size("smem_size"), lanes_y("lanes_y");
    constexpr int64_t BM = 64, BN = 16, BK = 64, WM = 64, WN = 16, TM = 1, TN = 1, TK = 8;
    block_x = block_x.bind(BM);
    block_y = block_y.bind(BN);
    warp_x = warp_x.bind(WM);
    warp_y = warp_y.bind(WN);
    thread_x = thread_x.bind(TM);
    thread_y = thread_y.bind(TN);
    thread_k = thread_k.bind(TK);
    k_dim = k_dim.bind(k);
    k_tiled = k_tiled.bind(BK);
    annot::MatrixMultiplyScalar mm(A, B, C);
    auto &mm_sp = mm[{{"k_dim", k_dim}}];
    // innermost first
    Composable per_lane = Stage(
        C, in_registers.getQueryFunction(), in_registers.getInsertFunction(),
        Stage(A, in_registers.getQueryFunction(),
              Stage(B, in_registers.getQueryFunction(),
                    Reduce(k_dim, thread_k)(Stage(A, view_of.getView(), Stage(B, view_of.getView(), mm_sp(A, B, C)))))));
    Composable lanes = (Tile(C["row"], thread_x) || Grid::Unit::THREAD_X_IN_WRAPS)(
        (Tile(C["col"], thread_y) || Grid::Unit::THREAD_Y_IN_WRAPS)(per_lane));
    Composable wavefronts = (Tile(C["row"], warp_x) || Grid::Unit::WARP_Y)((Tile(C["col"], warp_y) || Grid::Unit::WARP_X)(lanes));
    Composable program = Global((Tile(C["row"], block_x) || Grid::Unit::BLOCK_X)((Tile(C["col"], block_y) || Grid::Unit::BLOCK_Y)(
                                    Reduce(k_dim, k_tiled)(Stage(A, Stage(B, wavefronts))))),
                                // a wavefront unit in y would claim 64 threads (64 x 64 in all); 16 lanes in y are what WN needs
                                {{Grid::Dim::BLOCK_DIM_Y, lanes_y.bind(WN / TN)}}, smem_size, LdsManager(smem_size));
    Runner run(program);
    const bool ran = build(run, program);
    REQUIRE(last_source.find("stage_into_smem_flat") != std::string::npos);
    REQUIRE(last_source.find("(threadIdx.y / 64)") != std::string::npos);
    REQUIRE(last_source.find("(threadIdx.x % 64)") != std::string::npos);
    REQUIRE(last_source.find("(threadIdx.y % 64)") != std::string::npos);
    if (!ran) {
        return;
    }
    int64_t smem = 48 * 1024;
    check_schedule_product<m, n, k>(run, {{smem_size.getName(), &smem}});
}

CASE("schedule.gemm_float4_register_tiles") {  // gernels/mm/mm_registers.cu:13-88 of the reference
    constexpr int64_t m = 8, n = 8, k = 8;
    using AType = annot::MatrixGPUVec<m, k>;
    using BType = annot::MatrixGPUVec<k, n>;
    using CType = annot::MatrixGPUVec<m, n>;
    auto A = AbstractDataTypePtr(new const AType("A", false));
    auto B = AbstractDataTypePtr(new const BType("B", false));
    auto C = AbstractDataTypePtr(new const CType("C", false));
    Variable k_dim("k_dim"), c_row("c_row"), c_col("c_col"), k_tile("k_tile");
    c_row = c_row.bind(4);
    c_col = c_col.bind(8);
    k_tile = k_tile.bind(4);
    k_dim = k_dim.bind(k);
    annot::MatrixMultiplyReg mm(A, B, C);
    auto &mm_sp = mm[{{"k_dim", k_dim}}];
    Composable program = Global((Tile(C["row"], c_row) || Grid::Unit::THREAD_X)(
        (Tile(C["col"], c_col) || Grid::Unit::THREAD_Y)(Reduce(k_dim, k_tile)(mm_sp(A, B, C)))));
    Runner run(program);
    const bool ran = build(run, program);
    REQUIRE(last_source.find("matrix_multiply_reg") != std::string::npos);
    if (!ran) {
        return;
    }
    check_schedule_product<m, n, k>(run);
}

// One output element per thread, operands and result windows of the matrices in global memory: the
// schedules of gernels/mm/kernel_1.cu:13-64 (rows on x) and kernel_2.cu:13-65 (columns on x, so that the
// lanes of a wavefront read consecutive elements of B and write consecutive elements of C).
static void element_per_thread_schedule(bool columns_on_x) {
    constexpr int64_t m = 64, n = 64, k = 64;
    using AType = annot::MatrixGlobalToGlobal<m, k>;
    using BType = annot::MatrixGlobalToGlobal<k, n>;
    using CType = annot::MatrixGlobalToGlobal<m, n>;
    auto A = AbstractDataTypePtr(new const AType("A", false));
    auto B = AbstractDataTypePtr(new const BType("B", false));
    auto C = AbstractDataTypePtr(new const CType("C", false));
    Variable k_dim("k_dim"), block_x("block_x"), block_y("block_y"), thread_x("thread_x"), thread_y("thread_y");
    block_x = block_x.bind(32);
    block_y = block_y.bind(32);
    thread_x = thread_x.bind(1);
    thread_y = thread_y.bind(1);
    k_dim = k_dim.bind(k);
    annot::MatrixMultiplyScalar mm(A, B, C);
    auto &mm_sp = mm[{{"k_dim", k_dim}}];
    const Grid::Unit rows_on_blocks = columns_on_x ? Grid::Unit::BLOCK_Y : Grid::Unit::BLOCK_X;
    const Grid::Unit cols_on_blocks = columns_on_x ? Grid::Unit::BLOCK_X : Grid::Unit::BLOCK_Y;
    const Grid::Unit rows_on_threads = columns_on_x ? Grid::Unit::THREAD_Y : Grid::Unit::THREAD_X;
    const Grid::Unit cols_on_threads = columns_on_x ? Grid::Unit::THREAD_X : Grid::Unit::THREAD_Y;
    Composable program = Global((Tile(C["row"], block_x) || rows_on_blocks)((Tile(C["col"], block_y) || cols_on_blocks)(
        (Tile(C["row"], thread_x) || rows_on_threads)((Tile(C["col"], thread_y) || cols_on_threads)(mm_sp(A, B, C))))));
    Runner run(program);
    const bool ran = build(run, program);
    REQUIRE(last_source.find("query_global_2_global<thread_x, thread_y>") != std::string::npos);
    REQUIRE(last_source.find("__launch_bounds__(1024)") != std::string::npos);  // 32 x 32 threads
    // which index of the thread walks the columns of C
    const std::string col_index = columns_on_x ? "threadIdx.x" : "threadIdx.y";
    REQUIRE(last_source.find("((" + col_index + " / 1) % (((thread_y + (block_y - 0)) - 1) / thread_y))") != std::string::npos);
    if (!ran) {
        return;
    }
    check_schedule_product<m, n, k>(run);
}

CASE("schedule.gemm_one_element_per_thread") {  // gernels/mm/kernel_1.cu:13-92 of the reference
    element_per_thread_schedule(false);
}

CASE("schedule.gemm_one_element_per_thread_columns_on_x") {  // gernels/mm/kernel_2.cu:13-93 of the reference
    element_per_thread_schedule(true);
}

CASE("schedule.gemm_whole_product_in_one_call") {  // gernels/mm/mm_trivial.cu:13-78 of the reference
    // No tiling at all: one thread multiplies the whole matrices where they lie.
    constexpr int64_t m = 8, n = 8, k = 8;
    using AType = annot::MatrixQueryRegNoVector<m, k>;
    using BType = annot::MatrixQueryRegNoVector<k, n>;
    using CType = annot::MatrixQueryRegNoVector<m, n>;
    auto A = AbstractDataTypePtr(new const AType("A", false));
    auto B = AbstractDataTypePtr(new const BType("B", false));
    auto C = AbstractDataTypePtr(new const CType("C", false));
    Variable k_dim("k_dim");
    annot::MatrixMultiplyScalar mm(A, B, C);
    auto &mm_sp = mm[{{"k_dim", k_dim.bind(k)}}];
    Composable program = Global(mm_sp(A, B, C));
    Runner run(program);
    const bool ran = build(run, program);
    REQUIRE(last_source.find("gernels::matrix_multiply<k_dim>") != std::string::npos);
    REQUIRE(last_source.find("__launch_bounds__(1)") != std::string::npos);
    if (!ran) {
        return;
    }
    check_schedule_product<m, n, k>(run);
}

CASE("schedule.gemm_register_tiles_rows_on_threads") {  // gernels/mm/mm_shared.cu:13-97 of the reference
    // 2 x 8 tiles of C on the threads of one workgroup, each a register copy that is multiplied into over
    // one K tile and written back (the reference's file is named for LDS and stages nothing into it).
    constexpr int64_t m = 8, n = 8, k = 8;
    using AType = annot::MatrixGPUVec<m, k>;
    using BType = annot::MatrixGPUVec<k, n>;
    using CType = annot::MatrixGPUVec<m, n>;
    auto A = AbstractDataTypePtr(new const AType("A", false));
    auto B = AbstractDataTypePtr(new const BType("B", false));
    auto C = AbstractDataTypePtr(new const CType("C", false));
    Variable k_dim("k_dim"), c_row("c_row"), c_col("c_col"), k_tile("k_tile");
    c_row = c_row.bind(2);
    c_col = c_col.bind(8);
    k_tile = k_tile.bind(8);
    k_dim = k_dim.bind(k);
    annot::MatrixMultiplyReg mm(A, B, C);
    auto &mm_sp = mm[{{"k_dim", k_dim}}];
    Composable program = Global((Tile(C["row"], c_row) || Grid::Unit::THREAD_X)(
        (Tile(C["col"], c_col) || Grid::Unit::THREAD_Y)(Reduce(k_dim, k_tile)(mm_sp(A, B, C)))));
    Runner run(program);
    const bool ran = build(run, program);
    REQUIRE(last_source.find("matrix_multiply_reg") != std::string::npos);
    REQUIRE(last_source.find("query<c_row, k_tile>") != std::string::npos);
    if (!ran) {
        return;
    }
    check_schedule_product<m, n, k>(run);
}

// ---- FunctionPtr on the device -----------------------------------------------------------------

static Runner::Options deviceFunctionOptions(const std::string &file) {
    Runner::Options o;
    const char *tmp = std::getenv("GERN_TEST_TMP");
    o.prefix = tmp ? tmp : "/tmp";
    o.filename = file;
    o.include = " -I " + libraryDir() + " -I " + packageDir();
    return o;
}

// Like build(), with the directory of the device-function files on the include path.
static bool buildWithPrefix(Runner &run, Composable program, const Runner::Options &inner) {
    if (compileOnly()) {
        codegen::CodeGenerator cg;
        last_source = cg.generate_code(program);
        const std::string name = cg.getLaunchPlan().name_expression;
        const std::string i1 = "-I" + libraryDir(), i2 = "-I" + packageDir(), i3 = "-I" + inner.prefix;
        const char *names[1] = {name.c_str()};
        const char *opts[3] = {i1.c_str(), i2.c_str(), i3.c_str()};
        size_t size = 0;
        if (gern_hip_compile_only(last_source.c_str(), names, 1, opts, 3, "gfx950", &size) != 0) {
            impl::hipCheck(1);
        }
        return false;
    }
    Runner::Options o = inner;
    o.filename = "";
    run.compile(o);
    last_source = run.getSource();
    return true;
}

CASE("schedule.blur_chain_on_halo_tiles_staged_into_lds") {
    // A three-stage blur (x, y, x; the chain of apps/blur/blur.cpp:31-73) as a schedule at the level of the API:
    // every workgroup stages its input tile INTO LDS WITH THE HALO that the composed annotations infer
    // (16 x 64 outputs need 18 x 68 inputs), every thread takes the 4 x 8 window of it that its own 2 x 4
    // outputs need, and the two intermediates are register tiles of the thread (4 x 6, then 2 x 6).
    constexpr int64_t rows = 128, cols = 128, in_rows = rows + 2, in_cols = cols + 4;
    using InType = annot::MatrixGlobalToShared<in_rows, in_cols>;
    using OutType = annot::MatrixGlobalToGlobal<rows, cols>;
    using TempType = annot::MatrixQueryRegNoVector<in_rows, in_cols>;
    auto input = AbstractDataTypePtr(new const InType("input", false));
    auto output = AbstractDataTypePtr(new const OutType("output", false));
    auto t1 = AbstractDataTypePtr(new const TempType("t1", true));
    auto t2 = AbstractDataTypePtr(new const TempType("t2", true));
    InType view_of("input_view", false);
    Variable stride("stride"), block_r("block_r"), block_c("block_c"), thread_r("thread_r"), thread_c("thread_c"), smem_size("smem_size");
    std::map<std::string, Variable> three{{"stride", stride.bind(3)}};
    annot::BlurXPerThread first{input, t1};
    annot::BlurYPerThread second{t1, t2};
    annot::BlurXPerThread third{t2, output};
    Composable chain(new const Computation({first[three](input, t1), second[three](t1, t2), third[three](t2, output)}));
    Composable program = Global(
        (Tile(output["row"], block_r.bind(16)) || Grid::Unit::BLOCK_Y)((Tile(output["col"], block_c.bind(64)) || Grid::Unit::BLOCK_X)(
            Stage(input, (Tile(output["row"], thread_r.bind(2)) || Grid::Unit::THREAD_Y)((Tile(output["col"], thread_c.bind(4)) || Grid::Unit::THREAD_X)(
                             Stage(input, view_of.getView(), chain)))))),
        {}, smem_size, LdsManager(smem_size));
    Runner run(program);
    const bool ran = build(run, program);
    // the staged tile and the thread's window carry the inferred halo: (rows + 2) x (cols + 4)
    REQUIRE(last_source.find("stage_into_smem<((block_r + stride) - 1), ((((block_c + stride) - 1) + stride) - 1)>") != std::string::npos);
    REQUIRE(last_source.find("get_view<((thread_r + stride) - 1), ((((thread_c + stride) - 1) + stride) - 1)>") != std::string::npos);
    REQUIRE(last_source.find("blur_y_per_thread") != std::string::npos);
    if (!ran) {
        return;
    }
    impl::MatrixGPU in(in_rows, in_cols, in_cols), out(rows, cols, cols);
    std::vector<float> h(in_rows * in_cols);
    for (int64_t e = 0; e < in_rows * in_cols; e++) {
        h[e] = (float)((e * 37 + (e / in_cols) * 11) % 97) * 0.25f - 7.0f;
    }
    impl::hipCheck(gern_hip_memcpy_h2d(in.data, h.data(), sizeof(float) * h.size()));
    hip::GlobalMatrixF32 pin{in.data}, pout{out.data};
    int64_t smem = 18 * 72 * 4 + 1024;
    run.evaluate({{"input", &pin}, {"output", &pout}, {smem_size.getName(), &smem}});
    REQUIRE_EQ(run.ldsOverflows(), (int64_t)0);
    // the stages one after the other on the host, same order of additions, same division
    std::vector<float> a(in_rows * (in_cols - 2)), b(rows * (in_cols - 2)), want(rows * cols);
    for (int64_t i = 0; i < in_rows; i++) {
        for (int64_t j = 0; j < in_cols - 2; j++) {
            float sum = 0.0f;
            for (int64_t t = 0; t < 3; t++) {
                sum += h[i * in_cols + j + t];
            }
            a[i * (in_cols - 2) + j] = sum / 3.0f;
        }
    }
    for (int64_t i = 0; i < rows; i++) {
        for (int64_t j = 0; j < in_cols - 2; j++) {
            float sum = 0.0f;
            for (int64_t t = 0; t < 3; t++) {
                sum += a[(i + t) * (in_cols - 2) + j];
            }
            b[i * (in_cols - 2) + j] = sum / 3.0f;
        }
    }
    for (int64_t i = 0; i < rows; i++) {
        for (int64_t j = 0; j < cols; j++) {
            float sum = 0.0f;
            for (int64_t t = 0; t < 3; t++) {
                sum += b[i * (in_cols - 2) + j + t];
            }
            want[i * cols + j] = sum / 3.0f;
        }
    }
    std::vector<float> got = out.get();
    for (int64_t e = 0; e < rows * cols; e++) {
        REQUIRE_EQ(got[e], want[e]);
    }
    in.destroy();
    out.destroy();
}

CASE("function_ptr.device_function_called_from_a_kernel") {
    // The host-side cases are test/test-function-ptr.cpp:13-86 of the
    // reference; here the wrapped program is made of device gernels, so it is
    // emitted as a __device__ function and called from the generated kernel.
    auto in = AbstractDataTypePtr(new const annot::ArrayStaticGPU("input_con"));
    auto temp = AbstractDataTypePtr(new const annot::ArrayStaticGPU("temp", true));
    auto out = AbstractDataTypePtr(new const annot::ArrayStaticGPU("output_con"));
    annot::Add1GPUTemplate add_1;
    Variable step("step"), blk("blk");
    Runner::Options inner = deviceFunctionOptions("gern_test_device_fn.h");
    FunctionPtr add_2(Tile(out["size"], step.bind(1))(add_1(in, temp), add_1(temp, out)), inner);
    REQUIRE(add_2.getFunction().device);
    // The kernel hands the function views of its arrays (plain ArrayGPU
    // queries); the function cuts its register arrays out of those.
    auto in_view = arrayDS("in_view"), out_view = arrayDS("out_view");
    // (the function's template parameter is bound again where it is called)
    auto &add_2_bound = add_2[{{"step", step.bind(1)}}];
    Composable program = Global((Tile(out_view["size"], blk) || Grid::Unit::BLOCK_X)(add_2_bound(in_view, out_view)));
    Runner run(program);
    const bool ran = buildWithPrefix(run, program, inner);
    REQUIRE(last_source.find("gern_test_device_fn.h") != std::string::npos);
    if (!ran) {
        return;
    }
    impl::ArrayGPU a(10), b(10);
    a.ascending();
    int64_t blk_val = 5;
    REQUIRE_NOTHROW(run.evaluate({{in_view.getName(), &a}, {out_view.getName(), &b}, {blk.getName(), &blk_val}}));
    expect_offset(a, b, 2, 10);
    a.destroy();
    b.destroy();
}

// ---- gernels/cccl: block reduction + device-wide atomic ------------------------------------

CASE("reduce.grid_reduce_total") {  // gernels/cccl/global_reduce.cu:11-66: sum of 0..9 is 45
    annot::GridReduce grid_reduce;
    auto input = AbstractDataTypePtr(new const annot::ArrayF32("input"));
    auto output = AbstractDataTypePtr(new const annot::FloatPtr("output"));
    Variable block_size{"block_size"}, input_size{"input_size"};
    const int k_val = 10, threads = 2;
    input_size = input_size.bind(k_val);
    auto &specialized = grid_reduce[{{"k", input_size}}];
    Variable per_block = block_size.bind(threads);
    Composable program = Global((Reduce(input_size, per_block) || Grid::Unit::BLOCK_X)(specialized(output, input)),
                                {{Grid::BLOCK_DIM_X, per_block}});
    Runner run(program);
    if (!build(run, program)) {
        return;
    }
    impl::ArrayGPU in(k_val), out(1);
    in.ascending();
    run.evaluate({{input.getName(), &in}, {output.getName(), &out.data}});
    REQUIRE_EQ(out.get()[0], (float)(k_val * (k_val - 1) / 2));
    in.destroy();
    out.destroy();
}

static void block_reduce_then_global_sum(int threads, int temp_size_val);

CASE("reduce.block_reduce_whole_wavefronts") {
    // The same program with 128 threads per block: the sum inside a block is a
    // wavefront butterfly plus one LDS hop (all partial sums are integers
    // below 2^24, so the result is exact in any order).
    block_reduce_then_global_sum(128, 4);
}

CASE("reduce.block_reduce_then_global_sum") {  // gernels/cccl/rdom_mimic.cu:11-70: sum of 0..7 is 28
    block_reduce_then_global_sum(2, 4);
}

static void block_reduce_then_global_sum(int threads, int temp_size_val) {
    auto input = AbstractDataTypePtr(new const annot::ArrayF32("input"));
    auto output = AbstractDataTypePtr(new const annot::FloatPtr("output"));
    auto temp = AbstractDataTypePtr(new const annot::ArrayF32("temp", true));
    Variable threads_var{"var_thrds_per_blk"}, t1{"t1"}, temp_size("temp_size");
    Variable bound_threads = threads_var.bind(threads);
    temp_size = temp_size.bind(temp_size_val);
    annot::GlobalSum global_sum;
    annot::BlockReduce block_reduce;
    auto &block_reduce_sp = block_reduce[{{"block_size", bound_threads}}];
    (void)global_sum[{{"k", temp_size}}];  // the reference builds this specialisation and calls the plain one
    Composable program = Global((Reduce(temp_size, t1.bind(1)) || Grid::Unit::BLOCK_X)(block_reduce_sp(temp, input),
                                                                                         global_sum(output, temp)),
                                {{Grid::BLOCK_DIM_X, bound_threads}});
    Runner run(program);
    if (!build(run, program)) {
        return;
    }
    const int n = temp_size_val * threads;
    impl::ArrayGPU in(n), out(1);
    in.ascending();
    run.evaluate({{input.getName(), &in}, {output.getName(), &out.data}});
    REQUIRE_EQ(out.get()[0], (float)(n * (n - 1) / 2));
    in.destroy();
    out.destroy();
}

CHECK_MAIN()
