// Builds, with the REFERENCE library (compiled from /root/reference into
// oracle/_ref/), the CPU lowering of the composed pipelines of the hot path and
// leaves one shared object per pipeline in the output directory, plus a
// manifest naming each hook and its argument order.  Test infrastructure: the
// shared objects are the "reference" checker and CPU baseline.
//
// The annotation classes below are written against the reference's API.  The
// blur ones carry the dependency pattern of apps/common/annot/functions.h:175-249
// onto the CPU matrix type; the softmax ones follow :9-173 with the two
// changes the reference's own CPU annotations need to lower at all (a bound
// full-width variable for the row reductions, row-only tiling for the
// vector ops).
#include "annotations/abstract_function.h"
#include "compose/composable.h"
#include "compose/runner.h"
#include "config.h"
#include "library/array/annot/cpu-array.h"
#include "library/matrix/annot/cpu-matrix.h"

#include <cstdlib>
#include <fstream>
#include <iostream>

using namespace gern;

namespace refannot {

class BlurCPU : public AbstractFunction {
public:
    BlurCPU(AbstractDataTypePtr input, AbstractDataTypePtr output, bool along_x)
        : input(input), output(output), along_x(along_x) {
    }
    Annotation getAnnotation() override {
        Variable x("x"), y("y"), l_x("l_x"), l_y("l_y");
        std::vector<Expr> need = along_x ? std::vector<Expr>{x, y, l_x, l_y + stride - 1} :
                                           std::vector<Expr>{x, y, l_x + stride - 1, l_y};
        return annotate(Tileable(x = Expr(0), output["row"], l_x,
                                 Tileable(y = Expr(0), output["col"], l_y,
                                          Produces::Subset(output, {x, y, l_x, l_y}),
                                          Consumes::Subset(input, need))));
    }
    FunctionSignature getFunction() override {
        FunctionSignature f;
        f.name = along_x ? "gern::impl::blur_x" : "gern::impl::blur_y";
        f.args = {Parameter(input), Parameter(output)};
        f.template_args = {stride};
        return f;
    }
    std::vector<std::string> getHeader() override {
        return {"cpu-matrix.h", "ref_cpu_gernels.h"};
    }

private:
    AbstractDataTypePtr input, output;
    bool along_x;
    Variable stride{"stride", Datatype::Int64, true};
};

class RowReduceCPU : public AbstractFunction {
public:
    RowReduceCPU(AbstractDataTypePtr input, AbstractDataTypePtr output, std::string fn)
        : input(input), output(output), fn(fn) {
    }
    Annotation getAnnotation() override {
        Variable x("x"), l_x("l_x");
        return annotate(Tileable(x = Expr(0), output["size"], l_x,
                                 Produces::Subset(output, {x, l_x}),
                                 Consumes::Subset(input, {x, Expr(0), l_x, ncol})));
    }
    FunctionSignature getFunction() override {
        FunctionSignature f;
        f.name = fn;
        f.args = {Parameter(input), Parameter(output)};
        return f;
    }
    std::vector<std::string> getHeader() override {
        return {"cpu-matrix.h", "ref_cpu_gernels.h"};
    }

private:
    AbstractDataTypePtr input, output;
    std::string fn;
    Variable ncol{"ncol"};
};

class VecOpCPU : public AbstractFunction {
public:
    VecOpCPU(AbstractDataTypePtr vec, AbstractDataTypePtr input, AbstractDataTypePtr output, std::string fn)
        : vec(vec), input(input), output(output), fn(fn) {
    }
    Annotation getAnnotation() override {
        Variable x("x"), l_x("l_x");
        return annotate(Tileable(x = Expr(0), output["row"], l_x,
                                 Produces::Subset(output, {x, zero, l_x, ncol}),
                                 Consumes::Subsets(SubsetObjMany({
                                     SubsetObj(input, {x, Expr(0), l_x, ncol}),
                                     SubsetObj(vec, {x, l_x}),
                                 }))));
    }
    FunctionSignature getFunction() override {
        FunctionSignature f;
        f.name = fn;
        f.args = {Parameter(vec), Parameter(input), Parameter(output)};
        return f;
    }
    std::vector<std::string> getHeader() override {
        return {"cpu-matrix.h", "ref_cpu_gernels.h"};
    }

private:
    AbstractDataTypePtr vec, input, output;
    std::string fn;
    Variable ncol{"ncol"};
    Variable zero{"zero"};
};

class ExpCPU : public AbstractFunction {
public:
    ExpCPU(AbstractDataTypePtr input, AbstractDataTypePtr output)
        : input(input), output(output) {
    }
    Annotation getAnnotation() override {
        Variable x("x"), l_x("l_x");
        return annotate(Tileable(x = Expr(0), output["row"], l_x,
                                 Produces::Subset(output, {x, zero, l_x, ncol}),
                                 Consumes::Subset(input, {x, Expr(0), l_x, ncol})));
    }
    FunctionSignature getFunction() override {
        FunctionSignature f;
        f.name = "gern::impl::exp_matrix";
        f.args = {Parameter(input), Parameter(output)};
        return f;
    }
    std::vector<std::string> getHeader() override {
        return {"cpu-matrix.h", "ref_cpu_gernels.h"};
    }

private:
    AbstractDataTypePtr input, output;
    Variable ncol{"ncol"};
    Variable zero{"zero"};
};

}  // namespace refannot

static std::string g_out;
static std::ofstream g_manifest;

// Lowers `program` with the reference's Runner, then rebuilds the emitted
// source under a stable name (the Runner's own .so name is not exposed).
static void emit(const std::string &name, Composable program) {
    Runner run(program);
    Runner::Options o;
    o.filename = "ref_" + name + ".cpp";
    o.prefix = g_out;
    o.include = " -O2 -I " + std::string(GERN_ROOT_DIR) + "/test/ -I " + std::string(GERN_ROOT_DIR) +
                "/test/library/matrix/impl -I " + std::string(GERN_ROOT_DIR) + "/test/library/array/impl -I " +
                std::string(ORACLE_DIR);
    run.compile(o);
    FunctionSignature sig = run.getSignature();
    const std::string so = g_out + "/libref_" + name + ".so";
    const std::string cmd = "g++ -std=c++11 -fPIC " + o.include + " --shared -o " + so + " " + g_out + "/" + o.filename;
    if (std::system(cmd.c_str()) != 0) {
        std::cerr << "rebuild failed: " << cmd << std::endl;
        std::exit(1);
    }
    g_manifest << name << " hook_" << sig.name;
    for (const auto &a : sig.args) {
        g_manifest << " " << (isa<DSArg>(a) ? to<DSArg>(a)->getADTPtr().getName() : to<ExprArg>(a)->getVar().getName());
    }
    g_manifest << "\n";
}

static Composable blurChain(const std::string &pattern) {
    auto input = AbstractDataTypePtr(new const annot::MatrixCPU("input"));
    auto output = AbstractDataTypePtr(new const annot::MatrixCPU("output"));
    Variable stride("stride"), tr("tile_rows"), tc("tile_cols");
    std::vector<Composable> stages;
    AbstractDataTypePtr prev = input;
    for (size_t s = 0; s < pattern.size(); s++) {
        AbstractDataTypePtr next =
            (s + 1 == pattern.size()) ? output : AbstractDataTypePtr(new const annot::MatrixCPU("stage" + std::to_string(s)));
        refannot::BlurCPU f(prev, next, pattern[s] == 'x');
        stages.push_back(f[{{"stride", stride.bind(3)}}](prev, next));
        prev = next;
    }
    return Tile(output["row"], tr)(Tile(output["col"], tc)(Composable(stages)));
}

int main(int argc, char **argv) {
    if (argc < 2) {
        std::cerr << "usage: ref_driver <output dir>" << std::endl;
        return 2;
    }
    g_out = argv[1];
    g_manifest.open(g_out + "/manifest.txt");

    emit("blur_xy", blurChain("xy"));
    emit("blur_xyx", blurChain("xyx"));

    for (int64_t width : {int64_t(4096), int64_t(1000), int64_t(64)}) {
        auto input = AbstractDataTypePtr(new const annot::MatrixCPU("input"));
        auto output = AbstractDataTypePtr(new const annot::MatrixCPU("output"));
        auto shifted = AbstractDataTypePtr(new const annot::MatrixCPU("shifted"));
        auto expd = AbstractDataTypePtr(new const annot::MatrixCPU("expd"));
        auto row_max = AbstractDataTypePtr(new const annot::ArrayCPU("row_max"));
        auto row_sum = AbstractDataTypePtr(new const annot::ArrayCPU("row_sum"));
        Variable ncol("ncol"), tr("tile_rows"), zero("zero");
        refannot::RowReduceCPU max_row(input, row_max, "gern::impl::max_row");
        refannot::VecOpCPU sub(row_max, input, shifted, "gern::impl::subtract_vec_fixed");
        refannot::ExpCPU ex(shifted, expd);
        refannot::RowReduceCPU sum_row(expd, row_sum, "gern::impl::sum_row");
        refannot::VecOpCPU div(row_sum, expd, output, "gern::impl::divide_vec");
        std::map<std::string, Variable> b{{"ncol", ncol.bind(width)}, {"zero", zero.bind(0)}};
        emit("softmax_" + std::to_string(width), Tile(output["row"], tr)(max_row[b](input, row_max), sub[b](row_max, input, shifted),
                                                ex[b](shifted, expd), sum_row[b](expd, row_sum),
                                                div[b](row_sum, expd, output)));
    }
    {
        auto A = AbstractDataTypePtr(new const annot::MatrixCPU("A"));
        auto B = AbstractDataTypePtr(new const annot::MatrixCPU("B"));
        auto C = AbstractDataTypePtr(new const annot::MatrixCPU("C"));
        annot::MatrixMultiplyCPU mm;
        Variable ti("ti"), tj("tj"), tk("tk"), k_dim("k_dim");
        emit("gemm", Tile(C["row"], ti)(Tile(C["col"], tj)(Reduce(k_dim, tk)(mm(A, B, C, k_dim)))));
    }
    g_manifest.close();
    return 0;
}
