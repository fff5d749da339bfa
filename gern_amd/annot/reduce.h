// Annotations of the reduction gernels (gernels/reduce.h): a bare float* as
// the target of a device-wide sum, float arrays whose subsets are register
// arrays, and the three reduction functions.
//
// Mirrors the reference's gernels/cccl/gern_annot/adt.h:11-122 and
// gernels/cccl/gern_annot/functions.h:11-129.
#pragma once

#include "annot/table.h"

namespace gern {
namespace annot {

// A device pointer to one float: no fields, no subsets, nothing to allocate
// (all four calls are empty).
class FloatPtr : public TableADT {
public:
    explicit FloatPtr(const std::string &name)
        : TableADT(name, "float*") {
        free_call = FunctionSignature{};
    }
};

// Layout of the object handed to Runner::evaluate for an ArrayF32.
struct ArrayF32Layout {
    float *data;
    int64_t size;
};

// A float array in HBM whose subsets are per-thread register arrays of a
// compile-time length: query copies in, insert copies back, nothing is freed.
class ArrayF32 : public TableADT {
public:
    ArrayF32(const std::string &name, bool temp = false)
        : TableADT(name, temp ? "auto" : "gernels::ArrayF32") {
        fields = {x, len};
        allocate_call = call("gernels::allocate_local", {}, {len});
        query_call = call("template query", {x}, {len});
        insert_call = call("insert_array", {x}, {len});
        free_call = call("dummy");
        query_is_written_back = true;
        temporaries_are_freed = false;
    }
    bool readMember(const void *object, const std::string &member, int64_t &value) const override {
        if (member == "size") {
            value = static_cast<const ArrayF32Layout *>(object)->size;
        }
        return member == "size";
    }

private:
    Variable x{"x"};
    Variable len{"len"};
};

// What the three reduction gernels share: they are declared in
// gernels/reduce.h, take (output, input) in that order, and get their sizes as
// template arguments.
class ReductionGernel : public AbstractFunction {
public:
    FunctionSignature getFunction() override {
        FunctionSignature f;
        f.name = "gernels::" + gernel;
        f.args = {Parameter(output), Parameter(input)};
        f.template_args = sizes();
        return f;
    }
    std::vector<std::string> getHeader() override {
        return {"gernels/reduce.h"};
    }

protected:
    ReductionGernel(const std::string &gernel, const AbstractDataType *in, const AbstractDataType *out)
        : input(in), output(out), gernel(gernel) {
    }
    virtual std::vector<Variable> sizes() const = 0;
    // One call runs on all threads of a workgroup of exactly `block_size` threads.
    static Annotation onWholeBlock(Pattern p, Variable block_size) {
        return p.occupies({Grid::Unit::THREAD_X}).assumes({Grid::Dim::BLOCK_DIM_X == block_size});
    }
    AbstractDataTypePtr input, output;
    Variable k{"k", Datatype::Int64, true};
    Variable block_size{"block_size", Datatype::Int64, true};

private:
    std::string gernel;
};

// *output += sum(input[0 .. k)); every workgroup reduces block_size elements
// and adds its partial sum with one atomic.
struct GridReduce : ReductionGernel {
    GridReduce()
        : ReductionGernel("grid_reduce_total", new const ArrayF32("input"), new const FloatPtr("output")) {
    }
    Annotation getAnnotation() override {
        Variable i{"i"};
        return onWholeBlock(Computes(Produces::Subset(output, {}),
                                     Reducible(i = Expr(0), k, block_size, SubsetObj(input, {i, block_size}))),
                            block_size);
    }

protected:
    std::vector<Variable> sizes() const override {
        return {k, block_size};
    }
};

// output[i] = sum of block_size consecutive inputs, one per thread.
struct BlockReduce : ReductionGernel {
    BlockReduce()
        : ReductionGernel("block_reduce", new const ArrayF32("input"), new const ArrayF32("output")) {
    }
    Annotation getAnnotation() override {
        Variable i{"i"}, lx{"lx"};
        return onWholeBlock(Tileable(i = Expr(0), output["size"], lx, Produces::Subset(output, {i, lx}),
                                     Consumes::Subset(input, {i * block_size * lx, block_size * lx})),
                            block_size);
    }

protected:
    std::vector<Variable> sizes() const override {
        return {block_size};
    }
};

// *output += input[0] + ... + input[k - 1], sequentially.
struct GlobalSum : ReductionGernel {
    GlobalSum()
        : ReductionGernel("global_sum", new const ArrayF32("input"), new const FloatPtr("output")) {
    }
    Annotation getAnnotation() override {
        Variable i{"i"};
        Variable tk{"tk", Datatype::Int64, true};
        return annotate(Computes(Produces::Subset(output, {}), Reducible(i = Expr(0), k, tk, SubsetObj(input, {i, tk}))));
    }

protected:
    std::vector<Variable> sizes() const override {
        return {k};
    }
};

}  // namespace annot
}  // namespace gern
