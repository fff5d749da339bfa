// Annotations of the reduction gernels (gernels/reduce.h): a bare float* as
// the target of a device-wide sum, float arrays whose subsets are register
// arrays, and the three reduction functions.
//
// Mirrors the reference's gernels/cccl/gern_annot/adt.h:11-122 and
// gernels/cccl/gern_annot/functions.h:11-129.
#pragma once

#include "annotations/abstract_function.h"

namespace gern {
namespace annot {

// A device pointer to one float: no fields, no query, nothing to allocate.
class FloatPtr : public AbstractDataType {
public:
    explicit FloatPtr(const std::string &name)
        : name(name) {
    }
    std::string getType() const override {
        return "float*";
    }
    std::string getName() const override {
        return name;
    }
    std::vector<Variable> getFields() const override {
        return {};
    }
    FunctionSignature getQueryFunction() const override {
        return FunctionSignature{};
    }
    FunctionSignature getInsertFunction() const override {
        return FunctionSignature{};
    }
    FunctionSignature getAllocateFunction() const override {
        return FunctionSignature{};
    }
    FunctionSignature getFreeFunction() const override {
        return FunctionSignature{};
    }

private:
    std::string name;
};

// Layout of the object handed to Runner::evaluate for an ArrayF32.
struct ArrayF32Layout {
    float *data;
    int64_t size;
};

class ArrayF32 : public AbstractDataType {
public:
    ArrayF32(const std::string &name, bool temp = false)
        : name(name), temp(temp) {
    }
    std::string getName() const override {
        return name;
    }
    std::string getType() const override {
        return temp ? "auto" : "gernels::ArrayF32";
    }
    std::vector<Variable> getFields() const override {
        return {x, len};
    }
    FunctionSignature getAllocateFunction() const override {
        return FunctionSignature{.name = "gernels::allocate_local", .template_args = {len}};
    }
    FunctionSignature getFreeFunction() const override {
        return FunctionSignature{.name = "dummy"};
    }
    FunctionSignature getInsertFunction() const override {
        return FunctionSignature{.name = "insert_array", .args = {x}, .template_args = {len}};
    }
    FunctionSignature getQueryFunction() const override {
        return FunctionSignature{.name = "template query", .args = {x}, .template_args = {len}};
    }
    bool freeAlloc() const override {
        return false;
    }
    bool insertQuery() const override {
        return true;
    }
    bool readMember(const void *object, const std::string &member, int64_t &value) const override {
        if (member != "size") {
            return false;
        }
        value = static_cast<const ArrayF32Layout *>(object)->size;
        return true;
    }

private:
    std::string name;
    bool temp;
    Variable x{"x"};
    Variable len{"len"};
};

// *output += sum(input[0 .. k)); every workgroup reduces block_size elements
// and adds its partial sum with one atomic.
class GridReduce : public AbstractFunction {
public:
    GridReduce()
        : input(new const ArrayF32("input")), output(new const FloatPtr("output")) {
    }
    FunctionSignature getFunction() override {
        return FunctionSignature{
            .name = "gernels::grid_reduce_total",
            .args = {Parameter(output), Parameter(input)},
            .template_args = {k, block_size},
        };
    }
    Annotation getAnnotation() override {
        Variable i{"i"};
        return Computes(Produces::Subset(output, {}),
                        Reducible(i = Expr(0), k, block_size, SubsetObj(input, {i, block_size})))
            .occupies({Grid::Unit::THREAD_X})
            .assumes({Grid::Dim::BLOCK_DIM_X == block_size});
    }
    std::vector<std::string> getHeader() override {
        return {"gernels/reduce.h"};
    }

private:
    Variable k{"k", Datatype::Int64, true};
    Variable block_size{"block_size", Datatype::Int64, true};
    AbstractDataTypePtr input;
    AbstractDataTypePtr output;
};

// output[i] = sum of block_size consecutive inputs, one per thread.
class BlockReduce : public AbstractFunction {
public:
    BlockReduce()
        : input(new const ArrayF32("input")), output(new const ArrayF32("output")) {
    }
    FunctionSignature getFunction() override {
        return FunctionSignature{
            .name = "gernels::block_reduce",
            .args = {Parameter(output), Parameter(input)},
            .template_args = {block_size},
        };
    }
    Annotation getAnnotation() override {
        Variable i{"i"};
        Variable lx{"lx"};
        return Tileable(i = Expr(0), output["size"], lx,
                        Produces::Subset(output, {i, lx}),
                        Consumes::Subset(input, {i * block_size * lx, block_size * lx}))
            .occupies({Grid::Unit::THREAD_X})
            .assumes({Grid::Dim::BLOCK_DIM_X == block_size});
    }
    std::vector<std::string> getHeader() override {
        return {"gernels/reduce.h"};
    }

private:
    Variable block_size{"block_size", Datatype::Int64, true};
    AbstractDataTypePtr input;
    AbstractDataTypePtr output;
};

// *output += input[0] + ... + input[k - 1]
class GlobalSum : public AbstractFunction {
public:
    GlobalSum()
        : input(new const ArrayF32("input")), output(new const FloatPtr("output")) {
    }
    FunctionSignature getFunction() override {
        return FunctionSignature{
            .name = "gernels::global_sum",
            .args = {Parameter(output), Parameter(input)},
            .template_args = {k},
        };
    }
    Annotation getAnnotation() override {
        Variable i{"i"};
        Variable tk{"tk", Datatype::Int64, true};
        return annotate(Computes(Produces::Subset(output, {}), Reducible(i = Expr(0), k, tk, SubsetObj(input, {i, tk}))));
    }
    std::vector<std::string> getHeader() override {
        return {"gernels/reduce.h"};
    }

private:
    Variable k{"k", Datatype::Int64, true};
    AbstractDataTypePtr input;
    AbstractDataTypePtr output;
};

}  // namespace annot
}  // namespace gern
