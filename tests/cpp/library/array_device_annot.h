// Annotations of the device array library (array_device.h).
//
// Mirrors the reference's test annotations
// (test/library/array/annot/gpu-array.h:9-231).
#pragma once

#include "library/array_annot.h"

namespace gern {
namespace annot {

// Layout of the object handed to Runner::evaluate (and to the kernel).
struct ArrayGPULayout {
    float *data;
    int64_t size;
};

class ArrayGPU : public AbstractDataType {
public:
    ArrayGPU(const std::string &name = "test")
        : name(name) {
    }
    std::string getName() const override {
        return name;
    }
    std::string getType() const override {
        return "gern::impl::ArrayGPU";
    }
    std::vector<Variable> getFields() const override {
        return {x, len};
    }
    FunctionSignature getAllocateFunction() const override {
        return FunctionSignature{.name = "gern::impl::ArrayGPU::allocate", .args = {x, len}};
    }
    FunctionSignature getFreeFunction() const override {
        return FunctionSignature{.name = "destroy"};
    }
    FunctionSignature getInsertFunction() const override {
        return FunctionSignature{.name = "insert", .args = {x, len}};
    }
    FunctionSignature getQueryFunction() const override {
        return FunctionSignature{.name = "query", .args = {x, len}};
    }
    bool readMember(const void *object, const std::string &member, int64_t &value) const override {
        if (member != "size") {
            return false;
        }
        value = static_cast<const ArrayGPULayout *>(object)->size;
        return true;
    }

protected:
    std::string name;
    Variable x{"x"};
    Variable len{"len"};
};

// A scalar-unit device function.
class Add1GPU : public add_1 {
public:
    Annotation getAnnotation() override {
        Variable x("x");
        return Tileable(x = Expr(0), output["size"], step,
                        Produces::Subset(output, {x, step}),
                        Consumes::Subset(input, {x, step}))
            .occupies({Grid::Unit::SCALAR_UNIT});
    }
    std::vector<std::string> getHeader() override {
        return {"array_device.h"};
    }
};

class reductionGPU : public AbstractFunction {
public:
    reductionGPU()
        : input(new const ArrayGPU("input")), output(new const ArrayGPU("output")) {
    }
    Annotation getAnnotation() override {
        Variable x("x"), r("r"), step("step"), end("end");
        return Tileable(x = Expr(0), output["size"], step,
                        Produces::Subset(output, {x, step}),
                        Consumes::Subsets(Reducible(r = Expr(0), k, end, SubsetObj(input, {r, k}))))
            .occupies({Grid::Unit::SCALAR_UNIT});
    }
    std::vector<std::string> getHeader() override {
        return {"array_device.h"};
    }
    FunctionSignature getFunction() override {
        FunctionSignature f;
        f.name = "gern::impl::reduction";
        f.args = {Parameter(input), Parameter(output), Parameter(k)};
        return f;
    }

private:
    AbstractDataTypePtr input;
    AbstractDataTypePtr output;
    Variable k{"k"};
};

// Subsets are register arrays of a compile-time length, copied in by query
// and written back by insert.
class ArrayStaticGPU : public ArrayGPU {
public:
    ArrayStaticGPU(const std::string &name, bool temp = false)
        : ArrayGPU(name), temp(temp) {
    }
    std::string getType() const override {
        return temp ? "auto" : "gern::impl::ArrayGPU";
    }
    FunctionSignature getAllocateFunction() const override {
        return FunctionSignature{.name = "gern::impl::allocate_local", .template_args = {len}};
    }
    FunctionSignature getFreeFunction() const override {
        return FunctionSignature{.name = "dummy"};
    }
    FunctionSignature getInsertFunction() const override {
        return FunctionSignature{.name = "insert_array", .args = {x}, .template_args = {len}};
    }
    FunctionSignature getQueryFunction() const override {
        return FunctionSignature{.name = "query", .args = {x}, .template_args = {len}};
    }
    bool freeAlloc() const override {
        return false;
    }
    bool insertQuery() const override {
        return true;
    }

private:
    bool temp;
};

class Add1GPUTemplate : public Add1GPU {
public:
    FunctionSignature getFunction() override {
        FunctionSignature f;
        f.name = "gern::impl::add_1";
        f.args = {Parameter(input), Parameter(output)};
        f.template_args = {step};
        return f;
    }
};

// The same function claimed for the threads of a block, with a launch
// assumption on the block size.
class AddArrayThreads : public Add1GPU {
public:
    Annotation getAnnotation() override {
        return resetUnit(Add1GPU::getAnnotation(), {Grid::Unit::THREAD_X})
            .assumes(GridDim(Grid::Dim::BLOCK_DIM_X) >= step);
    }
};

}  // namespace annot
}  // namespace gern
