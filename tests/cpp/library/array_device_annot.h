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

class ArrayGPU : public TableADT {
public:
    ArrayGPU(const std::string &name = "test")
        : TableADT(name, "gern::impl::ArrayGPU") {
        fields = {x, len};
        allocate_call = call("gern::impl::ArrayGPU::allocate", fields);
        query_call = call("query", fields);
        insert_call = call("insert", fields);
    }
    // The launch is sized on the host from the caller's object.
    bool readMember(const void *object, const std::string &member, int64_t &value) const override {
        if (member == "size") {
            value = static_cast<const ArrayGPULayout *>(object)->size;
        }
        return member == "size";
    }

protected:
    Variable x{"x"};
    Variable len{"len"};
};

// A device function that one thread runs alone (SCALAR_UNIT).
struct Add1GPU : PiecewiseArrayFunction {
    Add1GPU()
        : PiecewiseArrayFunction("gern::impl::add_1", "array_device.h", AbstractDataTypePtr(new const ArrayCPU("input")),
                                 AbstractDataTypePtr(new const ArrayCPU("output"))) {
    }

protected:
    std::set<Grid::Unit> occupied_units() const override {
        return {Grid::Unit::SCALAR_UNIT};
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
// and written back by insert; a temporary is typed `auto` and never freed.
class ArrayStaticGPU : public ArrayGPU {
public:
    ArrayStaticGPU(const std::string &name, bool temp = false)
        : ArrayGPU(name) {
        type_name = temp ? "auto" : "gern::impl::ArrayGPU";
        allocate_call = call("gern::impl::allocate_local", {}, {len});
        query_call = call("query", {x}, {len});
        insert_call = call("insert_array", {x}, {len});
        free_call = call("dummy");
        query_is_written_back = true;
        temporaries_are_freed = false;
    }
};

struct Add1GPUTemplate : Add1GPU {
protected:
    bool step_is_a_template_argument() const override {
        return true;
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
