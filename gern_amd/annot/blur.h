// Annotations of the blur gernels (gernels/blur.h).  To produce an
// (l_x x l_y) tile at (x, y), blur_x consumes an l_x x (l_y + stride - 1)
// tile at the same origin and blur_y an (l_x + stride - 1) x l_y one: the
// halo the code generator propagates through a fused chain.
//
// Counterpart of the reference's apps/common/annot/functions.h:175-249.
#pragma once

#include "annot/matrix.h"

namespace gern {
namespace annot {

class BlurX : public AbstractFunction {
public:
    BlurX(AbstractDataTypePtr input, AbstractDataTypePtr output)
        : input(input), output(output) {
    }
    Annotation getAnnotation() override {
        Variable x("x");
        Variable y("y");
        Variable l_x("l_x", Datatype::Int64, true);
        Variable l_y("l_y", Datatype::Int64, true);
        return Tileable(x = Expr(0), ADTMember(output, "row", false), l_x,
                        Tileable(y = Expr(0), ADTMember(output, "col", false), l_y,
                                 Produces::Subset(output, {x, y, l_x, l_y}),
                                 Consumes::Subset(input, consumed(x, y, l_x, l_y))))
            // one wavefront cooperates on a tile
            .occupies({Grid::Unit::THREAD_X_IN_WRAPS});
    }
    FunctionSignature getFunction() override {
        FunctionSignature f;
        f.name = functionName();
        f.args = {Parameter(input), Parameter(output)};
        f.template_args = {stride};
        return f;
    }
    std::vector<std::string> getHeader() override {
        return {"gernels/blur.h"};
    }

protected:
    virtual std::vector<Expr> consumed(Variable x, Variable y, Variable l_x, Variable l_y) {
        return {x, y, l_x, l_y + stride - 1};
    }
    virtual std::string functionName() {
        return "gernels::blur_x";
    }
    AbstractDataTypePtr input;
    AbstractDataTypePtr output;
    Variable stride{"stride", Datatype::Int64, true};
};

class BlurY : public BlurX {
public:
    BlurY(AbstractDataTypePtr input, AbstractDataTypePtr output)
        : BlurX(input, output) {
    }

protected:
    std::vector<Expr> consumed(Variable x, Variable y, Variable l_x, Variable l_y) override {
        return {x, y, l_x + stride - 1, l_y};
    }
    std::string functionName() override {
        return "gernels::blur_y";
    }
};

// The same two functions for schedules in which ONE THREAD computes a tile (gernels/lds_blur.h): the
// dependency pattern is the same, the call occupies a single thread, and the data structures are those of
// annot/lds_matrix.h (a block's input tile staged into LDS with its halo, per-thread register tiles).
class BlurXPerThread : public BlurX {
public:
    using BlurX::BlurX;
    Annotation getAnnotation() override {
        Variable x("x");
        Variable y("y");
        Variable l_x("l_x", Datatype::Int64, true);
        Variable l_y("l_y", Datatype::Int64, true);
        return Tileable(x = Expr(0), ADTMember(output, "row", false), l_x,
                        Tileable(y = Expr(0), ADTMember(output, "col", false), l_y,
                                 Produces::Subset(output, {x, y, l_x, l_y}),
                                 Consumes::Subset(input, consumed(x, y, l_x, l_y))))
            .occupies({Grid::Unit::SCALAR_UNIT});
    }
    std::vector<std::string> getHeader() override {
        return {"gernels/lds_blur.h"};
    }

protected:
    std::string functionName() override {
        return "gernels::blur_x_per_thread";
    }
};

class BlurYPerThread : public BlurXPerThread {
public:
    using BlurXPerThread::BlurXPerThread;

protected:
    std::vector<Expr> consumed(Variable x, Variable y, Variable l_x, Variable l_y) override {
        return {x, y, l_x + stride - 1, l_y};
    }
    std::string functionName() override {
        return "gernels::blur_y_per_thread";
    }
};

}  // namespace annot
}  // namespace gern
