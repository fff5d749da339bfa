// Shared pieces of the test libraries' annotations: data structures are
// annot::TableADT tables (annot/table.h); the element-wise array functions
// share one annotation.
#pragma once

#include "annot/table.h"

#include <set>
#include <string>
#include <utility>
#include <vector>

namespace gern {
namespace annot {

// output[x .. x+step) is produced from input[x .. x+step): the annotation of
// every element-wise array function of the test libraries.
class PiecewiseArrayFunction : public AbstractFunction {
public:
    PiecewiseArrayFunction(std::string function, std::string header, AbstractDataTypePtr in, AbstractDataTypePtr out)
        : input(std::move(in)), output(std::move(out)), function(std::move(function)), header(std::move(header)) {
    }
    Annotation getAnnotation() override {
        Variable x("x");
        const auto pattern = Tileable(x = Expr(0), output["size"], step, Produces::Subset(output, {x, step}),
                                      Consumes::Subset(input, {x, step}));
        const std::set<Grid::Unit> units = occupied_units();
        return units.empty() ? annotate(pattern) : pattern.occupies(units);
    }
    FunctionSignature getFunction() override {
        FunctionSignature f;
        f.name = function;
        f.args = {Parameter(input), Parameter(output)};
        for (const auto &extra : trailing_arguments()) {
            f.args.push_back(Parameter(extra));
        }
        if (step_is_a_template_argument()) {
            f.template_args = {step};
        }
        return f;
    }
    std::vector<std::string> getHeader() override {
        return {header};
    }

protected:
    virtual std::vector<Variable> trailing_arguments() const {
        return {};
    }
    virtual bool step_is_a_template_argument() const {
        return false;
    }
    // Device functions say which grid units one call occupies.
    virtual std::set<Grid::Unit> occupied_units() const {
        return {};
    }
    AbstractDataTypePtr input, output;
    Variable step{"step"};

private:
    std::string function, header;
};

}  // namespace annot
}  // namespace gern
