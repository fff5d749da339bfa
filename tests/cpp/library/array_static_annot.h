// Annotations of array_static_host.h.
// Mirrors test/library/array/annot/cpu-array-template.h:11-114 of the reference.
#pragma once

#include "annot_table.h"

namespace gern {
namespace annot {

// Length is a compile-time constant: allocate / query / insert take it as a
// template argument, a query is a copy that is written back, and a temporary
// (typed `auto`: its length is only known where it is allocated) is not freed.
template<int Size>
class ArrayCPUTemplate : public TableADT {
public:
    ArrayCPUTemplate(const std::string &name = "test", bool temp = false)
        : TableADT(name, temp ? "auto" : "gern::impl::ArrayCPUTemplate<" + std::to_string(Size) + ">") {
        fields = {x, len};
        allocate_call = call("gern::impl::temp_allocate", {}, {len});
        query_call = call("query", {x}, {len});
        insert_call = call("insert", {x}, {len});
        query_is_written_back = true;
        temporaries_are_freed = false;
    }

protected:
    Variable x{"x"};
    Variable len{"len"};
};

struct addStaticStore : PiecewiseArrayFunction {
    addStaticStore()
        : PiecewiseArrayFunction("gern::impl::add", "array_static_host.h",
                                 AbstractDataTypePtr(new const ArrayCPUTemplate<10>("input")),
                                 AbstractDataTypePtr(new const ArrayCPUTemplate<10>("output"))) {
    }

protected:
    bool step_is_a_template_argument() const override {
        return true;
    }
};

}  // namespace annot
}  // namespace gern
