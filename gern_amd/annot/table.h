// A data structure described by data instead of one override per virtual: the
// type name, the fields of a subset, and the four calls (allocate, query,
// insert, free) that the code generator pastes, each with the fields it
// passes at run time and the fields it passes as template arguments.
#pragma once

#include "annotations/abstract_function.h"

#include <string>
#include <utility>
#include <vector>

namespace gern {
namespace annot {

class TableADT : public AbstractDataType {
public:
    TableADT(std::string name, std::string type)
        : AbstractDataType(std::move(name), ""), type_name(std::move(type)) {
    }
    std::string getType() const override {
        return type_name;
    }
    std::vector<Variable> getFields() const override {
        return fields;
    }
    FunctionSignature getAllocateFunction() const override {
        return allocate_call;
    }
    FunctionSignature getQueryFunction() const override {
        return query_call;
    }
    FunctionSignature getInsertFunction() const override {
        return insert_call;
    }
    FunctionSignature getFreeFunction() const override {
        return free_call;
    }
    bool insertQuery() const override {
        return query_is_written_back;
    }
    bool freeAlloc() const override {
        return temporaries_are_freed;
    }

protected:
    // name<constant...>(runtime...)
    static FunctionSignature call(const std::string &name, const std::vector<Variable> &runtime = {},
                                  const std::vector<Variable> &constant = {}) {
        FunctionSignature f;
        f.name = name;
        f.args = std::vector<Parameter>(runtime.begin(), runtime.end());
        f.template_args = constant;
        return f;
    }

    // Filled in by the constructor of the derived class (whose Variable
    // members exist only once the base is built).
    std::string type_name;
    std::vector<Variable> fields;
    FunctionSignature allocate_call, query_call, insert_call;
    FunctionSignature free_call = call("destroy");
    bool query_is_written_back = false;  // a queried subset is a copy: insert it after use
    bool temporaries_are_freed = true;   // an allocated temporary needs the free call
};

}  // namespace annot
}  // namespace gern
