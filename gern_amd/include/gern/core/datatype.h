// Scalar types of annotation variables and literals, and their C spelling in
// generated code.  Mirrors the public face of the reference's Datatype
// (include/gern/annotations/datatypes.h:16-67).
#pragma once

#include <complex>
#include <cstdint>
#include <ostream>
#include <string>

namespace gern {

class Datatype {
public:
    enum Kind {
        Bool,
        UInt8,
        UInt16,
        UInt32,
        UInt64,
        Int8,
        Int16,
        Int32,
        Int64,
        Float32,
        Float64,
        Complex64,
        Complex128,
        Undefined
    };

    Datatype()
        : kind(Undefined) {
    }
    Datatype(Kind k)
        : kind(k) {
    }

    Kind getKind() const {
        return kind;
    }
    bool isUInt() const {
        return kind >= UInt8 && kind <= UInt64;
    }
    bool isInt() const {
        return kind >= Int8 && kind <= Int64;
    }
    bool isFloat() const {
        return kind == Float32 || kind == Float64;
    }
    bool isComplex() const {
        return kind == Complex64 || kind == Complex128;
    }
    bool isBool() const {
        return kind == Bool;
    }
    int getNumBits() const;
    int getNumBytes() const {
        return (getNumBits() + 7) / 8;
    }
    // The type's spelling in generated C++ ("int64_t", "float", ...).
    std::string str() const;

private:
    Kind kind;
};

std::ostream &operator<<(std::ostream &, const Datatype &);
inline bool operator==(const Datatype &a, const Datatype &b) {
    return a.getKind() == b.getKind();
}
inline bool operator!=(const Datatype &a, const Datatype &b) {
    return !(a == b);
}

// Maps a C++ type to its Datatype (used by literal construction).
template<typename T>
inline Datatype type() {
    if constexpr (std::is_same_v<T, bool>) return Datatype::Bool;
    else if constexpr (std::is_same_v<T, float>) return Datatype::Float32;
    else if constexpr (std::is_same_v<T, double>) return Datatype::Float64;
    else if constexpr (std::is_same_v<T, std::complex<float>>) return Datatype::Complex64;
    else if constexpr (std::is_same_v<T, std::complex<double>>) return Datatype::Complex128;
    else if constexpr (std::is_integral_v<T> && std::is_unsigned_v<T>) {
        return sizeof(T) == 1 ? Datatype::UInt8 : sizeof(T) == 2 ? Datatype::UInt16 :
               sizeof(T) == 4 ? Datatype::UInt32 : Datatype::UInt64;
    } else if constexpr (std::is_integral_v<T>) {
        return sizeof(T) == 1 ? Datatype::Int8 : sizeof(T) == 2 ? Datatype::Int16 :
               sizeof(T) == 4 ? Datatype::Int32 : Datatype::Int64;
    } else {
        return Datatype::Undefined;
    }
}

}  // namespace gern
