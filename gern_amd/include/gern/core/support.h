// Small support pieces shared by the whole front end: reference-counted node
// handles, the two exception types, and the process-wide unique-name counter.
//
// Public names and behaviour follow the reference's utilities
// (include/gern/utils/uncopyable.h, utils/error.h:10-35,
// src/utils/name_generator.cpp:7-12); the implementation is this project's.
#pragma once

#include <atomic>
#include <exception>
#include <string>

namespace gern {

namespace util {

// Base for nodes handled through IntrusivePtr: carries the reference count.
template<typename T>
class Manageable {
public:
    Manageable() = default;
    Manageable(const Manageable &) {
    }
    Manageable &operator=(const Manageable &) {
        return *this;
    }
    virtual ~Manageable() = default;

private:
    template<typename U>
    friend class IntrusivePtr;
    mutable std::atomic<long> refs_{0};
};

class Uncopyable {
protected:
    Uncopyable() = default;
    ~Uncopyable() = default;

private:
    Uncopyable(const Uncopyable &) = delete;
    Uncopyable &operator=(const Uncopyable &) = delete;
};

// A shared handle whose count lives inside the pointee.  `ptr` is public, as
// user code compares and dereferences it directly.
template<typename T>
class IntrusivePtr {
public:
    T *ptr;

    IntrusivePtr()
        : ptr(nullptr) {
    }
    IntrusivePtr(T *p)
        : ptr(p) {
        retain();
    }
    IntrusivePtr(const IntrusivePtr &o)
        : ptr(o.ptr) {
        retain();
    }
    IntrusivePtr(IntrusivePtr &&o) noexcept
        : ptr(o.ptr) {
        o.ptr = nullptr;
    }
    IntrusivePtr &operator=(const IntrusivePtr &o) {
        if (o.ptr != ptr) {
            T *old = ptr;
            ptr = o.ptr;
            retain();
            drop(old);
        }
        return *this;
    }
    IntrusivePtr &operator=(IntrusivePtr &&o) noexcept {
        if (this != &o) {
            T *old = ptr;
            ptr = o.ptr;
            o.ptr = nullptr;
            drop(old);
        }
        return *this;
    }
    virtual ~IntrusivePtr() {
        drop(ptr);
        ptr = nullptr;
    }

    bool defined() const {
        return ptr != nullptr;
    }
    T *get() const {
        return ptr;
    }

private:
    void retain() {
        if (ptr != nullptr) {
            ptr->refs_.fetch_add(1, std::memory_order_relaxed);
        }
    }
    static void drop(T *p) {
        if (p != nullptr && p->refs_.fetch_sub(1, std::memory_order_acq_rel) == 1) {
            delete p;
        }
    }
};

}  // namespace util

namespace error {

class Error : public std::exception {
public:
    explicit Error(const std::string &msg)
        : message(msg) {
    }
    const char *what() const noexcept override {
        return message.c_str();
    }

protected:
    std::string message;
};

// The caller used the API wrongly (bad arguments, illegal composition,
// generated code that does not compile).
class UserError : public Error {
public:
    explicit UserError(const std::string &msg)
        : Error("User Error: " + msg) {
    }
};

// An invariant of the library itself was broken.
class InternalError : public Error {
public:
    explicit InternalError(const std::string &msg)
        : Error("Internal Error: " + msg) {
    }
};

}  // namespace error

// prefix + "_" + a process-wide counter (pre-incremented, starts at 1).
std::string getUniqueName(const std::string &prefix = "_gern_");

}  // namespace gern
