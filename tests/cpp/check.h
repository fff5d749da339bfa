// A tiny registration-based test harness for the C++ front-end tests: each
// translation unit registers CASE(name) bodies; main() runs them all (or the
// ones named on the command line), prints one line per case and returns the
// number of failed cases.
#pragma once

#include <cstdio>
#include <exception>
#include <functional>
#include <sstream>
#include <stdexcept>
#include <string>
#include <vector>

namespace check {

struct Case {
    std::string name;
    std::function<void()> body;
};

inline std::vector<Case> &cases() {
    static std::vector<Case> all;
    return all;
}

struct Registrar {
    Registrar(const char *name, std::function<void()> body) {
        cases().push_back({name, std::move(body)});
    }
};

struct Failure : std::runtime_error {
    using std::runtime_error::runtime_error;
};

inline void fail(const char *file, int line, const std::string &what) {
    std::ostringstream os;
    os << file << ":" << line << ": " << what;
    throw Failure(os.str());
}

// The text of anything printable with whitespace removed.
template<typename T>
std::string stripped(const T &v) {
    std::ostringstream os;
    os << v;
    std::string s = os.str(), out;
    for (char c : s) {
        if (c != ' ' && c != '\n' && c != '\t') {
            out.push_back(c);
        }
    }
    return out;
}

inline int run_all(int argc, char **argv) {
    int failed = 0, ran = 0;
    for (const auto &c : cases()) {
        bool selected = argc <= 1;
        for (int i = 1; i < argc; i++) {
            selected = selected || c.name == argv[i];
        }
        if (!selected) {
            continue;
        }
        ran++;
        try {
            c.body();
            std::printf("[  ok  ] %s\n", c.name.c_str());
        } catch (const std::exception &e) {
            failed++;
            std::printf("[ FAIL ] %s: %s\n", c.name.c_str(), e.what());
        }
        std::fflush(stdout);
    }
    std::printf("%d cases, %d failed\n", ran, failed);
    return failed;
}

}  // namespace check

#define CHECK_CAT2(a, b) a##b
#define CHECK_CAT(a, b) CHECK_CAT2(a, b)
#define CASE(name)                                                            \
    static void CHECK_CAT(case_body_, __LINE__)();                            \
    static check::Registrar CHECK_CAT(case_reg_, __LINE__)(name, CHECK_CAT(case_body_, __LINE__)); \
    static void CHECK_CAT(case_body_, __LINE__)()

#define REQUIRE(cond)                                         \
    do {                                                      \
        if (!(cond)) {                                        \
            check::fail(__FILE__, __LINE__, "not true: " #cond); \
        }                                                     \
    } while (0)

#define REQUIRE_EQ(a, b)                                                          \
    do {                                                                          \
        auto check_a = (a);                                                       \
        auto check_b = (b);                                                       \
        if (!(check_a == check_b)) {                                              \
            std::ostringstream check_os;                                          \
            check_os << #a " == " #b " failed: " << check_a << " vs " << check_b; \
            check::fail(__FILE__, __LINE__, check_os.str());                      \
        }                                                                         \
    } while (0)

#define REQUIRE_THROWS_AS(stmt, Exc)                                      \
    do {                                                                  \
        bool check_thrown = false;                                        \
        try {                                                             \
            (void)(stmt);                                                 \
        } catch (const Exc &) {                                           \
            check_thrown = true;                                          \
        } catch (const std::exception &e) {                               \
            check::fail(__FILE__, __LINE__, std::string("wrong exception from " #stmt ": ") + e.what()); \
        }                                                                 \
        if (!check_thrown) {                                              \
            check::fail(__FILE__, __LINE__, "no " #Exc " from " #stmt);   \
        }                                                                 \
    } while (0)

#define REQUIRE_NOTHROW(stmt)                                             \
    do {                                                                  \
        try {                                                             \
            (void)(stmt);                                                 \
        } catch (const std::exception &e) {                               \
            check::fail(__FILE__, __LINE__, std::string("exception from " #stmt ": ") + e.what()); \
        }                                                                 \
    } while (0)

#define CHECK_MAIN()                    \
    int main(int argc, char **argv) {   \
        return check::run_all(argc, argv); \
    }
