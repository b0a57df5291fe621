// A small test harness that understands the subset of the doctest macro vocabulary which IOM's
// backend-agnostic conformance scenarios use (test/backend/backend_conformance_*.hpp include
// <doctest/doctest.h>, test/backend/backend_conformance_common.hpp:13).  It is not doctest and
// shares no code with it: it exists so that those scenario headers can be compiled, unchanged and
// in place, against this repository's backend on a machine that has no doctest installed.
//
// Semantics kept, because the scenarios rely on them:
//   * CHECK*   records a failure and continues; REQUIRE* records it and leaves the test case by
//     throwing (so a REQUIRE inside a destructor or a noexcept function terminates, as it would
//     under doctest);
//   * *_MESSAGE(cond, a << b << c) and INFO(a << b) / CAPTURE(x) build their text lazily, only
//     when an assertion fails while they are in scope;
//   * CHECK_THROWS_AS strips const and reference from the type it is given;
//   * an exception that escapes a test case fails that case and the run goes on with the next.
//
// Added for the log a test run keeps: every case prints how many assertions it evaluated and how
// many failed.  Command line: --list, --test-case=<pattern with *> (several: comma separated),
// --test-case-exclude=<pattern>.  Header only; every definition is inline.
#pragma once

#include <atomic>
#include <cstddef>
#include <cstdio>
#include <cstring>
#include <exception>
#include <functional>
#include <iostream>
#include <mutex>
#include <sstream>
#include <string>
#include <string_view>
#include <type_traits>
#include <typeinfo>
#include <vector>

namespace doctest {

namespace detail {

struct TestCase {
    const char* name;
    const char* file;
    int line;
    void (*body)();
};

inline std::vector<TestCase>& registry() {
    static std::vector<TestCase> cases;
    return cases;
}

inline int enroll(const char* name, const char* file, int line, void (*body)()) {
    registry().push_back(TestCase{name, file, line, body});
    return 0;
}

// Thrown by a failed REQUIRE*; deliberately not derived from std::exception so that scenario code
// catching std::exception does not swallow it.
struct LeaveTestCase {};

struct Tally {
    std::atomic<std::size_t> asserts{0};
    std::atomic<std::size_t> failures{0};
};

inline Tally& tally() {
    static Tally t;
    return t;
}

inline std::mutex& print_mutex() {
    static std::mutex m;
    return m;
}

template <class T>
std::string to_text(const T& value) {
    if constexpr (std::is_same_v<T, bool>) {
        return value ? "true" : "false";
    } else if constexpr (std::is_same_v<T, std::nullptr_t>) {
        return "nullptr";
    } else if constexpr (std::is_same_v<T, std::byte>) {
        return std::to_string(static_cast<unsigned>(value));
    } else if constexpr (std::is_same_v<T, unsigned char> || std::is_same_v<T, signed char>) {
        return std::to_string(static_cast<int>(value));
    } else if constexpr (requires(std::ostream& os, const T& v) { os << v; }) {
        std::ostringstream os;
        os << value;
        return os.str();
    } else if constexpr (std::is_enum_v<T>) {
        return std::to_string(static_cast<long long>(static_cast<std::underlying_type_t<T>>(value)));
    } else {
        return std::string("{") + typeid(T).name() + "}";
    }
}

// Lazily built text: `Text() * a << b << c` parses as ((Text() * a) << b) << c.
class Text {
public:
    template <class T>
    Text& operator*(const T& value) {
        text_ += to_text(value);
        return *this;
    }
    template <class T>
    Text& operator<<(const T& value) {
        text_ += to_text(value);
        return *this;
    }
    [[nodiscard]] const std::string& str() const { return text_; }

private:
    std::string text_;
};

// INFO / CAPTURE: a scope object on a per-thread stack, rendered only when an assertion fails.
class ContextScope;
inline std::vector<const ContextScope*>& context_stack() {
    thread_local std::vector<const ContextScope*> stack;
    return stack;
}

class ContextScope {
public:
    explicit ContextScope(std::function<std::string()> render) : render_(std::move(render)) {
        context_stack().push_back(this);
    }
    ContextScope(const ContextScope&) = delete;
    ContextScope& operator=(const ContextScope&) = delete;
    ~ContextScope() {
        auto& stack = context_stack();
        if (!stack.empty() && stack.back() == this) {
            stack.pop_back();
        }
    }
    [[nodiscard]] std::string render() const { return render_(); }

private:
    std::function<std::string()> render_;
};

inline void pass() { tally().asserts.fetch_add(1, std::memory_order_relaxed); }

inline void fail(const char* file, int line, const char* macro, const std::string& expression,
                 const std::string& detail, bool leave) {
    tally().asserts.fetch_add(1, std::memory_order_relaxed);
    tally().failures.fetch_add(1, std::memory_order_relaxed);
    {
        const std::lock_guard<std::mutex> lock(print_mutex());
        std::cout << file << ":" << line << ": FAILED: " << macro << "( " << expression << " )\n";
        if (!detail.empty()) {
            std::cout << "    " << detail << "\n";
        }
        for (const ContextScope* scope : context_stack()) {
            std::cout << "    with: " << scope->render() << "\n";
        }
        std::cout.flush();
    }
    if (leave) {
        throw LeaveTestCase{};
    }
}

inline void truth(bool ok, const char* file, int line, const char* macro, const char* expression,
                  bool leave, const std::function<std::string()>& message = {}) {
    if (ok) {
        pass();
        return;
    }
    fail(file, line, macro, expression, message ? message() : std::string(), leave);
}

#if defined(__GNUC__)
#pragma GCC diagnostic push
#pragma GCC diagnostic ignored "-Wsign-compare"
#endif
struct Eq { template <class L, class R> static bool test(const L& l, const R& r) { return l == r; } static constexpr const char* sign = "=="; };
struct Ne { template <class L, class R> static bool test(const L& l, const R& r) { return l != r; } static constexpr const char* sign = "!="; };
struct Lt { template <class L, class R> static bool test(const L& l, const R& r) { return l < r; } static constexpr const char* sign = "<"; };
struct Le { template <class L, class R> static bool test(const L& l, const R& r) { return l <= r; } static constexpr const char* sign = "<="; };
struct Gt { template <class L, class R> static bool test(const L& l, const R& r) { return l > r; } static constexpr const char* sign = ">"; };
struct Ge { template <class L, class R> static bool test(const L& l, const R& r) { return l >= r; } static constexpr const char* sign = ">="; };
#if defined(__GNUC__)
#pragma GCC diagnostic pop
#endif

template <class Relation, class L, class R>
void compare(const L& lhs, const R& rhs, const char* file, int line, const char* macro,
             const char* expression, bool leave) {
    if (Relation::test(lhs, rhs)) {
        pass();
        return;
    }
    fail(file, line, macro, expression,
         "values: " + to_text(lhs) + " " + Relation::sign + " " + to_text(rhs) + " does not hold", leave);
}

inline bool wildcard_match(std::string_view pattern, std::string_view text) {
    std::size_t p = 0, t = 0, star = std::string_view::npos, mark = 0;
    while (t < text.size()) {
        if (p < pattern.size() && (pattern[p] == text[t] || pattern[p] == '?')) {
            ++p;
            ++t;
        } else if (p < pattern.size() && pattern[p] == '*') {
            star = p++;
            mark = t;
        } else if (star != std::string_view::npos) {
            p = star + 1;
            t = ++mark;
        } else {
            return false;
        }
    }
    while (p < pattern.size() && pattern[p] == '*') {
        ++p;
    }
    return p == pattern.size();
}

inline std::vector<std::string> split_patterns(std::string_view list) {
    std::vector<std::string> result;
    std::size_t begin = 0;
    while (begin <= list.size()) {
        const std::size_t comma = list.find(',', begin);
        const std::size_t end = comma == std::string_view::npos ? list.size() : comma;
        if (end > begin) {
            result.emplace_back(list.substr(begin, end - begin));
        }
        if (comma == std::string_view::npos) {
            break;
        }
        begin = comma + 1;
    }
    return result;
}

inline bool matches_any(const std::vector<std::string>& patterns, std::string_view name) {
    for (const std::string& pattern : patterns) {
        if (wildcard_match(pattern, name)) {
            return true;
        }
    }
    return false;
}

}  // namespace detail

// Runs the registered cases.  run() returns 0 when every assertion of every selected case held and
// no exception escaped a case, 1 otherwise.
class Context {
public:
    Context() = default;
    Context(int argc, const char* const* argv) { applyCommandLine(argc, argv); }

    void applyCommandLine(int argc, const char* const* argv) {
        for (int i = 1; i < argc; ++i) {
            const std::string_view arg(argv[i]);
            if (arg == "--list" || arg == "-ltc" || arg == "--list-test-cases") {
                list_only_ = true;
            } else if (arg.starts_with("--test-case=")) {
                include_ = detail::split_patterns(arg.substr(12));
            } else if (arg.starts_with("-tc=")) {
                include_ = detail::split_patterns(arg.substr(4));
            } else if (arg.starts_with("--test-case-exclude=")) {
                exclude_ = detail::split_patterns(arg.substr(20));
            } else if (arg.starts_with("-tce=")) {
                exclude_ = detail::split_patterns(arg.substr(5));
            }
        }
    }

    [[nodiscard]] bool shouldExit() const { return false; }

    int run() {
        std::size_t ran = 0, failed_cases = 0, total_asserts = 0, total_failures = 0;
        for (const detail::TestCase& test : detail::registry()) {
            if (!include_.empty() && !detail::matches_any(include_, test.name)) {
                continue;
            }
            if (detail::matches_any(exclude_, test.name)) {
                continue;
            }
            if (list_only_) {
                std::cout << test.name << "\n";
                continue;
            }
            std::cout << "[ case ] " << test.name << std::endl;
            const std::size_t asserts_before = detail::tally().asserts.load();
            const std::size_t failures_before = detail::tally().failures.load();
            bool escaped = false;
            try {
                test.body();
            } catch (const detail::LeaveTestCase&) {
                // already counted by the REQUIRE that threw
            } catch (const std::exception& error) {
                escaped = true;
                std::cout << test.file << ":" << test.line << ": FAILED: exception escaped the case: "
                          << typeid(error).name() << ": " << error.what() << std::endl;
            } catch (...) {
                escaped = true;
                std::cout << test.file << ":" << test.line
                          << ": FAILED: unknown exception escaped the case" << std::endl;
            }
            detail::context_stack().clear();
            const std::size_t asserts = detail::tally().asserts.load() - asserts_before;
            const std::size_t failures =
                    detail::tally().failures.load() - failures_before + (escaped ? 1 : 0);
            std::cout << "[ " << (failures == 0 ? " ok " : "FAIL") << " ] " << test.name << ": "
                      << asserts << " assertions, " << failures << " failed" << std::endl;
            ++ran;
            failed_cases += failures != 0;
            total_asserts += asserts;
            total_failures += failures;
        }
        if (!list_only_) {
            std::cout << "[ done ] " << ran << " cases, " << failed_cases << " failed; "
                      << total_asserts << " assertions, " << total_failures << " failed" << std::endl;
        }
        return total_failures == 0 ? 0 : 1;
    }

private:
    std::vector<std::string> include_;
    std::vector<std::string> exclude_;
    bool list_only_ = false;
};

}  // namespace doctest

#define IOMX_DT_CAT2(a, b) a##b
#define IOMX_DT_CAT(a, b) IOMX_DT_CAT2(a, b)
#define IOMX_DT_UNIQUE(stem) IOMX_DT_CAT(stem, __COUNTER__)

#define IOMX_DT_TEST_CASE(function, name)                                                       \
    static void function();                                                                     \
    [[maybe_unused]] static const int IOMX_DT_CAT(function, _enrolled) =                        \
            ::doctest::detail::enroll(name, __FILE__, __LINE__, &function);                     \
    static void function()
#define TEST_CASE(name) IOMX_DT_TEST_CASE(IOMX_DT_UNIQUE(iomx_dt_case_), name)

#define IOMX_DT_INFO(scope, ...)                                                                \
    const ::doctest::detail::ContextScope scope([&]() -> std::string {                          \
        ::doctest::detail::Text text;                                                           \
        text * __VA_ARGS__;                                                                     \
        return text.str();                                                                      \
    })
#define INFO(...) IOMX_DT_INFO(IOMX_DT_UNIQUE(iomx_dt_info_), __VA_ARGS__)
#define CAPTURE(x) INFO(#x " := " << x)

#define MESSAGE(...)                                                                            \
    do {                                                                                        \
        ::doctest::detail::Text text;                                                           \
        text * __VA_ARGS__;                                                                     \
        const std::lock_guard<std::mutex> lock(::doctest::detail::print_mutex());               \
        std::cout << __FILE__ << ":" << __LINE__ << ": MESSAGE: " << text.str() << std::endl;   \
    } while (false)

#define IOMX_DT_FAIL(macro, leave, ...)                                                         \
    do {                                                                                        \
        ::doctest::detail::Text text;                                                           \
        text * __VA_ARGS__;                                                                     \
        ::doctest::detail::fail(__FILE__, __LINE__, macro, text.str(), std::string(), leave);   \
    } while (false)
#define FAIL(...) IOMX_DT_FAIL("FAIL", true, __VA_ARGS__)
#define FAIL_CHECK(...) IOMX_DT_FAIL("FAIL_CHECK", false, __VA_ARGS__)

#define IOMX_DT_TRUTH(macro, leave, negate, ...)                                                \
    ::doctest::detail::truth((negate) != static_cast<bool>(__VA_ARGS__), __FILE__, __LINE__,    \
                             macro, #__VA_ARGS__, leave)
#define CHECK(...) IOMX_DT_TRUTH("CHECK", false, false, __VA_ARGS__)
#define REQUIRE(...) IOMX_DT_TRUTH("REQUIRE", true, false, __VA_ARGS__)
#define CHECK_FALSE(...) IOMX_DT_TRUTH("CHECK_FALSE", false, true, __VA_ARGS__)
#define REQUIRE_FALSE(...) IOMX_DT_TRUTH("REQUIRE_FALSE", true, true, __VA_ARGS__)
#define CHECK_UNARY(...) IOMX_DT_TRUTH("CHECK_UNARY", false, false, __VA_ARGS__)
#define REQUIRE_UNARY(...) IOMX_DT_TRUTH("REQUIRE_UNARY", true, false, __VA_ARGS__)
#define CHECK_UNARY_FALSE(...) IOMX_DT_TRUTH("CHECK_UNARY_FALSE", false, true, __VA_ARGS__)
#define REQUIRE_UNARY_FALSE(...) IOMX_DT_TRUTH("REQUIRE_UNARY_FALSE", true, true, __VA_ARGS__)

#define IOMX_DT_TRUTH_MESSAGE(macro, leave, negate, cond, ...)                                  \
    ::doctest::detail::truth((negate) != static_cast<bool>(cond), __FILE__, __LINE__, macro,    \
                             #cond, leave, [&]() -> std::string {                               \
                                 ::doctest::detail::Text text;                                  \
                                 text * __VA_ARGS__;                                            \
                                 return text.str();                                             \
                             })
#define CHECK_MESSAGE(cond, ...) IOMX_DT_TRUTH_MESSAGE("CHECK", false, false, cond, __VA_ARGS__)
#define REQUIRE_MESSAGE(cond, ...) IOMX_DT_TRUTH_MESSAGE("REQUIRE", true, false, cond, __VA_ARGS__)
#define CHECK_FALSE_MESSAGE(cond, ...) \
    IOMX_DT_TRUTH_MESSAGE("CHECK_FALSE", false, true, cond, __VA_ARGS__)
#define REQUIRE_FALSE_MESSAGE(cond, ...) \
    IOMX_DT_TRUTH_MESSAGE("REQUIRE_FALSE", true, true, cond, __VA_ARGS__)

#define IOMX_DT_COMPARE(macro, leave, relation, ...)                                            \
    ::doctest::detail::compare<::doctest::detail::relation>(__VA_ARGS__, __FILE__, __LINE__,    \
                                                            macro, #__VA_ARGS__, leave)
#define CHECK_EQ(...) IOMX_DT_COMPARE("CHECK_EQ", false, Eq, __VA_ARGS__)
#define CHECK_NE(...) IOMX_DT_COMPARE("CHECK_NE", false, Ne, __VA_ARGS__)
#define CHECK_LT(...) IOMX_DT_COMPARE("CHECK_LT", false, Lt, __VA_ARGS__)
#define CHECK_LE(...) IOMX_DT_COMPARE("CHECK_LE", false, Le, __VA_ARGS__)
#define CHECK_GT(...) IOMX_DT_COMPARE("CHECK_GT", false, Gt, __VA_ARGS__)
#define CHECK_GE(...) IOMX_DT_COMPARE("CHECK_GE", false, Ge, __VA_ARGS__)
#define REQUIRE_EQ(...) IOMX_DT_COMPARE("REQUIRE_EQ", true, Eq, __VA_ARGS__)
#define REQUIRE_NE(...) IOMX_DT_COMPARE("REQUIRE_NE", true, Ne, __VA_ARGS__)
#define REQUIRE_LT(...) IOMX_DT_COMPARE("REQUIRE_LT", true, Lt, __VA_ARGS__)
#define REQUIRE_LE(...) IOMX_DT_COMPARE("REQUIRE_LE", true, Le, __VA_ARGS__)
#define REQUIRE_GT(...) IOMX_DT_COMPARE("REQUIRE_GT", true, Gt, __VA_ARGS__)
#define REQUIRE_GE(...) IOMX_DT_COMPARE("REQUIRE_GE", true, Ge, __VA_ARGS__)

// An expression under test may itself hold a REQUIRE that fails: that must leave the case, not be
// taken for the exception (or the absence of one) that the outer assertion looks for.
#define IOMX_DT_THROWS(macro, leave, ...)                                                       \
    do {                                                                                        \
        bool iomx_dt_threw = false;                                                             \
        try {                                                                                   \
            static_cast<void>(__VA_ARGS__);                                                     \
        } catch (const ::doctest::detail::LeaveTestCase&) {                                     \
            throw;                                                                              \
        } catch (...) {                                                                         \
            iomx_dt_threw = true;                                                               \
        }                                                                                       \
        ::doctest::detail::truth(iomx_dt_threw, __FILE__, __LINE__, macro, #__VA_ARGS__, leave, \
                                 [] { return std::string("no exception was thrown"); });        \
    } while (false)
#define CHECK_THROWS(...) IOMX_DT_THROWS("CHECK_THROWS", false, __VA_ARGS__)
#define REQUIRE_THROWS(...) IOMX_DT_THROWS("REQUIRE_THROWS", true, __VA_ARGS__)

#define IOMX_DT_THROWS_AS(macro, leave, expression, ...)                                        \
    do {                                                                                        \
        int iomx_dt_outcome = 0; /* 0 nothing thrown, 1 the type, 2 another type */             \
        std::string iomx_dt_what;                                                               \
        try {                                                                                   \
            static_cast<void>(expression);                                                      \
        } catch (const ::doctest::detail::LeaveTestCase&) {                                     \
            throw;                                                                              \
        } catch (const std::remove_cv_t<std::remove_reference_t<__VA_ARGS__>>&) {               \
            iomx_dt_outcome = 1;                                                                \
        } catch (const std::exception& iomx_dt_error) {                                         \
            iomx_dt_outcome = 2;                                                                \
            iomx_dt_what = std::string(typeid(iomx_dt_error).name()) + ": " +                   \
                    iomx_dt_error.what();                                                       \
        } catch (...) {                                                                         \
            iomx_dt_outcome = 2;                                                                \
            iomx_dt_what = "an exception that is not a std::exception";                         \
        }                                                                                       \
        ::doctest::detail::truth(                                                               \
                iomx_dt_outcome == 1, __FILE__, __LINE__, macro,                                \
                #expression ", " #__VA_ARGS__, leave, [&] {                                     \
                    return iomx_dt_outcome == 0 ? std::string("no exception was thrown")        \
                                                : "threw instead: " + iomx_dt_what;             \
                });                                                                             \
    } while (false)
#define CHECK_THROWS_AS(expression, ...) \
    IOMX_DT_THROWS_AS("CHECK_THROWS_AS", false, expression, __VA_ARGS__)
#define REQUIRE_THROWS_AS(expression, ...) \
    IOMX_DT_THROWS_AS("REQUIRE_THROWS_AS", true, expression, __VA_ARGS__)

#define IOMX_DT_THROWS_WITH(macro, leave, expression, ...)                                      \
    do {                                                                                        \
        int iomx_dt_outcome = 0; /* 0 nothing thrown, 1 text matches, 2 other text or type */   \
        std::string iomx_dt_what;                                                               \
        try {                                                                                   \
            static_cast<void>(expression);                                                      \
        } catch (const ::doctest::detail::LeaveTestCase&) {                                     \
            throw;                                                                              \
        } catch (const std::exception& iomx_dt_error) {                                         \
            iomx_dt_what = iomx_dt_error.what();                                                \
            iomx_dt_outcome = iomx_dt_what == std::string(__VA_ARGS__) ? 1 : 2;                 \
        } catch (const char* iomx_dt_text) {                                                    \
            iomx_dt_what = iomx_dt_text;                                                        \
            iomx_dt_outcome = iomx_dt_what == std::string(__VA_ARGS__) ? 1 : 2;                 \
        } catch (...) {                                                                         \
            iomx_dt_outcome = 2;                                                                \
            iomx_dt_what = "an exception without text";                                         \
        }                                                                                       \
        ::doctest::detail::truth(                                                               \
                iomx_dt_outcome == 1, __FILE__, __LINE__, macro,                                \
                #expression ", " #__VA_ARGS__, leave, [&] {                                     \
                    return iomx_dt_outcome == 0 ? std::string("no exception was thrown")        \
                                                : "threw with: " + iomx_dt_what;                \
                });                                                                             \
    } while (false)
#define CHECK_THROWS_WITH(expression, ...) \
    IOMX_DT_THROWS_WITH("CHECK_THROWS_WITH", false, expression, __VA_ARGS__)
#define REQUIRE_THROWS_WITH(expression, ...) \
    IOMX_DT_THROWS_WITH("REQUIRE_THROWS_WITH", true, expression, __VA_ARGS__)

#define IOMX_DT_NOTHROW(macro, leave, ...)                                                      \
    do {                                                                                        \
        std::string iomx_dt_what;                                                               \
        bool iomx_dt_threw = false;                                                             \
        try {                                                                                   \
            static_cast<void>(__VA_ARGS__);                                                     \
        } catch (const ::doctest::detail::LeaveTestCase&) {                                     \
            throw;                                                                              \
        } catch (const std::exception& iomx_dt_error) {                                         \
            iomx_dt_threw = true;                                                               \
            iomx_dt_what = std::string(typeid(iomx_dt_error).name()) + ": " +                   \
                    iomx_dt_error.what();                                                       \
        } catch (...) {                                                                         \
            iomx_dt_threw = true;                                                               \
            iomx_dt_what = "an exception that is not a std::exception";                         \
        }                                                                                       \
        ::doctest::detail::truth(!iomx_dt_threw, __FILE__, __LINE__, macro, #__VA_ARGS__,       \
                                 leave, [&] { return "threw: " + iomx_dt_what; });              \
    } while (false)
#define CHECK_NOTHROW(...) IOMX_DT_NOTHROW("CHECK_NOTHROW", false, __VA_ARGS__)
#define REQUIRE_NOTHROW(...) IOMX_DT_NOTHROW("REQUIRE_NOTHROW", true, __VA_ARGS__)
