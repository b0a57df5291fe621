// Checks the assertion harness in doctest/doctest.h itself: cases built to fail must be reported as
// failed with the right counts, cases built to pass as passed.  The program prints one line per
// expectation and returns 0 only if the harness behaved as documented.  CPU only.
#include <doctest/doctest.h>

#include <cstdio>
#include <sstream>
#include <stdexcept>
#include <string>

namespace {

enum class Colour { red = 3, green = 5 };

int g_after_require = 0;

void throws_invalid() { throw std::invalid_argument("bad argument"); }
void throws_nothing() {}

}  // namespace

TEST_CASE("pass: every assertion form holds") {
    CHECK(1 + 1 == 2);
    CHECK_FALSE(1 + 1 == 3);
    REQUIRE(true);
    REQUIRE_FALSE(false);
    CHECK_EQ(2, 2u);
    CHECK_NE(2, 3);
    CHECK_LT(2, 3);
    CHECK_LE(3, 3);
    CHECK_GT(4, 3);
    CHECK_GE(3, 3);
    REQUIRE_EQ(std::string("a"), "a");
    CHECK_EQ(Colour::red, Colour::red);
    CHECK_MESSAGE(true, "never rendered " << 1);
    REQUIRE_MESSAGE(true, "never rendered");
    CHECK_THROWS(throws_invalid());
    CHECK_THROWS_AS(throws_invalid(), std::invalid_argument);
    CHECK_THROWS_AS(throws_invalid(), const std::invalid_argument&);
    CHECK_THROWS_AS(throws_invalid(), std::logic_error);
    CHECK_THROWS_WITH(throws_invalid(), "bad argument");
    CHECK_NOTHROW(throws_nothing());
    REQUIRE_NOTHROW(throws_nothing());
    const int captured = 7;
    CAPTURE(captured);
    INFO("label " << captured);
    CHECK(captured == 7);
}

TEST_CASE("fail: six CHECK forms fail and the case continues") {
    CHECK(1 + 1 == 3);                                        // 1
    CHECK_EQ(Colour::red, Colour::green);                     // 2
    CHECK_MESSAGE(false, "rendered " << 42);                  // 3
    CHECK_THROWS_AS(throws_invalid(), std::runtime_error);    // 4
    CHECK_THROWS_AS(throws_nothing(), std::runtime_error);    // 5
    CHECK_NOTHROW(throws_invalid());                          // 6
    CHECK(true);
}

TEST_CASE("fail: REQUIRE leaves the case") {
    CHECK(true);
    REQUIRE_EQ(1, 2);
    ++g_after_require;  // must not run
    CHECK(true);
}

TEST_CASE("fail: a REQUIRE inside CHECK_NOTHROW leaves the case instead of counting as a throw") {
    CHECK_NOTHROW([] { REQUIRE(false); }());
    ++g_after_require;  // must not run
}

TEST_CASE("fail: an escaped exception fails the case") {
    CHECK(true);
    throw std::runtime_error("escaped");
}

TEST_CASE("pass: context of an earlier case does not leak") {
    CHECK(true);
}

int main() {
    // capture the harness's own report
    std::ostringstream report;
    std::streambuf* previous = std::cout.rdbuf(report.rdbuf());
    doctest::Context context;
    const int status = context.run();
    std::cout.rdbuf(previous);
    const std::string text = report.str();

    int wrong = 0;
    const auto expect = [&](bool ok, const char* what) {
        std::printf("%s: %s\n", ok ? "ok" : "WRONG", what);
        wrong += ok ? 0 : 1;
    };
    const auto has = [&](const char* needle) { return text.find(needle) != std::string::npos; };

    expect(status == 1, "run() reports failure");
    expect(has("pass: every assertion form holds: 22 assertions, 0 failed"), "passing case counted");
    expect(has("fail: six CHECK forms fail and the case continues: 7 assertions, 6 failed"),
           "CHECK failures counted, case continued");
    expect(has("values: 3 == 5 does not hold"), "enum operands rendered by value");
    expect(has("rendered 42"), "message rendered on failure");
    expect(!has("never rendered"), "message not rendered on success");
    expect(has("threw instead: "), "wrong exception type reported");
    expect(has("no exception was thrown"), "missing exception reported");
    expect(has("fail: REQUIRE leaves the case: 2 assertions, 1 failed"), "REQUIRE left the case");
    expect(g_after_require == 0, "nothing ran after a failed REQUIRE");
    expect(has("instead of counting as a throw: 1 assertions, 1 failed"),
           "nested REQUIRE is not taken for a thrown exception");
    expect(has("exception escaped the case"), "escaped exception reported");
    expect(has("fail: an escaped exception fails the case: 1 assertions, 1 failed"),
           "escaped exception fails the case");
    expect(has("does not leak: 1 assertions, 0 failed"), "later case is clean");
    expect(has("[ done ] 6 cases, 4 failed; 34 assertions, 9 failed"), "totals");
    if (wrong != 0) {
        std::printf("---- harness report ----\n%s", text.c_str());
    }
    return wrong == 0 ? 0 : 1;
}
