// A very small test runner with gtest-like macros, enough to restate the reference's
// test/test_tensor, test/test_op cases (which use gtest, absent from this image).
// Every test carries a flag saying whether it needs a GPU; the runner selects by that flag.
#ifndef KX_MINI_TEST_H
#define KX_MINI_TEST_H

#include <cmath>
#include <functional>
#include <sstream>
#include <stdexcept>
#include <string>
#include <vector>

namespace mini {

struct Failure : std::runtime_error {
    using std::runtime_error::runtime_error;
};

// thrown by the fatal handler the runner installs: a CHECK / LOG(FATAL) inside the library
struct Fatal : std::runtime_error {
    using std::runtime_error::runtime_error;
};

struct TestCase {
    std::string suite, name;
    bool needs_gpu;
    std::function<void()> body;
};

std::vector<TestCase>& registry();

struct Registrar {
    Registrar(const char* suite, const char* name, bool needs_gpu, std::function<void()> body) {
        registry().push_back({suite, name, needs_gpu, std::move(body)});
    }
};

template <typename A, typename B>
std::string describe(const char* expr_a, const char* expr_b, const A& a, const B& b, const char* op,
                     const char* file, int line) {
    std::ostringstream os;
    os << file << ":" << line << ": expected " << expr_a << " " << op << " " << expr_b;
    (void)a;
    (void)b;
    return os.str();
}

}  // namespace mini

#define KX_TEST_IMPL(suite, name, gpu)                                                        \
    static void suite##_##name##_body();                                                      \
    static ::mini::Registrar suite##_##name##_reg(#suite, #name, gpu, suite##_##name##_body); \
    static void suite##_##name##_body()
#define TEST_CPU(suite, name) KX_TEST_IMPL(suite, name, false)
#define TEST_GPU(suite, name) KX_TEST_IMPL(suite, name, true)

#define KX_FAIL(msg) throw ::mini::Failure(std::string(__FILE__) + ":" + std::to_string(__LINE__) + ": " + (msg))
#define ASSERT_TRUE(c) do { if (!(c)) KX_FAIL("expected " #c); } while (0)
#define ASSERT_FALSE(c) do { if (c) KX_FAIL("expected !(" #c ")"); } while (0)
#define ASSERT_EQ(a, b) do { if (!((a) == (b))) KX_FAIL("expected " #a " == " #b); } while (0)
#define ASSERT_NE(a, b) do { if (!((a) != (b))) KX_FAIL("expected " #a " != " #b); } while (0)
#define ASSERT_LE(a, b) do { if (!((a) <= (b))) KX_FAIL("expected " #a " <= " #b); } while (0)
#define ASSERT_NEAR(a, b, tol) do { if (!(std::fabs((a) - (b)) <= (tol))) KX_FAIL("expected |" #a " - " #b "| <= " #tol); } while (0)
// the statement must end in a library CHECK failure / LOG(FATAL)
#define ASSERT_FATAL(stmt)                                      \
    do {                                                        \
        bool kx_died = false;                                   \
        try { stmt; } catch (const ::mini::Fatal&) { kx_died = true; } \
        if (!kx_died) KX_FAIL("expected a fatal check in: " #stmt); \
    } while (0)

#endif  // KX_MINI_TEST_H
