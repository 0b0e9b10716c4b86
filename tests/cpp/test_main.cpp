// Runner:  test_kuiper --cpu | --gpu | --all   [--list] [--only suite.name]
// Prints one "[ OK ] suite.name" / "[FAIL] suite.name: reason" line per test; exit code 1 on any
// failure.  (Role of the reference's test/test_main.cpp:4-16.)
#include <cstdio>
#include <cstring>
#include <string>

#include "base/log.h"
#include "mini_test.h"

namespace mini {
std::vector<TestCase>& registry() {
    static std::vector<TestCase> tests;
    return tests;
}
}  // namespace mini

static void throwing_fatal_handler(const std::string& message) {
    throw mini::Fatal(message);
}

int main(int argc, char** argv) {
    bool want_cpu = false, want_gpu = false, list = false;
    std::string only;
    for (int i = 1; i < argc; i++) {
        if (!std::strcmp(argv[i], "--cpu")) want_cpu = true;
        else if (!std::strcmp(argv[i], "--gpu")) want_gpu = true;
        else if (!std::strcmp(argv[i], "--all")) want_cpu = want_gpu = true;
        else if (!std::strcmp(argv[i], "--list")) list = true;
        else if (!std::strcmp(argv[i], "--only") && i + 1 < argc) only = argv[++i];
    }
    if (!want_cpu && !want_gpu) want_cpu = true;
    base::set_fatal_handler(throwing_fatal_handler);
    base::set_min_log_severity(base::LogSeverity::kFatal);  // expected errors are not noise

    int failed = 0, ran = 0;
    for (const auto& t : mini::registry()) {
        const std::string full = t.suite + "." + t.name;
        if (t.needs_gpu ? !want_gpu : !want_cpu) continue;
        if (!only.empty() && only != full) continue;
        if (list) {
            std::printf("%s\n", full.c_str());
            continue;
        }
        std::printf("[ RUN ] %s\n", full.c_str());
        std::fflush(stdout);
        ran++;
        try {
            t.body();
            std::printf("[ OK ] %s\n", full.c_str());
        } catch (const mini::Failure& f) {
            failed++;
            std::printf("[FAIL] %s: %s\n", full.c_str(), f.what());
        } catch (const mini::Fatal& f) {
            failed++;
            std::printf("[FAIL] %s: unexpected fatal check: %s\n", full.c_str(), f.what());
        } catch (const std::exception& e) {
            failed++;
            std::printf("[FAIL] %s: exception: %s\n", full.c_str(), e.what());
        }
        std::fflush(stdout);
    }
    if (!list) std::printf("%d run, %d failed\n", ran, failed);
    return failed ? 1 : 0;
}
