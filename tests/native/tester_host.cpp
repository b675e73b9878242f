// The gradient testers compiled by a plain host compiler: every case runs on the calling thread.
#include "tester_suite.cuh"
#include "concept_checks.cuh"

extern "C" int xad_test_tester_suite_host(char* text, std::size_t capacity, unsigned* self_checks) {
    return xad_suite::export_suite(text, capacity, self_checks);
}

extern "C" const char* xad_test_host_source_digest(void) { return XAD_TEST_SOURCE_DIGEST; }
