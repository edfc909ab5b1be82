// Tiny assertion helper for the test programs: count failures, exit code = number of failures.
#ifndef CTORCH_AMD_HOST_TEST_CHECK_H
#define CTORCH_AMD_HOST_TEST_CHECK_H
#include <cmath>
#include <cstdio>
#include <string>
#include <vector>

#include "Tensor.h"

static int g_failures = 0;

#define CHECK(cond, what)                                                        \
    do {                                                                         \
        if (!(cond)) {                                                           \
            std::printf("FAIL %s:%d %s\n", __FILE__, __LINE__, what);            \
            ++g_failures;                                                        \
        } else {                                                                 \
            std::printf("ok   %s\n", what);                                      \
        }                                                                        \
    } while (0)

inline bool all_close(const Tensor& t, const std::vector<float>& want, float tol) {
    std::vector<float> got = t.to_vector();
    if (got.size() != want.size()) return false;
    for (size_t i = 0; i < got.size(); ++i)
        if (!(std::fabs(got[i] - want[i]) <= tol)) return false;
    return true;
}
inline bool all_equal_to(const Tensor& t, float v, float tol) {
    return all_close(t, std::vector<float>(t.numel(), v), tol);
}
inline Tensor device_tensor(const std::vector<size_t>& shape, const std::vector<float>& values) {
    return Tensor::from_host(values.data(), shape, DeviceType::kAMD);
}
#endif
