#ifndef KX_TEST_UTILS_H
#define KX_TEST_UTILS_H
#include <cstdint>
// Fills a GPU fp32 array with one value and waits for it (role of the reference's
// test/utils.cu:19-38).
void set_value_cu(float* arr_cu, int32_t size, float value = 1.f);
#endif
