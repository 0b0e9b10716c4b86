// Host matmul kernels (explicit DeviceCPU layers only).
#include "matmul_kernel.h"

#include "bf16.h"

#include <cstring>
#include <vector>

namespace kernel {
namespace {

// column of nibble i inside a packed word: 0, 2, 4, 6, 1, 3, 5, 7
inline int column_of_nibble(int i) {
    return i < 4 ? 2 * i : 2 * (i - 4) + 1;
}

// [M, inner] or [inner] -> M
int32_t rows_of(const tensor::Tensor& t, int32_t inner) {
    if (t.dims_size() == 1) {
        CHECK_EQ(t.get_dim(0), inner);
        return 1;
    }
    CHECK_EQ(t.dims_size(), 2);
    CHECK_EQ(t.get_dim(1), inner);
    return t.get_dim(0);
}

}  // namespace

void matmul_kernel_cpu(const tensor::Tensor& input, const tensor::Tensor& weight,
                       const tensor::Tensor& output, void* stream) {
    UNUSED(stream);
    CHECK_EQ(input.is_empty(), false);
    CHECK_EQ(weight.is_empty(), false);
    CHECK_EQ(output.is_empty(), false);
    CHECK_EQ(weight.dims_size(), 2);
    const int32_t N = weight.get_dim(0);
    const int32_t K = weight.get_dim(1);
    const int32_t M = rows_of(input, K);
    CHECK_EQ(rows_of(output, N), M);

    const uint16_t* x = input.ptr<uint16_t>();
    const uint16_t* w = weight.ptr<uint16_t>();
    uint16_t* y = const_cast<uint16_t*>(output.ptr<uint16_t>());
    for (int32_t m = 0; m < M; m++) {
        for (int32_t n = 0; n < N; n++) {
            float acc = 0.0f;
            for (int32_t k = 0; k < K; k++) {
                acc += bf16_to_float(x[static_cast<size_t>(m) * K + k]) * bf16_to_float(w[static_cast<size_t>(n) * K + k]);
            }
            y[static_cast<size_t>(m) * N + n] = float_to_bf16(acc);
        }
    }
}

void matmul_kernel_awq_cpu(const tensor::Tensor& input, const tensor::Tensor& qweight,
                           const tensor::Tensor& scales, const tensor::Tensor& qzeros,
                           const tensor::Tensor& output, int32_t group_size, void* stream) {
    UNUSED(stream);
    CHECK_EQ(input.is_empty(), false);
    CHECK_EQ(qweight.is_empty(), false);
    CHECK_EQ(scales.is_empty(), false);
    CHECK_EQ(qzeros.is_empty(), false);
    CHECK_EQ(output.is_empty(), false);
    CHECK_EQ(qweight.dims_size(), 2);
    CHECK_GT(group_size, 0);
    const int32_t K = qweight.get_dim(0);
    const int32_t words = qweight.get_dim(1);
    const int32_t N = words * 8;
    CHECK_EQ(K % group_size, 0);
    const int32_t groups = K / group_size;
    CHECK_EQ(scales.size(), static_cast<size_t>(groups) * N);
    CHECK_EQ(qzeros.size(), static_cast<size_t>(groups) * words);
    const int32_t M = rows_of(input, K);
    CHECK_EQ(rows_of(output, N), M);

    const uint16_t* x = input.ptr<uint16_t>();
    const uint32_t* qw = qweight.ptr<uint32_t>();
    const uint16_t* sc = scales.ptr<uint16_t>();
    const uint32_t* qz = qzeros.ptr<uint32_t>();
    uint16_t* y = const_cast<uint16_t*>(output.ptr<uint16_t>());

    // per group: sum_k q*x and sum_k x first, then one (.. - z * sum x) * s per column
    std::vector<float> total(N), qx(N);
    for (int32_t m = 0; m < M; m++) {
        std::fill(total.begin(), total.end(), 0.0f);
        for (int32_t g = 0; g < groups; g++) {
            std::fill(qx.begin(), qx.end(), 0.0f);
            float xsum = 0.0f;
            for (int32_t k = g * group_size; k < (g + 1) * group_size; k++) {
                const float xv = bf16_to_float(x[static_cast<size_t>(m) * K + k]);
                xsum += xv;
                const uint32_t* row = qw + static_cast<size_t>(k) * words;
                for (int32_t j = 0; j < words; j++) {
                    const uint32_t word = row[j];
                    for (int i = 0; i < 8; i++) {
                        qx[8 * j + column_of_nibble(i)] += static_cast<float>((word >> (4 * i)) & 0xfu) * xv;
                    }
                }
            }
            for (int32_t j = 0; j < words; j++) {
                const uint32_t zword = qz[static_cast<size_t>(g) * words + j];
                for (int i = 0; i < 8; i++) {
                    const int32_t n = 8 * j + column_of_nibble(i);
                    const float z = static_cast<float>((zword >> (4 * i)) & 0xfu);
                    total[n] += fp16_to_float(sc[static_cast<size_t>(g) * N + n]) * (qx[n] - z * xsum);
                }
            }
        }
        for (int32_t n = 0; n < N; n++) {
            y[static_cast<size_t>(m) * N + n] = float_to_bf16(total[n]);
        }
    }
}

}  // namespace kernel
