// C++ consumer of the device classes, in the spirit of the reference's examples/cuda/example.cu:
// allocates device buffers with the HIP runtime, evaluates through
// sphericart::cuda::SphericalHarmonics<T> / SolidHarmonics<T> (include/sphericart_cuda.hpp)
// and writes the results to a file for the test-suite to compare.
//
//   device_example <f32|f64> <spherical|solid> <l_max> <n_samples> <xyz.bin> <out.bin>
//
// xyz.bin holds n_samples * 3 numbers of the chosen type; out.bin receives sph, dsph and ddsph one
// after the other. Built by sphericart_amd/build.py with hipcc (host code only: it needs
// hip_runtime_api.h for the allocations, the header of the classes needs no HIP at all) and linked
// against libsphericart_amd.so.

#include <hip/hip_runtime_api.h>

#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <memory>
#include <stdexcept>
#include <string>
#include <vector>

#include "sphericart_cuda.hpp"

#define HIP_CHECK(call)                                                                        \
    do {                                                                                       \
        hipError_t status_ = (call);                                                           \
        if (status_ != hipSuccess) {                                                           \
            std::fprintf(stderr, "HIP error at %s:%d - %s\n", __FILE__, __LINE__,              \
                         hipGetErrorString(status_));                                          \
            std::exit(EXIT_FAILURE);                                                           \
        }                                                                                      \
    } while (0)

template <typename T> static int run(bool solid, size_t l_max, size_t n, const char* in, const char* out) {
    const size_t ny = (l_max + 1) * (l_max + 1);
    std::vector<T> xyz(n * 3);
    FILE* f = std::fopen(in, "rb");
    if (!f || std::fread(xyz.data(), sizeof(T), xyz.size(), f) != xyz.size()) {
        std::fprintf(stderr, "cannot read %s\n", in);
        return 2;
    }
    std::fclose(f);

    // the solid class derives from the spherical one: hold either through the base
    std::unique_ptr<sphericart::cuda::SphericalHarmonics<T>> calculator;
    if (solid) {
        calculator = std::make_unique<sphericart::cuda::SolidHarmonics<T>>(l_max);
    } else {
        calculator = std::make_unique<sphericart::cuda::SphericalHarmonics<T>>(l_max);
    }

    T *d_xyz = nullptr, *d_sph = nullptr, *d_dsph = nullptr, *d_ddsph = nullptr;
    HIP_CHECK(hipMalloc(reinterpret_cast<void**>(&d_xyz), n * 3 * sizeof(T)));
    HIP_CHECK(hipMalloc(reinterpret_cast<void**>(&d_sph), n * ny * sizeof(T)));
    HIP_CHECK(hipMalloc(reinterpret_cast<void**>(&d_dsph), n * 3 * ny * sizeof(T)));
    HIP_CHECK(hipMalloc(reinterpret_cast<void**>(&d_ddsph), n * 9 * ny * sizeof(T)));
    HIP_CHECK(hipMemcpy(d_xyz, xyz.data(), n * 3 * sizeof(T), hipMemcpyHostToDevice));

    hipStream_t stream;
    HIP_CHECK(hipStreamCreate(&stream));
    calculator->compute(d_xyz, n, d_sph);                                  // default stream
    calculator->compute_with_gradients(d_xyz, n, d_sph, d_dsph, stream);   // a stream of the caller's
    HIP_CHECK(hipStreamSynchronize(stream));
    calculator->compute_with_hessians(d_xyz, n, d_sph, d_dsph, d_ddsph, stream);
    HIP_CHECK(hipStreamSynchronize(stream));

    // errors are exceptions with the reference's messages
    bool thrown = false;
    try {
        calculator->compute_with_gradients(d_xyz, n, d_sph, nullptr);
    } catch (const std::runtime_error& e) {
        thrown = std::strstr(e.what(), "dsph != nullptr") != nullptr;
    }
    if (!thrown) {
        std::fprintf(stderr, "a null dsph did not raise the expected exception\n");
        return 3;
    }
    calculator->compute(nullptr, 0, nullptr); // no samples: returns before looking at pointers

    std::vector<T> result(n * ny * 13);
    HIP_CHECK(hipMemcpy(result.data(), d_sph, n * ny * sizeof(T), hipMemcpyDeviceToHost));
    HIP_CHECK(hipMemcpy(result.data() + n * ny, d_dsph, n * 3 * ny * sizeof(T), hipMemcpyDeviceToHost));
    HIP_CHECK(hipMemcpy(result.data() + n * 4 * ny, d_ddsph, n * 9 * ny * sizeof(T), hipMemcpyDeviceToHost));
    f = std::fopen(out, "wb");
    if (!f || std::fwrite(result.data(), sizeof(T), result.size(), f) != result.size()) {
        std::fprintf(stderr, "cannot write %s\n", out);
        return 2;
    }
    std::fclose(f);
    HIP_CHECK(hipStreamDestroy(stream));
    HIP_CHECK(hipFree(d_xyz));
    HIP_CHECK(hipFree(d_sph));
    HIP_CHECK(hipFree(d_dsph));
    HIP_CHECK(hipFree(d_ddsph));
    std::printf("device_example: ok\n");
    return 0;
}

int main(int argc, char** argv) {
    if (argc != 7) {
        std::fprintf(stderr, "usage: %s <f32|f64> <spherical|solid> <l_max> <n_samples> <xyz.bin> <out.bin>\n",
                     argv[0]);
        return 2;
    }
    const bool f64 = std::string(argv[1]) == "f64";
    const bool solid = std::string(argv[2]) == "solid";
    const size_t l_max = std::strtoul(argv[3], nullptr, 10);
    const size_t n = std::strtoul(argv[4], nullptr, 10);
    try {
        return f64 ? run<double>(solid, l_max, n, argv[5], argv[6]) : run<float>(solid, l_max, n, argv[5], argv[6]);
    } catch (const std::exception& e) {
        std::fprintf(stderr, "exception: %s\n", e.what());
        return 1;
    }
}
