// Memory-safety run of the host build of the quantizers (mxq_host.cpp), compiled together with this file
// under AddressSanitizer and UndefinedBehaviorSanitizer: random shapes (empty, one element, ragged last
// tiles, tiles longer than the axis, several shared axes), all dtypes, formats, roundings and flags, with
// every buffer allocated at exactly the size the call describes, so that an index past the end of an
// operand is reported instead of reading a neighbour.  One call in 150 is large enough for the library's
// threads to start.  Also checked: a call that returns an error leaves the output untouched.
//
//   usage: host_abi_sanitize [seconds]      exit status 0 and "ok <calls>" when nothing was reported
#include <chrono>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <random>
#include <vector>

#include "mxq.h"

namespace {

std::mt19937_64 rng(12345);
int64_t pick(int64_t lo, int64_t hi) { return lo + (int64_t)(rng() % (uint64_t)(hi - lo + 1)); }

int elem_size(int dtype) { return dtype == MXQ_DTYPE_F32 ? 4 : 2; }

// n elements of `dtype` with arbitrary bit patterns (NaN, Inf, subnormals included), as a heap block of
// exactly n * size bytes
std::vector<unsigned char>* random_tensor(int64_t n, int dtype) {
    auto* v = new std::vector<unsigned char>((size_t)(n * elem_size(dtype)));
    for (auto& b : *v) b = (unsigned char)rng();
    return v;
}
// noise in [0, 1): bit patterns of 0 .. just below 1 in the dtype
std::vector<unsigned char>* noise_tensor(int64_t n, int dtype) {
    auto* v = new std::vector<unsigned char>((size_t)(n * elem_size(dtype)));
    for (int64_t i = 0; i < n; ++i) {
        if (dtype == MXQ_DTYPE_F32) {
            const float f = (float)(rng() % 16777216) / 16777216.0f;
            memcpy(v->data() + 4 * i, &f, 4);
        } else {
            const uint16_t top = dtype == MXQ_DTYPE_BF16 ? 0x3F80 : 0x3C00;      // 1.0
            const uint16_t h = (uint16_t)(rng() % top);
            memcpy(v->data() + 2 * i, &h, 2);
        }
    }
    return v;
}

struct Format { int ebits, mbits; float max_norm; };
const Format kFormats[] = {{4, 5, 448.0f}, {5, 4, 57344.0f}, {3, 4, 28.0f}, {2, 5, 7.5f}, {2, 3, 6.0f},
                           {0, 8, 1.984375f}, {0, 4, 1.75f}, {0, 2, 1.0f}, {8, 9, 3.3895313892515355e38f},
                           {5, 12, 65504.0f}, {1, 4, 1.75f}, {0, 6, 7.5f}};

long calls = 0, refused = 0;

void check(bool ok, const char* what) {
    if (!ok) {
        printf("FAILED: %s\n", what);
        exit(1);
    }
}

void one_call() {
    const int dtype = (int)pick(0, 2);
    const Format f = kFormats[pick(0, (int64_t)(sizeof(kFormats) / sizeof(kFormats[0])) - 1)];
    const int scale_bits = (int)pick(1, 8), rmode = (int)pick(0, 2), flush = (int)pick(0, 1);
    const int flags = (int)(pick(0, 3) == 0 ? pick(0, 3) : 0);                // exact exponent / every-op now and then
    const int kind = (int)pick(0, 5);
    int64_t n = 0;
    std::vector<unsigned char>*in = nullptr, *aux = nullptr;
    int rc = 0;
    std::vector<unsigned char>* out = nullptr;
    // now and then a call large enough for the library to spread it over several threads
    const bool big = pick(0, 150) == 0;
    if (kind <= 2) {                                                          // by tile, given max, dither by tile
        const int64_t pre = big ? pick(1, 40) : pick(0, 5), axis = big ? pick(200, 2000) : pick(0, 70),
                      post = big ? pick(1, 12) : pick(0, 9);
        int64_t tile = pick(-1, 80);
        n = pre * axis * post;
        in = random_tensor(n, dtype);
        out = new std::vector<unsigned char>(in->size(), 0xA5);
        if (kind == 0) {
            rc = mxq_host_quantize_mx_by_tile(in->data(), out->data(), dtype, pre, axis, post, scale_bits, f.ebits,
                                              f.mbits, f.max_norm, tile, flush, rmode, flags);
        } else if (kind == 1) {
            aux = random_tensor(pre * post, dtype);
            rc = mxq_host_quantize_mx_given_max(in->data(), out->data(), aux->data(), dtype, pre, axis, post,
                                                scale_bits, f.ebits, f.mbits, f.max_norm, flush, rmode, flags);
        } else {
            aux = noise_tensor(n, dtype);
            rc = mxq_host_quantize_mx_dither_by_tile(in->data(), aux->data(), out->data(), dtype, pre, axis, post,
                                                     scale_bits, f.ebits, f.mbits, f.max_norm, tile, flush, flags);
        }
    } else if (kind == 3) {                                                   // several shared axes
        const int n_axes = (int)pick(1, 3);
        int64_t ext[7];
        n = 1;
        for (int i = 0; i <= 2 * n_axes; ++i) {
            ext[i] = (i % 2 == 0) ? pick(1, 3) : pick(1, big ? 90 : 40);
            if (pick(0, 40) == 0) ext[i] = 0;
            n *= ext[i];
        }
        in = random_tensor(n, dtype);
        out = new std::vector<unsigned char>(in->size(), 0xA5);
        rc = mxq_host_quantize_mx_axes(in->data(), out->data(), dtype, n_axes, ext, scale_bits, f.ebits, f.mbits,
                                       f.max_norm, pick(-1, 48), flush, rmode, flags);
    } else {                                                                  // elementwise, plain and dither
        n = big ? pick(200000, 600000) : pick(0, 3000);
        const int bits = (int)pick(2, 24), exp_bits = (int)pick(0, 8), sat = (int)pick(0, 1), den = (int)pick(0, 1);
        const float max_norm = pick(0, 1) ? f.max_norm : 1.5f * (float)(1 << pick(0, 20));
        in = random_tensor(n, dtype);
        out = new std::vector<unsigned char>(in->size(), 0xA5);
        if (kind == 4) {
            rc = mxq_host_quantize_elemwise(in->data(), out->data(), dtype, n, bits, exp_bits, max_norm, rmode, sat, den,
                                            flags);
        } else {
            aux = noise_tensor(n, dtype);
            rc = mxq_host_quantize_elemwise_dither(in->data(), aux->data(), out->data(), dtype, n, bits, exp_bits,
                                                   max_norm, sat, den, flags);
        }
    }
    ++calls;
    if (rc != MXQ_OK) {
        ++refused;
        check(mxq_host_last_error()[0] != 0, "an error code without a message");
        for (unsigned char b : *out) check(b == 0xA5, "a refused call wrote to the output");
    }
    delete in;
    delete aux;
    delete out;
}

}  // namespace

int main(int argc, char** argv) {
    const double seconds = argc > 1 ? atof(argv[1]) : 20.0;
    const auto t0 = std::chrono::steady_clock::now();
    while (std::chrono::duration<double>(std::chrono::steady_clock::now() - t0).count() < seconds)
        for (int i = 0; i < 20; ++i) one_call();
    check(refused * 2 < calls, "more than half of the calls were refused: the driver's parameters are off");
    printf("ok %ld calls, %ld refused with a message\n", calls, refused);
    return 0;
}
