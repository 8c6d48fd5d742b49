// Host check of the fp32 <-> fp16 conversions of mxq_core.h (the form a compiler without _Float16
// gets, or the _Float16 form under clang): reads fp32 values from argv[1], writes for each the
// fp16 bit pattern to argv[2] and the fp32 value of that pattern to argv[3].  The test compares
// both files with torch's own conversions.
#include <stdio.h>
#include <stdlib.h>

#include <vector>

#include "mxq_core.h"

int main(int argc, char** argv) {
    if (argc != 4) return 2;
    FILE* f = fopen(argv[1], "rb");
    if (!f) return 2;
    fseek(f, 0, SEEK_END);
    const long n = ftell(f) / 4;
    fseek(f, 0, SEEK_SET);
    std::vector<float> x(n);
    if (fread(x.data(), 4, n, f) != (size_t)n) return 2;
    fclose(f);
    std::vector<unsigned short> h(n);
    std::vector<float> back(n);
    for (long i = 0; i < n; ++i) {
        h[i] = mxq_f16_bits(x[i]);
        back[i] = mxq_f16_value(h[i]);
    }
    f = fopen(argv[2], "wb");
    fwrite(h.data(), 2, n, f);
    fclose(f);
    f = fopen(argv[3], "wb");
    fwrite(back.data(), 4, n, f);
    fclose(f);
    printf("%ld values converted\n", n);
    return 0;
}
