// Host build of zenu_amd/csrc/zmath.hpp as a filter: zmath_host_eval <function> reads f32 values from
// stdin and writes the function's f32 results to stdout.  The GPU tests use it to show that a device
// function built from IEEE operations only returns the same bits on the device and on the host, so
// that what was checked exhaustively on the host holds for the kernel.
#include <cstdio>
#include <cstring>
#include <vector>

#include "../../zenu_amd/csrc/zmath.hpp"

int main(int argc, char **argv)
{
    if (argc != 2) return 2;
    float (*fn)(float) = nullptr;
    if (!strcmp(argv[1], "tanh_ulp2")) fn = [](float x) { return zmath::tanhf_ulp2(x); };
    else if (!strcmp(argv[1], "tanh")) fn = [](float x) { return zmath::tanhf_simd(x); };
    else if (!strcmp(argv[1], "sigmoid")) fn = [](float x) { return zmath::sigmoidf_zenu(x); };
    else return 2;
    std::vector<float> buf(1 << 16);
    size_t n;
    while ((n = fread(buf.data(), sizeof(float), buf.size(), stdin)) > 0) {
        for (size_t i = 0; i < n; i++) buf[i] = fn(buf[i]);
        if (fwrite(buf.data(), sizeof(float), n, stdout) != n) return 1;
    }
    return 0;
}
