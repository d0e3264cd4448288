// Host-only driver for tests/test_host_sanitizers.py, built with -fsanitize=address,undefined: the
// bundle reader's JSON parser and bounds checks (QW/src/weights.cpp:22-140 is what it stands for)
// against thousands of damaged meta files, and the two quantisers on edge inputs.  Prints a
// summary; any sanitizer report fails the test.
#include "mi_linear.h"
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <string>
#include <vector>
#include <random>
extern "C" {   // the device half of the library is not linked here
void* mi_malloc(size_t) { return nullptr; }
int mi_free(void*) { return 1; }
int mi_memcpy_h2d(void*, const void*, size_t, void*) { return 0; }
int mi_register_int8_weight(const void*, const void*, int, int) { return 0; }
int mi_register_q4_weight(const void*, const void*, int, int) { return 0; }
int mi_unregister_weight(const void*) { return 0; }
}
static void write(const char* p, const std::string& s) { FILE* f = fopen(p, "wb"); fwrite(s.data(), 1, s.size(), f); fclose(f); }
int main(int argc, char** argv) {
    const std::string dir = argc > 1 ? argv[1] : "/tmp";
    const std::string bin_path = dir + "/b.bin", meta_path = dir + "/m.json", meta2_path = dir + "/m2.json";
    std::mt19937 rng(7);
    // quantisers: zero rows, subnormals, inf/nan, max values, K not multiple of 32 for q4
    for (int K : {32, 64, 96, 896, 4864}) {
        const int N = 7;
        std::vector<uint16_t> w(N * K);
        for (auto& v : w) v = static_cast<uint16_t>(rng());
        for (int k = 0; k < K; ++k) w[k] = 0;                      // a zero row
        std::vector<int8_t> q(N * K); std::vector<uint16_t> s(N), s4(N * (K / 32)); std::vector<uint8_t> p(N * K / 2);
        mi_quantize_int8(w.data(), N, K, q.data(), s.data());
        mi_quantize_q4(w.data(), N, K, p.data(), s4.data());
    }
    std::vector<uint16_t> w(5 * 40); std::vector<uint8_t> p(5 * 20); std::vector<uint16_t> s4(5 * 2);
    printf("q4 with K = 40: rc %d (expected refusal)\n", mi_quantize_q4(w.data(), 5, 40, p.data(), s4.data()));
    // bundle: a good file, then mutations of its meta
    std::string bin(4096, 'x');
    write(bin_path.c_str(), bin);
    const std::string good = R"({"model_id": "m", "format": "binary", "tensors": {"a.weight": {"offset": 0, "shape": [4, 8], "dtype": "float16", "num_elements": 32, "size_bytes": 64}, "b.weight": {"offset": 64, "shape": [8, 16], "dtype": "int8", "num_elements": 128, "size_bytes": 128}, "b.weight.scale": {"offset": 192, "shape": [8], "dtype": "float16", "num_elements": 8, "size_bytes": 16}}})";
    write(meta_path.c_str(), good);
    void* b = mi_bundle_open(bin_path.c_str(), meta_path.c_str());
    printf("good bundle: %p, %d tensors\n", b, mi_bundle_count(b));
    for (int i = 0; i < mi_bundle_count(b); ++i) {
        const void* hp; size_t nb; int shape[8]; int rank; const char* dt;
        (void)hp; (void)nb; (void)shape; (void)rank; (void)dt;
        printf("  %s\n", mi_bundle_name(b, i));
    }
    mi_bundle_close(b);
    int opened = 0, refused = 0;
    for (int it = 0; it < 6000; ++it) {
        std::string m = good;
        const int kind = rng() % 6;
        if (kind == 0) m.resize(rng() % m.size());                                     // truncated
        else if (kind == 1) m[rng() % m.size()] = static_cast<char>(rng());              // a random byte
        else if (kind == 2) m.erase(rng() % m.size(), 1 + rng() % 8);                    // a hole
        else if (kind == 3) m.insert(rng() % m.size(), std::string(1 + rng() % 5, "{}[]\",:0-9e.\\"[rng() % 14]));
        else if (kind == 4) { size_t at = m.find("\"offset\": 64"); m.replace(at + 10, 2, std::to_string(rng() % 2 ? 1u << 31 : 5000)); }
        else { size_t at = m.find("\"size_bytes\": 128"); m.replace(at + 14, 3, std::to_string((rng() % 2) ? 99999999999ull : 4090)); }
        write(meta2_path.c_str(), m);
        void* h = mi_bundle_open(bin_path.c_str(), meta2_path.c_str());
        if (h) { ++opened; for (int i = 0; i < mi_bundle_count(h); ++i) (void)mi_bundle_name(h, i); mi_bundle_close(h); } else ++refused;
    }
    printf("mutated metas: %d opened, %d refused\n", opened, refused);
    return 0;
}
