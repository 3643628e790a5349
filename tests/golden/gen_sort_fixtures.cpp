// Writes the sort fixtures used by tests/test_oracle_sort.py and tests/test_gpu_units.py.
//
// Inputs follow the recipes of the reference's own sort tests, regenerated with libstdc++:
//   tests/test_bitonic.cu:73-80    mt19937(42), uniform_real_distribution<float>(0,100),
//                                  n = 64, 128, 256, value = index
//   tests/test_sort_impl.cu:64-81  mt19937(42), uniform_real_distribution<float>(0,1000),
//                                  n = 64, 128, 256, 512, value = index
// Expected output = std::sort of the (key,value) pairs, as in test_bitonic.cu:110-117.
// Build and run:  g++ -O1 -std=c++17 gen_sort_fixtures.cpp -o /tmp/gen && /tmp/gen > sort_fixtures.json
#include <algorithm>
#include <cstdint>
#include <cstdio>
#include <cstring>
#include <random>
#include <utility>
#include <vector>

static void emit(const char* name, float hi, int n, bool last) {
    std::mt19937 gen(42);
    std::uniform_real_distribution<float> dis(0.0f, hi);
    std::vector<std::pair<float, uint32_t>> v(n);
    for (int i = 0; i < n; ++i) v[i] = {dis(gen), (uint32_t)i};
    auto sorted = v;
    std::sort(sorted.begin(), sorted.end());
    auto bits = [](float f) { uint32_t u; std::memcpy(&u, &f, 4); return u; };
    std::printf("  {\"recipe\": \"%s\", \"n\": %d, \"hi\": %g,\n   \"key_bits\": [", name, n, hi);
    for (int i = 0; i < n; ++i) std::printf("%s%u", i ? "," : "", bits(v[i].first));
    std::printf("],\n   \"sorted_key_bits\": [");
    for (int i = 0; i < n; ++i) std::printf("%s%u", i ? "," : "", bits(sorted[i].first));
    std::printf("],\n   \"sorted_vals\": [");
    for (int i = 0; i < n; ++i) std::printf("%s%u", i ? "," : "", sorted[i].second);
    std::printf("]}%s\n", last ? "" : ",");
}

int main() {
    std::printf("[\n");
    for (int n : {64, 128, 256}) emit("test_bitonic", 100.0f, n, false);
    for (int n : {64, 128, 256, 512}) emit("test_sort_impl", 1000.0f, n, n == 512);
    std::printf("]\n");
    return 0;
}
