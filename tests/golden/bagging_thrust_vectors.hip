// Generator of tests/golden/bagging_thrust_vectors.json: the indices that
// thrust::default_random_engine + thrust::uniform_int_distribution<int> produce for the bagging draws of the
// reference (src/thundergbm/row_sampler.cu:15-22), computed on the host with the thrust headers this ROCm
// image ships (rocThrust). Host code only; no GPU is touched.
//   hipcc -O2 -std=c++17 --offload-arch=gfx950 tests/golden/bagging_thrust_vectors.hip -o /tmp/bagvec
//   /tmp/bagvec > tests/golden/bagging_thrust_vectors.json
#include <thrust/random.h>

#include <cstdio>

int main() {
    const int seeds[] = {0, 1, 12345, 1804289383, 2147483646, 2147483647};
    const int sizes[] = {1, 7, 1000, 1605, 20000000};
    const int positions[] = {0, 1, 2, 3, 5, 63, 64, 999, 1604, 65535, 1000000, 19999999};
    std::printf("[\n");
    bool first = true;
    for (int seed : seeds)
        for (int n_instances : sizes) {
            std::printf("%s{\"seed\": %d, \"N\": %d, \"draws\": {", first ? "" : ",\n", seed, n_instances);
            first = false;
            bool f2 = true;
            for (int i : positions) {
                if (i >= n_instances) continue;
                thrust::default_random_engine rng(seed);
                thrust::uniform_int_distribution<int> uniform_dist(0, n_instances - 1);
                rng.discard(i);
                std::printf("%s\"%d\": %d", f2 ? "" : ", ", i, uniform_dist(rng));
                f2 = false;
            }
            std::printf("}}");
        }
    std::printf("\n]\n");
    return 0;
}
