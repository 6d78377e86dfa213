// TEST INFRASTRUCTURE ONLY.
//
// The reference builds its kept-index lists with std::random_shuffle driven by
// glibc rand() (StreamMaskedGEMM/perf/basic_nn.cu:697-718).  This file calls the
// real std::random_shuffle / std::sort of the C++ standard library shipped with
// the compiler, so that the plain-C restatement in tw_oracle.c (ora_mask_gen)
// can be checked against the library routine itself on the same rand() stream.
// It contains none of the reference's code: only the standard-library calls.
#include <algorithm>
#include <cstdint>
#include <cstdlib>
#include <vector>

extern "C" void ora_std_srand(unsigned seed) { std::srand(seed); }

extern "C" void ora_std_mask_gen(int n, int n_kept, int32_t *offsets)
{
    std::vector<int> keep(n);
    for (int i = 0; i < n; ++i)
        keep[i] = i;
    std::random_shuffle(keep.begin(), keep.end());
    std::vector<int> host(keep.begin(), keep.begin() + n_kept);
    std::sort(host.begin(), host.end());
    for (int i = 0; i < n_kept; ++i)
        offsets[i] = host[i] - i;
}
