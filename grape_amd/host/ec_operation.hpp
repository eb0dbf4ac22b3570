// Host helpers around challenges and generators: the interface of the reference's
// include/ec_operation.cuh / src/ec_operation.cu.
#pragma once
#include <vector>
#include "fr.hpp"
#include "fr_tensor.hpp"

// N generators (scalars from Fr::random_element times the standard generator, derived on the GPU;
// the scalars are wiped afterwards) and the
// reference-format table out[w*N + i] = w*G_i, w < W, on the device
// (precompute_generators + naive_msm, src/ec_operation.cu:15-49).  `out` is device memory for
// W*N affine points.
std::vector<bn128> precompute_generators(uint N, uint W, affine_t* out);

std::vector<Fr> random_vec(uint len);                                             // src/ec_operation.cu:51-57
void generate_random_eval_points(size_t data_size, std::vector<Fr>& eval_point);  // :59-71
void ReassembleVectors(std::vector<Fr>& first, std::vector<Fr>& second, size_t first_size, size_t same_size,
                       size_t last_size);                                         // :74-122

// Host multilinear fold of an array of field elements or group elements, LSB first, missing
// partner of an odd tail = zero (include/ec_operation.cuh:38-57).
template <typename T>
T host_partial_me(T* points, uint inputsize, typename std::vector<Fr>::const_iterator begin,
                  typename std::vector<Fr>::const_iterator end) {
    if (begin >= end) return points[0];
    uint outputsize = (inputsize + 1) / 2;
    std::vector<T> next(outputsize);
    for (uint i = 0; i < outputsize; i++) {
        uint id0 = i * 2, id1 = i * 2 + 1;
        if (id1 < inputsize) next[i] = points[id0] + *begin * (points[id1] - points[id0]);
        else next[i] = points[id0] - *begin * points[id0];
    }
    return host_partial_me(next.data(), outputsize, begin + 1, end);
}
