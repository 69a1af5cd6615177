#include "dense.hpp"

namespace psig {

DenseChoice dense_choice(size_t, int64_t, int, bool, const int64_t *, int64_t, int64_t, int64_t, bool) {
    return DenseChoice{false, -1, 1, 0, 0};
}

template <typename T>
hipError_t launch_dense_forward(const T *, T *, const SigShape &, const LevelPlan &, const int64_t *,
                                const DenseChoice &, void *, hipStream_t) {
    return hipErrorNotSupported;
}
template <typename T>
hipError_t launch_dense_backward(const T *, const T *, const T *, T *, const SigShape &, const LevelPlan &,
                                 const int64_t *, const DenseChoice &, void *, hipStream_t) {
    return hipErrorNotSupported;
}

#define PSIG_INSTANTIATE(T)                                                                                  \
    template hipError_t launch_dense_forward<T>(const T *, T *, const SigShape &, const LevelPlan &,         \
                                                const int64_t *, const DenseChoice &, void *, hipStream_t);  \
    template hipError_t launch_dense_backward<T>(const T *, const T *, const T *, T *, const SigShape &,     \
                                                 const LevelPlan &, const int64_t *, const DenseChoice &,    \
                                                 void *, hipStream_t);
PSIG_INSTANTIATE(float)
PSIG_INSTANTIATE(double)
#undef PSIG_INSTANTIATE

}  // namespace psig
