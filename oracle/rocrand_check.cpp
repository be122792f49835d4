// TEST INFRASTRUCTURE ONLY.  Host-side calls into ROCm's rocRAND device header (its
// Philox4x32-10 engine is __host__ __device__): rocrand_init(seed, subsequence, offset)
// followed by one rocrand (the raw 32-bit draw), the library routine that takes the same
// three arguments as the curand_init behind the reference's sampler
// (craftax_full.cu:9732-9736) and weight init (:9123-9131).  tests/ hold cfo_philox_draw
// to it.  (rocrand_uniform is not compared: rocRAND maps the draw x to x * 2^-32 + 2^-32,
// cuRAND to x * 2^-32 + 2^-33.)
#include <cstdint>

#include <hip/hip_runtime.h>
#include <rocrand/rocrand_philox4x32_10.h>

extern "C" void cfo_rocrand_draws(uint64_t seed, const uint64_t* subsequence,
                                  const uint64_t* offset, int count, uint32_t* out) {
    for (int i = 0; i < count; i++) {
        rocrand_state_philox4x32_10 st;
        rocrand_init(seed, subsequence[i], offset[i], &st);
        out[i] = rocrand(&st);
    }
}
