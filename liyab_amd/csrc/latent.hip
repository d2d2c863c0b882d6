// The cached row of latent attention: one compressed row a position, from which every head's keys
// and values are made.
//
// liyab_latent_store: c_t = src_t[col_off : col_off + rank] / sqrt(mean(.^2) + eps) * w (32-bit
// sums and scaling, rounded once to the cache's type), written to the token's place in the pages,
// cache [pages, 1, page_size, rank] at row slots[t] = page * page_size + offset. A slot outside
// [0, num_slots) is not written (rows behind the step's tokens carry -1). A wave a row.
#include "common.h"
#include "launchers.h"

namespace liyab {

template <typename T>
__global__ void __launch_bounds__(256)
latent_store_kernel(T* __restrict__ cache, const T* __restrict__ src, int64_t src_stride, int col_off, const float* __restrict__ w, float eps,
                    const int* __restrict__ slots, int n, int rank, uint32_t num_slots) {
    const int lane = threadIdx.x % kWave, t = blockIdx.x * (256 / kWave) + threadIdx.x / kWave;
    if (t >= n) return;
    const int slot = slots[t];
    if (static_cast<uint32_t>(slot) >= num_slots) return;
    const T* row = src + static_cast<int64_t>(t) * src_stride + col_off;
    float ss = 0.0f;
    for (int i = lane; i < rank; i += kWave) {
        const float v = to_float<T>(row[i]);
        ss += v * v;
    }
    const float scale = 1.0f / sqrtf(wave_sum(ss) / static_cast<float>(rank) + eps);
    T* dst = cache + static_cast<int64_t>(slot) * rank;
    for (int i = lane; i < rank; i += kWave) {
        float v = to_float<T>(row[i]) * scale;
        if (w != nullptr) v *= w[i];
        dst[i] = from_float<T>(v);
    }
}

}  // namespace liyab

using namespace liyab;

extern "C" int liyab_latent_store(void* cache, int dtype, const void* src, int64_t src_stride, int col_off, const float* w, float eps,
                                  const int* slots, int n, int rank, int page_size, int num_pages, hipStream_t stream) {
    LIYAB_REQUIRE(cache && src && slots, "latent_store: null pointer");
    LIYAB_REQUIRE(dtype == kF32 || dtype == kBF16, "latent_store: unknown dtype %d", dtype);
    LIYAB_REQUIRE(n >= 0 && rank > 0 && col_off >= 0 && src_stride >= col_off + rank && page_size > 0 && num_pages > 0, "latent_store: bad sizes");
    LIYAB_REQUIRE(static_cast<int64_t>(page_size) * num_pages < (1ll << 31), "latent_store: slots must fit 31 bits");
    if (n == 0) return 0;
    const uint32_t num_slots = static_cast<uint32_t>(page_size) * static_cast<uint32_t>(num_pages);
    const int grid = (n + 3) / 4;
    if (dtype == kF32)
        latent_store_kernel<float><<<grid, 256, 0, stream>>>(static_cast<float*>(cache), static_cast<const float*>(src), src_stride, col_off, w, eps,
                                                             slots, n, rank, num_slots);
    else
        latent_store_kernel<bf16_t><<<grid, 256, 0, stream>>>(static_cast<bf16_t*>(cache), static_cast<const bf16_t*>(src), src_stride, col_off, w,
                                                              eps, slots, n, rank, num_slots);
    return check_launch("latent_store");
}
