// Launchers of the rearrangement kernels (space-to-depth, phase merge, channels-last transposes) and of the zero fill.
#include "phx_kernels_s2d.h"
#include "phx_launch.h"

namespace phx {

// Zero fill by a kernel: unlike a memset node it replays correctly when the caller captures the stream in a graph.
__global__ void __launch_bounds__(WG_THREADS) fill_zero_kernel(unsigned char* dst, size_t bytes) {
    const size_t words = bytes / 16;
    u32x4* d16 = reinterpret_cast<u32x4*>(dst);
    const bool aligned = (reinterpret_cast<size_t>(dst) & 15) == 0;
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    const size_t tid = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (aligned) {
        for (size_t i = tid; i < words; i += stride) d16[i] = u32x4{0u, 0u, 0u, 0u};
        for (size_t i = words * 16 + tid; i < bytes; i += stride) dst[i] = 0;
    } else {
        for (size_t i = tid; i < bytes; i += stride) dst[i] = 0;
    }
}

static int blocks_for(long items) { return (int)std::min<long>((items + WG_THREADS - 1) / WG_THREADS, 1 << 16); }

int launch_s2d_input(bool half_storage, const S2dArgs& a, hipStream_t st) {
    const long items = a.planes * a.H2 * ((a.W2 + 3) / 4);
    if (half_storage) hipLaunchKernelGGL((s2d_input_kernel<_Float16>), dim3(blocks_for(items)), dim3(WG_THREADS), 0, st, a);
    else hipLaunchKernelGGL((s2d_input_kernel<float>), dim3(blocks_for(items)), dim3(WG_THREADS), 0, st, a);
    return 0;
}

int launch_subsample(bool half_storage, const SubsampleArgs& a, hipStream_t st) {
    const long items = a.planes * a.H2 * ((a.W2 + 7) / 8);
    if (half_storage) hipLaunchKernelGGL((subsample_kernel<_Float16>), dim3(blocks_for(items)), dim3(WG_THREADS), 0, st, a);
    else hipLaunchKernelGGL((subsample_kernel<float>), dim3(blocks_for(items)), dim3(WG_THREADS), 0, st, a);
    return 0;
}

int launch_s2d_filter(bool half_storage, const S2dFilterArgs& a, bool to_caller, hipStream_t st) {
    const long items = 4L * a.Co * 4 * a.Ci * a.K2h * a.K2w;
    if (half_storage)
        hipLaunchKernelGGL((s2d_filter_kernel<_Float16>), dim3(blocks_for(items)), dim3(WG_THREADS), 0, st, a, to_caller);
    else hipLaunchKernelGGL((s2d_filter_kernel<float>), dim3(blocks_for(items)), dim3(WG_THREADS), 0, st, a, to_caller);
    return 0;
}

int launch_fill_zero(void* dst, size_t bytes, hipStream_t st) {
    if (bytes == 0) return 0;
    hipLaunchKernelGGL(fill_zero_kernel, dim3(blocks_for((long)((bytes + 15) / 16))), dim3(WG_THREADS), 0, st,
                       static_cast<unsigned char*>(dst), bytes);
    return 0;
}

int launch_phase_merge(bool half_storage, const PhaseMergeArgs& a, hipStream_t st) {
    const long items = a.planes * a.H * ((a.W + 3) / 4);  // at most: 16-byte words
    if (items == 0) return 0;
    if (half_storage) hipLaunchKernelGGL((phase_merge_kernel<_Float16>), dim3(blocks_for(items)), dim3(WG_THREADS), 0, st, a);
    else hipLaunchKernelGGL((phase_merge_kernel<float>), dim3(blocks_for(items)), dim3(WG_THREADS), 0, st, a);
    return 0;
}

int launch_transpose(bool half_storage, const TransposeArgs& a, hipStream_t st) {
    const int T = half_storage ? 64 : 32;  // tile edge of one wave
    const long tiles = a.batch * ((a.R + T - 1) / T) * ((a.Cc + T - 1) / T);
    if (tiles == 0) return 0;
    const int blocks = (int)std::min<long>((tiles + 3) / 4, 1 << 16);
    if (half_storage) hipLaunchKernelGGL((transpose_kernel<_Float16>), dim3(blocks), dim3(WG_THREADS), 0, st, a);
    else hipLaunchKernelGGL((transpose_kernel<float>), dim3(blocks), dim3(WG_THREADS), 0, st, a);
    return 0;
}

}  // namespace phx
