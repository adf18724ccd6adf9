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

int launch_patch_depth(bool half_storage, const PatchArgs& a0, bool to_caller, hipStream_t st) {
    if (a0.rows <= 0 || a0.C <= 0 || (long)a0.H * a0.W <= 0) return 0;
    PatchArgs a = a0;
    // channels per item: a power of two that divides C, for items of a few thousand elements
    const long per_channel = std::max((long)a.kw * a.Ho * a.Wo, (long)((a.H + a.kh - 1) / a.kh) * a.W);
    a.CB = 1;
    while (a.C % (a.CB * 2) == 0 && per_channel * a.CB * 2 <= 4096) a.CB *= 2;
    if (per_channel * a.CB >= (1L << 24)) return -1;  // the kernel divides an item's element counts in fp32
    const long items = a.rows * (a.C / a.CB) * a.kh;
    const dim3 grid((unsigned int)std::min<long>(items, 1L << 20));
    if (half_storage) hipLaunchKernelGGL((patch_depth_kernel<_Float16>), grid, dim3(WG_THREADS), 0, st, a, (int)to_caller);
    else hipLaunchKernelGGL((patch_depth_kernel<float>), grid, dim3(WG_THREADS), 0, st, a, (int)to_caller);
    return 0;
}

int launch_strided_gather(bool half_storage, const StridedGatherArgs& a, hipStream_t st) {
    const long items = a.planes * a.H2 * a.W2;
    if (items <= 0) return 0;
    if (half_storage) hipLaunchKernelGGL((strided_gather_kernel<_Float16>), dim3(blocks_for(items)), dim3(WG_THREADS), 0, st, a);
    else hipLaunchKernelGGL((strided_gather_kernel<float>), dim3(blocks_for(items)), dim3(WG_THREADS), 0, st, a);
    return 0;
}

int launch_dilation_phases(bool half_storage, const DilationPhaseArgs& a0, bool to_caller, hipStream_t st) {
    if (a0.rows <= 0 || a0.C <= 0 || a0.H <= 0 || a0.W <= 0) return 0;
    DilationPhaseArgs a = a0;
    // channels per item: a power of two that divides C, for items of a few thousand elements
    const long per_channel = (long)a.Hp * a.Wp * a.dw;
    a.CB = 1;
    while (a.C % (a.CB * 2) == 0 && per_channel * a.CB * 2 <= 4096) a.CB *= 2;
    // a workgroup's element count, divided in fp32: (Hp * max(Wp * dw, W)) * CB
    if (per_channel * a.CB >= (1L << 24) || (long)a.Hp * a.W * a.CB >= (1L << 24)) return -1;
    const long items = a.rows * (a.C / a.CB) * a.dh;
    const unsigned int blocks = (unsigned int)(items < (1L << 20) ? items : (1L << 20));
    if (half_storage)
        hipLaunchKernelGGL((dilation_phase_kernel<_Float16>), dim3(blocks), dim3(WG_THREADS), 0, st, a, (int)to_caller);
    else
        hipLaunchKernelGGL((dilation_phase_kernel<float>), dim3(blocks), dim3(WG_THREADS), 0, st, a, (int)to_caller);
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

int launch_merge_filter(bool half_storage, const MergeFilterArgs& a, bool to_caller, hipStream_t st) {
    const long items = 4L * a.Co * a.m * a.ci * a.Kh * a.Kw;
    if (items == 0) return 0;
    if (half_storage)
        hipLaunchKernelGGL((merge_filter_kernel<_Float16>), dim3(blocks_for(items)), dim3(WG_THREADS), 0, st, a, to_caller);
    else hipLaunchKernelGGL((merge_filter_kernel<float>), dim3(blocks_for(items)), dim3(WG_THREADS), 0, st, a, to_caller);
    return 0;
}

int launch_fill_zero(void* dst, size_t bytes, hipStream_t st) {
    if (bytes == 0) return 0;
    hipLaunchKernelGGL(fill_zero_kernel, dim3(blocks_for((long)((bytes + 15) / 16))), dim3(WG_THREADS), 0, st,
                       static_cast<unsigned char*>(dst), bytes);
    return 0;
}

// phase_merge_kernel for fp16 tensors with two column phases and fewer than 2^31 16-byte words in dx (32-bit index
// arithmetic): a word is four elements of each of the two phase rows that feed the dx row (two 8-byte runs of two
// buffers instead of eight 2-byte loads), interleaved in registers.
__global__ void __launch_bounds__(WG_THREADS) phase_merge_f16_sw2_kernel(const PhaseMergeArgs A) {
    const _Float16* buf = static_cast<const _Float16*>(A.buf);
    _Float16* dx = static_cast<_Float16*>(A.dx);
    const unsigned int cpr = (unsigned int)(A.W + 7) / 8u;
    const unsigned int total = (unsigned int)A.planes * (unsigned int)A.H * cpr;
    const int Wp0 = (A.W + 1) >> 1, Wp1 = A.W >> 1;
    for (unsigned int idx = blockIdx.x * blockDim.x + threadIdx.x; idx < total; idx += gridDim.x * blockDim.x) {
        const unsigned int r = idx / cpr;
        const int w0 = (int)(idx - r * cpr) * 8;
        const unsigned int plane = r / (unsigned int)A.H;
        const int h = (int)(r - plane * (unsigned int)A.H);
        const int a = h % A.sh, hp = h / A.sh;
        const int Hp = (A.H - a + A.sh - 1) / A.sh;
        const long o0 = A.off[a * 2], o1 = A.off[a * 2 + 1];
        const long row = (long)plane * Hp + hp;
        _Float16 v[8];
        if (w0 + 8 <= A.W) {
            f16x2 e01{}, e23{}, o01{}, o23{};
            if (o0 >= 0) {
                const _Float16* p = buf + o0 + row * Wp0 + (w0 >> 1);
                e01 = __builtin_bit_cast(f16x2, load4_a2(p));
                e23 = __builtin_bit_cast(f16x2, load4_a2(p + 2));
            }
            if (o1 >= 0) {
                const _Float16* p = buf + o1 + row * Wp1 + (w0 >> 1);
                o01 = __builtin_bit_cast(f16x2, load4_a2(p));
                o23 = __builtin_bit_cast(f16x2, load4_a2(p + 2));
            }
            v[0] = e01[0]; v[1] = o01[0]; v[2] = e01[1]; v[3] = o01[1];
            v[4] = e23[0]; v[5] = o23[0]; v[6] = e23[1]; v[7] = o23[1];
            u32x4 raw;
            __builtin_memcpy(&raw, v, 16);
            *reinterpret_cast<__attribute__((address_space(1))) u32x4_a2*>(
                (__attribute__((address_space(1))) _Float16*)(dx + (long)r * A.W + w0)) = raw;
        } else {
            for (int i = 0; w0 + i < A.W; ++i) {
                const int w = w0 + i, b = w & 1;
                const long o = b ? o1 : o0;
                dx[(long)r * A.W + w] = o >= 0 ? buf[o + row * (b ? Wp1 : Wp0) + (w >> 1)] : (_Float16)0;
            }
        }
    }
}

int launch_phase_merge(bool half_storage, const PhaseMergeArgs& a, hipStream_t st) {
    const long items = a.planes * a.H * ((a.W + 3) / 4);  // at most: 16-byte words
    if (items == 0) return 0;
    if (half_storage && a.sw == 2 && items < (1L << 31))
        hipLaunchKernelGGL(phase_merge_f16_sw2_kernel, dim3(blocks_for(a.planes * a.H * ((a.W + 7) / 8))), dim3(WG_THREADS), 0, st, a);
    else if (half_storage) hipLaunchKernelGGL((phase_merge_kernel<_Float16>), dim3(blocks_for(items)), dim3(WG_THREADS), 0, st, a);
    else hipLaunchKernelGGL((phase_merge_kernel<float>), dim3(blocks_for(items)), dim3(WG_THREADS), 0, st, a);
    return 0;
}

// dst[i] += src[i] in the tensors' own arithmetic (an fp16 sum is rounded once, like the elementwise add of a
// framework): what follows an input gradient that could not add its addend in its own epilogue.  16-byte words
// where both pointers allow it, element by element otherwise and for the tail.
template <typename TS>
__global__ void __launch_bounds__(WG_THREADS) add_inplace_kernel(TS* dst, const TS* src, long count) {
    constexpr int V = 16 / (int)sizeof(TS);
    const long stride = (long)gridDim.x * blockDim.x, tid = (long)blockIdx.x * blockDim.x + threadIdx.x;
    const bool aligned = ((reinterpret_cast<size_t>(dst) | reinterpret_cast<size_t>(src)) & 15) == 0;
    const long words = aligned ? count / V : 0;
    for (long i = tid; i < words; i += stride) {
        const u32x4 a = reinterpret_cast<const u32x4*>(dst)[i], b = reinterpret_cast<const u32x4*>(src)[i];
        u32x4 r;
        if constexpr (sizeof(TS) == 2) r = __builtin_bit_cast(u32x4, __builtin_bit_cast(f16x8, a) + __builtin_bit_cast(f16x8, b));
        else r = __builtin_bit_cast(u32x4, __builtin_bit_cast(f32x4, a) + __builtin_bit_cast(f32x4, b));
        reinterpret_cast<u32x4*>(dst)[i] = r;
    }
    for (long i = words * V + tid; i < count; i += stride) dst[i] = dst[i] + src[i];
}

int launch_add_inplace(bool half_storage, void* dst, const void* src, long count, hipStream_t st) {
    if (count <= 0) return 0;
    const int blocks = blocks_for((count + 7) / 8);
    if (half_storage)
        hipLaunchKernelGGL((add_inplace_kernel<_Float16>), dim3(blocks), dim3(WG_THREADS), 0, st, static_cast<_Float16*>(dst),
                           static_cast<const _Float16*>(src), count);
    else
        hipLaunchKernelGGL((add_inplace_kernel<float>), dim3(blocks), dim3(WG_THREADS), 0, st, static_cast<float*>(dst),
                           static_cast<const float*>(src), count);
    return 0;
}

// dst = sum of `slices` tensors of `count` elements each lying `count` elements apart (+ bias per channel: element e
// belongs to channel (e / plane) % channels of component e / comp_count; then + addend, element by element, in the storage
// type): what closes a forward / input-gradient pass whose reduction over the channels was cut into slices.  fp32 sums,
// one rounding.
template <typename TS>
__global__ void __launch_bounds__(WG_THREADS) slice_sum_kernel(const TS* partial, int slices, long count, TS* dst, const TS* bias,
                                                               const TS* addend, int plane, int channels, long comp_count) {
    const long stride = (long)gridDim.x * blockDim.x;
    for (long e = (long)blockIdx.x * blockDim.x + threadIdx.x; e < count; e += stride) {
        float acc = 0.0f;
        for (int z = 0; z < slices; ++z) acc += (float)partial[z * count + e];
        if (bias) acc += (float)bias[(e / comp_count) * channels + (e / plane) % channels];
        TS r = (TS)acc;
        if (addend) r = (TS)((float)r + (float)addend[e]);  // (as the separate in-place pass would: the rounded result plus the addend)
        dst[e] = r;
    }
}

int launch_slice_sum(bool half_storage, const void* partial, int slices, long count, void* dst, const void* bias, const void* addend,
                     int plane, int channels, long comp_count, hipStream_t st) {
    if (count <= 0) return 0;
    const int blocks = blocks_for(count);
    if (half_storage)
        hipLaunchKernelGGL((slice_sum_kernel<_Float16>), dim3(blocks), dim3(WG_THREADS), 0, st, static_cast<const _Float16*>(partial),
                           slices, count, static_cast<_Float16*>(dst), static_cast<const _Float16*>(bias),
                           static_cast<const _Float16*>(addend), plane, channels, comp_count);
    else
        hipLaunchKernelGGL((slice_sum_kernel<float>), dim3(blocks), dim3(WG_THREADS), 0, st, static_cast<const float*>(partial), slices,
                           count, static_cast<float*>(dst), static_cast<const float*>(bias), static_cast<const float*>(addend), plane,
                           channels, comp_count);
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
