// Host-side launch interface between the C ABI translation unit and the translation units that
// instantiate the kernel templates (split so that they compile in parallel).
#pragma once

#include "../../include/phx_qconv.h"
#include "phx_kernels_f32.h"
#include "phx_kernels_realx.h"
#include "phx_kernels_s2d.h"

namespace phx {

// Kernels that need more dynamic LDS than the default 64 KiB must opt in with hipFuncSetAttribute.  That call does
// not belong inside a launch (a launch may sit in a stream capture, and a first-use flag would be shared by
// threads): every such kernel registers itself while the library loads, and the opt-in is applied to all of them
// once per device by phx_init() or by the first compute call made with that device current.
bool register_big_lds_kernel(const void* fn);
template <auto Kernel>
struct BigLds {
    static inline const bool registered = register_big_lds_kernel(reinterpret_cast<const void*>(Kernel));
};

// grid rows of a launch that runs every group of a grouped convolution (one row otherwise)
inline unsigned int grid_rows(int groups) { return groups > 1 ? (unsigned int)groups : 1u; }

bool tuning_noearly();  // PHX_TUNE_NOEARLY, read once with the other planner overrides
bool tuning_thin_notile();  // PHX_TUNE_THIN_NOTILE

// which instantiation of the forward / input-gradient kernel to run
struct FwdVariant {
    bool half_storage;  // tensors are fp16 (else fp32)
    bool f16_mfma;      // fp16 matrix-core arithmetic (else fp32)
    int mode, map;      // 16 / 8, MAP_FWD / MAP_DGRAD
    int WCO, NTW, CK, P2LOG;
    bool lds_filters;   // fp16 MFMA only: filters staged through LDS (qconv_fwd_f16_lds_kernel)
    int ngroups;        // tap groups per chunk for that kernel
    bool vstage;        // fp32 MFMA: activations staged as groups of 4 positions (no zero insertion)
    bool pairs;         // fp16 MFMA: activations staged as aligned position pairs
    bool chunks;        // fp16 MFMA, filters in LDS: activations staged as 8-position chunks
    int pw;             // pointwise convolution run as a column of pw virtual taps over 16-channel sub-chunks (0 = off)
    int wgs;
    size_t lds_bytes;
};

int launch_pack_filters(const FwdVariant& v, const PackArgs& a, int blocks, hipStream_t st);
int launch_fwd_f32(const FwdVariant& v, const ConvArgs& a, hipStream_t st);
int launch_fwd_f16(const FwdVariant& v, const ConvArgs& a, hipStream_t st);
int launch_fwd_f16_lds8(const FwdVariant& v, const ConvArgs& a, hipStream_t st);  // 8-product, filters through LDS
int launch_fwd_f16_lds16_real(const FwdVariant& v, const ConvArgs& a, hipStream_t st);  // 16-product, chunk staging, real-valued input
int launch_pack_filters_f16(const FwdVariant& v, const PackArgs& a, int blocks, hipStream_t st);

// pointwise fp16-MFMA kernels with raw operand copies (phx_kernels_pw16.h); WCO = 32-channel sub-tiles per workgroup
struct PwxArgs;
int launch_pwx_f16(int WCO, const PwxArgs& a, int blocks, hipStream_t st);
int launch_pwr_f16(int WCO, const PwxArgs& a, int blocks, hipStream_t st);  // packed filter resident in LDS
size_t pwr_lds_bytes(int WCO, int nsteps);
int launch_pwx_nhwc_f16(int WCO, const PwxArgs& a, int blocks, hipStream_t st);  // channels-last tensors
size_t pwx_packed_bytes(int WCO, int co_tiles, int nsteps);
int launch_pack_filters_pwx(int map, int WCO, int nsteps, const PackArgs& a, hipStream_t st);

// Several filter images packed by one launch (phx_launch_pack.hip): a convolution's forward and input-gradient
// images, the sub-filters of a strided input gradient's phases, the groups of a grouped convolution.  A job is one
// call of one of the packing kernels above; the workgroups of the launch are dealt to the jobs in order.
enum PackKind { PACK_F32 = 0, PACK_F16 = 1, PACK_F16_LDS = 2, PACK_PWX = 3 };
struct PackJob {
    PackArgs a;
    int kind;                    // PackKind
    int half_storage;            // PACK_F32: the filter is stored as fp16
    int mode, map;               // 16 / 8, MAP_FWD / MAP_DGRAD
    int WCO, ngroups, pw;        // PACK_F16_LDS (PackLdsArgs), PACK_PWX (WCO)
    int nsteps;                  // PACK_PWX
    int block0, nblocks;         // this job's workgroups: [block0, block0 + nblocks)
};
constexpr int PACK_JOBS_MAX = 12;
struct PackJobs {
    int n;
    PackJob job[PACK_JOBS_MAX];
};
int launch_pack_jobs(const PackJobs& jobs, hipStream_t st);

// wave sets (reduction slices) per workgroup of the fp32-MFMA filter-gradient kernel
constexpr int wgrad_f32_ksets(int mode, bool vec) { return (mode == 8 && vec) ? 2 : 1; }
int launch_wgrad_f32(bool half_storage, bool vec, int mode, const WgradArgs& a, dim3 grid, size_t lds_bytes,
                     hipStream_t st);  // vec: windows staged as groups of 4 positions
// fp16-MFMA filter gradient: channel tile 32*MT x 32*NT, TPW taps per workgroup (1 or 3), stride SW along W (1 or 2)
int launch_wgrad_f16(int mode, int MT, int NT, int TPW, int SW, const WgradArgs& a, int nblocks, size_t lds_bytes,
                     hipStream_t st);
int launch_wgrad_f16_p16(int MT, int NT, int TPW, int SW, const WgradArgs& a, int nblocks, size_t lds_bytes, hipStream_t st);
int launch_wgrad_f16_p16t3(int MT, int NT, const WgradArgs& a, int nblocks, size_t lds_bytes, hipStream_t st);
// real-valued input, few channels: the whole filter gradient as one matrix product (phx_kernels_realx.h)
int launch_wgrad_f16_cl(int TPW, const WgradArgs& a, int nblocks, size_t lds_bytes, hipStream_t st);  // channels-last tensors
int launch_wgrad_f16_realx(const RealWgArgs& a, int nblocks, size_t lds_bytes, hipStream_t st);
int launch_wgrad_f16_p8(int MT, int NT, int SW, const WgradArgs& a, int nblocks, size_t lds_bytes, hipStream_t st);
int launch_reduce_wgrad(bool half_storage, const ReduceArgs& a, hipStream_t st);

// Dense on fp32 FMA threads for small problems (phx_launch_dense_small.hip); (a, b) = (x, w) forward, (grad, w) input
// gradient, (x, grad) filter gradient; filter element (r, i, o) at r * wcs + o * so + i * si
struct DenseSmallArgs {
    const void* a;
    const void* b;
    const void* bias;  // forward only, or null
    void* out;
    long wcs, so, si;
    int n, ni, no;
};
int launch_dense_small(bool half_storage, int pass, const DenseSmallArgs& a, hipStream_t st);

// Grouped convolutions with very few channels per group (depthwise and the like) on fp32 FMA threads, on the caller's
// channels-first tensors and filter (phx_launch_thin.hip).  in = x (forward, filter gradient) or the output gradient
// (input gradient); out = y, dx or dw.  Filter element (r, co, i, kh, kw), co over all groups and i inside its group,
// at r * wcs + co * so + i * si + kh * skh + kw * skw.
struct ThinDiv {  // t / d == umulhi(t, m) + (t & one): m = ceil(2^32 / d), one = 0, or m = 0, one = ~0 for d == 1; exact while t * d < 2^32
    unsigned int m, one;
};
struct ThinArgs {
    const void* in;
    const void* w;
    const void* bias;  // forward: [4][all output channels] or null
    void* out;
    const void* grad;  // filter gradient: the output gradient
    float* partial;    // filter gradient: [Z][output channel x input channel of its group][tap][4] partial sums
    long wcs, so, si, skh, skw;
    int N, groups, cig, cog;  // images, groups, input / output channels of one group
    int H, W, Ho, Wo;         // input and output image of the forward pass
    int Kh, Kw, sh, sw, dh, dw, pt, pl;
    int Z;                    // filter gradient: slices of the images summed by separate workgroups
    int real_x;               // x is real-valued: [N][channels][H][W], its imaginary components are zero and not stored
    unsigned int mh, mw;      // strided input gradient: ceil(2^32 / sh), ceil(2^32 / sw); 0 for a unit stride
    int kchunk;               // per-tap forward / input gradient (set by launch_thin): filters per LDS chunk
    // the tiled kernels (set by launch_thin): a workgroup works on R output rows of J images from a window tile of
    // J x rows x cols entries in LDS; bands = such tiles per image group; d_* = the divisions they make
    int tile_R, tile_J, tile_rows, tile_cols, tile_bands;
    int tile_row0, tile_col0;  // strided input gradient by phases: the tile's first row / column relative to its first output block
    ThinDiv d_cols, d_rows, d_wout, d_R;
};
// < 0: not launched; 1: ran on the kernel that stages window tiles in LDS, 2: the strided input gradient by phases from
// such tiles; 0 otherwise
int launch_thin(bool half_storage, int pass, const ThinArgs& a, hipStream_t st);
int thin_wgrad_slices(bool half_storage, const ThinArgs& a);  // Z of the filter gradient (sizes `partial`)

// space-to-depth rearrangements (stride-2 convolutions with very few input channels)
int launch_s2d_input(bool half_storage, const S2dArgs& a, hipStream_t st);
int launch_subsample(bool half_storage, const SubsampleArgs& a, hipStream_t st);
int launch_patch_depth(bool half_storage, const PatchArgs& a, bool to_caller, hipStream_t st);  // the patches of a stride == filter convolution as channels
int launch_strided_gather(bool half_storage, const StridedGatherArgs& a, hipStream_t st);  // the input positions of one residue class of taps
int launch_dilation_phases(bool half_storage, const DilationPhaseArgs& a, bool to_caller, hipStream_t st);  // phase images of a dilated convolution
int launch_s2d_filter(bool half_storage, const S2dFilterArgs& a, bool to_caller, hipStream_t st);
int launch_phase_merge(bool half_storage, const PhaseMergeArgs& a, hipStream_t st);
int launch_merge_filter(bool half_storage, const MergeFilterArgs& a, bool to_caller, hipStream_t st);  // block-diagonal filters of merged groups
// batched matrix transposes between channels-last tensors and the kernels' channels-first layout
int launch_transpose(bool half_storage, const TransposeArgs& a, hipStream_t st);
int launch_fill_zero(void* dst, size_t bytes, hipStream_t st);  // a kernel, so that it can be captured in a graph
int launch_add_inplace(bool half_storage, void* dst, const void* src, long count, hipStream_t st);  // dst += src
// dst = the sum of `slices` partial tensors of `count` elements (+ bias of the element's channel, + addend); partial results
// of a pass whose channel reduction was cut into slices
int launch_slice_sum(bool half_storage, const void* partial, int slices, long count, void* dst, const void* bias, const void* addend,
                     int plane, int channels, long comp_count, hipStream_t st);

// REAL / COMPLEX / GA_300 as compositions on the quaternion entry points (phx_algebra.hip); pass = phx_pass,
// (a, b) = (x, w) forward, (grad, w) input gradient, (x, grad) filter gradient
size_t algebra_conv_workspace_bytes(const phx_qconv_desc* d, int pass);
size_t algebra_dense_workspace_bytes(const phx_qdense_desc* d, int pass);
int algebra_conv_pass(const phx_qconv_desc* d, int pass, phx_stream_t stream, const void* a, const void* b,
                      const void* bias, void* out, void* ws, size_t ws_bytes);
int algebra_dense_pass(const phx_qdense_desc* d, int pass, phx_stream_t stream, const void* a, const void* b,
                       const void* bias, void* out, void* ws, size_t ws_bytes);

}  // namespace phx
