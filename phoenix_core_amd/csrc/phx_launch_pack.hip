// One launch that packs several filter images (PackJobs in phx_launch.h): every workgroup finds the job its index
// falls into and runs that packing kernel's body over the job's own index range.
#include "phx_kernels_pw16.h"
#include "phx_launch.h"

namespace phx {

template <int MODE, int MAP>
static __device__ __forceinline__ void pack_job_as(const PackJob& j, long first, long stride) {
    if (j.kind == PACK_F32) {
        if (j.half_storage) pack_filters_f32_body<_Float16, MODE, MAP>(j.a, first, stride);
        else pack_filters_f32_body<float, MODE, MAP>(j.a, first, stride);
    } else if (j.kind == PACK_F16) {
        pack_filters_f16_body<MODE, MAP>(j.a, first, stride);
    } else if (j.kind == PACK_F16_LDS) {
        const PackLdsArgs la{j.a, j.WCO, j.ngroups, j.pw};
        pack_filters_f16_lds_body<MODE, MAP>(la, first, stride);
    } else if (MODE == 16) {  // PACK_PWX (16-product form only)
        const PackPwxArgs pa{j.a, j.WCO, j.nsteps};
        pack_filters_pwx_body<MAP>(pa, first, stride);
    }
}

__global__ void __launch_bounds__(WG_THREADS) pack_jobs_kernel(const PackJobs J) {
    int k = 0;
    while (k + 1 < J.n && (int)blockIdx.x >= J.job[k + 1].block0) ++k;
    const PackJob& j = J.job[k];
    const long first = (long)((int)blockIdx.x - j.block0) * WG_THREADS + threadIdx.x;
    const long stride = (long)j.nblocks * WG_THREADS;
    if (j.mode == 16) {
        if (j.map == MAP_FWD) pack_job_as<16, MAP_FWD>(j, first, stride);
        else pack_job_as<16, MAP_DGRAD>(j, first, stride);
    } else {
        if (j.map == MAP_FWD) pack_job_as<8, MAP_FWD>(j, first, stride);
        else pack_job_as<8, MAP_DGRAD>(j, first, stride);
    }
}

int launch_pack_jobs(const PackJobs& jobs, hipStream_t st) {
    if (jobs.n <= 0) return 0;
    if (jobs.n > PACK_JOBS_MAX) return -1;
    const PackJob& last = jobs.job[jobs.n - 1];
    hipLaunchKernelGGL(pack_jobs_kernel, dim3(last.block0 + last.nblocks), dim3(WG_THREADS), 0, st, jobs);
    return 0;
}

}  // namespace phx
