// Job kernels.  A job is the work of one kernel launch as a struct: its arguments, `blocks` (how many 256-thread
// workgroups it needs) and `run(block)`, the body of one workgroup.  `job_kernel` runs one job; `job_pair_kernel`
// runs two independent jobs in a single grid, the first job's blocks first: the second job's blocks fill the machine
// while the first one drains, and the pause between two dependent launches of a stream is paid once.
//
// Wave priorities.  A job's workgroup computes its addresses, requests its input, works on it for a few thousand
// vector instructions and stores.  Eight such waves share a SIMD, and left alone they move in step: a new wave's few
// dozen address instructions queue behind seven neighbours' arithmetic, its loads go out late, and memory idles while
// the arithmetic runs and the reverse.  A job kernel therefore starts at the highest wave priority and the job calls
// job_requests_issued() once its loads are out (back to the lowest), so that a fresh wave's requests overtake the
// running waves' arithmetic.  Measured on several MI355X: forward quantizer of 8192 x 4096 19.4 -> 17.4-18.3 us,
// stochastic-rounding quantizer -4 to -6 %, inverse rotation -3 %, transposing and re-quantizing kernels -1 to -2 %;
// on two slower-clocked chips of the pool the forward quantizer was unchanged and the others gained the same.
// Priorities order waves of one SIMD only; results do not depend on them.
#pragma once
#include <hip/hip_runtime.h>

namespace qm {

__device__ __forceinline__ void job_starts() { __builtin_amdgcn_s_setprio(3); }
__device__ __forceinline__ void job_requests_issued() { __builtin_amdgcn_s_setprio(0); }
// before the final stores: a wave that is about to leave makes room for the next one sooner
__device__ __forceinline__ void job_stores_next() { __builtin_amdgcn_s_setprio(3); }

template <class A>
__global__ __launch_bounds__(256) void job_kernel(A a) {
    job_starts();
    a.run(blockIdx.x);
}

template <class A, class B>
__global__ __launch_bounds__(256) void job_pair_kernel(A a, B b) {
    job_starts();
    if (blockIdx.x < a.blocks) a.run(blockIdx.x);
    else b.run(blockIdx.x - a.blocks);
}

template <class A>
void launch_job(const A& job, hipStream_t stream) {
    job_kernel<<<dim3(job.blocks), dim3(256), 0, stream>>>(job);
}

template <class A, class B>
void launch_job_pair(const A& a, const B& b, hipStream_t stream) {
    job_pair_kernel<<<dim3(a.blocks + b.blocks), dim3(256), 0, stream>>>(a, b);
}

}  // namespace qm
