// Job kernels.  A job is the work of one kernel launch as a struct: its arguments, `blocks` (how many 256-thread
// workgroups it needs) and `run(block)`, the body of one workgroup.  `job_kernel` runs one job; `job_pair_kernel`
// runs two independent jobs in a single grid, the first job's blocks first: the second job's blocks fill the machine
// while the first one drains, and the pause between two dependent launches of a stream is paid once.
#pragma once
#include <hip/hip_runtime.h>

namespace qm {

template <class A>
__global__ __launch_bounds__(256) void job_kernel(A a) {
    a.run(blockIdx.x);
}

template <class A, class B>
__global__ __launch_bounds__(256) void job_pair_kernel(A a, B b) {
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
