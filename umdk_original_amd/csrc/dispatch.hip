// Token permutation with fused per-token int8 quantisation (bandwidth-bound).
//
// Reference semantics (paths relative to the reference tree):
//   send side   src/cam/comm_operator/ascend_kernels/moe_dispatch_normal/op_kernel/moe_dispatch_normal.h:330-396
//   quant       the same file :278-316 (scale = 127/(max|x| + 1e-12)), and the fused kernel's QuantToken,
//               src/cam/comm_operator/ascend_kernels/fused_deep_moe/op_kernel/fused_deep_moe/gemm/kernel/
//               grouped_matmul_slice_m_per_token_dequant_swiglu_quant_multistage_workspace.h:780-818 (no epsilon)
//   receive     moe_dispatch_normal.h:486-535 (rows land at recvCount[i-1] + j; triple and scale per row)
//
// Design.  The reference reads a token once per top-k copy and moves every row twice (sender ->
// window -> output).  Here one wavefront owns one token: lane l loads the 16-byte chunks l, l+64, ...
// of the row (each load instruction covers 1 KB of contiguous memory) exactly once, the row maximum
// is reduced with wave shuffles alone (no LDS, no workgroup barrier, so waves never wait for each
// other), the row is quantised in registers and each chunk's 8 result bytes are stored, again 512
// contiguous bytes per instruction, to each of the K destination rows.  HBM traffic is the
// algorithmic minimum: H*2 bytes read and K*H bytes written per token.
#include "cam_device.h"
#include "cam_kernels.h"
#include "permute_device.h"
#include "sched_device.h"

namespace cam {

namespace {

// Output row of entry (t,k), or -1.
__device__ __forceinline__ long long dispatch_row(const DispatchArgs &a, int t, int k)
{
    const long long i = (long long)t * a.K + k;
    if (a.dst_row != nullptr) {
        return a.dst_row[i];
    }
    const int e = a.idx[i];
    if (e < 0 || e >= a.E) {
        return -1;
    }
    const long long window_row = (long long)a.send_offset[e] + a.send_token_idx[i];
    const long long pre = e == 0 ? 0 : a.recv_count[e - 1];
    return pre + (window_row - a.recv_offset[e]);
}

// Four workgroups per CU (128 registers a lane) keep all 1024 workgroups of a 4096-token batch resident at once;
// the FP8 variant would spill at that size and stays at three.
template <int QUANT, int ACT>
__global__ __launch_bounds__(kDispWaves * kWave, QUANT == 3 ? 3 : 4) void dispatch_kernel(DispatchArgs a)
{
    // The first workgroups of the launch build the GEMM schedules (they start first and finish under the row
    // traffic of the others); they depend on nothing this launch writes.
    __shared__ SchedShared sched_s;
    const int builders = a.sched.nspec * a.sched.parts;
    if ((int)blockIdx.x < builders) {
        build_sched_part<kDispWaves * kWave>(sched_s, a.sched, (int)blockIdx.x / a.sched.parts,
                                             (int)blockIdx.x % a.sched.parts, a.sched.parts);
        return;
    }
    const int t = ((int)blockIdx.x - builders) * kDispWaves + (threadIdx.x >> 6);
    const int lane = threadIdx.x & (kWave - 1);
    if (t >= a.T) {
        return;
    }
    TokenRow r;
    load_token_row(a.x, t, a.H, lane, r);
    if (QUANT != 0) {
        quant_token_row<QUANT, ACT>(r);
    }
    for (int k = 0; k < a.K; ++k) {
        const long long row = dispatch_row(a, t, k);
        if (row < 0 || row >= a.A) {
            continue;
        }
        store_token_row<QUANT>(r, a.out, a.scales, a.src_info, a.src_rank, row, t, k, a.H, lane);
    }
}

// The quantising permute with per-expert smooth scales: every copy of a token is quantised on its own, under the
// scale row of its destination expert (moe_dispatch_shmem.h:492-549,693-733).  One wave per token; the token row
// is loaded once and stays in registers across its copies.
template <int ACT>
__global__ __launch_bounds__(kDispWaves * kWave) void dispatch_smooth_kernel(DispatchArgs a)
{
    const int t = (int)blockIdx.x * kDispWaves + (threadIdx.x >> 6);
    const int lane = threadIdx.x & (kWave - 1);
    if (t >= a.T) {
        return;
    }
    TokenRow r;
    load_token_row(a.x, t, a.H, lane, r);
    for (int k = 0; k < a.K; ++k) {
        const long long row = dispatch_row(a, t, k);
        const int e = a.idx[(long long)t * a.K + k];
        if (row < 0 || row >= a.A || e < 0 || e >= a.E) {
            continue;
        }
        quant_token_row_smooth<ACT>(r, a.smooth + (long long)e * a.H, a.H, lane);
        store_token_row<2>(r, a.out, a.scales, a.src_info, a.src_rank, row, t, k, a.H, lane);
    }
}

}  // namespace

hipError_t launch_dispatch(const DispatchArgs &a_in, hipStream_t stream)
{
    if (a_in.T <= 0) {
        if (a_in.sched.nspec > 0) {  // no rows to move, but the schedules are still owed
            return launch_build_sched(a_in.sched.group_list, a_in.sched.cumulative, a_in.sched.G, a_in.sched.max_rows,
                                      a_in.sched.nspec, a_in.sched.spec, stream);
        }
        return hipSuccess;
    }
    const DispatchArgs &a0 = a_in;
    if (a0.H % 8 != 0 || a0.H / 8 > kDispMaxChunks * kWave || (a0.quant == 3 && a0.H % 128 != 0)) {
        return hipErrorInvalidValue;
    }
    DispatchArgs a = a_in;
    if (a.sched.nspec != 0) {
        if (a.sched.nspec < 0 || a.sched.nspec > 2 || a.sched.G <= 0 || a.sched.G > kMaxExperts ||
            a.sched.group_list == nullptr) {
            return hipErrorInvalidValue;
        }
        const hipError_t qe = gemm_workgroups(&a.sched.queues);
        if (qe != hipSuccess) {
            return qe;
        }
        // a turn of items per builder workgroup where the item tables could be full
        const int cap = max(a.sched.spec[0].max_items, a.sched.spec[a.sched.nspec - 1].max_items);
        a.sched.parts = min(max((cap + kDispWaves * kWave - 1) / (kDispWaves * kWave), 1), 8);
    } else {
        a.sched.parts = 1;
    }
    dim3 grid((a.T + kDispWaves - 1) / kDispWaves + a.sched.nspec * a.sched.parts), block(kDispWaves * kWave);
    if (a.smooth != nullptr) {
        if (a.quant != 2 || a.idx == nullptr || a.sched.nspec != 0) {
            return hipErrorInvalidValue;
        }
        if (a.x_is_fp16) {
            hipLaunchKernelGGL((dispatch_smooth_kernel<1>), grid, block, 0, stream, a);
        } else {
            hipLaunchKernelGGL((dispatch_smooth_kernel<0>), grid, block, 0, stream, a);
        }
        return hipGetLastError();
    }
    if (a.quant == 0) {
        hipLaunchKernelGGL((dispatch_kernel<0, 0>), grid, block, 0, stream, a);  // a copy does not look at the format
    } else if (a.quant == 1) {
        if (a.x_is_fp16) {
            hipLaunchKernelGGL((dispatch_kernel<1, 1>), grid, block, 0, stream, a);
        } else {
            hipLaunchKernelGGL((dispatch_kernel<1, 0>), grid, block, 0, stream, a);
        }
    } else if (a.quant == 3) {
        if (a.x_is_fp16) {
            hipLaunchKernelGGL((dispatch_kernel<3, 1>), grid, block, 0, stream, a);
        } else {
            hipLaunchKernelGGL((dispatch_kernel<3, 0>), grid, block, 0, stream, a);
        }
    } else {
        if (a.x_is_fp16) {
            hipLaunchKernelGGL((dispatch_kernel<2, 1>), grid, block, 0, stream, a);
        } else {
            hipLaunchKernelGGL((dispatch_kernel<2, 0>), grid, block, 0, stream, a);
        }
    }
    return hipGetLastError();
}

}  // namespace cam
