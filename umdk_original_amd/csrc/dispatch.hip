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
// window -> output).  Here one workgroup owns one token: each thread loads 16 contiguous bf16 values
// (two 16-byte loads) exactly once, the row maximum is reduced with wave shuffles and one LDS
// exchange, the row is quantised in registers and the 16 resulting bytes are stored with one 16-byte
// store to each of the K destination rows.  HBM traffic is therefore the algorithmic minimum:
// H*2 bytes read and K*H bytes written per token.
#include "cam_device.h"
#include "cam_kernels.h"

namespace cam {

namespace {

constexpr int kDispMaxWaves = 8;  // H <= 7168 -> at most 448 threads

// Output row of entry (t,k), or -1.
__device__ __forceinline__ long long dispatch_row(const DispatchArgs &a, int t, int k)
{
    const int i = t * a.K + k;
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

__device__ __forceinline__ uint32_t pack4(int a, int b, int c, int d)
{
    return (uint32_t)(a & 0xff) | ((uint32_t)(b & 0xff) << 8) | ((uint32_t)(c & 0xff) << 16) |
           ((uint32_t)(d & 0xff) << 24);
}

template <int QUANT>
__global__ __launch_bounds__(kDispMaxWaves * kWave) void dispatch_kernel(DispatchArgs a)
{
    __shared__ float wave_max_s[kDispMaxWaves];
    const int t = blockIdx.x;
    const int tid = threadIdx.x;
    const int chunks = a.H >> 4;  // 16 elements per thread
    const bool active = tid < chunks;

    v4u lo = {0u, 0u, 0u, 0u};
    v4u hi = {0u, 0u, 0u, 0u};
    if (active) {
        const v4u *src = (const v4u *)(a.x + (long long)t * a.H) + 2 * tid;
        lo = __builtin_nontemporal_load(src);
        hi = __builtin_nontemporal_load(src + 1);
    }

    v4u q = {0u, 0u, 0u, 0u};
    float scale_out = 0.0f;
    if (QUANT != 0) {
        float f[16];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            f[2 * j] = bf16_bits_to_f32(lo[j] & 0xffffu);
            f[2 * j + 1] = bf16_bits_to_f32(lo[j] >> 16);
            f[8 + 2 * j] = bf16_bits_to_f32(hi[j] & 0xffffu);
            f[8 + 2 * j + 1] = bf16_bits_to_f32(hi[j] >> 16);
        }
        float m = 0.0f;
#pragma unroll
        for (int j = 0; j < 16; ++j) {
            m = fmaxf(m, fabsf(f[j]));
        }
        m = wave_max(m);
        const int nw = (blockDim.x + kWave - 1) / kWave;
        if (nw > 1) {
            if ((tid & (kWave - 1)) == 0) {
                wave_max_s[tid >> 6] = m;
            }
            __syncthreads();
            m = wave_max_s[0];
            for (int w = 1; w < nw; ++w) {
                m = fmaxf(m, wave_max_s[w]);
            }
        }
        float s;
        bool zero_row = false;
        if (QUANT == 1) {
            s = __fdiv_rn(127.0f, __fadd_rn(m, 1e-12f));
        } else {
            zero_row = (m == 0.0f);
            s = zero_row ? 0.0f : __fdiv_rn(127.0f, m);
        }
        scale_out = zero_row ? 0.0f : __fdiv_rn(1.0f, s);
        int qi[16];
#pragma unroll
        for (int j = 0; j < 16; ++j) {
            qi[j] = (int)rintf(__fmul_rn(f[j], s));
        }
        q[0] = pack4(qi[0], qi[1], qi[2], qi[3]);
        q[1] = pack4(qi[4], qi[5], qi[6], qi[7]);
        q[2] = pack4(qi[8], qi[9], qi[10], qi[11]);
        q[3] = pack4(qi[12], qi[13], qi[14], qi[15]);
    }

    for (int k = 0; k < a.K; ++k) {
        const long long row = dispatch_row(a, t, k);
        if (row < 0 || row >= a.A) {
            continue;
        }
        if (active) {
            if (QUANT != 0) {
                v4u *dst = (v4u *)((int8_t *)a.out + row * a.H) + tid;
                __builtin_nontemporal_store(q, dst);
            } else {
                v4u *dst = (v4u *)((uint16_t *)a.out + row * a.H) + 2 * tid;
                __builtin_nontemporal_store(lo, dst);
                __builtin_nontemporal_store(hi, dst + 1);
            }
        }
        if (tid == 0) {
            if (QUANT != 0) {
                a.scales[row] = scale_out;
            }
            if (a.src_info != nullptr) {
                a.src_info[3 * row + 0] = a.src_rank;
                a.src_info[3 * row + 1] = t;
                a.src_info[3 * row + 2] = k;
            }
        }
    }
}

}  // namespace

hipError_t launch_dispatch(const DispatchArgs &a, hipStream_t stream)
{
    if (a.T <= 0) {
        return hipSuccess;
    }
    const int chunks = a.H / 16;
    const int threads = ((chunks + kWave - 1) / kWave) * kWave;
    if (a.H % 16 != 0 || threads > kDispMaxWaves * kWave) {
        return hipErrorInvalidValue;
    }
    dim3 grid(a.T), block(threads);
    if (a.quant == 0) {
        hipLaunchKernelGGL(dispatch_kernel<0>, grid, block, 0, stream, a);
    } else if (a.quant == 1) {
        hipLaunchKernelGGL(dispatch_kernel<1>, grid, block, 0, stream, a);
    } else {
        hipLaunchKernelGGL(dispatch_kernel<2>, grid, block, 0, stream, a);
    }
    return hipGetLastError();
}

}  // namespace cam
