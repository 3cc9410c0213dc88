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

namespace cam {

namespace {

constexpr int kDispWaves = 4;         // tokens (waves) per workgroup
constexpr int kDispMaxChunks = 14;    // 16-byte chunks per lane: H <= 14 * 64 * 8 = 7168

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

__device__ __forceinline__ uint32_t pack4(int a, int b, int c, int d)
{
    return (uint32_t)(a & 0xff) | ((uint32_t)(b & 0xff) << 8) | ((uint32_t)(c & 0xff) << 16) |
           ((uint32_t)(d & 0xff) << 24);
}

template <int QUANT>
__global__ __launch_bounds__(kDispWaves * kWave) void dispatch_kernel(DispatchArgs a)
{
    const int t = blockIdx.x * kDispWaves + (threadIdx.x >> 6);
    const int lane = threadIdx.x & (kWave - 1);
    if (t >= a.T) {
        return;
    }
    const int nch = a.H >> 3;  // 8 bf16 values per chunk
    const v4u *src = (const v4u *)(a.x + (long long)t * a.H);
    v4u raw[kDispMaxChunks];
#pragma unroll
    for (int j = 0; j < kDispMaxChunks; ++j) {
        const int c = j * kWave + lane;
        raw[j] = v4u{0u, 0u, 0u, 0u};
        if (c < nch) {
            raw[j] = __builtin_nontemporal_load(src + c);
        }
    }

    v2u q[kDispMaxChunks];
    float scale_out = 0.0f;
    if (QUANT != 0) {
        float m = 0.0f;
#pragma unroll
        for (int j = 0; j < kDispMaxChunks; ++j) {
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                m = fmaxf(m, fabsf(bf16_bits_to_f32(raw[j][i] & 0xffffu)));
                m = fmaxf(m, fabsf(bf16_bits_to_f32(raw[j][i] >> 16)));
            }
        }
        m = wave_max(m);
        float s;
        bool zero_row = false;
        if (QUANT == 1) {
            s = __fdiv_rn(127.0f, __fadd_rn(m, 1e-12f));
        } else {
            zero_row = (m == 0.0f);
            s = zero_row ? 0.0f : __fdiv_rn(127.0f, m);
        }
        scale_out = zero_row ? 0.0f : __fdiv_rn(1.0f, s);
#pragma unroll
        for (int j = 0; j < kDispMaxChunks; ++j) {
            int v[8];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                v[2 * i] = (int)rintf(__fmul_rn(bf16_bits_to_f32(raw[j][i] & 0xffffu), s));
                v[2 * i + 1] = (int)rintf(__fmul_rn(bf16_bits_to_f32(raw[j][i] >> 16), s));
            }
            q[j] = v2u{pack4(v[0], v[1], v[2], v[3]), pack4(v[4], v[5], v[6], v[7])};
        }
    }

    for (int k = 0; k < a.K; ++k) {
        const long long row = dispatch_row(a, t, k);
        if (row < 0 || row >= a.A) {
            continue;
        }
        if (QUANT != 0) {
            v2u *dst = (v2u *)((int8_t *)a.out + row * a.H);
#pragma unroll
            for (int j = 0; j < kDispMaxChunks; ++j) {
                const int c = j * kWave + lane;
                if (c < nch) {
                    __builtin_nontemporal_store(q[j], dst + c);
                }
            }
        } else {
            v4u *dst = (v4u *)((uint16_t *)a.out + row * a.H);
#pragma unroll
            for (int j = 0; j < kDispMaxChunks; ++j) {
                const int c = j * kWave + lane;
                if (c < nch) {
                    __builtin_nontemporal_store(raw[j], dst + c);
                }
            }
        }
        if (lane == 0) {
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
    if (a.H % 8 != 0 || a.H / 8 > kDispMaxChunks * kWave) {
        return hipErrorInvalidValue;
    }
    dim3 grid((a.T + kDispWaves - 1) / kDispWaves), block(kDispWaves * kWave);
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
