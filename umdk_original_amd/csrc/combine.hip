// Weighted un-permute and reduce back to token order (bandwidth-bound gather).
//
// Reference semantics (paths relative to the reference tree):
//   src/cam/comm_operator/ascend_kernels/moe_combine_normal/op_kernel/moe_combine_normal.h:303-338
//   src/cam/comm_operator/ascend_kernels/fused_deep_moe/op_kernel/fused_deep_moe/raw_distributed/
//   cam_moe_distribute_combine.h:726-780
// acc = 0 (fp32); for k ascending, skipping absent slots: acc = acc + (float(row) * w[t,k]) with the
// multiply and the add rounded separately; out = bf16 round-to-nearest-even of acc.
//
// Design.  The reference scatters every row into a per-(token,k) window slot and then reads the slots
// back; here the rows are gathered straight from the expert-major buffer.  A workgroup of 128
// threads owns 1024 contiguous columns of one token, so row indices and weights are uniform across
// the workgroup; each thread issues up to eight independent 16-byte row loads before it starts the
// ordered accumulation, then stores 16 bytes of bf16.  Every row byte is read exactly once.
#include "cam_device.h"
#include "cam_kernels.h"

namespace cam {

namespace {

constexpr int kCombThreads = 128;
constexpr int kCombBatch = 8;

// Rows at or beyond *row_limit (the receive total, epRecvCounts[E-1] of moe_combine_normal.h:206-207) were
// never written by the dispatch that filled the buffers; whatever triple they hold is ignored.
__global__ void invert_src_info_kernel(const int32_t *src_info, long long A, const int32_t *row_limit, int T, int K,
                                       int32_t *slot_row)
{
    long long r = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (row_limit != nullptr) {
        A = min(A, (long long)*row_limit);
    }
    if (r >= A) {
        return;
    }
    int t = src_info[3 * r + 1];
    int k = src_info[3 * r + 2];
    if (t >= 0 && t < T && k >= 0 && k < K) {
        slot_row[(long long)t * K + k] = (int32_t)r;
    }
}

__global__ __launch_bounds__(kCombThreads) void combine_kernel(CombineArgs a, int segs)
{
    const int t = blockIdx.x / segs;
    const int seg = blockIdx.x - t * segs;
    const int col = (seg * kCombThreads + threadIdx.x) * 8;
    if (col >= a.H) {
        return;
    }
    float acc[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
        acc[j] = 0.0f;
    }
    const bool live = a.t_active == nullptr || t < *a.t_active;
    const long long rows = a.row_limit == nullptr ? a.A : min(a.A, (long long)*a.row_limit);
    if (live) {
        for (int k0 = 0; k0 < a.K; k0 += kCombBatch) {
            v4u v[kCombBatch];
            float w[kCombBatch];
            bool ok[kCombBatch];
#pragma unroll
            for (int j = 0; j < kCombBatch; ++j) {
                const int k = k0 + j;
                ok[j] = false;
                w[j] = 0.0f;
                v[j] = v4u{0u, 0u, 0u, 0u};
                if (k < a.K) {
                    const long long slot = (long long)t * a.K + k;
                    const long long row = a.slot_row[slot];
                    bool good = row >= 0 && row < rows;
                    if (good && a.src_info != nullptr) {
                        // The inverse map is not pre-cleared: accept a row only if it names this slot.
                        good = a.src_info[3 * row + 1] == t && a.src_info[3 * row + 2] == k;
                    }
                    if (good) {
                        ok[j] = true;
                        w[j] = a.w[slot];
                        v[j] = __builtin_nontemporal_load((const v4u *)(a.y + row * a.H + col));
                    }
                }
            }
#pragma unroll
            for (int j = 0; j < kCombBatch; ++j) {
                if (ok[j]) {
#pragma unroll
                    for (int c = 0; c < 4; ++c) {
                        float x0 = bf16_bits_to_f32(v[j][c] & 0xffffu);
                        float x1 = bf16_bits_to_f32(v[j][c] >> 16);
                        acc[2 * c] = __fadd_rn(acc[2 * c], __fmul_rn(x0, w[j]));
                        acc[2 * c + 1] = __fadd_rn(acc[2 * c + 1], __fmul_rn(x1, w[j]));
                    }
                }
            }
        }
    }
    v4u o;
#pragma unroll
    for (int c = 0; c < 4; ++c) {
        o[c] = f32_to_bf16_bits(acc[2 * c]) | (f32_to_bf16_bits(acc[2 * c + 1]) << 16);
    }
    __builtin_nontemporal_store(o, (v4u *)(a.out + (long long)t * a.H + col));
}

}  // namespace

hipError_t launch_invert_src_info(const int32_t *src_info, int64_t A, const int32_t *row_limit, int T, int K,
                                  int32_t *slot_row, hipStream_t stream)
{
    if (A <= 0) {
        return hipSuccess;
    }
    hipLaunchKernelGGL(invert_src_info_kernel, dim3((unsigned)((A + 255) / 256)), dim3(256), 0, stream, src_info,
                       (long long)A, row_limit, T, K, slot_row);
    return hipGetLastError();
}

hipError_t launch_combine(const CombineArgs &a, hipStream_t stream)
{
    if (a.T <= 0) {
        return hipSuccess;
    }
    if (a.H % 8 != 0) {
        return hipErrorInvalidValue;
    }
    const int segs = (a.H / 8 + kCombThreads - 1) / kCombThreads;
    const long long blocks = (long long)a.T * segs;
    if (blocks > 0x7fffffffll) {
        return hipErrorInvalidValue;
    }
    hipLaunchKernelGGL(combine_kernel, dim3((unsigned)blocks), dim3(kCombThreads), 0, stream, a, segs);
    return hipGetLastError();
}

}  // namespace cam
