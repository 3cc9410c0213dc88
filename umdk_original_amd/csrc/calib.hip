// Calibration micro-benchmarks for the MI355X this library is measured on.  NOT part of the product library: built
// into lib/libcam_calib.so and loaded only by `bench.py --only calib`.  They put numbers behind the ceilings that the
// kernels of the library are compared with:
//   * what the int8 matrix cores sustain and at which clock, alone and with LDS traffic beside them;
//   * what 7 KB rows stored to scattered row slots reach against the same bytes stored linearly (the dispatch);
//   * what streaming reads reach with plain and with non-temporal loads (combine, weight streaming);
//   * the dispatch's permute + quantise done in DESTINATION order (a wave per output row), in one pass and in two.
// Every entry point allocates what it needs, runs warm-up launches, times `reps` launches with HIP events on the null
// stream and frees everything again.
#include <hip/hip_runtime.h>

#include <algorithm>
#include <cstdint>
#include <numeric>
#include <random>
#include <vector>

namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef unsigned int v4u __attribute__((ext_vector_type(4)));
typedef unsigned int v2u __attribute__((ext_vector_type(2)));

#define CALIB_TRY(x)                 \
    do {                             \
        hipError_t e_ = (x);         \
        if (e_ != hipSuccess) {      \
            return (int)e_;          \
        }                            \
    } while (0)

struct Buffers {  // frees what was allocated when it goes out of scope
    std::vector<void *> p;
    ~Buffers()
    {
        for (void *q : p) {
            (void)hipFree(q);
        }
    }
    hipError_t get(void **out, size_t bytes)
    {
        hipError_t e = hipMalloc(out, bytes);
        if (e == hipSuccess) {
            p.push_back(*out);
        }
        return e;
    }
};

template <typename F>
int time_launches(F launch, int warm, int reps, double *us)
{
    hipEvent_t e0, e1;
    CALIB_TRY(hipEventCreate(&e0));
    CALIB_TRY(hipEventCreate(&e1));
    for (int i = 0; i < warm; ++i) {
        launch(i);
    }
    CALIB_TRY(hipDeviceSynchronize());
    CALIB_TRY(hipEventRecord(e0, 0));
    for (int i = 0; i < reps; ++i) {
        launch(i);
    }
    CALIB_TRY(hipEventRecord(e1, 0));
    CALIB_TRY(hipEventSynchronize(e1));
    float ms = 0.f;
    CALIB_TRY(hipEventElapsedTime(&ms, e0, e1));
    CALIB_TRY(hipGetLastError());
    (void)hipEventDestroy(e0);
    (void)hipEventDestroy(e1);
    *us = (double)ms * 1e3 / reps;
    return 0;
}

// ---------------------------------------------------------------------------------------------------------------
// Matrix cores.  Every wave runs `iters` rounds of 16 independent v_mfma_i32_32x32x32_i8 (the instruction and the
// count per sub-step of the GEMM kernel's tall tiles).  MODE 0: operands stay in registers and never change.  MODE 1:
// the operand fragments are read from LDS again in every round, 12 KB per wave like a tall tile's sub-step, always the
// same bytes.  MODE 2: the same reads from a window that moves through 96 KB of random bytes, so that the operands
// of consecutive instructions differ like real data.  clocks[0..1] = shader clock ticks and 100 MHz ticks that one
// wave saw from its first to its last round.
template <int MODE>
__global__ __launch_bounds__(512, 1) void mfma_loop_kernel(int iters, int seed, int *sink, long long *clocks)
{
    __shared__ v4i frag_s[MODE > 0 ? 12 * 64 * 8 : 1];  // 12 KB per wave
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    v4i a[4], b[2];
    for (int i = 0; i < 4; ++i) {
        a[i] = v4i{seed + lane * 3 + i, seed ^ (lane << 3), seed * 5 + i, lane};
    }
    for (int i = 0; i < 2; ++i) {
        b[i] = v4i{seed - lane + i, seed ^ (lane << 7), seed * 3 + i, lane * 9};
    }
    if (MODE > 0) {
        for (int i = 0; i < 12; ++i) {
            v4i v = i < 8 ? a[i & 3] : b[i & 1];
            if (MODE == 2) {  // pseudo-random bytes
                unsigned h = (unsigned)((wave * 12 + i) * 64 + lane) * 2654435761u + (unsigned)seed;
                for (int j = 0; j < 4; ++j) {
                    h = h * 1664525u + 1013904223u;
                    v[j] = (int)(h ^ (h >> 15));
                }
            }
            frag_s[(wave * 12 + i) * 64 + lane] = v;
        }
        __syncthreads();
    }
    v16i acc[4][2];
    for (int m = 0; m < 4; ++m) {
        for (int n = 0; n < 2; ++n) {
            for (int i = 0; i < 16; ++i) {
                acc[m][n][i] = 0;
            }
        }
    }
    const long long c0 = (long long)__builtin_readcyclecounter();  // s_memtime: shader clock
    const long long w0 = (long long)wall_clock64();                // 100 MHz
    for (int it = 0; it < iters; ++it) {
        if (MODE > 0) {
            const int win = MODE == 2 ? ((wave + it) & 7) : wave;  // whose 12 KB this round reads
            v4i alo[4], ahi[4], blo[2], bhi[2];
            for (int m = 0; m < 4; ++m) {
                alo[m] = frag_s[(win * 12 + m) * 64 + lane];
                ahi[m] = frag_s[(win * 12 + 4 + m) * 64 + lane];
            }
            for (int n = 0; n < 2; ++n) {
                blo[n] = frag_s[(win * 12 + 8 + n) * 64 + lane];
                bhi[n] = frag_s[(win * 12 + 10 + n) * 64 + lane];
            }
            for (int m = 0; m < 4; ++m) {
                for (int n = 0; n < 2; ++n) {
                    acc[m][n] = __builtin_amdgcn_mfma_i32_32x32x32_i8(blo[n], alo[m], acc[m][n], 0, 0, 0);
                    acc[m][n] = __builtin_amdgcn_mfma_i32_32x32x32_i8(bhi[n], ahi[m], acc[m][n], 0, 0, 0);
                }
            }
        } else {
            for (int kk = 0; kk < 2; ++kk) {
                for (int m = 0; m < 4; ++m) {
                    for (int n = 0; n < 2; ++n) {
                        acc[m][n] = __builtin_amdgcn_mfma_i32_32x32x32_i8(b[n], a[m], acc[m][n], 0, 0, 0);
                    }
                }
            }
        }
    }
    const long long c1 = (long long)__builtin_readcyclecounter();
    const long long w1 = (long long)wall_clock64();
    int s = 0;
    for (int m = 0; m < 4; ++m) {
        for (int n = 0; n < 2; ++n) {
            for (int i = 0; i < 16; ++i) {
                s ^= acc[m][n][i];
            }
        }
    }
    if (s == 0x7fffffff) {  // never true in practice; keeps the accumulators alive
        sink[0] = s;
    }
    if (blockIdx.x == 0 && threadIdx.x == 0) {
        clocks[0] = c1 - c0;
        clocks[1] = w1 - w0;
    }
}

// ---------------------------------------------------------------------------------------------------------------
// Row stores: one wave per 7168-byte row (7 x 64 lanes x 16 bytes), to the row slot slot[r] of the output.
__global__ __launch_bounds__(256) void store_rows_kernel(const int *slot, int rows, int8_t *out, int nt)
{
    const int r = blockIdx.x * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63;
    if (r >= rows) {
        return;
    }
    v4u *dst = (v4u *)(out + (size_t)slot[r] * 7168);
    const v4u v = {(unsigned)r, (unsigned)lane, 3u, 4u};
#pragma unroll
    for (int i = 0; i < 7; ++i) {
        if (nt) {
            __builtin_nontemporal_store(v, dst + i * 64 + lane);
        } else {
            dst[i * 64 + lane] = v;
        }
    }
}

// The same rows with a whole workgroup of four waves on each row (448 of its 512 16-byte pieces: two stores a thread).
__global__ __launch_bounds__(256) void store_rows_wg_kernel(const int *slot, int rows, int8_t *out, int nt)
{
    const int r = blockIdx.x;
    if (r >= rows) {
        return;
    }
    v4u *dst = (v4u *)(out + (size_t)slot[r] * 7168);
    const v4u v = {(unsigned)r, threadIdx.x, 3u, 4u};
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        const int piece = i * 256 + (int)threadIdx.x;
        if (piece < 448) {
            if (nt) {
                __builtin_nontemporal_store(v, dst + piece);
            } else {
                dst[piece] = v;
            }
        }
    }
}

// A plain fill of the same bytes: 16 bytes per thread, consecutive threads on consecutive pieces.
__global__ __launch_bounds__(256) void fill_kernel(v4u *out, long long n, int nt)
{
    const long long i = (long long)blockIdx.x * 256 + threadIdx.x;
    if (i < n) {
        const v4u v = {(unsigned)i, 2u, 3u, 4u};
        if (nt) {
            __builtin_nontemporal_store(v, out + i);
        } else {
            out[i] = v;
        }
    }
}

// Streaming read: 16 bytes per thread, one element per thread.
__global__ __launch_bounds__(256) void stream_read_kernel(const v4u *in, long long n, int nt, unsigned *sink)
{
    const long long i = (long long)blockIdx.x * 256 + threadIdx.x;
    if (i < n) {
        const v4u v = nt ? __builtin_nontemporal_load(in + i) : in[i];
        if (v[0] == 0x12345678u && v[3] == 0x9abcdef0u) {  // never true for the zero-filled buffer
            sink[0] = v[1];
        }
    }
}

// ---------------------------------------------------------------------------------------------------------------
// Destination-ordered permute + quantise at the dispatch's headline shape (4096 tokens x 7168 bf16, top-8).
constexpr int kH = 7168, kT = 4096, kK = 8, kE = 256, kA = kT * kK;

__device__ __forceinline__ void quant_row(const uint16_t *__restrict__ x, int8_t *__restrict__ out, float *scale_out,
                                          int lane)
{
    v4u v[14];  // 7168 bf16 = 14 x (64 lanes x 8 values)
#pragma unroll
    for (int i = 0; i < 14; ++i) {
        v[i] = ((const v4u *)x)[i * 64 + lane];
    }
    float mx = 0.f;
#pragma unroll
    for (int i = 0; i < 14; ++i) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            mx = fmaxf(mx, fabsf(__uint_as_float(v[i][j] << 16)));
            mx = fmaxf(mx, fabsf(__uint_as_float(v[i][j] & 0xffff0000u)));
        }
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
        mx = fmaxf(mx, __shfl_xor(mx, o, 64));
    }
    const float s = mx > 0.f ? 127.0f / mx : 0.f;
#pragma unroll
    for (int i = 0; i < 14; ++i) {
        unsigned p[2];
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            const int q0 = (int)rintf(__uint_as_float(v[i][2 * h] << 16) * s);
            const int q1 = (int)rintf(__uint_as_float(v[i][2 * h] & 0xffff0000u) * s);
            const int q2 = (int)rintf(__uint_as_float(v[i][2 * h + 1] << 16) * s);
            const int q3 = (int)rintf(__uint_as_float(v[i][2 * h + 1] & 0xffff0000u) * s);
            p[h] = (q0 & 255) | ((q1 & 255) << 8) | ((q2 & 255) << 16) | ((unsigned)(q3 & 255) << 24);
        }
        ((v2u *)out)[i * 64 + lane] = v2u{p[0], p[1]};
    }
    if (lane == 0) {
        *scale_out = mx > 0.f ? mx / 127.0f : 0.f;
    }
}

__global__ __launch_bounds__(256) void dest_one_pass_kernel(const uint16_t *x, const int *token_of_row, int8_t *out,
                                                            float *scales)
{
    const int row = blockIdx.x * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63;
    if (row < kA) {
        quant_row(x + (size_t)token_of_row[row] * kH, out + (size_t)row * kH, scales + row, lane);
    }
}

__global__ __launch_bounds__(256) void quant_tokens_kernel(const uint16_t *x, int8_t *q, float *qs)
{
    const int t = blockIdx.x * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63;
    if (t < kT) {
        quant_row(x + (size_t)t * kH, q + (size_t)t * kH, qs + t, lane);
    }
}

__global__ __launch_bounds__(256) void dest_copy_kernel(const int8_t *q, const float *qs, const int *token_of_row,
                                                        int8_t *out, float *scales)
{
    const int row = blockIdx.x * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63;
    if (row >= kA) {
        return;
    }
    const int t = token_of_row[row];
    const v4u *src = (const v4u *)(q + (size_t)t * kH);
    v4u *dst = (v4u *)(out + (size_t)row * kH);
    v4u v[7];
#pragma unroll
    for (int i = 0; i < 7; ++i) {
        v[i] = src[i * 64 + lane];
    }
#pragma unroll
    for (int i = 0; i < 7; ++i) {
        dst[i * 64 + lane] = v[i];
    }
    if (lane == 0) {
        scales[row] = qs[t];
    }
}

// ---------------------------------------------------------------------------------------------------------------
// fp32 -> bf16: the library's arithmetic definition (round to nearest even on the bit pattern, NaN -> truncated payload
// with the quiet bit set) against the hardware conversion instruction, over every one of the 2^32 bit patterns.
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));

__device__ __forceinline__ unsigned bf16_by_definition(unsigned u)
{
    const unsigned rounded = (u + 0x7fffu + ((u >> 16) & 1u)) >> 16;
    const unsigned quiet = (u >> 16) | 0x0040u;
    return ((u & 0x7fffffffu) > 0x7f800000u ? quiet : rounded) & 0xffffu;
}

__global__ __launch_bounds__(256) void bf16_check_kernel(unsigned long long *mismatches, unsigned *first)
{
    // thread i checks patterns 2i and 2i + 1 of this launch's quarter of the space
    const unsigned long long i = ((unsigned long long)blockIdx.y << 31) + ((unsigned long long)blockIdx.x * 256 + threadIdx.x) * 2;
    const unsigned u0 = (unsigned)i, u1 = (unsigned)i + 1u;
    const f32x2 p = {__uint_as_float(u0), __uint_as_float(u1)};
    const bf16x2 h = __builtin_convertvector(p, bf16x2);
    const unsigned packed = __builtin_bit_cast(unsigned, h);
    const unsigned want = bf16_by_definition(u0) | (bf16_by_definition(u1) << 16);
    if (packed != want) {
        atomicAdd(mismatches, 1ull);
        atomicMin(first, (packed & 0xffffu) != (want & 0xffffu) ? u0 : u1);
    }
}

}  // namespace

#define CALIB_API extern "C" __attribute__((visibility("default")))

// mode: see mfma_loop_kernel.  out[0] = int8 operations per second (POP/s), out[1] = shader clock in GHz while the
// loop ran.
CALIB_API int camCalibMfmaInt8(int mode, double *out)
{
    hipDeviceProp_t prop;
    int dev = 0;
    CALIB_TRY(hipGetDevice(&dev));
    CALIB_TRY(hipGetDeviceProperties(&prop, dev));
    const int cus = prop.multiProcessorCount;
    const int iters = 20000;
    Buffers b;
    int *sink;
    long long *clocks;
    CALIB_TRY(b.get((void **)&sink, 64));
    CALIB_TRY(b.get((void **)&clocks, 64));
    double us = 0;
    const int rc = time_launches(
        [&](int i) {
            if (mode == 2) {
                hipLaunchKernelGGL(mfma_loop_kernel<2>, dim3(cus), dim3(512), 0, 0, iters, 17 + i, sink, clocks);
            } else if (mode == 1) {
                hipLaunchKernelGGL(mfma_loop_kernel<1>, dim3(cus), dim3(512), 0, 0, iters, 17 + i, sink, clocks);
            } else {
                hipLaunchKernelGGL(mfma_loop_kernel<0>, dim3(cus), dim3(512), 0, 0, iters, 17 + i, sink, clocks);
            }
        },
        1, 3, &us);
    if (rc != 0) {
        return rc;
    }
    long long hc[2] = {0, 1};
    CALIB_TRY(hipMemcpy(hc, clocks, sizeof(hc), hipMemcpyDeviceToHost));
    const double ops = (double)cus * 8 /*waves*/ * iters * 16 /*MFMAs*/ * (2.0 * 32 * 32 * 32);
    out[0] = ops / (us * 1e-6) / 1e15;
    out[1] = hc[1] > 0 ? (double)hc[0] / (double)hc[1] * 0.1 : 0.0;
    return 0;
}

// 32768 rows of 7168 bytes, four rotating outputs: out[0] = TB/s to scattered row slots, out[1] = TB/s to consecutive
// ones (a wave per row), out[2] = scattered with a workgroup per row, out[3] = a plain fill of the same bytes
// (non-temporal stores if nt != 0).
CALIB_API int camCalibRowStores(int nt, double *out)
{
    const int rows = kA, rot = 4;
    Buffers b;
    int8_t *o[rot];
    int *slot_scattered, *slot_linear;
    for (int i = 0; i < rot; ++i) {
        CALIB_TRY(b.get((void **)&o[i], (size_t)rows * kH));
    }
    CALIB_TRY(b.get((void **)&slot_scattered, rows * sizeof(int)));
    CALIB_TRY(b.get((void **)&slot_linear, rows * sizeof(int)));
    std::vector<int> perm(rows);
    std::iota(perm.begin(), perm.end(), 0);
    CALIB_TRY(hipMemcpy(slot_linear, perm.data(), rows * sizeof(int), hipMemcpyHostToDevice));
    std::mt19937 rng(1);
    std::shuffle(perm.begin(), perm.end(), rng);
    CALIB_TRY(hipMemcpy(slot_scattered, perm.data(), rows * sizeof(int), hipMemcpyHostToDevice));
    for (int which = 0; which < 2; ++which) {
        const int *slot = which == 0 ? slot_scattered : slot_linear;
        double us = 0;
        const int rc = time_launches(
            [&](int i) {
                hipLaunchKernelGGL(store_rows_kernel, dim3(rows / 4), dim3(256), 0, 0, slot, rows, o[i % rot], nt);
            },
            8, 40, &us);
        if (rc != 0) {
            return rc;
        }
        out[which] = (double)rows * kH / (us * 1e-6) / 1e12;
    }
    {  // out[2]: scattered rows, a workgroup per row; out[3]: a plain fill of the same bytes
        double us = 0;
        int rc = time_launches(
            [&](int i) {
                hipLaunchKernelGGL(store_rows_wg_kernel, dim3(rows), dim3(256), 0, 0, slot_scattered, rows, o[i % rot], nt);
            },
            8, 40, &us);
        if (rc != 0) {
            return rc;
        }
        out[2] = (double)rows * kH / (us * 1e-6) / 1e12;
        const long long n = (long long)rows * kH / 16;
        rc = time_launches(
            [&](int i) {
                hipLaunchKernelGGL(fill_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, 0, (v4u *)o[i % rot], n, nt);
            },
            8, 40, &us);
        if (rc != 0) {
            return rc;
        }
        out[3] = (double)rows * kH / (us * 1e-6) / 1e12;
    }
    return 0;
}

// 1.5 GiB read once per launch: out[0] = TB/s with plain loads, out[1] = with non-temporal loads.
CALIB_API int camCalibStreamRead(double *out)
{
    const long long n = (3ll << 29) / 16;
    Buffers b;
    v4u *in;
    unsigned *sink;
    CALIB_TRY(b.get((void **)&in, (size_t)n * 16));
    CALIB_TRY(b.get((void **)&sink, 64));
    CALIB_TRY(hipMemset(in, 0, (size_t)n * 16));
    for (int nt = 0; nt < 2; ++nt) {
        double us = 0;
        const int rc = time_launches(
            [&](int) {
                hipLaunchKernelGGL(stream_read_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, 0, in, n, nt, sink);
            },
            3, 10, &us);
        if (rc != 0) {
            return rc;
        }
        out[nt] = (double)n * 16 / (us * 1e-6) / 1e12;
    }
    return 0;
}

// The dispatch in destination order, microseconds per launch: out[0] one pass (every output row quantises its token
// again), out[1] token-major quantisation alone, out[2] row copy in destination order alone, out[3] both back to back.
CALIB_API int camCalibDestinationOrder(double *out)
{
    const int rot = 4;
    std::mt19937 rng(5);
    std::vector<std::pair<int, int>> slots;  // (expert, token) in flat (token, k) order
    slots.reserve(kA);
    for (int t = 0; t < kT; ++t) {
        int e[kK];
        for (int k = 0; k < kK; ++k) {
            bool again;
            do {
                e[k] = (int)(rng() % kE);
                again = false;
                for (int j = 0; j < k; ++j) {
                    again = again || e[j] == e[k];
                }
            } while (again);
            slots.push_back({e[k], t});
        }
    }
    std::stable_sort(slots.begin(), slots.end(),
                     [](const std::pair<int, int> &a, const std::pair<int, int> &b) { return a.first < b.first; });
    std::vector<int> tor(kA);
    for (int r = 0; r < kA; ++r) {
        tor[r] = slots[r].second;
    }
    std::vector<uint16_t> hx((size_t)kT * kH);
    for (auto &v : hx) {
        v = (uint16_t)((0x3c00 + (rng() & 0x3ff)) | ((rng() & 1) << 15));
    }
    Buffers b;
    uint16_t *x[rot];
    int8_t *o[rot], *q;
    float *sc, *qs;
    int *dtor;
    for (int i = 0; i < rot; ++i) {
        CALIB_TRY(b.get((void **)&x[i], (size_t)kT * kH * 2));
        CALIB_TRY(hipMemcpy(x[i], hx.data(), (size_t)kT * kH * 2, hipMemcpyHostToDevice));
        CALIB_TRY(b.get((void **)&o[i], (size_t)kA * kH));
    }
    CALIB_TRY(b.get((void **)&q, (size_t)kT * kH));
    CALIB_TRY(b.get((void **)&sc, kA * sizeof(float)));
    CALIB_TRY(b.get((void **)&qs, kT * sizeof(float)));
    CALIB_TRY(b.get((void **)&dtor, kA * sizeof(int)));
    CALIB_TRY(hipMemcpy(dtor, tor.data(), kA * sizeof(int), hipMemcpyHostToDevice));
    int rc = time_launches(
        [&](int i) {
            hipLaunchKernelGGL(dest_one_pass_kernel, dim3(kA / 4), dim3(256), 0, 0, x[i % rot], dtor, o[i % rot], sc);
        },
        8, 40, &out[0]);
    if (rc != 0) {
        return rc;
    }
    rc = time_launches(
        [&](int i) { hipLaunchKernelGGL(quant_tokens_kernel, dim3(kT / 4), dim3(256), 0, 0, x[i % rot], q, qs); }, 8, 40,
        &out[1]);
    if (rc != 0) {
        return rc;
    }
    rc = time_launches(
        [&](int i) { hipLaunchKernelGGL(dest_copy_kernel, dim3(kA / 4), dim3(256), 0, 0, q, qs, dtor, o[i % rot], sc); },
        8, 40, &out[2]);
    if (rc != 0) {
        return rc;
    }
    return time_launches(
        [&](int i) {
            hipLaunchKernelGGL(quant_tokens_kernel, dim3(kT / 4), dim3(256), 0, 0, x[i % rot], q, qs);
            hipLaunchKernelGGL(dest_copy_kernel, dim3(kA / 4), dim3(256), 0, 0, q, qs, dtor, o[i % rot], sc);
        },
        8, 40, &out[3]);
}

// out[0] = bit patterns (in pairs) on which the hardware fp32 -> bf16 conversion differs from the definition above,
// out[1] = the smallest such pattern (as an unsigned value) or 2^32 - 1 when there is none.
CALIB_API int camCalibBf16Conversion(double *out)
{
    Buffers b;
    unsigned long long *mism;
    unsigned *first;
    CALIB_TRY(b.get((void **)&mism, 8));
    CALIB_TRY(b.get((void **)&first, 4));
    CALIB_TRY(hipMemset(mism, 0, 8));
    CALIB_TRY(hipMemset(first, 0xff, 4));
    // 2^32 patterns = 2 (grid y) x 2^31; a thread takes two: 2^30 threads per y = 2^22 workgroups of 256
    hipLaunchKernelGGL(bf16_check_kernel, dim3(1u << 22, 2), dim3(256), 0, 0, mism, first);
    CALIB_TRY(hipGetLastError());
    CALIB_TRY(hipDeviceSynchronize());
    unsigned long long hm = 0;
    unsigned hf = 0;
    CALIB_TRY(hipMemcpy(&hm, mism, 8, hipMemcpyDeviceToHost));
    CALIB_TRY(hipMemcpy(&hf, first, 4, hipMemcpyDeviceToHost));
    out[0] = (double)hm;
    out[1] = (double)hf;
    return 0;
}
