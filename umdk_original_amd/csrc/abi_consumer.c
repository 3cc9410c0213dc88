/* A caller of the C ABI written in plain C with nothing but the HIP runtime beside it: no torch, no C++.  It is what
 * a binding in another language sees (the reference reaches its operators the same way, through a C entry-point pair
 * found with dlsym: src/cam/comm_operator/pybind/pytorch_extension/pytorch_npu_helper.hpp:533-582).
 *
 *   abi_consumer check   phase 1 only, no GPU touched: argument validation and workspace sizes
 *   abi_consumer run     DispatchLayout and NotifyDispatch on the current GPU, compared with a loop on the host
 *
 * Exit status 0 on success; every failure prints what it was. */
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#define __HIP_PLATFORM_AMD__ 1
#include <hip/hip_runtime_api.h>

#include "../../include/cam_mi355x.h"

#define T 96
#define K 4
#define E 24
#define R 3

static camTensor tensor(void *data, int32_t dtype, int ndim, int64_t d0, int64_t d1)
{
    camTensor t;
    memset(&t, 0, sizeof(t));
    t.data = data;
    t.dtype = dtype;
    t.ndim = ndim;
    t.sizes[0] = d0;
    t.sizes[1] = d1;
    t.strides[0] = ndim == 2 ? d1 : 1;
    t.strides[1] = 1;
    t.format = CAM_FORMAT_ND;
    return t;
}

#define FAIL(...)                     \
    do {                              \
        fprintf(stderr, __VA_ARGS__); \
        fprintf(stderr, "\n");        \
        return 1;                     \
    } while (0)

static int check_only(void)
{
    /* pointers are never dereferenced by phase 1; any non-null, 16-byte aligned value will do */
    void *fake = (void *)(uintptr_t)0x1000;
    camTensor idx = tensor(fake, CAM_DT_INT64, 2, T, K);
    camTensor per_rank = tensor(fake, CAM_DT_INT32, 1, R, 0);
    camTensor per_expert = tensor(fake, CAM_DT_INT32, 1, E, 0);
    camTensor in_rank = tensor(fake, CAM_DT_INT32, 2, T, R);
    uint64_t ws = 0;
    camOpExecutor *ex = NULL;
    camStatus st = camDispatchLayoutGetWorkspaceSize(&idx, T, R, E, K, &per_rank, &per_expert, &in_rank, &ws, &ex);
    if (st != CAM_OK) FAIL("DispatchLayout phase 1: status %d: %s", (int)st, camGetRecentErrMsg());
    if (ex == NULL) FAIL("DispatchLayout phase 1 returned no executor");
    if (camDestroyExecutor(ex) != CAM_OK) FAIL("camDestroyExecutor failed");
    st = camDispatchLayoutGetWorkspaceSize(NULL, T, R, E, K, &per_rank, &per_expert, &in_rank, &ws, &ex);
    if (st != CAM_ERR_NULL || strstr(camGetRecentErrMsg(), "topkIdx") == NULL)
        FAIL("a NULL topkIdx should be refused by name, got status %d: %s", (int)st, camGetRecentErrMsg());
    st = camDispatchLayoutGetWorkspaceSize(&idx, T, 385, 385, K, &per_rank, &per_expert, &in_rank, &ws, &ex);
    if (st != CAM_ERR_RANGE) FAIL("385 ranks should be out of range, got status %d", (int)st);
    printf("check ok: %s\n", camGetVersion());
    return 0;
}

#define HIP_TRY(x)                                                             \
    do {                                                                       \
        hipError_t e_ = (x);                                                   \
        if (e_ != hipSuccess) FAIL("%s: %s", #x, hipGetErrorString(e_));       \
    } while (0)

static int run_on_gpu(void)
{
    static int64_t h_idx[T * K];
    static int32_t want_rank[R], want_expert[E], want_in[T * R], got_rank[R], got_expert[E], got_in[T * R];
    static int32_t want_off[E], got_off[E], got_send[3 * E];
    uint32_t s = 12345u;
    for (int i = 0; i < T * K; ++i) {
        s = s * 1664525u + 1013904223u;
        h_idx[i] = (s >> 8) % 29 == 0 ? -1 : (int64_t)((s >> 8) % E); /* some slots name no expert */
    }
    memset(want_rank, 0, sizeof(want_rank));
    memset(want_expert, 0, sizeof(want_expert));
    memset(want_in, 0, sizeof(want_in));
    for (int t = 0; t < T; ++t) {
        for (int k = 0; k < K; ++k) {
            const int64_t e = h_idx[t * K + k];
            if (e < 0) continue;
            want_expert[e] += 1;
            const int r = (int)(e / (E / R));
            if (!want_in[t * R + r]) {
                want_in[t * R + r] = 1;
                want_rank[r] += 1;
            }
        }
    }
    int32_t run = 0;
    for (int e = 0; e < E; ++e) {
        want_off[e] = run;
        run += want_expert[e];
    }

    void *d_idx, *d_rank, *d_expert, *d_in, *d_off, *d_send, *d_recv, *d_ws = NULL;
    HIP_TRY(hipMalloc(&d_idx, sizeof(h_idx)));
    HIP_TRY(hipMalloc(&d_rank, sizeof(got_rank)));
    HIP_TRY(hipMalloc(&d_expert, sizeof(got_expert)));
    HIP_TRY(hipMalloc(&d_in, sizeof(got_in)));
    HIP_TRY(hipMalloc(&d_off, sizeof(got_off)));
    HIP_TRY(hipMalloc(&d_send, sizeof(got_send)));
    HIP_TRY(hipMalloc(&d_recv, sizeof(got_send)));
    HIP_TRY(hipMemcpy(d_idx, h_idx, sizeof(h_idx), hipMemcpyHostToDevice));
    HIP_TRY(hipMemset(d_rank, 0xff, sizeof(got_rank))); /* outputs need not be zeroed by the caller */
    HIP_TRY(hipMemset(d_expert, 0xff, sizeof(got_expert)));
    HIP_TRY(hipMemset(d_in, 0xff, sizeof(got_in)));

    camTensor idx = tensor(d_idx, CAM_DT_INT64, 2, T, K);
    camTensor per_rank = tensor(d_rank, CAM_DT_INT32, 1, R, 0);
    camTensor per_expert = tensor(d_expert, CAM_DT_INT32, 1, E, 0);
    camTensor in_rank = tensor(d_in, CAM_DT_INT32, 2, T, R);
    uint64_t ws = 0;
    camOpExecutor *ex = NULL;
    if (camDispatchLayoutGetWorkspaceSize(&idx, T, R, E, K, &per_rank, &per_expert, &in_rank, &ws, &ex) != CAM_OK)
        FAIL("DispatchLayout phase 1: %s", camGetRecentErrMsg());
    if (ws > 0) HIP_TRY(hipMalloc(&d_ws, ws));
    if (camDispatchLayout(d_ws, ws, ex, NULL) != CAM_OK) FAIL("DispatchLayout phase 2: %s", camGetRecentErrMsg());
    HIP_TRY(hipDeviceSynchronize());
    HIP_TRY(hipMemcpy(got_rank, d_rank, sizeof(got_rank), hipMemcpyDeviceToHost));
    HIP_TRY(hipMemcpy(got_expert, d_expert, sizeof(got_expert), hipMemcpyDeviceToHost));
    HIP_TRY(hipMemcpy(got_in, d_in, sizeof(got_in), hipMemcpyDeviceToHost));
    if (memcmp(got_rank, want_rank, sizeof(got_rank)) != 0) FAIL("numTokensPerRank differs from the host loop");
    if (memcmp(got_expert, want_expert, sizeof(got_expert)) != 0) FAIL("numTokensPerExpert differs from the host loop");
    if (memcmp(got_in, want_in, sizeof(got_in)) != 0) FAIL("isTokenInRank differs from the host loop");
    if (d_ws) HIP_TRY(hipFree(d_ws));
    d_ws = NULL;

    /* NotifyDispatch on one rank: exclusive prefix sum of the counts and the (count, offset, tokens) triplets */
    camTensor send = tensor(d_send, CAM_DT_INT32, 1, 3 * E, 0);
    camTensor recv = tensor(d_recv, CAM_DT_INT32, 1, 3 * E, 0);
    camTensor off = tensor(d_off, CAM_DT_INT32, 1, E, 0);
    char group[1] = {0};
    if (camNotifyDispatchGetWorkspaceSize(&send, &per_expert, 3 * E, T, group, 1, 0, 1, 0, &off, &recv, &ws, &ex) != CAM_OK)
        FAIL("NotifyDispatch phase 1: %s", camGetRecentErrMsg());
    if (ws > 0) HIP_TRY(hipMalloc(&d_ws, ws));
    if (camNotifyDispatch(d_ws, ws, ex, NULL) != CAM_OK) FAIL("NotifyDispatch phase 2: %s", camGetRecentErrMsg());
    HIP_TRY(hipDeviceSynchronize());
    HIP_TRY(hipMemcpy(got_off, d_off, sizeof(got_off), hipMemcpyDeviceToHost));
    HIP_TRY(hipMemcpy(got_send, d_recv, sizeof(got_send), hipMemcpyDeviceToHost));
    if (memcmp(got_off, want_off, sizeof(got_off)) != 0) FAIL("sendDataOffset differs from the host prefix sum");
    for (int e = 0; e < E; ++e) {
        if (got_send[3 * e] != want_expert[e] || got_send[3 * e + 1] != want_off[e] || got_send[3 * e + 2] != T)
            FAIL("recvData triplet %d is (%d, %d, %d)", e, got_send[3 * e], got_send[3 * e + 1], got_send[3 * e + 2]);
    }
    if (d_ws) HIP_TRY(hipFree(d_ws));
    printf("run ok: DispatchLayout and NotifyDispatch match the host loops (%d tokens, top-%d, %d experts, %d ranks)\n",
           T, K, E, R);
    return 0;
}

int main(int argc, char **argv)
{
    if (argc == 2 && strcmp(argv[1], "check") == 0) return check_only();
    if (argc == 2 && strcmp(argv[1], "run") == 0) return run_on_gpu();
    fprintf(stderr, "usage: %s check|run\n", argv[0]);
    return 2;
}
