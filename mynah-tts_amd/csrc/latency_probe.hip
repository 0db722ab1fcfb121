// Measurement helper: what one dependent stage costs on this device, with the bytes taken out.
//
// A decode step is a chain of stages, each of which needs a whole vector (768 to 3072 floats) that the workgroups of the
// stage before it have just written, from every XCD.  The probe runs that skeleton and nothing else: `nodes` kernel nodes
// in one captured graph, node i reading the vector node i - 1 wrote -- every workgroup all of it, as a matvec stage reads
// its activation row -- reducing it and writing its own share of the next vector.  No weights, no caches: the time per
// node is what the dependency itself costs (the gap between two graph nodes, one read of memory another XCD has just
// written, a workgroup-wide reduction, one store).  `chains` > 1 runs that many independent chains side by side, each on a
// stream of its own, which shows how much of a chain's time a second chain can hide.
#include "common.h"

namespace mynah {
namespace {

__global__ void __launch_bounds__(256) k_probe_node(const float *__restrict__ in, float *__restrict__ out, int floats) {
    __shared__ float s_wave[4];
    const int tid = threadIdx.x;
    float acc = 0.0f;
    if ((floats & 3) == 0) {   // 16-byte requests, as the stage kernels read their activation rows
        const float4 *in4 = reinterpret_cast<const float4 *>(in);
        for (int i = tid; i < (floats >> 2); i += 256) {
            const float4 v = in4[i];
            acc += (v.x + v.y) + (v.z + v.w);
        }
    } else {
        for (int i = tid; i < floats; i += 256) acc += in[i];
    }
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) acc += __shfl_xor(acc, off);
    if ((tid & 63) == 0) s_wave[tid >> 6] = acc;
    __syncthreads();
    const float total = (s_wave[0] + s_wave[1]) + (s_wave[2] + s_wave[3]);
    // this workgroup's share of the next vector: values stay bounded (the next node's sum is again of order `floats`)
    const int share = (floats + (int)gridDim.x - 1) / (int)gridDim.x;
    const int begin = (int)blockIdx.x * share;
    for (int i = begin + tid; i < begin + share && i < floats; i += 256) out[i] = 1.0f + total * 1.0e-12f;
}

__global__ void __launch_bounds__(256) k_probe_fill(float *p, int n) {
    const int i = (int)(blockIdx.x * 256 + threadIdx.x);
    if (i < n) p[i] = 1.0f;
}

}  // namespace
}  // namespace mynah

using namespace mynah;

extern "C" int mynah_hip_dependent_launch_probe(void *opaque, int nodes, int workgroups, int floats, int chains, int repeats, float *node_us,
                                                char *error, size_t capacity) {
    State *st = enter_state(opaque);
    MYNAH_NEED_STATE(st);
    if (node_us == nullptr || nodes < 1 || nodes > 4096 || workgroups < 1 || workgroups > 4096 || floats < 1 || floats > (1 << 20) || chains < 1 ||
        chains > kMaxLanes || repeats < 1 || repeats > 1000) {
        set_error(error, capacity, "launch probe: nodes 1..4096, workgroups 1..4096, floats 1..2^20, chains 1..3, repeats 1..1000");
        return -1;
    }
    *node_us = 0.0f;
    float *buffers = nullptr;
    hipStream_t streams[kMaxLanes] = {};
    hipGraphExec_t graphs[kMaxLanes] = {};
    int rc = hip_check(hipMalloc(reinterpret_cast<void **>(&buffers), (size_t)chains * 2 * floats * sizeof(float)), "malloc", error, capacity);
    if (rc == 0) {
        hipLaunchKernelGGL(k_probe_fill, dim3((unsigned)((chains * 2 * floats + 255) / 256)), dim3(256), 0, st->stream, buffers, chains * 2 * floats);
        rc = hip_check(hipGetLastError(), "probe fill", error, capacity);
    }
    for (int c = 0; c < chains && rc == 0; ++c) rc = lane_stream(st, c, &streams[c], error, capacity);   // the streams the step's lanes use
    hipEvent_t *const done = st->lane_done;
    const hipEvent_t fork = st->lane_fork;
    for (int c = 0; c < chains && rc == 0; ++c) {
        float *a = buffers + (size_t)c * 2 * floats, *b = a + floats;
        hipGraph_t graph = nullptr;
        rc = hip_check(hipStreamBeginCapture(streams[c], hipStreamCaptureModeThreadLocal), "begin capture", error, capacity);
        if (rc != 0) break;
        for (int i = 0; i < nodes; ++i) {
            hipLaunchKernelGGL(k_probe_node, dim3((unsigned)workgroups), dim3(256), 0, streams[c], (i & 1) ? b : a, (i & 1) ? a : b, floats);
        }
        rc = hip_check(hipGetLastError(), "probe launch", error, capacity);
        const hipError_t end = hipStreamEndCapture(streams[c], &graph);
        if (rc == 0) rc = hip_check(end, "end capture", error, capacity);
        if (rc == 0) rc = hip_check(hipGraphInstantiate(&graphs[c], graph, nullptr, nullptr, 0), "graph instantiate", error, capacity);
        if (graph != nullptr) (void)hipGraphDestroy(graph);
    }
    const auto run_once = [&]() -> int {
        if (chains > 1) {
            MYNAH_TRY(hipEventRecord(fork, streams[0]));
            for (int c = 1; c < chains; ++c) MYNAH_TRY(hipStreamWaitEvent(streams[c], fork, 0));
        }
        for (int c = chains - 1; c >= 0; --c) {
            MYNAH_TRY(hipGraphLaunch(graphs[c], streams[c]));
            if (c > 0) MYNAH_TRY(hipEventRecord(done[c], streams[c]));
        }
        for (int c = 1; c < chains; ++c) MYNAH_TRY(hipStreamWaitEvent(streams[0], done[c], 0));
        return 0;
    };
    if (rc == 0) rc = run_once();   // warm-up
    if (rc == 0) rc = run_once();
    if (rc == 0) rc = hip_check(hipStreamSynchronize(st->stream), "synchronise", error, capacity);
    float ms = 0.0f;
    if (rc == 0) rc = hip_check(hipEventRecord(st->ev0, st->stream), "event record", error, capacity);
    for (int r = 0; r < repeats && rc == 0; ++r) rc = run_once();
    if (rc == 0) rc = hip_check(hipEventRecord(st->ev1, st->stream), "event record", error, capacity);
    if (rc == 0) rc = hip_check(hipEventSynchronize(st->ev1), "event synchronise", error, capacity);
    if (rc == 0) rc = hip_check(hipEventElapsedTime(&ms, st->ev0, st->ev1), "event elapsed", error, capacity);
    if (rc == 0) *node_us = ms * 1000.0f / ((float)repeats * (float)nodes);
    (void)hipStreamSynchronize(st->stream);
    for (int c = 0; c < chains; ++c) {
        if (c > 0 && streams[c] != nullptr) (void)hipStreamSynchronize(streams[c]);
        if (graphs[c] != nullptr) (void)hipGraphExecDestroy(graphs[c]);
    }
    if (buffers != nullptr) (void)hipFree(buffers);
    return rc;
}
