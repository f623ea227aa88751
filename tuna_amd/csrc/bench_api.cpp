// Timing loops and self-tests of the diagnostic build (libtuna_amd_bench.so): what bench.py, the tuner and the tests
// use to time launches with HIP events on the launch stream, without Python between the launches.  The loops call
// the product entry points of tuna_amd.h (the same object code as in libtuna_amd.so); nothing here is part of the
// product library.
#include <hip/hip_runtime.h>

#include "bench_internal.h"

namespace tuna {

// Times `iters` enqueues of `launch(i)` with HIP events on `stream`.
template <typename F>
static int time_loop(F launch, int n_sets, int warmup, int iters, int use_graph, hipStream_t stream, float *elapsed_ms)
{
    if (iters <= 0 || warmup < 0 || n_sets <= 0 || !elapsed_ms) return fail(TUNA_ERR_INVALID_ARG, "bad timing arguments");
    int rc;
    hipError_t e;
    hipEvent_t t0 = nullptr, t1 = nullptr;
    if ((e = hipEventCreate(&t0)) != hipSuccess) return hip_fail(e, "hipEventCreate");
    if ((e = hipEventCreate(&t1)) != hipSuccess) {
        (void)hipEventDestroy(t0);
        return hip_fail(e, "hipEventCreate");
    }
    hipGraph_t graph = nullptr;
    hipGraphExec_t exec = nullptr, tail_exec = nullptr;
    hipGraph_t tail_graph = nullptr;
    hipStream_t cap_stream = nullptr;
    rc = TUNA_OK;
    do {
        for (int i = 0; i < warmup && !rc; ++i) rc = launch(i % n_sets, stream);
        if (rc) break;
        if (use_graph) {
            // one rotation over the weight sets per graph launch; capture on a private
            // stream so that the caller's stream (possibly the default one) is untouched
            if ((e = hipStreamCreateWithFlags(&cap_stream, hipStreamNonBlocking)) != hipSuccess) { rc = hip_fail(e, "hipStreamCreate"); break; }
            if ((e = hipStreamSynchronize(stream)) != hipSuccess) { rc = hip_fail(e, "hipStreamSynchronize"); break; }
            for (int i = 0; i < n_sets && !rc; ++i) rc = launch(i, cap_stream);  // workspace for cap_stream grows here, before capture
            if (rc) break;
            if ((e = hipStreamSynchronize(cap_stream)) != hipSuccess) { rc = hip_fail(e, "hipStreamSynchronize"); break; }
            if ((e = hipStreamBeginCapture(cap_stream, hipStreamCaptureModeThreadLocal)) != hipSuccess) { rc = hip_fail(e, "hipStreamBeginCapture"); break; }
            for (int i = 0; i < n_sets && !rc; ++i) rc = launch(i, cap_stream);
            e = hipStreamEndCapture(cap_stream, &graph);
            if (rc) break;
            if (e != hipSuccess) { rc = hip_fail(e, "hipStreamEndCapture"); break; }
            if ((e = hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0)) != hipSuccess) { rc = hip_fail(e, "hipGraphInstantiate"); break; }
            // exactly `iters` timed launches: `iters / n_sets` replays of the rotation and, when that leaves a
            // remainder, one replay of a second graph that holds the first `iters % n_sets` launches of it
            const int reps = iters / n_sets, rest = iters % n_sets;
            if (rest > 0) {
                if ((e = hipStreamBeginCapture(cap_stream, hipStreamCaptureModeThreadLocal)) != hipSuccess) { rc = hip_fail(e, "hipStreamBeginCapture"); break; }
                for (int i = 0; i < rest && !rc; ++i) rc = launch(i, cap_stream);
                e = hipStreamEndCapture(cap_stream, &tail_graph);
                if (rc) break;
                if (e != hipSuccess) { rc = hip_fail(e, "hipStreamEndCapture"); break; }
                if ((e = hipGraphInstantiate(&tail_exec, tail_graph, nullptr, nullptr, 0)) != hipSuccess) { rc = hip_fail(e, "hipGraphInstantiate"); break; }
                if ((e = hipGraphLaunch(tail_exec, cap_stream)) != hipSuccess) { rc = hip_fail(e, "hipGraphLaunch"); break; }
            }
            if ((e = hipGraphLaunch(exec, cap_stream)) != hipSuccess) { rc = hip_fail(e, "hipGraphLaunch"); break; }
            if ((e = hipEventRecord(t0, cap_stream)) != hipSuccess) { rc = hip_fail(e, "hipEventRecord"); break; }
            for (int r = 0; r < reps; ++r)
                if ((e = hipGraphLaunch(exec, cap_stream)) != hipSuccess) { rc = hip_fail(e, "hipGraphLaunch"); break; }
            if (rc) break;
            if (rest > 0 && (e = hipGraphLaunch(tail_exec, cap_stream)) != hipSuccess) { rc = hip_fail(e, "hipGraphLaunch"); break; }
            if ((e = hipEventRecord(t1, cap_stream)) != hipSuccess) { rc = hip_fail(e, "hipEventRecord"); break; }
            if ((e = hipEventSynchronize(t1)) != hipSuccess) { rc = hip_fail(e, "hipEventSynchronize"); break; }
            if ((e = hipEventElapsedTime(elapsed_ms, t0, t1)) != hipSuccess) { rc = hip_fail(e, "hipEventElapsedTime"); break; }
        } else {
            if ((e = hipEventRecord(t0, stream)) != hipSuccess) { rc = hip_fail(e, "hipEventRecord"); break; }
            for (int i = 0; i < iters && !rc; ++i) rc = launch((warmup + i) % n_sets, stream);
            if (rc) break;
            if ((e = hipEventRecord(t1, stream)) != hipSuccess) { rc = hip_fail(e, "hipEventRecord"); break; }
            if ((e = hipEventSynchronize(t1)) != hipSuccess) { rc = hip_fail(e, "hipEventSynchronize"); break; }
            if ((e = hipEventElapsedTime(elapsed_ms, t0, t1)) != hipSuccess) { rc = hip_fail(e, "hipEventElapsedTime"); break; }
        }
    } while (0);
    if (exec) (void)hipGraphExecDestroy(exec);
    if (graph) (void)hipGraphDestroy(graph);
    if (tail_exec) (void)hipGraphExecDestroy(tail_exec);
    if (tail_graph) (void)hipGraphDestroy(tail_graph);
    if (cap_stream) {
        (void)hipStreamSynchronize(cap_stream);
        drop_workspace(cap_stream);
        (void)hipStreamDestroy(cap_stream);
    }
    (void)hipEventDestroy(t0);
    (void)hipEventDestroy(t1);
    return rc;
}

// Times `iters` enqueues of `launch(i, stream)` dealt round-robin to `n_streams` streams of the default priority that
// this call creates: every stream waits for one start event, the end event waits for every stream.  What the time
// shows is whether independent launches on different streams overlap on the device.
template <typename F>
static int time_loop_streams(F launch, int n_streams, int use_graph, int warmup, int iters, float *elapsed_ms)
{
    if (iters <= 0 || warmup < 0 || n_streams < 1 || n_streams > 16 || !elapsed_ms) return fail(TUNA_ERR_INVALID_ARG, "bad timing arguments");
    hipStream_t streams[16] = {};
    hipEvent_t joins[16] = {};
    hipEvent_t t0 = nullptr, t1 = nullptr, fork = nullptr;
    hipGraph_t graph = nullptr;
    hipGraphExec_t exec = nullptr;
    hipError_t e = hipSuccess;
    int rc = TUNA_OK, made = 0;
    // fork: every stream waits for `ev`, recorded on stream 0; join: stream 0 waits for every other stream
    auto fork_all = [&](hipEvent_t ev) {
        if ((e = hipEventRecord(ev, streams[0])) != hipSuccess) return hip_fail(e, "hipEventRecord");
        for (int j = 1; j < n_streams; ++j)
            if ((e = hipStreamWaitEvent(streams[j], ev, 0)) != hipSuccess) return hip_fail(e, "hipStreamWaitEvent");
        return (int)TUNA_OK;
    };
    auto join_all = [&]() {
        for (int j = 1; j < n_streams; ++j) {
            if ((e = hipEventRecord(joins[j], streams[j])) != hipSuccess) return hip_fail(e, "hipEventRecord");
            if ((e = hipStreamWaitEvent(streams[0], joins[j], 0)) != hipSuccess) return hip_fail(e, "hipStreamWaitEvent");
        }
        return (int)TUNA_OK;
    };
    do {
        if ((e = hipEventCreate(&t0)) != hipSuccess || (e = hipEventCreate(&t1)) != hipSuccess ||
            (e = hipEventCreateWithFlags(&fork, hipEventDisableTiming)) != hipSuccess) { rc = hip_fail(e, "hipEventCreate"); break; }
        for (; made < n_streams; ++made) {
            if ((e = hipStreamCreateWithFlags(&streams[made], hipStreamNonBlocking)) != hipSuccess) { rc = hip_fail(e, "hipStreamCreate"); break; }
            if ((e = hipEventCreateWithFlags(&joins[made], hipEventDisableTiming)) != hipSuccess) {
                (void)hipStreamDestroy(streams[made]);
                rc = hip_fail(e, "hipEventCreate");
                break;
            }
        }
        if (rc) break;
        for (int i = 0; i < warmup * n_streams && !rc; ++i) rc = launch(i, i % n_streams, streams[i % n_streams]);
        if (rc) break;
        for (int j = 0; j < n_streams; ++j)
            if ((e = hipStreamSynchronize(streams[j])) != hipSuccess) { rc = hip_fail(e, "hipStreamSynchronize"); break; }
        if (rc) break;
        if (use_graph) {
            // one graph of up to 256 launches with n_streams parallel branches, replayed; the launches that do not fill
            // a whole replay are left out of the timed count (the caller gets the time scaled to `iters`)
            const int per_graph = iters < 256 ? iters : 256;
            const int reps = iters / per_graph;
            if ((e = hipStreamBeginCapture(streams[0], hipStreamCaptureModeThreadLocal)) != hipSuccess) { rc = hip_fail(e, "hipStreamBeginCapture"); break; }
            rc = fork_all(fork);
            for (int i = 0; i < per_graph && !rc; ++i) rc = launch(i, i % n_streams, streams[i % n_streams]);
            if (!rc) rc = join_all();
            e = hipStreamEndCapture(streams[0], &graph);
            if (rc) break;
            if (e != hipSuccess) { rc = hip_fail(e, "hipStreamEndCapture"); break; }
            if ((e = hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0)) != hipSuccess) { rc = hip_fail(e, "hipGraphInstantiate"); break; }
            if ((e = hipGraphLaunch(exec, streams[0])) != hipSuccess) { rc = hip_fail(e, "hipGraphLaunch"); break; }
            if ((e = hipEventRecord(t0, streams[0])) != hipSuccess) { rc = hip_fail(e, "hipEventRecord"); break; }
            for (int r = 0; r < reps; ++r)
                if ((e = hipGraphLaunch(exec, streams[0])) != hipSuccess) { rc = hip_fail(e, "hipGraphLaunch"); break; }
            if (rc) break;
            if ((e = hipEventRecord(t1, streams[0])) != hipSuccess) { rc = hip_fail(e, "hipEventRecord"); break; }
            if ((e = hipEventSynchronize(t1)) != hipSuccess) { rc = hip_fail(e, "hipEventSynchronize"); break; }
            float ms = 0.f;
            if ((e = hipEventElapsedTime(&ms, t0, t1)) != hipSuccess) { rc = hip_fail(e, "hipEventElapsedTime"); break; }
            *elapsed_ms = ms * (float)iters / (float)(reps * per_graph);
            break;
        }
        if ((rc = fork_all(t0))) break;
        for (int i = 0; i < iters && !rc; ++i) rc = launch(i, i % n_streams, streams[i % n_streams]);
        if (rc) break;
        if ((rc = join_all())) break;
        if ((e = hipEventRecord(t1, streams[0])) != hipSuccess) { rc = hip_fail(e, "hipEventRecord"); break; }
        if ((e = hipEventSynchronize(t1)) != hipSuccess) { rc = hip_fail(e, "hipEventSynchronize"); break; }
        if ((e = hipEventElapsedTime(elapsed_ms, t0, t1)) != hipSuccess) { rc = hip_fail(e, "hipEventElapsedTime"); break; }
    } while (0);
    if (exec) (void)hipGraphExecDestroy(exec);
    if (graph) (void)hipGraphDestroy(graph);
    for (int j = 0; j < made; ++j) {
        (void)hipStreamSynchronize(streams[j]);
        drop_workspace(streams[j]);
        (void)hipStreamDestroy(streams[j]);
        (void)hipEventDestroy(joins[j]);
    }
    if (t0) (void)hipEventDestroy(t0);
    if (t1) (void)hipEventDestroy(t1);
    if (fork) (void)hipEventDestroy(fork);
    return rc;
}

}  // namespace tuna

using namespace tuna;

extern "C" {

TUNA_EXPORT int tuna_time_matmul(const void *const *q_list, const void *const *absmax_list, int n_sets, const void *x,
                                 const void *code, void *out, int m, int n, int k, const tuna_gemm_config *cfg,
                                 int decode_mode, int warmup, int iters, int use_graph, void *stream, float *elapsed_ms)
{
    if (!q_list || !absmax_list) return fail(TUNA_ERR_INVALID_ARG, "q_list / absmax_list is null");
    auto launch = [&](int set, hipStream_t s) {
        return tuna_matmul_ex(q_list[set], x, code, absmax_list[set], out, m, n, k, cfg, decode_mode, s);
    };
    return time_loop(launch, n_sets, warmup, iters, use_graph, static_cast<hipStream_t>(stream), elapsed_ms);
}

TUNA_EXPORT int tuna_time_matmul_streams(const void *const *q_list, const void *const *absmax_list, int n_sets, const void *x,
                                         const void *code, void *const *out_list, int n_streams, int m, int n, int k,
                                         const tuna_gemm_config *cfg, int decode_mode, int use_graph, int warmup, int iters,
                                         float *elapsed_ms)
{
    if (!q_list || !absmax_list || !out_list) return fail(TUNA_ERR_INVALID_ARG, "q_list / absmax_list / out_list is null");
    if (n_sets <= 0) return fail(TUNA_ERR_INVALID_ARG, "n_sets must be positive");
    auto launch = [&](int i, int lane, hipStream_t s) {
        return tuna_matmul_ex(q_list[i % n_sets], x, code, absmax_list[i % n_sets], out_list[lane], m, n, k, cfg, decode_mode, s);
    };
    return time_loop_streams(launch, n_streams, use_graph, warmup, iters, elapsed_ms);
}

TUNA_EXPORT int tuna_time_empty_launches(void *sink, int blocks, int threads, int n_streams, int use_graph, int warmup, int iters,
                                         float *elapsed_ms)
{
    int rc;
    if ((rc = check_ptr(sink, "sink", 4))) return rc;
    if (blocks < 1 || threads < 1 || threads > 1024) return fail(TUNA_ERR_INVALID_ARG, "bad launch shape");
    if (n_streams > 1) {
        auto launch = [&](int, int, hipStream_t s) {
            hipError_t e = launch_empty(sink, blocks, threads, s);
            return e == hipSuccess ? (int)TUNA_OK : hip_fail(e, "empty launch");
        };
        return time_loop_streams(launch, n_streams, use_graph, warmup, iters, elapsed_ms);
    }
    hipStream_t st = nullptr;
    hipError_t e = hipStreamCreateWithFlags(&st, hipStreamNonBlocking);
    if (e != hipSuccess) return hip_fail(e, "hipStreamCreate");
    auto launch = [&](int, hipStream_t s) {
        hipError_t e2 = launch_empty(sink, blocks, threads, s);
        return e2 == hipSuccess ? (int)TUNA_OK : hip_fail(e2, "empty launch");
    };
    rc = time_loop(launch, 64, warmup, iters, use_graph, st, elapsed_ms);
    (void)hipStreamDestroy(st);
    return rc;
}

TUNA_EXPORT int tuna_measure_handover(int same_xcd, int store_sc1, int load_sc1, int reuse, int pairs, int iters, void *stream,
                                      double *out6)
{
    if (!out6 || pairs < 1 || pairs > 64 || iters < 1 || iters > 4096) return fail(TUNA_ERR_INVALID_ARG, "bad hand-over yardstick arguments");
    // workgroup L runs on XCD L mod 8 (what the yardstick reports back as the pairs that shared an XCD): partners 8
    // apart share one, neighbours do not
    const hipError_t e = run_handover_yardstick(same_xcd ? 8 : 1, pairs, store_sc1 != 0, load_sc1 != 0, reuse != 0, iters,
                                                static_cast<hipStream_t>(stream), out6);
    return e == hipSuccess ? (int)TUNA_OK : hip_fail(e, "hand-over yardstick");
}

TUNA_EXPORT int tuna_time_matmul_blockwise(const void *const *q_list, const void *const *absmax_list, int n_sets, const void *x,
                                           const void *code, void *out, int m, int n, int k, int block_size,
                                           const tuna_gemm_config *cfg, int warmup, int iters, int use_graph, void *stream,
                                           float *elapsed_ms)
{
    if (!q_list || !absmax_list) return fail(TUNA_ERR_INVALID_ARG, "q_list / absmax_list is null");
    auto launch = [&](int set, hipStream_t s) {
        return tuna_matmul_blockwise_ex(q_list[set], x, code, absmax_list[set], out, m, n, k, block_size, cfg, s);
    };
    return time_loop(launch, n_sets, warmup, iters, use_graph, static_cast<hipStream_t>(stream), elapsed_ms);
}

TUNA_EXPORT int tuna_time_matmul_multi(const tuna_gemm_problem *problems, int n_sets, int count, int warmup, int iters,
                                       int use_graph, void *stream, float *elapsed_ms)
{
    if (!problems || count < 1) return fail(TUNA_ERR_INVALID_ARG, "problems is null or count < 1");
    auto launch = [&](int set, hipStream_t s) { return tuna_matmul_multi(problems + (size_t)set * count, count, s); };
    return time_loop(launch, n_sets, warmup, iters, use_graph, static_cast<hipStream_t>(stream), elapsed_ms);
}

TUNA_EXPORT int tuna_time_matmul_grouped(const void *const *q_list, const void *const *absmax_list, int n_sets, const void *x,
                                         const void *code, void *out, int m_group, int n_groups, int k,
                                         const int32_t *token_offsets, const tuna_gemm_config *cfg, int decode_mode,
                                         int warmup, int iters, int use_graph, void *stream, float *elapsed_ms)
{
    if (!q_list || !absmax_list) return fail(TUNA_ERR_INVALID_ARG, "q_list / absmax_list is null");
    auto launch = [&](int set, hipStream_t s) {
        return tuna_matmul_grouped(q_list[set], x, code, absmax_list[set], out, m_group, n_groups, k, token_offsets, cfg,
                                   decode_mode, s);
    };
    return time_loop(launch, n_sets, warmup, iters, use_graph, static_cast<hipStream_t>(stream), elapsed_ms);
}

TUNA_EXPORT int tuna_time_dequant(const void *const *q_list, const void *const *absmax_list, int n_sets, const void *code,
                                  void *out, int m, int k, int warmup, int iters, void *stream, float *elapsed_ms)
{
    if (!q_list || !absmax_list) return fail(TUNA_ERR_INVALID_ARG, "q_list / absmax_list is null");
    auto launch = [&](int set, hipStream_t s) {
        return tuna_dequant(q_list[set], absmax_list[set], code, out, m, k, s);
    };
    return time_loop(launch, n_sets, warmup, iters, 0, static_cast<hipStream_t>(stream), elapsed_ms);
}

TUNA_EXPORT int tuna_time_copy(const void *src, void *dst, size_t bytes, int warmup, int iters, void *stream,
                               float *elapsed_ms)
{
    int rc;
    if ((rc = check_ptr(src, "src", 16)) || (rc = check_ptr(dst, "dst", 16))) return rc;
    if (bytes == 0 || bytes % 16) return fail(TUNA_ERR_INVALID_ARG, "bytes must be a positive multiple of 16");
    auto launch = [&](int, hipStream_t s) {
        hipError_t e = launch_copy(src, dst, bytes, s);
        return e == hipSuccess ? (int)TUNA_OK : hip_fail(e, "copy launch");
    };
    return time_loop(launch, 1, warmup, iters, 0, static_cast<hipStream_t>(stream), elapsed_ms);
}

TUNA_EXPORT int tuna_time_read(const void *src, void *sink, size_t bytes, int blocks, int variant, int warmup, int iters,
                               void *stream, float *elapsed_ms)
{
    int rc;
    if ((rc = check_ptr(src, "src", 16)) || (rc = check_ptr(sink, "sink", 4))) return rc;
    if (bytes == 0 || bytes % 16) return fail(TUNA_ERR_INVALID_ARG, "bytes must be a positive multiple of 16");
    if (variant < 0 || variant > 5) return fail(TUNA_ERR_INVALID_ARG, "variant %d outside 0..5", variant);
    auto launch = [&](int, hipStream_t s) {
        hipError_t e = launch_read(src, sink, bytes, blocks, variant, s);
        return e == hipSuccess ? (int)TUNA_OK : hip_fail(e, "read launch");
    };
    return time_loop(launch, 1, warmup, iters, 0, static_cast<hipStream_t>(stream), elapsed_ms);
}

TUNA_EXPORT int tuna_time_unit_rate(int unit, void *sink, int warmup, int iters, void *stream, float *elapsed_ms,
                                    double *work_per_launch)
{
    int rc;
    if ((rc = check_ptr(sink, "sink", 4))) return rc;
    if (unit < 0 || unit > 21) return fail(TUNA_ERR_INVALID_ARG, "unit %d outside 0..21", unit);
    if (!work_per_launch) return fail(TUNA_ERR_INVALID_ARG, "work_per_launch is null");
    int dev = 0, cus = 0;
    hipError_t e = device_cus(&dev, &cus);
    if (e != hipSuccess) return hip_fail(e, "device query");
    auto launch = [&](int, hipStream_t s) {
        hipError_t e2 = launch_unit_rate(unit, cus, static_cast<uint32_t *>(sink), work_per_launch, s);
        return e2 == hipSuccess ? (int)TUNA_OK : hip_fail(e2, "unit-rate launch");
    };
    return time_loop(launch, 1, warmup, iters, 0, static_cast<hipStream_t>(stream), elapsed_ms);
}

TUNA_EXPORT int tuna_selftest_quantizer_division(void *counts, void *stream)
{
    int rc = check_ptr(counts, "counts", 8);
    if (rc) return rc;
    hipError_t e = launch_division_selftest(static_cast<unsigned long long *>(counts), static_cast<hipStream_t>(stream));
    if (e != hipSuccess) return hip_fail(e, "selftest launch");
    return TUNA_OK;
}

}  // extern "C"
