// The direct-transport all-reduce under HIP graph capture: a captured sequence of
// launches must replay to the same bits as eager execution, every time.  Replays
// are interleaved with eager work and synchronisation, and every replay is checked.
#include <hip/hip_runtime.h>
#include <stdio.h>
#include <string.h>

#include <vector>

#include "vr_oracle.h"
#include "vrank_allreduce.h"

#define HIPCK(x)                                                                       \
  do {                                                                                 \
    hipError_t e = (x);                                                                \
    if (e != hipSuccess) {                                                             \
      printf("HIP error %s at %s:%d\n", hipGetErrorString(e), __FILE__, __LINE__);      \
      return 2;                                                                        \
    }                                                                                  \
  } while (0)
#define VRCK(x)                                                                        \
  do {                                                                                 \
    int rc = (x);                                                                      \
    if (rc) {                                                                          \
      printf("vr error %s (%s) at %s:%d\n", vr_strerror(rc), vr_last_error_detail(), __FILE__, __LINE__); \
      return 2;                                                                        \
    }                                                                                  \
  } while (0)

int main() {
  const int N = 8;
  const size_t n = 524288;   // the 1 MiB per rank latency configuration
  vr_ctx *ctx;
  VRCK(vr_ctx_create(0, N, &ctx));
  hipStream_t stream;
  HIPCK(hipStreamCreateWithFlags(&stream, hipStreamNonBlocking));

  std::vector<std::vector<uint16_t>> host(N, std::vector<uint16_t>(n));
  void *in[N], *mid[N], *out[N];
  std::vector<const uint16_t *> hp;
  for (int r = 0; r < N; ++r) {
    vro_generate(host[r].data(), n, 300 + r, VRO_DIST_NORMAL, 0.0, 1.0);
    hp.push_back(host[r].data());
    HIPCK(hipMalloc(&in[r], n * 2));
    HIPCK(hipMalloc(&mid[r], n * 2));
    HIPCK(hipMalloc(&out[r], n * 2));
    HIPCK(hipMemcpy(in[r], host[r].data(), n * 2, hipMemcpyHostToDevice));
  }
  // expected: small (rotated) out of place, then bisect in place on the result
  std::vector<uint16_t> s1(n), want(n);
  vro_allreduce_rotated(s1.data(), hp.data(), N, n);
  std::vector<const uint16_t *> same(N, s1.data());
  vro_allreduce_bisect(want.data(), same.data(), N, n);

  int small_id, bisect_id;
  VRCK(vr_algo_from_string("small", &small_id));
  VRCK(vr_algo_from_string("bisect", &bisect_id));
  uint32_t seq = 1;

  hipGraph_t graph;
  hipGraphExec_t exec;
  HIPCK(hipStreamBeginCapture(stream, hipStreamCaptureModeThreadLocal));
  VRCK(vr_allreduce(ctx, stream, small_id, VR_TRANSPORT_DIRECT, in, mid, n, &seq));
  // copy mid -> out with the library's own copy kernel, then reduce in place
  for (int r = 0; r < N; ++r) VRCK(vr_stream_probe(ctx, stream, VR_PROBE_COPY, out[r], mid[r], n * 2));
  VRCK(vr_allreduce(ctx, stream, bisect_id, VR_TRANSPORT_DIRECT, out, nullptr, n, &seq));
  HIPCK(hipStreamEndCapture(stream, &graph));
  HIPCK(hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0));

  std::vector<uint16_t> got(n);
  int failures = 0;
  for (int replay = 0; replay < 6; ++replay) {
    // eager work between replays: scribble over the outputs, synchronise
    for (int r = 0; r < N; ++r) {
      HIPCK(hipMemsetAsync(mid[r], 0x5a, n * 2, stream));
      HIPCK(hipMemsetAsync(out[r], 0xa5, n * 2, stream));
    }
    HIPCK(hipStreamSynchronize(stream));
    HIPCK(hipGraphLaunch(exec, stream));
    HIPCK(hipStreamSynchronize(stream));
    for (int r = 0; r < N; ++r) {
      HIPCK(hipMemcpy(got.data(), out[r], n * 2, hipMemcpyDeviceToHost));
      const size_t bad = vro_count_mismatch(got.data(), want.data(), n);
      if (bad) {
        printf("replay %d rank %d: %zu mismatches\n", replay, r, bad);
        ++failures;
      }
    }
  }
  // launch cost: 50 graph replays vs 50 eager sequences
  hipEvent_t e0, e1;
  HIPCK(hipEventCreate(&e0));
  HIPCK(hipEventCreate(&e1));
  float ms_graph = 0, ms_eager = 0;
  HIPCK(hipEventRecord(e0, stream));
  for (int i = 0; i < 50; ++i) HIPCK(hipGraphLaunch(exec, stream));
  HIPCK(hipEventRecord(e1, stream));
  HIPCK(hipEventSynchronize(e1));
  HIPCK(hipEventElapsedTime(&ms_graph, e0, e1));
  HIPCK(hipEventRecord(e0, stream));
  for (int i = 0; i < 50; ++i) {
    VRCK(vr_allreduce(ctx, stream, small_id, VR_TRANSPORT_DIRECT, in, mid, n, &seq));
    for (int r = 0; r < N; ++r) VRCK(vr_stream_probe(ctx, stream, VR_PROBE_COPY, out[r], mid[r], n * 2));
    VRCK(vr_allreduce(ctx, stream, bisect_id, VR_TRANSPORT_DIRECT, out, nullptr, n, &seq));
  }
  HIPCK(hipEventRecord(e1, stream));
  HIPCK(hipEventSynchronize(e1));
  HIPCK(hipEventElapsedTime(&ms_eager, e0, e1));
  printf("10-kernel sequence: graph replay %.1f us, eager %.1f us\n", ms_graph * 1e3 / 50, ms_eager * 1e3 / 50);

  // The wire transport refuses capture: its flag values are per-launch kernel
  // arguments, so a replay would read stale flags.
  {
    int parallel_id = -1;
    VRCK(vr_algo_from_string("parallel", &parallel_id));
    VRCK(vr_ctx_reserve_wire(ctx));
    hipGraph_t g2;
    HIPCK(hipStreamBeginCapture(stream, hipStreamCaptureModeThreadLocal));
    const int rc = vr_allreduce(ctx, stream, parallel_id, VR_TRANSPORT_WIRE, in, mid, n, &seq);
    HIPCK(hipStreamEndCapture(stream, &g2));
    (void)hipGraphDestroy(g2);
    if (rc != VR_ERR_INVALID) {
      printf("wire launch under capture returned %d, expected VR_ERR_INVALID\n", rc);
      ++failures;
    }
    // and works again outside capture
    VRCK(vr_allreduce(ctx, stream, parallel_id, VR_TRANSPORT_WIRE, in, mid, n, &seq));
    VRCK(vr_ctx_check(ctx, stream));
  }

  // The allocation-free wire all-reduce clears its sinks in every call and starts
  // its flags from 1, so a captured call replays correctly: six replays with
  // eager work in between, each compared with the oracle.
  {
    int parallel_id = -1;
    VRCK(vr_algo_from_string("parallel", &parallel_id));
    const std::vector<uint16_t> &sum = s1;       // the rotated-order sum of the inputs
    hipGraph_t g3;
    hipGraphExec_t e3;
    HIPCK(hipStreamBeginCapture(stream, hipStreamCaptureModeThreadLocal));
    VRCK(vr_allreduce_static(ctx, stream, parallel_id, in, mid, n));
    HIPCK(hipStreamEndCapture(stream, &g3));
    HIPCK(hipGraphInstantiate(&e3, g3, nullptr, nullptr, 0));
    for (int replay = 0; replay < 6; ++replay) {
      for (int r = 0; r < N; ++r) HIPCK(hipMemsetAsync(mid[r], 0x3c, n * 2, stream));
      // an eager call between replays leaves other flags in the shared sinks
      if (replay % 2) VRCK(vr_allreduce_static(ctx, stream, bisect_id, in, out, n));
      HIPCK(hipStreamSynchronize(stream));
      HIPCK(hipGraphLaunch(e3, stream));
      VRCK(vr_ctx_check(ctx, stream));
      for (int r = 0; r < N; ++r) {
        HIPCK(hipMemcpy(got.data(), mid[r], n * 2, hipMemcpyDeviceToHost));
        const size_t bad = vro_count_mismatch(got.data(), sum.data(), n);
        if (bad) {
          printf("static replay %d rank %d: %zu mismatches\n", replay, r, bad);
          ++failures;
        }
      }
    }
    (void)hipGraphExecDestroy(e3);
    (void)hipGraphDestroy(g3);
  }

  // A streaming launch under capture: two ranks of 80 MiB, out of place, run as a one-trip
  // grid whose residency is capped with 75 KiB of dynamic LDS per work-group.  This is the
  // first launch of that kernel in the process, so the kernel's dynamic-LDS allowance is
  // raised while the stream is capturing.  Three replays against the oracle.
  {
    const size_t n2 = 41943040;
    vr_ctx *c2;
    VRCK(vr_ctx_create(0, 2, &c2));
    int simple_id = -1;
    VRCK(vr_algo_from_string("simple", &simple_id));
    std::vector<std::vector<uint16_t>> h2(2, std::vector<uint16_t>(n2));
    void *i2[2], *o2[2];
    const uint16_t *hp2[2];
    for (int r = 0; r < 2; ++r) {
      vro_generate(h2[r].data(), n2, 900 + r, VRO_DIST_NORMAL, 0.0, 0.02);
      hp2[r] = h2[r].data();
      HIPCK(hipMalloc(&i2[r], n2 * 2));
      HIPCK(hipMalloc(&o2[r], n2 * 2));
      HIPCK(hipMemcpy(i2[r], h2[r].data(), n2 * 2, hipMemcpyHostToDevice));
    }
    std::vector<uint16_t> want2(n2), got2(n2);
    vro_allreduce_rotated(want2.data(), hp2, 2, n2);
    hipGraph_t g4;
    hipGraphExec_t e4;
    uint32_t seq2 = 1;
    HIPCK(hipStreamBeginCapture(stream, hipStreamCaptureModeThreadLocal));
    VRCK(vr_allreduce(c2, stream, simple_id, VR_TRANSPORT_DIRECT, i2, o2, n2, &seq2));
    HIPCK(hipStreamEndCapture(stream, &g4));
    HIPCK(hipGraphInstantiate(&e4, g4, nullptr, nullptr, 0));
    for (int replay = 0; replay < 3; ++replay) {
      for (int r = 0; r < 2; ++r) HIPCK(hipMemsetAsync(o2[r], 0x77, n2 * 2, stream));
      HIPCK(hipStreamSynchronize(stream));
      HIPCK(hipGraphLaunch(e4, stream));
      HIPCK(hipStreamSynchronize(stream));
      for (int r = 0; r < 2; ++r) {
        HIPCK(hipMemcpy(got2.data(), o2[r], n2 * 2, hipMemcpyDeviceToHost));
        const size_t bad = vro_count_mismatch(got2.data(), want2.data(), n2);
        if (bad) {
          printf("streaming replay %d rank %d: %zu mismatches\n", replay, r, bad);
          ++failures;
        }
      }
    }
    (void)hipGraphExecDestroy(e4);
    (void)hipGraphDestroy(g4);
    for (int r = 0; r < 2; ++r) {
      (void)hipFree(i2[r]);
      (void)hipFree(o2[r]);
    }
    vr_ctx_destroy(c2);
  }

  (void)hipGraphExecDestroy(exec);
  (void)hipGraphDestroy(graph);
  for (int r = 0; r < N; ++r) {
    (void)hipFree(in[r]);
    (void)hipFree(mid[r]);
    (void)hipFree(out[r]);
  }
  (void)hipStreamDestroy(stream);
  vr_ctx_destroy(ctx);
  if (failures) {
    printf("%d failure(s)\n", failures);
    return 1;
  }
  printf("graph ok\n");
  return 0;
}
