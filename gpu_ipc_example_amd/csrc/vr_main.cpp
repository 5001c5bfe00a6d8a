// vr_main — command-line harness of the virtual-rank all-reduce, with the flags
// and the run protocol of the reference's main.cpp:
//   -n/--nelems "8MB"  elements per rank, K/M/G suffix = x1024     (main.cpp:17-34, 177)
//   -g/--groups, -w/--subgroups, -s/--simd   launch grid           (main.cpp:179-187, 289-294)
//   -f/--flag          first sequence number (default 0xe00f100f)  (main.cpp:183)
//   -v/--verify        check run #1 against the host sum and stop  (main.cpp:75-84)
//   -a/--algo          small | simple | bisect | ... | allgather_* (main.cpp:190, 296)
// plus what one process driving all ranks needs:
//   -r/--ranks N       number of virtual ranks (the MPI world size of the reference)
//   -t/--transport     direct | wire
//   -d/--device        HIP device index
//   --dtype            f16 | bf16 (the reference is built for one test_type, main.cpp:45)
// and, for the reference's own shape of one process per rank (mpirun -np N ./main):
//   --rank R           this process is rank R of the -r N ranks; it owns its input and
//                      scratch, maps every peer's scratch through the IPC exchange
//                      (main.cpp:241-283, ipc_exchange.cpp) and launches its own wires only
//                      (all-reduce and all-gather alike, main.cpp:296-314)
//   --ranks-here K     with --rank R: this process holds the K ranks R .. R+K-1 (R a
//                      multiple of K) and enqueues them as one launch; N / K processes
//   -i/--instance S    socket-name suffix shared by the processes of one run (main.cpp:194)
//   --seed S           seeded N(0,1) inputs (rank r uses S + r) instead of fill_pattern
//   --dump FILE        write this rank's result (raw 16-bit elements) to FILE
// Run protocol (main.cpp:48-109): run #1 with `flag`; with -v verify and return;
// otherwise two more warm-ups (flag+100, flag+150), then the timed run (flag+200)
// whose kernel time is printed as "[rank] Running time: <ns>ns" for every rank.
// All runs are in place on the same inputs, exactly like the reference.

#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include <stdexcept>
#include <string>
#include <vector>

#include "vrank/allreduce.hpp"

namespace {

struct Options {
  std::string nelems = "8MB", algo = "small", transport = "default", dtype = "f16";
  size_t groups = 1, subgroups = 4, flag = 0xe00f100f;
  uint32_t simd = 16;
  bool verify = false, grid_given = false;
  int ranks = 8, device = 0;
  int rank = -1;                     // >= 0: one process per rank (or per ranks_here ranks)
  int ranks_here = 1;
  std::string instance = "0", dump;
  long long seed = -1;
  unsigned long long spin = 0;
};

bool take(int &i, int argc, char **argv, const char *s, const char *l, std::string *out) {
  const std::string a = argv[i];
  const std::string ls = std::string("--") + l, ss = std::string("-") + s;
  if (a == ls || a == ss) {
    if (i + 1 >= argc) throw std::invalid_argument("missing value for " + a);
    *out = argv[++i];
    return true;
  }
  if (a.rfind(ls + "=", 0) == 0) { *out = a.substr(ls.size() + 1); return true; }
  if (a.rfind(ss, 0) == 0 && a.size() > 2 && a[1] != '-') { *out = a.substr(2); return true; }  // -g64
  return false;
}

Options parse(int argc, char **argv) {
  Options o;
  for (int i = 1; i < argc; ++i) {
    std::string v;
    const std::string a = argv[i];
    if (a == "-v" || a == "--verify") { o.verify = true; continue; }
    if (a == "-h" || a == "--help") {
      printf("usage: vr_main [-n 8MB] [-r 8] [-a small|simple|bisect|parallel|small_ring|simple_ring|"
             "small_pcie|simple_pcie|small_pcie_p|simple_pcie_p|simple_transmit|allgather_small|allgather_simple]\n"
             "               [-g groups -w subgroups -s simd] [-f flag] [-t direct|wire] [-d device]\n"
             "               [--dtype f16|bf16] [-v]\n"
             "               [--rank R [--ranks-here K] -i instance [--seed S] [--dump FILE]]   one process per rank (or K ranks)\n");
      exit(0);
    }
    if (take(i, argc, argv, "n", "nelems", &v)) o.nelems = v;
    else if (take(i, argc, argv, "g", "groups", &v)) { o.groups = strtoull(v.c_str(), nullptr, 0); o.grid_given = true; }
    else if (take(i, argc, argv, "w", "subgroups", &v)) { o.subgroups = strtoull(v.c_str(), nullptr, 0); o.grid_given = true; }
    else if (take(i, argc, argv, "f", "flag", &v)) o.flag = strtoull(v.c_str(), nullptr, 0);
    else if (take(i, argc, argv, "s", "simd", &v)) o.simd = (uint32_t)strtoul(v.c_str(), nullptr, 0);
    else if (take(i, argc, argv, "a", "algo", &v)) o.algo = v;
    else if (take(i, argc, argv, "r", "ranks", &v)) o.ranks = atoi(v.c_str());
    else if (take(i, argc, argv, "t", "transport", &v)) o.transport = v;
    else if (take(i, argc, argv, "d", "device", &v)) o.device = atoi(v.c_str());
    else if (take(i, argc, argv, "D", "dtype", &v)) o.dtype = v;
    else if (take(i, argc, argv, "R", "rank", &v)) o.rank = atoi(v.c_str());
    else if (take(i, argc, argv, "K", "ranks-here", &v)) o.ranks_here = atoi(v.c_str());
    else if (take(i, argc, argv, "i", "instance", &v)) o.instance = v;
    else if (take(i, argc, argv, "S", "seed", &v)) o.seed = atoll(v.c_str());
    else if (take(i, argc, argv, "O", "dump", &v)) o.dump = v;
    else if (take(i, argc, argv, "P", "spin", &v)) o.spin = strtoull(v.c_str(), nullptr, 0);
    // the reference ignores what it does not know (allow_unrecognised_options)
  }
  return o;
}

// The element type of the run: the reference is compiled for one test_type
// (main.cpp:45); here --dtype picks it, and the checks of vrank/allreduce.hpp
// (verifyTransmit / verifyAllgather <- allreduce.cpp:519-585, 832-838) are called
// for that type.
int g_dtype = VR_DTYPE_F16;
typedef unsigned short half_bits;

size_t verify_reduced(std::vector<uint16_t> &got, int rank, int world, size_t nelems) {
  size_t bad = 0;
  if (g_dtype == VR_DTYPE_BF16)
    vrank::verifyTransmit<vrank::bfloat16>(nullptr, reinterpret_cast<vrank::bfloat16 *>(got.data()), 0, rank, world,
                                           16, nelems, &bad);
  else
    vrank::verifyTransmit<half_bits>(nullptr, got.data(), 0, rank, world, 16, nelems, &bad);
  return bad;
}

size_t verify_gathered(std::vector<uint16_t> &got, int rank, int world, size_t nelems) {
  size_t bad = 0;
  if (g_dtype == VR_DTYPE_BF16)
    vrank::verifyAllgather<vrank::bfloat16>(reinterpret_cast<vrank::bfloat16 *>(got.data()), rank, world, nelems, &bad);
  else
    vrank::verifyAllgather<half_bits>(got.data(), rank, world, nelems, &bad);
  return bad;
}

int verify_allreduce(std::vector<std::vector<uint16_t>> &got, int world, size_t nelems) {
  size_t bad = 0;
  for (int rank = 0; rank < world; ++rank) bad += verify_reduced(got[rank], rank, world, nelems);
  if (bad == 0) printf("verify: %d ranks x %zu elements match the host sum\n", world, nelems);
  else printf("verify: %zu mismatches\n", bad);
  return 0;   // the reference's verify never fails the process (allreduce.cpp:550)
}

int verify_allgather(std::vector<std::vector<uint16_t>> &got, int world, size_t nelems) {
  size_t bad = 0;
  for (int rank = 0; rank < world; ++rank) bad += verify_gathered(got[rank], rank, world, nelems);
  if (bad == 0) printf("verify: %d ranks x %zu gathered elements match\n", world, nelems * world);
  else printf("verify: %zu mismatches\n", bad);
  return 0;
}

// One process per rank, the reference's own arrangement (main.cpp:212-314): this
// process owns the input (for the all-gather also the output) and the scratch of
// its ranks (scatter sink | gather sink each, the ipcbuf0 | ipcbuf1 of
// main.cpp:241-243, in one allocation), zeroes the scratch once, maps every peer
// process's scratch (open_all_ipc_mems, main.cpp:256), builds peerbuf0 / peerbuf1
// (main.cpp:260-269), waits for all processes (MPI_Barrier, main.cpp:287) and runs
// its own wires against them: benchAllreduce / benchAllgather (main.cpp:48-166).
int run_as_rank(const Options &o, int algo, size_t nelems, bool gather) {
  const int world = o.ranks, first = o.rank, K = o.ranks_here;
  if (K < 1 || world % K || first % K || first + K > world)
    throw std::invalid_argument("--rank must be a multiple of --ranks-here, which must divide -r");
  if (K > 1 && o.grid_given)
    throw std::invalid_argument("-g / -w / -s apply to one rank per process (--ranks-here 1)");
  const int nprocs = world / K, proc = first / K;
  vrank::VirtualRanks ranks(world, o.device);
  ranks.setDtype(g_dtype);
  if (o.spin) vrank::check(vr_ctx_set_spin_limit(ranks.get(), o.spin));
  size_t sink = 0;
  vrank::check(vr_rank_scratch_bytes(ranks.get(), &sink));
  const size_t alloc = nelems * sizeof(uint16_t);
  void *input[VR_MAX_RANKS] = {}, *output[VR_MAX_RANKS] = {}, *scratch = nullptr;
  vrank::check(vr_malloc(o.device, 2 * sink * K, &scratch));
  vrank::check(vr_memset(scratch, 0, 2 * sink * K));                          // main.cpp:251
  std::vector<uint16_t> host(nelems);
  for (int i = 0; i < K; ++i) {
    const int rank = first + i;
    vrank::check(vr_malloc(o.device, alloc, &input[i]));
    if (o.seed >= 0) vr_generate_dt(g_dtype, host.data(), nelems, (uint64_t)o.seed + (uint64_t)rank, 1, 0.0, 1.0);
    else vr_fill_pattern_dt(g_dtype, host.data(), rank, nelems);
    vrank::check(vr_copy_to_device(input[i], host.data(), alloc));
    if (gather) {
      vrank::check(vr_malloc(o.device, alloc * world, &output[i]));
      vrank::check(vr_memset(output[i], 1, alloc * world));                   // main.cpp:300
    }
  }

  void *bases[VR_MAX_RANKS] = {};
  size_t offsets[VR_MAX_RANKS] = {};
  vrank::check(vr_ipc_open_all(scratch, proc, nprocs, bases, offsets, o.instance.c_str()));
  void *peerbuf0[VR_MAX_RANKS] = {}, *peerbuf1[VR_MAX_RANKS] = {};
  for (int r = 0; r < world; ++r) {
    peerbuf0[r] = static_cast<char *>(bases[r / K]) + offsets[r / K] + (size_t)(r % K) * 2 * sink;
    peerbuf1[r] = static_cast<char *>(peerbuf0[r]) + sink;
  }
  int generation = 0;
  vrank::check(vr_ipc_barrier(proc, nprocs, o.instance.c_str(), ++generation));   // every scratch is zeroed

  void *stream = nullptr;
  vrank::check(vr_stream_create(o.device, &stream));
  void *ev0 = nullptr, *ev1 = nullptr;
  vrank::check(vr_event_create(&ev0));
  vrank::check(vr_event_create(&ev1));
  // The reference's four runs use the fixed flags flag, +100, +150, +200 on scratch
  // that is zeroed once (main.cpp:67-106, 251): sound while one run consumes at most
  // 50 flag values.  A shape that needs more gets freshly zeroed sinks before every
  // further run instead of silently accepting stale messages.
  uint32_t flags_per_run = 0;
  vrank::check(vr_rank_flags_used(ranks.get(), algo, nelems, o.grid_given ? (uint32_t)o.groups : 0u,
                                  o.grid_given ? (uint32_t)o.subgroups : 0u, &flags_per_run));
  const bool rezero = flags_per_run > 50;
  auto run = [&](uint32_t flag) {
    uint32_t step = flag;
    vr_ctx *c = ranks.get();
    if (K > 1) {
      if (gather) vrank::check(vr_allgather_ranks(c, stream, algo, first, K, input, output, peerbuf0, peerbuf1, sink, nelems, &step));
      else vrank::check(vr_allreduce_ranks(c, stream, algo, first, K, input, nullptr, peerbuf0, peerbuf1, sink, nelems, &step));
    } else if (gather) {
      if (o.grid_given)   // testAllgather with the -g / -w / -s grid (main.cpp:110-166, 293-307)
        vrank::check(vr_allgather_rank_grid(c, stream, algo, first, input[0], output[0], peerbuf0[first], peerbuf1[first],
                                            peerbuf0, peerbuf1, sink, nelems, flag, (uint32_t)o.groups,
                                            (uint32_t)o.subgroups, o.simd));
      else
        vrank::check(vr_allgather_rank(c, stream, algo, first, input[0], output[0], peerbuf0[first], peerbuf1[first],
                                       peerbuf0, peerbuf1, sink, nelems, &step));
    } else if (o.grid_given) {   // testTransmit with the -g / -w / -s grid (main.cpp:67-71, 289-294)
      vrank::check(vr_allreduce_rank_grid(c, stream, algo, first, input[0], nullptr, peerbuf0[first], peerbuf1[first],
                                          peerbuf0, peerbuf1, sink, nelems, flag, (uint32_t)o.groups,
                                          (uint32_t)o.subgroups, o.simd));
    } else {
      vrank::check(vr_allreduce_rank(c, stream, algo, first, input[0], nullptr, peerbuf0[first], peerbuf1[first],
                                     peerbuf0, peerbuf1, sink, nelems, &step));
    }
  };
  auto fresh_sinks = [&]() {
    ranks.wait(stream);
    vrank::check(vr_ipc_barrier(proc, nprocs, o.instance.c_str(), ++generation));   // nobody still writes
    vrank::check(vr_memset(scratch, 0, 2 * sink * K));
    vrank::check(vr_ipc_barrier(proc, nprocs, o.instance.c_str(), ++generation));   // every scratch is zeroed
  };
  int status = 0;
  run((uint32_t)o.flag);
  ranks.wait(stream);
  if (o.verify || !o.dump.empty()) {
    const size_t count = gather ? nelems * world : nelems;
    for (int i = 0; i < K; ++i) {
      const int rank = first + i;
      std::vector<uint16_t> got(count);
      vrank::check(vr_copy_to_host(got.data(), gather ? output[i] : input[i], count * 2));
      if (!o.dump.empty()) {
        const std::string name = K > 1 ? o.dump + "." + std::to_string(rank) : o.dump;
        FILE *f = fopen(name.c_str(), "wb");
        if (!f || fwrite(got.data(), 2, count, f) != count) throw std::runtime_error("cannot write " + name);
        fclose(f);
      }
      if (o.verify && o.seed < 0) {
        // verifyTransmit / verifyAllgather for this rank's copy (main.cpp:75-84, 137-146)
        const size_t bad = gather ? verify_gathered(got, rank, world, nelems) : verify_reduced(got, rank, world, nelems);
        if (bad == 0) printf(gather ? "[%d] verify: %zu gathered elements match\n" : "[%d] verify: %zu elements match the host sum\n", rank, count);
        else printf("[%d] verify: %zu mismatches\n", rank, bad);
      }
    }
  } else {
    if (rezero) fresh_sinks();
    run((uint32_t)o.flag + 100);
    if (rezero) fresh_sinks();
    run((uint32_t)o.flag + 150);
    if (rezero) fresh_sinks();
    ranks.wait(stream);
    vrank::check(vr_ipc_barrier(proc, nprocs, o.instance.c_str(), ++generation));  // main.cpp:101, 157
    vrank::check(vr_event_record(ev0, stream));
    run((uint32_t)o.flag + 200);
    vrank::check(vr_event_record(ev1, stream));
    float ms = 0.f;
    vrank::check(vr_event_elapsed_ms(ev0, ev1, &ms));
    ranks.wait(stream);
    for (int i = 0; i < K; ++i)
      printf("[%d] Running time: %lluns\n", first + i, (unsigned long long)(ms * 1e6));
  }
  // nobody unmaps or frees while a peer may still be writing into it
  vrank::check(vr_ipc_barrier(proc, nprocs, o.instance.c_str(), ++generation));
  vrank::check(vr_ipc_close_all(proc, nprocs, bases));
  vr_event_destroy(ev0);
  vr_event_destroy(ev1);
  vr_stream_destroy(stream);
  for (int i = 0; i < K; ++i) {
    vr_free(input[i]);
    vr_free(output[i]);
  }
  vr_free(scratch);
  return status;
}

}  // namespace

int main(int argc, char **argv) try {
  const Options o = parse(argc, argv);
  size_t nelems = 0;
  vrank::check(vr_parse_nelems(o.nelems.c_str(), &nelems));
  const int world = o.ranks;
  const bool gather = o.algo.find("allgather") != std::string::npos;
  int algo = -1;
  vrank::check(vr_algo_from_string(o.algo.c_str(), &algo));

  if (o.grid_given && o.subgroups % 4 != 0)
    throw std::logic_error("Subgroup numbers must be multiple of 4");   // main.cpp:289-291

  if (o.dtype == "bf16") g_dtype = VR_DTYPE_BF16;
  else if (o.dtype != "f16") throw std::invalid_argument("dtype must be f16 or bf16");

  if (o.rank >= 0) return run_as_rank(o, algo, nelems, gather);

  vrank::VirtualRanks ranks(world, o.device);
  ranks.setDtype(g_dtype);
  if (o.transport == "direct") ranks.setTransport(VR_TRANSPORT_DIRECT);
  else if (o.transport == "wire") ranks.setTransport(VR_TRANSPORT_WIRE);
  else if (o.transport != "default") throw std::invalid_argument("transport must be direct or wire");

  const size_t alloc = nelems * sizeof(uint16_t);
  std::vector<void *> input(world, nullptr), output(world, nullptr);
  std::vector<uint16_t> host(nelems);
  for (int r = 0; r < world; ++r) {
    vrank::check(vr_malloc(o.device, alloc, &input[r]));
    vr_fill_pattern_dt(g_dtype, host.data(), r, nelems);
    vrank::check(vr_copy_to_device(input[r], host.data(), alloc));
    if (gather) {
      vrank::check(vr_malloc(o.device, alloc * world, &output[r]));
      vrank::check(vr_memset(output[r], 1, alloc * world));          // main.cpp:300
    }
  }
  void *stream = nullptr;
  vrank::check(vr_stream_create(o.device, &stream));
  void *ev0 = nullptr, *ev1 = nullptr;
  vrank::check(vr_event_create(&ev0));
  vrank::check(vr_event_create(&ev1));

  auto run = [&](uint32_t flag) {
    uint32_t step = flag;
    if (gather && o.grid_given) {   // testAllgather with the -g / -w / -s grid (main.cpp:293-307)
      vrank::check(vr_allgather_grid(ranks.get(), stream, algo, ranks.transportFor(algo),
                                     (const void *const *)input.data(), output.data(), nelems, flag,
                                     (uint32_t)o.groups, (uint32_t)o.subgroups, o.simd));
    } else if (gather) {
      vrank::check(vr_allgather(ranks.get(), stream, algo, ranks.transportFor(algo),
                                (const void *const *)input.data(), output.data(), nelems, &step));
    } else if (o.grid_given) {
      vrank::check(vr_allreduce_grid(ranks.get(), stream, algo, ranks.transportFor(algo), input.data(),
                                     nullptr, nelems, flag, (uint32_t)o.groups,
                                     (uint32_t)o.subgroups, o.simd));
    } else {
      vrank::check(vr_allreduce(ranks.get(), stream, algo, ranks.transportFor(algo), input.data(), nullptr,
                                nelems, &step));
    }
  };

  run((uint32_t)o.flag);
  ranks.wait(stream);

  if (o.verify) {
    std::vector<std::vector<uint16_t>> got(world);
    for (int r = 0; r < world; ++r) {
      got[r].resize(gather ? nelems * world : nelems);
      vrank::check(vr_copy_to_host(got[r].data(), gather ? output[r] : input[r], got[r].size() * 2));
    }
    return gather ? verify_allgather(got, world, nelems) : verify_allreduce(got, world, nelems);
  }

  run((uint32_t)o.flag + 100);
  run((uint32_t)o.flag + 150);
  printf("---------last run------------------\n");
  ranks.wait(stream);
  vrank::check(vr_event_record(ev0, stream));
  run((uint32_t)o.flag + 200);
  vrank::check(vr_event_record(ev1, stream));
  float ms = 0.f;
  vrank::check(vr_event_elapsed_ms(ev0, ev1, &ms));
  ranks.wait(stream);
  for (int r = 0; r < world; ++r) printf("[%d] Running time: %lluns\n", r, (unsigned long long)(ms * 1e6));
  const double bytes = gather ? (double)world * alloc + (double)world * world * alloc
                              : 2.0 * world * alloc;
  printf("%s: %d ranks x %zu halves, %.3f us, %.1f GB/s algorithmic (2*N*S%s)\n", o.algo.c_str(),
         world, nelems, ms * 1e3, bytes / (ms * 1e-3) / 1e9, gather ? " -> N*S + N*N*S" : "");

  vr_event_destroy(ev0);
  vr_event_destroy(ev1);
  vr_stream_destroy(stream);
  for (int r = 0; r < world; ++r) {
    vr_free(input[r]);
    vr_free(output[r]);
  }
  return 0;
} catch (const std::exception &e) {
  fprintf(stderr, "vr_main: %s\n", e.what());
  return 1;
}
