// Inter-process exchange of device-memory handles: what lets the ranks of an
// all-reduce live in separate processes, each owning its input and scratch and
// mapping every peer's scratch.  Follows the reference's ipc_exchange.cpp:
//   open_all_ipc_mems (l.277-311): base address + offset of the pointer, IPC handle
//     of the base, all-gather of {handle, offset, pid}, open every peer's handle;
//   un_allgather (l.173-265): every rank listens on an AF_UNIX socket named after
//     its rank and the instance, connects to every peer and sends its record.
// A HIP IPC handle is 64 plain bytes, so no descriptor passing (SCM_RIGHTS,
// l.60-99) is needed; the records travel as ordinary stream data.

#include <errno.h>
#include <poll.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <sys/socket.h>
#include <sys/types.h>
#include <sys/un.h>
#include <time.h>
#include <unistd.h>

#include <string>
#include <vector>

#include "vr_host.h"

static int api_fail(int status, const std::string &detail) { return vr::fail(status, detail); }

namespace {

// A peer that never shows up ends the exchange with an error after 30 s
// (VRANK_IPC_TIMEOUT_MS overrides, for tests of that path).
int timeout_ms() {
  const char *env = getenv("VRANK_IPC_TIMEOUT_MS");
  const int v = env ? atoi(env) : 0;
  return v > 0 ? v : 30000;
}

double now_ms() {
  timespec ts;
  clock_gettime(CLOCK_MONOTONIC, &ts);
  return ts.tv_sec * 1e3 + ts.tv_nsec * 1e-6;
}

// ipc_exchange.cpp:159-160: one socket name per rank and instance.
std::string socket_name(const char *instance, const char *tag, int rank) {
  const char *dir = getenv("TMPDIR");
  if (!dir || !*dir) dir = "/tmp";
  return std::string(dir) + "/vrank-ipc-" + instance + "-" + tag + "-rank_" + std::to_string(rank);
}

bool fill_addr(const std::string &name, sockaddr_un *un, socklen_t *len) {
  memset(un, 0, sizeof *un);
  un->sun_family = AF_UNIX;
  if (name.size() >= sizeof un->sun_path) return false;
  memcpy(un->sun_path, name.c_str(), name.size());
  *len = (socklen_t)(offsetof(sockaddr_un, sun_path) + name.size());
  return true;
}

bool send_all(int fd, const void *buf, size_t n) {
  const char *p = static_cast<const char *>(buf);
  while (n) {
    const ssize_t k = send(fd, p, n, MSG_NOSIGNAL);
    if (k < 0) {
      if (errno == EINTR) continue;
      return false;
    }
    p += k;
    n -= (size_t)k;
  }
  return true;
}

bool recv_all(int fd, void *buf, size_t n, double deadline) {
  char *p = static_cast<char *>(buf);
  while (n) {
    pollfd pf = {fd, POLLIN, 0};
    const double left = deadline - now_ms();
    if (left <= 0 || poll(&pf, 1, (int)left) <= 0) return false;
    const ssize_t k = recv(fd, p, n, 0);
    if (k < 0 && errno == EINTR) continue;
    if (k <= 0) return false;
    p += k;
    n -= (size_t)k;
  }
  return true;
}

// All-gather of one fixed-size record per rank (un_allgather, ipc_exchange.cpp:173-265):
// listen on the own name, connect to every peer in the order rank+1, rank+2, ...
// and send {rank, record}; accept world-1 connections and file what arrives under
// the sender's rank.  A pending connection waits in the listener's backlog, so
// all ranks may connect before any of them accepts.
int un_allgather(const void *send_rec, void *recv_recs, size_t rec_bytes, int rank, int world,
                 const char *instance, const char *tag) {
  const std::string mine = socket_name(instance, tag, rank);
  sockaddr_un un;
  socklen_t len;
  if (!fill_addr(mine, &un, &len)) return api_fail(VR_ERR_INVALID, "socket name too long: " + mine);
  const int lsock = socket(AF_UNIX, SOCK_STREAM, 0);
  if (lsock < 0) return api_fail(VR_ERR_INVALID, std::string("socket: ") + strerror(errno));
  unlink(mine.c_str());
  int rc = VR_OK;
  std::vector<char> msg(sizeof(int) + rec_bytes);
  const double deadline = now_ms() + timeout_ms();
  if (bind(lsock, (sockaddr *)&un, len) < 0 || listen(lsock, world + 8) < 0) {
    rc = api_fail(VR_ERR_INVALID, "bind/listen " + mine + ": " + strerror(errno));
  }
  // connect to the peers and send
  for (int i = 1; i < world && rc == VR_OK; ++i) {
    const int peer = (rank + i) % world;
    const std::string theirs = socket_name(instance, tag, peer);
    sockaddr_un pun;
    socklen_t plen;
    fill_addr(theirs, &pun, &plen);
    int fd = -1;
    for (;;) {
      fd = socket(AF_UNIX, SOCK_STREAM, 0);
      if (fd >= 0 && connect(fd, (sockaddr *)&pun, plen) == 0) break;
      const int err = errno;
      if (fd >= 0) close(fd);
      fd = -1;
      if ((err != ECONNREFUSED && err != ENOENT) || now_ms() > deadline) {
        rc = api_fail(VR_ERR_TIMEOUT, "rank " + std::to_string(rank) + " could not reach rank " +
                                          std::to_string(peer) + " (" + strerror(err) + ")");
        break;
      }
      usleep(1000);   // the peer has not bound its socket yet (ipc_exchange.cpp:147-151)
    }
    if (fd < 0) break;
    memcpy(msg.data(), &rank, sizeof(int));
    memcpy(msg.data() + sizeof(int), send_rec, rec_bytes);
    if (!send_all(fd, msg.data(), msg.size()))
      rc = api_fail(VR_ERR_INVALID, std::string("send: ") + strerror(errno));
    close(fd);
  }
  // accept the peers' records
  for (int got = 0; got < world - 1 && rc == VR_OK; ++got) {
    pollfd pf = {lsock, POLLIN, 0};
    const double left = deadline - now_ms();
    if (left <= 0 || poll(&pf, 1, (int)left) <= 0) {
      rc = api_fail(VR_ERR_TIMEOUT, "rank " + std::to_string(rank) + " heard from " + std::to_string(got) +
                                        " of " + std::to_string(world - 1) + " peers");
      break;
    }
    const int fd = accept(lsock, nullptr, nullptr);
    if (fd < 0) {
      rc = api_fail(VR_ERR_INVALID, std::string("accept: ") + strerror(errno));
      break;
    }
    int from = -1;
    if (!recv_all(fd, msg.data(), msg.size(), deadline)) {
      rc = api_fail(VR_ERR_TIMEOUT, "short record from a peer");
    } else {
      memcpy(&from, msg.data(), sizeof(int));
      if (from < 0 || from >= world || from == rank)
        rc = api_fail(VR_ERR_INVALID, "record from rank " + std::to_string(from));
      else
        memcpy(static_cast<char *>(recv_recs) + (size_t)from * rec_bytes, msg.data() + sizeof(int), rec_bytes);
    }
    close(fd);
  }
  memcpy(static_cast<char *>(recv_recs) + (size_t)rank * rec_bytes, send_rec, rec_bytes);
  close(lsock);
  unlink(mine.c_str());
  return rc;
}

struct ExchangeContents {       // ipc_exchange.cpp:38-47
  hipIpcMemHandle_t ipc_handle;
  size_t offset;
  int pid;
};

}  // namespace

extern "C" int vr_ipc_open_all(void *ptr, int rank, int world, void *peer_bases[], size_t offsets[],
                               const char *instance) {
  if (!ptr || !peer_bases || !offsets || !instance) return api_fail(VR_ERR_INVALID, "null argument");
  if (world < 2 || world > VR_MAX_RANKS || rank < 0 || rank >= world)
    return api_fail(VR_ERR_INVALID, "rank / world out of range");
  // Step 1: base address of the allocation the pointer lies in (zeMemGetAddressRange, l.285-287).
  hipDeviceptr_t base = nullptr;
  size_t base_size = 0;
  hipError_t e = hipMemGetAddressRange(&base, &base_size, ptr);
  if (e != hipSuccess) return api_fail(VR_ERR_HIP, std::string("hipMemGetAddressRange: ") + hipGetErrorString(e));
  // Opening a mapping of 2 GiB or more has been seen not to return.
  if (base_size >= (2ull << 30))
    return api_fail(VR_ERR_INVALID, "shared allocations must stay under 2 GiB, this one has " +
                                        std::to_string(base_size) + " bytes");
  // Step 2: handle of the base, offset of the pointer inside it (l.289-296).
  ExchangeContents mine;
  memset(&mine, 0, sizeof mine);
  e = hipIpcGetMemHandle(&mine.ipc_handle, base);
  if (e != hipSuccess) return api_fail(VR_ERR_HIP, std::string("hipIpcGetMemHandle: ") + hipGetErrorString(e));
  mine.offset = (size_t)(static_cast<char *>(ptr) - static_cast<char *>(base));
  mine.pid = (int)getpid();
  // Step 3: exchange (l.298-301).
  std::vector<ExchangeContents> all((size_t)world);
  if (int rc = un_allgather(&mine, all.data(), sizeof mine, rank, world, instance, "mem")) return rc;
  // Step 4: open every peer's handle (l.303-320).
  for (int i = 0; i < world; ++i) {
    if (i == rank) {
      peer_bases[i] = ptr;
      offsets[i] = 0;
      continue;
    }
    void *peer = nullptr;
    e = hipIpcOpenMemHandle(&peer, all[(size_t)i].ipc_handle, hipIpcMemLazyEnablePeerAccess);
    if (e != hipSuccess) {
      for (int j = 0; j < i; ++j)
        if (j != rank) (void)hipIpcCloseMemHandle(peer_bases[j]);
      return api_fail(VR_ERR_HIP, "hipIpcOpenMemHandle(rank " + std::to_string(i) + ", pid " +
                                      std::to_string(all[(size_t)i].pid) + "): " + hipGetErrorString(e));
    }
    peer_bases[i] = peer;
    offsets[i] = all[(size_t)i].offset;
  }
  return VR_OK;
}

extern "C" int vr_ipc_close_all(int rank, int world, void *const peer_bases[]) {
  if (!peer_bases) return api_fail(VR_ERR_INVALID, "null argument");
  int rc = VR_OK;
  for (int i = 0; i < world; ++i) {
    if (i == rank || !peer_bases[i]) continue;
    const hipError_t e = hipIpcCloseMemHandle(peer_bases[i]);
    if (e != hipSuccess) rc = api_fail(VR_ERR_HIP, std::string("hipIpcCloseMemHandle: ") + hipGetErrorString(e));
  }
  return rc;
}

extern "C" int vr_ipc_barrier(int rank, int world, const char *instance, int generation) {
  if (!instance || world < 1 || world > VR_MAX_RANKS || rank < 0 || rank >= world)
    return api_fail(VR_ERR_INVALID, "bad argument");
  if (world == 1) return VR_OK;
  // Every rank hears from every other rank: nobody leaves before all have arrived.
  int token = generation, seen[VR_MAX_RANKS];
  const std::string tag = "barrier" + std::to_string(generation);
  if (int rc = un_allgather(&token, seen, sizeof token, rank, world, instance, tag.c_str())) return rc;
  for (int i = 0; i < world; ++i)
    if (seen[i] != generation) return api_fail(VR_ERR_INVALID, "barrier generations differ");
  return VR_OK;
}
