#ifndef _GNU_SOURCE
#define _GNU_SOURCE 1
#endif
#include "ipc.h"

#include <errno.h>
#include <fcntl.h>
#include <poll.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <sys/file.h>
#include <sys/socket.h>
#include <sys/stat.h>
#include <sys/un.h>
#include <unistd.h>

#include <atomic>
#include <mutex>
#include <string>
#include <thread>
#include <vector>

#include <hip/hip_runtime_api.h>

#include "../../include/amem_nccl.h"
#include "ctx.h"
#include "engine.h"
#include "log.h"

namespace amem {

int amem_groupID_value() { return ::amem_groupID; }

namespace {

// Same numbering as the reference's gmm_ipc_op (gmm_common.h:106-150).
enum WireOp : int32_t { OP_REGISTER_PEER_INFO = 16, OP_UPDATE_PEER_INFO = 17, OP_RELEASE_PEER_HANDLE = 18 };

struct WireReq {
  uint32_t magic;
  int32_t op;
  int32_t sender_slot;
  int32_t pid;
  uint64_t src;  // REGISTER: owner's handle
  uint64_t tgt;  // REGISTER: importer's VA; UPDATE/RELEASE: receiver's VA
};
static constexpr uint32_t kMagic = 0x414d454d;  // "AMEM"

// One claimed slot: its lock file, its listening socket and the thread that serves it.
struct Service {
  int slot = -1;
  int dev = 0;
  int lock_fd = -1;
  int listen_fd = -1;
  int wake[2] = {-1, -1};
  std::string sock_path, lock_path;
  std::thread thr;
  std::atomic<bool> stop{false};
  std::atomic<uint64_t> served[3];  // requests answered with success: register, update, release
  Service() { for (auto& n : served) n.store(0); }
};
// A process normally holds one slot (`primary`). It may claim more, one per rank it hosts: each
// extra slot is a full peer with a lock, a socket and a service thread of its own, so that ranks
// living in one process reach each other exactly as ranks in different processes do.
struct Ipc {
  std::mutex mtx;  // guards primary / extra (not the services' own `stop`)
  Service primary;
  std::vector<Service*> extra;
  int conn[AMEM_MAX_DEVS];              // client connections, by target slot
  std::mutex conn_mtx[AMEM_MAX_DEVS];
  Ipc() { for (int& c : conn) c = -1; }
};
// Never destroyed: a service thread may outlive static destruction at exit.
Ipc& g_ipc = *new Ipc();
Service& g_svc = g_ipc.primary;
// The slot on whose behalf this thread registers imported regions; -1 = the primary slot.
thread_local int t_acting_slot = -1;

// Whether `slot` is one of this process's own. Takes g_ipc.mtx for the extra slots: callers must
// not hold it (none of the service threads' handlers comes here, so ipc_stop may join them under it).
bool own_slot(int slot) {
  if (slot < 0) return false;
  if (g_svc.slot == slot) return true;
  std::lock_guard<std::mutex> lk(g_ipc.mtx);
  for (Service* s : g_ipc.extra) if (s->slot == slot) return true;
  return false;
}
int acting_slot() { return t_acting_slot >= 0 ? t_acting_slot : g_svc.slot; }

std::string ipc_dir() {
  const char* d = getenv("GMM_IPC_DIR");  // gmm_server_impl.cpp:78-79
  return d ? d : "/tmp";
}
std::string sock_name(int slot) {
  char b[256];
  snprintf(b, sizeof(b), "%s/amem_worker_%x_%d.sock", ipc_dir().c_str(), amem_groupID_value(), slot);
  return b;
}
std::string lock_name(int slot) {
  char b[256];
  snprintf(b, sizeof(b), "%s/amem_slot_%x_%d.lock", ipc_dir().c_str(), amem_groupID_value(), slot);
  return b;
}

// One message with an optional descriptor; >0 bytes sent, else error.
ssize_t send_msg(int sock, const void* buf, size_t bytes, int fd) {
  struct iovec iov = {(void*)buf, bytes};
  struct msghdr msg = {};
  union { struct cmsghdr cm; char control[CMSG_SPACE(sizeof(int))]; } cu;
  msg.msg_iov = &iov;
  msg.msg_iovlen = 1;
  if (fd >= 0) {
    memset(&cu, 0, sizeof(cu));
    msg.msg_control = cu.control;
    msg.msg_controllen = sizeof(cu.control);
    struct cmsghdr* cm = CMSG_FIRSTHDR(&msg);
    cm->cmsg_level = SOL_SOCKET;
    cm->cmsg_type = SCM_RIGHTS;
    cm->cmsg_len = CMSG_LEN(sizeof(int));
    memcpy(CMSG_DATA(cm), &fd, sizeof(int));
  }
  ssize_t r;
  do { r = sendmsg(sock, &msg, MSG_NOSIGNAL); } while (r < 0 && errno == EINTR);
  if (r < 0) LOGGER(ERROR, "pid:%d sendmsg failed on connect:%d error:%s", getpid(), sock, strerror(errno));
  return r;
}

// Receive exactly `bytes`; a descriptor that rides along is stored in *fd (else -1).
ssize_t recv_msg(int sock, void* buf, size_t bytes, int* fd) {
  if (fd) *fd = -1;
  size_t got = 0;
  while (got < bytes) {
    struct iovec iov = {(char*)buf + got, bytes - got};
    struct msghdr msg = {};
    union { struct cmsghdr cm; char control[CMSG_SPACE(sizeof(int))]; } cu;
    msg.msg_iov = &iov;
    msg.msg_iovlen = 1;
    msg.msg_control = cu.control;
    msg.msg_controllen = sizeof(cu.control);
    ssize_t r = recvmsg(sock, &msg, 0);
    if (r < 0 && errno == EINTR) continue;
    if (r <= 0) return r;
    for (struct cmsghdr* cm = CMSG_FIRSTHDR(&msg); cm; cm = CMSG_NXTHDR(&msg, cm)) {
      if (cm->cmsg_level == SOL_SOCKET && cm->cmsg_type == SCM_RIGHTS && cm->cmsg_len == CMSG_LEN(sizeof(int))) {
        int f;
        memcpy(&f, CMSG_DATA(cm), sizeof(int));
        if (fd && *fd < 0) *fd = f; else close(f);
      }
    }
    got += (size_t)r;
  }
  return (ssize_t)got;
}

int handle_request(const WireReq& req, int fd) {
  switch (req.op) {
    case OP_REGISTER_PEER_INFO:  // gmm_worker_impl.cpp:375-382
      if (fd >= 0) close(fd);
      return amem_register_peer_info(req.src, req.tgt, req.sender_slot);
    case OP_UPDATE_PEER_INFO:    // gmm_worker_impl.cpp:384-390
      if (fd < 0) {
        LOGGER(ERROR, "pid:%d recvmsg done but unexpected control header setting", getpid());
        return 1;
      }
      return amem_update_peer_info(req.tgt, fd);
    case OP_RELEASE_PEER_HANDLE: // gmm_worker_impl.cpp:392-397
      if (fd >= 0) close(fd);
      return amem_release_peer_mapping(req.tgt);
    default:
      if (fd >= 0) close(fd);
      LOGGER(ERROR, "worker:%d invalid op:%d", g_svc.slot, req.op);
      return 1;
  }
}

void serve(Service* svc_p) {
  Service& g_svc = *svc_p;
  if (gpu_present()) (void)hipSetDevice(g_svc.dev);
  std::vector<struct pollfd> fds;
  fds.push_back({g_svc.listen_fd, POLLIN, 0});
  fds.push_back({g_svc.wake[0], POLLIN, 0});
  while (!g_svc.stop.load()) {
    int n = poll(fds.data(), fds.size(), -1);
    if (n < 0) { if (errno == EINTR) continue; break; }
    if (fds[1].revents) break;
    if (fds[0].revents & POLLIN) {
      int c = accept4(g_svc.listen_fd, nullptr, nullptr, SOCK_CLOEXEC);
      if (c >= 0) {
        // Requests change this process's address space: only this user's processes may send
        // them, and one that stops half-way through a message must not block the others.
        struct ucred cred = {};
        socklen_t len = sizeof(cred);
        if (getsockopt(c, SOL_SOCKET, SO_PEERCRED, &cred, &len) != 0 || cred.uid != geteuid()) {
          LOGGER(WARN, "pid:%d refused a connection from uid %d", getpid(), (int)cred.uid);
          close(c);
        } else {
          struct timeval tv = {5, 0};
          setsockopt(c, SOL_SOCKET, SO_RCVTIMEO, &tv, sizeof(tv));
          setsockopt(c, SOL_SOCKET, SO_SNDTIMEO, &tv, sizeof(tv));
          fds.push_back({c, POLLIN, 0});
        }
      }
    }
    for (size_t i = 2; i < fds.size();) {
      if (!(fds[i].revents & (POLLIN | POLLHUP | POLLERR))) { ++i; continue; }
      WireReq req;
      int fd = -1;
      ssize_t r = recv_msg(fds[i].fd, &req, sizeof(req), &fd);
      if (r != (ssize_t)sizeof(req) || req.magic != kMagic) {
        // peer went away (gmm_worker_impl.cpp:409-419): drop the connection
        if (fd >= 0) close(fd);
        close(fds[i].fd);
        fds.erase(fds.begin() + i);
        continue;
      }
      int32_t ret = handle_request(req, fd);
      if (ret == 0 && req.op >= OP_REGISTER_PEER_INFO && req.op <= OP_RELEASE_PEER_HANDLE)
        g_svc.served[req.op - OP_REGISTER_PEER_INFO].fetch_add(1, std::memory_order_relaxed);
      send_msg(fds[i].fd, &ret, sizeof(ret), -1);
      ++i;
    }
  }
  for (size_t i = 2; i < fds.size(); ++i) close(fds[i].fd);
}

bool claim(int slot, Service& g_svc) {
  std::string lp = lock_name(slot);
  for (int attempt = 0; attempt < 4; ++attempt) {
    // Only this user's processes form a group (the service refuses everybody else), so nobody
    // else needs to open the lock, and nobody else should be able to hold it and fake a live peer.
    int fd = open(lp.c_str(), O_CREAT | O_RDWR | O_CLOEXEC | O_NOFOLLOW, 0600);
    if (fd < 0) return false;
    if (flock(fd, LOCK_EX | LOCK_NB) != 0) { close(fd); return false; }
    // The lock is on the file, not on its name: if the name was removed or replaced between the
    // open and the lock (a /tmp cleaner), somebody else may hold a lock under the same name.
    struct stat a, b;
    if (fstat(fd, &a) == 0 && stat(lp.c_str(), &b) == 0 && a.st_ino == b.st_ino && a.st_dev == b.st_dev) {
      g_svc.lock_fd = fd;
      g_svc.lock_path = lp;
      g_svc.slot = slot;
      return true;
    }
    close(fd);
  }
  return false;
}

// True while some process holds the lock file of `slot`. The lock dies with its holder, so
// this is how a peer that crashed is told from one that is merely slow.
bool slot_claimed(int slot) {
  int fd = open(lock_name(slot).c_str(), O_RDWR | O_CLOEXEC | O_NOFOLLOW);
  if (fd < 0) return false;
  const bool held = flock(fd, LOCK_SH | LOCK_NB) != 0;
  if (!held) flock(fd, LOCK_UN);
  close(fd);
  return held;
}

// Connect to the service of `slot`, waiting for it to appear (connect_if_not,
// gmm_client_impl.cpp:288-347, with a bounded wait instead of an abort).
int connect_if_not(int slot) {
  if (g_ipc.conn[slot] >= 0) return g_ipc.conn[slot];
  int64_t budget_ms = options().peer_timeout_ms > 0 ? options().peer_timeout_ms : 30000;
  std::string path = sock_name(slot);
  struct sockaddr_un addr = {};
  addr.sun_family = AF_UNIX;
  strncpy(addr.sun_path, path.c_str(), sizeof(addr.sun_path) - 1);
  for (int64_t waited = 0;; waited += 20) {
    int s = socket(AF_UNIX, SOCK_STREAM | SOCK_CLOEXEC, 0);
    if (s < 0) return -1;
    if (connect(s, (struct sockaddr*)&addr, sizeof(addr)) == 0) {
      // Requests carry descriptors of this process's device memory: whoever listens on the path
      // must be a process of the same user, or it gets nothing.
      struct ucred cred = {};
      socklen_t clen = sizeof(cred);
      if (getsockopt(s, SOL_SOCKET, SO_PEERCRED, &cred, &clen) != 0 || cred.uid != geteuid()) {
        LOGGER(ERROR, "groupID:%d pid:%d %s is served by uid %d, not by this user; refusing to talk to it",
               amem_groupID_value(), getpid(), path.c_str(), (int)cred.uid);
        close(s);
        return -1;
      }
      if (options().peer_timeout_ms > 0) {
        struct timeval tv = {(time_t)(options().peer_timeout_ms / 1000), (suseconds_t)((options().peer_timeout_ms % 1000) * 1000)};
        setsockopt(s, SOL_SOCKET, SO_RCVTIMEO, &tv, sizeof(tv));
        setsockopt(s, SOL_SOCKET, SO_SNDTIMEO, &tv, sizeof(tv));
      }
      g_ipc.conn[slot] = s;
      return s;
    }
    close(s);
    // A peer is known by its slot only after it has claimed that slot, so an unclaimed slot
    // means its process is gone; a claimed one without a socket yet is still starting.
    if (!slot_claimed(slot)) {
      LOGGER(ERROR, "groupID:%d pid:%d the process of slot %d is gone (nobody holds %s)", amem_groupID_value(),
             getpid(), slot, lock_name(slot).c_str());
      return -1;
    }
    if (waited >= budget_ms) break;
    usleep(20000);
  }
  LOGGER(ERROR, "groupID:%d pid:%d error on connecting to %s after retry, error:%s", amem_groupID_value(),
         getpid(), path.c_str(), strerror(errno));
  return -1;
}

int rpc(int slot, const WireReq& req, int fd) {
  if (slot < 0 || slot >= AMEM_MAX_DEVS) return 1;
  std::lock_guard<std::mutex> lk(g_ipc.conn_mtx[slot]);
  int s = connect_if_not(slot);
  if (s < 0) return 1;
  int32_t ret = 1;
  const bool sent = send_msg(s, &req, sizeof(req), fd) == (ssize_t)sizeof(req);
  const bool answered = sent && recv_msg(s, &ret, sizeof(ret), nullptr) == (ssize_t)sizeof(ret);
  if (!answered) {
    // peer gone, or no answer within the timeout: drop the connection so that the next
    // request reconnects instead of reading a stale reply
    close(s);
    g_ipc.conn[slot] = -1;
    return 1;
  }
  return ret;
}

}  // namespace

int ipc_slot() { return g_svc.slot; }

bool peer_alive(int slot) { return slot >= 0 && slot < AMEM_MAX_DEVS && slot_claimed(slot); }

// Bind and serve the slot `svc` has claimed. On failure the claim is given up.
static bool start_service(Service& svc) {
  svc.dev = current_device();
  svc.sock_path = sock_name(svc.slot);
  unlink(svc.sock_path.c_str());  // a stale file of a dead holder of this slot
  svc.listen_fd = socket(AF_UNIX, SOCK_STREAM | SOCK_CLOEXEC, 0);
  struct sockaddr_un addr = {};
  addr.sun_family = AF_UNIX;
  strncpy(addr.sun_path, svc.sock_path.c_str(), sizeof(addr.sun_path) - 1);
  if (svc.listen_fd < 0 || bind(svc.listen_fd, (struct sockaddr*)&addr, sizeof(addr)) != 0 ||
      listen(svc.listen_fd, 64) != 0 || pipe2(svc.wake, O_CLOEXEC) != 0) {
    LOGGER(ERROR, "pid:%d failed to serve on %s error:%s", getpid(), svc.sock_path.c_str(), strerror(errno));
    if (svc.listen_fd >= 0) close(svc.listen_fd);
    svc.listen_fd = -1;
    close(svc.lock_fd);
    svc.lock_fd = -1;
    svc.slot = -1;
    return false;
  }
  svc.stop.store(false);
  for (auto& n : svc.served) n.store(0);
  svc.thr = std::thread(serve, &svc);
  LOGGER(DEBUG, "groupID:%d pid:%d serving slot %d on %s", amem_groupID_value(), getpid(), svc.slot,
         svc.sock_path.c_str());
  return true;
}

static void stop_service(Service& svc) {
  if (svc.slot < 0) return;
  svc.stop.store(true);
  char b = 1;
  if (write(svc.wake[1], &b, 1) < 0) { /* thread is woken by close below */ }
  if (svc.thr.joinable()) svc.thr.join();
  close(svc.listen_fd);
  close(svc.wake[0]);
  close(svc.wake[1]);
  unlink(svc.sock_path.c_str());
  // The lock file stays: removing the name while another process is between open() and flock()
  // on it would let two processes hold "the" lock of one slot.
  close(svc.lock_fd);
  svc.lock_fd = svc.listen_fd = -1;
  svc.slot = -1;
}

int ipc_start(int preferred) {
  std::lock_guard<std::mutex> lk(g_ipc.mtx);
  if (g_svc.slot >= 0) return g_svc.slot;
  const char* forced = getenv("AMEM_SLOT");
  bool ok = false;
  if (forced) {
    int s = atoi(forced);
    ok = s >= 0 && s < AMEM_MAX_DEVS && claim(s, g_svc);
  } else {
    if (preferred < 0 || preferred >= AMEM_MAX_DEVS) preferred = 0;
    for (int k = 0; k < AMEM_MAX_DEVS && !ok; ++k) ok = claim((preferred + k) % AMEM_MAX_DEVS, g_svc);
  }
  if (!ok) {
    LOGGER(WARN, "groupID:%d pid:%d no free slot under %s; cross-process regions stay out of pause scope",
           amem_groupID_value(), getpid(), ipc_dir().c_str());
    return -1;
  }
  if (!start_service(g_svc)) return -1;
  return g_svc.slot;
}

// One more slot for this process: a rank of its own with lock, socket and service thread.
int ipc_claim_extra() {
  std::lock_guard<std::mutex> lk(g_ipc.mtx);
  if (g_svc.slot < 0) return -1;
  Service* svc = new Service();
  bool ok = false;
  for (int k = 1; k < AMEM_MAX_DEVS && !ok; ++k) ok = claim((g_svc.slot + k) % AMEM_MAX_DEVS, *svc);
  if (!ok || !start_service(*svc)) {
    LOGGER(WARN, "groupID:%d pid:%d no further free slot under %s", amem_groupID_value(), getpid(), ipc_dir().c_str());
    delete svc;
    return -1;
  }
  g_ipc.extra.push_back(svc);
  return svc->slot;
}

int ipc_served(int slot, uint64_t out[3]) {
  std::lock_guard<std::mutex> lk(g_ipc.mtx);
  Service* svc = g_svc.slot == slot && slot >= 0 ? &g_svc : nullptr;
  for (Service* s : g_ipc.extra) if (s->slot == slot) svc = s;
  if (!svc) return 1;
  for (int i = 0; i < 3; ++i) out[i] = svc->served[i].load(std::memory_order_relaxed);
  return 0;
}

int ipc_act_as(int slot) {
  if (slot < 0) { t_acting_slot = -1; return 0; }
  if (!own_slot(slot)) return 1;
  t_acting_slot = slot;
  return 0;
}

void ipc_stop() {
  std::lock_guard<std::mutex> lk(g_ipc.mtx);
  if (g_svc.slot < 0) return;
  for (Service* svc : g_ipc.extra) { stop_service(*svc); delete svc; }
  g_ipc.extra.clear();
  t_acting_slot = -1;
  stop_service(g_svc);
  for (int i = 0; i < AMEM_MAX_DEVS; ++i) {
    std::lock_guard<std::mutex> lc(g_ipc.conn_mtx[i]);
    if (g_ipc.conn[i] >= 0) close(g_ipc.conn[i]);
    g_ipc.conn[i] = -1;
  }
}

int peer_register(uint64_t src_handle, uint64_t my_va, int owner_slot) {
  if (g_svc.slot < 0 || (own_slot(owner_slot) && !options().peer_loopback)) return 1;
  WireReq req = {kMagic, OP_REGISTER_PEER_INFO, acting_slot(), (int32_t)getpid(), src_handle, my_va};
  int ret = rpc(owner_slot, req, -1);
  if (ret != 0)
    LOGGER(WARN, "groupID:%d pid:%d peer_dev:%d dptr:%llx send|recv error", amem_groupID_value(), getpid(),
           owner_slot, (unsigned long long)my_va);
  return ret;
}

// One descriptor to several importers at once: every request goes out before the first answer is
// waited for, so the importers (one service thread each, usually one process each) import and map side
// by side instead of one after the other. Slots are taken in ascending order, each connection stays
// locked from its request to its answer.
void peer_update_many(const int* slots, const uint64_t* peer_vas, int n, int fd, int* rets) {
  int socks[AMEM_MAX_DEVS];
  bool locked[AMEM_MAX_DEVS];
  bool mine[AMEM_MAX_DEVS];
  if (n > AMEM_MAX_DEVS) n = AMEM_MAX_DEVS;
  // (asked before any connection is locked: own_slot takes the lock that ipc_stop holds while it
  // takes the connections' locks)
  for (int i = 0; i < n; ++i) mine[i] = own_slot(slots[i]);
  for (int i = 0; i < n; ++i) {
    socks[i] = -1;
    locked[i] = false;
    rets[i] = 1;
    const int slot = slots[i];
    if (slot < 0 || slot >= AMEM_MAX_DEVS || (i > 0 && slot <= slots[i - 1])) continue;
    if (mine[i] && !options().peer_loopback) { rets[i] = 0; continue; }
    if (g_svc.slot < 0) continue;
    g_ipc.conn_mtx[slot].lock();
    locked[i] = true;
    const int s = connect_if_not(slot);
    if (s < 0) continue;
    WireReq req = {kMagic, OP_UPDATE_PEER_INFO, g_svc.slot, (int32_t)getpid(), 0, peer_vas[i]};
    if (send_msg(s, &req, sizeof(req), fd) == (ssize_t)sizeof(req)) {
      socks[i] = s;
    } else {
      close(s);
      g_ipc.conn[slot] = -1;
    }
  }
  for (int i = 0; i < n; ++i) {
    if (!locked[i]) continue;
    const int slot = slots[i];
    if (socks[i] >= 0) {
      int32_t ret = 1;
      if (recv_msg(socks[i], &ret, sizeof(ret), nullptr) == (ssize_t)sizeof(ret)) {
        rets[i] = ret;
      } else {
        // peer gone, or no answer within the timeout: the next request reconnects
        close(socks[i]);
        g_ipc.conn[slot] = -1;
      }
    }
    g_ipc.conn_mtx[slot].unlock();
    if (rets[i] != 0)
      LOGGER(WARN, "groupID:%d pid:%d peer_dev:%d peer_dptr:%llx newFD:%d send|recv error", amem_groupID_value(),
             getpid(), slot, (unsigned long long)peer_vas[i], fd);
  }
}

int peer_update(int importer_slot, uint64_t peer_va, int fd) {
  if (own_slot(importer_slot) && !options().peer_loopback) return 0;
  if (g_svc.slot < 0) return 1;
  WireReq req = {kMagic, OP_UPDATE_PEER_INFO, g_svc.slot, (int32_t)getpid(), 0, peer_va};
  int ret = rpc(importer_slot, req, fd);
  if (ret != 0)
    LOGGER(WARN, "groupID:%d pid:%d peer_dev:%d peer_dptr:%llx newFD:%d send|recv error", amem_groupID_value(),
           getpid(), importer_slot, (unsigned long long)peer_va, fd);
  return ret;
}

}  // namespace amem
