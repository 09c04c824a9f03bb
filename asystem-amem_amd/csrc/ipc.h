// Cross-process peer bookkeeping: a small request/response service on a UNIX stream socket
// in every process, carrying at most one file descriptor per message (SCM_RIGHTS).
// Replaces, for the pause/resume path only, the reference's worker thread and client
// calls: gmm_client_ctx::register_peer / update_peer (amem_nccl_plugin/gmm_client_impl.cpp:479-532),
// the worker dispatch (gmm_worker_impl.cpp:375-397) and gmm_send / gmm_recv
// (gmm_common_impl.cpp:341-434). The reference's admin thread, shared-memory config block and
// per-device worker pools are not reproduced: rendezvous is a lock file and a socket path
// per (group id, slot).
#ifndef AMEM_IPC_H_
#define AMEM_IPC_H_

#include <stdint.h>

namespace amem {

int amem_groupID_value();

// Claim a slot (preferring `preferred`, or AMEM_SLOT when set), bind the service socket and
// start the service thread. Idempotent. Returns the slot, or -1.
int ipc_start(int preferred);
// Claim one more slot for this process (a further rank living in it), with its own lock, socket and
// service thread. Needs the primary service. Returns the slot, or -1.
int ipc_claim_extra();
// From now on this thread registers imported regions as `slot` (one of this process's own; -1 =
// the primary slot again). 0 ok, 1 when the process does not hold that slot.
int ipc_act_as(int slot);
// How many requests the service of this process's `slot` has answered with success since it
// started: out[0] registrations, out[1] re-exported descriptors mapped, out[2] release requests.
// 0 ok, 1 when the process does not hold that slot.
int ipc_served(int slot, uint64_t out[3]);
void ipc_stop();
int ipc_slot();
// Whether a process currently holds `slot` of this group (a crashed one no longer does).
bool peer_alive(int slot);

// Importer -> owner: "my VA `my_va` maps your handle `src_handle`".
// 0 ok; 1 when the owner is this process (the reference's is_sameProcess rule,
// gmm_client_impl.cpp:482-484), unreachable, or does not know the handle.
int peer_register(uint64_t src_handle, uint64_t my_va, int owner_slot);
// Owner -> importer: "map this fd at your VA `peer_va`". 0 ok (also when the importer is
// this process, gmm_client_impl.cpp:512-514).
int peer_update(int importer_slot, uint64_t peer_va, int fd);

// The same to `n` importers at once (slots strictly ascending): all requests are sent before the first
// answer is read. rets[i] as peer_update's return for slots[i].
void peer_update_many(const int* slots, const uint64_t* peer_vas, int n, int fd, int* rets);

// Handler of a peer's request to drop the mapping at `va` (gmm_worker_impl.cpp:392-397).
int amem_release_peer_mapping(uint64_t va);

}  // namespace amem
#endif
