// gpreempt.h — priority and preemption control.
//
// In the reference this header wraps ioctls of a patched driver: `set_priority(NvContext, int)`
// turns a context's timeslice into 1 s (priority 0) or 1 us (any other), and on HIP
// `hipSuspendStreams` / `hipResumeStreams` stop and restart hardware queues through a patched
// amdkfd (include/gpreempt.h:124-173,191-194; src/gpreempt.cpp:61-72,143-196).  Here nothing
// below user space is modified: a tenant's priority selects the cooperative preempt flag it
// obeys, "suspend" raises that flag (running best-effort kernels leave at their next tile
// boundary) and "resume" lowers it (the tenant then calls BLPExecutor::resume).  The call shapes
// are kept so that client code reads the same.
#pragma once
#include <atomic>
#include <mutex>
#include <vector>
#include "util/gpu_util.h"

// What the reference keeps per GPU context (NvContext: client / object handles and channel list
// found by NvRmQuery for the calling thread): here the tenant's stream and its priority level.
struct NvContext {
    GPUstream stream = nullptr;
    int priority = 1;  // 0 = high, larger = lower
};

// Fills ctx for the calling thread's tenant; with stock drivers there is nothing to look up, so
// this only validates the stream.  Returns 0 on success (the reference's NV_OK).
int NvRmQuery(NvContext *ctx);

// priority 0 = high, 1 = low (reference include/gpreempt.h:165-173); further levels are allowed.
// The context is passed by value as in the reference: what carries the level is the tenant's
// stream (the priority recorded on the gp_stream handle, which selects the flag word the tenant
// obeys).  Returns 0, or -1 for a bad argument or a context without a stream.
int set_priority(NvContext ctx, int priority);

// The HIP side of the reference's header (include/gpreempt.h:191-194) stops and restarts hardware
// queues through a patched amdkfd.  Here "queues" are priority levels of a PreemptDomain: a
// level is suspended by raising the flag word it obeys (its kernels leave at their next tile
// boundary) and resumed by lowering it (the tenant then calls BLPExecutor::resume).  `fd` names a
// PreemptDomain: hipGetFd() returns the handle of the process's newest live domain (-1: none), as
// the reference's returns the one KFD file of the process; PreemptDomain::fd() gives a particular
// one.  The others return 0 on success, -1 on a bad argument.
int hipGetFd();
int hipSuspendStreams(int fd, std::vector<int> &stream_ids);    // stream_ids: priority levels (>= 1) to stop
int hipResumeStreams(int fd, std::vector<int> &stream_ids);
int hipResetWavefronts(int fd);                                 // nothing to reset without the driver patch: returns 0

namespace foo {

// The preempt flags of one GPU: one word per priority boundary.  Level p tenants obey word p-1,
// which is up while any request of a level < p is active.  The reference has two levels and one
// word (src/cuda-clients/blpclient.cpp:36-41,185-195).
class PreemptDomain {
public:
    static constexpr int kMaxLevels = 8;
    // use_relay: keep a device-memory mirror of the flag words up to date with a small resident
    // kernel (gp_flag_relay_start) and hand the mirror to the executors, so that their kernels
    // poll device memory on every claim.  Call stop_relay() (the destructor does) before freeing
    // device memory elsewhere: frees synchronise the device and would wait for the relay.
    explicit PreemptDomain(int levels = 2, bool use_relay = false);
    void stop_relay();
    bool relayed() const { return relay_on_; }
    ~PreemptDomain();
    PreemptDomain(const PreemptDomain &) = delete;
    PreemptDomain &operator=(const PreemptDomain &) = delete;

    int levels() const { return levels_; }
    bool ok() const { return ok_; }
    int fd() const { return fd_; }  // the handle hipSuspendStreams / hipResumeStreams take
    // device address of the flag a level-p (p >= 1) best-effort executor polls: BLPExecutor::dpStop
    GPUdeviceptr flag_for(int priority) const;
    // current value of that word as the host sees it (-1: the level obeys no word)
    int flag_value(int priority) const;
    // a request of `priority` starts / ends: raises / lowers the words of every lower level
    void begin(int priority);
    void end(int priority);
    // requests currently active at levels above `priority`
    int active_above(int priority) const;
    // steady-clock nanoseconds at which the word obeyed by `priority` was last raised (0: never)
    int64_t raised_ns(int priority) const;
    // direct control, what hipSuspendStreams / hipResumeStreams call
    void suspend_below(int priority) { begin(priority); }
    void resume_below(int priority) { end(priority); }
    // raise / lower the one word that level `priority` (>= 1) obeys, whatever requests are active
    void suspend_level(int priority);
    void resume_level(int priority);

private:
    void update();
    int levels_;
    int fd_ = -1;
    bool ok_ = true;
    volatile int *host_[kMaxLevels] = {nullptr};
    void *dev_[kMaxLevels] = {nullptr};
    std::atomic<int> active_[kMaxLevels];
    int forced_[kMaxLevels] = {0};      // suspend_level counts per word
    std::atomic<int64_t> raised_[kMaxLevels];
    std::mutex mu_;
    bool relay_on_ = false;
    int *mirror_ = nullptr;             // device ints, one per word
    volatile int *quit_host_ = nullptr; // host flag that ends the relay
    void *quit_dev_ = nullptr;
    GPUstream relay_stream_ = nullptr;
};

}  // namespace foo
