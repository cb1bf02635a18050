// Priority / preemption control over the cooperative flag (see include/gpreempt.h).
#include "gpreempt.h"

#include <algorithm>
#include <chrono>

int NvRmQuery(NvContext *ctx) { return ctx && ctx->stream ? 0 : -1; }

int set_priority(NvContext ctx, int priority) {
    if (priority < 0 || priority >= foo::PreemptDomain::kMaxLevels || !ctx.stream) return -1;
    return gp_stream_set_priority(ctx.stream, priority) == 0 ? 0 : -1;
}

// ---- hipSuspendStreams / hipResumeStreams over the flag words ------------------------------------
namespace {
std::mutex g_fd_mu;
std::vector<foo::PreemptDomain *> g_fds;
foo::PreemptDomain *domain_of(int fd) {
    std::lock_guard<std::mutex> g(g_fd_mu);
    return fd >= 0 && (size_t)fd < g_fds.size() ? g_fds[fd] : nullptr;
}

int g_newest_fd = -1;
int register_domain(foo::PreemptDomain *domain) {
    std::lock_guard<std::mutex> g(g_fd_mu);
    size_t i = 0;
    while (i < g_fds.size() && g_fds[i] != nullptr) ++i;
    if (i == g_fds.size()) g_fds.push_back(domain);
    else g_fds[i] = domain;
    g_newest_fd = (int)i;
    return (int)i;
}
void unregister_domain(foo::PreemptDomain *domain) {
    std::lock_guard<std::mutex> g(g_fd_mu);
    for (size_t i = 0; i < g_fds.size(); ++i)
        if (g_fds[i] == domain) {
            g_fds[i] = nullptr;
            if (g_newest_fd == (int)i) {
                g_newest_fd = -1;
                for (size_t j = 0; j < g_fds.size(); ++j) if (g_fds[j]) g_newest_fd = (int)j;
            }
        }
}
}  // namespace

int hipGetFd() {
    std::lock_guard<std::mutex> g(g_fd_mu);
    return g_newest_fd;
}

static int each_level(int fd, std::vector<int> &ids, bool suspend) {
    // the table's lock is held across the calls: a domain destroyed on another thread unregisters itself
    // under the same lock first, so the pointer cannot go stale in between
    std::lock_guard<std::mutex> g(g_fd_mu);
    foo::PreemptDomain *d = fd >= 0 && (size_t)fd < g_fds.size() ? g_fds[fd] : nullptr;
    if (!d) return -1;
    for (int p : ids)
        if (p < 1 || p >= d->levels()) return -1;
    for (int p : ids) suspend ? d->suspend_level(p) : d->resume_level(p);
    return 0;
}
int hipSuspendStreams(int fd, std::vector<int> &stream_ids) { return each_level(fd, stream_ids, true); }
int hipResumeStreams(int fd, std::vector<int> &stream_ids) { return each_level(fd, stream_ids, false); }
int hipResetWavefronts(int fd) { return domain_of(fd) ? 0 : -1; }

namespace foo {

static int64_t steady_ns() {
    return std::chrono::duration_cast<std::chrono::nanoseconds>(std::chrono::steady_clock::now().time_since_epoch()).count();
}

PreemptDomain::PreemptDomain(int levels, bool use_relay) : levels_(std::min(std::max(levels, 2), kMaxLevels)) {
    for (int i = 0; i < kMaxLevels; ++i) { active_[i] = 0; raised_[i] = 0; }
    fd_ = register_domain(this);
    for (int j = 0; j + 1 < levels_; ++j)
        if (gp_flag_create(&host_[j], &dev_[j]) != 0) ok_ = false;
    if (ok_ && use_relay) {
        const int n = levels_ - 1;
        bool good = gp_malloc((void **)&mirror_, sizeof(int) * 16) == 0 && gp_fill32_async(mirror_, 0, 16, nullptr) == 0 &&
                    gp_stream_sync(nullptr) == 0 && gp_flag_create(&quit_host_, &quit_dev_) == 0 &&
                    gp_stream_create(0, &relay_stream_) == 0;
        // ~10 minutes of polling at most; a scenario is far shorter
        if (good) good = gp_flag_relay_start(dev_, mirror_, n, (const int *)quit_dev_, 400000000ull, relay_stream_) == 0;
        relay_on_ = good;
        if (!good) std::fprintf(stderr, "PreemptDomain: flag relay not started (%s); kernels poll host memory\n", gp_last_error());
    }
}

void PreemptDomain::stop_relay() {
    if (!relay_on_) return;
    *quit_host_ = 1;
    gp_stream_sync(relay_stream_);
    relay_on_ = false;
}

PreemptDomain::~PreemptDomain() {
    unregister_domain(this);
    stop_relay();
    if (relay_stream_) gp_stream_destroy(relay_stream_);
    if (quit_host_) gp_flag_destroy(quit_host_);
    if (mirror_) gp_free(mirror_);
    for (int j = 0; j + 1 < levels_; ++j)
        if (host_[j]) gp_flag_destroy(host_[j]);
}

GPUdeviceptr PreemptDomain::flag_for(int priority) const {
    int p = std::min(priority, levels_ - 1);
    if (p < 1) return nullptr;
    return relay_on_ ? (GPUdeviceptr)(mirror_ + (p - 1)) : dev_[p - 1];
}

int PreemptDomain::flag_value(int priority) const {
    int p = std::min(priority, levels_ - 1);
    return p < 1 ? -1 : *host_[p - 1];
}

// word j is up while any request of a level <= j is active
void PreemptDomain::update() {
    int run = 0;
    for (int j = 0; j + 1 < levels_; ++j) {
        run += active_[j].load();
        int want = run > 0 || forced_[j] > 0;
        if (*host_[j] != want) {
            if (want) raised_[j].store(steady_ns());
            *host_[j] = want;
        }
    }
}

void PreemptDomain::begin(int priority) {
    int p = std::min(priority, levels_ - 1);
    if (p + 1 >= levels_) return;  // the lowest level preempts nobody
    std::lock_guard<std::mutex> g(mu_);
    // the time stamp goes first: whoever sees the request counted must not pair it with the
    // stamp of an earlier raise
    const int64_t now = steady_ns();
    for (int j = p; j + 1 < levels_; ++j)
        if (*host_[j] == 0) raised_[j].store(now);
    active_[p].fetch_add(1, std::memory_order_acq_rel);
    update();
}

void PreemptDomain::end(int priority) {
    int p = std::min(priority, levels_ - 1);
    if (p + 1 >= levels_) return;
    std::lock_guard<std::mutex> g(mu_);
    active_[p].fetch_sub(1, std::memory_order_acq_rel);
    update();
}

void PreemptDomain::suspend_level(int priority) {
    int p = std::min(priority, levels_ - 1);
    if (p < 1) return;
    std::lock_guard<std::mutex> g(mu_);
    if (*host_[p - 1] == 0) raised_[p - 1].store(steady_ns());
    ++forced_[p - 1];
    update();
}

void PreemptDomain::resume_level(int priority) {
    int p = std::min(priority, levels_ - 1);
    if (p < 1) return;
    std::lock_guard<std::mutex> g(mu_);
    if (forced_[p - 1] > 0) --forced_[p - 1];
    update();
}

int PreemptDomain::active_above(int priority) const {
    int p = std::min(priority, levels_ - 1), n = 0;
    for (int i = 0; i < p; ++i) n += active_[i].load(std::memory_order_acquire);
    return n;
}

int64_t PreemptDomain::raised_ns(int priority) const {
    int p = std::min(priority, levels_ - 1);
    return p >= 1 ? raised_[p - 1].load() : 0;
}

}  // namespace foo
