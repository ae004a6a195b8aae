// Refinement-record upgrade engine: record file -> pinned host entry -> device slot -> mailbox stage row -> seq, for one
// rank's record file and one GPU. Host code only (HIP runtime + POSIX); the C ABI is nq_stream_* in include/nq_moe_hip.h.
//
// Same contract as the reference's engine (streaming/nqstream.cu:1-26): an upgrade's three device writes (record bytes
// into the slot, the table row into the mailbox's stage, the sequence number) are issued in that order on ONE side stream,
// so the mailbox kernel of a later layer call can only see the new sequence number after the bytes have landed; a
// downgrade writes only row and seq. Ops start in arrival order. The host entries are both the bounce buffers of the reads
// and a cache of recently read records (least recently used entry without a user is replaced); an optional pinned RAM
// tier holds chosen records for the life of the engine; an op that has touched neither a drive nor the device can be
// cancelled; a failed or short read reports the op as failed and never writes its row.
//
// Built differently from the reference: no io_uring (liburing is not part of this toolchain). A record here is megabytes
// (9.5 MB at H = 6144, I = 2048), so one blocking pread per reader thread loses nothing against a submission ring: each
// drive gets `qd` reader threads, which is the drive's queue depth; a director thread owns all bookkeeping, hands reads
// to the drive with the fewest in flight, issues the copies and retires them by polling their events. The side stream
// has the default priority.
#include "nq_host.hpp"
#include <fcntl.h>
#include <unistd.h>
#include <sys/stat.h>
#include <errno.h>
#include <string.h>
#include <time.h>
#include <stdlib.h>
#include <atomic>
#include <condition_variable>
#include <deque>
#include <mutex>
#include <string>
#include <thread>
#include <unordered_map>
#include <unordered_set>
#include <vector>
#include "../../include/nq_moe_hip.h"

namespace {

constexpr int ROW_W = NQ_TBL_W;
constexpr double CANCELLED = -1e9;       // t_read and t_e2e of a cancelled op, as the reference reports it (nqstream.cu:207)

double now()
{
    timespec t; clock_gettime(CLOCK_MONOTONIC, &t);
    return (double)t.tv_sec + 1e-9 * (double)t.tv_nsec;
}

struct Op
{
    int64_t tag = 0, rec = -1;
    bool read = false;                   // upgrade from the record file (record bytes + row + seq); otherwise row-only or upload
    int nspans = 0;                      // upload: spans of the caller's pinned memory copied before the row (no file, no entry)
    const void* sp_src[NQ_STREAM_MAX_SPANS]; void* sp_dst[NQ_STREAM_MAX_SPANS]; int64_t sp_n[NQ_STREAM_MAX_SPANS];
    void* slot = nullptr; void* stage = nullptr; void* seqp = nullptr;
    int32_t seq = 0;
    int64_t row[ROW_W];
    double t0 = 0, t_rd = 0, t_sub = 0;
    int entry = -1, ring = -1, drive = -1;
    bool hit = false, copy_failed = false;   // copy_failed: a HIP call of this op's copies failed (seq was not written)
    const uint8_t* tier_src = nullptr;
    int64_t got = 0;                     // bytes the read returned, or -errno
    hipEvent_t ev = nullptr;
};

struct Engine
{
    // configuration
    int dev = 0, nh = 0, nd = 1;
    size_t rb = 0;
    int fds[2] = {-1, -1}, bfds[2] = {-1, -1}, qd[2] = {0, 0};   // O_DIRECT descriptor (or -1) and buffered descriptor per drive
    std::atomic<int> direct[2] = {{0}, {0}};                    // reads of the drive currently go through the O_DIRECT descriptor
    // pinned memory
    uint8_t* host = nullptr;             // nh entries of rb bytes
    int64_t* rows = nullptr; int32_t* seqs = nullptr;   // staging of row and seq per ring slot
    int nring = 0;
    std::vector<int> ring_free;
    // cache of the host entries (director thread only)
    std::vector<int64_t> ent_rec;        // record held (-1 = none)
    std::vector<int> ent_users;          // ops reading into or copying out of the entry
    std::vector<uint64_t> ent_stamp;     // last use; smallest unused stamp is replaced
    uint64_t clock = 0;
    std::unordered_map<int64_t, int> where;
    // RAM tier: 0 none, 1 active, 2 drop requested, 3 dropped
    std::atomic<int> tier_state{0};
    uint8_t* tier_mem = nullptr; size_t tier_n = 0; int tier_users = 0;
    std::unordered_map<int64_t, const uint8_t*> tier_at;
    // threads
    hipStream_t st = nullptr;
    std::mutex mu;                       // guards: inbox, cancel_req, landed, done, jobs, counters read by stats()
    std::condition_variable cv;          // wakes the director
    std::condition_variable rcv[2];      // wake a drive's readers
    std::deque<Op*> inbox, jobs[2];
    std::vector<int64_t> cancel_req;
    std::vector<Op*> landed;             // reads that returned, not yet seen by the director
    std::vector<NqStreamDone> done;
    std::vector<std::thread> readers;
    std::thread director;
    std::atomic<bool> stop{false};
    bool closed = false;
    std::vector<hipEvent_t> evpool;
    std::string fail;                    // first HIP failure of the director (reported by stats / poll)
    // director-side queues
    std::deque<Op*> waiting, ready;
    std::vector<Op*> copying;
    std::atomic<int> infl[2] = {{0}, {0}}, n_reading{0}, n_copying{0};   // written by the director, read by stats()
    // counters (under mu)
    int64_t n_up = 0, n_post = 0, n_hit = 0, bytes = 0, n_cancel = 0, n_fault = 0, n_tier_hit = 0, tier_bytes = 0, n_wait = 0, n_upload = 0, upload_bytes = 0;
    int64_t d_reads[2] = {0, 0}, d_bytes[2] = {0, 0}; double d_rdt[2] = {0, 0};
    // fault injection (streaming/nqstream.cu:68-70): minimum spacing between drive reads; share of reads reported as failed
    std::atomic<int64_t> fault_gap_us{0}, fault_ppm{0};
    double next_ok = 0; uint64_t frng = 88172645463325252ull;

    bool hip_ok(hipError_t e, const char* what)
    {
        if (e == hipSuccess) return true;
        std::lock_guard<std::mutex> g(mu);
        if (fail.empty()) fail = std::string(what) + ": " + hipGetErrorString(e);
        return false;
    }

    // ---- reader threads: one blocking pread per record ----
    void read_loop(int d)
    {
        for (;;)
        {
            Op* o;
            {
                std::unique_lock<std::mutex> g(mu);
                rcv[d].wait(g, [&] { return stop.load() || !jobs[d].empty(); });
                if (jobs[d].empty()) return;                       // stop, nothing left
                o = jobs[d].front(); jobs[d].pop_front();
            }
            o->got = read_record(d, host + (size_t)o->entry * rb, o->rec);
            { std::lock_guard<std::mutex> g(mu); landed.push_back(o); }
            cv.notify_one();
        }
    }

    // ---- director ----
    int take_entry(int64_t rec, bool& hit)
    {
        auto it = where.find(rec);
        if (it != where.end()) { hit = true; int e = it->second; ent_users[e]++; ent_stamp[e] = ++clock; return e; }
        hit = false;
        int best = -1;
        for (int e = 0; e < nh; ++e)
            if (ent_users[e] == 0 && (best < 0 || ent_stamp[e] < ent_stamp[best])) best = e;
        if (best < 0) return -1;
        if (ent_rec[best] >= 0) where.erase(ent_rec[best]);
        ent_rec[best] = -1; ent_users[best] = 1; ent_stamp[best] = ++clock;
        return best;
    }
    int pick_drive() const                                        // fewest reads in flight among the drives with room
    {
        int b = -1;
        for (int d = 0; d < nd; ++d)
            if (infl[d] < qd[d] && (b < 0 || infl[d] < infl[b])) b = d;
        return b;
    }
    hipEvent_t get_event()
    {
        if (!evpool.empty()) { hipEvent_t e = evpool.back(); evpool.pop_back(); return e; }
        hipEvent_t e = nullptr;
        hip_ok(hipEventCreateWithFlags(&e, hipEventDisableTiming), "hipEventCreate");
        return e;
    }
    void report(int64_t tag, bool hit, double t_read, double t_e2e)
    {
        std::lock_guard<std::mutex> g(mu);
        done.push_back(NqStreamDone{tag, hit ? 1 : 0, 0, t_read, t_e2e});
    }
    // record bytes (upgrade only) -> stage row -> seq, in this order on the side stream
    void issue_copies(Op* o)
    {
        o->ring = ring_free.back(); ring_free.pop_back();
        int64_t* r = rows + (size_t)o->ring * ROW_W;
        memcpy(r, o->row, sizeof o->row);
        seqs[o->ring] = o->seq;
        bool ok = true;
        for (int i = 0; i < o->nspans && ok; ++i)
            ok = hip_ok(hipMemcpyAsync(o->sp_dst[i], o->sp_src[i], (size_t)o->sp_n[i], hipMemcpyHostToDevice, st), "hipMemcpyAsync(span)");
        if (o->read)
        {
            const void* src = o->tier_src ? (const void*)o->tier_src : (const void*)(host + (size_t)o->entry * rb);
            ok = hip_ok(hipMemcpyAsync(o->slot, src, rb, hipMemcpyHostToDevice, st), "hipMemcpyAsync(record)");
        }
        ok = ok && hip_ok(hipMemcpyAsync(o->stage, r, ROW_W * 8, hipMemcpyHostToDevice, st), "hipMemcpyAsync(row)");
        ok = ok && hip_ok(hipMemcpyAsync(o->seqp, seqs + o->ring, 4, hipMemcpyHostToDevice, st), "hipMemcpyAsync(seq)");
        o->copy_failed = !ok;                                    // the chain stops at the first failure, so seq is never written after one
        o->ev = get_event();
        if (!o->ev || !hip_ok(hipEventRecord(o->ev, st), "hipEventRecord"))
        {
            // no event to watch: the op may not be retired (its pinned row, seq and host entry handed to the next op) while its
            // copies can still be in flight, so wait for the stream here, once, instead
            if (o->ev) { evpool.push_back(o->ev); o->ev = nullptr; }
            if (!hip_ok(hipStreamSynchronize(st), "hipStreamSynchronize")) o->copy_failed = true;
        }
        copying.push_back(o); n_copying++;
    }
    void retire_copies()
    {
        for (size_t i = 0; i < copying.size();)
        {
            Op* o = copying[i];
            if (o->ev)
            {
                const hipError_t q = hipEventQuery(o->ev);
                if (q == hipErrorNotReady) { ++i; continue; }
                if (q != hipSuccess) { hip_ok(q, "hipEventQuery"); o->copy_failed = true; }   // a real error is a failed op, not a landed one
                evpool.push_back(o->ev);
            }
            ring_free.push_back(o->ring);
            if (o->tier_src) tier_users--;
            else if (o->read) ent_users[o->entry]--;
            if (o->copy_failed) report(o->tag, false, -(double)EIO, -1.0);   // as a failed read: the row was never committed
            else report(o->tag, o->hit, o->t_rd - o->t0, now() - o->t0);
            delete o;
            copying[i] = copying.back(); copying.pop_back(); n_copying--;
        }
    }
    // start waiting ops in arrival order; returns true when the fault spacing held the head back
    bool start_ops()
    {
        const bool tier_on = tier_state.load(std::memory_order_acquire) == 1;
        const double gap = 1e-6 * (double)fault_gap_us.load();
        while (!ready.empty() && !ring_free.empty()) { issue_copies(ready.front()); ready.pop_front(); }
        while (ready.empty() && !waiting.empty() && !ring_free.empty())
        {
            Op* o = waiting.front();
            if (!o->read)
            {
                waiting.pop_front(); o->t_rd = o->t0;
                {
                    std::lock_guard<std::mutex> g(mu);
                    if (o->nspans) { n_upload++; for (int i = 0; i < o->nspans; ++i) upload_bytes += o->sp_n[i]; }
                    else n_post++;
                }
                issue_copies(o);
                continue;
            }
            if (tier_on)
            {
                auto ti = tier_at.find(o->rec);
                if (ti != tier_at.end())
                {
                    waiting.pop_front(); o->tier_src = ti->second; o->hit = true; tier_users++; o->t_rd = now();
                    { std::lock_guard<std::mutex> g(mu); n_up++; n_tier_hit++; tier_bytes += (int64_t)rb; }
                    issue_copies(o);
                    continue;
                }
            }
            const bool cached = where.count(o->rec) != 0;
            int d = -1;
            if (!cached)
            {
                d = pick_drive();
                if (d < 0) break;
                if (gap > 0 && now() < next_ok) return true;
            }
            bool hit; const int e = take_entry(o->rec, hit);
            if (e < 0) break;
            waiting.pop_front(); o->entry = e; o->hit = hit;
            if (hit)
            {
                o->t_rd = now();
                { std::lock_guard<std::mutex> g(mu); n_up++; n_hit++; }
                issue_copies(o);
                continue;
            }
            o->drive = d; o->t_sub = now(); infl[d]++; n_reading++;
            if (gap > 0) next_ok = o->t_sub + gap;
            { std::lock_guard<std::mutex> g(mu); n_up++; jobs[d].push_back(o); }
            rcv[d].notify_one();
        }
        return false;
    }
    void reap_reads(std::vector<Op*>& got)
    {
        for (Op* o : got)
        {
            const double t = now();
            infl[o->drive]--; n_reading--;
            bool inject = false;
            if (const int64_t ppm = fault_ppm.load())
            {
                frng ^= frng << 13; frng ^= frng >> 7; frng ^= frng << 17;
                inject = (int64_t)(frng % 1000000) < ppm;
            }
            {
                std::lock_guard<std::mutex> g(mu);
                d_reads[o->drive]++; d_rdt[o->drive] += t - o->t_sub; n_fault += inject;
            }
            if (o->got != (int64_t)rb || inject)
            {   // the expert stays where it is: no row, no seq; t_read < 0 carries the read's result
                ent_users[o->entry]--;
                const double res = (double)(o->got < -1 ? o->got : -1);
                report(o->tag, false, res, -1.0);
                delete o;
                continue;
            }
            o->t_rd = t; ent_rec[o->entry] = o->rec; where[o->rec] = o->entry;
            { std::lock_guard<std::mutex> g(mu); bytes += (int64_t)rb; d_bytes[o->drive] += (int64_t)rb; }
            if (ring_free.empty()) ready.push_back(o); else issue_copies(o);
        }
        got.clear();
    }
    void direct_loop()
    {
        hip_ok(hipSetDevice(dev), "hipSetDevice");
        std::vector<Op*> got;
        bool throttled = false;
        while (!stop.load())
        {
            {
                std::unique_lock<std::mutex> g(mu);
                if (inbox.empty() && landed.empty() && cancel_req.empty())
                {
                    // nothing new: sleep until woken; copies in flight are polled, a throttled head is retried
                    const bool idle = copying.empty() && waiting.empty() && ready.empty() && n_reading == 0 && tier_state.load() != 2;
                    const auto nap = idle ? std::chrono::microseconds(2000)
                                          : (!copying.empty() ? std::chrono::microseconds(30)
                                                              : std::chrono::microseconds(throttled ? 200 : 500));
                    cv.wait_for(g, nap);
                }
                while (!inbox.empty()) { waiting.push_back(inbox.front()); inbox.pop_front(); }
                got.swap(landed);
                if (!cancel_req.empty())
                {   // ops still waiting here have touched neither a drive nor the device
                    std::unordered_set<int64_t> cs(cancel_req.begin(), cancel_req.end());
                    cancel_req.clear();
                    std::deque<Op*> keep;
                    for (Op* o : waiting)
                        if (cs.count(o->tag)) { done.push_back(NqStreamDone{o->tag, 0, 1, CANCELLED, CANCELLED}); n_cancel++; delete o; }
                        else keep.push_back(o);
                    waiting.swap(keep);
                }
            }
            retire_copies();
            if (tier_state.load(std::memory_order_acquire) == 2 && tier_users == 0)
            {
                tier_at.clear();
                hip_ok(hipHostFree(tier_mem), "hipHostFree(tier)");
                tier_mem = nullptr;
                { std::lock_guard<std::mutex> g(mu); tier_n = 0; }
                tier_state.store(3);
            }
            reap_reads(got);
            throttled = start_ops();
            { std::lock_guard<std::mutex> g(mu); n_wait = (int64_t)(waiting.size() + ready.size()); }
        }
    }

    // ---- life cycle ----
    int open_files(const char* path, const char* alt)
    {
        const char* p[2] = {path, alt};
        for (int d = 0; d < nd; ++d)
        {
            bfds[d] = ::open(p[d], O_RDONLY);
            if (bfds[d] < 0) return nq::set_error("nq_stream_open: open %s: %s", p[d], strerror(errno));
            fds[d] = ::open(p[d], O_RDONLY | O_DIRECT);           // -1: no O_DIRECT on this file system
            direct[d] = fds[d] >= 0;
        }
        if (nd == 2)
        {
            struct stat a, b; fstat(bfds[0], &a); fstat(bfds[1], &b);
            if (a.st_size != b.st_size) return nq::set_error("nq_stream_open: alt_path size differs from path");
        }
        return 0;
    }
    // One record (or a part) into pinned memory. O_DIRECT needs the kernel to pin the destination pages itself, which it
    // refuses for the pinned memory of some driver stacks (EFAULT on the first byte): such a drive is read through the
    // page cache from then on, and the cached pages of each record are dropped after the read so that a long run does not
    // fill host memory with them. Returns the bytes read, or -errno.
    int64_t read_record(int d, uint8_t* dst, int64_t rec)
    {
        for (;;)
        {
            const bool dio = direct[d].load() != 0;
            const int fd = dio ? fds[d] : bfds[d];
            size_t got = 0; int64_t err = 0;
            while (got < rb)
            {
                ssize_t r = pread(fd, dst + got, rb - got, (off_t)((size_t)rec * rb + got));
                if (r < 0 && errno == EINTR) continue;
                if (r <= 0) { err = r < 0 ? -(int64_t)errno : 0; break; }
                got += (size_t)r;
            }
            if (dio && got == 0 && (err == -EFAULT || err == -EINVAL)) { direct[d] = 0; continue; }
            if (!dio) posix_fadvise(fd, (off_t)((size_t)rec * rb), (off_t)rb, POSIX_FADV_DONTNEED);
            return got == rb ? (int64_t)rb : (err < 0 ? err : (int64_t)got);
        }
    }
    int start()
    {
        hipError_t e;
        if ((e = hipSetDevice(dev)) != hipSuccess) return nq::set_error("nq_stream_open: hipSetDevice(%d): %s", dev, hipGetErrorString(e));
        if ((e = hipStreamCreateWithFlags(&st, hipStreamNonBlocking)) != hipSuccess) return nq::set_error("nq_stream_open: stream: %s", hipGetErrorString(e));
        nring = (qd[0] + qd[1]) * 4;
        if ((nh && (e = hipHostMalloc((void**)&host, (size_t)nh * rb, hipHostMallocPortable)) != hipSuccess) ||
            (e = hipHostMalloc((void**)&rows, (size_t)nring * ROW_W * 8, hipHostMallocPortable)) != hipSuccess ||
            (e = hipHostMalloc((void**)&seqs, (size_t)nring * 4, hipHostMallocPortable)) != hipSuccess)
            return nq::set_error("nq_stream_open: pinned memory (%zu bytes of entries): %s", (size_t)nh * rb, hipGetErrorString(e));
        if (nh) memset(host, 0, (size_t)nh * rb);                          // first touch of pinned pages is slow (2.7 GB/s against 23): pay it here
        for (int i = 0; i < nring; ++i) ring_free.push_back(i);
        ent_rec.assign(nh, -1); ent_users.assign(nh, 0); ent_stamp.assign(nh, 0);
        if (const char* v = getenv("NQ_FAULT_READ_MS")) fault_gap_us = (int64_t)(atof(v) * 1e3);
        if (const char* v = getenv("NQ_FAULT_FAIL_PPM")) fault_ppm = atoll(v);
        for (int d = 0; d < nd; ++d)
            for (int i = 0; i < qd[d]; ++i) readers.emplace_back([this, d] { read_loop(d); });
        director = std::thread([this] { direct_loop(); });
        return 0;
    }
    void close()
    {
        if (closed) return;
        closed = true;
        stop.store(true);
        { std::lock_guard<std::mutex> g(mu); for (int d = 0; d < 2; ++d) { for (Op* o : jobs[d]) delete o; jobs[d].clear(); } }
        cv.notify_all(); rcv[0].notify_all(); rcv[1].notify_all();
        if (director.joinable()) director.join();
        for (auto& t : readers) if (t.joinable()) t.join();
        if (st) { (void)hipSetDevice(dev); (void)hipStreamSynchronize(st); }
        for (Op* o : copying) { if (o->ev) evpool.push_back(o->ev); delete o; }
        for (Op* o : waiting) delete o;
        for (Op* o : ready) delete o;
        for (Op* o : landed) delete o;
        for (Op* o : inbox) delete o;
        copying.clear(); waiting.clear(); ready.clear(); landed.clear(); inbox.clear();
        for (auto e : evpool) (void)hipEventDestroy(e);
        evpool.clear();
        if (tier_mem) (void)hipHostFree(tier_mem);
        if (host) (void)hipHostFree(host);
        if (rows) (void)hipHostFree(rows);
        if (seqs) (void)hipHostFree(seqs);
        if (st) (void)hipStreamDestroy(st);
        for (int d = 0; d < 2; ++d) { if (fds[d] >= 0) ::close(fds[d]); if (bfds[d] >= 0) ::close(bfds[d]); }
        tier_mem = nullptr; host = nullptr; rows = nullptr; seqs = nullptr; st = nullptr; fds[0] = fds[1] = bfds[0] = bfds[1] = -1;
    }
    ~Engine() { close(); }

    int enqueue(Op* o, const int64_t* row)
    {
        memcpy(o->row, row, sizeof o->row);
        o->t0 = now();
        { std::lock_guard<std::mutex> g(mu); inbox.push_back(o); }
        cv.notify_one();
        return 0;
    }
};

}  // namespace

struct NqStream { Engine e; };

extern "C" {

NqStream* nq_stream_open(const char* path, const char* alt_path, int64_t rec_bytes, int n_host, int qd, int qd_alt, int device)
{
    const bool two = alt_path && alt_path[0];
    const int q1 = two ? (qd_alt > 0 ? qd_alt : qd) : 0;
    const bool no_file = !path || !path[0];                      // uploads and row-only ops only: no drive, no host entries
    if (no_file)
    {
        if (two) { nq::set_error("nq_stream_open: alt_path without path"); return nullptr; }
        NqStream* s = new NqStream;
        Engine& e = s->e;
        e.dev = device; e.nh = 0; e.rb = 0; e.nd = 0; e.qd[0] = qd > 0 ? qd : 8; e.qd[1] = 0;
        if (e.start()) { delete s; return nullptr; }
        return s;
    }
    if (rec_bytes <= 0 || rec_bytes % 4096 != 0 || qd < 1 || n_host < qd + q1)
    {
        nq::set_error("nq_stream_open: need rec_bytes %% 4096 == 0 and n_host >= qd (+ qd_alt) >= 1 (rec_bytes %lld, n_host %d, qd %d, qd_alt %d)",
                      (long long)rec_bytes, n_host, qd, q1);
        return nullptr;
    }
    NqStream* s = new NqStream;
    Engine& e = s->e;
    e.dev = device; e.nh = n_host; e.rb = (size_t)rec_bytes; e.nd = two ? 2 : 1; e.qd[0] = qd; e.qd[1] = q1;
    if (e.open_files(path, alt_path) || e.start()) { delete s; return nullptr; }
    return s;
}

int nq_stream_upgrade(NqStream* s, int64_t tag, int64_t rec, void* slot, void* stage_row, const int64_t* row_host, void* seq_ptr, int32_t seq)
{
    NQ_REQUIRE(s && !s->e.closed, "nq_stream_upgrade: engine is closed");
    NQ_REQUIRE(s->e.nd > 0, "nq_stream_upgrade: this engine was opened without a record file");
    NQ_REQUIRE(rec >= 0 && slot && stage_row && row_host && seq_ptr, "nq_stream_upgrade: null pointer or negative record index");
    Op* o = new Op; o->tag = tag; o->rec = rec; o->read = true; o->slot = slot; o->stage = stage_row; o->seqp = seq_ptr; o->seq = seq;
    return s->e.enqueue(o, row_host);
}

int nq_stream_post(NqStream* s, int64_t tag, void* stage_row, const int64_t* row_host, void* seq_ptr, int32_t seq)
{
    NQ_REQUIRE(s && !s->e.closed, "nq_stream_post: engine is closed");
    NQ_REQUIRE(stage_row && row_host && seq_ptr, "nq_stream_post: null pointer");
    Op* o = new Op; o->tag = tag; o->stage = stage_row; o->seqp = seq_ptr; o->seq = seq;
    return s->e.enqueue(o, row_host);
}

int nq_stream_upload(NqStream* s, int64_t tag, int nspans, const void* const* src_host, void* const* dst, const int64_t* nbytes,
                     void* stage_row, const int64_t* row_host, void* seq_ptr, int32_t seq)
{
    NQ_REQUIRE(s && !s->e.closed, "nq_stream_upload: engine is closed");
    NQ_REQUIRE(nspans >= 1 && nspans <= NQ_STREAM_MAX_SPANS && src_host && dst && nbytes, "nq_stream_upload: 1..%d spans", NQ_STREAM_MAX_SPANS);
    NQ_REQUIRE(stage_row && row_host && seq_ptr, "nq_stream_upload: null pointer");
    Op* o = new Op; o->tag = tag; o->stage = stage_row; o->seqp = seq_ptr; o->seq = seq; o->nspans = nspans;
    for (int i = 0; i < nspans; ++i)
    {
        if (!src_host[i] || !dst[i] || nbytes[i] <= 0) { delete o; return nq::set_error("nq_stream_upload: span %d is empty or null", i); }
        o->sp_src[i] = src_host[i]; o->sp_dst[i] = dst[i]; o->sp_n[i] = nbytes[i];
    }
    return s->e.enqueue(o, row_host);
}

int nq_stream_cancel(NqStream* s, int64_t tag)
{
    NQ_REQUIRE(s && !s->e.closed, "nq_stream_cancel: engine is closed");
    { std::lock_guard<std::mutex> g(s->e.mu); s->e.cancel_req.push_back(tag); }
    s->e.cv.notify_one();
    return 0;
}

int nq_stream_poll(NqStream* s, NqStreamDone* out, int max)
{
    if (!s || !out || max <= 0) return 0;
    std::lock_guard<std::mutex> g(s->e.mu);
    auto& d = s->e.done;
    const int n = (int)d.size() < max ? (int)d.size() : max;
    for (int i = 0; i < n; ++i) out[i] = d[i];
    d.erase(d.begin(), d.begin() + n);
    return n;
}

int64_t nq_stream_tier_load(NqStream* s, const int64_t* recs, int64_t n)
{
    if (!s || s->e.closed) { nq::set_error("nq_stream_tier_load: engine is closed"); return -1; }
    Engine& e = s->e;
    if (e.tier_state.load() != 0) { nq::set_error("nq_stream_tier_load: tier already loaded / dropped"); return -1; }
    if (n <= 0) return 0;
    if (e.nd == 0 || e.rb == 0) { nq::set_error("nq_stream_tier_load: this engine was opened without a record file (uploads and row-only ops only)"); return -1; }
    if (!recs) { nq::set_error("nq_stream_tier_load: null record list"); return -1; }
    hipError_t he = hipSetDevice(e.dev);
    uint8_t* m = nullptr;
    if (he == hipSuccess) he = hipHostMalloc((void**)&m, (size_t)n * e.rb, hipHostMallocPortable);
    if (he != hipSuccess) { nq::set_error("nq_stream_tier_load: %lld bytes of pinned memory: %s", (long long)n * (long long)e.rb, hipGetErrorString(he)); return -1; }
    std::atomic<int64_t> next{0}, bad{0};
    std::vector<std::thread> ths;
    for (int t = 0; t < 8; ++t)
        ths.emplace_back([&, t] {
            const int d = t % e.nd;
            for (int64_t i; (i = next.fetch_add(1)) < n;)
            {
                const int64_t got = e.read_record(d, m + (size_t)i * e.rb, recs[i]);
                if (got != (int64_t)e.rb) bad++;
            }
        });
    for (auto& t : ths) t.join();
    if (bad.load()) { (void)hipHostFree(m); nq::set_error("nq_stream_tier_load: %lld short reads", (long long)bad.load()); return -1; }
    {
        std::lock_guard<std::mutex> g(e.mu);       // the director reads tier_at only after it has seen state 1
        e.tier_mem = m; e.tier_n = (size_t)n;
        for (int64_t i = 0; i < n; ++i) e.tier_at[recs[i]] = m + (size_t)i * e.rb;
    }
    e.tier_state.store(1, std::memory_order_release);
    e.cv.notify_one();
    return n;
}

int nq_stream_tier_drop(NqStream* s)
{
    NQ_REQUIRE(s && !s->e.closed, "nq_stream_tier_drop: engine is closed");
    int one = 1;
    s->e.tier_state.compare_exchange_strong(one, 2);
    s->e.cv.notify_one();
    return 0;
}

int nq_stream_set_fault(NqStream* s, double read_ms, int64_t fail_ppm)
{
    NQ_REQUIRE(s && !s->e.closed, "nq_stream_set_fault: engine is closed");
    s->e.fault_gap_us = (int64_t)(read_ms * 1e3);
    s->e.fault_ppm = fail_ppm;
    return 0;
}

int nq_stream_stats(NqStream* s, NqStreamStats* out)
{
    NQ_REQUIRE(s && out, "nq_stream_stats: null pointer");
    Engine& e = s->e;
    std::lock_guard<std::mutex> g(e.mu);
    memset(out, 0, sizeof *out);
    out->upgrades = e.n_up; out->posts = e.n_post; out->host_hits = e.n_hit; out->bytes_read = e.bytes;
    out->fault_injected = e.n_fault; out->queued = (int64_t)e.inbox.size();
    out->reading = (int64_t)e.n_reading.load(); out->copying = (int64_t)e.n_copying.load();
    out->drives = e.nd; out->n_host = e.nh;
    for (int d = 0; d < 2; ++d)
    {
        out->drive_qd[d] = e.qd[d]; out->drive_inflight[d] = e.infl[d].load(); out->drive_reads[d] = e.d_reads[d];
        out->drive_bytes[d] = e.d_bytes[d]; out->drive_read_s[d] = e.d_rdt[d]; out->drive_direct[d] = e.direct[d].load();
    }
    out->tier_state = e.tier_state.load(); out->tier_recs = (int64_t)e.tier_n; out->tier_hits = e.n_tier_hit;
    out->tier_bytes = e.tier_bytes; out->cancelled = e.n_cancel; out->waiting = e.n_wait; out->now = now();
    out->uploads = e.n_upload; out->upload_bytes = e.upload_bytes;
    out->failed = e.fail.empty() ? 0 : 1;
    if (!e.fail.empty()) nq::set_error("nq_stream: %s", e.fail.c_str());
    return 0;
}

void nq_stream_close(NqStream* s)
{
    if (!s) return;
    s->e.close();
    delete s;
}

}  // extern "C"
