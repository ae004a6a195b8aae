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
    int entry = -1, stg = -1, drive = -1;   // host entry, row-staging index, drive that read the record
    bool hit = false, copy_failed = false;   // copy_failed: a HIP call of this op's copies failed (seq was not written)
    const uint8_t* tier_src = nullptr;
    int64_t got = 0;                     // bytes the read returned, or -errno
    hipEvent_t ev = nullptr;
};

// One drive (a copy of the record file): its descriptors, queue depth, the reads handed to its reader threads, its counters
struct Drive
{
    int fd_direct = -1, fd_buffered = -1;   // O_DIRECT descriptor (-1: the file system has none) and page-cache descriptor
    int depth = 0;                          // reader threads = reads in flight at most
    std::atomic<int> use_direct{0};         // reads currently go through fd_direct
    std::atomic<int> in_flight{0};          // written by the director, read by stats()
    std::deque<Op*> queue;                  // under Upgrader::mu
    std::condition_variable wake;           // wakes this drive's readers
    int64_t reads = 0, bytes = 0; double read_s = 0;   // under Upgrader::mu
};

// The pinned host entries as a cache of records (director thread only): which record an entry holds complete, how many ops
// are reading into it or in_copy out of it, and when it was last taken. A record that is not held takes the entry that has
// gone unused longest among those nobody uses.
struct HostCache
{
    struct Entry { int64_t record = -1; int users = 0; uint64_t last_use = 0; };
    std::vector<Entry> entry;
    std::unordered_map<int64_t, int> index;
    uint64_t tick = 0;
    void reset(int n) { entry.assign((size_t)n, Entry{}); index.clear(); tick = 0; }
    bool holds(int64_t rec) const { return index.find(rec) != index.end(); }
    int acquire(int64_t rec, bool& hit)     // -1: every entry is in use
    {
        const auto found = index.find(rec);
        hit = found != index.end();
        int e = hit ? found->second : -1;
        if (!hit)
        {
            for (int i = 0; i < (int)entry.size(); ++i)
                if (entry[i].users == 0 && (e < 0 || entry[i].last_use < entry[e].last_use)) e = i;
            if (e < 0) return -1;
            if (entry[e].record >= 0) index.erase(entry[e].record);
            entry[e].record = -1;
        }
        entry[e].users += 1;
        entry[e].last_use = ++tick;
        return e;
    }
    void filled(int e, int64_t rec) { entry[e].record = rec; index[rec] = e; }
    void release(int e) { entry[e].users -= 1; }
};

// pinned staging of (row, seq) pairs: the source of an op's last two copies must stay put until they have completed
struct RowStaging
{
    int64_t* row = nullptr; int32_t* seq = nullptr;
    int n = 0;
    std::vector<int> unused;
    bool any() const { return !unused.empty(); }
    int put(const int64_t* r, int32_t q)
    {
        const int i = unused.back(); unused.pop_back();
        memcpy(row + (size_t)i * ROW_W, r, ROW_W * sizeof(int64_t));
        seq[i] = q;
        return i;
    }
    void give_back(int i) { unused.push_back(i); }
};

struct Upgrader
{
    // configuration
    int dev = 0, nh = 0, nd = 1;
    size_t rb = 0;
    Drive drive[2];
    // pinned memory
    uint8_t* host = nullptr;             // nh entries of rb bytes
    RowStaging staging;
    HostCache cache;
    // RAM tier phases: 0 none, 1 active, 2 drop requested, 3 dropped
    std::atomic<int> ram_tier_phase{0};
    uint8_t* ram_tier_buf = nullptr; size_t ram_tier_count = 0; int ram_tier_readers = 0;
    std::unordered_map<int64_t, const uint8_t*> ram_tier_index;
    // threads
    hipStream_t st = nullptr;
    std::mutex mu;                       // guards: inbox, to_cancel, landed, done, the drives' queues, counters read by stats()
    std::condition_variable cv;          // wakes the director
    std::deque<Op*> inbox;
    std::vector<int64_t> to_cancel;
    std::vector<Op*> landed;             // reads that returned, not yet seen by the director
    std::vector<NqStreamDone> done;
    std::vector<std::thread> readers;
    std::thread director;
    std::atomic<bool> stop{false};
    bool closed = false;
    std::vector<hipEvent_t> spare_events;
    std::string fail;                    // first HIP failure of the director (reported by stats / poll)
    // director-side queues
    std::deque<Op*> pending, read_done;  // not started yet; read complete, pending for row staging
    std::vector<Op*> in_copy;
    std::atomic<int> n_reading{0}, n_copying{0};   // written by the director, read by stats()
    // counters (under mu)
    int64_t n_up = 0, n_post = 0, n_hit = 0, bytes = 0, n_cancel = 0, n_fault = 0, n_tier_hit = 0, tier_bytes = 0, n_wait = 0, n_upload = 0, upload_bytes = 0;
    // fault injection (streaming/nqstream.cu:68-70): minimum spacing between drive reads; share of reads reported as failed
    std::atomic<int64_t> fault_gap_us{0}, fault_ppm{0};
    double next_ok = 0;
    uint64_t fault_lcg = 0x9E3779B97F4A7C15ull;                  // 64-bit linear congruential generator; the top bits decide
    bool fault_draw(int64_t ppm)
    {
        fault_lcg = fault_lcg * 6364136223846793005ull + 1442695040888963407ull;
        return (int64_t)((fault_lcg >> 33) % 1000000ull) < ppm;
    }

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
                drive[d].wake.wait(g, [&] { return stop.load() || !drive[d].queue.empty(); });
                if (drive[d].queue.empty()) return;                       // stop, nothing left
                o = drive[d].queue.front(); drive[d].queue.pop_front();
            }
            o->got = read_record(d, host + (size_t)o->entry * rb, o->rec);
            { std::lock_guard<std::mutex> g(mu); landed.push_back(o); }
            cv.notify_one();
        }
    }

    // ---- director ----
    int least_busy_drive() const                                  // among the drives with a free reader; -1: none
    {
        int best = -1, load = 0;
        for (int d = 0; d < nd; ++d)
        {
            const int n = drive[d].in_flight.load();
            if (n >= drive[d].depth) continue;
            if (best < 0 || n < load) { best = d; load = n; }
        }
        return best;
    }
    hipEvent_t get_event()
    {
        if (!spare_events.empty()) { hipEvent_t e = spare_events.back(); spare_events.pop_back(); return e; }
        hipEvent_t e = nullptr;
        hip_ok(hipEventCreateWithFlags(&e, hipEventDisableTiming), "hipEventCreate");
        return e;
    }
    void report(int64_t tag, bool hit, double t_read, double t_e2e)
    {
        std::lock_guard<std::mutex> g(mu);
        done.push_back(NqStreamDone{tag, hit ? 1 : 0, 0, t_read, t_e2e});
    }
    // The op's device writes, in the order the mailbox relies on, all on the side stream: payload (upload spans, or the record
    // from the RAM tier / its host entry), then the row into the mailbox's stage, then the sequence number. The chain stops at
    // the first HIP failure, so seq is never written after one.
    void push_to_device(Op* o)
    {
        o->stg = staging.put(o->row, o->seq);
        struct Copy { void* dst; const void* src; size_t n; const char* what; };
        std::vector<Copy> chain;
        for (int i = 0; i < o->nspans; ++i) chain.push_back({o->sp_dst[i], o->sp_src[i], (size_t)o->sp_n[i], "hipMemcpyAsync(span)"});
        if (o->read) chain.push_back({o->slot, o->tier_src ? (const void*)o->tier_src : (const void*)(host + (size_t)o->entry * rb), rb, "hipMemcpyAsync(record)"});
        chain.push_back({o->stage, staging.row + (size_t)o->stg * ROW_W, ROW_W * sizeof(int64_t), "hipMemcpyAsync(row)"});
        chain.push_back({o->seqp, staging.seq + o->stg, sizeof(int32_t), "hipMemcpyAsync(seq)"});
        for (const Copy& c : chain)
            if (!hip_ok(hipMemcpyAsync(c.dst, c.src, c.n, hipMemcpyHostToDevice, st), c.what)) { o->copy_failed = true; break; }
        o->ev = get_event();
        if (!o->ev || !hip_ok(hipEventRecord(o->ev, st), "hipEventRecord"))
        {
            // no event to watch: the op may not be retired (its pinned row, seq and host entry handed to the next op) while its
            // copies can still be in flight, so wait for the stream here, once, instead
            if (o->ev) { spare_events.push_back(o->ev); o->ev = nullptr; }
            if (!hip_ok(hipStreamSynchronize(st), "hipStreamSynchronize")) o->copy_failed = true;
        }
        in_copy.push_back(o); n_copying++;
    }
    void collect_finished_copies()
    {
        for (size_t i = 0; i < in_copy.size();)
        {
            Op* o = in_copy[i];
            if (o->ev)
            {
                const hipError_t q = hipEventQuery(o->ev);
                if (q == hipErrorNotReady) { ++i; continue; }
                if (q != hipSuccess) { hip_ok(q, "hipEventQuery"); o->copy_failed = true; }   // a real error is a failed op, not a landed one
                spare_events.push_back(o->ev);
            }
            staging.give_back(o->stg);
            if (o->tier_src) ram_tier_readers--;
            else if (o->read) cache.release(o->entry);
            if (o->copy_failed) report(o->tag, false, -(double)EIO, -1.0);   // as a failed read: the row was never committed
            else report(o->tag, o->hit, o->t_rd - o->t0, now() - o->t0);
            delete o;
            in_copy[i] = in_copy.back(); in_copy.pop_back(); n_copying--;
        }
    }
    // start pending ops in arrival order; returns true when the fault spacing held the head back
    bool start_ops()
    {
        const bool tier_on = ram_tier_phase.load(std::memory_order_acquire) == 1;
        const double gap = 1e-6 * (double)fault_gap_us.load();
        while (!read_done.empty() && staging.any()) { push_to_device(read_done.front()); read_done.pop_front(); }
        while (read_done.empty() && !pending.empty() && staging.any())
        {
            Op* o = pending.front();
            if (!o->read)
            {
                pending.pop_front(); o->t_rd = o->t0;
                {
                    std::lock_guard<std::mutex> g(mu);
                    if (o->nspans) { n_upload++; for (int i = 0; i < o->nspans; ++i) upload_bytes += o->sp_n[i]; }
                    else n_post++;
                }
                push_to_device(o);
                continue;
            }
            if (tier_on)
            {
                auto ti = ram_tier_index.find(o->rec);
                if (ti != ram_tier_index.end())
                {
                    pending.pop_front(); o->tier_src = ti->second; o->hit = true; ram_tier_readers++; o->t_rd = now();
                    { std::lock_guard<std::mutex> g(mu); n_up++; n_tier_hit++; tier_bytes += (int64_t)rb; }
                    push_to_device(o);
                    continue;
                }
            }
            const bool cached = cache.holds(o->rec);
            int d = -1;
            if (!cached)
            {
                d = least_busy_drive();
                if (d < 0) break;
                if (gap > 0 && now() < next_ok) return true;
            }
            bool hit; const int e = cache.acquire(o->rec, hit);
            if (e < 0) break;
            pending.pop_front(); o->entry = e; o->hit = hit;
            if (hit)
            {
                o->t_rd = now();
                { std::lock_guard<std::mutex> g(mu); n_up++; n_hit++; }
                push_to_device(o);
                continue;
            }
            o->drive = d; o->t_sub = now(); drive[d].in_flight++; n_reading++;
            if (gap > 0) next_ok = o->t_sub + gap;
            { std::lock_guard<std::mutex> g(mu); n_up++; drive[d].queue.push_back(o); }
            drive[d].wake.notify_one();
        }
        return false;
    }
    void reap_reads(std::vector<Op*>& got)
    {
        for (Op* o : got)
        {
            const double t = now();
            drive[o->drive].in_flight--; n_reading--;
            bool inject = false;
            if (const int64_t ppm = fault_ppm.load()) inject = fault_draw(ppm);
            {
                std::lock_guard<std::mutex> g(mu);
                drive[o->drive].reads++; drive[o->drive].read_s += t - o->t_sub; n_fault += inject;
            }
            if (o->got != (int64_t)rb || inject)
            {   // the expert stays where it is: no row, no seq; t_read < 0 carries the read's result
                cache.release(o->entry);
                const double res = (double)(o->got < -1 ? o->got : -1);
                report(o->tag, false, res, -1.0);
                delete o;
                continue;
            }
            o->t_rd = t; cache.filled(o->entry, o->rec);
            { std::lock_guard<std::mutex> g(mu); bytes += (int64_t)rb; drive[o->drive].bytes += (int64_t)rb; }
            if (staging.any()) push_to_device(o); else read_done.push_back(o);
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
                if (inbox.empty() && landed.empty() && to_cancel.empty())
                {
                    // nothing new: sleep until woken; copies in flight are polled, a throttled head is retried
                    const bool idle = in_copy.empty() && pending.empty() && read_done.empty() && n_reading == 0 && ram_tier_phase.load() != 2;
                    const auto nap = idle ? std::chrono::microseconds(2000)
                                          : (!in_copy.empty() ? std::chrono::microseconds(30)
                                                              : std::chrono::microseconds(throttled ? 200 : 500));
                    cv.wait_for(g, nap);
                }
                while (!inbox.empty()) { pending.push_back(inbox.front()); inbox.pop_front(); }
                got.swap(landed);
                if (!to_cancel.empty())
                {   // ops still pending here have touched neither a drive nor the device
                    std::unordered_set<int64_t> cs(to_cancel.begin(), to_cancel.end());
                    to_cancel.clear();
                    std::deque<Op*> keep;
                    for (Op* o : pending)
                        if (cs.count(o->tag)) { done.push_back(NqStreamDone{o->tag, 0, 1, CANCELLED, CANCELLED}); n_cancel++; delete o; }
                        else keep.push_back(o);
                    pending.swap(keep);
                }
            }
            collect_finished_copies();
            if (ram_tier_phase.load(std::memory_order_acquire) == 2 && ram_tier_readers == 0)
            {
                ram_tier_index.clear();
                hip_ok(hipHostFree(ram_tier_buf), "hipHostFree(tier)");
                ram_tier_buf = nullptr;
                { std::lock_guard<std::mutex> g(mu); ram_tier_count = 0; }
                ram_tier_phase.store(3);
            }
            reap_reads(got);
            throttled = start_ops();
            { std::lock_guard<std::mutex> g(mu); n_wait = (int64_t)(pending.size() + read_done.size()); }
        }
    }

    // ---- life cycle ----
    int open_files(const char* path, const char* alt)
    {
        const char* p[2] = {path, alt};
        for (int d = 0; d < nd; ++d)
        {
            drive[d].fd_buffered = ::open(p[d], O_RDONLY);
            if (drive[d].fd_buffered < 0) return nq::set_error("nq_stream_open: open %s: %s", p[d], strerror(errno));
            drive[d].fd_direct = ::open(p[d], O_RDONLY | O_DIRECT);           // -1: no O_DIRECT on this file system
            drive[d].use_direct = drive[d].fd_direct >= 0;
        }
        if (nd == 2)
        {
            struct stat a, b; fstat(drive[0].fd_buffered, &a); fstat(drive[1].fd_buffered, &b);
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
            const bool dio = drive[d].use_direct.load() != 0;
            const int fd = dio ? drive[d].fd_direct : drive[d].fd_buffered;
            size_t got = 0; int64_t err = 0;
            while (got < rb)
            {
                ssize_t r = pread(fd, dst + got, rb - got, (off_t)((size_t)rec * rb + got));
                if (r < 0 && errno == EINTR) continue;
                if (r <= 0) { err = r < 0 ? -(int64_t)errno : 0; break; }
                got += (size_t)r;
            }
            if (dio && got == 0 && (err == -EFAULT || err == -EINVAL)) { drive[d].use_direct = 0; continue; }
            if (!dio) posix_fadvise(fd, (off_t)((size_t)rec * rb), (off_t)rb, POSIX_FADV_DONTNEED);
            return got == rb ? (int64_t)rb : (err < 0 ? err : (int64_t)got);
        }
    }
    int start()
    {
        hipError_t e;
        if ((e = hipSetDevice(dev)) != hipSuccess) return nq::set_error("nq_stream_open: hipSetDevice(%d): %s", dev, hipGetErrorString(e));
        if ((e = hipStreamCreateWithFlags(&st, hipStreamNonBlocking)) != hipSuccess) return nq::set_error("nq_stream_open: stream: %s", hipGetErrorString(e));
        staging.n = (drive[0].depth + drive[1].depth) * 4;
        if ((nh && (e = hipHostMalloc((void**)&host, (size_t)nh * rb, hipHostMallocPortable)) != hipSuccess) ||
            (e = hipHostMalloc((void**)&staging.row, (size_t)staging.n * ROW_W * 8, hipHostMallocPortable)) != hipSuccess ||
            (e = hipHostMalloc((void**)&staging.seq, (size_t)staging.n * 4, hipHostMallocPortable)) != hipSuccess)
            return nq::set_error("nq_stream_open: pinned memory (%zu bytes of entries): %s", (size_t)nh * rb, hipGetErrorString(e));
        if (nh) memset(host, 0, (size_t)nh * rb);                          // first touch of pinned pages is slow (2.7 GB/s against 23): pay it here
        for (int i = 0; i < staging.n; ++i) staging.give_back(i);
        cache.reset(nh);
        if (const char* v = getenv("NQ_FAULT_READ_MS")) fault_gap_us = (int64_t)(atof(v) * 1e3);
        if (const char* v = getenv("NQ_FAULT_FAIL_PPM")) fault_ppm = atoll(v);
        for (int d = 0; d < nd; ++d)
            for (int i = 0; i < drive[d].depth; ++i) readers.emplace_back([this, d] { read_loop(d); });
        director = std::thread([this] { direct_loop(); });
        return 0;
    }
    void close()
    {
        if (closed) return;
        closed = true;
        stop.store(true);
        { std::lock_guard<std::mutex> g(mu); for (int d = 0; d < 2; ++d) { for (Op* o : drive[d].queue) delete o; drive[d].queue.clear(); } }
        cv.notify_all(); drive[0].wake.notify_all(); drive[1].wake.notify_all();
        if (director.joinable()) director.join();
        for (auto& t : readers) if (t.joinable()) t.join();
        if (st) { (void)hipSetDevice(dev); (void)hipStreamSynchronize(st); }
        for (Op* o : in_copy) { if (o->ev) spare_events.push_back(o->ev); delete o; }
        for (Op* o : pending) delete o;
        for (Op* o : read_done) delete o;
        for (Op* o : landed) delete o;
        for (Op* o : inbox) delete o;
        in_copy.clear(); pending.clear(); read_done.clear(); landed.clear(); inbox.clear();
        for (auto e : spare_events) (void)hipEventDestroy(e);
        spare_events.clear();
        if (ram_tier_buf) (void)hipHostFree(ram_tier_buf);
        if (host) (void)hipHostFree(host);
        if (staging.row) (void)hipHostFree(staging.row);
        if (staging.seq) (void)hipHostFree(staging.seq);
        if (st) (void)hipStreamDestroy(st);
        for (int d = 0; d < 2; ++d) { if (drive[d].fd_direct >= 0) ::close(drive[d].fd_direct); if (drive[d].fd_buffered >= 0) ::close(drive[d].fd_buffered); }
        ram_tier_buf = nullptr; host = nullptr; staging.row = nullptr; staging.seq = nullptr; st = nullptr;
        for (int d = 0; d < 2; ++d) drive[d].fd_direct = drive[d].fd_buffered = -1;
    }
    ~Upgrader() { close(); }

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

struct NqStream { Upgrader e; };

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
        Upgrader& e = s->e;
        e.dev = device; e.nh = 0; e.rb = 0; e.nd = 0; e.drive[0].depth = qd > 0 ? qd : 8; e.drive[1].depth = 0;
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
    Upgrader& e = s->e;
    e.dev = device; e.nh = n_host; e.rb = (size_t)rec_bytes; e.nd = two ? 2 : 1; e.drive[0].depth = qd; e.drive[1].depth = q1;
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
    { std::lock_guard<std::mutex> g(s->e.mu); s->e.to_cancel.push_back(tag); }
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
    Upgrader& e = s->e;
    if (e.ram_tier_phase.load() != 0) { nq::set_error("nq_stream_tier_load: tier already loaded / dropped"); return -1; }
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
        std::lock_guard<std::mutex> g(e.mu);       // the director reads ram_tier_index only after it has seen state 1
        e.ram_tier_buf = m; e.ram_tier_count = (size_t)n;
        for (int64_t i = 0; i < n; ++i) e.ram_tier_index[recs[i]] = m + (size_t)i * e.rb;
    }
    e.ram_tier_phase.store(1, std::memory_order_release);
    e.cv.notify_one();
    return n;
}

int nq_stream_tier_drop(NqStream* s)
{
    NQ_REQUIRE(s && !s->e.closed, "nq_stream_tier_drop: engine is closed");
    int one = 1;
    s->e.ram_tier_phase.compare_exchange_strong(one, 2);
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
    Upgrader& e = s->e;
    std::lock_guard<std::mutex> g(e.mu);
    memset(out, 0, sizeof *out);
    out->upgrades = e.n_up; out->posts = e.n_post; out->host_hits = e.n_hit; out->bytes_read = e.bytes;
    out->fault_injected = e.n_fault; out->queued = (int64_t)e.inbox.size();
    out->reading = (int64_t)e.n_reading.load(); out->copying = (int64_t)e.n_copying.load();
    out->drives = e.nd; out->n_host = e.nh;
    for (int d = 0; d < 2; ++d)
    {
        out->drive_qd[d] = e.drive[d].depth; out->drive_inflight[d] = e.drive[d].in_flight.load(); out->drive_reads[d] = e.drive[d].reads;
        out->drive_bytes[d] = e.drive[d].bytes; out->drive_read_s[d] = e.drive[d].read_s; out->drive_direct[d] = e.drive[d].use_direct.load();
    }
    out->tier_state = e.ram_tier_phase.load(); out->tier_recs = (int64_t)e.ram_tier_count; out->tier_hits = e.n_tier_hit;
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
