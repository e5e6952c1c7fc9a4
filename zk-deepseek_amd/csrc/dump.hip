// Witness dump writer: raw little-endian bytes of a contiguous tensor into a file, as the reference's saveTensor
// writes them (inference/model.py:94-102 and its ~30 call sites per layer), without stalling the host.
//
// The reference copies every tensor to the host synchronously and writes the file before it goes on.  Here a
// dump enqueues a device-to-host copy on the null stream, behind the kernels that produced the tensor and ahead of
// anything launched later that may overwrite it, into a pinned staging slot, and returns; a writer thread waits
// for the copy's event and writes the file.  Tensors larger than a slot go through in pieces that are appended
// in order.  zk_dump_flush() waits for everything queued so far.  The bytes in the files are identical.
#include "common.h"
#include "../../include/int64gemm.h"

#include <condition_variable>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <deque>
#include <mutex>
#include <string>
#include <thread>

namespace zk {

constexpr size_t kSlotBytes = (size_t)4 << 20;       // staging slots of 4 MB, allocated when first needed,
constexpr int kSlots = 128;                          // 512 MB at most (a layer's worth of dumps queues without waiting)

struct DumpJob {
    std::string path;
    int slot;
    size_t bytes;
    bool append;             // a later piece of a large tensor
    hipEvent_t ev;           // null for host data (already in the slot)
};

struct DumpState {
    std::mutex mu;
    std::condition_variable cv_jobs, cv_slots, cv_idle;
    std::deque<DumpJob> jobs;
    unsigned char *slot_mem[kSlots] = {};
    hipEvent_t slot_ev[kSlots] = {};
    bool slot_busy[kSlots] = {};
    bool have_gpu = false, started = false;
    int in_flight = 0;       // jobs queued or being written
    long failures = 0;
    std::string first_failure;
};

// never destroyed: the detached writer thread may still be waiting on it when the process exits
static DumpState &g_dump = *new DumpState;

static void dump_writer()
{
    for (;;) {
        DumpJob job;
        {
            std::unique_lock<std::mutex> lock(g_dump.mu);
            g_dump.cv_jobs.wait(lock, [] { return !g_dump.jobs.empty(); });
            job = g_dump.jobs.front();
            g_dump.jobs.pop_front();
        }
        bool ok = true;
        std::string why;
        if (job.ev && hipEventSynchronize(job.ev) != hipSuccess) { ok = false; why = "device-to-host copy failed"; }
        if (ok) {
            FILE *f = fopen(job.path.c_str(), job.append ? "ab" : "wb");
            if (!f) { ok = false; why = "cannot open " + job.path; }
            else {
                if (job.bytes && fwrite(g_dump.slot_mem[job.slot], 1, job.bytes, f) != job.bytes) { ok = false; why = "short write to " + job.path; }
                if (fclose(f) != 0 && ok) { ok = false; why = "cannot close " + job.path; }
            }
        }
        {
            std::lock_guard<std::mutex> lock(g_dump.mu);
            if (!ok) {
                if (g_dump.failures++ == 0) g_dump.first_failure = why;
            }
            g_dump.slot_busy[job.slot] = false;
            g_dump.in_flight--;
        }
        g_dump.cv_slots.notify_all();
        g_dump.cv_idle.notify_all();
    }
}

// called with the lock held
static bool dump_start()
{
    if (g_dump.started) return true;
    int ndev = 0;
    g_dump.have_gpu = hipGetDeviceCount(&ndev) == hipSuccess && ndev > 0;
    if (!g_dump.have_gpu) (void)hipGetLastError();
    std::thread(dump_writer).detach();
    g_dump.started = true;
    return true;
}

// called with the lock held: memory (pinned when a device is there, plain otherwise) and event of a slot
static bool dump_slot_ready(int i)
{
    if (g_dump.slot_mem[i]) return true;
    void *p = nullptr;
    if (g_dump.have_gpu) {
        if (hipHostMalloc(&p, kSlotBytes, hipHostMallocDefault) != hipSuccess) { (void)hipGetLastError(); return false; }
        if (hipEventCreateWithFlags(&g_dump.slot_ev[i], hipEventDisableTiming) != hipSuccess) { (void)hipGetLastError(); (void)hipHostFree(p); return false; }
    } else {
        p = malloc(kSlotBytes);
        if (!p) return false;
    }
    g_dump.slot_mem[i] = static_cast<unsigned char *>(p);
    return true;
}

static int dump_enqueue(const char *name, const char *path, const void *src, size_t bytes, bool device)
{
    if (!path || (!src && bytes)) { set_error(kBadArgument, "%s: null pointer", name); return -1; }
    size_t done = 0;
    bool first = true;
    do {
        const size_t n = bytes - done < kSlotBytes ? bytes - done : kSlotBytes;
        int slot = -1;
        {
            std::unique_lock<std::mutex> lock(g_dump.mu);
            if (!dump_start()) { set_error(kLaunchFailure, "%s: cannot start the writer", name); return -1; }
            if (device && !g_dump.have_gpu) { set_error(kLaunchFailure, "%s: no device", name); return -1; }
            // the lowest free slot, so memory is only allocated for as many slots as are ever in flight at once
            g_dump.cv_slots.wait(lock, [&] {
                for (int i = 0; i < kSlots; i++)
                    if (!g_dump.slot_busy[i]) { slot = i; return true; }
                return false;
            });
            if (!dump_slot_ready(slot)) { set_error(kLaunchFailure, "%s: cannot allocate a staging buffer", name); return -1; }
            g_dump.slot_busy[slot] = true;
            g_dump.in_flight++;
        }
        DumpJob job{ path, slot, n, !first, nullptr };
        bool ok = true;
        if (device) {
            ok = n == 0 || hipMemcpyAsync(g_dump.slot_mem[slot], static_cast<const unsigned char *>(src) + done, n, hipMemcpyDeviceToHost, 0) == hipSuccess;
            ok = ok && hipEventRecord(g_dump.slot_ev[slot], 0) == hipSuccess;
            job.ev = g_dump.slot_ev[slot];
        } else if (n) {
            memcpy(g_dump.slot_mem[slot], static_cast<const unsigned char *>(src) + done, n);
        }
        {
            std::lock_guard<std::mutex> lock(g_dump.mu);
            if (!ok) {
                (void)hipGetLastError();
                g_dump.slot_busy[slot] = false;
                g_dump.in_flight--;
            } else {
                g_dump.jobs.push_back(job);
            }
        }
        if (!ok) {
            g_dump.cv_slots.notify_all();
            set_error(kLaunchFailure, "%s: cannot enqueue the copy of %s", name, path);
            return -1;
        }
        g_dump.cv_jobs.notify_one();
        done += n;
        first = false;
    } while (done < bytes);
    return 0;
}

}  // namespace zk

extern "C" {

int zk_dump_device(const char *path, const void *device_ptr, size_t bytes)
{
    return zk::dump_enqueue("zk_dump_device", path, device_ptr, bytes, true);
}

int zk_dump_host(const char *path, const void *host_ptr, size_t bytes)
{
    return zk::dump_enqueue("zk_dump_host", path, host_ptr, bytes, false);
}

long zk_dump_flush(void)
{
    std::unique_lock<std::mutex> lock(zk::g_dump.mu);
    zk::g_dump.cv_idle.wait(lock, [] { return zk::g_dump.in_flight == 0; });
    const long failed = zk::g_dump.failures;
    if (failed) {
        const std::string why = zk::g_dump.first_failure;
        zk::g_dump.failures = 0;
        zk::g_dump.first_failure.clear();
        lock.unlock();
        zk::set_error(zk::kLaunchFailure, "zk_dump_flush: %ld dump(s) failed, the first: %s", failed, why.c_str());
    }
    return failed;
}

}  // extern "C"
