// Self-tests of host-layer pieces that have no other way in from a test: the device buffer type that stands in for
// the reference's SyncArray (the cases of src/test/test_syncmem.cpp and test_syncarray.cpp that apply), the kernel-row
// cache's bookkeeping, and the host's bounded wait for the local solver.  Built into a library of its own, next to
// the tests; the product libraries do not contain it.
#include <chrono>
#include <stdexcept>
#include <string>
#include <vector>

#include "../../thundersvm_amd/host/device.h"
#include "../../thundersvm_amd/host/row_cache.h"
#include "../../thundersvm_amd/host/solver.h"

namespace {

thread_local std::string g_selftest_error;

#define SELFTEST_GUARD(body)                       \
    try {                                          \
        body;                                      \
        return 0;                                  \
    } catch (const std::exception &e) {            \
        g_selftest_error = e.what();               \
        return -1;                                 \
    }

using tsvm::RowCache;

// Drives RowCache the way a solve does (first working set of ws rows, then q = ws / 2 new rows per iteration while the
// previous new half stays pinned) on a cyclic sequence of n_ids ids, and checks after every step that each row of the
// working set has a slot of its own and that the tables agree.  Returns the number of hits, or -1 with `what` set.
long long row_cache_selftest(int n_ids, int slots, int ws, int iterations, std::string &what) {
    if (n_ids < ws || slots < 2 * ws || ws < 2 || ws % 2) { what = "bad arguments"; return -1; }
    RowCache c;
    c.init(n_ids, slots);
    const int q = ws / 2;
    std::vector<int> ids(ws), slot(ws);
    long long hits = 0;
    int next_id = 0;
    for (int it = 0; it < iterations; ++it) {
        const int n_new = it == 0 ? ws : q, first_new = it == 0 ? 0 : q;
        if (it > 0) {
            for (int t = 0; t < q; ++t) c.release(slot[t]);
            for (int t = 0; t < q; ++t) { ids[t] = ids[t + q]; slot[t] = slot[t + q]; }
        }
        for (int t = 0; t < n_new; ++t) {
            const int id = next_id;
            next_id = (next_id + 1) % n_ids;
            int s = c.lookup(id);
            if (s >= 0) ++hits;
            else s = c.insert(id);
            if (s < 0) { what = "no slot left for a working-set row"; return -1; }
            ids[first_new + t] = id;
            slot[first_new + t] = s;
        }
        std::vector<char> taken(slots, 0);
        for (int t = 0; t < ws; ++t) {
            if (slot[t] < 0 || slot[t] >= slots || c.slot_of[ids[t]] != slot[t] || c.id_of[slot[t]] != ids[t]) {
                what = "a working-set row lost its slot";
                return -1;
            }
            if (taken[slot[t]] && n_ids >= 2 * ws) { what = "two working-set rows share a slot"; return -1; }
            taken[slot[t]] = 1;
            if (c.pins[slot[t]] < 1) { what = "a working-set row is not pinned"; return -1; }
        }
        int listed = 0;
        for (int s2 = c.head; s2 >= 0; s2 = c.next[s2]) {
            if (c.pins[s2] != 0) { what = "a pinned row is on the eviction list"; return -1; }
            if (++listed > slots) { what = "the eviction list has a cycle"; return -1; }
        }
        int pinned = 0;
        for (int s2 = 0; s2 < c.used; ++s2) pinned += c.pins[s2] > 0;
        if (listed + pinned != c.used) { what = "rows neither pinned nor listed"; return -1; }
    }
    return hits;
}

}  // namespace

extern "C" {

const char *tsvm_selftest_last_error(void) { return g_selftest_error.c_str(); }

// Needs a device.  0 on success, -1 with a message otherwise.
int tsvm_selftest_device_buffer(void) {
    SELFTEST_GUARD({
        using tsvm::DeviceBuffer;
        auto expect = [](bool ok, const char *what) { if (!ok) throw std::runtime_error(std::string("DeviceBuffer: ") + what); };
        const size_t base = tsvm::device_bytes_in_use();
        {
            DeviceBuffer<char> a(100);
            expect(a.data() != nullptr && a.size() == 100, "allocation");
            expect(tsvm::device_bytes_in_use() == base + 100, "one allocation counted");
            DeviceBuffer<char> b;                       // nothing allocated, nothing counted
            expect(b.data() == nullptr && tsvm::device_bytes_in_use() == base + 100, "empty buffer");
            b.resize(100);
            expect(tsvm::device_bytes_in_use() == base + 200, "second allocation counted");
            {
                DeviceBuffer<char> t(100);
                expect(tsvm::device_bytes_in_use() == base + 300, "third allocation counted");
                DeviceBuffer<char> moved(std::move(t));   // ownership moves, the bytes are counted once
                expect(t.data() == nullptr && t.size() == 0 && moved.size() == 100, "move");
                expect(tsvm::device_bytes_in_use() == base + 300, "move does not count twice");
            }
            expect(tsvm::device_bytes_in_use() == base + 200, "destruction releases");
            DeviceBuffer<int> d(100);
            expect(d.size() == 100 && tsvm::device_bytes_in_use() == base + 200 + 100 * sizeof(int), "typed size");
            d.resize(20);                               // a resize starts over, as SyncArray::resize does
            expect(d.size() == 20 && tsvm::device_bytes_in_use() == base + 200 + 20 * sizeof(int), "resize");
            std::vector<int> host(10);
            for (int i = 0; i < 10; ++i) host[i] = i;
            d.upload(host.data(), 10, 5);               // interior offsets are accepted
            for (int i = 0; i < 10; ++i) host[i] = -1;
            d.download(host.data(), 10, 5);
            for (int i = 0; i < 10; ++i) expect(host[i] == i, "round trip");
            d.zero();
            const std::vector<int> z = d.to_host();
            for (int v : z) expect(v == 0, "zero fill");
        }
        expect(tsvm::device_bytes_in_use() == base, "everything released");
    })
}

// No device needed.  Returns the number of hits, or -1 (tsvm_selftest_last_error says what broke).
long long tsvm_selftest_row_cache(int n_ids, int slots, int ws, int iterations) {
    std::string what;
    const long long hits = row_cache_selftest(n_ids, slots, ws, iterations, what);
    if (hits < 0) g_selftest_error = "row cache: " + what;
    return hits;
}

// No device needed: waits on a word that nobody writes, with a stream that reports "still running", and returns 0 when
// the wait gave up with its time-out error after timeout_ms (within a second of it), -1 otherwise.  never_written != 0
// makes the stream report "drained" instead: the wait must then fail with its "finished without reporting" error at once.
int tsvm_selftest_solver_wait(int timeout_ms, int never_written) {
    static volatile uint64_t word;
    word = 0x7ff8dead00000001ull;
    const auto t0 = std::chrono::steady_clock::now();
    try {
        if (never_written)
            tsvm::wait_while_pending(&word, word, timeout_ms, [](void *) { return hipSuccess; }, nullptr);
        else
            tsvm::wait_while_pending(&word, word, timeout_ms, [](void *) { return hipErrorNotReady; }, nullptr);
    } catch (const std::runtime_error &e) {
        const double ms = std::chrono::duration<double, std::milli>(std::chrono::steady_clock::now() - t0).count();
        g_selftest_error = e.what();
        const bool timed_out = g_selftest_error.find("TSVM_SOLVER_TIMEOUT_MS") != std::string::npos;
        if (never_written) return !timed_out && ms < 1000.0 ? 0 : -1;
        return timed_out && ms >= timeout_ms && ms < timeout_ms + 1000.0 ? 0 : -1;
    }
    g_selftest_error = "the wait returned although the word never changed";
    return -1;
}

}  // extern "C"
