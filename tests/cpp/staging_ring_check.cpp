// Host-only check of the slot state machine behind fkrt_params_upload / fkrt_params_release
// (fusedkernellibrary_amd/csrc/fk_staging_ring.h), with stand-ins for the GPU runtime: "device" buffers are host memory, an
// event completes when the test says so.  Built with g++ -pthread, no GPU and no GPU header involved.
#include <atomic>
#include <cstdio>
#include <cstdlib>
#include <thread>
#include <vector>

#include "fk_staging_ring.h"

namespace {
struct FakeEvent {
    std::atomic<bool> recorded{ false };
    std::atomic<bool> done{ true };
};
std::atomic<int> syncs{ 0 }, allocations{ 0 };
std::atomic<bool> auto_complete{ true }; // a recorded event is complete at once
std::atomic<void (*)()> during_sync{ nullptr };

int current_device(int* d) { *d = 0; return 0; }
int alloc_slot(void** host, void** device, void** event, size_t bytes) {
    *host = std::malloc(bytes);
    *device = std::malloc(bytes);
    *event = new FakeEvent();
    ++allocations;
    return 0;
}
void free_slot(void* host, void* device, void* event) {
    std::free(host);
    std::free(device);
    delete static_cast<FakeEvent*>(event);
}
int copy_to_device(void* device, const void* host, size_t bytes, void*) {
    std::memcpy(device, host, bytes); // "stream order" is program order here
    return 0;
}
int event_record(void* event, void*) {
    FakeEvent* e = static_cast<FakeEvent*>(event);
    e->recorded = true;
    e->done = auto_complete.load();
    return 0;
}
int event_sync(void* event) {
    ++syncs;
    if (void (*hook)() = during_sync.load()) hook();
    FakeEvent* e = static_cast<FakeEvent*>(event);
    while (!e->done.load()) std::this_thread::yield();
    return 0;
}
int event_done(void* event, bool* done) {
    *done = static_cast<FakeEvent*>(event)->done.load();
    return 0;
}
const fkrt::RingBackend BACKEND{ current_device, alloc_slot, free_slot, copy_to_device, event_record, event_sync, event_done };

int failures = 0;
#define CHECK(cond)                                                          \
    do {                                                                     \
        if (!(cond)) {                                                       \
            std::printf("FAILED line %d: %s\n", __LINE__, #cond);            \
            ++failures;                                                      \
        }                                                                    \
    } while (0)

// 1. eight blocks leased: a ninth upload fails after its wait instead of taking a slot; every block keeps its own buffer
void nine_uploads_without_a_release() {
    fkrt::StagingRing& ring = *new fkrt::StagingRing(BACKEND, 30); // (rings are left alone at the end: their slots' buffers live as long as the process, as in the library)
    void* dev[9] = {};
    for (int i = 0; i < 8; ++i) {
        const int token = 1000 + i;
        CHECK(ring.upload(&dev[i], &token, sizeof(token), nullptr) == 0);
    }
    for (int i = 0; i < 8; ++i) {
        for (int j = 0; j < i; ++j) CHECK(dev[i] != dev[j]);
        CHECK(*static_cast<int*>(dev[i]) == 1000 + i);
    }
    CHECK(ring.leased() == 8);
    const int token = 7;
    CHECK(ring.upload(&dev[8], &token, sizeof(token), nullptr) == fkrt::StagingRing::RING_FULL);
    for (int i = 0; i < 8; ++i) CHECK(*static_cast<int*>(dev[i]) == 1000 + i); // nothing was overwritten
    // a release makes room, and the slot that comes back is the released one
    CHECK(ring.release(dev[3], nullptr) == 0);
    CHECK(ring.upload(&dev[8], &token, sizeof(token), nullptr) == 0);
    CHECK(dev[8] == dev[3] && *static_cast<int*>(dev[8]) == 7);
    CHECK(ring.release(dev[3], nullptr) == 0);
    CHECK(ring.release(dev[3], nullptr) == fkrt::StagingRing::NOT_A_LEASED_SLOT); // released twice
    int other = 0;
    CHECK(ring.release(&other, nullptr) == fkrt::StagingRing::NOT_A_LEASED_SLOT);
}

// 2. a released slot whose kernel has not finished is not handed out before its event completes, the wait happens with the
//    ring open (another thread's release goes through while the upload waits), and the first released slot is the one taken
fkrt::StagingRing* open_ring = nullptr;
void* to_release = nullptr;
std::atomic<int> released_during_sync{ -1 };
std::atomic<FakeEvent*> last_recorded{ nullptr };
int remembering_record(void* event, void* stream) {
    last_recorded = static_cast<FakeEvent*>(event);
    return event_record(event, stream);
}
void release_another_slot_then_complete() {
    FakeEvent* const awaited = last_recorded.load();                // the event the upload is waiting for
    released_during_sync = open_ring->release(to_release, nullptr); // would deadlock if the upload held the ring's mutex
    awaited->done = true;
}
void reclaim_waits_outside_the_lock() {
    fkrt::RingBackend remembering = BACKEND;
    remembering.event_record = remembering_record;
    fkrt::StagingRing& ring = *new fkrt::StagingRing(remembering, 1000);
    void* dev[8] = {};
    int token = 1;
    for (int i = 0; i < 8; ++i) CHECK(ring.upload(&dev[i], &token, sizeof(token), nullptr) == 0);
    auto_complete = false;                     // events stay pending until completed by hand
    CHECK(ring.release(dev[5], nullptr) == 0); // slot 5 drains, its kernel "has not finished"
    open_ring = &ring;
    to_release = dev[2];
    during_sync = release_another_slot_then_complete;
    const int before = syncs.load();
    void* got = nullptr;
    token = 99;
    CHECK(ring.upload(&got, &token, sizeof(token), nullptr) == 0);
    during_sync = nullptr;
    CHECK(syncs.load() == before + 1);       // it waited for the event
    CHECK(released_during_sync.load() == 0); // and the other release went through meanwhile
    CHECK(got == dev[5]);                    // the slot released first
    CHECK(*static_cast<int*>(got) == 99);
    auto_complete = true;
}

// 3. many host threads, more than slots: every block reaches its "kernel" intact
void threads_never_see_each_others_blocks() {
    fkrt::StagingRing& ring = *new fkrt::StagingRing(BACKEND, 5000);
    std::atomic<int> bad{ 0 };
    std::vector<std::thread> pool;
    for (int t = 0; t < 12; ++t) {
        pool.emplace_back([&, t] {
            for (int i = 0; i < 2000; ++i) {
                int block[64];
                for (int k = 0; k < 64; ++k) block[k] = t * 100000 + i;
                void* dev = nullptr;
                if (ring.upload(&dev, block, sizeof(block), nullptr) != 0) {
                    ++bad;
                    continue;
                }
                std::this_thread::yield(); // the "launch" happens some time after the upload
                for (int k = 0; k < 64; ++k) bad += static_cast<int*>(dev)[k] != t * 100000 + i ? 1 : 0;
                if (ring.release(dev, nullptr) != 0) ++bad;
            }
        });
    }
    for (std::thread& th : pool) th.join();
    CHECK(bad.load() == 0);
    CHECK(ring.leased() == 0);
}

// 4. a block larger than a slot makes the slot grow; nothing is allocated per upload otherwise
void slots_grow_and_are_reused() {
    fkrt::StagingRing& ring = *new fkrt::StagingRing(BACKEND, 100);
    const int before = allocations.load();
    std::vector<char> big(200 * 1024, 'x');
    void* dev = nullptr;
    for (int i = 0; i < 100; ++i) {
        CHECK(ring.upload(&dev, big.data(), big.size(), nullptr) == 0);
        CHECK(static_cast<char*>(dev)[big.size() - 1] == 'x');
        CHECK(ring.release(dev, nullptr) == 0);
    }
    CHECK(allocations.load() - before <= 8);
}
} // namespace

int main() {
    nine_uploads_without_a_release();
    reclaim_waits_outside_the_lock();
    threads_never_see_each_others_blocks();
    slots_grow_and_are_reused();
    if (failures == 0) std::printf("staging ring: ok\n");
    return failures == 0 ? 0 : 1;
}
