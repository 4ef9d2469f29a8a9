// fk_staging_ring.h — the slot state machine behind fkrt_params_upload / fkrt_params_release, free of any GPU header:
// the runtime layer drives it with the HIP runtime, its host-only check (tests/cpp/staging_ring_check.cpp) with stand-ins.
//
// A slot is a pinned host buffer, a device buffer and an event.  Its life:
//
//   FREE --upload--> LEASED --release (event recorded behind the kernel)--> DRAINING --event completed--> FREE
//
// A slot is handed out only when it is FREE, or DRAINING with its event completed; an upload that finds neither takes the
// DRAINING slot that was released first and waits for its event WITHOUT holding the ring's mutex (the slot is marked
// RECLAIMING meanwhile, so that no other upload takes it); an upload that finds every slot LEASED waits for a release, at
// most `wait_ms`, and then fails with RING_FULL instead of overwriting a block whose kernel has not run.
#ifndef FK_STAGING_RING_H
#define FK_STAGING_RING_H

#include <chrono>
#include <condition_variable>
#include <cstddef>
#include <cstring>
#include <mutex>

namespace fkrt {

// What the ring needs from a GPU runtime.  Every function returns 0 for success, anything else is passed to the caller.
struct RingBackend {
    int (*current_device)(int* device);
    int (*alloc_slot)(void** host, void** device, void** event, size_t bytes);
    void (*free_slot)(void* host, void* device, void* event);
    int (*copy_to_device)(void* device, const void* host, size_t bytes, void* stream); // stream-ordered, from pinned memory
    int (*event_record)(void* event, void* stream);
    int (*event_sync)(void* event);            // blocks until the event has completed
    int (*event_done)(void* event, bool* done); // does not block
};

class StagingRing {
public:
    static constexpr int SLOTS = 8;
    static constexpr size_t MIN_BYTES = 64 * 1024;
    static constexpr int RING_FULL = -1001;      // every slot stayed leased for wait_ms
    static constexpr int NOT_A_LEASED_SLOT = -1002;

    explicit StagingRing(const RingBackend& backend, unsigned wait_ms = 2000) : backend_(backend), wait_ms_(wait_ms) {}
    StagingRing(const StagingRing&) = delete;
    StagingRing& operator=(const StagingRing&) = delete;

    // Copies `bytes` from host_src into a slot (host_src may be released when the call returns), enqueues the slot's copy to
    // the device on `stream` and leases the slot to the caller until release().
    int upload(void** device_out, const void* host_src, size_t bytes, void* stream) {
        int current = 0;
        if (const int e = backend_.current_device(&current)) return e;
        int slot = -1;
        if (const int e = lease(slot)) return e;
        Slot& s = slots_[slot]; // ours alone from here on: LEASED
        int e = 0;
        if (s.bytes < bytes || s.owner != current || s.event == nullptr) {
            if (s.event != nullptr || s.host != nullptr || s.device != nullptr) backend_.free_slot(s.host, s.device, s.event);
            s.host = s.device = s.event = nullptr;
            s.bytes = 0;
            const size_t wanted = bytes > MIN_BYTES ? bytes : MIN_BYTES;
            e = backend_.alloc_slot(&s.host, &s.device, &s.event, wanted);
            if (e == 0) {
                s.bytes = wanted;
                s.owner = current;
            }
        }
        if (e == 0) {
            std::memcpy(s.host, host_src, bytes);
            e = backend_.copy_to_device(s.device, s.host, bytes, stream);
        }
        if (e != 0) { // hand the slot back
            std::lock_guard<std::mutex> hold(lock_);
            s.state = FREE;
            changed_.notify_all();
            return e;
        }
        *device_out = s.device;
        return 0;
    }

    // After the kernel that reads the block has been enqueued on `stream`: the slot may be used again once that kernel is done.
    int release(void* device_params, void* stream) {
        std::lock_guard<std::mutex> hold(lock_);
        for (Slot& s : slots_) {
            if (s.state == LEASED && s.device == device_params && device_params != nullptr) {
                const int e = backend_.event_record(s.event, stream);
                // (a record that fails leaves nothing to wait for: the slot is free for the next upload either way)
                s.state = e == 0 ? DRAINING : FREE;
                s.released = ++releases_;
                changed_.notify_all();
                return e;
            }
        }
        return NOT_A_LEASED_SLOT;
    }

    int leased() {
        std::lock_guard<std::mutex> hold(lock_);
        int n = 0;
        for (const Slot& s : slots_) n += s.state == LEASED ? 1 : 0;
        return n;
    }

private:
    enum State { FREE, LEASED, DRAINING, RECLAIMING };
    struct Slot {
        void* host = nullptr;
        void* device = nullptr;
        void* event = nullptr;
        size_t bytes = 0;
        int owner = 0; // device of the slot's buffers
        State state = FREE;
        unsigned long long released = 0; // order of the releases
    };

    int lease(int& out) {
        std::unique_lock<std::mutex> hold(lock_);
        // (the system clock: its timed wait is the one that thread sanitizers of every vintage understand)
        const auto deadline = std::chrono::system_clock::now() + std::chrono::milliseconds(wait_ms_);
        for (;;) {
            int oldest = -1;
            for (int i = 0; i < SLOTS; ++i) {
                Slot& s = slots_[i];
                if (s.state == FREE) {
                    s.state = LEASED;
                    out = i;
                    return 0;
                }
                if (s.state == DRAINING) {
                    bool done = false;
                    if (backend_.event_done(s.event, &done) == 0 && done) {
                        s.state = LEASED;
                        out = i;
                        return 0;
                    }
                    if (oldest < 0 || s.released < slots_[oldest].released) oldest = i;
                }
            }
            if (oldest >= 0) { // wait for the kernel that reads it, with the ring open to everybody else
                Slot& s = slots_[oldest];
                s.state = RECLAIMING;
                void* const event = s.event;
                hold.unlock();
                const int e = backend_.event_sync(event);
                hold.lock();
                if (e != 0) {
                    s.state = DRAINING;
                    changed_.notify_all();
                    return e;
                }
                s.state = LEASED;
                out = oldest;
                return 0;
            }
            // every slot is between its upload and its release (or being reclaimed by another upload)
            if (changed_.wait_until(hold, deadline) == std::cv_status::timeout) return RING_FULL;
        }
    }

    RingBackend backend_;
    unsigned wait_ms_;
    std::mutex lock_;
    std::condition_variable changed_;
    Slot slots_[SLOTS];
    unsigned long long releases_ = 0;
};

} // namespace fkrt
#endif
