// Host-only check of the workspace rules (aether-ml_amd/csrc/ws_ledger.h) with a fake
// allocator: prints one "ok <name>" line per rule and exits non-zero at the first failure.
#include <stdio.h>
#include <stdlib.h>
#include <set>

#include "ws_ledger.h"

static std::set<void*> g_alive;
static int g_quiesced = 0;
static bool g_fail_alloc = false;

static void* fake_alloc(int64_t bytes) {
    if (g_fail_alloc) return nullptr;
    (void)bytes;
    static uintptr_t next = 0x1000;                     // addresses are never reused, so identity tests are exact
    void* p = reinterpret_cast<void*>(next);
    next += 0x1000;
    g_alive.insert(p);
    return p;
}
static void fake_release(void* p) {
    if (!g_alive.count(p)) { printf("FAIL release of a pointer that is not alive\n"); exit(1); }
    g_alive.erase(p);
}
static void quiesce() { ++g_quiesced; }

#define CHECK(cond, name)                                                     \
    do {                                                                      \
        if (!(cond)) { printf("FAIL %s: %s\n", name, #cond); return 1; }      \
    } while (0)

int main() {
    using aeth::WorkspaceLedger;
    WorkspaceLedger w;
    void* p = nullptr;

    // 1. first request allocates with slack, a smaller one reuses the buffer
    CHECK(w.acquire(1000, &p, fake_alloc, fake_release, quiesce) == WorkspaceLedger::kOk, "first");
    void* first = p;
    CHECK(w.cur_bytes == (1 << 20) && g_alive.size() == 1 && w.generation == 1, "first");
    CHECK(w.acquire(500, &p, fake_alloc, fake_release, quiesce) == WorkspaceLedger::kOk && p == first, "reuse");
    CHECK(w.generation == 1, "reuse");
    printf("ok reuse\n");

    // 2. no recording alive: growth frees the old buffer after the device has gone idle
    CHECK(w.acquire(4 << 20, &p, fake_alloc, fake_release, quiesce) == WorkspaceLedger::kOk, "grow");
    CHECK(p != nullptr && !g_alive.count(first) && g_alive.size() == 1 && g_quiesced == 1, "grow");
    CHECK(w.generation == 2 && w.cur_bytes == (5 << 20), "grow");
    printf("ok grow_frees_old\n");

    // 3. while a recording is open the workspace must not move
    void* second = p;
    w.recording_open = true;
    CHECK(w.acquire(64 << 20, &p, fake_alloc, fake_release, quiesce) == WorkspaceLedger::kWhileRecording, "open");
    CHECK(w.cur == second && g_alive.size() == 1, "open");
    CHECK(w.acquire(1 << 20, &p, fake_alloc, fake_release, quiesce) == WorkspaceLedger::kOk && p == second, "open");
    w.recording_open = false;
    w.recording_ended_ok();
    printf("ok no_growth_while_recording\n");

    // 4. a live recording keeps the buffer it was made with alive across growth
    CHECK(w.acquire(64 << 20, &p, fake_alloc, fake_release, quiesce) == WorkspaceLedger::kOk, "retire");
    CHECK(p != second && g_alive.count(second) && g_alive.size() == 2 && w.retired.size() == 1, "retire");
    CHECK(g_quiesced == 1, "retire");                                  // nothing was freed, nothing to wait for
    void* third = p;
    w.recording_ended_ok();                                            // a second recording, made with `third`
    CHECK(w.acquire(256 << 20, &p, fake_alloc, fake_release, quiesce) == WorkspaceLedger::kOk, "retire2");
    CHECK(g_alive.count(second) && g_alive.count(third) && g_alive.size() == 3, "retire2");
    printf("ok live_recordings_keep_their_workspace\n");

    // 5. retired buffers go when the LAST recording is destroyed
    w.recording_destroyed(fake_release);
    CHECK(g_alive.size() == 3 && w.live_recordings == 1, "destroy1");
    w.recording_destroyed(fake_release);
    CHECK(g_alive.size() == 1 && g_alive.count(p) && w.retired.empty() && w.live_recordings == 0, "destroy2");
    printf("ok retired_freed_with_last_recording\n");

    // 6. a failed allocation leaves no dangling current pointer
    g_fail_alloc = true;
    void* q = nullptr;
    CHECK(w.acquire((int64_t)1 << 40, &q, fake_alloc, fake_release, quiesce) == WorkspaceLedger::kAllocFailed, "oom");
    CHECK(w.cur == nullptr && w.cur_bytes == 0 && g_alive.empty(), "oom");
    g_fail_alloc = false;
    CHECK(w.acquire(100, &q, fake_alloc, fake_release, quiesce) == WorkspaceLedger::kOk && q != nullptr, "after oom");
    printf("ok alloc_failure\n");

    // 7. reset frees everything
    w.recording_ended_ok();
    CHECK(w.acquire(8 << 20, &q, fake_alloc, fake_release, quiesce) == WorkspaceLedger::kOk, "pre-reset");
    CHECK(g_alive.size() == 2, "pre-reset");
    w.reset(fake_release);
    CHECK(g_alive.empty() && w.cur == nullptr && w.live_recordings == 0 && w.retired.empty(), "reset");
    printf("ok reset\n");
    return 0;
}
