// Model test of the hand-over protocol of the one-launch transforms (ckks_llm_amd/csrc/pair_protocol.hpp), on the host: one
// thread per workgroup runs the very decision functions the kernels compile, with the tile passes replaced by bookkeeping that
// catches a first-pass tile run twice or not at all, a second-pass tile that starts before the limb's first pass is complete,
// and a second-pass tile run twice or not at all.  Scenarios: any number of workgroups resident at once (down to one), any
// start order, late starters, spin limits from zero upwards (every wait runs out) to generous, the form without taking over
// (the key switch's last launch), many launches in a row on the same words (replays), and two launches with words of their own
// that compete for the same residency slots.  Built by tests/cpp/Makefile with hipcc in host-only mode.
#include <algorithm>
#include <atomic>
#include <chrono>
#include <condition_variable>
#include <cstdio>
#include <cstdlib>
#include <mutex>
#include <random>
#include <thread>
#include <vector>

#include "../../ckks_llm_amd/csrc/pair_protocol.hpp"

using namespace ckks;

namespace {

struct Slots {                      // residency: at most `free` workgroups run at a time
    std::mutex m;
    std::condition_variable cv;
    int free;
    explicit Slots(int n) : free(n) {}
    void acquire() { std::unique_lock<std::mutex> l(m); cv.wait(l, [&] { return free > 0; }); free--; }
    void release() { { std::lock_guard<std::mutex> l(m); free++; } cv.notify_one(); }
};

struct Limb {
    alignas(128) unsigned words[pair::WORDS] = {};
    std::atomic<int> p1[16], p2[16];
    std::atomic<int> errors{0};
    Limb() { for (int i = 0; i < 16; i++) { p1[i] = 0; p2[i] = 0; } }
    void begin_launch() { for (int i = 0; i < 16; i++) { p1[i] = 0; p2[i] = 0; } }
};

void fail(Limb& L, const char* what, unsigned tile) {
    if (L.errors++ == 0) fprintf(stderr, "protocol violation: %s (tile %u)\n", what, tile);
}
void pass1(Limb& L, unsigned t, int work_us) {
    if (L.p1[t].exchange(1) != 0) fail(L, "first-pass tile run twice", t);
    if (work_us) std::this_thread::sleep_for(std::chrono::microseconds(work_us));
    L.p1[t] = 2;                                             // complete (its stores acknowledged)
}
void pass2(Limb& L, unsigned t) {
    for (int i = 0; i < 16; i++)
        if (L.p1[i] != 2) { fail(L, "second pass started before the first pass was complete", t); break; }
    if (L.p2[t].fetch_add(1) != 0) fail(L, "second-pass tile run twice", t);
}

// what pair_run does on the device, lane 0's part and the workgroup's part in one thread
void workgroup(Limb& L, unsigned tile, bool stealing, unsigned spin_steal, unsigned spin_max, int work_us, bool broken) {
    unsigned* w = L.words;
    unsigned act = pair::claim_own(w, tile, stealing), mine = 0;
    if (broken) act = tile;                                  // a workgroup that ignores that its tile was taken: the model must object
    while (act < pair::TILES) {
        pass1(L, act, work_us);
        mine |= 1u << act;
        act = pair::tile_done_then_decide(w, stealing, spin_steal, spin_max);
    }
    if (act == pair::DEFER) pair::defer(w, mine);
    const unsigned last = pair::leave(w);                    // counted out ahead of the own second pass, as on the device
    unsigned todo = act == pair::GO ? mine : 0u;
    while (todo) { const unsigned t = (unsigned)__builtin_ctz(todo); todo &= todo - 1u; pass2(L, t); }
    if (!(last & 0x80000000u)) return;
    unsigned rest = last & pair::ALL;
    const unsigned finished = rest;
    while (rest) { const unsigned t = (unsigned)__builtin_ctz(rest); rest &= rest - 1u; pass2(L, t); }
    pair::reset(w, finished);
}

struct Scenario { int resident; int order; bool stealing; unsigned spin_steal, spin_max; int work_us; int late_us; bool broken = false; };

// one launch over `limbs` (each with words of its own); returns the number of violations
int launch(std::vector<Limb*>& limbs, Slots& slots, const Scenario& sc, std::mt19937& rng) {
    struct Job { Limb* L; unsigned tile; };
    std::vector<Job> jobs;
    for (Limb* L : limbs) { L->begin_launch(); for (unsigned t = 0; t < 16; t++) jobs.push_back({L, t}); }
    if (sc.order == 1) std::reverse(jobs.begin(), jobs.end());
    if (sc.order == 2) std::shuffle(jobs.begin(), jobs.end(), rng);
    std::vector<std::thread> th;
    for (const Job& j : jobs) {
        th.emplace_back([&, j] {
            slots.acquire();
            workgroup(*j.L, j.tile, sc.stealing, sc.spin_steal, sc.spin_max, sc.work_us, sc.broken);
            slots.release();
        });
        if (sc.late_us) std::this_thread::sleep_for(std::chrono::microseconds(rng() % (unsigned)sc.late_us));
    }
    for (auto& t : th) t.join();
    int bad = 0;
    for (Limb* L : limbs) {
        for (int i = 0; i < 16; i++) {
            if (L->p1[i] != 2) { fail(*L, "first-pass tile never run", (unsigned)i); }
            if (L->p2[i] != 1) { fail(*L, "second-pass tile not run exactly once", (unsigned)i); }
        }
        for (int k : {pair::CLAIM, pair::DONE, pair::LEFT, pair::TODO})
            if (L->words[k] != 0) fail(*L, "a protocol word is not zero after the launch", (unsigned)k);
        bad += L->errors;
    }
    return bad;
}

}  // namespace

int main(int argc, char** argv) {
    const int rounds = argc > 1 ? atoi(argv[1]) : 3;
    std::mt19937 rng(12345);
    int bad = 0, launches = 0;
    unsigned long deferred = 0, stolen = 0;
    for (int resident : {1, 2, 3, 5, 16, 40})
        for (int order : {0, 1, 2})
            for (int steal : {1, 0})
                for (auto spins : {std::pair<unsigned, unsigned>{0u, 0u}, {0u, 50u}, {4u, 2000u}, {32u, 400000u}})
                    for (int work_us : {0, 30}) {
                        // without taking over and with unbounded patience a workgroup would wait for ones that cannot start: the form
                        // without taking over always runs with every workgroup resident on the device
                        if (!steal && resident < 16 && spins.second > 2000u) continue;
                        Scenario sc{resident, order, steal != 0, spins.first, spins.second, work_us, work_us ? 20 : 0};
                        Slots slots(resident);
                        Limb a, b;                                   // two limbs: two sets of words, one pool of slots
                        std::vector<Limb*> limbs{&a, &b};
                        for (int r = 0; r < rounds; r++) {           // launches in a row on the same words: replays
                            bad += launch(limbs, slots, sc, rng);
                            launches++;
                        }
                        deferred += a.words[pair::DEFERRED_TOTAL] + b.words[pair::DEFERRED_TOTAL];
                        stolen += a.words[pair::STOLEN_TOTAL] + b.words[pair::STOLEN_TOTAL];
                    }
    {
        // the model's own check: a broken workgroup (it runs its tile although another has taken it) must be caught
        Scenario sc{2, 0, true, 0u, 50u, 30, 20, true};
        Slots slots(2);
        Limb a;
        std::vector<Limb*> limbs{&a};
        FILE* quiet = freopen("/dev/null", "w", stderr);
        (void)quiet;
        const int caught = launch(limbs, slots, sc, rng);
        if (!freopen("/dev/stderr", "w", stderr)) return 2;
        if (caught == 0) { printf("the model did not notice a workgroup that ignores its claim\n"); return 1; }
    }
    printf("%d launches, %d violations, %lu tiles taken over, %lu second-pass tiles left to the last workgroup out\n", launches, bad, stolen, deferred);
    if (stolen == 0 || deferred == 0) { fprintf(stderr, "the scenarios never took a tile over or never deferred one: they prove nothing\n"); return 1; }
    return bad ? 1 : 0;
}
