// CPU model of the in-launch split-K exchange: the protocol of juliavision_amd/csrc/sk_exchange.hpp -- the very
// header the HIP kernel instantiates -- run by one host thread per wave.  Built and run by
// tests/test_sk_exchange_protocol.py (g++ -O1 -pthread); prints one line per scenario and exits nonzero on a failure.
//
// Memory model of the host stand-in: the kernel orders "partials stored" before "flag published" with
// s_waitcnt vmcnt(0) and reads the partials only after the flag; here the flag store is a release and the flag load
// an acquire, which is the same edge.
#include <atomic>
#include <chrono>
#include <cstdio>
#include <cstring>
#include <thread>
#include <vector>

#include "../juliavision_amd/csrc/sk_exchange.hpp"

struct HostMem {
    static unsigned load(const unsigned *p) { return __atomic_load_n(p, __ATOMIC_ACQUIRE); }
    static void store(unsigned *p, unsigned v) { __atomic_store_n(p, v, __ATOMIC_RELEASE); }
    static unsigned fetch_add(unsigned *p, unsigned v) { return __atomic_fetch_add(p, v, __ATOMIC_ACQ_REL); }
    static void pause() { std::this_thread::yield(); }
};
using Ex = sk::Exchange<HostMem>;

constexpr int WAVES = 2, TILES = 2, WORDS = 256;     // words [0, WORDS): flags, [WORDS, 2 WORDS): counters

struct Bank {
    unsigned w[2 * WORDS];
    // what wave `wave` of slice `src` sent to slice `owner` of `tile`
    unsigned part[TILES][4][4][WAVES];
    void zero() { std::memset(this, 0, sizeof(*this)); }
    bool clean() const {
        for (unsigned v : w) if (v) return false;
        return true;
    }
};

struct Sync {                                         // the launch boundary: every wave of a launch has finished
    std::atomic<int> count{0}, gen{0};
    int n;
    explicit Sync(int n_) : n(n_) {}
    void wait() {
        const int g = gen.load();
        if (count.fetch_add(1) + 1 == n) { count.store(0); gen.fetch_add(1); }
        else while (gen.load() == g) std::this_thread::yield();
    }
};

static unsigned payload(int round, int tile, int src, int owner, int wave) {
    return 0x9e3779b9u * (unsigned)(round + 1) + (unsigned)(((tile * 4 + src) * 4 + owner) * WAVES + wave);
}

struct Plan {
    int S, rounds, limit;
    bool same_epoch;          // a replayed graph: every launch carries the epoch it was captured with
    int late_slice = -1;      // this slice publishes only after late_ms (one tile, one wave: tile 0, wave 0)
    int late_ms = 0;
    int odd_xcc_slice = -1;   // this slice reports another XCD
};

struct Outcome { std::atomic<int> stale{0}, timed_out{0}, other_xcd{0}, arrived{0}; };

static void wave_thread(Bank *bank, Sync *sync, const Plan &pl, Outcome *out, int tile, int s, int wave) {
    const int S = pl.S;
    for (int round = 0; round < pl.rounds; round++) {
        const unsigned epoch = sk::epoch_of(pl.same_epoch ? 77u : 0x0ffffffeu + (unsigned)round);      // crosses the 28-bit wrap
        const unsigned xcc = (s == pl.odd_xcc_slice) ? 3u : 2u;
        for (int owner = 0; owner < S; owner++)
            if (owner != s) bank->part[tile][owner][s][wave] = payload(round, tile, s, owner, wave);
        if (s == pl.late_slice && tile == 0 && wave == 0 && round == 0) std::this_thread::sleep_for(std::chrono::milliseconds(pl.late_ms));
        unsigned *mine = bank->w + (tile * S + s) * WAVES + wave;
        Ex::publish(mine, epoch, xcc);
        unsigned *fl[3];
        for (int bi = 0; bi < 3; bi++) {
            const int src = S == 4 ? bi + (bi >= s ? 1 : 0) : 1 - s;
            fl[bi] = bank->w + (tile * S + src) * WAVES + wave;
        }
        const unsigned *const cfl[3] = {fl[0], fl[1], fl[2]};
        const sk::WaitResult wr = Ex::wait(cfl, S == 4 ? 3 : 1, epoch, 2u, pl.limit);
        if (wr == sk::ARRIVED) {
            out->arrived++;
            for (int bi = 0; bi < (S == 4 ? 3 : 1); bi++) {
                const int src = S == 4 ? bi + (bi >= s ? 1 : 0) : 1 - s;
                if (bank->part[tile][s][src][wave] != payload(round, tile, src, s, wave)) out->stale++;
            }
            for (int bi = 0; bi < (S == 4 ? 3 : 1); bi++) Ex::release(fl[bi], fl[bi] + WORDS, S == 4 ? 3 : 1);
        } else if (wr == sk::TIMED_OUT) out->timed_out++;
        else out->other_xcd++;
        sync->wait();                                  // end of the launch
        if (pl.late_slice < 0 && pl.odd_xcc_slice < 0 && tile == 0 && s == 0 && wave == 0 && !bank->clean()) out->stale += 1000;
        sync->wait();
    }
}

static void run(Bank &bank, const Plan &pl, Outcome &out) {
    const int n = TILES * pl.S * WAVES;
    Sync sync(n);
    std::vector<std::thread> th;
    for (int tile = 0; tile < TILES; tile++)
        for (int s = 0; s < pl.S; s++)
            for (int wave = 0; wave < WAVES; wave++) th.emplace_back(wave_thread, &bank, &sync, std::cref(pl), &out, tile, s, wave);
    for (auto &t : th) t.join();
}

int main() {
    int bad = 0;
    static Bank bank;
    // 1. ordinary launches and replays: nobody reads partials that were not written for this launch, every launch
    //    leaves the bank zeroed (checked after each one), with two and with four slices, fresh and repeated epochs.
    for (int S : {2, 4})
        for (bool same : {false, true}) {
            bank.zero();
            Plan pl{S, 400, 1 << 22, same};
            Outcome out;
            run(bank, pl, out);
            const int want = TILES * S * WAVES * pl.rounds;
            const bool ok = out.stale == 0 && out.timed_out == 0 && out.other_xcd == 0 && out.arrived == want && bank.clean();
            std::printf("exchange S=%d %s epochs: arrived %d/%d stale %d -> %s\n", S, same ? "replayed" : "fresh", out.arrived.load(), want,
                        out.stale.load(), ok ? "ok" : "FAIL");
            bad += !ok;
        }
    // 2. a partner that shows up after the bound: its waiters report TIMED_OUT and release nothing, so the late
    //    publication stays in the bank; a replay with the same epoch would take it for an arrival, hence the rule that
    //    the host zeroes the banks after a nonzero status.  After that zeroing the next launch is clean again.
    for (int S : {2, 4}) {
        bank.zero();
        Plan pl{S, 1, 8, true};
        pl.late_slice = 1; pl.late_ms = 100;
        Outcome out;
        run(bank, pl, out);
        const int waiters = S - 1;                    // wave 0 of the other slices of tile 0
        bool ok = out.timed_out >= waiters && out.stale == 0 && !bank.clean();
        const unsigned left = bank.w[(0 * S + 1) * WAVES + 0];
        ok = ok && (left & sk::EPOCH_MASK) == 77u;     // the stale "arrived" a replay would have seen
        bank.zero();                                   // mi_device_status(reset = 1)
        Plan again{S, 50, 1 << 22, true};
        Outcome out2;
        run(bank, again, out2);
        ok = ok && out2.stale == 0 && out2.timed_out == 0 && bank.clean();
        std::printf("late partner S=%d: timed out %d (>= %d), bank dirty until zeroed, clean afterwards -> %s\n", S, out.timed_out.load(), waiters,
                    ok ? "ok" : "FAIL");
        bad += !ok;
    }
    // 3. a partner on another XCD: everyone who waits for it says so; it arrives, but nothing of it is consumed.
    {
        bank.zero();
        Plan pl{2, 1, 1 << 22, true};
        pl.odd_xcc_slice = 0;
        Outcome out;
        run(bank, pl, out);
        const bool ok = out.other_xcd == TILES * WAVES && out.arrived == TILES * WAVES && out.stale == 0;
        std::printf("partner on another XCD: reported by %d waiters -> %s\n", out.other_xcd.load(), ok ? "ok" : "FAIL");
        bad += !ok;
    }
    // 4. epochs: never zero, 28 bits, XCD id in the top four
    {
        bool ok = sk::epoch_of(0) == 1 && sk::epoch_of(1u << 28) == 1 && sk::epoch_of(0x1234567) == 0x1234567 &&
                  sk::word_of(5, 9) == ((9u << 28) | 5u) && (sk::word_of(sk::EPOCH_MASK, 15) & sk::EPOCH_MASK) == sk::EPOCH_MASK;
        std::printf("epoch words -> %s\n", ok ? "ok" : "FAIL");
        bad += !ok;
    }
    return bad ? 1 : 0;
}
