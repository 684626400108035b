// Arrival-flag protocol of the in-launch split-K exchange (gemm_w4_kernel, SK instance), written once for the
// device and for a host model: the kernel instantiates it over agent-scope HIP atomics, the CPU test of the protocol
// (tests/sk_exchange_host_test.cpp) over the compiler's __atomic builtins with one thread per wave.  No HIP header is
// needed to read this file.
//
// One word per (tile, K-slice, wave) and one counter behind it.  A wave that has stored its partials for its partners
// and seen them acknowledged PUBLISHES: word = (xcc << 28) | epoch.  A wave then WAITS, for a bounded number of polls,
// until the same wave of every partner has published this launch's epoch, and checks that each partner reported the
// XCD it runs on itself (the partials are exchanged through one XCD's L2 with plain stores and loads; partners on
// different XCDs would read stale lines).  After it has consumed a partner's partials it RELEASES that partner's word:
// the last consumer (the only one with two slices, the third to count itself in with four) writes zero to the word and
// its counter, so that every launch leaves its bank zeroed and a replayed launch -- same epoch -- starts clean.
//
// A wait that expires, or a partner on another XCD, is an error the caller must make visible: the waiter releases
// nothing (the bank stays dirty and has to be zeroed by the host before it is used again) and reports the reason.
#pragma once

namespace sk {

constexpr unsigned EPOCH_BITS = 28, EPOCH_MASK = (1u << EPOCH_BITS) - 1;
enum WaitResult { ARRIVED = 0, TIMED_OUT = 1, OTHER_XCD = 2 };

#if defined(__HIP_DEVICE_COMPILE__) || defined(__HIPCC__)
#define SK_FN __host__ __device__ inline __attribute__((always_inline))
#else
#define SK_FN inline __attribute__((always_inline))
#endif

// Launch counter -> the epoch a launch publishes: 28 bits, never zero (zero is what a clean word holds).
SK_FN unsigned epoch_of(unsigned launch_counter) {
    const unsigned e = launch_counter & EPOCH_MASK;
    return e ? e : 1u;
}

SK_FN unsigned word_of(unsigned epoch, unsigned xcc) { return ((xcc & 15u) << EPOCH_BITS) | (epoch & EPOCH_MASK); }

// Mem supplies: static unsigned load(const unsigned *), void store(unsigned *, unsigned),
// unsigned fetch_add(unsigned *, unsigned), void pause().
template <class Mem>
struct Exchange {
    SK_FN static void publish(unsigned *word, unsigned epoch, unsigned xcc) { Mem::store(word, word_of(epoch, xcc)); }

    // Polls the n (1 or 3) partner words together, at most `limit` rounds.
    SK_FN static WaitResult wait(const unsigned *const (&w)[3], int n, unsigned epoch, unsigned my_xcc, int limit) {
        const unsigned want = epoch & EPOCH_MASK;
        for (int round = 0; round < limit; round++) {
            const unsigned u0 = Mem::load(w[0]);
            const unsigned u1 = n > 1 ? Mem::load(w[1]) : u0;
            const unsigned u2 = n > 2 ? Mem::load(w[2]) : u0;
            if ((u0 & EPOCH_MASK) == want && (u1 & EPOCH_MASK) == want && (u2 & EPOCH_MASK) == want) {
                const unsigned x = (my_xcc & 15u) << EPOCH_BITS;
                return ((u0 & ~EPOCH_MASK) == x && (u1 & ~EPOCH_MASK) == x && (u2 & ~EPOCH_MASK) == x) ? ARRIVED : OTHER_XCD;
            }
            Mem::pause();
        }
        return TIMED_OUT;
    }

    // This wave has consumed what the owner of `word` sent.  consumers = partners that read it (1 or 3).
    SK_FN static void release(unsigned *word, unsigned *counter, int consumers) {
        bool last = true;
        if (consumers > 1) {
            last = Mem::fetch_add(counter, 1u) == (unsigned)(consumers - 1);
            if (last) Mem::store(counter, 0u);
        }
        if (last) Mem::store(word, 0u);
    }
};

}  // namespace sk
