// Hand-counted waits, checked at compile time.
//
// A wave's vector memory loads complete in the order they were issued, and `s_waitcnt vmcnt(N)` waits until at most N
// of them are outstanding. A kernel that issues its loads by hand therefore waits for a particular load by giving N =
// the number of loads it has issued since. That number follows from the kernel's issue order alone, so it is not
// written down a second time: each such kernel describes its schedule (what it issues, in which order, and where it
// needs which load) to the queue below in a constexpr function, and a static_assert holds every N it uses against the
// count the schedule gives - never larger (the load would still be in flight) and, in the steady state, not smaller
// either (the loop would wait for loads it does not need yet).
#pragma once

namespace mtq {

struct VmQueue {
    static constexpr int CAP = 1024;
    int tag[CAP] = {};
    int n = 0;      // loads issued
    int done = 0;   // loads known to have landed: the oldest `done`
    constexpr void issue(int t, int count) {
        for (int i = 0; i < count && n < CAP; i++) tag[n++] = t;
    }
    // s_waitcnt vmcnt(N): everything but the youngest N has landed
    constexpr void wait(int N) {
        if (n - N > done) done = n - N;
    }
    // true once every load tagged `t` has landed (false if none was issued)
    constexpr bool landed(int t) const {
        for (int i = n - 1; i >= 0; i--)
            if (tag[i] == t) return i < done;
        return false;
    }
    // Loads issued after the last one tagged `t`: the largest N whose wait guarantees that `t` has landed (-1: never issued).
    constexpr int younger_than(int t) const {
        for (int i = n - 1; i >= 0; i--)
            if (tag[i] == t) return n - 1 - i;
        return -1;
    }
};
// A load's tag: what it is (a small integer the kernel chooses) and the iteration (turn) it belongs to.
constexpr int vm_tag(int kind, int turn) { return kind * 4096 + turn; }

}  // namespace mtq
