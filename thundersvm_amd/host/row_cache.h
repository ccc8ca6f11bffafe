// The kernel-row cache's bookkeeping on the host (which instance has which slot of the row arena, and which row
// goes when a slot is needed).
#pragma once
#include <vector>

namespace tsvm {

// Kernel-row cache bookkeeping (host side).  Rows of the kernel matrix live in slots of one HBM pool;
// slot_of maps an instance id to its slot, an intrusive doubly linked list keeps the slots that may be evicted in
// eviction order (tail first).  The device only ever sees slot numbers.  The reference keeps no rows
// beyond the previous working set's second half (csmosolver.cpp:33-42,65-77); cached rows are the
// rows get_rows would recompute, so the cache cannot change a result.
//
// Which row goes.  A row is pinned (out of the list) while it is in the working set, two outer iterations as a rule.
// When it leaves, a row that was found in the cache when it entered goes to the front of the list; a row that had to
// be computed goes to the tail, where the next misses take its slot first (all but every 64th such row, which goes
// to the front, so that the cache's content can drift).  Plain least-recently-used order loses against SMO's access
// pattern whenever the rows that keep coming back outnumber the slots: the selection works through them in turn,
// and every row is evicted shortly before it is wanted again (a 426,315-instance class pair with 35,000 slots: 1 %
// hits; with this order 26 %, and the best any order could do, knowing the future, is 39 %).
struct RowCache {
    int cap = 0, used = 0, head = -1, tail = -1;
    long long released_misses = 0;
    std::vector<int> slot_of, id_of, prev, next, pins;
    std::vector<char> was_hit;
    void init(int n, int capacity) {
        cap = capacity;
        slot_of.assign(n, -1);
        id_of.assign(cap, -1);
        prev.assign(cap, -1);
        next.assign(cap, -1);
        pins.assign(cap, 0);
        was_hit.assign(cap, 0);
    }
    void unlink(int s) {
        if (prev[s] >= 0) next[prev[s]] = next[s]; else head = next[s];
        if (next[s] >= 0) prev[next[s]] = prev[s]; else tail = prev[s];
    }
    void push_front(int s) {
        prev[s] = -1;
        next[s] = head;
        if (head >= 0) prev[head] = s;
        head = s;
        if (tail < 0) tail = s;
    }
    void push_back(int s) {
        next[s] = -1;
        prev[s] = tail;
        if (tail >= 0) next[tail] = s;
        tail = s;
        if (head < 0) head = s;
    }
    int lookup(int id) {                 // slot of a cached row, pinned from now on, or -1
        const int s = slot_of[id];
        if (s >= 0) {
            if (pins[s]++ == 0) { unlink(s); was_hit[s] = 1; }
        }
        return s;
    }
    int insert(int id) {                 // slot for a new row, pinned: a free one, else the list's tail (-1: every slot is pinned)
        int s;
        if (used < cap) {
            s = used++;
        } else {
            s = tail;
            if (s < 0) return -1;
            unlink(s);
            slot_of[id_of[s]] = -1;
        }
        id_of[s] = id;
        slot_of[id] = s;
        pins[s] = 1;
        was_hit[s] = 0;
        return s;
    }
    void release(int s) {                // the row has left the working set
        if (--pins[s] > 0) return;
        if (was_hit[s] || (++released_misses & 63) == 0) push_front(s);
        else push_back(s);
    }
};

}  // namespace tsvm
