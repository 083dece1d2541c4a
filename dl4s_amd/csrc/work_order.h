// The order in which the workgroups of an attention launch take their work items.  Plain integer arithmetic with no
// dependency on the HIP headers, so that a host compiler can build it too (tests/test_work_order.py checks on the CPU
// that every order hands out every item exactly once).
#pragma once

#if defined(__HIPCC__)
#define DL4S_WORK_ORDER_FN __host__ __device__ __forceinline__
#else
#define DL4S_WORK_ORDER_FN inline
#endif

namespace dl4s_work_order {

DL4S_WORK_ORDER_FN int imin(int a, int b) { return a < b ? a : b; }
DL4S_WORK_ORDER_FN int imax(int a, int b) { return a > b ? a : b; }

// Work order of a launch of `total_blocks` = (batch*head pairs) x `nunits` workgroups.  Workgroups are handed to the 8
// XCDs round-robin by index, so every XCD gets one contiguous run of the pair-major order (workgroups sharing a K/V pair
// share an L2).  Inside the run the order is pair-major by default; with `lpt` the items are handed out by ascending
// unit -- the callers number a pair's units longest first -- so that the hardware dispatcher does
// longest-processing-time scheduling and the launch ends on the cheapest items.  Returns false for padding workgroups.
DL4S_WORK_ORDER_FN bool work_item_at(const int block, const int nunits, const int total_blocks, const int lpt, int &bh, int &unit,
                                     const int snake = 0) {
    const int npairs = total_blocks / nunits;
    int bid = block;
    if (snake > 0) {
        // Launches that fit the chip at once: the dispatcher deals an XCD's workgroups out to its `snake` CUs in turn,
        // so CU c holds the XCD's items c, c + snake, ...  Reversing every second round of the longest-first order pairs
        // long items with short ones on each CU.
        const int x = bid & 7, wl = bid >> 3;
        const int n = (npairs & 7) == 0 ? (npairs >> 3) * nunits : imin((total_blocks + 7) / 8, total_blocks - x * ((total_blocks + 7) / 8));
        const int r = wl / snake;
        if ((r & 1) && wl < n) {
            const int len_r = imin(snake, n - r * snake);
            bid = (r * snake + (len_r - 1 - (wl - r * snake))) * 8 + x;
        }
    }
    if ((npairs & 7) == 0) {
        // A pair count that divides by 8: XCD x takes the pairs x, x + 8, ... instead of a contiguous run.  Work that
        // depends on the batch element (valid lengths, padding masks) then spreads evenly over the XCDs, whose runs
        // would otherwise each hold a few whole batch elements.
        const int x = bid & 7, wl = bid >> 3, cnt = npairs >> 3;
        if (wl >= cnt * nunits) return false;
        if (lpt) {
            unit = wl / cnt;
            bh = x + 8 * (wl % cnt);
        }
        else { bh = x + 8 * (wl / nunits); unit = wl % nunits; }
        return true;
    }
    const int chunk = (total_blocks + 7) / 8;
    const int w = (bid % 8) * chunk + bid / 8;
    if (w >= total_blocks) return false;
    bh = w / nunits;
    unit = w % nunits;
    if (lpt) {
        // The run is w in [a, a + n).  Item `wl` of the run in (unit ascending, w ascending) order: every unit occurs c
        // times, the `rem` units of the cyclic interval starting at s once more.
        const int a = (bid % 8) * chunk;
        const int n = imin(chunk, total_blocks - a);
        const int wl = bid / 8;
        const int c = n / nunits, rem = n % nunits, s = a % nunits;
        const int wrap = s + rem - nunits;   // > 0: the interval wraps around to units [0, wrap)
        auto before = [&](int U) {           // items with unit < U
            const int extra = wrap > 0 ? imin(U, wrap) + imax(0, U - s) : imin(imax(U - s, 0), rem);
            return c * U + extra;
        };
        int lo = 0, hi = nunits - 1;         // largest U with before(U) <= wl
        while (lo < hi) {
            const int mid = (lo + hi + 1) >> 1;
            if (before(mid) <= wl) lo = mid; else hi = mid - 1;
        }
        unit = lo;
        const int j = wl - before(lo);
        bh = (a + (lo - s + nunits) % nunits + j * nunits) / nunits;
    }
    return true;
}

// A launch whose items are each cut into `nsplit` shares: grid x = the items (padded to a multiple of 8), grid y = the shares.
// Workgroups start in the order of bx + gx * by and go to XCD (bx + gx * by) % 8 = bx % 8.  Returns the item index `blk` (to be
// passed to work_item_at) and the share `sp` such that an XCD's sequence runs over its items in their order with the shares of
// an item next to each other - with the longest-first order every share of a long item starts before any share of a
// shorter one, which a share-major walk (all first shares, then all second shares) does not give.
DL4S_WORK_ORDER_FN void split_item_at(const int bx, const int by, const int gx, const int nsplit, int &blk, int &sp) {
    const long long lin = (long long)by * gx + bx;
    const long long wl = lin >> 3;
    sp = (int)(wl % nsplit);
    blk = (int)(wl / nsplit) * 8 + (int)(lin & 7);
}

}  // namespace dl4s_work_order
