// Which (query head, tile group) a workgroup of the prompt-attention kernel takes.  Plain C++ so that the
// arithmetic can be replayed on the host for every head count and group count before a kernel uses it.
#pragma once

#if defined(__HIPCC__)
#define LEONE_HD __host__ __device__
#else
#define LEONE_HD
#endif

namespace leone {

constexpr int kPrefillDies = 8;

struct PrefillWork {
    int head;
    int group;
};

// Workgroups go round the chip's eight dies in turn (block b runs on die b % 8), each die has a cache of
// its own, and a compute unit holds two workgroups.  When the heads divide evenly over the dies and the
// groups pair up, a die gets q_heads / 8 neighbouring heads (few key/value heads, whose keys its cache
// then keeps) with all their groups, and the second half of a die's workgroups takes the groups in falling
// order, so that a compute unit tends to hold a group that sees few keys beside one that sees many.
// Otherwise blocks are numbered head by head.  Either way every (head, group) pair with head < q_heads and
// group < n_groups belongs to exactly one block of the q_heads * n_groups that are launched.
LEONE_HD inline bool prefill_die_order(int q_heads, int n_groups) {
    return q_heads % kPrefillDies == 0 && n_groups % 2 == 0;
}

LEONE_HD inline PrefillWork prefill_work(int block, int q_heads, int n_groups) {
    PrefillWork w;
    if (prefill_die_order(q_heads, n_groups)) {
        const int heads_here = q_heads / kPrefillDies;            // at least 1
        const int half = heads_here * (n_groups / 2);             // workgroups of one half of a die
        const int spot = block / kPrefillDies;                    // 0 .. 2 * half - 1
        const int late = spot / half, r = spot % half;
        const int pair = r / heads_here;
        w.head = (block % kPrefillDies) * heads_here + r % heads_here;
        w.group = late ? n_groups - 1 - pair : pair;
    } else {
        w.head = block / n_groups;
        w.group = block % n_groups;
    }
    return w;
}

}  // namespace leone
