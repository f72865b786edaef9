// Replays the prompt-attention kernel's numbering of workgroups on the host: for every head count and
// group count each (head, group) pair must come up exactly once among the launched blocks.
#include <cstdio>
#include <vector>
#include "prefill_order.h"

int main() {
    for (int q_heads = 1; q_heads <= 64; ++q_heads) {
        for (int n_groups = 1; n_groups <= 32; ++n_groups) {
            std::vector<int> seen(q_heads * n_groups, 0);
            for (int block = 0; block < q_heads * n_groups; ++block) {
                const leone::PrefillWork w = leone::prefill_work(block, q_heads, n_groups);
                if (w.head < 0 || w.head >= q_heads || w.group < 0 || w.group >= n_groups) {
                    std::printf("heads %d groups %d block %d: (%d, %d) out of range\n", q_heads, n_groups, block, w.head, w.group);
                    return 1;
                }
                ++seen[w.head * n_groups + w.group];
            }
            for (int i = 0; i < q_heads * n_groups; ++i) {
                if (seen[i] != 1) {
                    std::printf("heads %d groups %d: pair (%d, %d) taken %d times\n", q_heads, n_groups, i / n_groups, i % n_groups, seen[i]);
                    return 1;
                }
            }
        }
    }
    std::printf("ok\n");
    return 0;
}
