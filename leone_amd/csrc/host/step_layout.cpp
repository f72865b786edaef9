#include "step_layout.h"

#include <algorithm>
#include <string>
#include <unordered_set>

namespace leone::host {

namespace {

bool tiled(const StepEntryView& e, const StepShape& shape, const RowTiling& t) {
    return !shape.all_rows_wanted && e.count >= t.min_rows;
}

// How many of the tilings cut this entry: thresholds nest, so the entries a tiling cuts are those that reach
// a certain number.
int tilings_met(const StepEntryView& e, const StepShape& shape) {
    int met = 0;
    for (const RowTiling& t : shape.tilings) met += tiled(e, shape, t) ? 1 : 0;
    return met;
}

// Places the tiles of a portion of `count` rows take: whole groups.
long tile_places(int count, const RowTiling& t) {
    const long tiles = (count + t.tile_rows - 1) / t.tile_rows;
    return (tiles + t.group_tiles - 1) / t.group_tiles * t.group_tiles;
}

void check(const std::vector<StepEntryView>& entries, const StepShape& shape) {
    if (entries.empty()) throw StepRefused("a step needs at least one entry");
    std::unordered_set<RequestKey> seen;
    for (const StepEntryView& e : entries) {
        const std::string who = "request " + std::to_string(e.request);
        if (!seen.insert(e.request).second) throw StepRefused(who + " appears twice in one step");
        if (e.count <= 0) throw StepRefused(who + " brings no tokens");
        for (int i = 0; i < e.count; ++i)
            if (e.tokens[i] < 0 || e.tokens[i] >= shape.vocab_size)
                throw StepRefused(who + ": token " + std::to_string(e.tokens[i]) + " is outside the vocabulary of " +
                                  std::to_string(shape.vocab_size));
        for (int i = 0; i < e.want_count; ++i)
            if (e.want[i] < 0 || e.want[i] >= e.count)
                throw StepRefused(who + ": wanted place " + std::to_string(e.want[i]) + " is outside its " +
                                  std::to_string(e.count) + " tokens");
    }
}

}  // namespace

StepSections step_sections(const CacheManager& cache, const std::vector<StepEntryView>& entries, const StepShape& shape) {
    long rows = 0, wanted = 0;
    std::vector<long> tiles(shape.tilings.size(), 0);
    for (const StepEntryView& e : entries) {
        rows += e.count;
        wanted += e.want_count;
        for (size_t i = 0; i < shape.tilings.size(); ++i)
            if (tiled(e, shape, shape.tilings[i])) tiles[i] += tile_places(e.count, shape.tilings[i]);
    }
    if (shape.all_rows_wanted) wanted = rows;
    const long n = static_cast<long>(entries.size());
    StepSections s;
    s.offsets = {0, rows, 2 * rows, 3 * rows, 3 * rows + n, 3 * rows + n + wanted};
    for (long count : tiles) s.offsets.push_back(s.offsets.back() + 3 * count);
    for (int g = 0; g < cache.group_count(); ++g) s.offsets.push_back(s.offsets.back() + n * cache.max_blocks(g));
    return s;
}

StepSummary pack_step(const CacheManager& cache, const std::vector<StepEntryView>& entries, const StepShape& shape,
                      const StepSections& sections, std::int32_t* out, std::vector<PlacedEntry>& placed) {
    check(entries, shape);
    for (const StepEntryView& e : entries) cache.length(e.request);   // throws for a request that is not admitted

    const int n = static_cast<int>(entries.size());
    std::vector<int> order(n);
    for (int i = 0; i < n; ++i) order[i] = i;
    std::stable_sort(order.begin(), order.end(),
                     [&](int a, int b) { return tilings_met(entries[a], shape) > tilings_met(entries[b], shape); });

    std::int32_t* tokens = out + sections.offsets[0];
    std::int32_t* positions = out + sections.offsets[1];
    std::int32_t* row_entry = out + sections.offsets[2];
    std::int32_t* slots = out + sections.offsets[3];
    std::int32_t* want_rows = out + sections.offsets[4];
    const int n_tilings = static_cast<int>(shape.tilings.size());
    const int first_table = 5 + n_tilings;          // index of the first block table's offset

    StepSummary summary;
    summary.tiled.assign(n_tilings, TiledRows{});
    placed.assign(n, PlacedEntry{});
    std::vector<int> first_row(n, 0);
    int row = 0;
    for (int ei = 0; ei < n; ++ei) {
        const StepEntryView& e = entries[order[ei]];
        const int start = cache.length(e.request);
        first_row[order[ei]] = row;
        for (int i = 0; i < e.count; ++i) {
            tokens[row + i] = e.tokens[i];
            positions[row + i] = start + i;
            row_entry[row + i] = ei;
        }
        slots[ei] = cache.slot(e.request);
        for (int g = 0; g < cache.group_count(); ++g) {
            const std::vector<int>& table = cache.table(e.request, g);
            const int width = cache.max_blocks(g);
            std::int32_t* dst = out + sections.offsets[first_table + g] + static_cast<long>(ei) * width;
            const int held = std::min<int>(width, static_cast<int>(table.size()));
            std::copy(table.begin(), table.begin() + held, dst);
            std::fill(dst + held, dst + width, -1);
        }
        for (int ti = 0; ti < n_tilings; ++ti) {
            const RowTiling& t = shape.tilings[ti];
            if (!tiled(e, shape, t)) continue;
            std::int32_t* tiles = out + sections.offsets[5 + ti];
            int& tile = summary.tiled[ti].tiles;
            const int n_tiles = (e.count + t.tile_rows - 1) / t.tile_rows;
            const long places = tile_places(e.count, t);
            for (long index = 0; index < places; ++index) {
                const bool used = index < n_tiles;
                const int at = static_cast<int>(index) * t.tile_rows;
                tiles[3 * tile] = ei;
                tiles[3 * tile + 1] = used ? row + at : row;
                tiles[3 * tile + 2] = used ? std::min(t.tile_rows, e.count - at) : 0;
                ++tile;
            }
            summary.tiled[ti].rows = row + e.count;
        }
        if (e.count != 1) summary.decode_only = false;
        summary.max_position = std::max(summary.max_position, start + e.count - 1);
        placed[ei] = PlacedEntry{order[ei], slots[ei], row, e.count, start};
        row += e.count;
    }
    int wanted = 0;
    if (shape.all_rows_wanted) {
        for (int r = 0; r < row; ++r) want_rows[wanted++] = r;
    } else {
        for (int i = 0; i < n; ++i)
            for (int w = 0; w < entries[i].want_count; ++w) want_rows[wanted++] = first_row[i] + entries[i].want[w];
    }
    summary.rows = row;
    summary.wanted = wanted;
    return summary;
}

}  // namespace leone::host
