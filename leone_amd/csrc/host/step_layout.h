// Lays out the metadata of one step for the device: every kernel of the step reads its rows'
// tokens, positions, owners, state slots, wanted rows, query tiles and block tables from one
// buffer, so a step needs one upload.
//
// A part that works on tiles of consecutive rows of one request declares a tiling: portions of at least
// `min_rows` rows are cut into tiles of `tile_rows` rows, `group_tiles` tiles in a row make a group (what one
// workgroup of such a kernel takes, reading the portion's cache once for all its tiles), and a portion's last
// group is filled up with tiles of no rows.  A step may carry several tilings (parts with kernels of
// different shapes); each gets its own tile list.  Inside the step the entries that meet more of the
// tilings' thresholds come first, so that for every tiling the rows of its tiled portions are the step's
// first rows; short portions and single decoded tokens come last; logits keep the caller's order of
// entries.  The layout knows nothing of what the parts do with the tiles.  A step is refused as a whole, before anything is written, if an entry
// is empty, a request appears twice, a token lies outside the vocabulary or a wanted place outside
// its entry.
#pragma once

#include <cstdint>
#include <stdexcept>
#include <vector>

#include "cache_manager.h"

namespace leone::host {

struct StepRefused : std::runtime_error {
    using std::runtime_error::runtime_error;
};

struct StepEntryView {
    RequestKey request;
    const std::int32_t* tokens;
    int count;
    const std::int32_t* want;   // indices into tokens
    int want_count;
};

// Where an entry landed: entries are listed in the order they run in.
struct PlacedEntry {
    int given_index;   // position in the caller's list
    int slot;
    int first_row;
    int count;
    int start;         // absolute position of its first token
};

struct TiledRows {
    int rows = 0;            // rows [0, rows) of the step belong to portions this tiling cuts
    int tiles = 0;           // places in its tile list, unused ones included
};

struct StepSummary {
    int rows = 0;
    int max_position = 0;
    int wanted = 0;
    bool decode_only = true;
    std::vector<TiledRows> tiled;   // one per tiling of the shape
};

// Section offsets into the packed buffer, in 32-bit words: tokens, positions, row_entry, slots,
// want_rows, one tile list per tiling (entry, first row, rows; group_tiles to a group), then one block
// table [entries, max_blocks] per cache group; the last offset is the total.
struct StepSections {
    std::vector<long> offsets;
    long total() const { return offsets.back(); }
};

struct RowTiling {
    int tile_rows;        // rows of one tile
    int min_rows;         // portions at least this long are tiled
    int group_tiles;      // tiles that make a group
};

struct StepShape {
    int vocab_size;
    bool all_rows_wanted; // decode recording: the wanted rows are all rows, whatever the entries ask; nothing is tiled
    std::vector<RowTiling> tilings;
};

StepSections step_sections(const CacheManager& cache, const std::vector<StepEntryView>& entries, const StepShape& shape);

// Checks the step and writes it to `out` (which holds step_sections(...).total() words).
StepSummary pack_step(const CacheManager& cache, const std::vector<StepEntryView>& entries, const StepShape& shape,
                      const StepSections& sections, std::int32_t* out, std::vector<PlacedEntry>& placed);

}  // namespace leone::host
