// Lays out the metadata of one step for the device: every kernel of the step reads its rows'
// tokens, positions, owners, state slots, wanted rows, query tiles and block tables from one
// buffer, so a step needs one upload.
//
// Inside the step, prompt portions long enough for the tiled prompt-attention kernel come first,
// short portions and single decoded tokens after; logits keep the caller's order of entries.  A
// tiled portion is cut into tiles of `tile_rows` rows; `group_tiles` tiles in a row make a group (one
// workgroup of that kernel, which reads the portion's keys once for all its tiles).  A portion's
// last group is filled up with tiles of no rows.  A step is refused as a whole, before anything is written, if an entry
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

struct StepSummary {
    int rows = 0;
    int prefill_rows = 0;    // rows [0, prefill_rows) belong to tiled prompt portions
    int max_position = 0;
    int tiles = 0;           // places in the tile list, unused ones included
    int wanted = 0;
    bool decode_only = true;
};

// Section offsets into the packed buffer, in 32-bit words: tokens, positions, row_entry, slots,
// want_rows, tiles (entry, first row, rows; group_tiles to a group), then one block table
// [entries, max_blocks] per cache group; the last offset is the total.
struct StepSections {
    std::vector<long> offsets;
    long total() const { return offsets.back(); }
};

struct StepShape {
    int vocab_size;
    int tile_rows;        // rows of one query tile of the prompt-attention kernel
    int min_tile_rows;    // portions at least this long are tiled
    bool all_rows_wanted; // decode recording: the wanted rows are all rows, whatever the entries ask
    int group_tiles;      // tiles one workgroup of the prompt-attention kernel takes
};

StepSections step_sections(const CacheManager& cache, const std::vector<StepEntryView>& entries, const StepShape& shape);

// Checks the step and writes it to `out` (which holds step_sections(...).total() words).
StepSummary pack_step(const CacheManager& cache, const std::vector<StepEntryView>& entries, const StepShape& shape,
                      const StepSections& sections, std::int32_t* out, std::vector<PlacedEntry>& placed);

}  // namespace leone::host
