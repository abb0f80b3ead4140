// moe_tuning.hpp — the tuning store of the MoE launch shapes.
//
// Winners of a measured sweep, kept per (stage, K, ncols, bucket of routed rows) and
// consulted by the launchers before the compiled-in rules of moe_heuristics.hpp.  On
// disk it is the reference's native tier (`vk-native-tuning/2`,
// src/c/vkernels/core/tuning.hpp:11-25): one line-based `moe_fused.gfx950.tune` under
// $VKERNELS_TUNING_CACHE (default ~/.cache/vkernels/tuning; the value "off" disables
// it), `#` comments, `key=stage,K,ncols,rows` starting a record, `name=value` lines
// (variant, waves, nt, depth) after it.  Malformed lines and shapes that are not
// compiled are skipped: a stale store degrades to the compiled-in rules, never to an
// error.
#pragma once

#include <string>

#include "moe_heuristics.hpp"

namespace vk {

constexpr const char* kMoeTuningFile = "moe_fused.gfx950.tune";
constexpr const char* kMoeTuningArch = "gfx950";  // the one architecture this library is compiled for

// Bucket of the routed rows a record is kept under: the power of two at or above
// n_flat up to the decode limit, one bucket beyond it.
int moe_rows_bucket(int n_flat);

// Store directory ("" when disabled).
std::string moe_tuning_dir();

// Reads `dir`/moe_fused.gfx950.tune (null: the store directory) into the process's
// table, replacing what a file put there before; records set by moe_tuning_set stay.
// Returns the number of records taken, 0 when there is no file.  A file whose first line
// is not `# vk-native-tuning/2`, or whose `# arch=` comment names another architecture,
// counts as no file.
int moe_tuning_load(const char* dir);

// Parses a .tune body into the table (what moe_tuning_load does with the file).
int moe_tuning_parse(const std::string& text);

// The record of this problem, if any.  The first call loads the default store.
bool moe_tuning_find(int stage, int K, int ncols, int n_flat, MoeTile* tile);

// Sets (tile != null; must be a candidate of the stage) or removes the record.
bool moe_tuning_set(int stage, int K, int ncols, int n_flat, const MoeTile* tile);

// Every record as a .tune body (what a sweep writes to the store).
std::string moe_tuning_dump(const char* written_by);

}  // namespace vk
