// moe_tuning.cpp — see moe_tuning.hpp.
#include "moe_tuning.hpp"

#include <array>
#include <atomic>
#include <cstdio>
#include <cstdlib>
#include <fstream>
#include <map>
#include <mutex>
#include <sstream>

namespace vk {
namespace {

using Key = std::array<int, 4>;  // stage, K, ncols, rows bucket

struct Record {
  MoeTile tile;
  bool from_file;
};

std::mutex g_lock;
std::map<Key, Record> g_table;
std::atomic<int> g_records{0};  // launches skip the lock while the table is empty
std::atomic<unsigned> g_version{0};  // bumped by every change of the table (under the lock)
std::once_flag g_default_loaded;

Key make_key(int stage, int K, int ncols, int n_flat) {
  return Key{stage, K, ncols, moe_rows_bucket(n_flat)};
}

bool parse_ints(const std::string& text, long long* out, int want) {
  const char* p = text.c_str();
  for (int i = 0; i < want; ++i) {
    char* end = nullptr;
    out[i] = strtoll(p, &end, 10);
    if (end == p) return false;
    p = end;
    if (i + 1 < want) {
      if (*p != ',') return false;
      ++p;
    }
  }
  while (*p == ' ' || *p == '\t' || *p == '\r') ++p;
  return *p == 0;
}

// Takes the record being assembled if it is complete and names a compiled shape.
void commit(bool open, const long long (&key)[4], const long long (&val)[4], unsigned seen, int* taken) {
  if (!open || seen != 0xFu) return;
  const MoeTile tile{(int)val[0], (int)val[1], (int)val[2], (int)val[3]};
  const int stage = (int)key[0];
  if ((stage != 0 && stage != 1) || !is_moe_tile_candidate(stage, tile)) return;
  if (key[1] <= 0 || key[2] <= 0 || key[3] <= 0 || key[1] > (1 << 24) || key[2] > (1 << 24)) return;
  const Key k{stage, (int)key[1], (int)key[2], moe_rows_bucket((int)key[3])};
  auto it = g_table.find(k);
  if (it != g_table.end() && !it->second.from_file) return;  // a record set by hand wins
  g_table[k] = Record{tile, true};
  ++*taken;
}

int parse_locked(const std::string& text) {
  for (auto it = g_table.begin(); it != g_table.end();)
    it = it->second.from_file ? g_table.erase(it) : std::next(it);
  static const char* names[4] = {"variant", "waves", "nt", "depth"};
  std::istringstream in(text);
  std::string line;
  long long key[4] = {0, 0, 0, 0}, val[4] = {0, 0, 0, 0};
  unsigned seen = 0;
  bool open = false;
  int taken = 0;
  while (std::getline(in, line)) {
    const size_t first = line.find_first_not_of(" \t\r");
    if (first == std::string::npos || line[first] == '#') continue;
    const size_t eq = line.find('=', first);
    if (eq == std::string::npos) continue;
    const std::string name = line.substr(first, eq - first), value = line.substr(eq + 1);
    if (name == "key") {
      commit(open, key, val, seen, &taken);
      seen = 0;
      open = parse_ints(value, key, 4);
      continue;
    }
    for (int i = 0; i < 4; ++i) {
      long long v = 0;
      if (name == names[i] && parse_ints(value, &v, 1)) {
        val[i] = v;
        seen |= 1u << i;
      }
    }
  }
  commit(open, key, val, seen, &taken);
  g_version.fetch_add(1u, std::memory_order_relaxed);
  g_records.store((int)g_table.size(), std::memory_order_release);
  return taken;
}

}  // namespace

int moe_rows_bucket(int n_flat) {
  if (n_flat > kMoeDecodeMaxRows) return 2 * kMoeDecodeMaxRows;
  int b = 1;
  while (b < n_flat) b <<= 1;
  return b;
}

std::string moe_tuning_dir() {
  const char* env = getenv("VKERNELS_TUNING_CACHE");
  if (env != nullptr && *env != 0) return std::string(env) == "off" ? std::string() : std::string(env);
  const char* home = getenv("HOME");
  if (home == nullptr || *home == 0) return std::string();
  return std::string(home) + "/.cache/vkernels/tuning";
}

int moe_tuning_parse(const std::string& text) {
  std::lock_guard<std::mutex> hold(g_lock);
  return parse_locked(text);
}

// True for a body this library may take records from: it starts with the format's header
// line, as the reference requires of a store file (src/c/vkernels/core/tuning.cpp:195), and
// the architecture it names in its `# arch=` comment, if it names one, is the one this
// library is compiled for (the reference keys its stores by that token,
// core/tuning.cpp:137-150; records swept on another device say nothing about this one).
bool moe_tuning_body_ok(const std::string& body) {
  static const char kHeader[] = "# vk-native-tuning/2";
  if (body.rfind(kHeader, 0) != 0) return false;
  std::istringstream in(body);
  std::string line;
  while (std::getline(in, line)) {
    const size_t first = line.find_first_not_of(" \t\r");
    if (first == std::string::npos) continue;
    if (line[first] != '#') break;  // the header comments are over
    const size_t at = line.find("arch=", first);
    if (at == std::string::npos) continue;
    std::string arch = line.substr(at + 5);
    arch = arch.substr(0, arch.find_first_of(" \t\r"));
    return arch == kMoeTuningArch;
  }
  return true;
}

int moe_tuning_load(const char* dir) {
  const std::string root = dir != nullptr ? std::string(dir) : moe_tuning_dir();
  std::string body;
  if (!root.empty()) {
    std::ifstream in(root + "/" + kMoeTuningFile, std::ios::binary);
    if (in) {
      std::ostringstream all;
      all << in.rdbuf();
      body = all.str();
    }
  }
  // a file of another format or another device is as good as no file
  if (!moe_tuning_body_ok(body)) body.clear();
  return moe_tuning_parse(body);
}

bool moe_tuning_find(int stage, int K, int ncols, int n_flat, MoeTile* tile) {
  std::call_once(g_default_loaded, [] { (void)moe_tuning_load(nullptr); });
  if (g_records.load(std::memory_order_acquire) == 0) return false;
  // A serving loop asks for the same few problems call after call: each thread keeps
  // its last answer per stage and takes the lock only when the problem or the table
  // has changed since.
  struct Last {
    unsigned version;
    Key key;
    bool valid, found;
    MoeTile tile;
  };
  thread_local Last last[2] = {};
  const Key key = make_key(stage, K, ncols, n_flat);
  Last& l = last[stage & 1];
  const unsigned version = g_version.load(std::memory_order_acquire);
  if (!(l.valid && l.version == version && l.key == key)) {
    std::lock_guard<std::mutex> hold(g_lock);
    const auto it = g_table.find(key);
    l.version = g_version.load(std::memory_order_relaxed);
    l.key = key;
    l.valid = true;
    l.found = it != g_table.end();
    if (l.found) l.tile = it->second.tile;
  }
  if (!l.found) return false;
  *tile = l.tile;
  return true;
}

bool moe_tuning_set(int stage, int K, int ncols, int n_flat, const MoeTile* tile) {
  if ((stage != 0 && stage != 1) || K <= 0 || ncols <= 0 || n_flat <= 0) return false;
  if (tile != nullptr && !is_moe_tile_candidate(stage, *tile)) return false;
  std::call_once(g_default_loaded, [] { (void)moe_tuning_load(nullptr); });
  std::lock_guard<std::mutex> hold(g_lock);
  const Key k = make_key(stage, K, ncols, n_flat);
  if (tile != nullptr) g_table[k] = Record{*tile, false};
  else g_table.erase(k);
  g_version.fetch_add(1u, std::memory_order_relaxed);
  g_records.store((int)g_table.size(), std::memory_order_release);
  return true;
}

std::string moe_tuning_dump(const char* written_by) {
  std::lock_guard<std::mutex> hold(g_lock);
  std::ostringstream out;
  out << "# vk-native-tuning/2\n# arch=" << kMoeTuningArch << " written_by=" << (written_by != nullptr ? written_by : "unknown") << "\n";
  for (const auto& kv : g_table) {
    const Key& k = kv.first;
    const MoeTile& t = kv.second.tile;
    out << "key=" << k[0] << ',' << k[1] << ',' << k[2] << ',' << k[3] << "\nvariant=" << t.variant
        << "\nwaves=" << t.waves << "\nnt=" << t.nt << "\ndepth=" << t.depth << "\n";
  }
  return out.str();
}

}  // namespace vk
