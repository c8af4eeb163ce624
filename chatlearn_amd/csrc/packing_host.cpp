// Host-side bin packing for dynamic batching (plain C++, no GPU work): the
// reference does this on the CPU too, in interpreted loops over Python lists.
// Same decisions, item for item: stable longest-first order, strict-fit
// best-fit for the open-ended packer, lightest-bin-first for the fixed-count
// packer followed by a descending (total, id-list) ordering of the bins.
#include <algorithm>
#include <numeric>
#include <vector>
#include "common.hpp"

namespace {

std::vector<int64_t> longest_first(const int64_t* len, int64_t n) {
  std::vector<int64_t> idx(n);
  std::iota(idx.begin(), idx.end(), 0);
  std::stable_sort(idx.begin(), idx.end(), [&](int64_t a, int64_t b) { return len[a] > len[b]; });
  return idx;
}

void emit(const std::vector<std::vector<int64_t>>& bins, int64_t* order, int64_t* offsets) {
  int64_t pos = 0;
  for (size_t b = 0; b < bins.size(); ++b) {
    offsets[b] = pos;
    for (int64_t id : bins[b]) order[pos++] = id;
  }
  offsets[bins.size()] = pos;
}

}  // namespace

extern "C" int clgrpo_bin_packing(const int64_t* seq_len, int64_t n, int64_t max_train_token, int64_t* order,
                                  int64_t* bin_offsets, int64_t* n_bins) {
  if (n < 0) return clgrpo::fail(CLGRPO_EINVAL, "clgrpo_bin_packing: n=%lld", (long long)n);
  if (!bin_offsets || !n_bins || (n > 0 && (!seq_len || !order)))
    return clgrpo::fail(CLGRPO_ENULL, "clgrpo_bin_packing: NULL pointer");
  std::vector<std::vector<int64_t>> bins;
  std::vector<int64_t> load;
  for (int64_t id : longest_first(seq_len, n)) {
    const int64_t need = seq_len[id];
    int64_t pick = -1, pick_free = 0;
    for (size_t b = 0; b < bins.size(); ++b) {
      const int64_t free_ = max_train_token - load[b];
      if (free_ > need && (pick < 0 || free_ < pick_free)) { pick = (int64_t)b; pick_free = free_; }
    }
    if (pick < 0) { bins.push_back({id}); load.push_back(need); }
    else { bins[pick].push_back(id); load[pick] += need; }
  }
  emit(bins, order, bin_offsets);
  *n_bins = (int64_t)bins.size();
  return CLGRPO_OK;
}

extern "C" int clgrpo_bin_packing_fix_bin(const int64_t* seq_len, int64_t n, int64_t bin_size, int64_t* order,
                                          int64_t* bin_offsets) {
  if (n < 0 || bin_size <= 0)
    return clgrpo::fail(CLGRPO_EINVAL, "clgrpo_bin_packing_fix_bin: n=%lld bin_size=%lld", (long long)n, (long long)bin_size);
  if (!bin_offsets || (n > 0 && (!seq_len || !order)))
    return clgrpo::fail(CLGRPO_ENULL, "clgrpo_bin_packing_fix_bin: NULL pointer");
  std::vector<std::vector<int64_t>> bins(bin_size);
  std::vector<int64_t> load(bin_size, 0);
  for (int64_t id : longest_first(seq_len, n)) {
    int64_t pick = 0;
    for (int64_t b = 1; b < bin_size; ++b)
      if (load[b] < load[pick]) pick = b;
    bins[pick].push_back(id);
    load[pick] += seq_len[id];
  }
  // Descending by (total, id list): equal totals are ordered by comparing the lists, as tuples compare.
  std::vector<int64_t> perm(bin_size);
  std::iota(perm.begin(), perm.end(), 0);
  std::stable_sort(perm.begin(), perm.end(), [&](int64_t a, int64_t b) {
    if (load[a] != load[b]) return load[a] > load[b];
    return std::lexicographical_compare(bins[b].begin(), bins[b].end(), bins[a].begin(), bins[a].end());
  });
  std::vector<std::vector<int64_t>> sorted;
  sorted.reserve(bin_size);
  for (int64_t b : perm) sorted.push_back(bins[b]);
  emit(sorted, order, bin_offsets);
  return CLGRPO_OK;
}
