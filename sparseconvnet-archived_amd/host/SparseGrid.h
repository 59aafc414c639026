// Host-side SparseGrid: what a Picture fills in codifyInputData().
//
// Same surface as the reference's SparseGrid / SparseGridMap (SparseGrid.h):
// `backgroundCol` and a map `mp` from site key to feature-matrix row with
// operator[], find, insert, erase, size and iteration.  Iteration is in
// ascending key, the order of the reference's vectorHash back-end
// (SparseGrid.h:15-16, vectorHash.cpp:40-55); it is the order that fixes the
// row numbering of every rule book.  Storage is an insertion-ordered entry
// list with an open-addressing index, so codify stays O(1) per site on large
// lattices; deeper layers never use this class (their grids live in HBM).
#pragma once
#include <stdint.h>
#include <algorithm>
#include <utility>
#include <vector>

class SparseGridMap {
public:
  typedef std::pair<int64_t, int> value_type;
  typedef std::vector<value_type>::iterator iterator;

  SparseGridMap() : live_(0), sorted_(true) {}

  int &operator[](int64_t key) {
    size_t slot = 0;
    int at = lookup(key, &slot);
    if (at < 0)
      at = append(key, 0, slot);
    return entries_[at].second;
  }
  std::pair<iterator, bool> insert(const value_type &kv) {
    size_t slot = 0;
    int at = lookup(kv.first, &slot);
    bool fresh = at < 0;
    if (fresh)
      at = append(kv.first, kv.second, slot);
    return std::make_pair(entries_.begin() + at, fresh);
  }
  iterator find(int64_t key) {
    int at = lookup(key);
    return at < 0 ? entries_.end() : entries_.begin() + at;
  }
  // begin() puts the entries in ascending key before iteration starts
  iterator begin() {
    order();
    return entries_.begin();
  }
  iterator end() { return entries_.end(); }
  void erase(iterator it) {
    size_t at = it - entries_.begin();
    entries_.erase(entries_.begin() + at);
    reindex();
  }
  size_t size() const { return entries_.size(); }
  // room for n sites without growing on the way (optional)
  void reserve(size_t n) {
    entries_.reserve(n);
    size_t cap = 16;
    while (cap < 2 * n + 2)
      cap *= 2;
    if (cap > index_.size()) {
      index_.assign(cap, -1);
      for (size_t i = 0; i < entries_.size(); ++i)
        place((int)i);
    }
  }
  void clear() {
    entries_.clear();
    index_.clear();
    sorted_ = true;
  }
  // entries in insertion order unless an ordered view has been requested
  const std::vector<value_type> &entries() const { return entries_; }

private:
  std::vector<value_type> entries_;
  std::vector<int> index_; // open addressing over entries_, -1 = empty
  size_t live_;
  bool sorted_;

  static size_t mix(int64_t k) {
    uint64_t x = (uint64_t)k * 0x9E3779B97F4A7C15ull;
    return (size_t)(x ^ (x >> 29));
  }
  // the entry of `key`, or -1 and (if asked) the empty slot its probe ended at
  int lookup(int64_t key, size_t *emptySlot = nullptr) const {
    if (index_.empty())
      return -1;
    size_t mask = index_.size() - 1, s = mix(key) & mask;
    for (;;) {
      int at = index_[s];
      if (at < 0) {
        if (emptySlot)
          *emptySlot = s;
        return -1;
      }
      if (entries_[at].first == key)
        return at;
      s = (s + 1) & mask;
    }
  }
  void place(int at) {
    size_t mask = index_.size() - 1, s = mix(entries_[at].first) & mask;
    while (index_[s] >= 0)
      s = (s + 1) & mask;
    index_[s] = at;
  }
  void reindex() {
    size_t cap = 16;
    while (cap < 2 * entries_.size() + 2)
      cap *= 2;
    index_.assign(cap, -1);
    for (size_t i = 0; i < entries_.size(); ++i)
      place((int)i);
  }
  // slot: where lookup(key) gave up (valid unless the index has to grow)
  int append(int64_t key, int row, size_t slot) {
    if (!entries_.empty() && key < entries_.back().first)
      sorted_ = false;
    entries_.push_back(value_type(key, row));
    if (index_.size() < 2 * entries_.size() + 2)
      reindex();
    else
      index_[slot] = (int)entries_.size() - 1;
    return (int)entries_.size() - 1;
  }
  void order() {
    if (sorted_)
      return;
    std::sort(entries_.begin(), entries_.end());
    sorted_ = true;
    reindex();
  }
};

class SparseGrid {
public:
  int backgroundCol; // -1: no "null vector" row needed
  SparseGridMap mp;
  SparseGrid() : backgroundCol(-1) {}
};
