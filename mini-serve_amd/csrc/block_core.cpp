// C++ page bookkeeping: allocator, per-request block table, batch packing. Host code only.
//
// Same contract as the Python implementation, page id for page id: a fresh allocator hands out
// 0, 1, 2, ...; freed pages are reused newest first; allocate is all or nothing; free validates the
// whole call before it changes anything. The language boundary is crossed once per unit of work:
// one call packs all tables of a batch, one call yields all new slots of a request.
//
// C ABI with status codes (mapped to Python exceptions by the caller):
//   0 ok, 1 out of blocks, 2 bad argument, 3 block id out of range, 4 incref of a free block,
//   5 more releases than holders, 6 position out of range / page given back, 7 invariant broken,
//   8 buffer too small, 9 duplicate block in prefix.
#include <cstddef>
#include <cstdint>
using std::size_t;
#include <unordered_map>
#include <unordered_set>
#include <vector>

namespace {

enum Status { OK = 0, OUT_OF_BLOCKS, BAD_ARG, BAD_ID, INCREF_FREE, OVER_RELEASE, BAD_POS, BROKEN, TOO_SMALL, DUP_PREFIX };

constexpr int NO_BLOCK = -1;

struct Allocator {
  int num_blocks, block_size;
  std::vector<int> free_;     // stack: back() is handed out first
  std::vector<int> holders_;  // 0 = free
  std::unordered_map<int, int> drops_;  // scratch of free()

  Allocator(int n, int bs) : num_blocks(n), block_size(bs), holders_(n, 0) {
    free_.reserve(n);
    for (int b = n - 1; b >= 0; --b) free_.push_back(b);
  }
  bool valid(int b) const { return b >= 0 && b < num_blocks; }

  int allocate(int n, int* out) {
    if (n < 0) return BAD_ARG;
    if ((size_t)n > free_.size()) return OUT_OF_BLOCKS;
    for (int i = 0; i < n; ++i) {
      const int b = free_.back();
      free_.pop_back();
      holders_[b] = 1;
      out[i] = b;
    }
    return OK;
  }
  int incref(const int* blocks, int n) {
    for (int i = 0; i < n; ++i) {
      if (!valid(blocks[i])) return BAD_ID;
      if (holders_[blocks[i]] == 0) return INCREF_FREE;
    }
    for (int i = 0; i < n; ++i) ++holders_[blocks[i]];
    return OK;
  }
  int release(const int* blocks, int n) {
    drops_.clear();
    for (int i = 0; i < n; ++i) {
      if (!valid(blocks[i])) return BAD_ID;
      ++drops_[blocks[i]];
    }
    for (const auto& kv : drops_)
      if (holders_[kv.first] < kv.second) return OVER_RELEASE;
    for (int i = 0; i < n; ++i)
      if (--holders_[blocks[i]] == 0) free_.push_back(blocks[i]);
    return OK;
  }
  int check() const {
    std::unordered_set<int> seen(free_.begin(), free_.end());
    if (seen.size() != free_.size()) return BROKEN;
    for (int b = 0; b < num_blocks; ++b) {
      if (holders_[b] < 0) return BROKEN;
      if ((holders_[b] == 0) != (seen.count(b) == 1)) return BROKEN;
    }
    return OK;
  }
};

struct Table {
  Allocator* alloc;
  std::vector<int> blocks;
  int num_tokens = 0;
  int first_live = 0;

  int needed(int n) const {
    const int bs = alloc->block_size;
    const int want = (num_tokens + n + bs - 1) / bs - (int)blocks.size();
    return want > 0 ? want : 0;
  }
  int append(int n, int* fresh, int cap, int* n_fresh) {
    if (n < 0) return BAD_ARG;
    const int k = needed(n);
    if (k > cap) return TOO_SMALL;
    const int st = alloc->allocate(k, fresh);
    if (st != OK) return st;
    blocks.insert(blocks.end(), fresh, fresh + k);
    num_tokens += n;
    *n_fresh = k;
    return OK;
  }
  int slot(int pos, int* out) const {
    if (pos < 0 || pos >= num_tokens) return BAD_POS;
    const int bs = alloc->block_size;
    const int b = blocks[pos / bs];
    if (b == NO_BLOCK) return BAD_POS;
    *out = b * bs + pos % bs;
    return OK;
  }
  int tail_slots(int n, int* out) const {
    if (n < 0 || n > num_tokens) return BAD_POS;
    const int bs = alloc->block_size;
    const int start = num_tokens - n;
    if (n > 0 && start / bs < first_live) return BAD_POS;
    for (int p = start; p < num_tokens; ++p) out[p - start] = blocks[p / bs] * bs + p % bs;
    return OK;
  }
  int rewind(int n) {
    if (n < 0 || n > num_tokens) return BAD_POS;
    if (n > 0 && (num_tokens - n) / alloc->block_size < first_live) return BAD_POS;
    num_tokens -= n;
    return OK;
  }
  int release_before(int pos, int* freed) {
    int upto = (pos > 0 ? pos : 0) / alloc->block_size;
    if (upto > (int)blocks.size()) upto = (int)blocks.size();
    *freed = 0;
    if (upto <= first_live) return OK;
    const int st = alloc->release(blocks.data() + first_live, upto - first_live);
    if (st != OK) return st;
    for (int i = first_live; i < upto; ++i) blocks[i] = NO_BLOCK;
    *freed = upto - first_live;
    first_live = upto;
    return OK;
  }
  int release_all() {
    const int st = alloc->release(blocks.data() + first_live, (int)blocks.size() - first_live);
    if (st != OK) return st;
    blocks.clear();
    num_tokens = 0;
    first_live = 0;
    return OK;
  }
};

}  // namespace

extern "C" {

void* msb_allocator_new(int num_blocks, int block_size) {
  if (num_blocks < 1 || block_size < 1) return nullptr;
  return new Allocator(num_blocks, block_size);
}
void msb_allocator_delete(void* a) { delete static_cast<Allocator*>(a); }
int msb_allocator_num_free(void* a) { return (int)static_cast<Allocator*>(a)->free_.size(); }
int msb_allocator_refcount(void* a, int block, int* out) {
  auto* al = static_cast<Allocator*>(a);
  if (!al->valid(block)) return BAD_ID;
  *out = al->holders_[block];
  return OK;
}
int msb_allocator_allocate(void* a, int n, int* out) { return static_cast<Allocator*>(a)->allocate(n, out); }
int msb_allocator_incref(void* a, const int* blocks, int n) { return static_cast<Allocator*>(a)->incref(blocks, n); }
int msb_allocator_free(void* a, const int* blocks, int n) { return static_cast<Allocator*>(a)->release(blocks, n); }
int msb_allocator_check(void* a) { return static_cast<Allocator*>(a)->check(); }

void* msb_table_new(void* a, const int* prefix, int n, int* status) {
  auto* al = static_cast<Allocator*>(a);
  std::unordered_set<int> seen(prefix, prefix + n);
  if ((int)seen.size() != n) {
    *status = DUP_PREFIX;
    return nullptr;
  }
  *status = al->incref(prefix, n);
  if (*status != OK) return nullptr;
  auto* t = new Table{al, {}, 0, 0};
  t->blocks.assign(prefix, prefix + n);
  t->num_tokens = n * al->block_size;
  return t;
}
void msb_table_delete(void* t) { delete static_cast<Table*>(t); }
int msb_table_num_tokens(void* t) { return static_cast<Table*>(t)->num_tokens; }
int msb_table_num_blocks(void* t) { return (int)static_cast<Table*>(t)->blocks.size(); }
int msb_table_first_live(void* t) { return static_cast<Table*>(t)->first_live; }
int msb_table_blocks_needed(void* t, int n) { return n < 0 ? -1 : static_cast<Table*>(t)->needed(n); }
int msb_table_append(void* t, int n, int* fresh, int cap, int* n_fresh) {
  return static_cast<Table*>(t)->append(n, fresh, cap, n_fresh);
}
int msb_table_slot(void* t, int pos, int* out) { return static_cast<Table*>(t)->slot(pos, out); }
int msb_table_tail_slots(void* t, int n, int* out) { return static_cast<Table*>(t)->tail_slots(n, out); }
int msb_table_rewind(void* t, int n) { return static_cast<Table*>(t)->rewind(n); }
int msb_table_release_before(void* t, int pos, int* freed) { return static_cast<Table*>(t)->release_before(pos, freed); }
int msb_table_release(void* t) { return static_cast<Table*>(t)->release_all(); }
int msb_table_blocks(void* t, int* out, int cap) {
  auto* tb = static_cast<Table*>(t);
  if ((int)tb->blocks.size() > cap) return TOO_SMALL;
  for (size_t i = 0; i < tb->blocks.size(); ++i) out[i] = tb->blocks[i];
  return OK;
}

// Rows of a dense int32 matrix out[rows, width]: row i = table i's entries, padded with pad_block;
// then pad_rows rows of pad_block alone. One call per batch.
int msb_pack_tables(void* const* tables, int n, int* out, int rows, int width, int pad_rows, int pad_block, int* total) {
  if (pad_rows < 0 || n < 0) return BAD_ARG;
  if (rows < n + pad_rows) return TOO_SMALL;
  int sum = 0;
  for (int i = 0; i < n; ++i) {
    const auto* tb = static_cast<const Table*>(tables[i]);
    const int k = (int)tb->blocks.size();
    if (k > width) return TOO_SMALL;
    int* row = out + (size_t)i * width;
    for (int j = 0; j < k; ++j) row[j] = tb->blocks[j];
    for (int j = k; j < width; ++j) row[j] = pad_block;
    sum += k;
  }
  for (int i = n; i < n + pad_rows; ++i)
    for (int j = 0; j < width; ++j) out[(size_t)i * width + j] = pad_block;
  *total = sum;
  return OK;
}

}  // extern "C"
