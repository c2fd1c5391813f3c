// Page and slot pools and the cache manager of the host runtime; see module.cpp for what the
// module is and which parts of the reference it stands for.
#pragma once
#include <pybind11/numpy.h>
#include <pybind11/pybind11.h>
#include <pybind11/stl.h>

#include <algorithm>
#include <cstdint>
#include <map>
#include <set>
#include <sstream>
#include <stdexcept>
#include <string>
#include <unordered_map>
#include <vector>

namespace py = pybind11;

namespace mshost {

struct CacheError : std::runtime_error {
    using std::runtime_error::runtime_error;
};
struct OutOfPages : CacheError {
    using CacheError::CacheError;
};

template <typename... A> static std::string cat(A&&... a) {
    std::ostringstream s;
    (s << ... << a);
    return s.str();
}

// A LIFO free list over a bump pointer, with a bitmap of live pages so that freeing a page twice,
// or one that was never handed out, fails at once.
class BlockPool {
public:
    explicit BlockPool(int num_pages) : num_pages_(num_pages), live_(num_pages > 0 ? num_pages : 0, 0) {
        if (num_pages < 1) throw CacheError(cat("a pool needs at least one page, got ", num_pages));
    }
    int num_pages() const { return num_pages_; }
    int available() const { return (int)free_.size() + (num_pages_ - next_); }
    int alloc() {  // -1: exhausted
        int p;
        if (!free_.empty()) {
            p = free_.back();
            free_.pop_back();
        } else if (next_ < num_pages_) {
            p = next_++;
        } else {
            return -1;
        }
        if (live_[p]) throw CacheError(cat("page ", p, " handed out while live"));
        live_[p] = 1;
        return p;
    }
    void free(int page) {
        if (page < 0 || page >= num_pages_ || !live_[page])
            throw CacheError(cat("page ", page, " freed twice or never handed out (pool of ", num_pages_, ")"));
        live_[page] = 0;
        free_.push_back(page);
    }
    std::vector<int> live_pages() const {
        std::vector<int> out;
        for (int p = 0; p < num_pages_; ++p)
            if (live_[p]) out.push_back(p);
        return out;
    }

private:
    int num_pages_, next_ = 0;
    std::vector<int> free_;
    std::vector<char> live_;
};

// Indices into the per-request arrays of fixed size; lowest free index first.
class SlotPool {
public:
    explicit SlotPool(int n) : n_(n), live_(n > 0 ? n : 0, 0) {
        for (int i = 0; i < n; ++i) free_.insert(i);
    }
    int num_slots() const { return n_; }
    int available() const { return (int)free_.size(); }
    int alloc() {
        if (free_.empty()) return -1;
        int s = *free_.begin();
        free_.erase(free_.begin());
        live_[s] = 1;
        return s;
    }
    void free(int slot) {
        if (!is_live(slot)) throw CacheError(cat("slot ", slot, " freed twice or never handed out"));
        live_[slot] = 0;
        free_.insert(slot);
    }
    bool is_live(int slot) const { return slot >= 0 && slot < n_ && live_[slot]; }

private:
    int n_;
    std::set<int> free_;
    std::vector<char> live_;
};

struct Group {
    std::string name;
    int window;  // keys a row may see; 0 = all
    BlockPool pool;
    std::unordered_map<int, std::vector<int>> tables;  // slot -> logical page -> physical page, -1 = given back
    std::unordered_map<int, int> first_live;           // slot -> first logical page not yet given back
    Group(std::string n, int w, int pages) : name(std::move(n)), window(w), pool(pages) {}
};

class CacheCore {
public:
    CacheCore(int page_size, int max_requests) : page_size_(page_size), slots_(max_requests) {
        if (page_size < 16 || page_size % 16) throw CacheError(cat("page size ", page_size, " must be a positive multiple of 16"));
        if (max_requests < 1) throw CacheError("at least one request slot is needed");
    }
    int add_group(const std::string& name, int window, int num_pages) {
        groups_.emplace_back(name, window, num_pages);
        return (int)groups_.size() - 1;
    }
    int page_size() const { return page_size_; }
    int max_requests() const { return slots_.num_slots(); }
    int num_groups() const { return (int)groups_.size(); }
    const std::string& group_name(int g) const { return groups_.at(g).name; }
    int group_window(int g) const { return groups_.at(g).window; }
    int group_pages(int g) const { return groups_.at(g).pool.num_pages(); }
    int group_available(int g) const { return groups_.at(g).pool.available(); }
    std::vector<int> group_live_pages(int g) const { return groups_.at(g).pool.live_pages(); }
    // A page beyond every pool (id = the pool's size) and a slot beyond the request slots (id = max_requests): never
    // handed out.  Rows that only fill a captured step up to its size write there, so that they change nothing a
    // request owns: neither a key nor a state.  The device arrays are one page and one slot larger for them.
    int scratch_page(int g) const { return groups_.at(g).pool.num_pages(); }
    int scratch_slot() const { return slots_.num_slots(); }
    int slots_available() const { return slots_.available(); }
    bool slot_is_live(int s) const { return slots_.is_live(s); }

    int admit() {
        int slot = slots_.alloc();
        if (slot < 0) throw CacheError(cat("all ", slots_.num_slots(), " request slots are in use"));
        lengths_[slot] = 0;
        for (auto& g : groups_) {
            g.tables[slot] = {};
            g.first_live[slot] = 0;
        }
        return slot;
    }
    int length(int slot) const {
        auto it = lengths_.find(slot);
        if (it == lengths_.end()) throw CacheError(cat("slot ", slot, " is not in use"));
        return it->second;
    }
    std::map<int, int> lengths() const { return lengths_; }
    std::vector<int> pages_needed(int slot, int n_new) const {
        const int end = length(slot) + n_new;
        std::vector<int> need;
        for (auto& g : groups_) {
            const int have = (int)g.tables.at(slot).size();
            need.push_back(std::max(0, (end + page_size_ - 1) / page_size_ - have));
        }
        return need;
    }
    bool can_extend(int slot, int n_new, const std::vector<int>& reserved) const {
        auto need = pages_needed(slot, n_new);
        for (size_t g = 0; g < groups_.size(); ++g) {
            const int res = g < reserved.size() ? reserved[g] : 0;
            if (groups_[g].pool.available() - res < need[g]) return false;
        }
        return true;
    }
    void extend(int slot, int n_new) {  // all groups or none
        if (!slots_.is_live(slot)) throw CacheError(cat("slot ", slot, " is not in use"));
        auto need = pages_needed(slot, n_new);
        for (size_t g = 0; g < groups_.size(); ++g)
            if (groups_[g].pool.available() < need[g])
                throw OutOfPages(cat("group ", groups_[g].name, ": ", need[g], " pages needed for ", n_new, " tokens of slot ", slot,
                                     ", ", groups_[g].pool.available(), " free"));
        for (size_t g = 0; g < groups_.size(); ++g)
            for (int i = 0; i < need[g]; ++i) groups_[g].tables[slot].push_back(groups_[g].pool.alloc());
    }
    void commit(int slot, int n_new) {
        const int L = (lengths_.at(slot) += n_new);
        for (auto& g : groups_) {
            if (g.window <= 0) continue;
            // the next row is at position L and sees keys > L - window
            auto& table = g.tables[slot];
            const int dead = std::min((int)table.size(), std::max(0, L - g.window + 1) / page_size_);
            int& first = g.first_live[slot];
            for (int p = first; p < dead; ++p)
                if (table[p] >= 0) {
                    g.pool.free(table[p]);
                    table[p] = -1;
                }
            first = std::max(first, dead);
        }
    }
    void release(int slot) {
        if (!slots_.is_live(slot)) throw CacheError(cat("slot ", slot, " released twice or never admitted"));
        for (auto& g : groups_) {
            for (int p : g.tables[slot])
                if (p >= 0) g.pool.free(p);
            g.tables.erase(slot);
            g.first_live.erase(slot);
        }
        lengths_.erase(slot);
        slots_.free(slot);
    }
    const std::vector<int>& table(int g, int slot) const {
        auto& t = groups_.at(g).tables;
        auto it = t.find(slot);
        if (it == t.end()) throw CacheError(cat("slot ", slot, " is not in use"));
        return it->second;
    }
    int slot_of_position(int g, int slot, int pos) const {
        const auto& t = table(g, slot);
        if (pos < 0 || pos / page_size_ >= (int)t.size()) throw py::index_error(cat("position ", pos, " of slot ", slot, " has no page"));
        const int page = t[pos / page_size_];
        if (page < 0) throw CacheError(cat("group ", groups_[g].name, ": position ", pos, " of slot ", slot, " lies in a page already given back"));
        return page * page_size_ + pos % page_size_;
    }
    std::vector<int> live_requests() const {
        std::vector<int> out;
        for (auto& kv : lengths_) out.push_back(kv.first);
        return out;
    }
    // A page is owned by at most one table entry, and every live page of a pool is owned.
    void check() const {
        for (auto& g : groups_) {
            std::map<int, int> owned;
            for (auto& kv : g.tables)
                for (int p : kv.second) {
                    if (p < 0) continue;
                    if (owned.count(p)) throw CacheError(cat("group ", g.name, ": page ", p, " held by slot ", owned[p], " and slot ", kv.first));
                    owned[p] = kv.first;
                }
            auto live = g.pool.live_pages();
            if (live.size() != owned.size() || !std::all_of(live.begin(), live.end(), [&](int p) { return owned.count(p) > 0; }))
                throw CacheError(cat("group ", g.name, ": ", live.size(), " live pages differ from ", owned.size(), " owned pages"));
            if ((int)live.size() + g.pool.available() != g.pool.num_pages())
                throw CacheError(cat("group ", g.name, ": ", live.size(), " live + ", g.pool.available(), " free != ", g.pool.num_pages()));
        }
    }

    // The int32 buffer of a step.  Entries are (slot, number of tokens); tokens and wanted rows come
    // flattened.  Sections, each starting on a 16-byte boundary, in this order: tokens, positions,
    // seq_q_start, seq_q_len, seq_pos0, seq_slot, want_rows, then per group "table/<name>" [S, width]
    // and "slot_map/<name>" [T], then per entry of heads_per_kv "work/<g>" [n, 2].  `table_multiple`
    // rounds the widths of the block tables up (captured graphs want few distinct widths).  `pad_rows` appends that
    // many requests of one row each that belong to nobody: token 0 at position 0 of the scratch slot, whose one page
    // is the scratch page; their rows run like any other and leave no trace in what requests own.  "positions" is
    // [T, axes]: on every axis a row's index in its request's cache, unless `explicit_positions` ([T, axes]
    // flattened, rows of the entries only) gives the caller's own (where a row sits in the cache never follows them).
    //
    // `fill_rows`, `fill_seqs`, `fill_want` > 0 fill a step of any mix up to a size that many steps share (one
    // captured graph then serves them all): requests of the scratch slot are appended until there are `fill_seqs`
    // requests and `fill_rows` rows, the last of them taking what rows are left (token 0 at positions 0, 1, ...,
    // all of its pages being the scratch page, so rows a page apart write the same place: nobody reads it); the
    // wanted rows are filled up to `fill_want` with the step's last row; and every work list is filled up, with
    // items of request -1 that the attention kernel skips, to the most items that any step of this size can have,
    // fill_rows * g / rows_per_block + fill_seqs.  Needs fill_rows - rows >= fill_seqs - entries >= 1, or both zero (a step
    // that has the size already: only its wanted rows and work lists are filled up).
    py::tuple build_step(const std::vector<int>& slots_in, const std::vector<int>& counts_in, const std::vector<int>& tokens_in,
                         const std::vector<int>& want_in, const std::vector<int>& heads_per_kv, int rows_per_block,
                         int table_multiple, int pad_rows, int axes, const std::vector<int>& explicit_positions,
                         int fill_rows, int fill_seqs, int fill_want) const {
        const int S_real = (int)slots_in.size();
        if (S_real == 0 || counts_in.size() != slots_in.size()) throw CacheError("a step needs at least one entry");
        if (pad_rows < 0) throw CacheError("pad_rows must not be negative");
        std::vector<int> slots(slots_in), counts(counts_in), tokens(tokens_in), want_rows(want_in);
        slots.insert(slots.end(), pad_rows, scratch_slot());
        counts.insert(counts.end(), pad_rows, 1);
        tokens.insert(tokens.end(), pad_rows, 0);
        const int T_real = (int)tokens_in.size();
        if (fill_rows > 0) {
            if (pad_rows) throw CacheError("a step is filled up with single rows or to a size, not both");
            const int more_seqs = fill_seqs - S_real, more_rows = fill_rows - T_real;
            if (more_seqs < 0 || more_rows < more_seqs || (more_seqs == 0 && more_rows > 0))
                throw CacheError(cat("a step of ", S_real, " requests and ", T_real, " rows cannot be filled up to ", fill_seqs, " and ", fill_rows));
            if ((int)want_rows.size() > fill_want) throw CacheError(cat(want_rows.size(), " wanted rows exceed ", fill_want));
            if (more_seqs > 0) {
                slots.insert(slots.end(), more_seqs, scratch_slot());
                counts.insert(counts.end(), more_seqs - 1, 1);
                counts.push_back(more_rows - (more_seqs - 1));
                tokens.insert(tokens.end(), more_rows, 0);
            }
            want_rows.insert(want_rows.end(), fill_want - want_rows.size(), fill_rows - 1);
        }
        const int S = (int)slots.size();
        std::vector<int> q_start(S), pos0(S);
        int T = 0;
        for (int i = 0; i < S; ++i) {
            q_start[i] = T;
            pos0[i] = i < S_real ? length(slots[i]) : 0;
            if (counts[i] < 1) throw CacheError(cat("slot ", slots[i], ": an entry needs at least one token"));
            T += counts[i];
        }
        if ((int)tokens.size() != T) throw CacheError(cat("the step has ", T - pad_rows, " rows but ", tokens_in.size(), " tokens"));
        std::vector<std::pair<std::string, std::vector<int32_t>>> sections;
        auto add = [&](const std::string& name, std::vector<int32_t> v) { sections.emplace_back(name, std::move(v)); };
        if (axes < 1) throw CacheError(cat("positions have ", axes, " axes"));
        if (!explicit_positions.empty() && explicit_positions.size() != (size_t)T_real * axes)
            throw CacheError(cat("positions given for ", explicit_positions.size(), " numbers, the step has ", T_real, " rows of ", axes));
        std::vector<int32_t> positions((size_t)T * axes);
        for (int i = 0; i < S; ++i)
            for (int j = 0; j < counts[i]; ++j)
                for (int a = 0; a < axes; ++a) positions[(size_t)(q_start[i] + j) * axes + a] = pos0[i] + j;
        std::copy(explicit_positions.begin(), explicit_positions.end(), positions.begin());
        add("tokens", std::vector<int32_t>(tokens.begin(), tokens.end()));
        add("positions", positions);
        add("seq_q_start", std::vector<int32_t>(q_start.begin(), q_start.end()));
        add("seq_q_len", std::vector<int32_t>(counts.begin(), counts.end()));
        add("seq_pos0", std::vector<int32_t>(pos0.begin(), pos0.end()));
        add("seq_slot", std::vector<int32_t>(slots.begin(), slots.end()));
        add("want_rows", std::vector<int32_t>(want_rows.begin(), want_rows.end()));
        py::dict widths;
        for (size_t gi = 0; gi < groups_.size(); ++gi) {
            const Group& g = groups_[gi];
            int width = 1;
            for (int i = 0; i < S_real; ++i) width = std::max(width, (int)g.tables.at(slots[i]).size());
            for (int i = S_real; i < S; ++i) width = std::max(width, (counts[i] + page_size_ - 1) / page_size_);
            if (table_multiple > 1) width = (width + table_multiple - 1) / table_multiple * table_multiple;
            std::vector<int32_t> table((size_t)S * width, -1), slot_map(T);
            for (int i = S_real; i < S; ++i) {  // rows that belong to nobody: every page is the scratch page
                for (int p = 0; p * page_size_ < counts[i]; ++p) table[(size_t)i * width + p] = scratch_page((int)gi);
                for (int j = 0; j < counts[i]; ++j) slot_map[q_start[i] + j] = scratch_page((int)gi) * page_size_ + j % page_size_;
            }
            for (int i = 0; i < S_real; ++i) {
                const auto& t = g.tables.at(slots[i]);
                std::copy(t.begin(), t.end(), table.begin() + (size_t)i * width);
                for (int j = 0; j < counts[i]; ++j) {
                    const int pos = pos0[i] + j, lp = pos / page_size_;
                    if (lp >= (int)t.size() || t[lp] < 0)
                        throw CacheError(cat("group ", g.name, ": slot ", slots[i], " writes position ", pos, " into a page it does not hold"));
                    slot_map[q_start[i] + j] = t[lp] * page_size_ + pos % page_size_;
                }
            }
            add("table/" + g.name, std::move(table));
            add("slot_map/" + g.name, std::move(slot_map));
            widths[py::str(g.name)] = width;
        }
        // Blocks of rows for the attention kernels, those with the longest contexts first: a block's
        // work grows with the keys its last row sees, and the kernel spreads the blocks over the chip
        // by their place in this order.
        for (int hk : heads_per_kv) {
            struct Item { int keys, seq, r0; };
            std::vector<Item> items;
            for (int i = 0; i < S; ++i)
                for (int r0 = 0; r0 < counts[i] * hk; r0 += rows_per_block)
                    items.push_back({pos0[i] + std::min(counts[i], (r0 + rows_per_block + hk - 1) / hk), i, r0});
            std::stable_sort(items.begin(), items.end(), [](const Item& a, const Item& b) { return a.keys > b.keys; });
            std::vector<int32_t> work;
            work.reserve(items.size() * 2);
            for (const Item& it : items) {
                work.push_back(it.seq);
                work.push_back(it.r0);
            }
            if (fill_rows > 0) {  // as many items as any step of this size can have; the kernel skips request -1
                const size_t most = (size_t)(fill_rows * hk + rows_per_block - 1) / rows_per_block + fill_seqs;
                while (work.size() < 2 * most) {
                    work.push_back(-1);
                    work.push_back(0);
                }
            }
            add("work/" + std::to_string(hk), std::move(work));
        }
        size_t total = 0;
        py::dict offsets;
        for (auto& s : sections) {
            offsets[py::str(s.first)] = py::make_tuple(total, s.second.size());
            total += (s.second.size() + 3) / 4 * 4;
        }
        py::array_t<int32_t> buf(std::max<size_t>(total, 4));
        auto* p = buf.mutable_data();
        std::fill(p, p + buf.size(), 0);
        size_t off = 0;
        for (auto& s : sections) {
            std::copy(s.second.begin(), s.second.end(), p + off);
            off += (s.second.size() + 3) / 4 * 4;
        }
        return py::make_tuple(buf, offsets, widths);
    }

private:
    int page_size_;
    SlotPool slots_;
    std::map<int, int> lengths_;
    std::vector<Group> groups_;
};

}  // namespace mshost
