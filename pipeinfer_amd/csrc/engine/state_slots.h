// Host-side table of recurrent-state slots: which slot of the per-layer state arrays belongs to which sequence.
//
// The companion of kv_cells for mixers that carry a fixed-size state from token to token instead of one cache cell per token: a sequence owns one slot from its first
// token until it is removed; a slot that is handed out again starts from a zero state (the first run that uses it is told so, nothing is cleared in between).
#pragma once

#include <cstdint>
#include <vector>

namespace pi {

class state_slots {
public:
    explicit state_slots(int n_slots) : owner_(n_slots, -1), fresh_(n_slots, 0), last_(n_slots, -1) {}
    int  size() const { return (int) owner_.size(); }
    int  used() const { int n = 0; for (int o : owner_) n += o >= 0; return n; }
    int  find(int seq) const { for (int i = 0; i < size(); i++) if (owner_[i] == seq) return i; return -1; }
    // the slot of `seq`, allotted now if it has none (-1: every slot is taken)
    int  acquire(int seq) {
        int s = find(seq);
        if (s >= 0) return s;
        for (int i = 0; i < size(); i++) if (owner_[i] < 0) { owner_[i] = seq; fresh_[i] = 1; last_[i] = -1; return i; }
        return -1;
    }
    // true once per allotment: the caller's next run must start the slot's state from zero
    bool take_fresh(int slot) { const bool f = fresh_[slot] != 0; fresh_[slot] = 0; return f; }
    void mark_fresh(int slot) { fresh_[slot] = 1; }                 // (a run that was told so could not be started)
    bool is_fresh(int slot) const { return fresh_[slot] != 0; }
    void release(int seq) { const int s = find(seq); if (s >= 0) { owner_[s] = -1; fresh_[s] = 0; } }
    void keep(int seq) { for (int i = 0; i < size(); i++) if (owner_[i] != seq) { owner_[i] = -1; fresh_[i] = 0; } }
    void clear() { for (int i = 0; i < size(); i++) { owner_[i] = -1; fresh_[i] = 0; } }
    int  owner(int slot) const { return owner_[slot]; }
    // the last token the slot's sequence was fed (-1: none yet): models whose embedding looks at the previous token
    int  last_token(int slot) const { return last_[slot]; }
    void set_last_token(int slot, int token) { last_[slot] = token; }
private:
    std::vector<int32_t> owner_;
    std::vector<uint8_t> fresh_;
    std::vector<int32_t> last_;
};

}  // namespace pi
