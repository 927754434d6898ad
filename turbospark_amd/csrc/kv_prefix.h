// The token ids the KV rows were built from (crates/runtime/src/kv_prefix.rs:49-137): pure host
// state beside the cache cursor.  Invariant: fed[0..len) are exactly the ids behind positions
// [0, len), in order; a state that took in anything the ids do not describe is tainted and is
// never offered for reuse.
#pragma once
#include <algorithm>
#include <cstdint>
#include <vector>

struct tsv_prefix {
    std::vector<int32_t> fed;
    bool tainted = false;

    // clear(): paired with whatever empties the cache itself (kv_prefix.rs:60-63)
    void clear() {
        fed.clear();
        tainted = false;
    }
    // taint(): sticky until clear() (:68-70)
    void taint() { tainted = true; }
    // record(tokens, pos0) (:79-92): a write that starts inside the record replaces its tail (a
    // rewind is describable); one that starts past its end leaves a gap nobody can name, so the
    // record is dropped and tainted rather than padded.
    void record(const int32_t* tokens, int64_t n, int64_t pos0) {
        const int64_t len = (int64_t)fed.size();
        if (pos0 != len) {
            if (pos0 >= 0 && pos0 < len) {
                fed.resize((size_t)pos0);
            } else {
                fed.clear();
                tainted = true;
                return;
            }
        }
        if (n > 0) fed.insert(fed.end(), tokens, tokens + n);
    }
    // rewind_to(position) (:96-100): longer than the record is a no-op
    void rewind_to(int64_t position) {
        if (position >= 0 && position < (int64_t)fed.size()) fed.resize((size_t)position);
    }
    // untainted_len() (:104-106): -1 stands for None
    int64_t untainted_len() const { return tainted ? -1 : (int64_t)fed.size(); }
    // common_prefix(prompt) (:129-137): the longest common prefix, capped one below the prompt's
    // length so that at least one token is always left to feed.
    int64_t common_prefix(const int32_t* prompt, int64_t n) const {
        if (tainted || fed.empty() || n <= 0) return 0;
        const int64_t ceiling = std::min<int64_t>((int64_t)fed.size(), n - 1);
        int64_t i = 0;
        while (i < ceiling && fed[(size_t)i] == prompt[i]) i++;
        return i;
    }
};
