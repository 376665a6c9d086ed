// engine/sequence_model.h -- what the engine, the trace runner and the C API need from a model family, and the registry that picks the family.
//
// A family registers a factory under the "architecture" string of its config.json (a static FamilyRegistrar in its .cpp).  open_model(path) reads
// that string and builds the object; GGUF files stay with nt::Model (engine/model.h), which the engine holds directly.
// A SequenceModel owns its weights and a slot cache: every live sequence holds one slot, tokens are appended with forward() in portions of any size,
// and a released slot is handed to the next sequence as it is (nothing a sequence reads lies beyond its own length; what a slot holds besides rows per
// position -- a recurrent state, the last inputs of a convolution -- is not read by a sequence's first token).
#pragma once
#include <cstdint>
#include <functional>
#include <memory>
#include <string>
#include <vector>

namespace nt {

struct SeqModelInfo {
    std::string architecture;
    int vocab = 0, width = 0, n_layers = 0, n_layer_runs = 0, max_context = 0;
    int bos = -1, eos = -1;          // -1: the model folder names none
};

struct SeqLoadOptions {
    int max_context = 4096;          // positions a slot can hold
    int slots = 1;                   // sequences alive at once
    bool float32 = false;            // every product in true F32 (weights widened at load) instead of bf16 products with F32 sums
};

class SequenceModel {
public:
    virtual ~SequenceModel() {}
    virtual int load(const std::string& dir, const SeqLoadOptions& opt) = 0;
    virtual const SeqModelInfo& info() const = 0;
    virtual const std::string& error() const = 0;
    virtual uint64_t weight_bytes() const = 0;
    // ---- the slot cache
    virtual int acquire_slot() = 0;                 // slot id >= 0 (length 0), or NTK_E_NOMEM when all are taken
    virtual int release_slot(int slot) = 0;
    virtual int slot_length(int slot) const = 0;    // positions the slot holds, negative if it is not live
    virtual int truncate_slot(int slot, int length) = 0;   // forget everything from position `length` on (a family with recurrent state: only back to 0 or not at all)
    // ---- the step: append `n` tokens to `slot`; the logits of the tokens want[0 .. n_want) (indices into this portion) are left on the device,
    //      [n_want][vocab] F32, and returned (stream ordered: sync() or copy_logits() before the host reads).  nullptr on failure.
    virtual float* forward(int slot, const int* tokens, int n, const int* want, int n_want) = 0;
    virtual int copy_logits(float* host, int rows) = 0;    // blocking copy of the last forward's rows
    // residual stream after every layer run of the LAST forward portion, [layer runs][n][width] (host); only while debug capture is on
    virtual int set_capture(bool on) = 0;
    virtual int copy_capture(float* host) = 0;
    virtual int sync() = 0;
    virtual void* stream() const = 0;
};

using FamilyFactory = std::function<std::unique_ptr<SequenceModel>()>;
struct FamilyRegistrar { FamilyRegistrar(const char* architecture, FamilyFactory make); };
// the families linked into this binary
std::vector<std::string> registered_families();
// nullptr (and *why) if the path is not a model folder or its architecture has no family here
std::unique_ptr<SequenceModel> make_family(const std::string& architecture);
std::unique_ptr<SequenceModel> open_model(const std::string& path, const SeqLoadOptions& opt, std::string* why);

// The slot cache: `slots` regions of `capacity` positions; a live slot has a length.  Device memory belongs to the model (per layer run: cache rows
// [slots][capacity][row], and per slot whatever state its mixers carry); this class is the bookkeeping every family shares.
class SlotTable {
public:
    void reset(int slots, int capacity) { len_.assign((size_t)slots, -1); cap_ = capacity; }
    int slots() const { return (int)len_.size(); }
    int capacity() const { return cap_; }
    int acquire() {
        for (size_t i = 0; i < len_.size(); ++i)
            if (len_[i] < 0) { len_[i] = 0; return (int)i; }
        return -1;
    }
    bool live(int s) const { return s >= 0 && s < (int)len_.size() && len_[(size_t)s] >= 0; }
    int length(int s) const { return live(s) ? len_[(size_t)s] : -1; }
    bool release(int s) { if (!live(s)) return false; len_[(size_t)s] = -1; return true; }
    bool set_length(int s, int n) { if (!live(s) || n < 0 || n > cap_) return false; len_[(size_t)s] = n; return true; }

private:
    std::vector<int> len_;
    int cap_ = 0;
};

}  // namespace nt
