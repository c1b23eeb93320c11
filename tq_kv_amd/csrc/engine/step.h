// What one step knows about its batch, on the host and on the device.
//
// A step runs the tokens it is given as one packed batch: the tokens of sequence 0, then of
// sequence 1, and so on.  For each token the device knows which sequence of the step it
// belongs to and its absolute position; for each sequence its slot, how many positions the
// cache held before the step and how many tokens it brings; for each group of the cache the
// page table of the step's sequences.  All of it is laid out by tqe_plan_step as one int32
// array and uploaded in one copy.
#pragma once
#include <map>
#include <vector>

#include "core.h"

struct tqe_cache;

namespace tq {

struct StepArrays {
    const int32_t* tokens = nullptr;
    const int32_t* tok_seq = nullptr;
    const int32_t* tok_pos = nullptr;
    const int32_t* seq_slot = nullptr;
    const int32_t* seq_start = nullptr;
    const int32_t* seq_new = nullptr;
    const int32_t* cu = nullptr;
    const int32_t* want_rows = nullptr;
    const int32_t* last_rows = nullptr;
    const int32_t* want_in_last = nullptr;
    const int32_t* last_seq = nullptr;
    const int32_t* last_pos = nullptr;
};

struct Tiles {
    const int32_t* seq = nullptr;
    const int32_t* tok0 = nullptr;
    const int32_t* count = nullptr;
    int n = 0;
};

struct StepShape {
    int n_tokens, n_seqs, n_want;
    std::vector<int> widths;
    bool operator<(const StepShape& o) const {
        if (n_tokens != o.n_tokens) return n_tokens < o.n_tokens;
        if (n_seqs != o.n_seqs) return n_seqs < o.n_seqs;
        if (n_want != o.n_want) return n_want < o.n_want;
        return widths < o.widths;
    }
};

struct StepContext {
    // what runs the step
    hipStream_t stream = nullptr;
    Workspace* ws = nullptr;
    Staging* staging = nullptr;
    int act_dtype = BF16;

    // the batch
    int n_seqs = 0, n_tokens = 0, n_want = 0, n_last = 0, max_new = 0, max_end = 0;
    bool all_decode = false, prune_last = false;
    bool capturing = false;                          // the step is being recorded into a graph: nothing may be uploaded
    bool fuse_small = false, fuse_mid = false;       // set by the model from what parts/linear says of the step
    std::vector<int32_t> packed;                     // the host copy
    StepArrays host, dev;
    int32_t* flat = nullptr;                         // the device copy (workspace, or a captured graph's own buffer)
    size_t flat_count = 0;
    struct Table { const int32_t* host = nullptr; const int32_t* dev = nullptr; int width = 0; };
    std::vector<Table> tables;                       // one page table [n_seqs][width] per group of the cache
    std::vector<int32_t> lens;

    // Lays the step out.  cache may be null (then starts must be given and there are no page
    // tables).  Nothing is uploaded yet.
    void plan(const tqe_cache* cache, int n_seqs, const int32_t* slots, const int32_t* starts, const int32_t* n_new,
              const int32_t* tokens, const int32_t* want_counts, const int32_t* want_idx, int width_step);
    // Copies the arrays to the device: into `into` (a buffer of flat_count values that a captured
    // graph reads) or into workspace memory.
    void upload(int32_t* into = nullptr);
    StepShape shape() const;

    // The step's tokens cut into tiles of up to `tile` consecutive queries of one sequence
    // (sequence of the step, first packed token, number of queries), on the device, longest
    // reach first; built and uploaded when a mixer first asks for this size.
    Tiles query_tiles(int tile);
    // The same for the step's last_rows, in their own numbering.
    Tiles last_tiles(int tile);

    Tensor alloc(int dtype, std::initializer_list<int64_t> dims) { return ws->tensor(dtype, dims); }

    // scratch of the model for a step whose last block goes on with a few rows
    std::unique_ptr<struct Stream> sub_stream;
    std::map<std::string, int> memo;                 // what parts remember for the length of a step (the prompt kernel's tile)

    StepContext();
    ~StepContext();
private:
    std::map<std::pair<int, int>, Tiles> tiles_;
    Tiles upload_tiles(std::vector<int32_t>& seq, std::vector<int32_t>& tok0, std::vector<int32_t>& count, const std::vector<long long>& reach);
    void carve(StepArrays& out, const int32_t* base, const int32_t* meta);
    int32_t meta_[TQE_META_SIZE];
};

}  // namespace tq
