// Launches over tiny tensors collected into one.
//
// A decode step spends a dozen launches on tensors of a few hundred elements (a position turned into
// rotary tables, scatter indices, a mask): each costs a launch and a trip to memory for operands the
// kernel before it has just written, however little it computes. While a batch is collecting on a
// stream, the entry points of the broadcast binary ops, the contiguous maps, Cast, Where, Expand and
// Concat hand such calls over as records instead of launching them; one block then runs the records
// (records that do not touch each other's data side by side on the block's wavefronts, a barrier
// where one reads or overwrites what an earlier one wrote), with the same element functors as the
// kernels they replace.
// Anything else issued on the stream (as_stream, common.hpp) sends the collected records out first,
// so the order of effects on the stream is the order of the calls.
#pragma once

#include "common.hpp"

namespace rmlk {

// Output elements of an operator that may be collected: what one block gets through in a few trips.
// (At 4096 the collected launch of a 512-token prefill, four integer operators of that size, took
// 22 us for work that 3 us kernels of several blocks each had done.)
constexpr int64_t kBatchMaxElems = 1024;
constexpr int kBatchMaxOps = 24;           // records of one launch (they travel as kernel arguments)
constexpr int kBatchMaxRank = 4;           // dims of a record after coalescing

enum SmallKind : int32_t { kSmallBinary = 0, kSmallUnary, kSmallCast, kSmallWhere, kSmallCopy };

struct SmallOp {
    int32_t kind;
    int32_t op;              // rmlk_binary_op / rmlk_unary_op
    int32_t dt, dt2;         // element type (Cast: source, destination; Where / copy: element size in dt)
    int32_t n, rank;
    // set when the batch goes out: the record's place among the records that may run side by side
    // (none of them touches what another writes), and whether the block meets after it
    int32_t group_size, group_index, sync, reserved;
    int32_t dim[kBatchMaxRank];
    int32_t st[4][kBatchMaxRank];   // element strides of in[0..2] and of out
    const void *in[3];
    void *out;
};

// Fills n, rank, dim and st of `op` from a shape and the element strides of `n_in` inputs followed
// by the output's (strides[n_in]); dims of 1 are dropped and dims that every operand walks as one
// run are merged. False when the result does not fit a record.
bool small_op_layout(SmallOp &op, int rank, const int64_t *shape, int n_in, const int64_t (*strides)[kMaxRank]);

// True: the record was taken and will run with the stream's batch. False: no batch is collecting
// on `s`; the caller launches the work itself.
bool batch_take(hipStream_t s, const SmallOp &op);

inline bool batch_collecting() { return g_open_batches.load(std::memory_order_relaxed) > 0; }

}  // namespace rmlk
