// Which fused kernel for which problem: estimated durations of the kernel families, in microseconds.
//
// The families differ in how they spread the work, not in what they compute, so the choice is a matter of time only:
//   four-tile     one workgroup per unit (four state tiles sharing B) walks the whole sequence with the state in its
//                 accumulators: nothing is read back and nothing waits, but a unit is one compute unit's work;
//   token-split   one workgroup per tile, four waves splitting every chunk's tokens: the shortest chunk when tiles
//                 are scarce, four times the B traffic;
//   pair          a chunk-state launch over (unit, run of chunks) that fills every compute unit, then the streaming
//                 recurrence over what it wrote: three more passes over the states;
//   chain         work items of R chunks of a unit drawn from a ticket counter, linked by flags: fills every compute
//                 unit whatever the number of units, pays a start, a read-back per item and a link per item.
// The formulas are fits to one sweep of 36 shapes around the benchmark configurations (batch 1 - 32, 512 - 65 536
// tokens, 24 - 128 heads, dstate 64 / 128, chunk 128 / 256, 1 / 8 groups, with and without packed sequences) on an
// MI355X at steady clocks; every quantity is per compute unit, so another compute-unit count rescales them.  They
// are good to about 10 %, which is enough to rank the families; tests/test_cost_model_cpu.py holds the sweep and a
// second one of 18 other shapes that the fit has not seen, and checks that the family picked is never more than a few
// per cent slower than the best one the dispatcher could have picked.
// The constants (microseconds per unit-chunk, per link, the 5 TB/s of the streaming pair) are this one device's: an
// MI355X with 256 compute units in 8 XCDs of 32 at its steady clocks.  Another compute-unit count rescales them
// linearly and nothing has been measured at any other value; another part needs its own sweep.
#pragma once

#include <stdint.h>

namespace ssd {
namespace cost {

struct Problem {
    int64_t units;      // groups of four state tiles (32 headdim rows x dstate) that share (batch, group)
    int chunks;         // chunks per sequence
    int chunk_size, dstate;
    int n_cu;           // compute units of the device
};

// Time of one unit-chunk relative to dstate 128, chunk 256: the part that shrinks with the tile (arithmetic, x and B
// traffic) and the part that does not (per-chunk bookkeeping, the state's way out).  dstate 64: 0.71 measured, chunk
// 128: 0.75.
inline double work(const Problem &q) { return 0.45 + 0.55 * (q.dstate / 128.0) * (q.chunk_size / 256.0); }

inline int64_t ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }

// Chain kernel with R chunks per item.  Throughput: a compute unit takes an item after the other, 8 us per unit-chunk
// at R = 4 (more links and read-backs per chunk below that), and the launch ends with its fullest compute unit, whose
// last item nothing overlaps; 15 us of start and drain.  Latency: the items of a unit form a chain whose links
// (flag, read-back, recurrence, store, acknowledge: 3 us) follow one another however many compute units there are.
inline double chain_us(const Problem &q, int R)
{
    const int64_t items_per_unit = ceil_div(q.chunks, R);
    const double per_item = (double)q.chunks / (double)items_per_unit;       // chunks of an average item
    const double items_per_cu = (double)(q.units * items_per_unit) / q.n_cu;
    const double rounds = (double)ceil_div(q.units * items_per_unit, q.n_cu);
    const double t_chunk = (R >= 4 ? 8.0 : R == 2 ? 8.4 : 10.0) * work(q);
    const double throughput = 15.0 + t_chunk * per_item * (items_per_cu > 0.95 * rounds ? items_per_cu : 0.95 * rounds);
    const double latency = 3.0 * (double)items_per_unit + t_chunk * per_item;
    return throughput > latency ? throughput : latency;
}

// The best R of {4, 2, 1} for the chain kernel, and its estimate.
inline int chain_chunks_per_item(const Problem &q, double *us)
{
    int best = 4;
    double t = chain_us(q, 4);
    for (int R = 2; R >= 1; --R) {
        const double c = chain_us(q, R);
        if (c < 0.97 * t) { t = c; best = R; }      // fewer links unless the gain is clear
    }
    if (us) *us = t;
    return best;
}

// Four-tile kernel: a wave walks its tile's chunks one after the other, 4.7 us each on an otherwise idle device and
// 7.1 us when every compute unit has a workgroup; beyond that workgroups share compute units and take turns at
// their instruction issue, and the launch lasts as long as the compute unit with the most of them.
inline double four_tile_us(const Problem &q)
{
    const double k = (double)q.units / q.n_cu;
    const double most = (double)ceil_div(q.units, q.n_cu);
    const double t_chunk = k <= 1.0 ? 4.7 + 2.4 * k : 7.1 * (1.0 + 0.95 * (most - 1.0) + 0.3 * (k - 1.0));
    return 4.0 + q.chunks * t_chunk * work(q);
}

// Token-split kernel: 2.35 us per chunk while every workgroup (one per tile) has a compute unit of its own; with w
// workgroups per compute unit 1.6 times that up to w = 1.5 and a further 1.1 times per workgroup beyond.  (Measured up
// to 32 chunks; longer sequences run about a third slower per chunk, but there this family is not a candidate.)
inline double token_split_us(const Problem &q)
{
    const double w = 4.0 * (double)q.units / q.n_cu;
    const double share = w <= 1.0 ? 1.0 : 1.6 + (w > 1.5 ? 1.1 * (w - 1.5) : 0.0);
    return 3.5 + q.chunks * 2.35 * share * work(q);
}

// Chunk-state launch + recurrence: x read and the chunk states written, then read, and the passed states written
// (read and write share the bandwidth: about 5 TB/s over the lot).
inline double pair_us(const Problem &q)
{
    const double x_bytes = (double)q.units * q.chunks * 256.0 * q.chunk_size;       // 4 tiles x 32 rows x Q x bf16
    const double s_bytes = (double)q.units * q.chunks * 512.0 * q.dstate;           // 4 tiles x 32 rows x N x fp32
    return 6.0 + (x_bytes + 3.0 * s_bytes) / 5.0e6 * (256.0 / q.n_cu);
}

}  // namespace cost
}  // namespace ssd
