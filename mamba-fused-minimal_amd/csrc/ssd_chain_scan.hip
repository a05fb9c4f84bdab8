// The instantiations of the ticket / flag-chain kernel (ssd_chain_kernel.h) whose chain step also consumes the passed
// states: y (+)= exp(dA_cumsum) [same sequence] C . (state entering the chunk), the state-dependent half of the chunk
// scan (kernels/ssd_chunk_scan.py:94-117), computed while a wave holds that state in registers -- with `out` absent the
// passed states never reach memory beyond one fp32 slot per state tile and work item.  A translation unit of its own so
// that the two families of instantiations compile side by side.
#include "ssd_chain_kernel.h"

namespace ssd {

// Work items are two chunks long: with four, the states entering the chunks (256 registers with dstate 128), the bf16
// hi + lo operands of one of them (64) and what the step loop keeps across the chain step do not fit the 512 registers
// of a wave (chain_chunks_per_item says so to the launch plan).
template <bool SEQ, bool LOCAL, int OUTM>
static hipError_t launch_scan_r(const Params &p, int n_wg, hipStream_t s)
{
    const int nt = p.dstate / 16, spc = p.Q / 32;
    if (nt == 8 && spc == 8) return chain::launch_kernel<8, 8, 2, SEQ, LOCAL, OUTM, true>(p, n_wg, s);
    if (nt == 8 && spc == 4) return chain::launch_kernel<8, 4, 2, SEQ, LOCAL, OUTM, true>(p, n_wg, s);
    if (nt == 4 && spc == 8) return chain::launch_kernel<4, 8, 2, SEQ, LOCAL, OUTM, true>(p, n_wg, s);
    return chain::launch_kernel<4, 4, 2, SEQ, LOCAL, OUTM, true>(p, n_wg, s);
}

template <bool SEQ, bool LOCAL>
static hipError_t launch_scan_t(const Params &p, int n_wg, hipStream_t s)
{
    return p.out ? launch_scan_r<SEQ, LOCAL, 0>(p, n_wg, s) : launch_scan_r<SEQ, LOCAL, 2>(p, n_wg, s);
}

hipError_t launch_chain_scan(const Params &p, int r, bool local, int n_wg, hipStream_t s)
{
    if (r != 2 || !p.y || !p.Cm || (p.out && p.dt_out != DT_F32)) return hipErrorInvalidValue;
    if (p.seq) return local ? launch_scan_t<true, true>(p, n_wg, s) : launch_scan_t<true, false>(p, n_wg, s);
    return local ? launch_scan_t<false, true>(p, n_wg, s) : launch_scan_t<false, false>(p, n_wg, s);
}

}  // namespace ssd
