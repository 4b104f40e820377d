// Shape of the coefficient slabs of the straight-line contraction kernel (smx_kernels_poly.hip): shared by the loader,
// which lays the coefficients out, and the launcher.  No device code: a host compiler can include this file.
#pragma once

#include "smx_poly_tables.inc"

namespace smx {

// Coefficient slabs of the straight-line contraction kernel.  The monomials of polynomials 0..NP-1 follow one another,
// each list padded with zero coefficients to a multiple of four; a slab holds them for one species and CB channels
// as [monomial / V][CB][V], V = 16 / sizeof(F): a thread reads V coefficients of its channel with one 16-byte LDS
// read, the lanes of a wavefront side by side.  The loader lays the coefficients out with the same function.
constexpr int poly_spec_padded(int n) { return (n + 3) / 4 * 4; }
constexpr int poly_spec_offset(int lm)   // padded monomials in front of polynomial lm (lm = NP: all of them)
{
    int o = 0;
    for (int q = 0; q < lm && q < kPolyTables; ++q) o += poly_spec_padded(kPolyTableLen[q]);
    return o;
}
struct PolySpecShape {
    int CB, AG, kblocks;      // channels per block, atoms per pass (AG * CB <= 256 threads), blocks per channel axis
    int blocks_per_cu;        // resident blocks the LDS and the registers allow
    unsigned slab_bytes;      // poly_spec_offset(NP) * CB * sizeof(F)
};
inline PolySpecShape poly_spec_shape(int elem, int K, int NP)
{
    const int Kpad = (K + 15) / 16 * 16, mono = poly_spec_offset(NP);
    const int reg_blocks = elem == 8 ? 4 : 5;   // 256-thread blocks per CU within the register file (128 / 96 registers)
    // Channel blocks of at least 128 bytes per atom row are preferred; narrower ones are taken when no such block
    // fits, or when it would leave one block per CU where narrower blocks leave several.
    PolySpecShape best[2] = {};
    long best_score[2] = {-1, -1};
    for (int pass = 0; pass < 2; ++pass)
        for (int CB = 16; CB <= 128 && CB <= Kpad; CB += 16) {
            if (Kpad % CB != 0 || (pass == 0 && CB * elem < 128 && CB < Kpad)) continue;
            const long slab = (long)mono * CB * elem;
            int blocks = (int)(160 * 1024 / slab);
            if (blocks < 1) continue;
            if (blocks > reg_blocks) blocks = reg_blocks;
            const int AG = 256 / CB;
            const long score = (long)blocks * AG * CB;
            if (score >= best_score[pass]) {
                best_score[pass] = score;
                best[pass] = PolySpecShape{CB, AG, Kpad / CB, blocks, (unsigned)slab};
            }
        }
    if (best_score[0] < 0 || (best[0].blocks_per_cu == 1 && best[1].blocks_per_cu > 1)) return best[1];
    return best[0];
}

}  // namespace smx
