// Host-side check of the slab shapes the contraction kernel and the loader agree on: every channel count and every
// number of polynomials must give a shape the kernel can run (prints one line per case; the caller asserts).
#include "smx_poly_shape.hpp"

#include <cstdio>
#include <initializer_list>

int main()
{
    int bad = 0;
    for (int elem : {4, 8})
        for (int NP : {1, 4, 9})
            for (int K = 1; K <= 512; ++K) {
                const smx::PolySpecShape sh = smx::poly_spec_shape(elem, K, NP);
                const int Kpad = (K + 15) / 16 * 16;
                const bool ok = sh.CB > 0 && sh.CB % 16 == 0 && sh.CB <= 128 && Kpad % sh.CB == 0 && sh.kblocks * sh.CB == Kpad &&
                                sh.AG >= 1 && sh.AG * sh.CB <= 256 && sh.blocks_per_cu >= 1 &&
                                sh.slab_bytes == (unsigned)(smx::poly_spec_offset(NP) * sh.CB * elem) && sh.slab_bytes % 16 == 0 &&
                                (long)sh.slab_bytes * sh.blocks_per_cu <= 160L * 1024;
                if (!ok) { ++bad; std::printf("BAD elem %d NP %d K %d: CB %d AG %d kblocks %d blocks %d slab %u\n", elem, NP, K, sh.CB, sh.AG, sh.kblocks, sh.blocks_per_cu, sh.slab_bytes); }
                if (K == 96 || K == 128)
                    std::printf("elem %d NP %d K %d: CB %d AG %d kblocks %d blocks %d slab %u\n", elem, NP, K, sh.CB, sh.AG, sh.kblocks, sh.blocks_per_cu, sh.slab_bytes);
            }
    std::printf("offsets %d %d %d\n", smx::poly_spec_offset(1), smx::poly_spec_offset(4), smx::poly_spec_offset(9));
    return bad ? 1 : 0;
}
