// Arguments of the tiled Newton-Schulz GEMM (ns_fast.hip), shared with the entry point in ns.hip.
#pragma once
#include "common.hpp"

namespace viola {

struct NsArgs {
    const uint16_t* a;          // [batch, m, k]
    const uint16_t* b;          // [batch, n, k], or [batch, k, n] when b_kn
    const uint16_t* residual;   // [batch, m, n] or null
    uint16_t* out;              // [batch, m, n]
    uint16_t* out_diag;         // second copy with add_diag on the diagonal, or null
    int64_t batch, m, n, k;
    float add_diag;
    int transpose_out;          // store out (and out_diag) as [batch, n, m]
    int symmetric;              // b == a, m == n: compute tiles with tn >= tm only and mirror them
    int tiles_m, tiles_n;
    int group_m;                // tile rows per band of the work order (ns_fast.hip)
    int64_t tiles;              // batch * tiles_m * tiles_n
};

// Tile shapes of the tiled kernel (rows x columns of output per block); NS_TILE_GENERIC is the kernel in ns.hip that
// takes every shape the tiled one refuses.
enum NsTile { NS_TILE_GENERIC = 0, NS_TILE_64x64 = 1, NS_TILE_128x64 = 2, NS_TILE_128x128 = 3, NS_TILE_192x192 = 4, NS_TILE_384x192 = 5 };
NsTile ns_choose_tile(int64_t batch, int64_t m, int64_t n, bool symmetric);
bool ns_fast_takes(const NsArgs& args);

// Launches the tiled kernel when the shape qualifies (16-byte aligned rows, k and n multiples of 8,
// one matrix below 2 GiB); returns false without launching otherwise.
bool launch_ns_gemm_fast(const NsArgs& args, bool is_bf16, bool b_kn, int epilogue, hipStream_t stream);

}  // namespace viola
