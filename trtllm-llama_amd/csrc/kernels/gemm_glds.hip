// MFMA GEMM for prefill-shaped problems, LDS-DMA staged:  C[m,n] = epi( sum_k A[m,k] * W[n,k] )   (W_INT8_SQ, W_FP16)
//
// Both operands are row-major with K contiguous (activations [M][K], weights [N][K]), so one staging scheme serves
// both: a K-tile is 128 BYTES of every tile row (128 int8 | 64 fp16), brought HBM/L2 -> LDS by
// `global_load_lds_dwordx4` (no VGPR round trip, no ds_write pass), double-buffered, ONE barrier per K-tile: the DMA of
// tile t+1 is in flight while the MFMAs of tile t run.
//
// LDS image: [row][128 B], 16-byte column index XOR-swizzled with (row >> 1) & 7 so that the 16 lanes of a
// ds_read_b128 phase (16 consecutive rows, same k-chunk) hit 16 different 16-byte bank groups.  The DMA writes LDS
// lane-linearly (wave-uniform base + lane * 16), so the swizzle is applied to the per-lane GLOBAL source address: the
// 8 lanes of a row read the 8 pieces of that row's 128-byte line in permuted order - still one full line per row.
//
// MFMA: v_mfma_i32_32x32x32_i8 (exact int32) / v_mfma_f32_32x32x16_f16 - identical byte geometry (a k-step is 32
// bytes, lane l holds row l & 31, bytes [16 * (l >> 5), +16)).  Tile shapes are template parameters (waves WM x WN,
// each wave MT x NT MFMA tiles); the launcher picks the shape that fills the 256 CUs best for the problem
// (M = 1024 prefill shapes are one to three workgroup rounds: tile quantisation matters as much as the inner loop).
//
// Epilogue: per-column x per-row scales exactly as the reference's epilogue_per_row_per_col_scale.h:279-347
// (float(acc) * (s_col * s_row)), transposed through LDS so that every lane stores 16 contiguous bytes of a C row.
#include "dev_utils.h"
#include "gemm_glds_impl.h"
#include "kernels.h"
#include "launch_util.h"
#include <atomic>
#include <map>

namespace tllm
{
namespace kernels
{
using namespace dev;

int gemm_tune_cfg = 0; // test/bench override of the tile shape (0 = heuristic)
int launch_gemm_sqp(const GemmParams& p, int cfg, hipStream_t stream); // gemm_sqp.hip: phased SmoothQuant kernel, ids 13..
int launch_gemm_f16p(const GemmParams& p, int cfg, hipStream_t stream); // gemm_sqp.hip: the same pipeline on fp16 operands, ids 50..
extern void* gemm_clock_probe;                                              // gemm_sqp.hip (microbench hook)

namespace
{

// production tile shapes: id -> (BM, BN); the ids index launch_wt's table, the other ids there are the measured
// alternatives kept for the microbench sweep (prefill GEMM)
struct Shape
{
    int id, bm, bn;
    // measured time per (workgroup round x tile area), relative to the phased 256 x 192 tile of the same operand type.  fp16:
    // profiles/r04_tile256x128.txt.  SmoothQuant (r05): relative to the PERSISTENT 256 x 192 tile (profiles/r05_sqgemm_persistent.txt:
    // O at M = 8192 117 us against 135 for 256 x 256 in two rounds, O at M = 4096 63 us for 256 x 128 against 69)
    double f, f_sq;
};
// id 42 is the phased 256 x 128 tile of gemm_sqp.hip (its fp16 sibling is id 54): it has no lock-step form in this file
constexpr int kPhased256x128 = 42;
constexpr Shape kShapes[] = {{8, 128, 128, 1.40, 1.80}, {6, 256, 192, 1.0, 1.0}, {2, 256, 256, 1.04, 1.30}, {4, 128, 256, 1.39, 1.60},
    {kPhased256x128, 256, 128, 1.08, 1.37}};
constexpr int kNumCfg = 12;

template <int WT>
int launch_wt(const GemmParams& p, int cfg, hipStream_t stream)
{
    switch (cfg)
    {
    // production shapes:        waves  MFMA tiles  BKB stages
    case 1: return launch_cfg<WT, 2, 2, 2, 2, 1, 64, 4>(p, stream);  // 128 x 128, 64 KB  -> 2 workgroups per CU
    case 2: return launch_cfg<WT, 2, 4, 4, 2, 1, 64, 4>(p, stream);  // 256 x 256, 128 KB
    case 3: return launch_cfg<WT, 4, 2, 2, 3, 1, 64, 5>(p, stream);  // 256 x 192, 140 KB
    case 4: return launch_cfg<WT, 2, 2, 2, 4, 1, 64, 4>(p, stream);  // 128 x 256, 96 KB
    // experiments
    case 5: return launch_cfg<WT, 2, 2, 2, 2, 1, 128, 2>(p, stream); // 128 x 128, one stage ahead
    case 6: // 256 x 192, one stage ahead
        return launch_cfg<WT, 4, 2, 2, 3, 1, 128, 2>(p, stream);
    case 7: return launch_cfg<WT, 2, 4, 2, 1, 1, 64, 4>(p, stream);  // 128 x 128 on 8 waves
    case 8: return launch_cfg<WT, 2, 2, 2, 2, 1, 128, 4>(p, stream); // 128 x 128, 128-byte stages, 3 ahead (1 per CU)
    case 9: return launch_cfg<WT, 2, 2, 4, 3, 1, 128, 2>(p, stream); // 256 x 192 on 4 waves (128 x 96 per wave)
    case 10: return launch_cfg<WT, 2, 2, 4, 4, 1, 128, 2>(p, stream); // 256 x 256 on 4 waves (128 x 128 per wave)
    case 11: return launch_cfg<WT, 2, 2, 4, 3, 2, 128, 2>(p, stream); // 256 x 192, 2 K-groups of 4 waves (128 x 96 per wave)
    case 12: return launch_cfg<WT, 2, 2, 2, 2, 2, 128, 2>(p, stream);  // 128 x 128, 2 K-groups of 4 waves (64 x 64 per wave)
    case 36: return launch_cfg<WT, 4, 2, 2, 3, 1, 64, 5, 4>(p, stream);  // 256 x 192, 64-byte stages 4 ahead, 8 compute + 4 loader waves
    case 37: return launch_cfg<WT, 4, 2, 2, 3, 1, 128, 2, 4>(p, stream); // 256 x 192, one 128-byte stage ahead, 8 + 4 waves
    default: return launch_cfg<WT, 2, 2, 2, 2, 1, 128, 4>(p, stream);
    }
}

} // namespace

static bool glds_serves(const GemmParams& p)
{
    const bool sq = p.wtype == W_INT8_SQ;
    if (!sq && p.wtype != W_FP16)
        return false;
    const int es = sq ? 1 : 2;
    if ((reinterpret_cast<uintptr_t>(p.a) & 15) || ((p.lda * es) & 15) || (reinterpret_cast<uintptr_t>(p.w) & 15)
        || (p.ldw & 15) || ((p.K * es) % 128) || p.K <= 0 || p.M < 32)
        return false;
    if (!sq && p.out_dtype == DT_INT32)
        return false;
    if (p.residual
        && (p.out_dtype != DT_HALF || (p.ldc & 7) || (p.N & 7) || (reinterpret_cast<uintptr_t>(p.c) & 15)
            || (reinterpret_cast<uintptr_t>(p.residual) & 15)))
        return false; // the fused residual lives in the vector epilogue (a mis-aligned residual: launch_gemm adds it in a pass)
    if (p.silu_gate
        && (sq || p.residual || p.out_dtype != DT_HALF || (p.ldc & 7) || (p.N & 7) || (reinterpret_cast<uintptr_t>(p.c) & 15)
            || (reinterpret_cast<uintptr_t>(p.silu_gate) & 15)))
        return false; // so does the fused SwiGLU gate (fp16 operands only)
    return true;
}

// The static rule: fewest workgroup rounds over the CUs x the tile's area x what a tile of that kind costs per area (the 128-wide
// lock-step tiles pay ~40 % for their lower MFMA : LDS ratio and their exposed prologue / epilogue).  `phased_ok` = false leaves
// out the tile that exists in gemm_sqp.hip only (its launcher refused the problem: alignment, 32-bit DMA offsets).
static int static_shape_cfg(const GemmParams& p, bool phased_ok = true)
{
    const int cus = launch_util::device_cus();
    double best = 1e30;
    int cfg = 8;
    for (const Shape& s : kShapes)
    {
        if (s.id == kPhased256x128 && !phased_ok)
            continue;
        const int64_t tiles = (int64_t) ((p.M + s.bm - 1) / s.bm) * ((p.N + s.bn - 1) / s.bn);
        // beyond two rounds the 256 x 128 tile loses to 256 x 256 / 256 x 192 (M = 8192: 162 vs 136 us on O, 467 vs 377 on gate / up)
        if (s.id == kPhased256x128 && tiles > 2 * cus)
            continue;
        const double cost = (double) ((tiles + cus - 1) / cus) * s.bm * s.bn * (p.wtype == W_INT8_SQ ? s.f_sq : s.f);
        if (cost < best)
        {
            best = cost;
            cfg = s.id;
        }
    }
    return cfg;
}

// the kernel id launch_gemm_glds runs for this problem when no profile entry exists (the tactic profiler's incumbent)
int gemm_static_cfg(const GemmParams& p)
{
    if (!glds_serves(p))
        return 0;
    const int cfg = static_shape_cfg(p);
    // (SmoothQuant: the persistent forms 62 / 63 of gemm_sqp.hip serve fp16 output on 16-byte rows; launch_gemm_glds falls back
    // to the one-tile-per-workgroup forms 42 / 20 for the rest)
    const bool persist = p.out_dtype == DT_HALF && !(p.ldc & 7) && !(p.N & 7) && !(reinterpret_cast<uintptr_t>(p.c) & 15)
        && p.K >= 256;
    if (cfg == kPhased256x128)
        return p.wtype == W_INT8_SQ ? (persist ? 62 : 42) : (persist ? 56 : 54);
    // the 256 x 192 tile runs its phased sibling (gemm_sqp.hip)
    return cfg == 6 ? (p.wtype == W_INT8_SQ ? (persist ? 63 : 20) : (persist ? 55 : 50)) : cfg;
}

// exactly kernel `cfg`, no fall-back: 0 launched, -1 launch error, 1 this kernel does not serve the problem (the tactic profiler)
int launch_gemm_cfg(const GemmParams& p, int cfg, hipStream_t stream)
{
    if (!glds_serves(p))
        return 1;
    const bool sq = p.wtype == W_INT8_SQ;
    if ((cfg >= 1 && cfg <= kNumCfg) || cfg == 36 || cfg == 37)
    {
        // a tile far larger than the problem only burns time in the sweep
        return sq ? launch_wt<W_INT8_SQ>(p, cfg, stream) : launch_wt<W_FP16>(p, cfg, stream);
    }
    return sq ? launch_gemm_sqp(p, cfg, stream) : launch_gemm_f16p(p, cfg, stream);
}

// returns 0 on success, -1 on a launch error, 1 when the shape / type is not served by this kernel
int launch_gemm_glds(const GemmParams& p, hipStream_t stream)
{
    const bool sq = p.wtype == W_INT8_SQ;
    if (!glds_serves(p))
        return 1;
    int cfg = gemm_tune_cfg;
    bool from_table = false;
    if (cfg <= 0)
    {
        // the kernel the on-device profile found fastest for this shape (gemm_tactics.hip), else the static rule below
        cfg = gemm_tactic_lookup(p.wtype, p.M, p.N, p.K);
        from_table = cfg > 0;
    }
    const bool glds_id = (cfg >= 1 && cfg <= kNumCfg) || cfg == 36 || cfg == 37; // ids served by this file's table
    if (cfg > kNumCfg && !glds_id)
    {
        const int r = sq ? launch_gemm_sqp(p, cfg, stream) : launch_gemm_f16p(p, cfg, stream);
        if (r <= 0)
            return r;
        cfg = 0; // not served there (shape / alignment): the heuristic below picks a lock-step shape
    }
    if (cfg <= 0 || !((cfg >= 1 && cfg <= kNumCfg) || cfg == 36 || cfg == 37))
    {
        cfg = static_shape_cfg(p);
        if (cfg == kPhased256x128)
        {
            // one round of 256 x 128 tiles where 128 x 128 would take two (O / down at M = 2048: 34 vs 44 us, 84 vs 107 us)
            int r = sq ? launch_gemm_sqp(p, 62, stream) : launch_gemm_f16p(p, 56, stream); // the persistent form first (r05)
            if (r > 0)
                r = sq ? launch_gemm_sqp(p, 42, stream) : launch_gemm_f16p(p, 54, stream);
            if (r <= 0)
                return r;
            cfg = static_shape_cfg(p, false);
        }
    }
    if (!sq && cfg == 6 && gemm_tune_cfg <= 0 && !from_table)
    {
        // the same sibling on fp16 operands (r04): 6 - 7 % faster on QKV / gate / up at M = 1024 (profiles/r04_fp16_gemm_sweep.txt)
        int r = launch_gemm_f16p(p, 55, stream); // (r05: its persistent form first)
        if (r > 0)
            r = launch_gemm_f16p(p, 50, stream);
        if (r <= 0)
            return r;
    }
    if (sq && cfg == 6 && gemm_tune_cfg <= 0 && !from_table)
    {
        // the 256 x 192 SmoothQuant tile has a phased sibling (gemm_sqp.hip) that measures 2-5 % faster at the 7B prefill
        // shapes; exact either way
        // ... and that one a persistent form (r05: one workgroup per CU walks its tiles, the next tile's first K-tiles are
        // requested under the epilogue, tiles ordered in bands of 4 row tiles): 3 - 10 % on top (profiles/r05_sqgemm_persistent.txt)
        int r = launch_gemm_sqp(p, 63, stream);
        if (r > 0)
            r = launch_gemm_sqp(p, 20, stream);
        if (r <= 0)
            return r;
    }
    if (sq && gemm_clock_probe)
    {
        GemmParams q = p;
        q.clock_probe = gemm_clock_probe;
        return launch_wt<W_INT8_SQ>(q, cfg, stream);
    }
    return sq ? launch_wt<W_INT8_SQ>(p, cfg, stream) : launch_wt<W_FP16>(p, cfg, stream);
}

} // namespace kernels
} // namespace tllm
