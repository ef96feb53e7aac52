// Algo index space, raster choice and the analytic tile issue order.
#include <atomic>
#include <mutex>

#include "fo_common.h"

namespace {

fo_algo_entry g_table[128];
int g_count = 0;
std::once_flag g_once;
std::atomic<bool> g_row_waves{true};

// Same enumeration rule as the reference generator (tool/generate_instances.py:5-37):
// nested product with TbM slowest and Swizzle fastest, minus the shapes CUTLASS
// could not instantiate; the index is the position among the survivors.
void build_table() {
    const int tb[] = {128, 256}, tk[] = {32, 64}, stages[] = {3, 4, 5};
    const int swz[] = {1, 2, 3, 4, 6, 8};
    int n = 0;
    for (int tbm : tb)
        for (int tbn : tb)
            for (int tbk : tk)
                for (int wk : tk)
                    for (int st : stages)
                        for (int sw : swz) {
                            const bool wide = (tbm == 128 && tbn == 256) || (tbm == 256 && tbn == 128);
                            if (tbm == 256 && tbn == 256) continue;
                            if (wide && tbk == 64 && (wk == 32 || st >= 4)) continue;
                            if (tbk % wk) continue;
                            const int32_t row[12] = {tbm, tbn, tbk, 64, 64, wk, 16, 8, 16, st, sw, 1};
                            for (int i = 0; i < 12; i++) g_table[n].f[i] = row[i];
                            n++;
                        }
    g_count = n;
}

}  // namespace

const fo_algo_entry *fo_algo_lookup(int algo) {
    std::call_once(g_once, build_table);
    if (algo < 0 || algo >= g_count) return nullptr;
    return &g_table[algo];
}

int fo_pick_raster(int algo, int M, int N, fo_raster *r) {
    const fo_algo_entry *e = fo_algo_lookup(algo);
    if (!e) return FO_ERR_ALGO;
    const int bm = e->f[0], bn = e->f[1];
    if (M <= 0 || N <= 0) return FO_ERR_ARG;
    if (M % bm || N % bn) return FO_ERR_SHAPE;
    // The workgroup (macro) tile may cover several reorder tiles: 256x256 when it
    // divides the problem and leaves more than half a wave of workgroups.  (With
    // exactly half a wave, 128 tiles of 256x256, the Algo's own tile fills every CU
    // in a single round instead: 2048x4096x4096 73 us against 88, 8192x1024x8192
    // 134 against 162; from 129 tiles on it would need a second round and loses.)
    r->mtm = bm;
    r->mtn = bn;
    if (M % 256 == 0 && N % 256 == 0 && (long)(M / 256) * (N / 256) > 128) {
        r->mtm = 256;
        r->mtn = 256;
    }
    r->grid_m = M / r->mtm;
    r->grid_n = N / r->mtn;
    r->panel = e->f[10] < r->grid_m ? e->f[10] : r->grid_m;
    r->xcd_remap = (r->grid_m * r->grid_n >= 16) ? 1 : 0;
    r->tail_tiles = 0;
    r->resident = 0;
    r->tail_sub_m = r->tail_sub_n = 1;
    if (r->mtm == 256 && r->mtn == 256) {
        // The 256x256 launch is persistent on as many workgroups as stay resident (one
        // per CU: 256).  When at most half a wave is left after the last full one, those
        // positions go to a second launch with the Algo's own tile, which fits them into a
        // single wave of its own (two resident workgroups of 128x128 per CU, one of 128x256
        // or 256x128).  Measured against one more wave of mostly idle CUs: +5 % on
        // 8192x7168x4096 (3.5 waves), +15 % on 4096x5120x4096 (1.25 waves).
        const int resident = fo_main_tile_resident();
        r->resident = resident;
        const int nt = r->grid_m * r->grid_n, rem = nt % resident;
        const int per = (256 / bm) * (256 / bn);
        if (nt > resident && rem != 0 && per > 1 && rem * per <= (per == 4 ? 2 * resident : resident)) {
            r->tail_tiles = rem;
            r->tail_sub_m = 256 / bm;
            r->tail_sub_n = 256 / bn;
        }
        // Waves of whole tile rows (fo_row_wave_tile) when the tiles are whole waves and a wave is whole rows
        // that split into 8 power-of-two blocks; otherwise the panels above.
        const int per_xcd = resident / 8;
        if (g_row_waves.load(std::memory_order_relaxed) && r->xcd_remap && rem == 0 && resident % 8 == 0 &&
            per_xcd > 0 && (per_xcd & (per_xcd - 1)) == 0 && (r->grid_n & (r->grid_n - 1)) == 0) {
            int log_per = 0, log_gn = 0;
            while ((1 << log_per) < per_xcd) log_per++;
            while ((1 << log_gn) < r->grid_n) log_gn++;
            // blocks as close to square as the row length allows: block width 2^log_bw, 2^log_xc blocks per row
            int best = -1, best_cost = 0;
            for (int log_xc = 0; log_xc <= 3; log_xc++) {
                const int log_bw = log_gn - log_xc, log_bh = log_per - log_bw;
                if (log_bw < 0 || log_bh < 0) continue;
                const int cost = (1 << log_bh) + (1 << log_bw);  // operand panels an XCD reads per K step
                if (best < 0 || cost < best_cost || (cost == best_cost && log_bw > log_bh)) {
                    best = log_xc;
                    best_cost = cost;
                }
            }
            if (best >= 0) {
                const int log_bw = log_gn - best, log_bh = log_per - log_bw;
                r->xcd_remap = 2;
                r->panel = fo_pack_row_waves(log_bh, log_bw, best, resident);
            }
        }
    }
    return FO_OK;
}

void fo_set_row_waves(bool on) { g_row_waves.store(on, std::memory_order_relaxed); }

extern "C" int fo_gemm_set_row_waves(int on) {
    fo_set_row_waves(on != 0);
    return FO_OK;
}

extern "C" int fo_algo_count(void) {
    std::call_once(g_once, build_table);
    return g_count;
}

extern "C" int fo_algo_info(int algo, int32_t info[12]) {
    const fo_algo_entry *e = fo_algo_lookup(algo);
    if (!e) return FO_ERR_ALGO;
    if (!info) return FO_ERR_ARG;
    for (int i = 0; i < 12; i++) info[i] = e->f[i];
    return FO_OK;
}

extern "C" int fo_schedule_order(int algo, int M, int N, int32_t *order) {
    if (!order) return FO_ERR_ARG;
    fo_raster r;
    int rc = fo_pick_raster(algo, M, N, &r);
    if (rc) return rc;
    const fo_algo_entry *e = fo_algo_lookup(algo);
    const int bm = e->f[0], bn = e->f[1];
    const int tn = N / bn;
    const int sub_m = r.mtm / bm, sub_n = r.mtn / bn;
    int k = 0;
    const int nt = r.grid_m * r.grid_n, main_tiles = nt - r.tail_tiles;
    for (int wg = 0; wg < main_tiles; wg++) {
        int pm, pn;
        fo_wg_to_tile(wg, r.grid_m, r.grid_n, r.panel, r.xcd_remap, &pm, &pn);
        for (int s = 0; s < sub_m * sub_n; s++)
            order[k++] = (pm * sub_m + s / sub_n) * tn + pn * sub_n + s % sub_n;
    }
    // the tail launch walks the remaining positions in the Algo's own tile (one reorder tile per unit)
    for (int u = 0; u < r.tail_tiles * r.tail_sub_m * r.tail_sub_n; u++) {
        int pm, pn;
        fo_unit_to_tile(u, main_tiles, r.tail_sub_m, r.tail_sub_n, r.grid_m, r.grid_n, r.panel, r.xcd_remap, &pm,
                        &pn);
        order[k++] = pm * tn + pn;
    }
    return FO_OK;
}

extern "C" int fo_workgroup_tiles(int algo, int M, int N, int32_t *tiles_per_workgroup, int32_t *workgroups) {
    fo_raster r;
    int rc = fo_pick_raster(algo, M, N, &r);
    if (rc) return rc;
    const fo_algo_entry *e = fo_algo_lookup(algo);
    if (tiles_per_workgroup) *tiles_per_workgroup = (r.mtm / e->f[0]) * (r.mtn / e->f[1]);
    if (workgroups) *workgroups = r.grid_m * r.grid_n;
    return FO_OK;
}

extern "C" int fo_version(void) { return 100; }

extern "C" const char *fo_error_string(int code) {
    switch (code) {
        case FO_OK: return "ok";
        case FO_ERR_ARG: return "null pointer or non-positive size";
        case FO_ERR_SHAPE: return "shape not divisible by the tile (M % BM, N % BN, K % 8, dim % 8)";
        case FO_ERR_ALGO: return "Algo index out of range";
        case FO_ERR_DTYPE: return "dtype must be FO_F16 or FO_BF16";
        case FO_ERR_SEGMENTS: return "cSeg does not partition the tiles (or too many groups for monitor mode)";
        case FO_ERR_STATE: return "fo_overlap handle used before its init call, or a launch that does not fit this device";
        case FO_ERR_LIMIT: return "more groups than the static scratch of the allocation-free call holds (4096)";
        default: return code > 0 ? hipGetErrorString((hipError_t)code) : "unknown error";
    }
}
