/*
 * fo_oracle.c -- TEST INFRASTRUCTURE, NOT PRODUCT CODE.
 *
 * A plain-C, CPU-only restatement of the FlashOverlap overlap hot path, used
 * solely as the checker by tests/, by __graft_entry__.smoke() and by the
 * cpu_baseline leg of bench.py.  Nothing in the shipped package imports,
 * links or executes this file; the product path is the HIP library and fails
 * loudly when that library is missing.
 *
 * Every function cites the reference lines (paths relative to the
 * infinigence/FlashOverlap tree) whose behaviour it restates.  Integer
 * results (permutations, row maps, signal counts, monitor stamps, storage
 * addresses) are the bit-exact contract; floating point follows the
 * fp32-accumulate parity target (the reference's CUTLASS fp16-accumulate
 * rounding lives in an un-vendored third-party library and is not the
 * target).
 *
 * Pinning status (what fixes each function independently of this file):
 *   reorder_indices, row_mapping, cseg_from_waves, tile_group : hand-derived
 *       vectors + permutation/stability invariants + closed form.
 *   gemm_signal / gemm_scatter : torch/numpy fp32 matmul, all-ones input
 *       (every C == K), brute-force address map on tiny tiles, round trip
 *       unpermute(permute(C)) == C, counts == cSeg, stamps a permutation.
 *   wait : semantic spec (CAS-to-zero on equality), threaded counter test.
 *   consumer_reduce : closed form ACC_k = k * C'.
 *   reorder_rmsnorm / rmsnorm : textbook fp32 RMSNorm on the un-permuted
 *       matrix, constant-row closed form, identity-RA reduction.
 *   predict_latency : hand-computed pipelines (single group => gemm+comm).
 *   algo table : the 102 12-tuples listed in the reference's generated table.
 * No function here is "parity unpinned".
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define FO_F16 0
#define FO_BF16 1

/* ------------------------------------------------------------------ */
/* 16-bit float conversions (IEEE binary16 and bfloat16), RNE.          */
/* ------------------------------------------------------------------ */
static float f16_to_f32(uint16_t h) {
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1f;
    uint32_t man = h & 0x3ffu;
    uint32_t out;
    if (exp == 0) {
        if (man == 0) {
            out = sign;
        } else { /* subnormal: normalise */
            int e = -1;
            do { man <<= 1; e++; } while (!(man & 0x400u));
            man &= 0x3ffu;
            out = sign | ((uint32_t)(127 - 15 - e) << 23) | (man << 13);
        }
    } else if (exp == 31) {
        out = sign | 0x7f800000u | (man << 13);
    } else {
        out = sign | ((exp + 112) << 23) | (man << 13);
    }
    float f;
    memcpy(&f, &out, 4);
    return f;
}

static uint16_t f32_to_f16(float f) {
    uint32_t x;
    memcpy(&x, &f, 4);
    uint32_t sign = (x >> 16) & 0x8000u;
    uint32_t absx = x & 0x7fffffffu;
    if (absx >= 0x7f800000u) { /* inf / nan */
        return (uint16_t)(sign | 0x7c00u | ((absx > 0x7f800000u) ? 0x200u : 0));
    }
    if (absx >= 0x477ff000u) { /* rounds to >= 65520 -> inf */
        return (uint16_t)(sign | 0x7c00u);
    }
    if (absx < 0x33000001u) { /* below half of the smallest subnormal */
        return (uint16_t)sign;
    }
    int32_t e = (int32_t)(absx >> 23) - 127;
    uint32_t man = (absx & 0x7fffffu) | 0x800000u;
    uint32_t shift, half_exp;
    if (e < -14) { /* subnormal result */
        shift = (uint32_t)(13 + (-14 - e));
        half_exp = 0;
    } else {
        shift = 13;
        half_exp = (uint32_t)(e + 15);
    }
    uint32_t q = man >> shift;
    uint32_t rem = man & ((1u << shift) - 1);
    uint32_t halfway = 1u << (shift - 1);
    if (rem > halfway || (rem == halfway && (q & 1))) q++;
    uint32_t out;
    if (half_exp == 0) {
        out = q; /* may carry into exponent 1: correct */
    } else {
        out = ((half_exp - 1) << 10) + q; /* q carries the implicit bit */
    }
    return (uint16_t)(sign | out);
}

static float bf16_to_f32(uint16_t h) {
    uint32_t x = (uint32_t)h << 16;
    float f;
    memcpy(&f, &x, 4);
    return f;
}

static uint16_t f32_to_bf16(float f) {
    uint32_t x;
    memcpy(&x, &f, 4);
    if ((x & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((x >> 16) | 0x40u);
    uint32_t lsb = (x >> 16) & 1u;
    x += 0x7fffu + lsb;
    return (uint16_t)(x >> 16);
}

static inline float to_f32(int dtype, uint16_t v) {
    return dtype == FO_BF16 ? bf16_to_f32(v) : f16_to_f32(v);
}
static inline uint16_t from_f32(int dtype, float v) {
    return dtype == FO_BF16 ? f32_to_bf16(v) : f32_to_f16(v);
}

/* exported for the conversion self-tests */
float fo_oracle_f16_to_f32(uint16_t h) { return f16_to_f32(h); }
uint16_t fo_oracle_f32_to_f16(float f) { return f32_to_f16(f); }
float fo_oracle_bf16_to_f32(uint16_t h) { return bf16_to_f32(h); }
uint16_t fo_oracle_f32_to_bf16(float f) { return f32_to_bf16(f); }

/* ------------------------------------------------------------------ */
/* Layout builders.                                                    */
/* ------------------------------------------------------------------ */

/* example/utils.py:6-22 (duplicated at test/test.py:23-39, tune/search.py:237-253):
 * RA[hint[i]] = i; the tile ids not in hint, ascending, take the slots
 * len(hint).. .  RA maps original tile id -> storage slot. */
int fo_oracle_reorder_indices(int S, const int *hint, int nhint, int32_t *RA) {
    if (S < 0 || nhint < 0 || nhint > S) return -1;
    for (int t = 0; t < S; t++) RA[t] = -1;
    for (int i = 0; i < nhint; i++) {
        if (hint[i] < 0 || hint[i] >= S) return -1;
        RA[hint[i]] = i; /* a repeated hint entry keeps the last index, as the list assignment does */
    }
    int next = nhint;
    for (int t = 0; t < S; t++) {
        int in_hint = 0;
        for (int i = 0; i < nhint; i++) {
            if (hint[i] == t) { in_hint = 1; break; }
        }
        if (!in_hint) RA[t] = next++;
    }
    return 0;
}

/* tune/search.py:88-94: tiles per wave group; the last group takes the
 * remainder.  Returns the number of groups. */
int fo_oracle_cseg_from_waves(int T, int wsize, int32_t *cseg) {
    if (T <= 0 || wsize <= 0) return -1;
    int G = (T + wsize - 1) / wsize;
    for (int i = 0; i < G; i++) {
        int left = T - i * wsize;
        cseg[i] = left < wsize ? left : wsize;
    }
    return G;
}

/* example/utils.py:24-52 (dup. tune/search.py:53-81): inside each group's
 * row range, rows are stably sorted by (row % W); RE[orig_row] = new_row. */
int fo_oracle_row_mapping(int M, int N, int BM, int BN, const int32_t *cseg, int G, int W,
                          int32_t *RE) {
    int64_t tiles = ((int64_t)M * N) / ((int64_t)BM * BN);
    int64_t sum = 0;
    for (int g = 0; g < G; g++) sum += cseg[g];
    if (sum != tiles || W <= 0) return -1;
    int64_t row0 = 0;
    for (int g = 0; g < G; g++) {
        int64_t R = (int64_t)cseg[g] * BM;
        int64_t k = 0;
        for (int q = 0; q < W; q++) {
            for (int64_t l = 0; l < R; l++) {
                int64_t row = row0 + l;
                if (row % W == q) {
                    RE[row] = (int32_t)(row0 + k);
                    k++;
                }
            }
        }
        row0 += R;
    }
    return 0;
}

/* example/utils.py:54-65: order[k] = k-th row after a stable sort by row % W. */
void fo_oracle_rows_by_world_size(int M, int W, int32_t *order) {
    int k = 0;
    for (int q = 0; q < W; q++)
        for (int r = 0; r < M; r++)
            if (r % W == q) order[k++] = r;
}

/* src/overlap/gemm_with_signal.h:343-349: linear scan over cSeg prefix sums;
 * group of storage slot r = smallest g with cSeg[0]+..+cSeg[g] > r. */
int fo_oracle_tile_group(const int32_t *cseg, int G, int r) {
    int bound = cseg[0];
    int g = 0;
    while (bound <= r) {
        g++;
        if (g >= G) return -1;
        bound += cseg[g];
    }
    return g;
}

/* ------------------------------------------------------------------ */
/* Signal GEMM.                                                        */
/* ------------------------------------------------------------------ */

/* src/overlap/gemm_with_signal.h:236-256 (reshape, map_to_d), :291-334 (store),
 * :337-361 (end_epilogue), src/overlap/gemm_signal.cu:71-91 (argument
 * wiring), src/overlap/gemm_with_scatter.h:229 + CUTLASS ScatterD (row map).
 *
 * C = A . B^T with A[M,K], B[N,K] (src/overlap_impl.cu:227-229), fp32
 * accumulate, one rounding to the 16-bit output type.  Tile t = tm*TN + tn is
 * stored at slot r = RA[t]: origin ((r / rLDN)*BM, (r % rLDN)*BN) of
 * C' = C viewed as [(M*N)/(rLDN*BN), rLDN*BN].  With RE != NULL, row rho of
 * C' lands on row RE[rho].  After a tile's store: MM[group(r)] += 1; in
 * monitor mode o = MM[TN-1]++ and MM[TN + r] = o.
 *
 * `order` (length T, may be NULL = ascending tile id) is the sequence in
 * which tiles complete; it only affects monitor stamps.  RA == NULL means
 * plain GEMM (src/gemm/gemm.cu:23-110): row-major C, no signalling.
 */
int fo_oracle_gemm_signal(int dtype, int M, int N, int K, int BM, int BN, int rLDN,
                          const uint16_t *A, const uint16_t *B, uint16_t *C, int32_t *MM,
                          const int32_t *RA, const int32_t *RE, const int32_t *cseg, int G,
                          int monitor, const int32_t *order) {
    if (M <= 0 || N <= 0 || K <= 0 || BM <= 0 || BN <= 0) return -1;
    if (M % BM || N % BN) return -2;
    int TM = M / BM, TN = N / BN, T = TM * TN;
    if (RA) {
        if (rLDN <= 0 || T % rLDN) return -2;
        int64_t s = 0;
        for (int g = 0; g < G; g++) s += cseg[g];
        if (s != T) return -3;
    }
    float *Af = (float *)malloc(sizeof(float) * (size_t)M * K);
    float *Bf = (float *)malloc(sizeof(float) * (size_t)N * K);
    if (!Af || !Bf) { free(Af); free(Bf); return -4; }
    for (size_t i = 0; i < (size_t)M * K; i++) Af[i] = to_f32(dtype, A[i]);
    for (size_t i = 0; i < (size_t)N * K; i++) Bf[i] = to_f32(dtype, B[i]);
    int64_t ldp = (int64_t)rLDN * BN; /* leading dimension of C' */

#pragma omp parallel for schedule(dynamic, 1)
    for (int t = 0; t < T; t++) {
        int tm = t / TN, tn = t % TN;
        int r = RA ? RA[t] : 0;
        for (int i = 0; i < BM; i++) {
            const float *a = Af + (size_t)(tm * BM + i) * K;
            uint16_t *dst;
            if (RA) {
                int64_t prow = (int64_t)(r / rLDN) * BM + i;
                if (RE) prow = RE[prow];
                dst = C + prow * ldp + (int64_t)(r % rLDN) * BN;
            } else {
                dst = C + (size_t)(tm * BM + i) * N + (size_t)tn * BN;
            }
            for (int j = 0; j < BN; j++) {
                const float *b = Bf + (size_t)(tn * BN + j) * K;
                float acc = 0.f;
#pragma omp simd reduction(+ : acc)
                for (int k = 0; k < K; k++) acc += a[k] * b[k];
                dst[j] = from_f32(dtype, acc);
            }
        }
    }
    free(Af);
    free(Bf);
    if (RA && MM) {
        for (int s = 0; s < T; s++) {
            int t = order ? order[s] : s;
            int r = RA[t];
            int g = fo_oracle_tile_group(cseg, G, r);
            if (g < 0) return -3;
            MM[g] += 1;
            if (monitor) {
                int o = MM[TN - 1];
                MM[TN - 1] = o + 1;
                MM[TN + r] = o;
            }
        }
    }
    return 0;
}

/* Inverse of the storage map, for round-trip checks: rebuild row-major C from
 * the reordered (and optionally row-scattered) buffer.  Follows the index
 * math of src/rmsnorm/rmsnorm.cuh:80-86 generalised to whole rows. */
int fo_oracle_unpermute(int M, int N, int BM, int BN, int rLDN, const uint16_t *Cp,
                        const int32_t *RA, const int32_t *RE, uint16_t *C) {
    if (M % BM || N % BN) return -2;
    int TN = N / BN;
    int64_t ldp = (int64_t)rLDN * BN;
    for (int m = 0; m < M; m++) {
        for (int tn = 0; tn < TN; tn++) {
            int r = RA[(m / BM) * TN + tn];
            int64_t prow = (int64_t)(r / rLDN) * BM + m % BM;
            if (RE) prow = RE[prow];
            memcpy(C + (size_t)m * N + (size_t)tn * BN, Cp + prow * ldp + (int64_t)(r % rLDN) * BN,
                   sizeof(uint16_t) * BN);
        }
    }
    return 0;
}

/* ------------------------------------------------------------------ */
/* Wait + host schedule + consumer.                                    */
/* ------------------------------------------------------------------ */

/* src/wait.cuh:5-9: one poll of the spin loop.  atomicCAS(addr, that, 0)
 * == that  -> the counter is reset to 0 and the waiter is released (returns
 * 1); otherwise nothing changes and the waiter keeps spinning (returns 0). */
int fo_oracle_wait_poll(int expect, int32_t *counter) {
    if (*counter == expect) {
        *counter = 0;
        return 1;
    }
    return 0;
}

/* 1-GPU stand-in for the in-place ncclAllReduce of src/overlap_impl.cu:256:
 * acc[i] = round(float(acc[i]) + float(src[i])), one rounding. */
void fo_oracle_consumer_reduce(int dtype, const uint16_t *src, uint16_t *acc, int64_t n) {
    for (int64_t i = 0; i < n; i++)
        acc[i] = from_f32(dtype, to_f32(dtype, acc[i]) + to_f32(dtype, src[i]));
}

/* src/overlap_impl.cu:246-258 (all-reduce flavour) and :302-315
 * (reduce-scatter flavour), executed after the signal GEMM has finished:
 * for each group i: wait(cSeg[i], &MM[i]) then consume the contiguous range
 * C_flat[acc : acc + n_i], n_i = cSeg[i]*BM*BN, acc += n_i.
 *   W == 1 : ACC_flat[acc : acc+n_i] += C_flat[acc : acc+n_i].
 *   W  > 1 : the group holds W equal chunks; chunk q is accumulated into
 *            ACC[q] (each ACC[q] is [M/W, N], stride seg_stride elements) at
 *            offset acc/W, mirroring ncclReduceScatter(C+acc -> D+acc/W).
 * Returns 0, or 1+i if group i's wait could never be satisfied (the
 * reference would spin forever). */
int fo_oracle_host_schedule(int dtype, int64_t tile_elems, const int32_t *cseg, int G, int32_t *MM,
                            const uint16_t *C, uint16_t *ACC, int W, int64_t seg_stride) {
    int64_t acc = 0;
    for (int i = 0; i < G; i++) {
        int64_t n = (int64_t)cseg[i] * tile_elems;
        if (!fo_oracle_wait_poll(cseg[i], &MM[i])) return 1 + i;
        if (ACC) {
            if (W <= 1) {
                fo_oracle_consumer_reduce(dtype, C + acc, ACC + acc, n);
            } else {
                int64_t chunk = n / W;
                for (int q = 0; q < W; q++)
                    fo_oracle_consumer_reduce(dtype, C + acc + q * chunk,
                                              ACC + q * seg_stride + acc / W, chunk);
            }
        }
        acc += n;
    }
    return 0;
}

/* ------------------------------------------------------------------ */
/* RMSNorm.                                                            */
/* ------------------------------------------------------------------ */

/* src/rmsnorm/rmsnorm.cuh:64-117 + launcher src/rmsnorm/rmsnorm.cu:14-30
 * (ldn = dim / BN) + example/RMSNorm.py:13-18.  For output row b and column
 * j: t = (b/BM)*ldn + j/BN, r = RA[t], source element
 * Xp[(r/rldn)*BM + b%BM, (r%rldn)*BN + j%BN] with Xp = X viewed as
 * [.., rldn*BN].  ss = sum float(x)^2 (fp32), s = 1/sqrt(ss/dim + eps),
 * y = round16( round16(float(x)*s) * w )  -- the second product is a 16-bit
 * multiply (rmsnorm.cuh:110-112), i.e. one rounding of the exact product.
 * RA == NULL means plain RMSNorm (rmsnorm.cuh:14-59).  The reference
 * hard-codes eps = 1e-5 (rmsnorm.cuh:102); here it is an argument. */
int fo_oracle_reorder_rmsnorm(int dtype, const uint16_t *X, uint16_t *Y, const uint16_t *Wt,
                              int bs, int dim, int BM, int BN, int rldn, const int32_t *RA,
                              float eps) {
    if (bs <= 0 || dim <= 0) return -1;
    if (RA && (BM <= 0 || BN <= 0 || rldn <= 0 || dim % BN || bs % BM)) return -2;
    int ldn = RA ? dim / BN : 0;
    float *row = (float *)malloc(sizeof(float) * (size_t)dim);
    if (!row) return -4;
    for (int b = 0; b < bs; b++) {
        for (int j = 0; j < dim; j++) {
            size_t src;
            if (RA) {
                int r = RA[(b / BM) * ldn + j / BN];
                int64_t nr = (int64_t)(r / rldn) * BM + b % BM;
                int64_t nc = (int64_t)(r % rldn) * BN + j % BN;
                src = (size_t)(nr * ((int64_t)rldn * BN) + nc);
            } else {
                src = (size_t)b * dim + j;
            }
            row[j] = to_f32(dtype, X[src]);
        }
        float ss = 0.f;
        for (int j = 0; j < dim; j++) ss += row[j] * row[j];
        float s = 1.0f / sqrtf(ss / (float)dim + eps);
        for (int j = 0; j < dim; j++) {
            float xn = to_f32(dtype, from_f32(dtype, row[j] * s));
            Y[(size_t)b * dim + j] = from_f32(dtype, xn * to_f32(dtype, Wt[j]));
        }
    }
    free(row);
    return 0;
}

/* ------------------------------------------------------------------ */
/* Algo index space.                                                   */
/* ------------------------------------------------------------------ */

/* tool/generate_instances.py:5-37: cartesian product (first key slowest) of
 * TbM{128,256} TbN{128,256} TbK{32,64} WarpM{64} WarpN{64} WarpK{32,64}
 * Inst{16,8,16} Stages{3,4,5} Swizzle{1,2,3,4,6,8} SplitK{1}, minus the
 * filtered combinations; index = position in the surviving list.  Returns the
 * number of entries written (12 ints each). */
int fo_oracle_algo_table(int32_t *out, int cap) {
    static const int tbm_[] = {128, 256}, tbn_[] = {128, 256}, tbk_[] = {32, 64};
    static const int wk_[] = {32, 64}, st_[] = {3, 4, 5}, sw_[] = {1, 2, 3, 4, 6, 8};
    int n = 0;
    for (int a = 0; a < 2; a++)
        for (int b = 0; b < 2; b++)
            for (int c = 0; c < 2; c++)
                for (int d = 0; d < 2; d++)
                    for (int e = 0; e < 3; e++)
                        for (int f = 0; f < 6; f++) {
                            int tbm = tbm_[a], tbn = tbn_[b], tbk = tbk_[c], wk = wk_[d];
                            int st = st_[e], sw = sw_[f];
                            if (tbm == 128 && tbn == 256 && tbk == 64 && wk == 64 && st >= 4) continue;
                            if (tbm == 128 && tbn == 256 && tbk == 64 && wk == 32) continue;
                            if (tbm == 256 && tbn == 128 && tbk == 64 && wk == 32) continue;
                            if (tbm == 256 && tbn == 128 && tbk == 64 && wk == 64 && st >= 4) continue;
                            if (tbm == 256 && tbn == 256) continue;
                            if (tbk % wk) continue; /* tbm % 64 and tbn % 64 always hold */
                            if (n < cap) {
                                int32_t *o = out + 12 * n;
                                o[0] = tbm; o[1] = tbn; o[2] = tbk; o[3] = 64; o[4] = 64; o[5] = wk;
                                o[6] = 16; o[7] = 8; o[8] = 16; o[9] = st; o[10] = sw; o[11] = 1;
                            }
                            n++;
                        }
    return n;
}

/* ------------------------------------------------------------------ */
/* Predictive wave-group latency model.                                */
/* ------------------------------------------------------------------ */

/* tune/search.py:180-205: linear interpolation (numpy.interp semantics,
 * clamped at both ends) of a measured (elements, GiB/ms) curve, then
 * latency = x * bytes_factor / bw / 2^30, where bytes_factor is
 * 2*2*(W-1) for all_reduce and 2*(W-1) for reduce_scatter in the
 * reference; the caller passes it so that the 1-GPU consumer (6 bytes per
 * element) uses the same code. */
double fo_oracle_interp_latency(const double *sizes, const double *bw, int n, double x,
                                double bytes_factor) {
    double y;
    if (x <= sizes[0]) {
        y = bw[0];
    } else if (x >= sizes[n - 1]) {
        y = bw[n - 1];
    } else {
        int i = 1;
        while (sizes[i] < x) i++;
        double t = (x - sizes[i - 1]) / (sizes[i] - sizes[i - 1]);
        y = bw[i - 1] + t * (bw[i] - bw[i - 1]);
    }
    return x * bytes_factor / y / (1024.0 * 1024.0 * 1024.0);
}

/* tune/search.py:207-235.  wave = tiles per wave when co-running with the
 * communication stage (reference: sm_count-2), full_wave = tiles per wave
 * when the GEMM runs alone (reference: sm_count). */
double fo_oracle_predict_latency(int64_t M, int64_t N, double gemm_dur, const double *sizes,
                                 const double *bw, int ncurve, const int32_t *gp, int ngp,
                                 int tile_num, int wave, int full_wave, double bytes_factor) {
    int64_t per_tile = M * N / tile_num;
    if (ngp == 1)
        return fo_oracle_interp_latency(sizes, bw, ncurve, (double)(per_tile * gp[0]), bytes_factor) +
               gemm_dur;
    int old_waves = (tile_num + full_wave - 1) / full_wave;
    int new_waves = (tile_num + wave - 1) / wave;
    double g = gemm_dur / old_waves * new_waves;
    double acc_comm = 0, acc_comp = 0;
    for (int i = 0; i < ngp; i++) {
        double comm = 0;
        if (i > 0)
            comm = fo_oracle_interp_latency(sizes, bw, ncurve, (double)(per_tile * gp[i - 1]),
                                            bytes_factor);
        acc_comm = (acc_comp > acc_comm ? acc_comp : acc_comm) + comm;
        acc_comp += g / new_waves * ((gp[i] + wave - 1) / wave);
    }
    acc_comm = (acc_comp > acc_comm ? acc_comp : acc_comm) +
               fo_oracle_interp_latency(sizes, bw, ncurve, (double)(per_tile * gp[ngp - 1]),
                                        bytes_factor);
    return acc_comm;
}

/* tune/search.py:376-385: all compositions (ordered partitions) of n, in the
 * reference's recursion order (first part ascending).  out receives parts
 * back to back, lens the part count of each composition.  Returns the number
 * of compositions (2^(n-1)). */
static void compositions_rec(int remaining, int *path, int depth, int32_t *out, int32_t *lens,
                             int *count, int *pos) {
    if (remaining == 0) {
        for (int i = 0; i < depth; i++) out[(*pos)++] = path[i];
        lens[(*count)++] = depth;
        return;
    }
    for (int i = 1; i <= remaining; i++) {
        path[depth] = i;
        compositions_rec(remaining - i, path, depth + 1, out, lens, count, pos);
    }
}

int fo_oracle_compositions(int n, int32_t *out, int32_t *lens) {
    int path[64];
    int count = 0, pos = 0;
    if (n <= 0 || n > 20) return -1;
    compositions_rec(n, path, 0, out, lens, &count, &pos);
    return count;
}
