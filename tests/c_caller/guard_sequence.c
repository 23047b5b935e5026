/* guard_sequence.c -- a C11 consumer of libcwick_hip.so, written the way the engine would call
 * it: every hot loop is guarded by one call that returns 1 when the GPU produced the result and
 * 0 when the caller has to run its own CPU loop (the convention of src/h3.c:562-564).
 *
 *   latent cache:  create -> write_f32 (quantised on the device) -> mla_decode
 *   K/V cache:     create -> write_f32 (narrowed on the device)  -> gqa_decode
 *   selection:     force(0): the same calls decline, the CPU loops below produce the result;
 *                  force(1): the GPU path again
 *
 * The CPU loops are this program's own plain double-precision attention over what the caches
 * hold (read back through the ABI), so the check does not depend on anything but the header.
 * Exit status 0: every result inside max-abs 2e-3 / relative 1e-2, every decline clean.
 * Without a GPU the program reports the backend as unavailable and checks only the declines. */
#include <math.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "cwick_hip.h"

static uint32_t rng_state = 0x2545F491u;
static float frand(void) {           /* uniform in [-1, 1) */
    rng_state ^= rng_state << 13; rng_state ^= rng_state >> 17; rng_state ^= rng_state << 5;
    return (float)(rng_state >> 8) * (1.0f / 8388608.0f) - 1.0f;
}
static float bf16_to_f32(uint16_t b) { uint32_t u = (uint32_t)b << 16; float f; memcpy(&f, &u, 4); return f; }
static uint16_t f32_to_bf16(float f) { uint32_t u; memcpy(&u, &f, 4); u += 0x7FFFu + ((u >> 16) & 1u); return (uint16_t)(u >> 16); }
static float e4m3_to_f32(uint8_t b) {      /* bias 7, subnormal step 2^-9, 0x7F / 0xFF NaN (src/tensor.c:344-368) */
    int e = (b >> 3) & 15, m = b & 7;
    float v = e == 0 ? (float)m * 0x1p-9f : (e == 15 && m == 7) ? NAN : ldexpf(1.0f + (float)m / 8.0f, e - 7);
    return (b & 0x80) ? -v : v;
}

static int check(const char *what, const float *got, const double *ref, int n) {
    double d = 0, m = 0;
    for (int i = 0; i < n; i++) {
        if (!(got[i] == got[i])) { printf("FAIL %s: NaN at %d\n", what, i); return 0; }
        double e = fabs((double)got[i] - ref[i]);
        if (e > d) d = e;
        if (fabs(ref[i]) > m) m = fabs(ref[i]);
    }
    printf("%-34s max-abs %.3e  rel %.3e\n", what, d, m > 0 ? d / m : d);
    return d <= 2e-3 && d <= 1e-2 * m;
}

/* CPU loop: absorbed-latent decode over the rows the cache holds (src/attention.c:749-811) */
static void cpu_mla(const uint8_t *rows, const float *scales, int n, const uint16_t *q, int nh, float scale, double *out) {
    double *s = malloc(sizeof(double) * (size_t)n);
    for (int h = 0; h < nh; h++) {
        double mx = -1e300, sum = 0;
        for (int t = 0; t < n; t++) {
            double d = 0;
            for (int i = 0; i < CWICK_HIP_LATENT_KDIM; i++)
                d += (double)bf16_to_f32(q[h * CWICK_HIP_LATENT_KDIM + i]) *
                     (double)(e4m3_to_f32(rows[(size_t)t * CWICK_HIP_LATENT_KDIM + i]) * scales[t * CWICK_HIP_LATENT_NBLK + i / CWICK_HIP_LATENT_BLOCK]);
            s[t] = d * scale;
            if (s[t] > mx) mx = s[t];
        }
        for (int t = 0; t < n; t++) { s[t] = exp(s[t] - mx); sum += s[t]; }
        for (int j = 0; j < CWICK_HIP_LATENT_VDIM; j++) {
            double a = 0;
            for (int t = 0; t < n; t++)
                a += s[t] * (double)(e4m3_to_f32(rows[(size_t)t * CWICK_HIP_LATENT_KDIM + j]) * scales[t * CWICK_HIP_LATENT_NBLK + j / CWICK_HIP_LATENT_BLOCK]);
            out[h * CWICK_HIP_LATENT_VDIM + j] = a / sum;
        }
    }
    free(s);
}

/* CPU loop: GQA decode over bf16 rows (src/q35_model.c:1656-1701) */
static void cpu_gqa(const uint16_t *k, const uint16_t *v, int n, int nkv, int hd, const uint16_t *q, int nh, float scale, double *out) {
    double *s = malloc(sizeof(double) * (size_t)n);
    for (int h = 0; h < nh; h++) {
        const int g = h / (nh / nkv);
        double mx = -1e300, sum = 0;
        for (int t = 0; t < n; t++) {
            double d = 0;
            for (int i = 0; i < hd; i++) d += (double)bf16_to_f32(q[h * hd + i]) * (double)bf16_to_f32(k[((size_t)t * nkv + g) * hd + i]);
            s[t] = d * scale;
            if (s[t] > mx) mx = s[t];
        }
        for (int t = 0; t < n; t++) { s[t] = exp(s[t] - mx); sum += s[t]; }
        for (int i = 0; i < hd; i++) {
            double a = 0;
            for (int t = 0; t < n; t++) a += s[t] * (double)bf16_to_f32(v[((size_t)t * nkv + g) * hd + i]);
            out[h * hd + i] = a / sum;
        }
    }
    free(s);
}

int main(void) {
    int ok = 1;
    char info[256];
    if (!cwick_hip_ready()) {
        printf("backend: unavailable (%s)\n", cwick_hip_last_error());
        /* the guards decline and leave their outputs alone */
        float out[4] = {7, 7, 7, 7};
        int64_t got = -1;
        int32_t idx[2] = {-5, -5};
        ok &= cwick_hip_topk(out, 4, 2, idx, &got) == 0 && got == -1 && idx[0] == -5;
        ok &= cwick_hip_latent_create(1, 16) == NULL && cwick_hip_kv_create(16, 4, 256) == NULL;
        ok &= cwick_hip_last_error()[0] != 0;
        printf(ok ? "declines: clean\nOK\n" : "FAIL: a decline touched its outputs\n");
        return ok ? 0 : 1;
    }
    cwick_hip_device_info(info, sizeof info);
    printf("backend: %s\n", info);

    /* ---- absorbed-latent MLA over a cache filled from fp32 rows ---- */
    enum { N = 700, NH = 16 };
    const float scale = 0.0721687836f;
    float *lat = malloc(sizeof(float) * N * CWICK_HIP_LATENT_KDIM);
    for (int i = 0; i < N * CWICK_HIP_LATENT_KDIM; i++) lat[i] = 1.5f * frand();
    uint16_t *q = malloc(sizeof(uint16_t) * NH * CWICK_HIP_LATENT_KDIM);
    for (int i = 0; i < NH * CWICK_HIP_LATENT_KDIM; i++) q[i] = f32_to_bf16(2.0f * frand());
    cwick_hip_latent *lc = cwick_hip_latent_create(2, 1024);
    if (!lc) { printf("FAIL latent_create: %s\n", cwick_hip_last_error()); return 1; }
    ok &= cwick_hip_latent_write_f32(lc, 1, 0, N, lat);
    uint8_t *rows = malloc((size_t)N * CWICK_HIP_LATENT_KDIM);
    float *scales = malloc(sizeof(float) * N * CWICK_HIP_LATENT_NBLK);
    ok &= cwick_hip_latent_read(lc, 1, 0, N, rows, scales);
    float *c_acc = malloc(sizeof(float) * NH * CWICK_HIP_LATENT_VDIM);
    double *ref = malloc(sizeof(double) * NH * CWICK_HIP_LATENT_VDIM);
    cpu_mla(rows, scales, N, q, NH, scale, ref);
    if (cwick_hip_mla_decode(lc, 1, NULL, N, q, NH, scale, c_acc)) ok &= check("mla_decode (GPU)", c_acc, ref, NH * CWICK_HIP_LATENT_VDIM);
    else { printf("FAIL mla_decode declined: %s\n", cwick_hip_last_error()); ok = 0; }
    /* what the quantiser stored is the nearest E4M3 point of value / scale */
    {
        double worst = 0;
        for (int i = 0; i < N * CWICK_HIP_LATENT_KDIM; i++) {
            const float s = scales[(i / CWICK_HIP_LATENT_KDIM) * CWICK_HIP_LATENT_NBLK + (i % CWICK_HIP_LATENT_KDIM) / CWICK_HIP_LATENT_BLOCK];
            const double e = fabs((double)e4m3_to_f32(rows[i]) * s - lat[i]) / (448.0 * s);
            if (e > worst) worst = e;
        }
        printf("%-34s worst error %.4f of the block maximum\n", "latent_write_f32 round trip", worst);
        ok &= worst <= 0.0358;                       /* half an E4M3 step at the top binade: 16 / 448 */
    }

    /* ---- the same guard with the backend deselected: declines, the CPU loop runs ---- */
    cwick_hip_force(0);
    for (int i = 0; i < NH * CWICK_HIP_LATENT_VDIM; i++) c_acc[i] = -3.0f;
    if (cwick_hip_mla_decode(lc, 1, NULL, N, q, NH, scale, c_acc)) { printf("FAIL: served while deselected\n"); ok = 0; }
    else {
        int untouched = 1;
        for (int i = 0; i < NH * CWICK_HIP_LATENT_VDIM; i++) untouched &= c_acc[i] == -3.0f;
        printf("%-34s declined (%s), outputs %s\n", "mla_decode after force(0)", cwick_hip_last_error(), untouched ? "untouched" : "TOUCHED");
        ok &= untouched;
        for (int i = 0; i < NH * CWICK_HIP_LATENT_VDIM; i++) c_acc[i] = (float)ref[i];     /* the CPU path */
    }
    ok &= cwick_hip_force(1) == 0;
    ok &= cwick_hip_mla_decode(lc, 1, NULL, N, q, NH, scale, c_acc) && check("mla_decode after force(1)", c_acc, ref, NH * CWICK_HIP_LATENT_VDIM);
    /* an index list with padding, as the selector emits it */
    {
        int32_t sel[64];
        for (int i = 0; i < 64; i++) sel[i] = (i * 37) % N;
        sel[5] = -1; sel[63] = -1;
        uint8_t *r2 = malloc(62 * CWICK_HIP_LATENT_KDIM); float *s2 = malloc(sizeof(float) * 62 * CWICK_HIP_LATENT_NBLK);
        int m = 0;
        for (int i = 0; i < 64; i++) if (sel[i] >= 0) {
            memcpy(r2 + (size_t)m * CWICK_HIP_LATENT_KDIM, rows + (size_t)sel[i] * CWICK_HIP_LATENT_KDIM, CWICK_HIP_LATENT_KDIM);
            memcpy(s2 + m * CWICK_HIP_LATENT_NBLK, scales + sel[i] * CWICK_HIP_LATENT_NBLK, sizeof(float) * CWICK_HIP_LATENT_NBLK);
            m++;
        }
        cpu_mla(r2, s2, m, q, NH, scale, ref);
        ok &= cwick_hip_mla_decode(lc, 1, sel, 64, q, NH, scale, c_acc) && check("mla_decode over sel[] with -1", c_acc, ref, NH * CWICK_HIP_LATENT_VDIM);
        sel[0] = 5000;                                /* outside the cache: refused on the host */
        ok &= cwick_hip_mla_decode(lc, 1, sel, 64, q, NH, scale, c_acc) == 0;
        free(r2); free(s2);
    }
    cwick_hip_latent_free(lc);

    /* ---- GQA decode over a K/V cache filled from fp32 rows ---- */
    enum { GK = 500, GH = 16, GKV = 4, GD = 256 };
    float *kf = malloc(sizeof(float) * GK * GKV * GD), *vf = malloc(sizeof(float) * GK * GKV * GD);
    for (int i = 0; i < GK * GKV * GD; i++) { kf[i] = frand(); vf[i] = frand(); }
    uint16_t *gq = malloc(sizeof(uint16_t) * GH * GD);
    for (int i = 0; i < GH * GD; i++) gq[i] = f32_to_bf16(frand());
    cwick_hip_kv *kv = cwick_hip_kv_create(GK, GKV, GD);
    if (!kv) { printf("FAIL kv_create: %s\n", cwick_hip_last_error()); return 1; }
    ok &= cwick_hip_kv_write_f32(kv, 0, GK, kf, vf);
    uint16_t *kb = malloc(sizeof(uint16_t) * GK * GKV * GD), *vb = malloc(sizeof(uint16_t) * GK * GKV * GD);
    ok &= cwick_hip_kv_read(kv, 0, GK, kb, vb);
    int same = 1;
    for (int i = 0; i < GK * GKV * GD; i++) same &= kb[i] == f32_to_bf16(kf[i]) && vb[i] == f32_to_bf16(vf[i]);
    printf("%-34s %s\n", "kv_write_f32 narrows with RNE", same ? "bit-equal" : "DIFFERS");
    ok &= same;
    float *go = malloc(sizeof(float) * GH * GD);
    double *gref = malloc(sizeof(double) * GH * GD);
    cpu_gqa(kb, vb, GK, GKV, GD, gq, GH, 0.0625f, gref);
    ok &= cwick_hip_gqa_decode(kv, GK, gq, GH, 0.0625f, go) && check("gqa_decode (GPU)", go, gref, GH * GD);
    ok &= cwick_hip_gqa_decode(kv, GK + 1, gq, GH, 0.0625f, go) == 0;       /* past the capacity: declined */

    /* ---- block-sparse decode: the selection of src/mm_model.c:1733-1780 and :1969-1976, then the
     * attention over the kept positions (:1962-2047), against this file's own loops ---- */
    {
        enum { IH = 4, ID = 128, BS = 64, KEEP = 3, MAXSEL = (KEEP + 1) * BS };
        uint16_t *ik = malloc(sizeof(uint16_t) * GK * ID);
        float *iq = malloc(sizeof(float) * IH * ID), *isc = malloc(sizeof(float) * GK);
        for (int i = 0; i < GK * ID; i++) ik[i] = f32_to_bf16(frand());
        for (int i = 0; i < IH * ID; i++) iq[i] = frand();
        cwick_hip_kv *idx = cwick_hip_kv_create(GK, 1, ID);
        if (!idx) { printf("FAIL kv_create (index keys): %s\n", cwick_hip_last_error()); return 1; }
        ok &= cwick_hip_kv_write(idx, 0, GK, ik, ik);
        for (int s = 0; s < GK; s++) {                      /* mm_index_scores */
            float tot = 0.0f;
            for (int h = 0; h < IH; h++) {
                float d = 0.0f;
                for (int i = 0; i < ID; i++) d = fmaf(iq[h * ID + i], bf16_to_f32(ik[s * ID + i]), d);
                if (d > 0.0f) tot += d;
            }
            isc[s] = tot;
        }
        enum { NBLK = (GK + BS - 1) / BS };
        float bmax[NBLK];
        int chosen[NBLK] = {0}, want_blk[KEEP + 1], nb = 0;
        for (int b = 0; b < NBLK; b++) {
            bmax[b] = -1e30f;
            for (int s = b * BS; s < (b + 1) * BS && s < GK; s++) bmax[b] = fmaxf(bmax[b], isc[s]);
        }
        for (int r = 0; r < KEEP; r++) {                    /* the KEEP best blocks (scores are tie-free here) */
            int best = -1;
            for (int b = 0; b < NBLK; b++) if (!chosen[b] && (best < 0 || bmax[b] > bmax[best])) best = b;
            chosen[best] = 1;
        }
        chosen[GK / BS] = 1;                                /* the newest block, always */
        for (int b = 0; b < NBLK; b++) if (chosen[b]) want_blk[nb++] = b;
        int32_t want_pos[MAXSEL], got_blk[KEEP + 1], got_pos[MAXSEL];
        int64_t n_want = 0, n_got = -1;
        for (int i = 0; i < nb; i++)
            for (int s = want_blk[i] * BS; s < (want_blk[i] + 1) * BS && s < GK; s++) want_pos[n_want++] = s;
        int sel_ok = cwick_hip_mm_select(idx, GK, iq, IH, BS, KEEP, got_blk, got_pos, MAXSEL, &n_got) && n_got == n_want;
        for (int i = 0; sel_ok && i < nb; i++) sel_ok &= got_blk[i] == want_blk[i];
        for (int64_t i = 0; sel_ok && i < n_want; i++) sel_ok &= got_pos[i] == want_pos[i];
        printf("%-34s %s (%lld positions in %d blocks)\n", "mm_select (GPU)", sel_ok ? "equal" : "DIFFERS",
               (long long)n_want, nb);
        ok &= sel_ok;
        uint16_t *kg = malloc(sizeof(uint16_t) * MAXSEL * GKV * GD), *vg = malloc(sizeof(uint16_t) * MAXSEL * GKV * GD);
        for (int64_t i = 0; i < n_want; i++) {
            memcpy(kg + i * GKV * GD, kb + (size_t)want_pos[i] * GKV * GD, sizeof(uint16_t) * GKV * GD);
            memcpy(vg + i * GKV * GD, vb + (size_t)want_pos[i] * GKV * GD, sizeof(uint16_t) * GKV * GD);
        }
        cpu_gqa(kg, vg, (int)n_want, GKV, GD, gq, GH, 0.0625f, gref);
        ok &= cwick_hip_gqa_decode_sel(kv, got_pos, n_got, gq, GH, 0.0625f, go) &&
              check("gqa_decode_sel over them (GPU)", go, gref, GH * GD);
        cwick_hip_kv_free(idx);
    }
    cwick_hip_kv_free(kv);
    cwick_hip_shutdown();
    printf(ok ? "OK\n" : "FAILED\n");
    return ok ? 0 : 1;
}
