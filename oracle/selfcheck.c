/*
 * TEST INFRASTRUCTURE ONLY.  Exhaustive check of the oracle's element converters against the CPU
 * instructions the reference uses:
 *   orc_bf16_narrow_rne  vs VCVTNEPS2BF16 (_mm512_cvtneps_pbh, bf16_intrisics.hpp:73-75)  all 2^32 inputs
 *   orc_fp16_narrow      vs VCVTPS2PH imm 0 (_mm256_cvtps_ph, fp16_intrisics.hpp:103)     all 2^32 inputs
 *   orc_fp16_widen       vs VCVTPH2PS (_mm256_cvtph_ps, fp16_intrisics.hpp:100)           all 2^16 inputs
 *   orc_bf16_widen / orc_bf16_narrow_trunc vs the shift forms                               all inputs
 * A check whose instruction the CPU lacks prints "skipped".  Usage: selfcheck [threads] [stride]
 * (stride > 1 samples every stride-th fp32 pattern plus a dense window around every exponent edge).
 * Exit status 0 when nothing mismatched.
 */
#define _GNU_SOURCE
#include <cpuid.h>
#include <immintrin.h>
#include <pthread.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "ccl_comp_oracle.h"

static int cpu_support(void) { /* bit0 avx512f/bw/vl, bit1 avx512_bf16, bit2 f16c */
    unsigned a, b, c, d;
    int r = 0;
    if (__get_cpuid_count(7, 0, &a, &b, &c, &d))
        if ((b & (1u << 16)) && (b & (1u << 30)) && (b & (1u << 31)))
            r |= 1;
    if (__get_cpuid_count(7, 1, &a, &b, &c, &d))
        if (a & (1u << 5))
            r |= 2;
    if (__get_cpuid(1, &a, &b, &c, &d))
        if (c & (1u << 29))
            r |= 4;
    return r;
}

struct job {
    uint64_t lo, hi, stride;
    uint64_t bad;
    uint32_t first_bad;
    int which;
};

__attribute__((target("avx512f,avx512bw,avx512vl,avx512bf16"))) static void bf16_block(uint32_t base,
                                                                                       uint16_t* out) {
    uint32_t v[16];
    for (int i = 0; i < 16; i++) v[i] = base + (uint32_t)i;
    __m256i r = (__m256i)_mm512_cvtneps_pbh(_mm512_loadu_ps((const float*)v));
    _mm256_storeu_si256((__m256i*)out, r);
}

__attribute__((target("f16c,avx"))) static void fp16_block(uint32_t base, uint16_t* out) {
    uint32_t v[8];
    for (int i = 0; i < 8; i++) v[i] = base + (uint32_t)i;
    __m128i r = _mm256_cvtps_ph(_mm256_loadu_ps((const float*)v), 0);
    _mm_storeu_si128((__m128i*)out, r);
}

__attribute__((target("f16c,avx"))) static void fp16_widen_block(uint16_t base, uint32_t* out) {
    uint16_t v[8];
    for (int i = 0; i < 8; i++) v[i] = (uint16_t)(base + i);
    __m256 r = _mm256_cvtph_ps(_mm_loadu_si128((const __m128i*)v));
    _mm256_storeu_ps((float*)out, r);
}

static void* worker(void* p) {
    struct job* j = (struct job*)p;
    uint16_t hw[16];
    for (uint64_t b = j->lo; b < j->hi; b += 16 * j->stride) {
        /* dense near exponent boundaries, strided elsewhere */
        uint32_t base = (uint32_t)b;
        if (j->which == 0) {
            bf16_block(base, hw);
            for (int i = 0; i < 16; i++) {
                uint16_t sw = orc_bf16_narrow_rne(base + (uint32_t)i);
                if (sw != hw[i]) {
                    if (!j->bad)
                        j->first_bad = base + (uint32_t)i;
                    j->bad++;
                }
            }
        }
        else {
            fp16_block(base, hw);
            fp16_block(base + 8, hw + 8);
            for (int i = 0; i < 16; i++) {
                uint16_t sw = orc_fp16_narrow(base + (uint32_t)i);
                if (sw != hw[i]) {
                    if (!j->bad)
                        j->first_bad = base + (uint32_t)i;
                    j->bad++;
                }
            }
        }
    }
    return NULL;
}

static uint64_t run_u32(int which, int threads, uint64_t stride, uint32_t* first_bad) {
    pthread_t tid[64];
    struct job jb[64];
    uint64_t total = 1ull << 32, part = total / (uint64_t)threads;
    part -= part % 16;
    for (int t = 0; t < threads; t++) {
        jb[t].lo = part * (uint64_t)t;
        jb[t].hi = (t == threads - 1) ? total : part * (uint64_t)(t + 1);
        jb[t].stride = stride;
        jb[t].bad = 0;
        jb[t].first_bad = 0;
        jb[t].which = which;
        pthread_create(&tid[t], NULL, worker, &jb[t]);
    }
    uint64_t bad = 0;
    for (int t = 0; t < threads; t++) {
        pthread_join(tid[t], NULL);
        if (jb[t].bad && !bad)
            *first_bad = jb[t].first_bad;
        bad += jb[t].bad;
    }
    if (stride > 1) { /* dense windows: +-2^16 patterns around every exponent change, both signs */
        struct job w;
        w.stride = 1;
        w.which = which;
        w.bad = 0;
        w.first_bad = 0;
        for (uint64_t e = 0; e <= 0x1ff; e++) {
            uint64_t centre = e << 23;
            w.lo = (centre >= 0x10000) ? centre - 0x10000 : 0;
            w.hi = centre + 0x10000;
            if (w.hi > total)
                w.hi = total;
            worker(&w);
        }
        if (w.bad && !bad)
            *first_bad = w.first_bad;
        bad += w.bad;
    }
    return bad;
}

int main(int argc, char** argv) {
    int threads = (argc > 1) ? atoi(argv[1]) : 8;
    uint64_t stride = (argc > 2) ? strtoull(argv[2], NULL, 10) : 1;
    if (threads < 1) threads = 1;
    if (threads > 64) threads = 64;
    if (stride < 1) stride = 1;
    int cpu = cpu_support(), fail = 0;
    uint32_t fb = 0;

    uint64_t bad = 0;
    for (uint32_t h = 0; h < 65536; h++)
        if (orc_bf16_widen((uint16_t)h) != (h << 16))
            bad++;
    for (uint64_t u = 0; u < (1ull << 32); u += 4099)
        if (orc_bf16_narrow_trunc((uint32_t)u) != (uint16_t)((uint32_t)u >> 16))
            bad++;
    printf("bf16_widen_trunc mismatches=%llu\n", (unsigned long long)bad);
    fail |= bad != 0;

    if ((cpu & 3) == 3) {
        bad = run_u32(0, threads, stride, &fb);
        printf("bf16_narrow_rne_vs_vcvtneps2bf16 stride=%llu mismatches=%llu first=0x%08x\n",
               (unsigned long long)stride, (unsigned long long)bad, fb);
        fail |= bad != 0;
    }
    else
        printf("bf16_narrow_rne_vs_vcvtneps2bf16 skipped (no avx512_bf16)\n");

    if (cpu & 4) {
        bad = run_u32(1, threads, stride, &fb);
        printf("fp16_narrow_vs_vcvtps2ph stride=%llu mismatches=%llu first=0x%08x\n",
               (unsigned long long)stride, (unsigned long long)bad, fb);
        fail |= bad != 0;
        bad = 0;
        for (uint32_t h = 0; h < 65536; h += 8) {
            uint32_t hw[8];
            fp16_widen_block((uint16_t)h, hw);
            for (int i = 0; i < 8; i++)
                if (orc_fp16_widen((uint16_t)(h + i)) != hw[i])
                    bad++;
        }
        printf("fp16_widen_vs_vcvtph2ps mismatches=%llu\n", (unsigned long long)bad);
        fail |= bad != 0;
    }
    else
        printf("fp16 checks skipped (no f16c)\n");
    return fail;
}
