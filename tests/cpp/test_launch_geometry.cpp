// Host-only test of the launch geometry of the copy-shaped kernels (oneccl_amd/csrc/launch_geometry.hpp): for sizes
// from one byte to 256 GiB and 1..16 destinations, every launch stays below HIP's limit of 2^32 lanes per grid, and
// the launches together give every group of elements to exactly one lane (intervals checked at every size; every
// lane enumerated at small sizes and with small artificial limits, through the same index function the kernel uses).
#include <stdio.h>

#include <map>
#include <vector>

#include "../../oneccl_amd/csrc/launch_geometry.hpp"

using namespace mi;

static int failed = 0, checks = 0;
#define EXPECT(c)                                                       \
    do {                                                                \
        checks++;                                                       \
        if (!(c)) {                                                     \
            failed++;                                                   \
            printf("FAILED %s:%d: %s\n", __FILE__, __LINE__, #c);       \
        }                                                               \
    } while (0)

static void check_lane_work(uint64_t addr, uint32_t esz, uint64_t count, uint32_t per, uint64_t limit, bool enumerate) {
    const LaneWork w = lane_work(addr, esz, count, per);
    EXPECT((uint64_t)w.head + w.ngroup * per + w.tail == count);
    EXPECT(w.tail < per && w.head < 16 / esz + 1);
    EXPECT(w.head == count || ((addr + (uint64_t)w.head * esz) & 15u) == 0);
    EXPECT(w.head + w.tail <= kGeomBlock);                 // one lane of block 0 each
    const uint64_t n = num_launches(w, kGeomBlock, limit);
    uint64_t next = 0, heads = 0, tails = 0;
    for (uint64_t i = 0; i < n; i++) {
        const LaunchPiece p = launch_piece(w, kGeomBlock, limit, i);
        EXPECT(p.group0 == next);
        EXPECT(p.grid >= 1 && (uint64_t)p.grid <= limit);
        EXPECT((uint64_t)p.grid * kGeomBlock < (1ull << 32));
        EXPECT((uint64_t)p.grid * kGeomBlock >= p.ngroup);              // a lane for every group
        EXPECT(p.ngroup + kGeomBlock > (uint64_t)p.grid * kGeomBlock || p.ngroup == 0);     // no idle block
        if (n > 1) EXPECT(p.ngroup > 0);
        if (enumerate) {
            std::vector<int> seen(p.ngroup, 0);
            for (uint32_t b = 0; b < p.grid; b++)
                for (uint32_t t = 0; t < kGeomBlock; t++) {
                    const uint64_t g = (uint64_t)b * kGeomBlock + t;    // what the kernels compute
                    if (g < p.ngroup) seen[g]++;
                }
            for (int s : seen) EXPECT(s == 1);
        }
        next += p.ngroup;
        heads += p.head;
        tails += p.tail;
    }
    EXPECT(next == w.ngroup && heads == w.head && tails == w.tail);
}

static void check_bcast(uint64_t addr, uint64_t bytes, int m, uint32_t max_sect, uint64_t limit, bool enumerate) {
    const BcastShape b = bcast_shape(addr, bytes, max_sect);
    EXPECT((uint64_t)b.head + b.nvec * 16 + b.tail == bytes);
    EXPECT(b.sect_tiles % 8 == 0 && b.sect_tiles <= max_sect && b.sect_tiles >= 8);
    EXPECT(b.sects * b.sect_tiles * kGeomBlock >= b.nvec);
    const uint64_t n = bcast_num_launches(b, m, limit);
    uint64_t next = 0, heads = 0, tails = 0;
    for (uint64_t i = 0; i < n; i++) {
        const BcastPiece p = bcast_piece(b, m, limit, i);
        EXPECT(p.vec0 == next);
        EXPECT((uint64_t)p.grid * kGeomBlock < (1ull << 32));
        EXPECT((uint64_t)p.grid <= limit || bcast_sects_per_launch(b, m, limit) == 1);
        EXPECT(p.grid % (b.sect_tiles * (uint32_t)m) == 0 && p.grid > 0);
        EXPECT((uint64_t)p.grid / m * kGeomBlock >= p.nvec);
        if (enumerate) {
            std::map<std::pair<uint32_t, uint64_t>, int> seen;
            for (uint32_t blk = 0; blk < p.grid; blk++)
                for (uint32_t t = 0; t < kGeomBlock; t += (blk % 7 == 0 ? 1 : 85)) {    // every lane of some blocks, a few of the others
                    const BcastLane l = bcast_lane(blk, t, b.sect_tiles, (uint32_t)m);
                    EXPECT(l.dst < (uint32_t)m);
                    if (l.vec < p.nvec) seen[{ l.dst, l.vec }]++;
                }
            for (auto& kv : seen) EXPECT(kv.second == 1);
            // every (destination, vector) pair of the piece has its lane: count the pairs block by block
            uint64_t pairs = 0;
            for (uint32_t blk = 0; blk < p.grid; blk++) {
                const BcastLane first = bcast_lane(blk, 0, b.sect_tiles, (uint32_t)m);
                if (first.vec < p.nvec) pairs += (p.nvec - first.vec < kGeomBlock) ? p.nvec - first.vec : kGeomBlock;
            }
            EXPECT(pairs == p.nvec * (uint64_t)m);
        }
        next += p.nvec;
        heads += p.head;
        tails += p.tail;
    }
    EXPECT(next == b.nvec && heads == b.head && tails == b.tail);
}

int main() {
    EXPECT(hip_block_limit(256) == (1u << 24) - 1);
    const uint64_t hw = hip_block_limit(kGeomBlock);
    // sizes 1 B ... 256 GiB (x2 steps, with odd neighbours), every misalignment class, the real limit
    for (int sh = 0; sh <= 38; sh++)
        for (int64_t d : { -17, -1, 0, 1, 4099 }) {
            const int64_t bytes = (int64_t)(1ull << sh) + d;
            if (bytes <= 0) continue;
            for (uint64_t addr : { 0x7f0000000000ull, 0x7f0000000003ull, 0x7f000000000eull }) {
                check_lane_work(addr, 1, (uint64_t)bytes, 16, hw, false);                        // copy
                check_lane_work(addr & ~1ull, 2, (uint64_t)bytes / 2 + 1, 8, hw, false);         // fp32 -> 16-bit
                check_lane_work(addr & ~3ull, 4, (uint64_t)bytes / 4 + 1, 4, hw, false);         // 16-bit -> fp32
                for (int m = 1; m <= 16; m++) check_bcast(addr, (uint64_t)bytes, m, 4096, hw, false);
            }
        }
    // a 64 GiB copy is the first that needs two launches; 1 -> 7 from 9.2 GiB likewise
    {
        const LaneWork w = lane_work(0, 1, 64ull << 30, 16);
        EXPECT(num_launches(w, kGeomBlock, hw) == 2);
        EXPECT(num_launches(lane_work(0, 1, (64ull << 30) - 4096, 16), kGeomBlock, hw) == 1);
        const BcastShape b = bcast_shape(0, 10ull << 30, 4096);
        EXPECT(bcast_num_launches(b, 7, hw) == 2 && bcast_num_launches(b, 6, hw) == 1);
    }
    // small sizes and small artificial limits, every lane enumerated
    for (uint64_t limit : { 1ull, 2ull, 3ull, 7ull, 64ull, 1000ull })
        for (uint64_t bytes : { 1ull, 15ull, 16ull, 17ull, 4095ull, 4096ull, 4097ull, 65536ull, 100003ull, 1048576ull + 5 })
            for (uint64_t addr : { 0ull, 5ull, 15ull }) {
                check_lane_work(addr, 1, bytes, 16, limit, true);
                check_lane_work(addr & ~1ull, 2, bytes, 8, limit, true);
                check_lane_work(addr & ~3ull, 4, bytes, 4, limit, true);
                for (int m : { 1, 2, 3, 7, 16 })
                    for (uint32_t max_sect : { 8u, 16u, 4096u }) check_bcast(addr, bytes, m, max_sect, limit, true);
            }
    // pack / unpack quarters: they tile the tensor exactly, none is longer than 4 KiB + 127, every quarter but the
    // first starts on a 128-byte line of the destination, and none exists beyond ceil(total / 4 KiB)
    for (uint64_t total : { 1ull, 2ull, 127ull, 128ull, 129ull, 4095ull, 4096ull, 4097ull, 4223ull, 4224ull, 8191ull, 8192ull, 16383ull, 16384ull,
                            16385ull, 100003ull, 4194304ull, 4194306ull, 12345678ull })
        for (uint64_t mis = 0; mis < 128; mis += (total < 20000 ? 1 : 7)) {
            const uint64_t dst = 0x7f0000100000ull + mis;
            const uint64_t nq = (total + kCopyQuarter - 1) / kCopyQuarter;
            uint64_t next = 0;
            for (uint64_t q = 0; q < nq; q++) {
                const CopyQuarter c = copy_quarter(total, dst, q);
                EXPECT(c.n > 0 && c.n <= kCopyQuarter + kCopyLine - 1);
                EXPECT(c.lo == next);
                EXPECT(q == 0 || ((dst + c.lo) & (kCopyLine - 1)) == 0);
                EXPECT(q + 1 == nq || c.n <= kCopyQuarter);
                next = c.lo + c.n;
            }
            EXPECT(next == total);
            for (uint64_t q = nq; q < nq + 4; q++) EXPECT(copy_quarter(total, dst, q).n == 0);
        }
    EXPECT(copy_quarter(0, 0x1000, 0).n == 0);
    // where a reduce's vectors start: the measured cases, then every choice against a brute-force minimum
    {
        const unsigned peers4[8] = { 0, 4, 4, 4, 4, 4, 4, 4 }, in2[8] = { 2, 2, 2, 2, 2, 2, 2, 2 }, al[8] = { 0 };
        const unsigned spread[8] = { 0, 2, 4, 6, 8, 10, 12, 14 };
        const unsigned o0[1] = { 0 }, o6[1] = { 6 };
        EXPECT(vector_grid(peers4, 8, o0, 1) == 0);     // seven peers 4 bytes off: loose reads on 4-byte boundaries are cheap
        EXPECT(vector_grid(in2, 8, o0, 1) == 2);        // eight inputs 2 bytes off: dearer than one loose output
        EXPECT(vector_grid(al, 8, o6, 1) == 0);         // the output alone off: it stays loose
        EXPECT(vector_grid(al, 8, o0, 1) == 0);
        EXPECT(vector_grid(spread, 8, o0, 1) == 0);
        EXPECT(vector_grid(in2, 1, o0, 1) == 0);        // one input 2 bytes off costs less than a loose output
        EXPECT(vector_grid(in2, 2, o0, 1) == 0 && vector_grid(in2, 3, o0, 1) == 2);
        // with the kernels' realignment in registers a read off the 4-byte boundary costs half: four such inputs are
        // worth a loose output, eight are not
        EXPECT(vector_grid(in2, 8, o0, 1, true) == 2 && vector_grid(in2, 4, o0, 1, true) == 0 && vector_grid(in2, 3, o0, 1, true) == 0);
        EXPECT(vector_grid(spread, 8, o0, 1, true) == 0 && vector_grid(peers4, 8, o6, 1, true) == 4);
        uint64_t x = 88172645463325252ull;
        for (int it = 0; it < 20000; it++) {
            unsigned in[8], out[3];
            x ^= x << 13; x ^= x >> 7; x ^= x << 17;
            const int n = 1 + (int)(x % 8), m = 1 + (int)((x >> 8) % 3);
            const unsigned gran = 1u << ((x >> 16) % 4);        // 1-, 2-, 4- and 8-byte elements
            for (int j = 0; j < n; j++) in[j] = (unsigned)((x >> (20 + 4 * j)) & 15u) / gran * gran;
            for (int k = 0; k < m; k++) out[k] = (unsigned)((x >> (52 + 4 * k)) & 15u) / gran * gran;
            const bool ra = (x >> 19) & 1;
            const unsigned g = vector_grid(in, n, out, m, ra);
            bool is_one = false;
            unsigned best = ~0u;
            for (int j = 0; j < n; j++) { is_one |= in[j] == g; const unsigned p = grid_price(in[j], in, n, out, m, ra); if (p < best) best = p; }
            for (int k = 0; k < m; k++) { is_one |= out[k] == g; const unsigned p = grid_price(out[k], in, n, out, m, ra); if (p < best) best = p; }
            EXPECT(is_one && grid_price(g, in, n, out, m, ra) == best);
            EXPECT(grid_price(out[0], in, n, out, m, ra) > best || g == out[0]);    // the first destination's among equals
        }
    }
    // which 128-byte line the vectors start on: the measured cases, then every choice against a brute-force minimum
    {
        const unsigned al[8] = { 0 }, all16[8] = { 16, 16, 16, 16, 16, 16, 16, 16 }, peers16[8] = { 0, 16, 16, 16, 16, 16, 16, 16 };
        const unsigned all2[8] = { 2, 2, 2, 2, 2, 2, 2, 2 }, own64[8] = { 64, 0, 0, 0, 0, 0, 0, 0 }, own16[8] = { 16, 0, 0, 0, 0, 0, 0, 0 };
        const unsigned o0[1] = { 0 }, o16[1] = { 16 }, o2[1] = { 2 }, o64[1] = { 64 };
        EXPECT(vector_start(al, 8, o0, 1, 0, true) == 0);
        EXPECT(vector_start(all16, 8, o16, 1, 0, true) == 112);         // everything 16 bytes off: 112 bytes of head put all of it on lines
        EXPECT(vector_start(all16, 8, o16, 1, 0, false) == 0);          // ... not asked for: the 16-byte boundary is enough
        EXPECT(vector_start(all2, 8, o2, 1, 2, true) == 126 && vector_start(all2, 8, o2, 1, 2, false) == 14);
        EXPECT(vector_start(peers16, 8, o0, 1, 0, true) == 0);          // the output's line is worth more than seven inputs'
        EXPECT(vector_start(al, 8, o16, 1, 0, true) == 112);            // the output alone off: the head follows it
        EXPECT(vector_start(own16, 8, o16, 1, 0, true) == 112);
        EXPECT(vector_start(own64, 8, o64, 1, 0, true) == 0);           // whole 64 bytes off: seven inputs outweigh it
        EXPECT(vector_start(own64, 2, o64, 1, 0, true) == 64);
        uint64_t x = 1234567891234567ull;
        for (int it = 0; it < 20000; it++) {
            unsigned in[8], out[3], in16[8], out16[3];
            x ^= x << 13; x ^= x >> 7; x ^= x << 17;
            const int n = 1 + (int)(x % 8), m = 1 + (int)((x >> 8) % 3);
            const unsigned gran = 1u << ((x >> 16) % 4);
            uint64_t y = x * 0x9e3779b97f4a7c15ull;
            for (int j = 0; j < n; j++) { in[j] = (unsigned)((y >> (7 * j)) & 127u) / gran * gran; in16[j] = in[j] & 15u; }
            for (int k = 0; k < m; k++) { out[k] = (unsigned)((x >> (40 + 7 * k)) & 127u) / gran * gran; out16[k] = out[k] & 15u; }
            const unsigned mis = vector_grid(in16, n, out16, m, false);
            if (mis % gran) continue;
            const unsigned h0 = (16u - mis) & 15u, s = vector_start(in, n, out, m, mis, true);
            EXPECT(s >= h0 && s < 128 && (s - h0) % 16 == 0 && s % gran == 0);
            EXPECT(vector_start(in, n, out, m, mis, false) == h0);
            unsigned best = ~0u;
            for (unsigned e = 0; e < 128; e += 16) { const unsigned p = line_price(h0 + e, in, n, out, m); if (p < best) best = p; }
            EXPECT(line_price(s, in, n, out, m) == best);
            EXPECT(line_price(h0, in, n, out, m) > best || s == h0);        // among equals the head stays as short as it can be
        }
    }
    // the write phase's pace: 8 MiB per group of stores at 7,300 GB/s on a 100 MHz clock is 1.149 us = 114.9 ticks
    {
        EXPECT(write_pace_ticks16(256ull * 512 * 16 * 4, 7300.0, 100000) == 1839);
        EXPECT(write_pace_ticks16(256ull * 512 * 16 * 4, 8030.0, 100000) == 1671);
        EXPECT(write_pace_ticks16(240ull * 512 * 16 * 4, 7300.0, 100000) == 1724);       // fewer CUs: less per group, a shorter pace
        EXPECT(write_pace_ticks16(256ull * 512 * 16 * 4, 7300.0, 25000) == 460);         // a slower clock: fewer ticks
        EXPECT(write_pace_ticks16(256ull * 512 * 16 * 4, 0.0, 100000) == 0 && write_pace_ticks16(1 << 23, 7300.0, 0) == 0);
        EXPECT(write_pace_ticks16(256ull * 512 * 16 * 4, 100.0, 100000) == 134218);      // the slowest setting: 8.4 ms per group
        EXPECT(write_pace_ticks16(~0ull, 1e-9, 100000) == 4294967295u);                  // saturates
    }
    // whether the phased form pays: the measured crossovers (one phase holds 88 MiB of results on 256 CUs)
    {
        const uint64_t per = 256ull * 512 * 44;
        auto mib = [](uint64_t m) { return (m << 20) / 16; };
        EXPECT(phases_full_enough(mib(85), per, 2) && !phases_full_enough(mib(128), per, 2) && phases_full_enough(mib(170), per, 2));
        EXPECT(phases_full_enough(mib(64), per, 3) && !phases_full_enough(mib(96), per, 3) && phases_full_enough(mib(128), per, 3));
        EXPECT(phases_full_enough(mib(51), per, 4) && !phases_full_enough(mib(38), per, 4));
        EXPECT(phases_full_enough(mib(28), per, 8) && !phases_full_enough(mib(21), per, 8));
        for (int n = 2; n <= 64; n++) EXPECT(phases_full_enough(mib(2000), per, n));    // long buffers always
        EXPECT(!phases_full_enough(0, per, 8) && !phases_full_enough(100, 0, 8));
    }
    // one more register group where it takes a phase off a launch of few phases (88 MiB per phase as usual, 96 MiB wider)
    {
        const uint64_t lanes = 256ull * 512;
        auto mib = [](uint64_t m) { return (m << 20) / 16; };
        EXPECT(phase_reg_groups(mib(64), lanes, 6, 20) == 6 && phase_reg_groups(mib(88), lanes, 6, 20) == 6);     // one phase either way
        EXPECT(phase_reg_groups(mib(88) + 1, lanes, 6, 20) == 7 && phase_reg_groups(mib(96), lanes, 6, 20) == 7);   // two phases -> one
        EXPECT(phase_reg_groups(mib(96) + 1, lanes, 6, 20) == 6 && phase_reg_groups(mib(176), lanes, 6, 20) == 6);  // two either way
        EXPECT(phase_reg_groups(mib(192), lanes, 6, 20) == 7 && phase_reg_groups(mib(256), lanes, 6, 20) == 6);
        EXPECT(phase_reg_groups(mib(384), lanes, 6, 20) == 7);                                                      // five -> four
        EXPECT(phase_reg_groups(mib(528), lanes, 6, 20) == 6 && phase_reg_groups(mib(570), lanes, 6, 20) == 6);     // six either way; seven -> six: too many to matter
        EXPECT(phase_reg_groups(mib(1024), lanes, 6, 20) == 6 && phase_reg_groups(1003782144ull / 8, lanes, 6, 20) == 6);
        EXPECT(phase_reg_groups(0, lanes, 6, 20) == 6 && phase_reg_groups(mib(96), 0, 6, 20) == 6);
        // with the wider phase 92 MiB from two inputs is one phase at fill 0.96: phased
        EXPECT(phases_full_enough(mib(92), lanes * 48, 2) && !phases_full_enough(mib(92), lanes * 44, 2));
    }
    printf("%d checks, %d failed\n", checks, failed);
    return failed ? 1 : 0;
}
