// Fusion-buffer kernels: pack / unpack of many tensors in one launch and the fused
// (tensors + peer fusion buffers -> tensors) reduce.  Layout follows oneCCL's fusion manager
// (src/fusion/fusion.cpp:283-362): tensor t lives at fusion_buf + off[t]; off is a running byte offset,
// optionally rounded up to an alignment.
//
// Work is cut into items of kFusionChunk bytes of one tensor; a block of the fused reduce takes items grid-stride
// (a block of pack / unpack takes a quarter of one item; the tiled form of the fused reduce takes tiles of two items'
// size).  The item list and the per-tensor offset, size and tile-count tables live in device memory owned by the
// plan; the tensor pointers of a call travel as kernel arguments: kFusionGroup tensors per launch of the fused
// reduce (two tables: inputs and outputs), more for pack and unpack (one table).
#pragma once

#include "batch_kernels.hpp"

namespace mi {

constexpr int kFusionGroup = 256;                 // tensors per launch (two pointer tables must fit the 4 KiB of kernel arguments)
constexpr int kFusionMaxPeers = 16;
constexpr uint32_t kFusionChunk = 16384;          // bytes of one tensor per work item = kBlock lanes x 16 B x 4

struct FusionItem {
    uint32_t t;     // tensor index
    uint32_t c;     // chunk index inside the tensor
};
// Device addresses fit 48 bits; a table keeps them as 32 low and 16 high bits, 1.5 KiB for kFusionGroup of them.
struct FusionPtrs {
    uint32_t lo[kFusionGroup];
    uint16_t hi[kFusionGroup];
    bool set(size_t i, const void* p) {
        const uint64_t v = (uint64_t)(uintptr_t)p;
        lo[i] = (uint32_t)v;
        hi[i] = (uint16_t)(v >> 32);
        return (v >> 48) == 0;
    }
    __device__ __forceinline__ uint64_t get(uint32_t i) const { return ((uint64_t)hi[i] << 32) | lo[i]; }
};
struct PeerPtrs {
    const void* p[kFusionMaxPeers];
};

struct FusionLaunchArgs {
    const void* const* own;       // host arrays of k device pointers
    void* const* out;
    const void* const* peers;     // n_peers fusion buffers
    int n_peers;
    int op;
    size_t k;
    const uint64_t* d_off;        // device tables of the plan
    const uint64_t* d_bytes;
    const FusionItem* d_items;
    const uint32_t* d_tile_end;   // device: tiles of kFusionTile bytes of tensors 0..t together
    const uint64_t* item_begin;   // host: first item of tensor t, k + 1 entries
    const uint64_t* tile_begin;   // host: first tile of tensor t, k + 1 entries
    hipStream_t stream;
    Tuning tune;
};

// Elements of a tensor chunk before its output's first 16-byte boundary, where its vectors start (none when the
// output is not even aligned to its element size).  Inputs that disagree with the output modulo 16 bytes -- the peers'
// copies of a tensor behind an odd-sized one in a tightly packed fusion buffer -- are read as loose vectors; aligning
// the peers and storing loose vectors instead measures 6 % slower.
template <uint32_t ES>
__device__ __forceinline__ uint32_t fusion_head(const void* out) {
    const uint32_t mis = (uint32_t)(uintptr_t)out & 15u;
    return (mis % ES) == 0 ? ((16u - mis) & 15u) / ES : 0;
}

// What the realignment in registers (load_vectors) needs of an item when any of its inputs' vectors start off a 4-byte
// boundary: the vector behind the last computed one must be readable.  Inside a tensor it is (the next item's data:
// `spare` bytes of the tensor follow the item); in a tensor's last item the last whole vector is left to the edge
// lanes instead.  Returns bit 0: vector nvec may be read; bit 1: nvec was the count before one vector was taken off.
// own / peer_off: where the item's vectors start in the own tensor and, as an offset, in every peer's buffer.
template <uint32_t ES>
__device__ __forceinline__ uint32_t fusion_beyond(const void* own, const PeerPtrs& peers, int n_peers, uint64_t peer_off,
                                                  uint32_t nvec, uint64_t spare, uint32_t realign) {
    if (ES >= 4 || !realign || nvec == 0) return 0;
    uint32_t odd = (uint32_t)(uintptr_t)own;
    for (int j = 0; j < n_peers; j++) odd |= (uint32_t)((uintptr_t)peers.p[j] + peer_off);
    if ((odd & 3u) == 0) return 0;
    return spare >= 16 ? 1u : 3u;
}

// out_t[i] = own_t[i] OP peer_0[off_t + i] OP ... : one pass, same arithmetic as reduce_multi_kernel
template <class TR, int OP>
__global__ void __launch_bounds__(kBlock)
fusion_reduce_kernel(FusionPtrs own, FusionPtrs out, PeerPtrs peers, int n_peers, const uint64_t* off,
                     const uint64_t* bytes, const FusionItem* items, uint32_t nitems, uint32_t t0, uint32_t realign) {
    typedef typename TR::elem_t E;
    kernel_prologue<TR, OP>();
    constexpr uint32_t ES = sizeof(E);
    const uint32_t tid = threadIdx.x;
    const uint64_t idx[4] = { tid, tid + (uint32_t)kBlock, tid + 2u * kBlock, tid + 3u * kBlock };
    for (uint32_t it = blockIdx.x; it < nitems; it += gridDim.x) {
        const FusionItem w = items[it];
        const uint64_t lo = (uint64_t)w.c * kFusionChunk;
        const uint64_t left = bytes[w.t] - lo;
        const uint32_t nb = left < kFusionChunk ? (uint32_t)left : kFusionChunk;
        const unsigned char* a = (const unsigned char*)(uintptr_t)own.get(w.t - t0) + lo;
        unsigned char* o = (unsigned char*)(uintptr_t)out.get(w.t - t0) + lo;
        const uint64_t poff = off[w.t] + lo;
        const uint32_t nelem = nb / ES;
        {
            uint32_t head = fusion_head<ES>(o);
            if (head > nelem) head = nelem;
            uint32_t nvec = (nelem - head) / TR::VEC;
            const uint32_t beyond = fusion_beyond<ES>(a + head * ES, peers, n_peers, poff + head * ES, nvec, left - nb, realign);
            nvec -= beyond >> 1;
            const uint32_t tail = nelem - head - nvec * TR::VEC;
            const uint64_t nload = nvec + (beyond & 1u);
            Accs<TR> acc[4];
            u32x4 x[4];
            load_vectors<ES, 4, false>(a + head * ES, idx, nvec, nload, x);
#pragma unroll
            for (int u = 0; u < 4; u++) acc[u] = vec_init<TR>(x[u]);
            for (int j = 0; j < n_peers; j++) {
                load_vectors<ES, 4, false>((const unsigned char*)peers.p[j] + poff + head * ES, idx, nvec, nload, x);
#pragma unroll
                for (int u = 0; u < 4; u++) vec_step<TR, OP>(x[u], acc[u]);
            }
            u32x4_u* d = (u32x4_u*)(o + head * ES);
#pragma unroll
            for (int u = 0; u < 4; u++)
                if (idx[u] < nvec) st_loose(d + idx[u], vec_finish<TR>(acc[u]));
            if (tid < head + tail) {
                const uint32_t i = (tid < head) ? tid : head + nvec * TR::VEC + (tid - head);
                typename TR::acc_t r = TR::init(ld_elem<E>(a, i));
                for (int j = 0; j < n_peers; j++)
                    r = TR::template step<OP>(ld_elem<E>((const unsigned char*)peers.p[j] + poff, i), r);
                st_elem<E>(o, i, TR::finish(r));
            }
        }
    }
}

// Items per phase of the phased fused kernel whose results wait in registers on top of the kPhaseU / 2 that wait in
// LDS (two vectors = 8 registers per item).  A traits class with heavier arithmetic specialises this before its
// kernels are instantiated; the build fails on any scratch use.
template <class TR>
struct FusionPhaseRegs {
    static constexpr int items(int nt) { return nt <= 8 ? 12 : 0; }     // with more, the slot selection no longer stays in registers
};

// The same reduce with reads and writes separated in time (see reduce_multi_phased_kernel): each block takes kPhaseU / 2
// work items per phase (an item is 16 KiB of one tensor = two vectors per lane), keeps their results in LDS, and
// writes them after the chip-wide barrier.  Item (phase, slot, block) = phase * slots * blocks + slot * blocks + block.
// Head/tail elements of chunks whose output does not start on a 16-byte boundary are written directly (they are a
// few bytes).  NT = 1 + number of peers.
template <class TR, int OP, int NT>
__global__ void __launch_bounds__(kPhaseBlock)
fusion_reduce_phased_kernel(FusionPtrs own, FusionPtrs out, PeerPtrs peers, const uint64_t* off, const uint64_t* bytes,
                            const FusionItem* items, uint32_t nitems, uint32_t t0, PhaseSync* ps, int early_loads,
                            int early_stores, long spin_ticks, uint32_t realign, uint32_t wave_runs, uint32_t write_pace16) {
    typedef typename TR::elem_t E;
    kernel_prologue<TR, OP>();
    constexpr uint32_t ES = sizeof(E);
    constexpr int S = kPhaseU / 2;                      // items per phase whose results wait in LDS
    constexpr int RI = FusionPhaseRegs<TR>::items(NT);  // ... and in registers (two vectors per lane each)
    constexpr int SLOTS = S + RI;
    constexpr int NP = NT - 1;
    static_assert(kFusionChunk == 2 * 16 * kPhaseBlock, "an item is two vectors per lane");
    static_assert(SLOTS <= 64, "one descriptor per lane of a wave");
    static_assert(RI <= 12, "the register slots are named one by one below");
    __shared__ u32x4 stage[kPhaseU * kPhaseBlock];
    u32x4 rs[2 * (RI > 0 ? RI : 1)];
    const uint32_t tid = threadIdx.x;
    const uint32_t lane = tid & 63u;
    bool give_up = false;
    unsigned gen = 0;
    if (tid == 0) gen = phase_generation(ps);
    const uint64_t per_phase = (uint64_t)SLOTS * gridDim.x;
    for (uint64_t p0 = 0; p0 < nitems; p0 += per_phase) {
        // Lane k of every wave fetches the descriptor of this block's k-th item of the phase, so that the chain
        // item -> tensor tables -> pointers is walked once, for all items at once, instead of once per item.
        uint64_t d_a = 0, d_o = 0, d_poff = 0;
        uint32_t d_nb = 0;      // 0: no item in this slot
        uint32_t d_head = 0;    // elements before the item's first vector (bits 0-7); bits 8-9: fusion_beyond's answer; bit 10: a buffer is off the 128-byte lines
        if (lane < (uint32_t)SLOTS) {
            const uint64_t it = p0 + (uint64_t)lane * gridDim.x + blockIdx.x;
            if (it < nitems) {
                const FusionItem w = items[it];
                const uint64_t lo = (uint64_t)w.c * kFusionChunk;
                const uint64_t left = bytes[w.t] - lo;
                d_nb = left < kFusionChunk ? (uint32_t)left : kFusionChunk;
                d_a = own.get(w.t - t0) + lo;
                d_o = out.get(w.t - t0) + lo;
                d_poff = off[w.t] + lo;
                d_head = fusion_head<ES>((const void*)(uintptr_t)d_o);
                const uint32_t ne = d_nb / ES;
                if (d_head > ne) d_head = ne;
                d_head |= fusion_beyond<ES>((const void*)(uintptr_t)(d_a + d_head * ES), peers, NP, d_poff + d_head * ES,
                                            (ne - d_head) / TR::VEC, left - d_nb, realign) << 8;
                const uint32_t hbytes = (d_head & 0xffu) * ES;
                uint32_t off_lines = (uint32_t)(d_a + hbytes) | (uint32_t)(d_o + hbytes);
                for (int j = 0; j < NP; j++) off_lines |= (uint32_t)((uintptr_t)peers.p[j] + d_poff + hbytes);
                if (off_lines & (kLineBytes - 1)) d_head |= 1u << 10;
            }
        }
        // The block reports its arrival at the barriers a little before it is done (see phase_arrive): in front of the
        // slot that leaves early_loads or fewer loads per lane to issue (a slot is two vectors of NT inputs), and in
        // front of the one that leaves early_stores or fewer stores (two per slot).
        const int nslots = __popcll(__ballot(d_nb != 0));
        const int lead_r = early_loads > 0 ? (early_loads >= 2 * NT ? early_loads / (2 * NT) : 1) : 0;
        const int arrive_r = nslots > lead_r ? nslots - lead_r : 0;
        bool arrived = false;
        for (int k = 0; k < SLOTS; k++) {
            if (lead_r > 0 && k == arrive_r) {
                if (tid == 0) phase_arrive(ps);
                arrived = true;
            }
            const uint32_t nb = __shfl(d_nb, k, 64);
            if (nb == 0) break;
            const unsigned char* a = (const unsigned char*)(uintptr_t)__shfl(d_a, k, 64);
            unsigned char* o = (unsigned char*)(uintptr_t)__shfl(d_o, k, 64);
            const uint64_t poff = __shfl(d_poff, k, 64);
            const uint32_t nelem = nb / ES;
            {
                const uint32_t hb = __shfl(d_head, k, 64);
                const uint32_t head = hb & 0xffu, beyond = (hb >> 8) & 1u;
                const uint32_t nvec = (nelem - head) / TR::VEC - ((hb >> 9) & 1u), tail = nelem - head - nvec * TR::VEC;
                const unsigned char* s[NT];
                s[0] = a + head * ES;
#pragma unroll
                for (int j = 0; j < NP; j++) s[j + 1] = (const unsigned char*)peers.p[j] + poff + head * ES;
                // the item's two vectors of a lane: half an item apart, or -- when a buffer of the item is off the
                // 128-byte lines -- 64 vectors apart, so that a wave covers 2 KiB in one run (fewer shared lines)
                const bool runs = wave_runs == 2 || (wave_runs == 1 && (hb >> 10));
                const uint32_t i0 = runs ? (tid & ~63u) * 2u + lane : tid;
                const uint64_t idx[2] = { i0, i0 + (runs ? 64u : (uint32_t)kPhaseBlock) };
                // The item's elements before its first and after its last vector (one per lane): their loads go out
                // in front of the vectors', so that the lanes that have one wait once per item, not twice.
                const bool edge = tid < head + tail;
                const uint32_t ei = (tid < head) ? tid : head + nvec * TR::VEC + (tid - head);
                E ev[NT];
                if (edge) {
                    ev[0] = ld_elem<E>(a, ei);
#pragma unroll
                    for (int j = 0; j < NP; j++) ev[j + 1] = ld_elem<E>((const unsigned char*)peers.p[j] + poff, ei);
                }
                u32x4 res[2];
                if (nvec >= 2u * kPhaseBlock)       // a whole item: no lane is out of range (the same answer for the whole block)
                    reduce_group<TR, OP, NT, 2, true>(s, idx, nvec, nvec + beyond, res);
                else
                    reduce_group<TR, OP, NT, 2, false>(s, idx, nvec, nvec + beyond, res);
                if (k < S) {
                    stage[(2 * k) * kPhaseBlock + tid] = res[0];
                    stage[(2 * k + 1) * kPhaseBlock + tid] = res[1];
                }
                else {
                    // a register file has no run-time index: the slot is picked by a (wave-uniform) branch
#define MI_RS_PUT(i) case i: if (i < RI) { rs[2 * (i < RI ? i : 0)] = res[0]; rs[2 * (i < RI ? i : 0) + 1] = res[1]; } break;
                    switch (k - S) {
                        MI_RS_PUT(0) MI_RS_PUT(1) MI_RS_PUT(2) MI_RS_PUT(3) MI_RS_PUT(4) MI_RS_PUT(5)
                        MI_RS_PUT(6) MI_RS_PUT(7) MI_RS_PUT(8) MI_RS_PUT(9) MI_RS_PUT(10) MI_RS_PUT(11)
                        default: break;
                    }
#undef MI_RS_PUT
                }
                if (edge) {
                    typename TR::acc_t r = TR::init(ev[0]);
#pragma unroll
                    for (int j = 0; j < NP; j++) r = TR::template step<OP>(ev[j + 1], r);
                    st_elem<E>(o, ei, TR::finish(r));
                }
            }
        }
        if (lead_r == 0) __syncthreads();           // "when done" means the whole block, and its loads have landed
        if (!arrived && tid == 0) phase_arrive(ps);
        phase_wait(ps, ++gen, give_up, spin_ticks);
        const bool more = p0 + per_phase < nitems;
        const int lead_w = early_stores / 2;
        const int arrive_w = nslots > lead_w ? nslots - lead_w : 0;
        arrived = false;
        // the clock paces the items' stores as it does in reduce_multi_phased_kernel (write_pace16: 1/16 ticks per item
        // of the whole grid; 0: unpaced)
        uint64_t pace_next16 = write_pace16 ? (uint64_t)wall_clock64() << 4 : 0;
        for (int k = 0; k < SLOTS; k++) {
            if (more && lead_w > 0 && k == arrive_w) {
                if (tid == 0) phase_arrive(ps);
                arrived = true;
            }
            const uint32_t nb = __shfl(d_nb, k, 64);
            if (nb == 0) break;
            if (write_pace16) {
                while (((uint64_t)wall_clock64() << 4) < pace_next16) __builtin_amdgcn_s_sleep(1);
                pace_next16 += write_pace16;
            }
            unsigned char* o = (unsigned char*)(uintptr_t)__shfl(d_o, k, 64);
            {
                const uint32_t nelem = nb / ES;
                const uint32_t hb = __shfl(d_head, k, 64);
                const uint32_t head = hb & 0xffu;
                const uint32_t nvec = (nelem - head) / TR::VEC - ((hb >> 9) & 1u);
                u32x4_u* d = (u32x4_u*)(o + head * ES);
                u32x4 v0 = { 0, 0, 0, 0 }, v1 = v0;
                if (k < S) {
                    v0 = stage[(2 * k) * kPhaseBlock + tid];
                    v1 = stage[(2 * k + 1) * kPhaseBlock + tid];
                }
                else {
#define MI_RS_GET(i) case i: if (i < RI) { v0 = rs[2 * (i < RI ? i : 0)]; v1 = rs[2 * (i < RI ? i : 0) + 1]; } break;
                    switch (k - S) {
                        MI_RS_GET(0) MI_RS_GET(1) MI_RS_GET(2) MI_RS_GET(3) MI_RS_GET(4) MI_RS_GET(5)
                        MI_RS_GET(6) MI_RS_GET(7) MI_RS_GET(8) MI_RS_GET(9) MI_RS_GET(10) MI_RS_GET(11)
                        default: break;
                    }
#undef MI_RS_GET
                }
                const bool runs = wave_runs == 2 || (wave_runs == 1 && (hb >> 10));
                const uint32_t i0 = runs ? (tid & ~63u) * 2u + lane : tid;
                const uint32_t i1 = i0 + (runs ? 64u : (uint32_t)kPhaseBlock);
                if (i0 < nvec) st_loose(d + i0, v0);
                if (i1 < nvec) st_loose(d + i1, v1);
            }
        }
        if (more) {
            if (lead_w == 0) __syncthreads();       // "when done": every wave's stores have been acknowledged
            if (!arrived && tid == 0) phase_arrive(ps);
            phase_wait(ps, ++gen, give_up, spin_ticks);
        }
    }
}

// ---------------------------------------------------------------------------------------------------
// The phased fused reduce in tiles: the scheme of reduce_batch_phased_kernel with the tensors of a plan as its jobs.  A
// tile is kFusionTile bytes of one tensor (four vectors per lane), the inputs -- the own tensor, then the peers' slices
// in argument order -- are taken one after the other with four vectors of one input in flight per lane, the number of
// peers is a run-time count, and what a tile needs to know (where it starts in the own tensor, in the output and in
// the peers' buffers, its size, head and the realignment's needs) is worked out by lane q of every wave for the
// block's q-th tile of a phase: the first phase's at the start, every later one's while the block waits at the
// barrier in the middle of the phase before.  Elements before a tile's first and after its last vector are computed
// phase by phase between the block's report of its write phase and its wait.  A phase holds 12 tiles per block (28 vectors per lane in registers, 20 in LDS; no type
// spills with them): the 256-tensor configuration of 191 MB then takes two phases instead of two and a small third
// (258 against 264 us), larger plans measure the same either way.
constexpr uint32_t kFusionTile = (uint32_t)kBatchPhaseTile * 16u;       // 32 KiB

struct FusionDesc {
    uint64_t a, o, poff;    // where the tile starts: own tensor, output tensor, offset into every peer's buffer
    uint32_t nb;            // bytes of the tile; 0: the phase has no such tile
    uint32_t headb;         // elements before the tile's first vector (bits 0-7); bits 8-9: fusion_beyond's answer;
                            // bit 10: a buffer's first vector is off the 128-byte lines
};

template <class TR>
__device__ __forceinline__ FusionDesc fusion_describe(const FusionPtrs& own, const FusionPtrs& out, const PeerPtrs& peers,
                                                      int n_peers, const uint64_t* off, const uint64_t* bytes,
                                                      const uint32_t* tile_end, uint32_t t0, uint32_t nt, uint32_t tile_base,
                                                      uint64_t tile, uint32_t ntiles, uint32_t realign) {
    typedef typename TR::elem_t E;
    constexpr uint32_t ES = sizeof(E);
    FusionDesc d = { 0, 0, 0, 0u, 0u };
    if (tile < ntiles) {
        const uint32_t key = tile_base + (uint32_t)tile;        // counted from the plan's first tensor, as tile_end is
        uint32_t lo = t0, hi = t0 + nt - 1;                     // first tensor whose tiles end beyond `key`
        while (lo < hi) {
            const uint32_t mid = (lo + hi) >> 1;
            if (tile_end[mid] > key) hi = mid;
            else lo = mid + 1;
        }
        const uint32_t beg = lo > t0 ? tile_end[lo - 1] : tile_base;
        const uint64_t at = (uint64_t)(key - beg) * kFusionTile;
        const uint64_t left = bytes[lo] - at;
        d.nb = left < kFusionTile ? (uint32_t)left : kFusionTile;
        d.a = own.get(lo - t0) + at;
        d.o = out.get(lo - t0) + at;
        d.poff = off[lo] + at;
        uint32_t head = fusion_head<ES>((const void*)(uintptr_t)d.o);
        const uint32_t ne = d.nb / ES;
        if (head > ne) head = ne;
        d.headb = head | fusion_beyond<ES>((const void*)(uintptr_t)(d.a + head * ES), peers, n_peers, d.poff + head * ES,
                                           (ne - head) / TR::VEC, left - d.nb, realign) << 8;
        const uint32_t hbytes = head * ES;
        uint32_t off_lines = (uint32_t)(d.a + hbytes) | (uint32_t)(d.o + hbytes);
        for (int j = 0; j < n_peers; j++) off_lines |= (uint32_t)((uintptr_t)peers.p[j] + d.poff + hbytes);
        if (off_lines & (kLineBytes - 1)) d.headb |= 1u << 10;
    }
    return d;
}

struct FusionSlot {             // a tile's description, the same in every lane
    const unsigned char* a;
    unsigned char* o;
    uint64_t poff;
    uint32_t nb, head, nvec, nload, tail;
    bool runs;
};
template <class TR>
__device__ __forceinline__ FusionSlot fusion_slot(const FusionDesc& d, int q, uint32_t wave_runs) {
    constexpr uint32_t ES = sizeof(typename TR::elem_t);
    FusionSlot s;
    s.nb = (uint32_t)__builtin_amdgcn_readlane((int)d.nb, q);
    const uint32_t hb = (uint32_t)__builtin_amdgcn_readlane((int)d.headb, q);
    s.a = (const unsigned char*)(uintptr_t)readlane64(d.a, q);
    s.o = (unsigned char*)(uintptr_t)readlane64(d.o, q);
    s.poff = readlane64(d.poff, q);
    const uint32_t ne = s.nb / ES;
    s.head = hb & 0xffu;
    s.nvec = (ne - s.head) / TR::VEC - ((hb >> 9) & 1u);
    s.nload = s.nvec + ((hb >> 8) & 1u);
    s.tail = ne - s.head - s.nvec * TR::VEC;
    s.runs = wave_runs == 2 || (wave_runs == 1 && ((hb >> 10) & 1u));
    return s;
}

template <class TR, int OP>
__device__ __forceinline__ void fusion_tile(const PeerPtrs& peers, int n_peers, const FusionSlot& s, u32x4 (&out)[kBatchPhaseG],
                                            PhaseSync* arrive_ps = nullptr, int arrive_k = 0) {
    typedef typename TR::elem_t E;
    constexpr int G = kBatchPhaseG;
    constexpr uint32_t ES = sizeof(E);
    Accs<TR> acc[G];
    u32x4 x[G];
    uint64_t idx[G];
#pragma unroll
    for (int g = 0; g < G; g++) idx[g] = batch_tile_vector(g, s.runs ? 1u : 0u);
    load_vectors<ES, G, false>(s.a + s.head * ES, idx, s.nvec, s.nload, x);
#pragma unroll
    for (int g = 0; g < G; g++) acc[g] = vec_init<TR>(x[g]);
    for (int j = 0; j < n_peers; j++) {
        if (j + 1 == arrive_k && threadIdx.x == 0) phase_arrive(arrive_ps);     // arrive_k == 0: never
        load_vectors<ES, G, false>((const unsigned char*)peers.p[j] + s.poff + s.head * ES, idx, s.nvec, s.nload, x);
#pragma unroll
        for (int g = 0; g < G; g++) vec_step<TR, OP>(x[g], acc[g]);
    }
#pragma unroll
    for (int g = 0; g < G; g++) out[g] = vec_finish<TR>(acc[g]);
}

template <class TR, int OP>
__global__ void __launch_bounds__(kPhaseBlock)
fusion_reduce_tiled_kernel(FusionPtrs own, FusionPtrs out, PeerPtrs peers, int n_peers, const uint64_t* off,
                           const uint64_t* bytes, const uint32_t* tile_end, uint32_t t0, uint32_t nt, uint32_t tile_base,
                           uint32_t ntiles, PhaseSync* ps, int early_loads, int early_stores, long spin_ticks,
                           uint32_t realign, uint32_t wave_runs, uint32_t write_pace16) {
    typedef typename TR::elem_t E;
    kernel_prologue<TR, OP>();
    constexpr uint32_t ES = sizeof(E);
    constexpr int G = kBatchPhaseG;
    constexpr int RG = MultiPhaseRegs<TR>::groups + 1;      // one more register-staged tile than the reduce: 12 tiles, 100 MB, per phase
    constexpr int LG = kPhaseU / G;
    static_assert(RG + LG <= 64, "one tile description per lane of a wave");
    __shared__ u32x4 stage[kPhaseU * kPhaseBlock];
    const int n = n_peers + 1;
    const uint64_t grid = gridDim.x;
    const uint64_t per_phase = grid * (uint64_t)(RG + LG);      // tiles
    const uint32_t lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
    static_assert(3 * TR::VEC - 2 <= 64, "a wave holds a tile's edge elements");
    auto describe = [&](uint64_t tile) {
        return fusion_describe<TR>(own, out, peers, n_peers, off, bytes, tile_end, t0, nt, tile_base, tile, ntiles, realign);
    };
    bool give_up = false;
    unsigned gen = 0;
    if (threadIdx.x == 0) gen = phase_generation(ps);
    FusionDesc desc = describe(lane < (uint32_t)(RG + LG) ? (uint64_t)lane * grid + blockIdx.x : (uint64_t)ntiles);
    for (uint64_t p0 = 0; p0 < ntiles; p0 += per_phase) {
        u32x4 rs[G * (RG > 0 ? RG : 1)];
#pragma unroll
        for (int q = 0; q < RG; q++) {
            const FusionSlot s = fusion_slot<TR>(desc, q, wave_runs);
            if (s.nb) {
                u32x4 v[G];
                fusion_tile<TR, OP>(peers, n_peers, s, v);
#pragma unroll
                for (int g = 0; g < G; g++) rs[q * G + g] = v[g];
            }
        }
        bool arrived = false;
        for (int q = 0; q < LG; q++) {
            const FusionSlot s = fusion_slot<TR>(desc, RG + q, wave_runs);
            if (!s.nb) break;                               // tiles ascend with q: nothing further in this phase
            const int rem = (LG - q) * n * G;               // loads per lane still to issue in this phase
            int arrive_k = 0;
            if (!arrived) {
                const int k = rem > early_loads ? (rem - early_loads + G - 1) / G : 0;
                if (k == 0 && threadIdx.x == 0) phase_arrive(ps);
                arrive_k = k < n ? k : 0;
                arrived = k < n;
            }
            u32x4 v[G];
            fusion_tile<TR, OP>(peers, n_peers, s, v, ps, arrive_k);
#pragma unroll
            for (int g = 0; g < G; g++) stage[(q * G + g) * kPhaseBlock + threadIdx.x] = v[g];
        }
        if (early_loads == 0) __syncthreads();              // "when done" means the whole block, and its loads have landed
        if (!arrived && threadIdx.x == 0) phase_arrive(ps);
        const uint64_t np = p0 + per_phase;
        const FusionDesc next = describe(lane < (uint32_t)(RG + LG) ? np + (uint64_t)lane * grid + blockIdx.x : (uint64_t)ntiles);
        phase_wait(ps, ++gen, give_up, spin_ticks);
        const bool more = np < ntiles;
        const int arrive_u = more ? kPhaseU - early_stores : -1;    // kPhaseU: after the last store
        // the clock paces the tiles' stores as it does in reduce_multi_phased_kernel (write_pace16: 1/16 ticks per tile
        // of the whole grid; 0: unpaced)
        uint64_t pace_next16 = write_pace16 ? (uint64_t)wall_clock64() << 4 : 0;
        auto paced = [&](bool valid) {
            if (write_pace16 && valid) {
                while (((uint64_t)wall_clock64() << 4) < pace_next16) __builtin_amdgcn_s_sleep(1);
                pace_next16 += write_pace16;
            }
        };
#pragma unroll
        for (int q = 0; q < RG; q++) {
            const FusionSlot s = fusion_slot<TR>(desc, q, wave_runs);
            paced(s.nb != 0);
            u32x4_u* d = (u32x4_u*)(s.o + s.head * ES);
#pragma unroll
            for (int g = 0; g < G; g++) {
                const uint32_t i = batch_tile_vector(g, s.runs ? 1u : 0u);
                if (i < s.nvec) st_loose(d + i, rs[q * G + g]);
            }
        }
        for (int q = 0; q < LG; q++) {
            const FusionSlot s = fusion_slot<TR>(desc, RG + q, wave_runs);
            paced(s.nb != 0);
            u32x4_u* d = (u32x4_u*)(s.o + s.head * ES);
#pragma unroll
            for (int g = 0; g < G; g++) {
                const uint32_t i = batch_tile_vector(g, s.runs ? 1u : 0u);
                if (q * G + g == arrive_u && threadIdx.x == 0) phase_arrive(ps);
                if (i < s.nvec) st_loose(d + i, stage[(q * G + g) * kPhaseBlock + threadIdx.x]);
            }
        }
        if (more && arrive_u == kPhaseU) {
            __syncthreads();                                // "when done": every wave's stores have been acknowledged
            if (threadIdx.x == 0) phase_arrive(ps);
        }
        // The elements before a tile's first and after its last vector, for this phase's tiles (lane q holds the q-th
        // one's description): those that have such elements go round the block's waves, one element per lane (at most
        // VEC - 1 in front and 2 VEC - 1 behind), the elements of eight inputs loaded before their steps so that the loads
        // are in flight together.  Here, after the block's report and before its wait, the round trip costs nothing
        // while other blocks still write; in front of the report it would hold the whole chip back.
        {
            const uint32_t ne = desc.nb / ES, eh = desc.headb & 0xffu;
            const uint32_t ev = desc.nb ? (ne - eh) / TR::VEC - ((desc.headb >> 9) & 1u) : 0u;
            unsigned long long todo = __ballot(desc.nb != 0 && (eh + (ne - eh - ev * TR::VEC)) != 0);
            for (uint32_t turn = 0; todo; turn++) {
                const int q = __builtin_ctzll(todo);
                todo &= todo - 1;
                if ((turn & (kPhaseBlock / 64 - 1)) != wave) continue;
                const FusionSlot s = fusion_slot<TR>(desc, q, 0);
                if (lane < s.head + s.tail) {
                    const uint32_t i = (lane < s.head) ? lane : s.head + s.nvec * TR::VEC + (lane - s.head);
                    typename TR::acc_t r = TR::init(ld_elem<E>(s.a, i));
                    for (int j0 = 0; j0 < n_peers; j0 += 8) {
                        E x[8];
#pragma unroll
                        for (int u = 0; u < 8; u++)
                            if (j0 + u < n_peers) x[u] = ld_elem<E>((const unsigned char*)peers.p[j0 + u] + s.poff, i);
#pragma unroll
                        for (int u = 0; u < 8; u++)
                            if (j0 + u < n_peers) r = TR::template step<OP>(x[u], r);
                    }
                    st_elem<E>(s.o, i, TR::finish(r));
                }
            }
        }
        if (more) phase_wait(ps, ++gen, give_up, spin_ticks);
        desc = next;
    }
}

// The write phase's pace for the phased fused kernels, in 1/16 clock ticks per `stores` stores of 16 bytes per lane of
// the whole grid (a tile: 4, an item: 2): 1.1 x Tuning::write_pace while own buffer and peers together are few enough
// inputs for the type (PhasePacedInputs), else unpaced.
template <class TR, int OP>
inline uint32_t fusion_write_pace16(const FusionLaunchArgs& a, int grid, int stores) {
    if (a.n_peers < 1 || a.n_peers + 1 > PhasePacedInputs<TR, OP>::value) return 0;
    return write_pace_ticks16((uint64_t)grid * kPhaseBlock * 16u * (uint32_t)stores, 1.1 * (double)a.tune.write_pace, a.tune.wall_khz);
}

template <class TR, int OP>
inline hipError_t launch_fusion_tiled(const FusionLaunchArgs& a, const FusionPtrs& own, const FusionPtrs& out,
                                      const PeerPtrs& pp, size_t t0, size_t t1) {
    const int grid = (a.tune.num_cus / kPhaseGroups) * kPhaseGroups;
    g_last_kernel = "fusion_reduce_tiled_kernel";
    const uint32_t pace16 = fusion_write_pace16<TR, OP>(a, grid, 4);
    hipLaunchKernelGGL((fusion_reduce_tiled_kernel<TR, OP>), dim3(grid), dim3(kPhaseBlock), 0, a.stream, own, out, pp, a.n_peers,
                       a.d_off, a.d_bytes, a.d_tile_end, (uint32_t)t0, (uint32_t)(t1 - t0), (uint32_t)a.tile_begin[t0],
                       (uint32_t)(a.tile_begin[t1] - a.tile_begin[t0]), a.tune.sync,
                       phase_early_loads<TR, OP>(a.tune, a.n_peers + 1, pace16 != 0), phase_early_stores<TR>(a.tune, 1),
                       a.tune.spin_ticks, (uint32_t)a.tune.realign, (uint32_t)a.tune.wave_runs, pace16);
    return hipGetLastError();
}

template <class TR, int OP, int NT>
inline hipError_t launch_fusion_phased(const FusionLaunchArgs& a, const FusionPtrs& own, const FusionPtrs& out,
                                       const PeerPtrs& pp, uint64_t i0, uint64_t i1, size_t t0) {
    int grid = (a.tune.num_cus / kPhaseGroups) * kPhaseGroups;
    g_last_kernel = "fusion_reduce_phased_kernel";
    const uint32_t pace16 = fusion_write_pace16<TR, OP>(a, grid, 2);
    hipLaunchKernelGGL((fusion_reduce_phased_kernel<TR, OP, NT>), dim3(grid), dim3(kPhaseBlock), 0, a.stream, own, out, pp,
                       a.d_off, a.d_bytes, a.d_items + i0, (uint32_t)(i1 - i0), (uint32_t)t0, a.tune.sync,
                       phase_early_loads<TR, OP>(a.tune, NT, pace16 != 0), phase_early_stores<TR>(a.tune, 1), a.tune.spin_ticks,
                       (uint32_t)a.tune.realign, (uint32_t)a.tune.wave_runs, pace16);
    return hipGetLastError();
}

template <class TR, int OP>
inline hipError_t launch_fusion_op(const FusionLaunchArgs& a) {
    PeerPtrs pp;
    for (int j = 0; j < kFusionMaxPeers; j++) pp.p[j] = (j < a.n_peers) ? a.peers[j] : nullptr;
    for (size_t t0 = 0; t0 < a.k; t0 += kFusionGroup) {
        const size_t t1 = (t0 + kFusionGroup < a.k) ? t0 + kFusionGroup : a.k;
        const uint64_t i0 = a.item_begin[t0], i1 = a.item_begin[t1];
        if (i1 == i0)
            continue;
        FusionPtrs own = {}, out = {};
        for (size_t t = t0; t < t1; t++)
            if (!own.set(t - t0, a.own[t]) || !out.set(t - t0, a.out[t])) return hipErrorInvalidValue;   // not a device address
        hipError_t e = hipSuccess;
        // Large groups with two or more peers (from 320 MB of traffic by default, 480 MB with three peers, 960 MB with
        // two): separate reads from writes in time (at most 16 KiB of padding per item is over-counted).  With two
        // peers and 1.07 GB of traffic the phased item kernel, its write phase paced, measures 6.61-6.66 against
        // 5.96-6.16 TB/s for the 32- and 64-bit types, 6.47-6.57 against 5.92-6.04 for fp16, 6.38-6.40 against 5.99-6.12
        // for the 8-bit ones and 6.24-6.27 against 6.04-6.17 for bfloat16; at half of that bfloat16 loses 4 %.  With one
        // peer the phased forms measure 2-20 % below the streaming one at every size and are only taken when forced.
        // From five peers on the tiled kernel (32 KiB tiles, the inputs one after the other, tile descriptions off the
        // critical path) is the faster phased form -- 7 peers: 256 tensors in the 256-byte layout 6.52 against 6.35
        // TB/s, 400 even-sized tensors packed tightly 6.73-6.75 against 6.18-6.28, 400 odd-sized ones 6.47 against 5.79 --
        // and with three and four the item kernel, which has all inputs of an item in flight at once (256 tensors, 3
        // peers: 6.33 against 6.08; 400 tensors: level).
        const uint64_t traffic = (uint64_t)(a.n_peers + 2) * (i1 - i0) * kFusionChunk;
        const uint64_t from = (uint64_t)a.tune.phased_min_bytes * (a.n_peers == 2 ? 6u : a.n_peers == 3 ? 3u : 2u);
        const bool phased = a.tune.sync && a.tune.num_cus >= kPhaseGroups && a.n_peers >= 1 &&
                            (a.tune.variant == 8 || (a.tune.variant == 0 && a.tune.max_blocks == 0 && a.n_peers >= 2 && traffic >= from));
        if (phased && a.n_peers >= 5) {
            e = launch_fusion_tiled<TR, OP>(a, own, out, pp, t0, t1);
        }
        else if (phased) {
            switch (a.n_peers) {
                case 1: e = launch_fusion_phased<TR, OP, 2>(a, own, out, pp, i0, i1, t0); break;
                case 2: e = launch_fusion_phased<TR, OP, 3>(a, own, out, pp, i0, i1, t0); break;
                case 3: e = launch_fusion_phased<TR, OP, 4>(a, own, out, pp, i0, i1, t0); break;
                default: e = launch_fusion_phased<TR, OP, 5>(a, own, out, pp, i0, i1, t0); break;
            }
        }
        else {
            int grid = grid_for(i1 - i0, a.tune);
            g_last_kernel = "fusion_reduce_kernel";
            hipLaunchKernelGGL((fusion_reduce_kernel<TR, OP>), dim3(grid), dim3(kBlock), 0, a.stream, own, out, pp,
                               a.n_peers, a.d_off, a.d_bytes, a.d_items + i0, (uint32_t)(i1 - i0), (uint32_t)t0,
                               (uint32_t)a.tune.realign);
            e = hipGetLastError();
        }
        if (e != hipSuccess)
            return e;
    }
    return hipSuccess;
}

template <class TR>
hipError_t launch_fusion_reduce(const FusionLaunchArgs& a) {
    switch (a.op) {
        case OP_SUM: return launch_fusion_op<TR, OP_SUM>(a);
        case OP_PROD: return launch_fusion_op<TR, OP_PROD>(a);
        case OP_MIN: return launch_fusion_op<TR, OP_MIN>(a);
        case OP_MAX: return launch_fusion_op<TR, OP_MAX>(a);
        default: return hipErrorInvalidValue;
    }
}

}  // namespace mi
