// The single-pass top-k path: two launches (included by topk.hip inside its namespace).
//
// k_topk_stream - blocks of the 1D grid, in dispatch order:
//   sample blocks   one per bucket, the first blocks of the grid.  8192 evenly spread
//                   elements of grad + residual -> the candidate window [lo, hi) and the
//                   predicted threshold; the block clears the bucket's counters and then
//                   publishes the call's epoch number in S_READY.
//   then, segment by segment (segment s = the tiles of bucket s, then the bin blocks of
//   bucket s - 1; the bin blocks of the last bucket close the grid):
//   streaming blocks one per 4096-element tile, in address order.  A wavefront loads its
//                   1024 elements, waits until the bucket's S_READY shows the epoch, stores
//                   residual <- grad + residual (0.0f at or above the predicted threshold)
//                   and stages its candidates (key >= lo) in LDS in index order; the block
//                   writes them to the tile's slots and counts itself into its group of
//                   tiles (at most 64 groups per bucket).
//   bin blocks      64 per bucket.  Block g waits until group g's tiles are finished (when it
//                   is dispatched - one bucket later - they are, except in the last bucket),
//                   counts the group's candidates per coarse window bin (64 bins), publishes
//                   the counts and copies the candidates, binned, to the bucket's per-bin
//                   lists.  It waits for nothing else.
// k_topk_select - 64 blocks per bucket; nothing crosses blocks any more: every block
//                   redundantly finds the bin that holds the k-th largest key (from the
//                   groups' counts), the exact threshold and the tie rule (from that bin's
//                   list) and the number of picks in the groups before its own, then writes
//                   its group's picks, in index order, at that offset of the payload and
//                   repairs the residual where the predicted threshold and the true one
//                   disagree.  A failed selection (threshold outside the window, a bin list
//                   overflow) hands the bucket to the exact selection, run by the bucket's 64
//                   blocks together through counter barriers; the launch covers at most 16
//                   buckets, so that all its blocks are resident at the same time.
//
// Progress in k_topk_stream.  The hardware deals the blocks of a grid to the XCDs round-robin
// and every XCD dispatches its share in grid order.  A streaming block waits only for its
// bucket's sample block, which precedes every streaming block in the grid.  A bin block waits
// only for streaming blocks that precede it in the grid.  Nothing waits for a later block.
// (Variants in which blocks of the streaming launch also performed the selection were built
// and measured: with the streaming block that finishes a group last going on as the group's
// emitter, the slowest XCD collects every emitter, slows down further and jams; with
// dedicated selection blocks in the grid nothing jams, but every dependent memory round trip
// of the selection takes 5 to 8 microseconds while the stream is in flight, the blocks live
// 50 to 100 microseconds each, and the stream loses a quarter of its block slots to them.)
// All waits are bounded all the same (`limit_ticks`): a block that gives up sets S_TIMEOUT,
// overwrites the bucket's payload header with kPoisonK and leaves; k_topk_select leaves such
// a bucket alone.
//
// Everything that crosses blocks inside a launch is written and read with agent-scope
// accesses (the XCDs' L2 caches are not coherent for plain ones), and a writer waits for
// its stores' acknowledgements before it signals.

constexpr int kFRegion = 1024;                // elements one wavefront streams
constexpr int kFWaves = kBlock / kWave;       // 4
constexpr int kFTile = kFRegion * kFWaves;    // elements per streaming block
constexpr int kFVecs = kFRegion / (kWave * 4);  // 16-byte vectors per lane and array: all issued at once
constexpr int kTileSlots = 128;               // candidate slots per tile
constexpr int kCoarse = 64;                   // coarse window bins; the last one holds keys >= hi
constexpr int kGroups = 64;                   // at most this many groups of tiles per bucket
constexpr int kCntStride = 64;                // words between two groups' arrival counters: 256 bytes, so that the
                                              // arrivals of a bucket's tiles spread over memory channels
constexpr int kHeld = 7;                      // tiles per wavefront whose slots a bin / select block keeps in registers
constexpr int kFSample = 8192;                // sampled elements per bucket
constexpr int kSelBuckets = 16;               // buckets per k_topk_select launch: 1024 blocks, all resident
constexpr uint32_t kPoisonK = 0xFFFFFFFFu;    // payload header of a bucket whose selection was abandoned
constexpr uint32_t kGaveUp = 0xFFFFFFFEu;     // a wavefront's count: its wait for the sample timed out
static_assert(kFVecs == 4, "the streaming role is written for four vectors per lane");

__device__ __forceinline__ uint64_t ld_agent64(const uint64_t* p) {
    return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void st_agent64(uint64_t* p, uint64_t v) {
    __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
// 16-byte streaming store written through to memory (agent scope): a later 4-byte
// repair of the same line by a block on another XCD must not be overwritten by a
// delayed write-back of this one.  A store of more than 8 bytes reads its data
// registers over the following cycles: the compiler keeps the next vector
// instruction from overwriting them for stores it emits itself, not for this one,
// hence the wait states inside the statement.
__device__ __forceinline__ void store_through(float* p, u4a v) {
    asm volatile("global_store_dwordx4 %0, %1, off sc1 nt\n\ts_nop 2" ::"v"(p), "v"(v) : "memory");
}

struct FusedGeo {       // per-bucket tiling, derived the same way by every block
    uint64_t bn;        // elements
    uint32_t k;
    uint32_t ntiles;    // streaming tiles
    uint32_t tpg;       // tiles per group
    uint32_t ng;        // groups
};
__device__ __forceinline__ FusedGeo fused_geo(const Geometry& g, BucketsArg bk, uint32_t b) {
    FusedGeo f;
    f.bn = bucket_count(g, bk, b);
    f.k = bucket_k(g, bk, b);
    f.ntiles = (uint32_t)((f.bn + kFTile - 1) / kFTile);
    f.tpg = (f.ntiles + kGroups - 1) / kGroups;
    f.ng = (f.ntiles + f.tpg - 1) / f.tpg;
    return f;
}

// Coarse window bin of a candidate key (key >= lo).
__device__ __forceinline__ uint32_t coarse_bin(uint32_t key, uint32_t lo, uint32_t hi, uint32_t shift) {
    return key >= hi ? (uint32_t)(kCoarse - 1) : (key - lo) >> shift;
}

// Waits until *p == want.  Called by a whole wavefront or a single thread; false when the wait timed out.
// Every poll is a memory transaction on one address (agent-scope loads are not cached):
// few pollers and a pause between polls, or the channel that holds the word becomes the
// bottleneck of every stream that crosses it.
__device__ __forceinline__ bool wait_word(const uint32_t* p, uint32_t want, uint64_t limit_ticks) {
    uint64_t t0 = 0;
    uint32_t polls = 0;
    while ((uint32_t)__builtin_amdgcn_readfirstlane((int)ld_agent(p)) != want) {
        __builtin_amdgcn_s_sleep(16);
        if ((++polls & 63u) == 0) {
            const uint64_t now = (uint64_t)wall_clock64();
            if (t0 == 0) t0 = now;
            else if (now - t0 > limit_ticks) return false;
        }
    }
    asm volatile("" ::: "memory");
    return true;
}

struct StreamLds {
    union {
        struct {  // sample block
            uint32_t lh[3][kBinsR];
            uint32_t scratch[3 * (kBlock / kWave + 2)];
        } s;
        struct {  // streaming block
            uint64_t stage[kFWaves][kWave];  // a wavefront's candidates, (bits << 32) | index, in index order
            uint32_t wcnt[kFWaves];
            uint32_t ready;
        } a;
        struct {  // bin block
            uint32_t dbuf[kFWaves][16 * kWave];  // dense_tile_walk's staging area, one per wavefront
            uint32_t cnt[kCoarse];
            uint32_t base[kCoarse];
            uint32_t flag;
        } e;
    };
};
struct SelectLds {
    uint32_t lh[kBins0];                 // radix rounds, tie-break, exact fallback
    // dense_tile_walk's staging area, one per wavefront; the threshold bin's list in between
    uint32_t dbuf[kFWaves][16 * kWave] __attribute__((aligned(8)));
    uint32_t part[kFWaves][kCoarse];
    uint32_t rcnt[kFWaves][kHeld];
    uint32_t wtot[kFWaves];
    uint32_t scratch[kBlock / kWave + 2];
    uint32_t flag;
};

// ---- sample ------------------------------------------------------------------------
// Radix-selects (11 + 10 key bits) three ranks of the sample: upper and lower end of the
// candidate window (6 sigma of the sampling noise away from the expected rank of the k-th
// largest key) and the predicted threshold; clears what the launch accumulates into;
// publishes the epoch.
__device__ __forceinline__ void fused_sample(BucketsArg bk, const Geometry& g, const Workspace& w, uint32_t b,
                                             uint32_t epoch, StreamLds& L) {
    const FusedGeo fg = fused_geo(g, bk, b);
#ifdef FUSED_TRACE
    const uint32_t tr_s0 = (uint32_t)wall_clock64();
#endif
    const uint64_t bn = fg.bn;
    const float* gp = bucket_grad(g, bk, b);
    const float* rp = bucket_residual(g, bk, b);
    const uint64_t nvec = bn / 4;
    constexpr int SV = kFSample / 4;     // sampled vectors
    constexpr int PV = SV / kBlock;      // vectors per thread; their 4 * PV keys stay in registers
    // sampled in runs of 8 vectors (one 128-byte line per array), runs evenly spread
    const uint32_t nsv = nvec < (uint64_t)SV ? (uint32_t)(nvec & ~7ull) : (uint32_t)SV;
    const uint64_t stride = nsv ? (nvec / (nsv / 8)) : 8;  // vectors between run starts (>= 8)
    // first of all, so that the acknowledgements are back long before the epoch is published: clear
    // what the launches accumulate into
    uint32_t* st = w.state + (uint64_t)b * kStateWords;
    if (threadIdx.x < kGroups) st_agent(w.grp_cnt + ((uint64_t)b * kGroups + threadIdx.x) * kCntStride, 0u);
    if (threadIdx.x < kCoarse) st_agent(w.bin_fill + (uint64_t)b * kCoarse + threadIdx.x, 0u);
    if (threadIdx.x == 0) {
        st_agent(st + S_BAR1, 0u);
        st_agent(st + S_OK, 0u);
        st_agent(st + S_TIMEOUT, 0u);
        st_agent(st + S_BARF, 0u); st_agent(st + S_BARF + 1, 0u); st_agent(st + S_BARF + 2, 0u); st_agent(st + S_BARF + 3, 0u);
    }
    // The sample is read twice (the second time from the cache): its keys need not stay in
    // registers, which this launch's streaming blocks could then not use either.
    auto for_keys = [&](auto&& body) {
        u4a gv[PV], rv[PV];
#pragma unroll
        for (int j = 0; j < PV; j++) {
            const uint32_t i = (uint32_t)j * kBlock + threadIdx.x;
            const uint32_t ii = i < nsv ? i : 0;
            const uint64_t v = (uint64_t)(ii >> 3) * stride + (ii & 7);
            gv[j] = nsv ? *(const u4u4*)(gp + v * 4) : u4a{0u, 0u, 0u, 0u};
            rv[j] = nsv ? *(const u4u4*)(rp + v * 4) : u4a{0u, 0u, 0u, 0u};
        }
#pragma unroll
        for (int j = 0; j < PV; j++) {
            if ((uint32_t)j * kBlock + threadIdx.x < nsv) {
#pragma unroll
                for (int q = 0; q < 4; q++) body(key_of(u2f(gv[j][q]) + u2f(rv[j][q])));
            }
        }
    };
    uint32_t* h0 = &L.s.lh[0][0];
    for (int i = threadIdx.x; i < 3 * kBinsR; i += kBlock) h0[i] = 0;
    const uint32_t S = nsv * 4;
    const float ks = (float)fg.k * (float)S / (float)bn;
    const float margin = 6.0f * sqrtf(ks) + 16.0f;
    // ranks: 0 upper end of the window, 1 lower end, 2 the predicted threshold itself
    constexpr int NR = 3;
    uint32_t rank[NR];
    rank[0] = ks - margin >= 1.0f ? (uint32_t)(ks - margin) : 0u;  // 0: no upper end
    rank[1] = (uint32_t)(ks + margin) + 1u;                       // > S: no lower end
    rank[2] = ks >= 1.0f ? (uint32_t)ks : 1u;
    uint32_t prefix[NR] = {0u, 0u, 0u}, want[NR] = {rank[0], rank[1], rank[2]};
    const bool active[NR] = {rank[0] >= 1u && rank[0] <= S, rank[1] <= S, rank[2] <= S};
    uint32_t rem[NR], bin[NR], left[NR];
    __syncthreads();
    // round 0, key[30:20]: lh[0] and lh[1] are adjacent, one 2048-bin histogram serves all ranks
    for_keys([&](uint32_t kq) { atomicAdd(&h0[kq >> 20], 1u); });
    __syncthreads();
#ifdef FUSED_TRACE
    const uint32_t tr_s1 = (uint32_t)wall_clock64();
#endif
#pragma unroll
    for (int z = 0; z < NR; z++) rem[z] = active[z] ? want[z] : 0u;
    {
        const uint32_t* const hs[NR] = {h0, h0, h0};
        pick_bins<kBins0, kBlock, NR>(hs, rem, bin, left, L.s.scratch);
    }
#pragma unroll
    for (int z = 0; z < NR; z++) {
        if (!active[z]) continue;
        prefix[z] |= bin[z] << 20;
        want[z] = left[z];
    }
#ifdef FUSED_TRACE
    const uint32_t tr_s2 = (uint32_t)wall_clock64();
#endif
    // round 1, key[19:10] among the keys that match a rank's first digit
    for (int i = threadIdx.x; i < NR * kBinsR; i += kBlock) h0[i] = 0;
    __syncthreads();
    for_keys([&](uint32_t kq) {
#pragma unroll
        for (int z = 0; z < NR; z++)
            if (active[z] && (kq >> 20) == (prefix[z] >> 20)) atomicAdd(&L.s.lh[z][(kq >> 10) & (kBinsR - 1)], 1u);
    });
    __syncthreads();
#ifdef FUSED_TRACE
    const uint32_t tr_s3 = (uint32_t)wall_clock64();
#endif
#pragma unroll
    for (int z = 0; z < NR; z++) rem[z] = active[z] ? want[z] : 0u;
    {
        const uint32_t* const hs[NR] = {L.s.lh[0], L.s.lh[1], L.s.lh[2]};
        pick_bins<kBinsR, kBlock, NR>(hs, rem, bin, left, L.s.scratch);
    }
#pragma unroll
    for (int z = 0; z < NR; z++) {
        if (!active[z]) continue;
        prefix[z] |= bin[z] << 10;
    }
#ifdef FUSED_TRACE
    const uint32_t tr_s4 = (uint32_t)wall_clock64();
#endif
    prefix[0] |= 0x3FFu;  // upper end of the window: rounded up
    prefix[2] |= 0x200u;  // predicted threshold: middle of its 1024-key cell
    // every store above must have arrived before the epoch is published
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    if (threadIdx.x == 0) {
        const uint32_t lo = active[1] ? prefix[1] : 0u;
        uint32_t hi = active[0] ? prefix[0] : 0x7FFFFFFFu;
        if (hi < lo) hi = lo;
        uint32_t shift = 0;
        while (((hi - lo) >> shift) >= (uint32_t)(kCoarse - 1)) shift++;
        // never below lo: every pre-zeroed element must be a listed candidate
        uint32_t that = active[2] ? prefix[2] : 0x7FFFFFFFu;
        if (that < lo) that = lo;
        st_agent(st + S_LO_KEY, lo);
        st_agent(st + S_HI_KEY, hi);
        st_agent(st + S_SHIFT, shift);
        st_agent(st + S_THAT, that);
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
#ifdef FUSED_TRACE
        st[25] = tr_s0;
        st[26] = (uint32_t)wall_clock64();
        st[27] = tr_s1; st[28] = tr_s2; st[29] = tr_s3; st[30] = tr_s4;
#endif
        st_agent(st + S_READY, epoch);
    }
    // off the critical path: the histograms of the exact selection, should the select launch need it
    for (int i = threadIdx.x; i < kHistWords; i += kBlock) w.hist[(uint64_t)b * kHistWords + i] = 0u;
}

// ---- a dense tile's elements ---------------------------------------------------------
// Calls f(index, bits, in_range) for every element of tile t of the bucket, 64 elements per
// step, every lane of the wavefront taking part in every step; the loads of 16 steps are in
// flight together and parked in LDS, so the code stays a loop.  AGENT: the residual was
// written by other blocks of the same launch.
template <bool AGENT, class F>
__device__ __forceinline__ void dense_tile_walk(const float* rp, uint64_t bn, uint32_t t, uint32_t* buf, F&& f) {
    const int lane = threadIdx.x & (kWave - 1);
    const uint64_t e0 = (uint64_t)t * kFTile;
    const uint64_t e1 = e0 + kFTile < bn ? e0 + kFTile : bn;
    constexpr int B = 16;
#pragma unroll 1
    for (uint64_t base = e0; base < e1; base += (uint64_t)B * kWave) {
        uint32_t v[B];
#pragma unroll
        for (int j = 0; j < B; j++) {
            const uint64_t i = base + (uint64_t)j * kWave + lane;
            if constexpr (AGENT) v[j] = i < e1 ? ld_agent((const uint32_t*)rp + i) : 0u;
            else v[j] = i < e1 ? f2u(rp[i]) : 0u;
        }
#pragma unroll
        for (int j = 0; j < B; j++) buf[j * kWave + lane] = v[j];  // a lane reads back only what it wrote
#pragma unroll 1
        for (int j = 0; j < B && base + (uint64_t)j * kWave < e1; j++) {  // wave-uniform trip count
            const uint64_t i = base + (uint64_t)j * kWave + lane;
            f((uint32_t)i, buf[j * kWave + lane], i < e1);
        }
    }
}

// ---- a group's tiles as a bin block / select block sees them ------------------------------
// The slots of up to kHeld tiles per wavefront stay in registers, the rest (buckets of more
// than 64 * 4 * kHeld tiles) are re-read from memory on every sweep.  AGENT: the slots were
// written by other blocks of the same launch (agent-scope loads), else by an earlier launch.
template <bool AGENT>
struct GroupTiles {
    const uint32_t* tcnt;
    const uint64_t* slots;
    uint32_t t0;        // the group's first tile
    uint32_t wt0, wt1;  // this wavefront's tiles: a contiguous quarter of the group's
    int lane;
    bool more;          // wave-uniform: dense tiles, or tiles past the register window
    uint32_t cnt[kHeld];            // candidates in the tile's slots, or kDense (wave-uniform)
    uint64_t e0[kHeld], e1[kHeld];  // slot `lane` and slot `64 + lane`

    static __device__ __forceinline__ uint32_t ld32(const uint32_t* p) {
        if constexpr (AGENT) return ld_agent(p);
        else return *p;
    }
    static __device__ __forceinline__ uint64_t ld64(const uint64_t* p) {
        if constexpr (AGENT) return ld_agent64(p);
        else return *p;
    }
    // every load issued at once
    __device__ __forceinline__ void load(const Geometry& g, const Workspace& w, uint32_t b, uint32_t grp,
                                         const FusedGeo& fg) {
        constexpr int NW = kBlock / kWave;
        lane = threadIdx.x & (kWave - 1);
        const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x / kWave));
        tcnt = w.tile_cnt + (uint64_t)b * g.ftiles;
        slots = w.slots + (uint64_t)b * g.ftiles * kTileSlots;
        t0 = grp * fg.tpg;
        const uint32_t t1 = t0 + fg.tpg < fg.ntiles ? t0 + fg.tpg : fg.ntiles;
        const uint32_t pw = (t1 - t0 + NW - 1) / NW;
        wt0 = t0 + wave * pw < t1 ? t0 + wave * pw : t1;
        wt1 = wt0 + pw < t1 ? wt0 + pw : t1;
#pragma unroll
        for (int h = 0; h < kHeld; h++) {
            const uint32_t t = wt0 + h < wt1 ? wt0 + h : t0;  // stays inside the bucket's arrays
            cnt[h] = (uint32_t)__builtin_amdgcn_readfirstlane((int)ld32(tcnt + t));
            e0[h] = ld64(slots + (uint64_t)t * kTileSlots + lane);  // slots past the count: ignored by the sweeps
            e1[h] = ld64(slots + (uint64_t)t * kTileSlots + kWave + lane);
        }
        bool any_dense = false;
#pragma unroll
        for (int h = 0; h < kHeld; h++) any_dense |= wt0 + h < wt1 && cnt[h] == kDense;
        more = any_dense || wt1 > wt0 + kHeld;
    }
    // nd(h, t, cnt, e0, e1) for every ordinary tile (h < kHeld: register-held, else ~0u), dn(h, t)
    // for every dense one.  Order: register-held ordinary tiles first, then the dense ones and
    // those past the register window, in index order.
    template <class ND, class DN>
    __device__ __forceinline__ void sweep(ND&& nd, DN&& dn) const {
#pragma unroll
        for (int h = 0; h < kHeld; h++)
            if (wt0 + h < wt1 && cnt[h] != kDense) nd((uint32_t)h, wt0 + h, cnt[h], e0[h], e1[h]);
        if (more) {
#pragma unroll 1
            for (uint32_t t = wt0; t < wt1; t++) {
                const uint32_t h = t - wt0 < (uint32_t)kHeld ? t - wt0 : ~0u;
                const uint32_t c = (uint32_t)__builtin_amdgcn_readfirstlane((int)ld32(tcnt + t));
                if (c == kDense) {
                    dn(h, t);
                } else if (h == ~0u) {
                    const uint64_t a0 = ld64(slots + (uint64_t)t * kTileSlots + lane);
                    const uint64_t a1 = ld64(slots + (uint64_t)t * kTileSlots + kWave + lane);
                    nd(h, t, c, a0, a1);
                }
            }
        }
    }
};
__device__ __forceinline__ uint32_t key64(uint64_t e) { return (uint32_t)(e >> 32) & 0x7FFFFFFFu; }

__device__ __forceinline__ void fused_give_up(uint32_t* st, uint32_t* out) {
    if (threadIdx.x == 0) {
        st_agent(st + S_TIMEOUT, 1u);
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        st_agent(out, kPoisonK);
    }
}

// ---- bin block -----------------------------------------------------------------------------
__device__ __forceinline__ void fused_bin(BucketsArg bk, const Geometry& g, const Workspace& w, uint32_t b,
                                          uint32_t grp, const FusedGeo& fg, uint32_t epoch, uint64_t limit_ticks,
                                          StreamLds& L) {
    uint32_t* st = w.state + (uint64_t)b * kStateWords;
    // the group's tiles are finished: all its streaming blocks have arrived
    {
        const uint32_t tg0 = grp * fg.tpg;
        const uint32_t in_group = (tg0 + fg.tpg < fg.ntiles ? tg0 + fg.tpg : fg.ntiles) - tg0;
        // the counter is only meaningful once the sample block has cleared it
        if (threadIdx.x == 0)
            L.e.flag = wait_word(st + S_READY, epoch, limit_ticks) &&
                       wait_word(w.grp_cnt + ((uint64_t)b * kGroups + grp) * kCntStride, in_group, limit_ticks);
        __syncthreads();
        if (!L.e.flag) {
            fused_give_up(st, bucket_wire(g, bk, b));
            return;
        }
    }
#ifdef FUSED_TRACE
    if (threadIdx.x == 0) w.list2[((uint64_t)b * kGroups + grp) * 4 + 0] = (uint32_t)wall_clock64();
#endif
    const uint32_t lo = ld_agent(st + S_LO_KEY), hi = ld_agent(st + S_HI_KEY), shift = ld_agent(st + S_SHIFT);
    const uint64_t bn = fg.bn;
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x / kWave));
    const float* rp = bucket_residual(g, bk, b);
    GroupTiles<true> G;
    G.load(g, w, b, grp, fg);
    // candidates per coarse bin
    if (threadIdx.x < kCoarse) L.e.cnt[threadIdx.x] = 0;
    __syncthreads();
    G.sweep([&](uint32_t, uint32_t, uint32_t cnt, uint64_t a0, uint64_t a1) {
                if ((uint32_t)lane < cnt) atomicAdd(&L.e.cnt[coarse_bin(key64(a0), lo, hi, shift)], 1u);
                if ((uint32_t)(kWave + lane) < cnt) atomicAdd(&L.e.cnt[coarse_bin(key64(a1), lo, hi, shift)], 1u);
            },
            [&](uint32_t, uint32_t t) {
                dense_tile_walk<true>(rp, bn, t, L.e.dbuf[wave], [&](uint32_t, uint32_t v, bool in) {
                    const uint32_t key = v & 0x7FFFFFFFu;
                    const bool cand = in && key >= lo;
                    wave_hist_add(L.e.cnt, cand, cand ? coarse_bin(key, lo, hi, shift) : 0u);
                });
            });
    __syncthreads();
    if (threadIdx.x < kCoarse) {
        const uint32_t c = L.e.cnt[threadIdx.x];
        w.ghist[((uint64_t)b * kGroups + grp) * kCoarse + threadIdx.x] = c;
        // the top bin (keys >= hi) holds picks for certain as long as the window holds: no list
        L.e.base[threadIdx.x] = (c && threadIdx.x < kCoarse - 1)
            ? __hip_atomic_fetch_add(w.bin_fill + (uint64_t)b * kCoarse + threadIdx.x, c, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)
            : 0u;
    }
    __syncthreads();
    // binned copies (read by the next launch: plain stores)
    uint64_t* bl = w.blist + (uint64_t)b * (kCoarse - 1) * g.lcapb;
    auto put = [&](bool valid, uint32_t cb, uint64_t e) {
        if (valid && cb < (uint32_t)(kCoarse - 1)) {
            const uint32_t pos = atomicAdd(&L.e.base[cb], 1u);
            if (pos < g.lcapb) bl[(uint64_t)cb * g.lcapb + pos] = e;
        }
    };
    G.sweep([&](uint32_t, uint32_t, uint32_t cnt, uint64_t a0, uint64_t a1) {
                put((uint32_t)lane < cnt, coarse_bin(key64(a0), lo, hi, shift), a0);
                put((uint32_t)(kWave + lane) < cnt, coarse_bin(key64(a1), lo, hi, shift), a1);
            },
            [&](uint32_t, uint32_t t) {
                dense_tile_walk<true>(rp, bn, t, L.e.dbuf[wave], [&](uint32_t i, uint32_t v, bool in) {
                    const uint32_t key = v & 0x7FFFFFFFu;
                    const bool cand = in && key >= lo;
                    put(cand, cand ? coarse_bin(key, lo, hi, shift) : 0u, (uint64_t)i | ((uint64_t)v << 32));
                });
            });
#ifdef FUSED_TRACE
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    if (threadIdx.x == 0) w.list2[((uint64_t)b * kGroups + grp) * 4 + 1] = (uint32_t)wall_clock64();
#endif
}

// ---- the streaming launch ------------------------------------------------------------------
__global__ __launch_bounds__(kBlock, 5) void k_topk_stream(Buckets, Geometry g, Workspace w, uint32_t epoch,
                                                        uint32_t first_wave, uint64_t limit_ticks) {
    const BucketsArg bk = buckets_arg();
    __shared__ StreamLds L;
    if (blockIdx.x < g.nbuckets) {
        fused_sample(bk, g, w, blockIdx.x, epoch, L);
        return;
    }
    // segment s of the grid: the tiles of bucket s, then the bin blocks of bucket s - 1 (whose
    // tiles are finished or about to be by then: a bin block that is dispatched early only
    // polls); after the last segment the bin blocks of the last bucket
    const uint32_t per = g.ftiles + kGroups;
    const uint32_t j = blockIdx.x - g.nbuckets;
    uint32_t b = j / per, t = j - b * per;
    bool emit = false;
    if (b >= g.nbuckets) {
        t = j - g.nbuckets * per;
        b = g.nbuckets - 1;
        emit = true;
    } else if (t >= g.ftiles) {
        if (b == 0) return;
        t -= g.ftiles;
        b -= 1;
        emit = true;
    }
#ifdef FUSED_TRACE
    const uint32_t tr_start = (uint32_t)wall_clock64();
#endif
    const FusedGeo fg = fused_geo(g, bk, b);
    if (emit) {
#ifdef FUSED_TRACE
        if (threadIdx.x == 0 && t < fg.ng) w.list2[((uint64_t)b * kGroups + t) * 4 + 2] = tr_start;
#endif
        if (t < fg.ng) fused_bin(bk, g, w, b, t, fg, epoch, limit_ticks, L);
        return;
    }
    if (t >= fg.ntiles) return;
    // The blocks that start together with the sample blocks would bury the samples' few loads under
    // 40 MB of their own and then wait for the samples all the same: they hold back for two
    // microseconds, and the memory system is busy with their loads while the samples are evaluated.
    if (blockIdx.x < first_wave) __builtin_amdgcn_s_sleep(80);
    const uint64_t bn = fg.bn;
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x / kWave));
    const uint64_t w0 = (uint64_t)t * kFTile + (uint64_t)wave * kFRegion;  // first element of this wave's region
    const bool live = w0 < bn;                                             // wave-uniform
    float* const rbase = bucket_residual(g, bk, b);
    const float* gp = bucket_grad(g, bk, b) + w0;
    float* rp = rbase + w0;
    const uint32_t len = live ? (uint32_t)((bn - w0) < (uint64_t)kFRegion ? (bn - w0) : (uint64_t)kFRegion) : 0u;
    const uint32_t nfull = len / 4;  // full vectors in this region
    u4a gv[kFVecs], rv[kFVecs];
#pragma unroll
    for (int u = 0; u < kFVecs; u++) {
        const uint32_t vi = (uint32_t)u * kWave + lane;
        if (vi < nfull) {
            gv[u] = __builtin_nontemporal_load((const u4u4*)(gp + vi * 4));
            rv[u] = __builtin_nontemporal_load((const u4u4*)(rp + vi * 4));
        }
    }
    uint32_t* st = w.state + (uint64_t)b * kStateWords;
    uint32_t* out = bucket_wire(g, bk, b);
    // the window of this bucket: wait for its sample block (one wavefront polls for the block)
    if (wave == 0) {
        const bool r0 = wait_word(st + S_READY, epoch, limit_ticks);
        if (lane == 0) L.a.ready = r0 ? 1u : 0u;
    }
    __syncthreads();
    const bool ready = L.a.ready != 0;
#ifdef FUSED_TRACE
    const uint32_t tr_ready = (uint32_t)wall_clock64();
#endif
    const uint32_t lo_key = ld_agent(st + S_LO_KEY), that_key = ld_agent(st + S_THAT);
    // both the same in every lane, and kept in scalar registers by saying so at every update
    uint32_t staged = 0;  // candidates of the region so far
    uint32_t dense = 0;   // 1: more candidates than slots
    uint64_t* const slots = L.a.stage[wave];
    auto lanes_below = [&](uint64_t m) {
        return (uint32_t)__builtin_amdgcn_mbcnt_hi((uint32_t)(m >> 32), __builtin_amdgcn_mbcnt_lo((uint32_t)m, 0u));
    };
    auto pick = [](const u4a& a, uint32_t q) {
        uint32_t v = a[0];
        v = q == 1 ? a[1] : v;
        v = q == 2 ? a[2] : v;
        return q == 3 ? a[3] : v;
    };
    // Puts back the region's staged candidates that were stored as zeros.
    auto restore_staged = [&]() {
        if ((uint32_t)lane < staged) {
            const uint64_t e = slots[lane];
            if (((uint32_t)(e >> 32) & 0x7FFFFFFFu) >= that_key) st_agent((uint32_t*)rbase + (uint32_t)e, (uint32_t)(e >> 32));
        }
    };
    // Appends the lanes' candidates (mask4: which of a lane's four elements) in index
    // order: lane-major, element-minor.  Nearly every call finds a few lanes with one
    // candidate each: one ballot, one 8-byte LDS store.
    auto append = [&](uint32_t mask4, const u4a& a, uint32_t first_idx) {
        const uint64_t m1 = __ballot(mask4 != 0);
        if (!m1) return;  // wave-uniform
        const uint32_t c = __popc(mask4);
        uint32_t before = lanes_below(m1), total = __popcll(m1);
        const uint64_t m2 = __ballot(c >= 2);
        if (m2) {  // wave-uniform
            before += lanes_below(m2);
            total += __popcll(m2);
            const uint64_t m3 = __ballot(c >= 3);
            if (m3) {
                const uint64_t m4 = __ballot(c >= 4);
                before += lanes_below(m3) + lanes_below(m4);
                total += __popcll(m3) + __popcll(m4);
            }
        }
        if (dense) return;
        total = (uint32_t)__builtin_amdgcn_readfirstlane((int)total);
        if (staged + total > (uint32_t)kWave) {
            // the region goes dense: its earlier candidates were stored as zeros where
            // they reached the predicted threshold; put those values back
            dense = 1u;
            restore_staged();
            return;
        }
        if (mask4) {
            uint32_t pos = staged + before;
            const uint32_t q = (uint32_t)__ffs((int)mask4) - 1u;
            slots[pos] = (uint64_t)(first_idx + q) | ((uint64_t)pick(a, q) << 32);
            uint32_t rest = mask4 & (mask4 - 1u);
            while (rest) {
                const uint32_t q2 = (uint32_t)__ffs((int)rest) - 1u;
                slots[++pos] = (uint64_t)(first_idx + q2) | ((uint64_t)pick(a, q2) << 32);
                rest &= rest - 1u;
            }
        }
        staged = (uint32_t)__builtin_amdgcn_readfirstlane((int)(staged + total));
    };
    if (ready) {
#pragma unroll
        for (int u = 0; u < kFVecs; u++) {
            const uint32_t vi = (uint32_t)u * kWave + lane;
            u4a a = {0u, 0u, 0u, 0u}, z = {0u, 0u, 0u, 0u};
            uint32_t mask4 = 0;
            if (vi < nfull) {
#pragma unroll
                for (int q = 0; q < 4; q++) {
                    const float adj = u2f(gv[u][q]) + u2f(rv[u][q]);
                    a[q] = f2u(adj);
                    z[q] = key_of(adj) >= that_key ? 0u : a[q];
                    mask4 |= (key_of(adj) >= lo_key ? 1u : 0u) << q;
                }
            }
            append(mask4, a, (uint32_t)w0 + vi * 4);  // may turn the region dense
            if (vi < nfull) store_through(rp + vi * 4, dense ? a : z);
        }
        // the bucket's last partial vector (bucket length not a multiple of 4) lies in its last region
        if (len & 3) {
            u4a a = {0u, 0u, 0u, 0u};
            uint32_t mask4 = 0;
            if (lane == 0) {
                for (uint32_t q = 0; q < (len & 3); q++) {
                    const float adj = gp[nfull * 4 + q] + rp[nfull * 4 + q];
                    a[q] = f2u(adj);
                    mask4 |= (key_of(adj) >= lo_key ? 1u : 0u) << q;
                }
            }
            append(mask4, a, (uint32_t)w0 + nfull * 4);
            if (lane == 0) {
                for (uint32_t q = 0; q < (len & 3); q++)
                    st_agent((uint32_t*)rp + nfull * 4 + q, (!dense && (a[q] & 0x7FFFFFFFu) >= that_key) ? 0u : a[q]);
            }
        }
    }
    // ---- the tile's candidates, in index order, to its slots ------------------------------
    if (lane == 0) L.a.wcnt[wave] = !ready ? kGaveUp : (dense ? kDense : staged);
    __syncthreads();
    uint32_t before = 0, total = 0;
    bool tile_dense = false, gave_up = false;
#pragma unroll
    for (int i = 0; i < kFWaves; i++) {
        const uint32_t c = L.a.wcnt[i];
        gave_up |= c == kGaveUp;
        tile_dense |= c == kDense;
        if (i < wave) before += c;
        total += c;
    }
    if (gave_up) {  // a wavefront never saw the sample arrive: the bucket's result is invalid
        fused_give_up(st, out);
        return;     // without counting the tile: the bucket's bin blocks give up as well
    }
    tile_dense |= total > (uint32_t)kTileSlots;
    if (tile_dense) {
        if (!dense) restore_staged();  // a tile is dense as a whole: its residual holds plain sums
    } else if ((uint32_t)lane < staged) {
        st_agent64(w.slots + ((uint64_t)b * g.ftiles + t) * kTileSlots + before + lane, slots[lane]);
    }
    if (threadIdx.x == 0) st_agent(w.tile_cnt + (uint64_t)b * g.ftiles + t, tile_dense ? kDense : total);
    // ---- the block counts itself into its group once all its stores have arrived ----------
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
#ifdef FUSED_TRACE
    if (threadIdx.x == 0) {
        w.tile_gt[(uint64_t)b * g.tiles + t] = tr_start;
        w.tile_eq[(uint64_t)b * g.tiles + t] = (uint32_t)wall_clock64();
        w.reg_cnt[(uint64_t)b * g.regions + t] = tr_ready;
    }
#endif
    if (threadIdx.x == 0)
        __hip_atomic_fetch_add(w.grp_cnt + ((uint64_t)b * kGroups + t / fg.tpg) * kCntStride, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// The need-th smallest index among the list's entries with key == T: radix select over
// the index, 11 + 11 + 10 bits.  Called by all threads of the block.
__device__ __forceinline__ uint32_t resolve_ties64(const uint64_t* l2, uint32_t count2, uint32_t T, uint32_t need,
                                                   uint32_t* lh /* kBins0 words */, uint32_t* scratch) {
    uint32_t iwant = need, iprefix = 0;
    const int shifts[3] = {21, 10, 0};
    const int widths[3] = {11, 11, 10};
    for (int r = 0; r < 3; r++) {
        const int bins = 1 << widths[r];
        for (int i = threadIdx.x; i < kBins0; i += kBlock) lh[i] = 0;
        __syncthreads();
        const int hs = shifts[r] + widths[r];
        for (uint32_t i = threadIdx.x; i < count2; i += kBlock) {
            const uint64_t e = l2[i];
            const uint32_t idx = (uint32_t)e, key = (uint32_t)(e >> 32) & 0x7FFFFFFFu;
            const bool match = hs >= 32 ? true : ((idx >> hs) == (iprefix >> hs));
            // bins stored reversed, so that pick_bin's top-down scan runs over ascending indices
            if (key == T && match) atomicAdd(&lh[(bins - 1) - ((idx >> shifts[r]) & (bins - 1))], 1u);
        }
        __syncthreads();
        uint32_t left;
        const uint32_t rb = pick_bin<kBins0, kBlock>(lh, iwant, 0, &left, scratch);
        iprefix |= ((uint32_t)(bins - 1) - (rb - (uint32_t)(kBins0 - bins))) << shifts[r];
        iwant = left;
    }
    return iprefix;
}


// The exact selection of one bucket by its select blocks together (same algorithm as the exact
// path: three radix rounds over the key, then an ordered emit), each on its own group's
// element range; four barriers.  Returns false when a barrier wait timed out.
__device__ __forceinline__ bool select_exact_group(BucketsArg bk, const Geometry& g, const Workspace& w, uint32_t b,
                                                   uint32_t grp, const FusedGeo& fg, uint32_t that_key,
                                                   const GroupTiles<false>& G, SelectLds& L, uint64_t limit_ticks) {
    uint32_t* st = w.state + (uint64_t)b * kStateWords;
    const uint64_t bn = fg.bn;
    float* rp = bucket_residual(g, bk, b);
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = threadIdx.x / kWave;
    const uint64_t below = (1ull << lane) - 1ull;
    const uint64_t e0 = (uint64_t)grp * fg.tpg * kFTile;
    const uint64_t e1r = e0 + (uint64_t)fg.tpg * kFTile;
    const uint64_t e1 = e1r < bn ? e1r : bn;
    // 1: put back what the streaming blocks stored as 0.0f in this group's tiles
    G.sweep([&](uint32_t, uint32_t, uint32_t cnt, uint64_t a0, uint64_t a1) {
                if ((uint32_t)lane < cnt && key64(a0) >= that_key) rp[(uint32_t)a0] = u2f((uint32_t)(a0 >> 32));
                if ((uint32_t)(kWave + lane) < cnt && key64(a1) >= that_key) rp[(uint32_t)a1] = u2f((uint32_t)(a1 >> 32));
            },
            [&](uint32_t, uint32_t) {});
    __syncthreads();  // a block only ever reads the range it restored itself: plain accesses
    // 2: radix select; every wavefront walks a contiguous quarter of the group's range
    constexpr int NW = kBlock / kWave;
    const uint64_t quarter = ((e1 - e0 + NW - 1) / NW + kWave - 1) / kWave * kWave;
    const uint64_t ws0 = e0 + (uint64_t)wave * quarter < e1 ? e0 + (uint64_t)wave * quarter : e1;
    const uint64_t ws1 = ws0 + quarter < e1 ? ws0 + quarter : e1;
    auto walk = [&](auto&& f) {
        constexpr int B = 8;
#pragma unroll 1
        for (uint64_t base = ws0; base < ws1; base += (uint64_t)B * kWave) {
            uint32_t v[B];
#pragma unroll
            for (int j = 0; j < B; j++) {
                const uint64_t i = base + (uint64_t)j * kWave + lane;
                v[j] = i < ws1 ? f2u(rp[i]) : 0u;
            }
#pragma unroll
            for (int j = 0; j < B; j++) {
                const uint64_t i = base + (uint64_t)j * kWave + lane;
                if (base + (uint64_t)j * kWave < ws1) f(i, v[j], i < ws1);  // wave-uniform
            }
        }
    };
    uint32_t* lh = L.lh;
    uint32_t* gh = w.hist + (uint64_t)b * kHistWords;  // cleared by the bucket's sample block
    uint32_t prefix = 0, remaining = fg.k;
#pragma unroll 1
    for (int round = 0; round < 3; round++) {
        const int bins = round == 0 ? kBins0 : kBinsR;
        const int shift = round == 0 ? 20 : (round == 1 ? 10 : 0);
        const int hi_shift = round == 0 ? 31 : shift + 10;
        uint32_t* ghr = gh + (round == 0 ? 0 : (round == 1 ? kBins0 : kBins0 + kBinsR));
        for (int i = threadIdx.x; i < kBins0; i += kBlock) lh[i] = 0;
        __syncthreads();
        walk([&](uint64_t, uint32_t v, bool valid) {
            const uint32_t key = v & 0x7FFFFFFFu;
            wave_hist_add(lh, valid && (key >> hi_shift) == (prefix >> hi_shift), (key >> shift) & (uint32_t)(bins - 1));
        });
        __syncthreads();
        for (int i = threadIdx.x; i < bins; i += kBlock) {
            const uint32_t c = lh[i];
            if (c) __hip_atomic_fetch_add(&ghr[i], c, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
        if (!bucket_barrier(st + S_BARF + round, fg.ng, &L.flag, limit_ticks)) return false;
        for (int i = threadIdx.x; i < bins; i += kBlock) lh[i] = ld_agent(&ghr[i]);
        __syncthreads();
        uint32_t left, bin;
        if (round == 0) bin = pick_bin<kBins0, kBlock>(lh, remaining, 0, &left, L.scratch);
        else bin = pick_bin<kBinsR, kBlock>(lh, remaining, 0, &left, L.scratch);
        prefix |= bin << shift;
        remaining = left;
    }
    const uint32_t T = prefix, need = remaining;
    // 3: keys above and at the threshold per wavefront range, per group, and in the groups before
    uint32_t gt_w = 0, eq_w = 0;  // wave-uniform
    walk([&](uint64_t, uint32_t v, bool valid) {
        const uint32_t key = v & 0x7FFFFFFFu;
        gt_w += (uint32_t)__popcll(__ballot(valid && key > T));
        eq_w += (uint32_t)__popcll(__ballot(valid && key == T));
    });
    uint32_t* wsum = lh;  // LDS words free again: [0..NW) above, [NW..2NW) equal
    __syncthreads();
    if (lane == 0) { wsum[wave] = gt_w; wsum[NW + wave] = eq_w; }
    __syncthreads();
    uint32_t gt_run = 0, eq_run = 0, gt_blk = 0, eq_blk = 0;
#pragma unroll
    for (int i = 0; i < NW; i++) {
        if (i < wave) { gt_run += wsum[i]; eq_run += wsum[NW + i]; }
        gt_blk += wsum[i];
        eq_blk += wsum[NW + i];
    }
    if (threadIdx.x == 0) {
        st_agent(&w.blk_above[(uint64_t)b * kGroups + grp], gt_blk);
        st_agent(&w.blk_eq[(uint64_t)b * kGroups + grp], eq_blk);
    }
    if (!bucket_barrier(st + S_BARF + 3, fg.ng, &L.flag, limit_ticks)) return false;
    {
        static_assert(kGroups <= kBlock, "one thread per group of the bucket");
        const uint32_t vg = threadIdx.x < grp ? ld_agent(&w.blk_above[(uint64_t)b * kGroups + threadIdx.x]) : 0u;
        const uint32_t ve = threadIdx.x < grp ? ld_agent(&w.blk_eq[(uint64_t)b * kGroups + threadIdx.x]) : 0u;
        uint32_t gt_before, eq_before;
        block_exclusive_scan(vg, L.scratch, &gt_before);
        block_exclusive_scan(ve, L.scratch, &eq_before);
        gt_run += gt_before;
        eq_run += eq_before;
    }
    // 4: this wavefront's picks, in index order
    uint32_t* out = bucket_wire(g, bk, b);
    walk([&](uint64_t i, uint32_t v, bool valid) {
        const uint32_t key = v & 0x7FFFFFFFu;
        const bool is_gt = valid && key > T, is_eq = valid && key == T;
        const uint64_t mg = __ballot(is_gt), me = __ballot(is_eq);
        const uint32_t gt_b = gt_run + (uint32_t)__popcll(mg & below);
        const uint32_t eq_b = eq_run + (uint32_t)__popcll(me & below);
        if (is_gt || (is_eq && eq_b < need)) {
            const uint32_t pos = gt_b + (eq_b < need ? eq_b : need);
            out[1 + 2 * (uint64_t)pos] = (uint32_t)i;
            out[2 + 2 * (uint64_t)pos] = v;
            rp[i] = 0.0f;
        }
        gt_run += (uint32_t)__popcll(mg);
        eq_run += (uint32_t)__popcll(me);
    });
    if (grp == 0 && threadIdx.x == 0) {
        st[S_T] = T;
        st[S_NEED] = need;
    }
    return true;
}


// ---- the select launch ----------------------------------------------------------------------
// blockIdx.x = group, blockIdx.y = bucket - first_bucket.  Everything the streaming launch
// left behind is read with plain loads; only the exact fallback talks across blocks.
__global__ __launch_bounds__(kBlock, 4) void k_topk_select(Buckets, Geometry g, Workspace w, uint32_t first_bucket,
                                                           uint64_t limit_ticks) {
    const BucketsArg bk = buckets_arg();
    __shared__ SelectLds L;
    constexpr int NW = kBlock / kWave;
    const uint32_t b = first_bucket + blockIdx.y, grp = blockIdx.x;
    const FusedGeo fg = fused_geo(g, bk, b);
    if (grp >= fg.ng) return;
    uint32_t* st = w.state + (uint64_t)b * kStateWords;
    uint32_t* out = bucket_wire(g, bk, b);
    if (st[S_TIMEOUT]) return;  // the streaming launch gave the bucket up: its payload header says so
    if (grp == 0 && threadIdx.x == 0) st[S_READY] = 0u;  // a replay of a captured launch carries the same epoch
    GroupTiles<false> G;
    G.load(g, w, b, grp, fg);
    const uint32_t lo = st[S_LO_KEY], hi = st[S_HI_KEY], shift = st[S_SHIFT], that_key = st[S_THAT];
    (void)hi;
    const uint32_t k = fg.k;
    const uint64_t bn = fg.bn;
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x / kWave));
    const uint64_t below = (1ull << lane) - 1ull;
    float* rp = bucket_residual(g, bk, b);

    bool failed = false;
    do {
    // ---- 3: threshold bin from the groups' counts -------------------------------------------
    // thread (wave, lane): bin `lane` of groups [16 wave, 16 wave + 16)
    constexpr int GPW = kGroups / NW;
    uint32_t gh[GPW];
    uint32_t mine = 0;
#pragma unroll
    for (int i = 0; i < GPW; i++) {
        const uint32_t gi = (uint32_t)(wave * GPW + i);
        gh[i] = gi < fg.ng ? w.ghist[((uint64_t)b * kGroups + gi) * kCoarse + lane] : 0u;
        mine += gh[i];
    }
    L.part[wave][lane] = mine;
    __syncthreads();
    // scanned from the top bin downwards: lane l looks at bin 63 - l
    uint32_t totr = 0;
#pragma unroll
    for (int i = 0; i < NW; i++) totr += L.part[i][kCoarse - 1 - lane];
    const uint32_t inc = wave_inclusive_scan(totr);
    const uint64_t reach = __ballot(inc >= k);
    if (!reach) {  // fewer than k candidates
        failed = true;
        break;
    }
    const int lstar = __ffsll((long long)reach) - 1;
    const uint32_t jstar = (uint32_t)(kCoarse - 1 - lstar);
    if (jstar == (uint32_t)(kCoarse - 1)) {  // the threshold lies at or above the window's upper end
        failed = true;
        break;
    }
    const uint32_t n2 = (uint32_t)__shfl((int)totr, lstar, kWave);          // candidates in the threshold bin
    const uint32_t above_total = (uint32_t)__shfl((int)inc, lstar, kWave) - n2;
    const uint32_t need = k - above_total;                                   // picks inside the bin, 1..n2
    // certain picks (bins above the threshold bin) in the groups before this one
    uint32_t ab = 0;
#pragma unroll
    for (int i = 0; i < GPW; i++)
        if ((uint32_t)lane > jstar && (uint32_t)(wave * GPW + i) < grp) ab += gh[i];
    uint32_t above_before;
    block_exclusive_scan(ab, L.scratch, &above_before);
    if (n2 > g.lcapb) {  // more keys in the threshold bin than its list holds (heavy ties, clustered values)
        failed = true;
        break;
    }

    // ---- 4: exact threshold from the bin's list ---------------------------------------------
    const uint64_t* l2 = w.blist + ((uint64_t)b * (kCoarse - 1) + jstar) * g.lcapb;
    // the first 2048 entries are parked in LDS (the dense walks' staging area is idle until the emit)
    constexpr uint32_t kL2Cached = kFWaves * 16 * kWave / 2;
    uint64_t* const lcache = (uint64_t*)&L.dbuf[0][0];
    {
        constexpr int PER = kL2Cached / kBlock;
        uint64_t ent[PER];
#pragma unroll
        for (int j = 0; j < PER; j++) {
            const uint32_t i = (uint32_t)j * kBlock + threadIdx.x;
            ent[j] = i < n2 ? l2[i] : 0ull;
        }
#pragma unroll
        for (int j = 0; j < PER; j++) lcache[(uint32_t)j * kBlock + threadIdx.x] = ent[j];  // a thread reads back only what it wrote
    }
    auto for_list2 = [&](auto&& body) {
#pragma unroll 1
        for (uint32_t i = threadIdx.x; i < n2; i += kBlock) {
            const uint64_t e = i < kL2Cached ? lcache[i] : l2[i];
            body((uint32_t)e, key64(e));
        }
    };
    uint32_t* lh = L.lh;
    const uint32_t bin_lo = lo + (jstar << shift);  // smallest key of the threshold bin
    uint32_t vprefix = 0, want = need;              // key - bin_lo: up to 30 bits, selected as 10 + 10 + 10
    // a bin spans 2^shift keys: rounds whose digits lie wholly above that are skipped
    const int first_round = shift <= 10 ? 2 : (shift <= 20 ? 1 : 0);
#pragma unroll 1
    for (int r = first_round; r < 3; r++) {
        const int sh = 20 - 10 * r;
        const int hs = sh + 10;
        for (int i = threadIdx.x; i < kBinsR; i += kBlock) lh[i] = 0;
        __syncthreads();
        for_list2([&](uint32_t, uint32_t key) {
            const uint32_t v = key - bin_lo;
            if ((v >> hs) == (vprefix >> hs)) atomicAdd(&lh[(v >> sh) & (kBinsR - 1)], 1u);
        });
        __syncthreads();
        uint32_t left;
        const uint32_t bin = pick_bin<kBinsR, kBlock>(lh, want, 0, &left, L.scratch);
        if (bin >= (uint32_t)kBinsR) {  // the list holds fewer matching keys than the counts promised
            failed = true;
            break;
        }
        vprefix |= bin << sh;
        want = left;
    }
    if (failed) break;
    const uint32_t T = bin_lo + vprefix;
    const uint32_t need2 = want;
    const uint32_t ties = lh[vprefix & (kBinsR - 1)];
    __syncthreads();
    // when only some keys equal to T are taken, they are the need2 lowest indices
    const uint32_t istar = ties != need2 ? resolve_ties64(l2, n2, T, need2, lh, L.scratch) : 0xFFFFFFFFu;
    auto is_pick = [&](bool valid, uint32_t key, uint32_t idx) {
        return valid && (key > T || (key == T && idx <= istar));
    };
    // the threshold bin's picks at indices below this group's first element
    uint32_t mine_before = 0, mine_all = 0;
    const uint64_t first_elem = (uint64_t)G.t0 * kFTile;
    for_list2([&](uint32_t idx, uint32_t key) {
        if (is_pick(true, key, idx)) {
            mine_all++;
            mine_before += (uint64_t)idx < first_elem ? 1u : 0u;
        }
    });
    uint32_t l2_before, l2_total;
    block_exclusive_scan(mine_before, L.scratch, &l2_before);
    block_exclusive_scan(mine_all, L.scratch, &l2_total);
    if (above_total + l2_total != k) {  // cannot happen with consistent lists
        failed = true;
        break;
    }

    // ---- 5: payload, in index order -----------------------------------------------------------
    // picks per tile first: the register-held tiles' into rcnt, the others' into the total
    uint32_t w_total = 0;
    G.sweep([&](uint32_t h, uint32_t, uint32_t cnt, uint64_t a0, uint64_t a1) {
              const uint32_t c = (uint32_t)__popcll(__ballot(is_pick((uint32_t)lane < cnt, key64(a0), (uint32_t)a0))) +
                                 (uint32_t)__popcll(__ballot(is_pick((uint32_t)(kWave + lane) < cnt, key64(a1), (uint32_t)a1)));
              if (h != ~0u) L.rcnt[wave][h] = c;
              w_total += c;
          },
          [&](uint32_t h, uint32_t t) {
              uint32_t c = 0;
              dense_tile_walk<false>(rp, bn, t, L.dbuf[wave], [&](uint32_t i, uint32_t v, bool in) {
                  c += (uint32_t)__popcll(__ballot(is_pick(in && (v & 0x7FFFFFFFu) >= lo, v & 0x7FFFFFFFu, i)));
              });
              if (h != ~0u) L.rcnt[wave][h] = c;
              w_total += c;
          });
    if (lane == 0) L.wtot[wave] = w_total;
    __syncthreads();
    uint32_t wave_off = above_before + l2_before;
    for (int i = 0; i < wave; i++) wave_off += L.wtot[i];
    auto emit_half = [&](bool valid, uint64_t e, uint32_t pos) {
        const uint32_t key = key64(e), idx = (uint32_t)e, bitsv = (uint32_t)(e >> 32);
        const bool pick = is_pick(valid, key, idx);
        const uint64_t m = __ballot(pick);
        if (pick) {
            const u2a pr = {idx, bitsv};
            *(u2a4*)(out + 1 + 2 * (uint64_t)(pos + (uint32_t)__popcll(m & below))) = pr;
        }
        // the streaming block stored 0.0f for key >= predicted threshold; repair where the prediction was wrong
        if (valid && pick != (key >= that_key)) rp[idx] = pick ? 0.0f : u2f(bitsv);
        return pos + (uint32_t)__popcll(m);
    };
    auto emit_dense = [&](uint32_t t, uint32_t pos) {
        // a dense tile's residual holds plain sums (nothing was stored as zero)
        dense_tile_walk<false>(rp, bn, t, L.dbuf[wave], [&](uint32_t i, uint32_t v, bool in) {
            const bool pick = is_pick(in && (v & 0x7FFFFFFFu) >= lo, v & 0x7FFFFFFFu, i);
            const uint64_t m = __ballot(pick);
            if (pick) {
                const uint32_t p = pos + (uint32_t)__popcll(m & below);
                out[1 + 2 * (uint64_t)p] = i;
                out[2 + 2 * (uint64_t)p] = v;
                rp[i] = 0.0f;
            }
            pos += (uint32_t)__popcll(m);
        });
        return pos;
    };
    {
        uint32_t pos = wave_off;
#pragma unroll
        for (int h = 0; h < kHeld; h++) {
            if (G.wt0 + h < G.wt1) {
                if (G.cnt[h] != kDense) {
                    pos = emit_half((uint32_t)lane < G.cnt[h], G.e0[h], pos);
                    pos = emit_half((uint32_t)(kWave + lane) < G.cnt[h], G.e1[h], pos);
                } else {
                    pos += L.rcnt[wave][h];  // written out by the loop below
                }
            }
        }
    }
    if (G.more) {
        uint32_t pos = wave_off;
#pragma unroll 1
        for (uint32_t t = G.wt0; t < G.wt1; t++) {
            const uint32_t cnt = (uint32_t)__builtin_amdgcn_readfirstlane((int)G.tcnt[t]);
            if (cnt == kDense) {
                pos = emit_dense(t, pos);
            } else if (t - G.wt0 < (uint32_t)kHeld) {
                pos += L.rcnt[wave][t - G.wt0];
            } else {
                const uint64_t a0 = G.slots[(uint64_t)t * kTileSlots + lane];
                const uint64_t a1 = G.slots[(uint64_t)t * kTileSlots + kWave + lane];
                pos = emit_half((uint32_t)lane < cnt, a0, pos);
                pos = emit_half((uint32_t)(kWave + lane) < cnt, a1, pos);
            }
        }
    }
    if (grp == 0 && threadIdx.x == 0) {
        st[S_T] = T;
        st[S_NEED] = need2;
        st[S_ISTAR] = istar;
        st[S_OK] = 1u;
    }
    } while (false);
    // the exact selection for a bucket the window could not finish (S_OK stays 0)
    if (failed) {
        if (!select_exact_group(bk, g, w, b, grp, fg, that_key, G, L, limit_ticks)) {
            fused_give_up(st, out);
            return;
        }
    }
    if (grp == 0 && threadIdx.x == 0 && !ld_agent(st + S_TIMEOUT)) out[0] = k;
}
