// Host-side rules of the Q8_0 kernels: which kernel and tile a product takes,
// how a launch is cut into work units, list capacities and workspace sizes.
// No device code and no HIP types: the dispatch planner (tm_hip.cpp) includes
// this header alone, so that it also builds with a plain C++ compiler for its
// CPU tests; the kernel headers include it for the same definitions, next to
// the kernels the rules describe.
#pragma once

#include <cstddef>
#include <cstdint>

// (xq_bpad / xq_bytes are also called from device code)
#if defined(__HIPCC__)
#define Q8_HD __host__ __device__
#else
#define Q8_HD
#endif

namespace q8 {

// ---- GEMV / small-batch list kernels (q8_gemv.hpp, q8_gemm_small.hpp) --------

// The list travels in the kernel-argument segment (read through the scalar
// cache): 224 * 64 + 40 = 14376 bytes, enough for a whole decode step of a
// 28-layer model (197 products) in one launch.
constexpr int GEMV_MAX_DESCS = 224;


// Most launches of a real step carry one to three products (q/k/v, gate/up, a
// lone projection between two dependent operators), at up to four tokens with
// a descriptor each: they use a short argument block (808 bytes) instead of the
// 14 KB one, which is copied and fetched per launch (q,k,v at 2 tokens: 6
// descriptors, a step of 115 such launches 727 -> 718 us).
constexpr int GEMV_FEW_DESCS = 12;


// ---- prefill GEMM on the f32 matrix cores (q8_gemm_mma.hpp) ------------------

constexpr int MMA_MAX_DESCS = 64;


// How many workgroups share each output tile of a launch, each with its own
// part of K: a launch with few output tiles and a long K otherwise leaves most
// of the chip idle (1024 x 2048 at 32 tokens is 32 tiles of 64 blocks each).
// Doubled while the launch's tiles, times it, stay within 256 workgroups and
// every wave keeps at least 4 blocks of the shortest K. It depends on what
// shares the launch, and with it the order of a product's f32 sums (the same
// launch gives the same bits every time).
constexpr uint32_t MMA_SHARED_MAX_TILES = 128;  // tiles x parts <= 256, parts >= 2
constexpr size_t MMA_SHARED_PARTIAL_FLOATS = 256u * 2u * 16u * 64u; // 256 partial tiles of 64 x 32
inline uint32_t mma_shared_parts(uint64_t tiles, uint32_t min_blocks) {
    uint32_t z = 1;
    while (z < 8u && tiles * (z * 2u) <= 256u && min_blocks / (4u * z * 2u) >= 4u) {
        z *= 2u;
    }
    return z;
}

struct MmaConfig {
    int tmw, tnw, s;
};

struct MmaProduct {
    const uint8_t *w;
    const float *x;
    float *y;
    uint32_t rows, cols, batch;
};

inline uint64_t mma_tiles(const MmaProduct &p, const MmaConfig &c) {
    return (uint64_t)((p.batch + 32u * c.tmw - 1) / (32u * c.tmw)) *
           ((p.rows + 32u * c.tnw - 1) / (32u * c.tnw));
}

// Tile and K split. Measured on MI355X at M = 512 over the Qwen3-0.6B
// projection shapes, alone and as one list launch: a 64-token x 32-row wave
// tile with K split over the 4 waves of a workgroup is best or tied
// everywhere (f32 MFMA is slow enough that filling all 1024 SIMDs with short
// MFMA streams matters more than operand reuse). Narrow batches use a
// 32-token tile; K is split no finer than one Q8_0 block per wave.
inline MmaConfig pick_mma_config(const MmaProduct *prods, int n) {
    uint32_t max_batch = 0, min_blocks = 0xffffffffu;
    for (int i = 0; i < n; ++i) {
        max_batch = prods[i].batch > max_batch ? prods[i].batch : max_batch;
        const uint32_t blocks = prods[i].cols / 32u;
        min_blocks = blocks < min_blocks ? blocks : min_blocks;
    }
    // Tokens per wave tile: 64, or 32 for narrow batches and for launches whose
    // last round of workgroups would be less than half full with 64 (the chip
    // runs 256 of these workgroups at a time; a 32-token tile makes twice the
    // workgroups, each half as long). Up to 128 output tiles of 64 tokens x 32
    // rows: 1024 x 2048 at 128 tokens 24 -> 15 us, 1024 x 1024 14 -> 9, 256 x 4096
    // 43 -> 26, 512 x 2048 at 512 tokens 23 -> 15; 257 to 384 tiles: the 0.6B gate
    // and up projections together at 128 tokens 27 -> 24; at 192 and at 256 tiles
    // the 64-token tile is ahead (1536 x 1024 at 256 tokens 14 against 16 us).
    uint64_t tiles64 = 0;
    for (int i = 0; i < n; ++i) {
        tiles64 += (uint64_t)((prods[i].batch + 63u) / 64u) * ((prods[i].rows + 31u) / 32u);
    }
    const bool short_last_round = tiles64 <= 128u || (tiles64 > 256u && tiles64 <= 384u);
    MmaConfig c;
    c.tmw = max_batch > 32u && !short_last_round ? 2 : 1;
    c.tnw = 1;
    c.s = min_blocks >= 4u ? 4 : (min_blocks >= 2u ? 2 : 1);
    return c;
}


// The same kernel fed with activations in split form (gemm_mma_kernel<..., XP>):
// always the 32-token tile. A wave's share of K is made of whole groups of four
// blocks, so K is split over four waves from 16 blocks on. Two row tiles per wave
// (the activations' pieces are then fetched once for both) from more than 256
// tiles of one, and from about 256 under a K of 96 blocks and more, where the
// halved tile count lets two workgroups share each tile. Measured alone (us, one
// row tile against two): 4096 x 1024 at 128 tokens 11.1 against 9.0, at 64 tokens
// (256 tiles) 7.1 against 8.5, at 256 tokens 19.8 against 14.9; 6144 x 1024 at 64
// tokens (384 tiles) 10.8 against 8.7, at 32 tokens (192 tiles) 6.9 against 8.3;
// 1024 x 3072 at 256 tokens (256 tiles) 17.3 against 14.3, at 128 tokens (two
// workgroups per tile either way) 11.1 against 11.9; 1024 x 2048 at 256 tokens
// 11.4 against 11.7.
inline MmaConfig pick_mma_split_config(const MmaProduct *prods, int n) {
    uint32_t min_blocks = 0xffffffffu;
    uint64_t tiles = 0;
    for (int i = 0; i < n; ++i) {
        const uint32_t blocks = prods[i].cols / 32u;
        min_blocks = blocks < min_blocks ? blocks : min_blocks;
        tiles += (uint64_t)((prods[i].batch + 31u) / 32u) * ((prods[i].rows + 31u) / 32u);
    }
    MmaConfig c;
    c.tmw = 1;
    c.s = min_blocks >= 16u ? 4 : (min_blocks >= 8u ? 2 : 1);
    c.tnw = c.s == 4 && (tiles > 256u || (tiles > 192u && min_blocks >= 96u)) ? 2 : 1;
    return c;
}

// ---- prefill GEMM on the bf16 matrix cores (q8_gemm_bf16x3.hpp) -------------

constexpr int SPLIT_MAX_DESCS = 16;

constexpr int BX3_MAX_DESCS = 64;
constexpr uint32_t BX3_CHUNK_BLOCKS = 16;   // K is cut into chunks of 512 columns or more
constexpr uint32_t BX3_MAX_SPLIT_TILES = 16384; // arrival counters per context


// How a product is cut into work units (output tile x K chunk): a function of
// the product's shape and of the tile its launch uses.
//
// Tile: 256 rows x 128 tokens (2 x 4 waves, two per SIMD), or x 64 tokens (1 x 4
// waves, one per SIMD) for some products that would make fewer than 192 units
// of the large tile (bx3_plan below). Measured alone, the small tile is 1.1-1.6 times as fast on such
// products (4096 x 1024 at 512 tokens: 35 against 40 us, 6144 x 2048 at 128
// tokens: 33 us against 48 on the f32 kernel) and 10-25 % slower on large ones
// (a quarter more operand bytes per product).
//
// K chunks: a product with few output tiles cuts K into at most BX3_MAX_CHUNKS
// chunks of 512 columns or more, as many as it takes to give the chip about
// BX3_UNITS_WANTED work units; one with many tiles does not cut K at all
// (14336 x 4096 at 512 tokens: 295 TFLOP/s whole, less in chunks). Measured
// alone with the large tile: chunks of 512 instead of 1024 columns make
// 6144 x 2048 at 256 tokens 47 us instead of 59 (f32 kernel: 69) and 8192 x 1024
// at 512 tokens 49 instead of 56 (f32: 93); chunks of 256 columns and less made
// the 0.6B projections slower, alone and together.
constexpr uint32_t BX3_TILE_ROWS = 256;
constexpr uint32_t BX3_UNITS_WANTED = 192;
constexpr uint32_t BX3_MAX_CHUNKS = 8;

struct Bx3Plan {
    uint32_t tile_tokens;  // 128 or 64
    uint32_t chunk_blocks; // Q8_0 blocks per K chunk
    uint32_t chunks;
    uint64_t tiles;        // output tiles
    uint64_t units;        // tiles x chunks
    uint64_t split_tiles;  // tiles that need an arrival counter (chunks > 1)
    uint64_t partial_floats; // floats of partial tiles (chunks > 1)
};

inline Bx3Plan bx3_plan_with(uint32_t rows, uint32_t cols, uint32_t batch, uint32_t tile_tokens) {
    Bx3Plan p;
    p.tile_tokens = tile_tokens;
    const uint32_t blocks = cols / 32u;
    p.tiles = (uint64_t)((batch + tile_tokens - 1u) / tile_tokens) *
              ((rows + BX3_TILE_ROWS - 1u) / BX3_TILE_ROWS);
    uint32_t most = (blocks + BX3_CHUNK_BLOCKS - 1u) / BX3_CHUNK_BLOCKS;
    most = most < BX3_MAX_CHUNKS ? most : BX3_MAX_CHUNKS;
    const uint64_t want = (BX3_UNITS_WANTED + p.tiles - 1u) / p.tiles;
    const uint32_t chunks = want < most ? (uint32_t)want : most;
    p.chunk_blocks = (blocks + chunks - 1u) / chunks;
    p.chunks = (blocks + p.chunk_blocks - 1u) / p.chunk_blocks;
    p.units = p.tiles * p.chunks;
    p.split_tiles = p.chunks > 1u ? p.tiles : 0u;
    p.partial_floats = p.split_tiles * p.chunks * tile_tokens * BX3_TILE_ROWS;
    return p;
}

// ---- K chunks: decided per launch ------------------------------------------
//
// What bx3_plan_with says about a product's chunks is what the product would get
// alone; bx3_launch_tile keeps using those unit counts as its measure of "enough
// work". How the products of a launch are actually cut is decided for the launch
// as a whole, because a work unit has a fixed cost that 16-block chunks pay too
// often: measured (1024 units of one product at 512 tokens, K = 512 ... 4096)
// a unit takes about 6 us plus 1.43 us per Q8_0 block, and a unit of a chunked
// tile about 10 us more (its 128 KiB partial tile goes to memory and comes back;
// a whole round of them is 33 MB at once). The seven projections of a Qwen3-0.6B
// layer at 512 tokens, each cut as if alone, were 480 units of 16 blocks, two
// rounds of the chip and 61 MB of partial tiles: 82 us. Cut for the launch they
// are 240 units of 32 blocks, one round, the five K = 1024 products whole: 66 us.
//
// The rule: every product gets chunks_i = ceil(blocks_i / L) (at most
// bx3_chunk_cap) for one target length L per launch; L runs over the lengths at
// which some product's chunk count changes, each candidate is priced by handing
// its units, longest first (the kernel's order), to the chip's workgroup slots
// as they come free, and the cheapest wins (ties: fewer units).
struct Bx3Shape3 {
    uint32_t rows, cols, batch;
};

// At most eight chunks, none below 512 columns, and no more than it takes to
// give a product about two rounds of units on its own: a product with many
// output tiles is never cut.
inline uint32_t bx3_chunk_cap(uint32_t rows, uint32_t cols, uint32_t batch, uint32_t tile_tokens) {
    const uint32_t blocks = cols / 32u;
    const uint64_t tiles = (uint64_t)((batch + tile_tokens - 1u) / tile_tokens) *
                           ((rows + BX3_TILE_ROWS - 1u) / BX3_TILE_ROWS);
    uint32_t cap = blocks / BX3_CHUNK_BLOCKS;
    cap = cap < BX3_MAX_CHUNKS ? cap : BX3_MAX_CHUNKS;
    const uint64_t by_tiles = (2u * 256u + tiles - 1u) / tiles;
    cap = by_tiles < cap ? (uint32_t)by_tiles : cap;
    return cap < 1u ? 1u : cap;
}

// The plan of a product cut into `chunks` chunks (as many as bx3_plan_launch gave it).
inline Bx3Plan bx3_plan_chunked(uint32_t rows, uint32_t cols, uint32_t batch, uint32_t tile_tokens,
                                uint32_t chunks) {
    Bx3Plan p;
    p.tile_tokens = tile_tokens;
    const uint32_t blocks = cols / 32u;
    p.tiles = (uint64_t)((batch + tile_tokens - 1u) / tile_tokens) *
              ((rows + BX3_TILE_ROWS - 1u) / BX3_TILE_ROWS);
    chunks = chunks < 1u ? 1u : chunks;
    p.chunk_blocks = (blocks + chunks - 1u) / chunks;
    p.chunks = (blocks + p.chunk_blocks - 1u) / p.chunk_blocks;
    p.units = p.tiles * p.chunks;
    p.split_tiles = p.chunks > 1u ? p.tiles : 0u;
    p.partial_floats = p.split_tiles * p.chunks * tile_tokens * BX3_TILE_ROWS;
    return p;
}

// A product's last rows may be cut off as a segment of their own with K in
// (more) chunks: the tail of a launch whose units do not fill its last round
// (bx3_plan_launch). row_tiles == 0: none.
struct Bx3Tail {
    uint32_t product = 0;   // index in the launch's list
    uint32_t row_tiles = 0; // row tiles (of BX3_TILE_ROWS rows) in the tail segment
    uint32_t chunks = 0;    // its K chunks
};
constexpr uint32_t BX3_TAIL_CHUNK_BLOCKS = 8; // a tail's chunks: 256 columns or more,
constexpr uint32_t BX3_TAIL_MAX_CHUNKS = 3;   // at most three

// Rows of a product's head segment (what the tail leaves), and of the tail.
inline uint32_t bx3_head_rows(uint32_t rows, uint32_t tail_row_tiles) {
    const uint32_t row_tiles = (rows + BX3_TILE_ROWS - 1u) / BX3_TILE_ROWS;
    return tail_row_tiles == 0u ? rows : (row_tiles - tail_row_tiles) * BX3_TILE_ROWS;
}

// Estimated duration (ns) of a launch whose products are cut as `chunks` says
// (and `tail`, if any): units in descending length to `slots` workgroup slots,
// each to the slot that comes free first. Units of one segment are alike, so
// the slots are tracked as groups that come free together.
inline uint64_t bx3_price(const Bx3Shape3 *shapes, const uint32_t *chunks, int n,
                          uint32_t tile_tokens, const Bx3Tail *tail = nullptr) {
    const uint32_t slots = tile_tokens == 128u ? 256u : 512u;
    const uint64_t unit_ns = tile_tokens == 128u ? 6000u : 4500u;
    const uint64_t block_ns = tile_tokens == 128u ? 1430u : 1100u;
    const uint64_t chunked_ns = tile_tokens == 128u ? 10000u : 5000u;
    struct Kind {
        uint64_t ns, units;
    };
    Kind kinds[BX3_MAX_DESCS + 1];
    int nk = 0;
    auto add = [&](uint32_t rows, uint32_t cols, uint32_t batch, uint32_t c) { // insertion sort, longest first
        const Bx3Plan p = bx3_plan_chunked(rows, cols, batch, tile_tokens, c);
        const Kind k{unit_ns + block_ns * p.chunk_blocks + (p.chunks > 1u ? chunked_ns + 1000u * p.chunks : 0u),
                     p.units};
        int at = nk++;
        while (at > 0 && kinds[at - 1].ns < k.ns) {
            kinds[at] = kinds[at - 1];
            --at;
        }
        kinds[at] = k;
    };
    for (int i = 0; i < n; ++i) {
        if (tail != nullptr && tail->row_tiles != 0u && tail->product == (uint32_t)i) {
            const uint32_t head = bx3_head_rows(shapes[i].rows, tail->row_tiles);
            add(head, shapes[i].cols, shapes[i].batch, chunks[i]);
            add(shapes[i].rows - head, shapes[i].cols, shapes[i].batch, tail->chunks);
        } else {
            add(shapes[i].rows, shapes[i].cols, shapes[i].batch, chunks[i]);
        }
    }
    struct Group {
        uint64_t free_at, count;
    };
    constexpr int MAX_GROUPS = 4 * BX3_MAX_DESCS + 8;
    Group groups[MAX_GROUPS]; // ascending free_at
    int ng = 1;
    groups[0] = Group{0u, slots};
    uint64_t end = 0;
    for (int i = 0; i < nk; ++i) {
        uint64_t left = kinds[i].units;
        while (left > 0) {
            // whole rounds of every slot at once when the class is large
            if (ng == 1 && left >= groups[0].count) {
                const uint64_t rounds = left / groups[0].count;
                groups[0].free_at += rounds * kinds[i].ns;
                left -= rounds * groups[0].count;
                end = groups[0].free_at > end ? groups[0].free_at : end;
                continue;
            }
            const uint64_t take = left < groups[0].count ? left : groups[0].count;
            const uint64_t done = groups[0].free_at + kinds[i].ns;
            end = done > end ? done : end;
            groups[0].count -= take;
            left -= take;
            if (groups[0].count == 0) { // drop it
                for (int g = 1; g < ng; ++g) {
                    groups[g - 1] = groups[g];
                }
                --ng;
            }
            // insert (done, take), merging with a group of the same time
            int at = 0;
            while (at < ng && groups[at].free_at < done) {
                ++at;
            }
            if (at < ng && groups[at].free_at == done) {
                groups[at].count += take;
            } else if (ng < MAX_GROUPS) {
                for (int g = ng; g > at; --g) {
                    groups[g] = groups[g - 1];
                }
                groups[at] = Group{done, take};
                ++ng;
            } else { // (cannot happen with these bounds; stay correct anyway)
                groups[ng - 1].count += take;
            }
        }
    }
    return end;
}

// chunks[i] for every product of a launch (see above). Deterministic: a function
// of the shapes in list order and the tile.
inline void bx3_plan_chunks(const Bx3Shape3 *shapes, int n, uint32_t tile_tokens, uint32_t *chunks) {
    uint32_t cap[BX3_MAX_DESCS];
    uint64_t tiles = 0;
    bool any = false;
    for (int i = 0; i < n; ++i) {
        cap[i] = bx3_chunk_cap(shapes[i].rows, shapes[i].cols, shapes[i].batch, tile_tokens);
        any = any || cap[i] > 1u;
        chunks[i] = 1u;
        tiles += bx3_plan_chunked(shapes[i].rows, shapes[i].cols, shapes[i].batch, tile_tokens, 1u).tiles;
    }
    if (!any || tiles >= 1024u) {
        return; // nothing to cut, or rounds enough as it is
    }
    // candidate lengths: where some product's chunk count changes
    uint32_t lengths[BX3_MAX_DESCS * BX3_MAX_CHUNKS];
    int nl = 0;
    for (int i = 0; i < n; ++i) {
        const uint32_t blocks = shapes[i].cols / 32u;
        for (uint32_t c = 1; c <= cap[i]; ++c) {
            const uint32_t len = (blocks + c - 1u) / c;
            bool seen = false;
            for (int j = 0; j < nl; ++j) {
                seen = seen || lengths[j] == len;
            }
            if (!seen) {
                lengths[nl++] = len;
            }
        }
    }
    uint64_t best_ns = ~0ull, best_units = ~0ull;
    uint32_t trial[BX3_MAX_DESCS];
    for (int j = 0; j < nl; ++j) {
        uint64_t units = 0;
        for (int i = 0; i < n; ++i) {
            const uint32_t blocks = shapes[i].cols / 32u;
            uint32_t c = (blocks + lengths[j] - 1u) / lengths[j];
            c = c > cap[i] ? cap[i] : c;
            trial[i] = c;
            units += bx3_plan_chunked(shapes[i].rows, shapes[i].cols, shapes[i].batch, tile_tokens, c).units;
        }
        const uint64_t ns = bx3_price(shapes, trial, n, tile_tokens);
        if (ns < best_ns || (ns == best_ns && units < best_units)) {
            best_ns = ns;
            best_units = units;
            for (int i = 0; i < n; ++i) {
                chunks[i] = trial[i];
            }
        }
    }
}

// The whole cut of a launch: chunks[i] for every product, and (when `tail` is
// given) at most one tail segment. A launch of more units than the chip has
// workgroup slots ends with a round that is partly empty: 594 whole-K units on
// 512 slots are two rounds, the second 16 % full. The units of that last round
// are then taken off the end of one whole-K product, as a segment of rows of its
// own whose K is cut into chunks: several short units in the place of each long
// one. Candidates: every whole-K product, 2 or 3 chunks of 256 columns or more;
// priced like everything else; taken when the estimate drops by 8 % or more (a
// launch with a segment in it runs on an instantiation of the kernel that is
// 3-4 % slower, gemm_bf16x3_kernel<..., SEG = true>).
// Measured on that instantiation (split pass included): 76800 x 1024 at 128
// tokens, 300 units on 256 slots, 99.4 us whole, 89.3 / 86.9 / 90.5 with the last
// 44 row tiles in 2 / 3 / 4 chunks; 151936 x 1024 at 128 tokens (594 units) 152.8
// whole, 147.0 / 150.2 / 176.4 (too little to pay for the instantiation: not taken). More chunks lose what they gain to their partial tiles, which cost more
// the more of them are on their way at once; on the 64-token tile (512 slots, half
// the arithmetic per partial byte) they cost too much for the estimate to be
// trusted (151936 x 1024 at 64 tokens: 88.1 whole, 83.8 / 85.1 / 94.8): no tails
// there. The tail's rows add in another order than the head's (another chunk
// count), like any product whose K is cut.
inline void bx3_plan_launch(const Bx3Shape3 *shapes, int n, uint32_t tile_tokens, uint32_t *chunks,
                            Bx3Tail *tail = nullptr) {
    bx3_plan_chunks(shapes, n, tile_tokens, chunks);
    if (tail == nullptr) {
        return;
    }
    *tail = Bx3Tail{};
    const uint32_t slots = tile_tokens == 128u ? 256u : 512u;
    uint64_t units = 0;
    for (int i = 0; i < n; ++i) {
        units += bx3_plan_chunked(shapes[i].rows, shapes[i].cols, shapes[i].batch, tile_tokens, chunks[i]).units;
    }
    const uint64_t ragged = units % slots;
    if (tile_tokens != 128u || units <= slots || ragged == 0u || n >= BX3_MAX_DESCS) {
        return;
    }
    const uint64_t base_ns = bx3_price(shapes, chunks, n, tile_tokens);
    uint64_t best_ns = base_ns;
    Bx3Tail best;
    for (int i = 0; i < n; ++i) {
        if (chunks[i] != 1u) {
            continue;
        }
        const uint32_t blocks = shapes[i].cols / 32u;
        uint32_t most = blocks / BX3_TAIL_CHUNK_BLOCKS;
        most = most < BX3_TAIL_MAX_CHUNKS ? most : BX3_TAIL_MAX_CHUNKS;
        const uint32_t tiles_t = (shapes[i].batch + tile_tokens - 1u) / tile_tokens;
        const uint32_t row_tiles = (shapes[i].rows + BX3_TILE_ROWS - 1u) / BX3_TILE_ROWS;
        const uint64_t t = (ragged + tiles_t - 1u) / tiles_t;
        if (most < 2u || t >= row_tiles) {
            continue; // (the head keeps at least one row tile)
        }
        // (one chunk more only for 5 % more: the estimate knows nothing of what
        // many partial tiles at once cost each other)
        Bx3Tail mine;
        uint64_t mine_ns = ~0ull;
        for (uint32_t c = 2; c <= most; ++c) {
            const Bx3Tail trial{(uint32_t)i, (uint32_t)t, c};
            const uint64_t ns = bx3_price(shapes, chunks, n, tile_tokens, &trial);
            if (mine_ns == ~0ull || ns * 100u < mine_ns * 95u) {
                mine_ns = ns;
                mine = trial;
            }
        }
        if (mine_ns < best_ns) {
            best_ns = mine_ns;
            best = mine;
        }
    }
    if (best.row_tiles != 0u && best_ns * 100u <= base_ns * 92u) {
        *tail = best;
    }
}

// Which tile the products of one launch take together, or 0 when the kernel does
// not pay for them: the rule of a single product, with the launch's sums in the
// place of the product's own figures (`shapes` = rows, cols, batch of every
// product; all with batch <= 32, all with 33..64, or all above).
//
// Up to 64 tokens there is one small tile of tokens. The kernel's time hardly
// depends on the batch here (27 us for 8192 x 1024, 97 us for 151936 x 1024), the
// f32 kernel's does: from 33 tokens (its 64-token tile) 16 M weights are the
// break-even (16384 x 1024 at 64 tokens: 30 against 29 us; 4096 x 4096: 34 against
// 47; 151936 x 1024: 97 against 219). At 32 tokens and below only the largest
// matrices would gain, and little: from 17 tokens (below, the exact small-batch
// kernel serves the entry point) the bar is 32 M weights.
//
// Above 64 tokens, in order of preference: the large tile with 192 units or more;
// the small tile with 192 units or more, in however many K chunks (alone, split
// pass included: 1024 x 4096 at 512 tokens in six chunks 37 us, against 47 on the
// large tile and 46 on the f32 kernel; 896 x 4864 39 against 51; 2048 x 4096 at 256
// tokens 35 against 45; 1024 x 3072 at 512 tokens 33 against 31 on the f32 kernel,
// 28 when the gated activation in front of it has written its split form; the
// seven Qwen3-0.6B projections at 128 tokens 34 us against 54 on the f32
// kernels); the large tile with 128 units or more (a product alone is then
// about even with the f32 kernel, products that share a launch far ahead);
// the small tile again for products of 3072 columns and more with at least 32
// units (alone, at 128 tokens: 1024 x 3072 29 us against 34 on the f32 kernel,
// 1024 x 4096 32 against 44, 1152 x 6912 38 against 71, 1536 x 8960 45 against 90;
// at 256 tokens 1024 x 4096 34 against 39; 2048 columns lose, 27 against 24). Measured alone at 512 tokens
// against the f32 kernel: small tile 3072 x 1024 34 against 35 us, 2048 x 2048 39
// against 49, 4096 x 1024 36 against 48, 2048 x 1024 (128 units) 31 against 28;
// large tile 8192 x 1024 49 against 93, 6144 x 2048 69 against 133. Together: the
// seven Qwen3-0.6B projections at 512 tokens 78 us on the large tile against 144
// on the f32 kernel.
inline uint32_t bx3_launch_tile(const Bx3Shape3 *shapes, int n) {
    if (n <= 0) {
        return 0;
    }
    uint64_t large = 0, small = 0, weights = 0;
    uint32_t least_cols = shapes[0].cols;
    for (int i = 0; i < n; ++i) {
        least_cols = shapes[i].cols < least_cols ? shapes[i].cols : least_cols;
        small += bx3_plan_with(shapes[i].rows, shapes[i].cols, shapes[i].batch, 64u).units;
        large += bx3_plan_with(shapes[i].rows, shapes[i].cols, shapes[i].batch, 128u).units;
        weights += (uint64_t)shapes[i].rows * shapes[i].cols;
    }
    if (shapes[0].batch <= 32u) {
        // half of the one token tile is padding: only twice the weights pay (the
        // f32 kernel's own tile is 32 tokens here; 20 x (6144 x 2048 + 2048 x 6144) at
        // 32 tokens: 385 us on the f32 kernels, about 300 us here)
        return weights >= (1ull << 25) && small >= 128u ? 64u : 0u;
    }
    if (shapes[0].batch <= 64u) {
        return weights >= (1ull << 24) && small >= 128u ? 64u : 0u;
    }
    if (large >= BX3_UNITS_WANTED) {
        return 128u;
    }
    if (small >= BX3_UNITS_WANTED) {
        return 64u;
    }
    if (large >= 128u) {
        return 128u;
    }
    // Few output tiles under a deep K: this kernel cuts K into chunks and takes
    // 22.5 + 2.3 us per 1024 columns, its split pass included. A wave of the f32
    // kernel takes 0.72 us per block of a 32-token tile (twice that for 64
    // tokens) after 4.5 us, over K divided by its 4 waves and by the workgroups
    // that share a tile (q8::mma_shared_parts), once per round of 256
    // workgroups: 1024 x 3072 at 128 tokens 14.8 us against 29.1 here, 1024 x 4096
    // at 192 tokens 26.4 against 33.1, but 1152 x 6912 at 128 tokens 42.0 against
    // 37.9 and 2048 x 8192 at 96 tokens 49.0 against 41.3. The cheaper estimate wins.
    if (least_cols < 3072u || small < 32u) {
        return 0u;
    }
    MmaProduct prods[MMA_MAX_DESCS];
    const int m = n < MMA_MAX_DESCS ? n : MMA_MAX_DESCS;
    uint32_t min_blocks = 0xffffffffu, max_blocks = 0;
    for (int i = 0; i < m; ++i) {
        prods[i] = MmaProduct{nullptr, nullptr, nullptr, shapes[i].rows, shapes[i].cols, shapes[i].batch};
        const uint32_t blocks = shapes[i].cols / 32u;
        min_blocks = blocks < min_blocks ? blocks : min_blocks;
        max_blocks = blocks > max_blocks ? blocks : max_blocks;
    }
    const MmaConfig c = pick_mma_config(prods, m);
    uint64_t tiles = 0;
    for (int i = 0; i < m; ++i) {
        tiles += mma_tiles(prods[i], c);
    }
    const uint32_t z = c.s == 4 ? mma_shared_parts(tiles, min_blocks) : 1u;
    const uint64_t rounds = (tiles * z + 255u) / 256u;
    const uint64_t per_wave = (max_blocks + 4u * z - 1u) / (4u * z);
    const uint64_t f32_us_x100 = 450u + 72u * (uint64_t)c.tmw * per_wave * rounds;
    const uint64_t here_us_x100 = 2250u + 230u * (uint64_t)(max_blocks * 32u) / 1024u;
    return here_us_x100 < f32_us_x100 ? 64u : 0u;
}

// Up to 32 tokens half of the staged kernel's 64-token tile is padding, and its time
// hardly depends on the batch. The launches it takes there (32 M weights and more)
// run on the 32-token tiles of the f32 kernel fed from the split form instead
// (gemm_mma_kernel<..., XP>), behind the same split pass. Measured, split pass
// included, staged against small tiles: 151936 x 1024 at 17 / 32 tokens 80 us against
// 53 / 57; 33000 x 1024 35 against 20 / 21; 262144 x 1152 at 32 tokens 136 against
// 127; forty 2B-class matrices (6144 x 2048, 2048 x 6144) in one launch at 32 tokens
// 277 against 231. From 33 tokens the small tiles need two token tiles and lose
// (the forty matrices at 64 tokens 284 against 382).
inline bool bx3_small_batch_tiles(uint32_t batch) { return batch <= 32u; }

// Below 17 tokens the MFMA entry point over sealed weights of 1024 columns and more
// normally runs the vector kernels (GEMV arithmetic). A large product does better on
// the 32-token tiles above, whose time hardly depends on the batch, from 9 tokens
// (32 M weights and more) or from 5 (128 M and more: the vocabulary projections).
// Measured against the vector kernel, split pass included: 151936 x 1024 at 5 / 8 /
// 12 / 16 tokens 72 / 70 / 125 / 129 us against 62; 262144 x 1152 at 8 / 16 tokens
// 222 / 386 against about 120; 33000 x 1024 at 5 / 8 tokens 25 / 24 against 27 (not
// taken), at 12 / 16 tokens 36 against 27.
inline bool mma_small_batch_on_tiles(uint32_t rows, uint32_t cols, uint32_t batch) {
    if (batch < 5u || batch > 16u) {
        return false;
    }
    const Bx3Shape3 one{rows, cols, batch};
    return (uint64_t)rows * cols >= (batch <= 8u ? (1ull << 27) : (1ull << 25)) &&
           bx3_launch_tile(&one, 1) != 0u;
}

// A product on its own: its plan, and whether the kernel pays for it (`worth`).
inline Bx3Plan bx3_plan(uint32_t rows, uint32_t cols, uint32_t batch, bool *worth) {
    const Bx3Shape3 one{rows, cols, batch};
    const uint32_t tile = bx3_launch_tile(&one, 1);
    *worth = tile != 0u;
    return bx3_plan_with(rows, cols, batch, tile != 0u ? tile : (batch <= 64u ? 64u : 128u));
}
inline Bx3Plan bx3_plan(uint32_t rows, uint32_t cols, uint32_t batch) {
    bool worth;
    return bx3_plan(rows, cols, batch, &worth);
}


// ---- int8-activation profile (q8_gemm_i8.hpp, q8_gemv_i8.hpp, q8_gemm_i8_lds.hpp)

// Layout of a quantized-activation buffer for `batch` rows of `cols`:
//   [batch][cols] int8 quants, then [cols/32][bpad] f32 scales with
//   bpad = batch rounded up to 4 (block-major, so that the four tokens a lane
//   rescales per MFMA are one aligned 16-byte load).
Q8_HD inline uint32_t xq_bpad(uint32_t batch) { return (batch + 3u) & ~3u; }
Q8_HD inline size_t xq_bytes(uint32_t cols, uint32_t batch) {
    return (size_t)batch * cols + (size_t)(cols / 32u) * xq_bpad(batch) * 4u;
}


constexpr int I8_MAX_DESCS = 64;


// 0: 16 tokens x 64 rows (batch <= 16), 1: 32 x 32 (batch <= 32), 2: 64 x 32,
// 3: 64 x 64 (large batches: operands are re-read from L2 per wave, so the
// larger tile halves that traffic per MFMA).
inline int pick_i8_config(uint32_t batch) {
    return batch <= 16u ? 0 : (batch <= 32u ? 1 : (batch < 128u ? 2 : 3));
}


constexpr uint32_t GEMV_I8_MAX_BATCH = 16; // above this the MFMA kernels only

inline int gemv_i8_tokens(uint32_t batch) {
    return batch == 1u ? 1 : (batch == 2u ? 2 : (batch <= 4u ? 4 : 8));
}


constexpr uint32_t GEMM_I8_LDS_MIN_BATCH = 5; // below: the streaming kernel (q8_gemv_i8.hpp)

// Workgroup shape for a batch. The bits do not depend on the shape.
//   0..3  batches up to 256: four waves side by side, each 16 rows for 1..4 token
//         tiles of 16; larger batches take several such tiles of equal height
//         (96 tokens: two of 48). While a weight byte is used a few times only,
//         what counts is the weight stream: whole 128-byte lines per fetched row
//         piece (stages of 4 blocks; 8 for one token tile, where LDS leaves
//         room), and many small workgroups per CU so that many stages are in
//         flight. Measured on 535 MB of 2B-class matrices: M = 128 364 us against
//         521 us for shape 4, M = 256 671 against 705, M = 512 1273 against 1165.
//   4     above 256: 2x2 waves over 128 tokens x 128 rows, stages of 2 blocks
//         (bound by the epilogue's f32 operations, not by the fetch).
inline int i8_lds_shape(uint32_t batch) {
    if (batch > 256u) {
        return 4;
    }
    const uint32_t tiles = (batch + 63u) / 64u;
    const uint32_t per_tile = (batch + tiles - 1u) / tiles;
    return (int)((per_tile + 15u) / 16u) - 1;
}


// ---- F16 weight twins (f16_gemv.hpp) ----------------------------------------

constexpr uint32_t F16_GEMM_MAX_BATCH = 32; // native/metal/tm_metal.m:1279-1283 (max_batch 32)

inline int f16_tokens(uint32_t batch) { return batch == 1u ? 1 : (batch == 2u ? 2 : (batch <= 4u ? 4 : 8)); }


// ---- the operators either side of a product, measurement kernels -------------

// rows per workgroup of rmsnorm_kernel (q8_neighbors.hpp), one wave each
constexpr uint32_t RMSNORM_ROWS = 1;
constexpr uint32_t ARGMAX_GROUPS = 64;   // partial results: 64 f32 values, then 64 u32 indices
constexpr uint32_t ARGMAX_PARTIAL_BYTES = ARGMAX_GROUPS * 8u;
// workgroups of xor_checksum_kernel = partial words it leaves (q8_misc.hpp)
constexpr uint32_t CHECKSUM_GROUPS = 2048;

} // namespace q8
