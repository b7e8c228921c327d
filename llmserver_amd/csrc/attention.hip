// Causal attention over the paged cache for a flat batch: portions of prompts and single decoded
// tokens go through the same kernel.  Compiled once per (element type, head size): -DLSA_ND=<head
// size / 16> and -DLSA_BF16=0|1.
//
// Work is a list of items made on the host.  An item is one wavefront's job: a tile of 16
// (token, head-of-the-group) pairs of one request against the keys [k_begin, k_end) of one KV
// head.  The wavefront walks the keys in steps, keeps a running maximum and sum per pair (online
// softmax, 32-bit) and accumulates the output in MFMA registers.  If the item covers every key
// its pairs can see, it writes the output; otherwise it writes its maximum, sum and unnormalised
// output to a partial slot and `merge` combines the slots by log-sum-exp; where a plan gives every
// tile four (or two) key ranges, the wavefronts of a workgroup are those ranges and combine them
// through LDS themselves, without slots and without the second launch.
//
// MFMA use (64-lane wavefront, lane = 16 * quad + col):
//   scores:  S^T[key][pair] = K[key][:] . Q[pair][:]      A = K rows (lane: key col, 8 or 4 dims of quad)
//                                                          B = Q^T    (lane: pair col, same dims)
//            result lane holds keys 4*quad..4*quad+3 of pair col, so the softmax of a pair is a
//            reduction inside a lane plus two shuffles, and
//   output:  O^T[dim][pair] += V^T[dim][key] . P^T[key][pair]   A = V^T rows (lane: dim col, keys of quad)
//                                                                B = P^T, exactly the registers S^T left.
// Keys are stored [page][kv_head][slot][dim], values transposed [page][kv_head][dim][slot], so
// both A operands are contiguous vector loads straight from the pages.
#include "common.hpp"

#ifndef LSA_ND
#error "compile with -DLSA_ND=<head_dim / 16>"
#endif
#ifndef LSA_BF16
#error "compile with -DLSA_BF16=0 or 1"
#endif

using namespace lsa;

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));

constexpr int ND = LSA_ND;          // 16-wide chunks of the head
constexpr int D = ND * 16;          // head size
constexpr float NEG_INF = -__builtin_huge_valf();

// Two wavefronts per SIMD while the double-buffered operands of a step fit into 256 registers.
#define LSA_MIN_WAVES (LSA_ND <= 8 ? 2 : 1)

struct Item { int row, q0, k_begin, k_end; };

struct Geometry {
    int n_q, n_kv, group, gheads, tokens_per_tile, gtiles, page_size, window;
    unsigned page_magic;      // ceil(2^32 / page_size): key / page_size == mulhi(key, page_magic) for key < 2^32 / page_size
    float scale;
};

// Decode steps (every row brings one token) can leave the per-head norm and the rotation of q and
// of the new key, and the new key's and value's way into the cache, to this kernel: a wavefront
// then reads its queries raw from the projection, and the one whose key range ends at the new
// token takes that token's key and value from the projection too (normalised, rotated, written to
// the cache on the side) instead of from the pages.  One launch less between the projection and
// the attention.  bfloat16 and head sizes in steps of 64 only.
struct DecodeFusion {
    const float* q_weight;     // [D] or null: no norm
    const float* k_weight;
    const float* cos_sin;      // [tokens, D] (cos of the D/2 pairs, then sin) or null: no rotation
    float eps;
    int mode;                  // 0: off; 1: q from the raw projection; 3: and the new key and value
};

#if LSA_BF16
typedef bf16_t elem_t;
constexpr int KEY_STEP = 32;                 // keys per loop step (one 16x16x32 MFMA in the output product)
constexpr int NS = (D + 31) / 32;            // 32-dim steps of the score product
#else
typedef float elem_t;
constexpr int KEY_STEP = 16;
constexpr int NS = D / 16;                   // 16-dim steps (four 16x16x4 MFMAs each)
#endif

// MODE is DecodeFusion::mode, known when the kernel is compiled: what a mode does not need is not in its code, and
// no branch stands between the loads of the item's start (a load inside a branch makes every later wait a wait
// for everything).
// PLAIN: the step has both norm weights and a rotation (then nothing of the fused start depends on a flag).
// WG_RANGES (0, 2 or 4): the four items of a workgroup are the four key ranges of one tile, or the two ranges of each
// of two tiles (the plan says so), and the workgroup merges them itself through LDS and writes the output: no partial
// results in memory, no merge launch.  For steps whose contexts are short, where that launch costs as much as the
// attention, and for steps of many rows, whose tiles get no more ranges than that anyway.
template <int MODE, bool PLAIN, int WG_RANGES>
__global__ __launch_bounds__(256, LSA_MIN_WAVES) void paged_attention_kernel(
    const elem_t* __restrict__ q, long q_token_stride, elem_t* __restrict__ out,
    const elem_t* keys, const elem_t* values,
    const int* __restrict__ table, int table_stride,
    const int* __restrict__ row_start, const int* __restrict__ row_len, const int* __restrict__ row_ctx,
    const Item* __restrict__ items, const int* __restrict__ item_slot, int n_items,
    float* __restrict__ part_acc, float* __restrict__ part_ml, Geometry g, DecodeFusion fusion) {
    const int lane = threadIdx.x & 63;
    // The wavefront's number, told to the compiler to be the same in all lanes: the item, its row and the key loop's bounds
    // then live in scalar registers and the loop's branches are scalar ones (a hundred branches on the execution mask
    // otherwise; batch 8 at context 4,096: 4.56 -> 4.53 ms a step).
    const int item_index = blockIdx.x * 4 + __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    constexpr bool WG_MERGE = WG_RANGES > 0;
    if (!WG_MERGE && item_index >= n_items) return;      // with WG_MERGE every wavefront has to reach the barrier at the end
    // The start of an item is a chain of loads, each of which needs the one before it (the item, its row, the row's
    // queries and table entries, the first keys).  Every link costs a trip to memory, so everything that can be
    // asked for is asked for as soon as its address is known, in the order in which it will be needed, and nothing
    // is used before all of it is under way: three trips (item; row, table entries and norm weights; queries,
    // rotation and first keys and values) instead of one per array.
    Item item = items[min(item_index, n_items - 1)];
    if (WG_MERGE && item_index >= n_items) item.k_begin = item.k_end;      // (the launcher refuses such a launch) no keys, no weight
    const int slot = item_slot[min(item_index, n_items - 1)];  // needed at the very end only
    const int kv_head = blockIdx.y / g.gtiles, gtile = blockIdx.y % g.gtiles;
    const int col = lane & 15, quad = lane >> 4;
    const int row = item.row;
    const int* row_table = table + (size_t)row * table_stride;
    const int ps = g.page_size;
    const size_t kv_head_keys = (size_t)kv_head * ps * D;      // offset of the head inside a key page
    const size_t kv_head_values = (size_t)kv_head * D * ps;
    const size_t page_elems = (size_t)g.n_kv * ps * D;

    // Page ids come from the block table 64 logical blocks at a time: lane l of `pages_cur` holds
    // the page of block 64 * chunk + l, and a lane fetches the entry it needs with a shuffle.  The
    // next 64 are requested when a chunk is entered, long before they are needed, so that no load
    // of keys or values ever waits for a table entry.
    int chunk = -1, pages_cur = 0, pages_next = 0;
    auto table_chunk = [&](int c) { return row_table[min(64 * c + lane, table_stride - 1)]; };
    auto enter_chunk = [&](int kt) {            // kt is uniform over the wavefront
        const int c = (int)__umulhi((unsigned)kt, g.page_magic) >> 6;
        if (c != chunk) {
            pages_cur = (chunk >= 0 && c == chunk + 1) ? pages_next : table_chunk(c);
            chunk = c;
            pages_next = table_chunk(c + 1);
        }
    };
    const int kt_first = (item.k_begin / KEY_STEP) * KEY_STEP;
    chunk = (int)__umulhi((unsigned)kt_first, g.page_magic) >> 6;      // the table entries of the first keys need the item only
    pages_cur = table_chunk(chunk);
    pages_next = table_chunk(chunk + 1);
#if LSA_BF16
    // Norm weights and rotation of a head in the operand layout (this lane: dims 32 s + 8 quad .. + 8 of every s).
    constexpr bool FUSABLE = NS % 2 == 0;                      // head sizes in steps of 64 only (the host checks)
    constexpr int NR = NS / 2 > 0 ? NS / 2 : 1;
    struct HeadWeights { f32x4 w[NS][2]; };
    struct Rotation { f32x4 c[NR][2], s[NR][2]; };
    auto load_weights = [&](HeadWeights& hw, const float* weight) {
#pragma unroll
        for (int s = 0; s < NS; ++s) {
            hw.w[s][0] = *reinterpret_cast<const f32x4*>(weight + 32 * s + 8 * quad);
            hw.w[s][1] = *reinterpret_cast<const f32x4*>(weight + 32 * s + 8 * quad + 4);
        }
    };
    constexpr bool FUSED_Q = FUSABLE && (MODE & 1), NEW_TOKEN = FUSABLE && (MODE & 2);
    // Where a step has no norm weights or no rotation, the loads read the start of the projection instead (any
    // readable 4 D bytes will do: a row of it has at least 6 D) and what they bring is not used.
    const float* readable = reinterpret_cast<const float*>(q);
    const bool normed = PLAIN || fusion.q_weight != nullptr, rotated = PLAIN || fusion.cos_sin != nullptr;
    HeadWeights q_weights;
    if constexpr (FUSED_Q) load_weights(q_weights, normed ? fusion.q_weight : readable);
#else
    constexpr bool NEW_TOKEN = false;
#endif
    const int n = row_len[row], ctx = row_ctx[row], first_pos = ctx - n, token0 = row_start[row] + item.q0;
    __builtin_amdgcn_sched_barrier(0);          // all of the above is asked for before any of it is waited for
    // The pair this lane's column stands for.
    const int pair_token = col / g.gheads, pair_head_in_group = gtile * g.gheads + col % g.gheads;
    const bool pair_valid = pair_token < g.tokens_per_tile && item.q0 + pair_token < n && pair_head_in_group < g.group;
    const int q_pos = pair_valid ? first_pos + item.q0 + pair_token : -1;
    const int head = kv_head * g.group + pair_head_in_group;
    // Decode steps: the item that ends at the row's new token takes that token's key and value from the projection,
    // and walks the pages up to the key before it.
    const bool takes_new_token = NEW_TOKEN && item.k_begin < item.k_end && item.k_end == ctx;
    const int k_begin = item.k_begin, k_end = takes_new_token ? item.k_end - 1 : item.k_end;
    // Q^T operand, kept in registers for the whole item.  Lanes without a pair read the first pair's (their
    // operand is zeroed below): no branch stands between the loads.
    const elem_t* q_lane = q + (size_t)(token0 + (pair_valid ? pair_token : 0)) * q_token_stride
                             + (size_t)(pair_valid ? head : kv_head * g.group) * D;
#if LSA_BF16
    bf16x8 qf[NS];
#pragma unroll
    for (int s = 0; s < NS; ++s) {
        const int dim = 32 * s + 8 * quad;
        if (32 * s + 32 <= D) {
            qf[s] = *reinterpret_cast<const bf16x8*>(q_lane + dim);
        } else {                                               // head size not a multiple of 32: the last step is half empty
            bf16x8 x = {0, 0, 0, 0, 0, 0, 0, 0};
            if (dim < D) x = *reinterpret_cast<const bf16x8*>(q_lane + dim);
            qf[s] = x;
        }
    }
    const float* token_cos_sin = rotated ? fusion.cos_sin + (size_t)token0 * D : readable;
    Rotation rotation;
    if constexpr (FUSED_Q || NEW_TOKEN) {
#pragma unroll
        for (int s = 0; s < NS / 2; ++s) {
            const float* c = token_cos_sin + 32 * s + 8 * quad;
            rotation.c[s][0] = *reinterpret_cast<const f32x4*>(c);
            rotation.c[s][1] = *reinterpret_cast<const f32x4*>(c + 4);
            rotation.s[s][0] = *reinterpret_cast<const f32x4*>(c + D / 2);
            rotation.s[s][1] = *reinterpret_cast<const f32x4*>(c + D / 2 + 4);
        }
    }
    const elem_t* token_qkv = q + (size_t)token0 * q_token_stride;
    bf16x8 kh[NS];
    bf16x4 vnew[ND];
    if constexpr (NEW_TOKEN) {                  // every item asks for them (they are there for every row): no branch
#pragma unroll
        for (int s = 0; s < NS; ++s) kh[s] = *reinterpret_cast<const bf16x8*>(token_qkv + (size_t)(g.n_q + kv_head) * D + 32 * s + 8 * quad);
        const elem_t* vh = token_qkv + (size_t)(g.n_q + g.n_kv + kv_head) * D + 4 * quad;
#pragma unroll
        for (int c = 0; c < ND; ++c) vnew[c] = *reinterpret_cast<const bf16x4*>(vh + 16 * c);
    }
#else
    f32x4 qf[NS];
#pragma unroll
    for (int s = 0; s < NS; ++s) qf[s] = *reinterpret_cast<const f32x4*>(q_lane + 16 * s + 4 * quad);
#endif

    // One step of KEY_STEP keys: the K rows and V^T pieces this lane feeds to the MFMAs.  Steps are
    // loaded one ahead of the step being computed, so the loads of the next step are in flight
    // while the softmax and the products of this one run.
    struct Step {
#if LSA_BF16
        bf16x8 k[2][NS];
        bf16x4 v[ND][2];
#else
        f32x4 k[NS];
        f32x4 v[ND];
#endif
    };

    // Element offset of key `key` inside the pool: page * page_elems (+ what the caller adds).
    auto locate_key = [&](int key, int& slot) {
        const int block = (int)__umulhi((unsigned)key, g.page_magic);
        slot = key - block * ps;
        return (size_t)__shfl(pages_cur, block - 64 * chunk, 64) * page_elems;
    };

    // Loads of a step are unconditional: a lane whose key lies outside the item's range reads a
    // key of the step that lies inside it (any valid address will do); scores of such keys are
    // masked and their values are zeroed before use.
    auto load_step = [&](Step& f, int kt) {
        enter_chunk(kt);
        const int lo = max(k_begin, kt), hi = min(k_end, kt + KEY_STEP) - 1;      // valid keys of this step
        // An item without keys (the first step is asked for before anybody looks) reads the start of the pool.
        const bool none = hi < lo;
        auto locate = [&](int key, int& slot) {
            const size_t page = locate_key(key, slot);
            if (none) slot = 0;
            return none ? (size_t)0 : page;
        };
#if LSA_BF16
        // A step that lies inside the item's range, with pages of a multiple of 16 keys: each half of the step lies in
        // one page, the same for all lanes, which one lane's table entry names (no exchange between lanes, and the
        // page's address is a scalar).
        if ((ps & 15) == 0 && kt >= k_begin && kt + KEY_STEP <= k_end) {
            size_t page[2];
            int slot0[2];
#pragma unroll
            for (int t2 = 0; t2 < 2; ++t2) {
                const int first = kt + 16 * t2;
                const int block = (int)__umulhi((unsigned)first, g.page_magic);
                slot0[t2] = first - block * ps;
                page[t2] = (size_t)__builtin_amdgcn_readlane(pages_cur, block - 64 * chunk) * page_elems;
            }
#pragma unroll
            for (int t2 = 0; t2 < 2; ++t2) {
                const elem_t* kp = keys + page[t2] + kv_head_keys + (size_t)(slot0[t2] + col) * D + 8 * quad;
#pragma unroll
                for (int s = 0; s < NS; ++s) {
                    if (32 * s + 32 <= D) {
                        f.k[t2][s] = *reinterpret_cast<const bf16x8*>(kp + 32 * s);
                    } else {
                        bf16x8 kf = *reinterpret_cast<const bf16x8*>(kp + 32 * s - (quad >= 2 ? 16 : 0));
                        if (quad >= 2) kf = (bf16x8){0, 0, 0, 0, 0, 0, 0, 0};
                        f.k[t2][s] = kf;
                    }
                }
            }
#pragma unroll
            for (int t2 = 0; t2 < 2; ++t2) {
                const elem_t* vp = values + page[t2] + kv_head_values + (size_t)col * ps + slot0[t2] + 4 * quad;
#pragma unroll
                for (int c = 0; c < ND; ++c) f.v[c][t2] = *reinterpret_cast<const bf16x4*>(vp + (size_t)(16 * c) * ps);
            }
            return;
        }
#pragma unroll
        for (int t2 = 0; t2 < 2; ++t2) {
            int slot;
            const int key = min(max(kt + 16 * t2 + col, lo), hi);
            const size_t page = locate(key, slot);
            const elem_t* kp = keys + page + kv_head_keys + (size_t)slot * D + 8 * quad;
#pragma unroll
            for (int s = 0; s < NS; ++s) {
                if (32 * s + 32 <= D) {
                    f.k[t2][s] = *reinterpret_cast<const bf16x8*>(kp + 32 * s);
                } else {                                   // head size not a multiple of 32: upper half of the last step is zero
                    bf16x8 kf = *reinterpret_cast<const bf16x8*>(kp + 32 * s - (quad >= 2 ? 16 : 0));
                    if (quad >= 2) kf = (bf16x8){0, 0, 0, 0, 0, 0, 0, 0};
                    f.k[t2][s] = kf;
                }
            }
        }
#pragma unroll
        for (int t2 = 0; t2 < 2; ++t2) {
            int slot;
            const int key0 = min(max(kt + 16 * t2 + 4 * quad, lo & ~3), hi & ~3);
            const size_t page = locate(key0, slot);
            const elem_t* vp = values + page + kv_head_values + (size_t)col * ps + slot;
#pragma unroll
            for (int c = 0; c < ND; ++c) f.v[c][t2] = *reinterpret_cast<const bf16x4*>(vp + (size_t)(16 * c) * ps);
        }
#else
        int slot;
        const int key = min(max(kt + col, lo), hi);
        const size_t page = locate(key, slot);
        const elem_t* kp = keys + page + kv_head_keys + (size_t)slot * D + 4 * quad;
#pragma unroll
        for (int s = 0; s < NS; ++s) f.k[s] = *reinterpret_cast<const f32x4*>(kp + 16 * s);
        const int key0 = min(max(kt + 4 * quad, lo & ~3), hi & ~3);
        const size_t vpage = locate(key0, slot);
        const elem_t* vp = values + vpage + kv_head_values + (size_t)col * ps + slot;
#pragma unroll
        for (int c = 0; c < ND; ++c) f.v[c] = *reinterpret_cast<const f32x4*>(vp + (size_t)(16 * c) * ps);
#endif
    };

    // The first step's keys and values: under way while the queries are prepared.
    Step a, b;
    load_step(a, kt_first);                     // also for an item without keys: see load_step
    __builtin_amdgcn_sched_barrier(0);          // and so are the queries, the rotation, the new key and value and the first keys

#if LSA_BF16
    // A head in the operand layout, normalised over the head and rotated as the separate kernel does it; the four
    // quads of a column share a head.
    auto norm_rotate = [&](bf16x8 (&h)[NS], bool normed, const HeadWeights& hw, bool rotated) {
        float x[NS][8];
        float sq = 0.f;
#pragma unroll
        for (int s = 0; s < NS; ++s)
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                x[s][e] = (float)h[s][e];
                sq += x[s][e] * x[s][e];
            }
        if (normed) {
            sq += __shfl_xor(sq, 16, 64);
            sq += __shfl_xor(sq, 32, 64);
            const float rstd = rsqrtf(sq / (float)D + fusion.eps);
#pragma unroll
            for (int s = 0; s < NS; ++s)
#pragma unroll
                for (int e = 0; e < 8; ++e) x[s][e] = x[s][e] * rstd * (e < 4 ? hw.w[s][0][e] : hw.w[s][1][e - 4]);
        }
        if (rotated) {
#pragma unroll
            for (int s = 0; s < NS / 2; ++s)
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    const float co = e < 4 ? rotation.c[s][0][e] : rotation.c[s][1][e - 4];
                    const float si = e < 4 ? rotation.s[s][0][e] : rotation.s[s][1][e - 4];
                    const float x1 = x[s][e], x2 = x[s + NS / 2][e];
                    x[s][e] = x1 * co - x2 * si;
                    x[s + NS / 2][e] = x2 * co + x1 * si;
                }
        }
#pragma unroll
        for (int s = 0; s < NS; ++s)
#pragma unroll
            for (int e = 0; e < 8; ++e) h[s][e] = (bf16_t)x[s][e];
    };
    if constexpr (FUSED_Q) norm_rotate(qf, normed, q_weights, rotated);
    HeadWeights k_weights;
    if constexpr (NEW_TOKEN) load_weights(k_weights, normed ? fusion.k_weight : readable);
#endif
    if (!pair_valid) {
#pragma unroll
        for (int s = 0; s < NS; ++s)
#if LSA_BF16
            qf[s] = (bf16x8){0, 0, 0, 0, 0, 0, 0, 0};
#else
            qf[s] = (f32x4){0.f, 0.f, 0.f, 0.f};
#endif
    }

    f32x4 acc[ND];
#pragma unroll
    for (int c = 0; c < ND; ++c) acc[c] = (f32x4){0.f, 0.f, 0.f, 0.f};
    float run_max = NEG_INF, run_sum = 0.f;    // run_sum: this lane's share (its keys) of the pair's sum

#if LSA_BF16
    if constexpr (NEW_TOKEN) if (takes_new_token) {
        // The online softmax starts from the new token's key (maximum = its score, sum = 1, output = its value);
        // column 0 puts key and value into the cache.
        const int new_pos = item.k_end - 1;
        norm_rotate(kh, normed, k_weights, rotated);
        float dot = 0.f;
#pragma unroll
        for (int s = 0; s < NS; ++s)
#pragma unroll
            for (int e = 0; e < 8; ++e) dot += (float)kh[s][e] * (float)qf[s][e];
        dot += __shfl_xor(dot, 16, 64);
        dot += __shfl_xor(dot, 32, 64);
        if (pair_valid) {
            run_max = dot * g.scale;
            run_sum = quad == 0 ? 1.f : 0.f;
#pragma unroll
            for (int c = 0; c < ND; ++c)
#pragma unroll
                for (int r = 0; r < 4; ++r) acc[c][r] = (float)vnew[c][r];
        }
        if (col == 0) {
            const int block = (int)__umulhi((unsigned)new_pos, g.page_magic);
            const int new_slot = new_pos - block * ps;
            const size_t page = (size_t)row_table[block] * page_elems;
            elem_t* kp = const_cast<elem_t*>(keys) + page + kv_head_keys + (size_t)new_slot * D + 8 * quad;
#pragma unroll
            for (int s = 0; s < NS; ++s) *reinterpret_cast<bf16x8*>(kp + 32 * s) = kh[s];
            elem_t* vp = const_cast<elem_t*>(values) + page + kv_head_values + (size_t)(4 * quad) * ps + new_slot;
#pragma unroll
            for (int c = 0; c < ND; ++c)
#pragma unroll
                for (int r = 0; r < 4; ++r) vp[(size_t)(16 * c + r) * ps] = vnew[c][r];
        }
    }
#endif

    auto compute_step = [&](Step& f, int kt) {
        const bool edge = kt < k_begin || kt + KEY_STEP > k_end;
#if LSA_BF16
        constexpr int NV = 8;
        float sv[NV];
        float tile_max = NEG_INF;
#pragma unroll
        for (int t2 = 0; t2 < 2; ++t2) {
            f32x4 s4 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int s = 0; s < NS; ++s) s4 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(f.k[t2][s], qf[s], s4, 0, 0, 0);
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int kpos = kt + 16 * t2 + 4 * quad + r;
                const bool seen = kpos >= k_begin && kpos < k_end && kpos <= q_pos && (g.window <= 0 || kpos > q_pos - g.window);
                const float v = seen ? s4[r] * g.scale : NEG_INF;
                sv[4 * t2 + r] = v;
                tile_max = fmaxf(tile_max, v);
            }
        }
#else
        constexpr int NV = 4;
        float sv[NV];
        float tile_max = NEG_INF;
        {
            f32x4 s4 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int s = 0; s < NS; ++s)
#pragma unroll
                for (int e = 0; e < 4; ++e) s4 = __builtin_amdgcn_mfma_f32_16x16x4f32(f.k[s][e], qf[s][e], s4, 0, 0, 0);
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int kpos = kt + 4 * quad + r;
                const bool seen = kpos >= k_begin && kpos < k_end && kpos <= q_pos && (g.window <= 0 || kpos > q_pos - g.window);
                const float v = seen ? s4[r] * g.scale : NEG_INF;
                sv[r] = v;
                tile_max = fmaxf(tile_max, v);
            }
        }
#endif
        tile_max = fmaxf(tile_max, __shfl_xor(tile_max, 16, 64));
        tile_max = fmaxf(tile_max, __shfl_xor(tile_max, 32, 64));
        const float new_max = fmaxf(run_max, tile_max);
        const float use_max = new_max == NEG_INF ? 0.f : new_max;
#if LSA_BF16
        const float alpha = __expf(run_max - use_max);   // run_max = -inf gives 0
#else
        const float alpha = expf(run_max - use_max);
#endif
        run_max = new_max;
        run_sum *= alpha;
#pragma unroll
        for (int c = 0; c < ND; ++c) acc[c] *= alpha;
#if LSA_BF16
        bf16x8 pf;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            const float p = __expf(sv[e] - use_max);
            run_sum += p;
            pf[e] = (bf16_t)p;
        }
#pragma unroll
        for (int c = 0; c < ND; ++c) {
            bf16x8 vf;
#pragma unroll
            for (int t2 = 0; t2 < 2; ++t2) {
                bf16x4 piece = f.v[c][t2];
                if (edge) {                      // keys outside the item's range may hold anything: keep them out of the sum
#pragma unroll
                    for (int r = 0; r < 4; ++r) {
                        const int kpos = kt + 16 * t2 + 4 * quad + r;
                        if (kpos < k_begin || kpos >= k_end) piece[r] = (bf16_t)0.f;
                    }
                }
#pragma unroll
                for (int r = 0; r < 4; ++r) vf[4 * t2 + r] = piece[r];
            }
            acc[c] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf, pf, acc[c], 0, 0, 0);
        }
#else
        float pv[4];
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            pv[r] = expf(sv[r] - use_max);
            run_sum += pv[r];
        }
#pragma unroll
        for (int c = 0; c < ND; ++c) {
            f32x4 vf = f.v[c];
            if (edge) {
#pragma unroll
                for (int r = 0; r < 4; ++r)
                    if (kt + 4 * quad + r < k_begin || kt + 4 * quad + r >= k_end) vf[r] = 0.f;
            }
#pragma unroll
            for (int r = 0; r < 4; ++r) acc[c] = __builtin_amdgcn_mfma_f32_16x16x4f32(vf[r], pv[r], acc[c], 0, 0, 0);
        }
#endif
    };

    if (k_begin < k_end) {
        int kt = (k_begin / KEY_STEP) * KEY_STEP;
        int steps = (k_end - kt + KEY_STEP - 1) / KEY_STEP;
        // Steady state without a branch between the loads of one step and the products of the
        // step before it, so that the wait for operands leaves the newer loads in flight.
        while (steps >= 3) {
            load_step(b, kt + KEY_STEP);
            compute_step(a, kt);
            load_step(a, kt + 2 * KEY_STEP);
            compute_step(b, kt + KEY_STEP);
            kt += 2 * KEY_STEP;
            steps -= 2;
        }
        if (steps == 2) {
            load_step(b, kt + KEY_STEP);
            compute_step(a, kt);
            compute_step(b, kt + KEY_STEP);
        } else {
            compute_step(a, kt);
        }
    }

    run_sum += __shfl_xor(run_sum, 16, 64);
    run_sum += __shfl_xor(run_sum, 32, 64);
    if constexpr (WG_MERGE) {
        // Every wavefront of the workgroup gets here (the launch has no workgroup with fewer than four items, and
        // nothing above returns).  The wavefronts of a tile are neighbours: all but the first leave their sums in LDS,
        // the first adds them up by log-sum-exp.
        constexpr int R = WG_RANGES > 0 ? WG_RANGES : 1, TILES = 4 / R;
        __shared__ f32x4 others_acc[4 - TILES][ND][64];
        __shared__ float ranges_max[4][16], ranges_sum[4][16];
        const int wave = threadIdx.x >> 6, first_wave = wave / R * R, member = wave - first_wave;
        if (quad == 0) {
            ranges_max[wave][col] = run_max;
            ranges_sum[wave][col] = run_sum;
        }
        if (member > 0) {
#pragma unroll
            for (int c = 0; c < ND; ++c) others_acc[first_wave / R * (R - 1) + member - 1][c][lane] = acc[c];
        }
        __syncthreads();
        if (member > 0 || !pair_valid) return;
        float top = NEG_INF;
#pragma unroll
        for (int w = 0; w < R; ++w) top = fmaxf(top, ranges_max[first_wave + w][col]);
        float weight[R], total = 0.f;
#pragma unroll
        for (int w = 0; w < R; ++w) {
            const float m = ranges_max[first_wave + w][col];
            weight[w] = m == NEG_INF ? 0.f : expf(m - top);
            total += weight[w] * ranges_sum[first_wave + w][col];
        }
        const float inv = total > 0.f ? 1.f / total : 0.f;
        elem_t* o = out + ((size_t)(token0 + pair_token) * g.n_q + head) * D + 4 * quad;
#pragma unroll
        for (int c = 0; c < ND; ++c) {
            f32x4 sum = acc[c] * weight[0];
#pragma unroll
            for (int w = 1; w < R; ++w) sum += others_acc[first_wave / R * (R - 1) + w - 1][c][lane] * weight[w];
#if LSA_BF16
            bf16x4 r4;
#pragma unroll
            for (int r = 0; r < 4; ++r) r4[r] = (bf16_t)(sum[r] * inv);
            *reinterpret_cast<bf16x4*>(o + 16 * c) = r4;
#else
            *reinterpret_cast<f32x4*>(o + 16 * c) = sum * inv;
#endif
        }
        return;
    }
    if (!pair_valid) return;
    if (slot < 0) {
        const float inv = run_sum > 0.f ? 1.f / run_sum : 0.f;
        elem_t* o = out + ((size_t)(token0 + pair_token) * g.n_q + head) * D + 4 * quad;
#pragma unroll
        for (int c = 0; c < ND; ++c) {
#if LSA_BF16
            bf16x4 r4;
#pragma unroll
            for (int r = 0; r < 4; ++r) r4[r] = (bf16_t)(acc[c][r] * inv);
            *reinterpret_cast<bf16x4*>(o + 16 * c) = r4;
#else
            *reinterpret_cast<f32x4*>(o + 16 * c) = acc[c] * inv;
#endif
        }
    } else {
        const size_t base = ((size_t)slot * gridDim.y + blockIdx.y) * 16 + col;
        float* pa = part_acc + base * D + 4 * quad;
#pragma unroll
        for (int c = 0; c < ND; ++c) *reinterpret_cast<f32x4*>(pa + 16 * c) = acc[c];
        if (quad == 0) {
            part_ml[base * 2] = run_max;
            part_ml[base * 2 + 1] = run_sum;
        }
    }
}

#if LSA_BF16
// ------------------------------------------------------------------------------------------------
// Portions of prompts: the four wavefronts of a workgroup take 4 * SUB consecutive tiles of 16 pairs
// of one request (SUB tiles each).  They see (almost) the same keys, so each step's 32 keys and values are fetched
// from the pages once per workgroup, straight into LDS (global_load_lds, 16 bytes a lane: no registers and no LDS
// stores on the way), into a ring of STAGES buffers: the loads of step i + STAGES - 1 are issued before the products
// of step i, one barrier a step, and every wavefront reads its MFMA operands from LDS, 16 bytes per lane and read
// (8-byte reads reach three quarters of the LDS rate at best).  Rows in LDS are padded so that the operand
// reads of a wavefront spread over the banks.  `tiles[i]` = {row, first token of the workgroup's tiles, k_begin, k_end}.
// The wavefronts of a workgroup come in one or two halves (HALVES, see below), each with a ring of its own.
//
// Key ranges: an entry of `tiles` may cover only a range [k_begin, k_end) of the keys that its tiles see, the other
// ranges being other entries (workgroups of their own).  `tile_slots[i]` = {first slot, slots between one tile and the
// next} then says where entry i leaves its partial results: tile j of the entry writes (max, sum, acc) of every valid
// pair to slot first + j * stride, in the layout of the wavefront-per-tile kernel, and merge_kernel combines the slots of
// a tile.  first = -1 (or no `tile_slots` at all): the entry has all keys of its tiles and writes the output itself.
// What the merge relies on: every slot that a merge entry names is written for every pair the merge reads, also by an
// entry none of whose keys a pair may see (it writes max = -inf, sum = 0, acc = 0, which the merge weighs with zero);
// pairs beyond the row's tokens or the group's heads are never read by the merge, and never written here.
//
// A load writes 64 lanes x 16 bytes to 1 KB of LDS in lane order, from wherever each lane points: a step's buffer is
// a row of such 1 KB chunks, and a lane's place in its chunk says which 16 bytes of the step it fetches (the padding
// of the rows, and the places behind the last row of a chunk, fetch a neighbour's bytes again).  Each of the four
// wavefronts fetches one quarter of a step: the keys of its first 16 keys, the keys of its last 16, the values of the
// first 16, the values of the last 16.  With pages of 16 keys or a multiple, such a quarter lies in one page: the
// wavefront looks one page up (a scalar), and every load is that page's address plus the lane's constant offset.
//   keys:   two blocks of 16 rows of D * 2 + 16 bytes.  The rows of a block are the 16 keys in page order, except that
//           in the second block rows i and i ^ 4 change places.  The score product t (of two) takes keys
//           8 a + b + 4 t (a, b = 0 .. 3) for its 16 rows: lane quad q is then left with keys 8 q + 4 t .. 8 q + 4 t + 3,
//           after both products a lane's eight scores are the step's keys 8 q .. 8 q + 7 in order; and the 16 rows of
//           a product lie at 16 different row numbers modulo 16 (that is what the exchange is for), so that their
//           reads spread over all banks.
//   values: two blocks (the first and the last 16 keys) of D rows (one head dimension) of 32 + 16 bytes: lane quad q
//           of the output product reads keys 8 q .. 8 q + 7 of its dimension as one 16-byte piece, the same 16 bytes
//           as in the page.
constexpr int K_ROW_SLOTS = D / 8 + 1, V_ROW_SLOTS = 3;            // 16-byte places of a row in LDS, the last one padding
constexpr int K_ROW = 16 * K_ROW_SLOTS, V_ROW = 16 * V_ROW_SLOTS;  // bytes of a key row, of a value row of one block
constexpr int K_BLOCK_CHUNKS = (16 * K_ROW_SLOTS + 63) / 64, V_BLOCK_CHUNKS = (D * V_ROW_SLOTS + 63) / 64;   // 1 KB each
constexpr int K_BLOCK_BYTES = 1024 * K_BLOCK_CHUNKS, V_BLOCK_BYTES = 1024 * V_BLOCK_CHUNKS;
constexpr int K_TILE_BYTES = 2 * K_BLOCK_BYTES, STEP_BYTES = K_TILE_BYTES + 2 * V_BLOCK_BYTES;
constexpr int STEP_LOADS = K_BLOCK_CHUNKS > V_BLOCK_CHUNKS ? K_BLOCK_CHUNKS : V_BLOCK_CHUNKS;     // of a wavefront per step
// Buffers in the ring: two (the loads of step i + 1 are under way while step i is multiplied).  A third, with the loads
// two steps ahead, was measured and gains nothing where the registers bound the wavefronts per SIMD, and costs the
// third workgroup per compute unit that the form with four tiles otherwise has room for (2,048 x 2,048: 95 against 78 us).
#ifndef LSA_TILE_STAGES
#define LSA_TILE_STAGES 2
#endif
constexpr int STAGES = LSA_TILE_STAGES;
// Tiles of 16 pairs per wavefront (SUB): with two, every key and value operand read from LDS feeds two products, which
// halves the LDS traffic per flop; the accumulators of two tiles fit the registers up to a head size of 128.
// The host picks one or two per launch: two pay when the rows are long (the longest workgroup then does not
// decide the time), one when they are short and there are few workgroups.
constexpr int MAX_SUB = LSA_ND <= 8 ? 2 : 1;
// Halves of a workgroup that split the keys between them (see the kernel): two where their buffers fit into LDS.
constexpr int MAX_HALVES = LSA_ND <= 8 ? 2 : 1;
// Wavefronts per SIMD wanted (they hide the latency of a step's dependent chain: LDS read, MFMA, softmax, MFMA),
// as far as the registers of SUB tiles allow.
#define LSA_TILE_MIN_WAVES(SUB) ((SUB) == 1 ? (LSA_ND <= 8 ? 3 : 1) : (LSA_ND <= 4 ? 3 : 2))
struct FullStep { static constexpr bool value = true; };        // every key of the step is seen by every pair
struct MaskedStep { static constexpr bool value = false; };
typedef unsigned u32x4 __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) unsigned char* lds_ptr_t;

// One load of a wavefront straight into LDS: lane i's 16 bytes go to `lds_address` + 16 i (a byte address in LDS, the
// same for all lanes).  Written out rather than called as a builtin: the compiler makes every later LDS read wait for
// all loads it knows to write LDS, and these are meant to stay in flight while the steps before them are read.
__device__ __forceinline__ void load_16_bytes_a_lane_to_lds(const void* source, unsigned lds_address) {
    asm volatile("s_mov_b32 m0, %1\n\tglobal_load_lds_dwordx4 %0, off" ::"v"(source), "s"(lds_address) : "memory", "m0");
}
// The same with one base for all lanes and a byte offset per lane.
__device__ __forceinline__ void load_16_bytes_a_lane_to_lds(const void* base, unsigned offset, unsigned lds_address) {
    asm volatile("s_mov_b32 m0, %2\n\tglobal_load_lds_dwordx4 %0, %1" ::"v"(offset), "s"(base), "s"(lds_address) : "memory", "m0");
}

// Waits until at most PENDING of this wavefront's loads are still under way (they land in the order they were
// issued), then for the workgroup.  Written out because __syncthreads() would wait for every load, also for those
// of the steps ahead, which are meant to stay in flight across the barrier.
template <int PENDING>
__device__ __forceinline__ void loads_landed_then_barrier() {
    static_assert(PENDING >= 0 && PENDING < 64, "the counter of loads in flight has six bits");
    asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)\n\ts_barrier" ::"n"(PENDING) : "memory");
}

// HALVES = 2: the workgroup has eight wavefronts; wavefronts 4 .. 7 take the same tiles as wavefronts 0 .. 3 and the
// second half of the keys' steps, through LDS buffers of their own, and leave their running maximum, sum and
// accumulators in LDS at the end, where the first four merge them by log-sum-exp.  The longest workgroup of a launch
// (the tiles that see the most keys) then walks half as many steps: a launch with few workgroups, which that
// workgroup bounds, ends sooner.  Both halves make the same number of trips through the loop (one of them may
// have a step less to compute), so that they meet at the same barriers.
//
// Key ranges: a plan may give the tiles of a workgroup a part of their keys only and the other parts to other
// workgroups (rows of few tiles behind long contexts: few workgroups, each with a long walk).  `tile_slots[i]` then
// names where entry i leaves its partial results, in the form the wavefront kernel leaves them (accumulators, running
// maximum in natural-logarithm units, sum): tile j of the workgroup writes slot `first + j * stride`, and `merge`
// combines a tile's slots.  first < 0 (or no `tile_slots` at all): the entry holds all keys and writes the output.
struct TileSlots { int first, stride; };

template <int SUB, int HALVES>
__global__ __launch_bounds__(256 * HALVES, LSA_TILE_MIN_WAVES(SUB)) void paged_attention_tile_kernel(
    const elem_t* __restrict__ q, long q_token_stride, elem_t* __restrict__ out,
    const elem_t* __restrict__ keys, const elem_t* __restrict__ values,
    const int* __restrict__ table, int table_stride,
    const int* __restrict__ row_start, const int* __restrict__ row_len, const int* __restrict__ row_ctx,
    const Item* __restrict__ tiles, const TileSlots* __restrict__ tile_slots, float* __restrict__ part_acc, float* __restrict__ part_ml,
    Geometry g) {
    __shared__ __attribute__((aligned(1024))) unsigned char lds_all[HALVES * STAGES * STEP_BYTES];
    const int half = HALVES > 1 ? __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 8)) : 0;     // (the same in all lanes, and known to be)
    const int lds_base = half * STAGES * STEP_BYTES;                  // this half's ring of buffers
    const unsigned lds_begin = (unsigned)__builtin_amdgcn_readfirstlane((int)((unsigned)(size_t)(lds_ptr_t)lds_all + (unsigned)lds_base));      // its byte address in LDS
    const int tid = threadIdx.x & 255, lane = tid & 63, wave = tid >> 6;
    // Workgroups are handed to the eight XCDs in turn, and each XCD has its own L2: with the KV head
    // running fastest over the workgroup index, an XCD keeps meeting the same few KV heads, whose
    // keys and values then stay in its L2 for all the tiles that read them.
    const int heads = g.n_kv * g.gtiles;
    const Item tile = tiles[blockIdx.x / heads];
    const int head_index = blockIdx.x % heads;
    const int kv_head = head_index / g.gtiles, gtile = head_index % g.gtiles;
    const int col = lane & 15, quad = lane >> 4;
    const int row = tile.row;
    const int n = row_len[row], first_pos = row_ctx[row] - n;
    const int q0 = tile.q0 + wave * SUB * g.tokens_per_tile;    // first token of this wavefront's SUB consecutive tiles
    const int pair_token = col / g.gheads, pair_head_in_group = gtile * g.gheads + col % g.gheads;
    const int head = kv_head * g.group + pair_head_in_group;
    bool pair_valid[SUB];
    int q_pos[SUB];
#pragma unroll
    for (int u = 0; u < SUB; ++u) {
        const int token = q0 + u * g.tokens_per_tile + pair_token;
        pair_valid[u] = pair_token < g.tokens_per_tile && token < n && pair_head_in_group < g.group;
        q_pos[u] = pair_valid[u] ? first_pos + token : -1;
    }
    const int* row_table = table + (size_t)row * table_stride;
    const int ps = g.page_size;
    const size_t kv_head_keys = (size_t)kv_head * ps * D, kv_head_values = (size_t)kv_head * D * ps;
    const size_t page_elems = (size_t)g.n_kv * ps * D;
    // Keys this wavefront's pairs can see at all: [wave_lo, wave_hi).
    const int wave_tokens = max(0, min(SUB * g.tokens_per_tile, n - q0));
    const int wave_hi = wave_tokens > 0 ? first_pos + q0 + wave_tokens : 0;
    const int wave_lo = g.window > 0 ? max(0, first_pos + q0 - g.window + 1) : 0;
    const int q_pos_min = first_pos + q0;                       // smallest position among the wavefront's valid pairs
    const float scale_log2 = g.scale * 1.44269504088896340736f;

    bf16x8 qf[SUB][NS];
    f32x4 acc[SUB][ND];
    float run_max[SUB], run_sum[SUB];
#pragma unroll
    for (int u = 0; u < SUB; ++u) {
#pragma unroll
        for (int s = 0; s < NS; ++s) {
            const int dim = 32 * s + 8 * quad;
            bf16x8 x = {0, 0, 0, 0, 0, 0, 0, 0};
            if (pair_valid[u] && dim < D)
                x = *reinterpret_cast<const bf16x8*>(q + (size_t)(row_start[row] + q0 + u * g.tokens_per_tile + pair_token) * q_token_stride +
                                                     (size_t)head * D + dim);
            qf[u][s] = x;
        }
#pragma unroll
        for (int c = 0; c < ND; ++c) acc[u][c] = (f32x4){0.f, 0.f, 0.f, 0.f};
        run_max[u] = NEG_INF;
        run_sum[u] = 0.f;
    }

    // The steps of 32 keys that cover the tile's keys, and this half's share of them: [k_begin, k_end).
    const int first_step = (tile.k_begin / 32) * 32;
    const int all_steps = tile.k_begin < tile.k_end ? (tile.k_end - 1 - first_step) / 32 + 1 : 0;
    const int trips = (all_steps + HALVES - 1) / HALVES;              // of every wavefront through the loop below
    const int cut = min(tile.k_end, first_step + 32 * trips);         // where the second half's keys begin
    const int k_begin = half ? cut : tile.k_begin, k_end = half ? tile.k_end : cut;
    const int my_steps = half ? all_steps - trips : trips;
    // The row's table, 64 entries at a time, one in each lane: a step's pages are read from there (64 pages hold a
    // whole number of steps).  After the load of the next 64 entries the wavefront waits for every load it has in
    // flight, this one included, and says so to the compiler: a wait that the compiler places itself would stand in
    // every trip (it cannot tell the trips that bring new entries from those that do not).
    // Each of the four wavefronts fetches one quarter of a step: keys or values (`of_values`), of the step's first or
    // last 16 keys (`late`); beside the page's number a lane keeps where the wavefront's kind of data begins in it.
    const int wave_uniform = __builtin_amdgcn_readfirstlane(wave);
    const bool of_values = wave_uniform >= 2;
    const int late = wave_uniform & 1;
    const char* const quarter_data = of_values ? reinterpret_cast<const char*>(values + kv_head_values) : reinterpret_cast<const char*>(keys + kv_head_keys);
    int chunk = -1, chunk_pages = 0;
    unsigned long long chunk_begins = 0;
    auto enter_chunk = [&](int kt) __attribute__((always_inline)) {
        const int c = (int)__umulhi((unsigned)kt, g.page_magic) >> 6;
        if (c != chunk) {
            chunk = c;
            chunk_pages = row_table[min(64 * c + lane, table_stride - 1)];
            __builtin_amdgcn_s_waitcnt(0x0F70);
            chunk_begins = (unsigned long long)(quarter_data + 2 * (size_t)chunk_pages * page_elems);
        }
    };

    // What this lane fetches in each of its wavefront's loads of a step: constant over the steps.  `piece_key` is the
    // piece's (first) key among those 16, `piece_at` the 16-byte piece of the key's row (keys) or the head dimension
    // (values), `piece_offset` its byte offset from where the first of the 16 keys lies in its page.
    const int quarter_chunks = of_values ? V_BLOCK_CHUNKS : K_BLOCK_CHUNKS;
    const unsigned quarter_lds = lds_begin + (unsigned)(of_values ? K_TILE_BYTES + late * V_BLOCK_BYTES : late * K_BLOCK_BYTES);
    int piece_key[STEP_LOADS], piece_at[STEP_LOADS];
    unsigned piece_offset[STEP_LOADS];
#pragma unroll
    for (int m = 0; m < STEP_LOADS; ++m) {
        const int place = 64 * min(m, quarter_chunks - 1) + lane;
        if (!of_values) {
            const int r = min(place / K_ROW_SLOTS, 15);
            piece_at[m] = min(place % K_ROW_SLOTS, D / 8 - 1);
            piece_key[m] = late ? (r ^ 4) : r;
            piece_offset[m] = (unsigned)(piece_key[m] * (2 * D) + 16 * piece_at[m]);
        } else {
            piece_at[m] = min(place / V_ROW_SLOTS, D - 1);
            piece_key[m] = 8 * min(place % V_ROW_SLOTS, 1);
            piece_offset[m] = (unsigned)(2 * (piece_at[m] * ps + piece_key[m]));
        }
    }
    const bool pages_of_16 = (ps & 15) == 0;        // then each half of a step (16 keys) lies inside one page
    auto issue_loads = [&](int stage, int kt) __attribute__((always_inline)) {
        enter_chunk(kt);
        const unsigned buffer = quarter_lds + (unsigned)(stage * STEP_BYTES);
        const int first_key = kt + 16 * late;
        if (pages_of_16 && kt >= k_begin && kt + 32 <= k_end) {
            // Interior step: one page lookup for the whole wavefront (scalar).
            const int block = (int)__umulhi((unsigned)first_key, g.page_magic), slot = first_key - block * ps;
            const unsigned low = (unsigned)__builtin_amdgcn_readlane((int)(unsigned)chunk_begins, block - 64 * chunk);
            const unsigned high = (unsigned)__builtin_amdgcn_readlane((int)(unsigned)(chunk_begins >> 32), block - 64 * chunk);
            const char* base = reinterpret_cast<const char*>(((unsigned long long)high << 32) | low) + (of_values ? 2 * slot : 2 * D * slot);
#pragma unroll
            for (int m = 0; m < STEP_LOADS; ++m)
                load_16_bytes_a_lane_to_lds(base, piece_offset[m], buffer + 1024u * (unsigned)min(m, quarter_chunks - 1));
            return;
        }
        // A step at an end of the key range, or pages that are no multiple of 16 keys: every lane looks its key's
        // page up.  Keys outside the range are never fetched (their pages may not be the request's): the nearest
        // key inside stands in, and the scores and values of such places are masked where they are used.
        const int lo = max(k_begin, kt), hi = min(k_end, kt + 32) - 1;
#pragma unroll
        for (int m = 0; m < STEP_LOADS; ++m) {
            const int key = of_values ? min(max(first_key + piece_key[m], lo & ~7), hi & ~7) : min(max(first_key + piece_key[m], lo), hi);
            const int block = (int)__umulhi((unsigned)key, g.page_magic), slot = key - block * ps;
            const size_t page = (size_t)__shfl(chunk_pages, block - 64 * chunk, 64) * page_elems;
            const char* source = of_values
                ? reinterpret_cast<const char*>(values + page + kv_head_values + (size_t)piece_at[m] * ps + slot)
                : reinterpret_cast<const char*>(keys + page + kv_head_keys + (size_t)slot * D + 8 * piece_at[m]);
            load_16_bytes_a_lane_to_lds(source, buffer + 1024u * (unsigned)min(m, quarter_chunks - 1));
        }
    };
    // Where this lane reads its operands in a step's buffer: the key row of each of the two score products (key
    // 8 a + b + 4 t for lane column 4 a + b), and its 16 bytes of a value row.
    int key_row_at[2];
#pragma unroll
    for (int t2 = 0; t2 < 2; ++t2) {
        const int key = 8 * (col >> 2) + (col & 3) + 4 * t2;
        key_row_at[t2] = (key >> 4) * K_BLOCK_BYTES + (key < 16 ? key : ((key - 16) ^ 4)) * K_ROW + 16 * quad;
    }
    const int value_at = K_TILE_BYTES + (quad >> 1) * V_BLOCK_BYTES + col * V_ROW + 16 * (quad & 1);
    // The steps that every pair of the wavefront sees completely (they need no mask) lie in [full_from, full_to]; the
    // steps that have anything for its pairs in (active_from, active_to).
    const bool whole_tiles = wave_tokens == SUB * g.tokens_per_tile && g.gheads * g.tokens_per_tile == 16 && (gtile + 1) * g.gheads <= g.group;
    const int full_from = !whole_tiles ? 0x7fffffff : g.window > 0 ? max(k_begin, first_pos + q0 + wave_tokens - g.window) : k_begin;
    const int full_to = min(k_end - 32, q_pos_min - 31);
    // Scores stay as the products left them; the scale (in units of ln 2, so that the exponential is one
    // instruction) goes into the multiply-add that also subtracts the running maximum.  FULL: every key of
    // the step is seen by every pair of the wavefront, nothing is masked.
    auto compute_step = [&](auto full_tag, int stage, int kt) __attribute__((always_inline)) {
        constexpr bool FULL = decltype(full_tag)::value;
        const unsigned char* buffer = lds_all + lds_base + stage * STEP_BYTES;
        float sv[SUB][8];
        float tile_max[SUB];
#pragma unroll
        for (int u = 0; u < SUB; ++u) tile_max[u] = NEG_INF;
#pragma unroll
        for (int t2 = 0; t2 < 2; ++t2) {
            f32x4 s4[SUB];
#pragma unroll
            for (int u = 0; u < SUB; ++u) s4[u] = (f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int s = 0; s < NS; ++s) {
                bf16x8 kf = {0, 0, 0, 0, 0, 0, 0, 0};
                if (32 * s + 32 <= D || quad < 2) kf = *reinterpret_cast<const bf16x8*>(buffer + key_row_at[t2] + 64 * s);
#pragma unroll
                for (int u = 0; u < SUB; ++u) s4[u] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf, qf[u][s], s4[u], 0, 0, 0);
            }
#pragma unroll
            for (int u = 0; u < SUB; ++u)
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    float v = s4[u][r];
                    if (!FULL) {
                        const int kpos = kt + 8 * quad + 4 * t2 + r;
                        const bool seen = kpos >= k_begin && kpos < k_end && kpos <= q_pos[u] && (g.window <= 0 || kpos > q_pos[u] - g.window);
                        v = seen ? v : NEG_INF;
                    }
                    sv[u][4 * t2 + r] = v;
                    tile_max[u] = fmaxf(tile_max[u], v);
                }
        }
        // Values of keys outside the range may be anything (a page's places behind the context were never written):
        // their weights are zero, and so that zero times anything stays zero they are cleared where they are read.
        u32x4 keep = {~0u, ~0u, ~0u, ~0u};
        if (!FULL) {
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int kpos = kt + 8 * quad + 2 * i;
                keep[i] = ((kpos >= k_begin && kpos < k_end) ? 0x0000ffffu : 0u) | ((kpos + 1 >= k_begin && kpos + 1 < k_end) ? 0xffff0000u : 0u);
            }
        }
        auto value_operand = [&](int c) __attribute__((always_inline)) {
            const u32x4 raw = *reinterpret_cast<const u32x4*>(buffer + value_at + 16 * c * V_ROW);
            return __builtin_bit_cast(bf16x8, FULL ? raw : (raw & keep));
        };
        // The value operands are asked for now, so that they arrive while the softmax runs, and the output products
        // of the first tile are issued before the softmax of the second: the MFMA pipe works on them meanwhile.
        // (With one tile per wavefront there is nothing to overlap them with; they are read where they are used.)
        bf16x8 vf[SUB > 1 ? ND : 1];
        if (SUB > 1) {
#pragma unroll
            for (int c = 0; c < ND; ++c) vf[c] = value_operand(c);
        }
        // The running maximum of a pair only moves when some key of this step beats it, which
        // soon becomes rare: then the exchange between the lanes of a pair and the rescaling of
        // the accumulators are skipped (the result is the same, the maximum being unchanged).
#pragma unroll
        for (int u = 0; u < SUB; ++u) {
            if (__any(tile_max[u] > run_max[u])) {
                float top = fmaxf(tile_max[u], __shfl_xor(tile_max[u], 16, 64));
                top = fmaxf(top, __shfl_xor(top, 32, 64));
                const float new_max = fmaxf(run_max[u], top);
                const float alpha = __builtin_amdgcn_exp2f((run_max[u] - (new_max == NEG_INF ? 0.f : new_max)) * scale_log2);
                run_max[u] = new_max;
                run_sum[u] *= alpha;
#pragma unroll
                for (int c = 0; c < ND; ++c) acc[u][c] *= alpha;
            }
            const float shift = run_max[u] == NEG_INF ? 0.f : -run_max[u] * scale_log2;
            bf16x8 pf;
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const float p = __builtin_amdgcn_exp2f(__builtin_fmaf(sv[u][e], scale_log2, shift));
                run_sum[u] += p;
                pf[e] = (bf16_t)p;
            }
#pragma unroll
            for (int c = 0; c < ND; ++c) {
                const bf16x8 value = SUB > 1 ? vf[SUB > 1 ? c : 0] : value_operand(c);
                acc[u][c] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(value, pf, acc[u][c], 0, 0, 0);
            }
        }
    };
    auto compute = [&](int stage, int kt) __attribute__((always_inline)) {
        if (kt >= wave_hi || kt + 32 <= wave_lo) return;          // nothing for this wavefront's pairs in this step
        if (kt >= full_from && kt <= full_to) compute_step(FullStep{}, stage, kt);
        else compute_step(MaskedStep{}, stage, kt);
    };

    if (all_steps > 0) {
        // Loads run STAGES - 1 steps ahead of the products.  They are issued unconditionally (past the end they fetch
        // the last step again; a half without keys fetches the step before its own), the same number by every
        // wavefront in every trip, so that counting them tells which have landed.  A trip: wait for this step's loads
        // (all but those of the steps ahead), meet the others (now everybody's pieces of this step are in LDS, and
        // everybody is through with the buffer of the step before, which the next loads overwrite), issue, compute.
        int kt = half ? first_step + 32 * trips : first_step;
        const int last = my_steps > 0 ? kt + 32 * (my_steps - 1) : max(first_step, kt - 32);
        if (my_steps == 0) kt = last;
        // (every load so far has landed before the first one into LDS is issued: the compiler, which does not see
        // those, then never waits for "all loads" inside the loop on behalf of the queries)
        __builtin_amdgcn_s_waitcnt(0x0F70);
#pragma unroll
        for (int ahead = 0; ahead < STAGES - 1; ++ahead) issue_loads(ahead, min(kt + 32 * ahead, last));
        int stage = 0;
        for (int trip = 0; trip < trips; ++trip) {
            loads_landed_then_barrier<(STAGES - 2) * STEP_LOADS>();
            issue_loads(stage == 0 ? STAGES - 1 : stage - 1, min(kt + 32 * (STAGES - 1), last));
            if (trip < my_steps) compute(stage, kt);
            stage = stage + 1 == STAGES ? 0 : stage + 1;
            kt += 32;
        }
    }
    // Where this entry's results go: the output, or a slot per tile (asked for here, at the end, where it is needed).
    TileSlots slots = {-1, 0};
    if (tile_slots != nullptr) slots = tile_slots[blockIdx.x / heads];
    if constexpr (HALVES > 1) {
        // The second half's wavefronts hand over what they have; the first half's add it to theirs.  The buffers
        // of keys and values are free once every load has landed and everybody has passed the barrier.
        loads_landed_then_barrier<0>();
        float* handed = reinterpret_cast<float*>(lds_all);
        constexpr int PER_WAVE = SUB * (ND * 256 + 32);               // floats: accumulators (ND x 64 lanes x 4), then max and sum of 16 pairs
        static_assert(4 * PER_WAVE * sizeof(float) <= sizeof(lds_all), "the buffers of keys and values hold what the second half hands over");
        float* mine = handed + (size_t)wave * PER_WAVE;
#pragma unroll
        for (int u = 0; u < SUB; ++u) {
            float total = run_sum[u];
            total += __shfl_xor(total, 16, 64);
            total += __shfl_xor(total, 32, 64);
            run_sum[u] = total;                                       // the pair's whole sum, in every lane of the pair
        }
        if (half) {
#pragma unroll
            for (int u = 0; u < SUB; ++u) {
                float* block = mine + u * (ND * 256 + 32);
#pragma unroll
                for (int c = 0; c < ND; ++c) *reinterpret_cast<f32x4*>(block + (c * 64 + lane) * 4) = acc[u][c];
                if (quad == 0) {
                    block[ND * 256 + col] = run_max[u];
                    block[ND * 256 + 16 + col] = run_sum[u];
                }
            }
        }
        __syncthreads();
        if (half) return;
#pragma unroll
        for (int u = 0; u < SUB; ++u) {
            const float* block = mine + u * (ND * 256 + 32);
            const float other_max = block[ND * 256 + col], other_sum = block[ND * 256 + 16 + col];
            const float top = fmaxf(run_max[u], other_max);
            const float w0 = run_max[u] == NEG_INF ? 0.f : __builtin_amdgcn_exp2f((run_max[u] - top) * scale_log2);
            const float w1 = other_max == NEG_INF ? 0.f : __builtin_amdgcn_exp2f((other_max - top) * scale_log2);
            const float total = w0 * run_sum[u] + w1 * other_sum;
            if (!pair_valid[u]) continue;
            if (slots.first >= 0) {
                const size_t base = ((size_t)(slots.first + (wave * SUB + u) * slots.stride) * heads + head_index) * 16 + col;
                float* pa = part_acc + base * D + 4 * quad;
#pragma unroll
                for (int c = 0; c < ND; ++c) {
                    const f32x4 other = *reinterpret_cast<const f32x4*>(block + (c * 64 + lane) * 4);
                    *reinterpret_cast<f32x4*>(pa + 16 * c) = acc[u][c] * w0 + other * w1;
                }
                if (quad == 0) {
                    part_ml[base * 2] = top == NEG_INF ? NEG_INF : top * g.scale;
                    part_ml[base * 2 + 1] = total;
                }
                continue;
            }
            const float inv = total > 0.f ? 1.f / total : 0.f;
            elem_t* o = out + ((size_t)(row_start[row] + q0 + u * g.tokens_per_tile + pair_token) * g.n_q + head) * D + 4 * quad;
#pragma unroll
            for (int c = 0; c < ND; ++c) {
                const f32x4 other = *reinterpret_cast<const f32x4*>(block + (c * 64 + lane) * 4);
                bf16x4 r4;
#pragma unroll
                for (int r = 0; r < 4; ++r) r4[r] = (bf16_t)((acc[u][c][r] * w0 + other[r] * w1) * inv);
                *reinterpret_cast<bf16x4*>(o + 16 * c) = r4;
            }
        }
        return;
    }
    // (the loads issued past the end still write LDS: a wavefront ends only when they have landed)
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
#pragma unroll
    for (int u = 0; u < SUB; ++u) {
        float total = run_sum[u];
        total += __shfl_xor(total, 16, 64);
        total += __shfl_xor(total, 32, 64);
        if (!pair_valid[u]) continue;
        if (slots.first >= 0) {
            const size_t base = ((size_t)(slots.first + (wave * SUB + u) * slots.stride) * heads + head_index) * 16 + col;
            float* pa = part_acc + base * D + 4 * quad;
#pragma unroll
            for (int c = 0; c < ND; ++c) *reinterpret_cast<f32x4*>(pa + 16 * c) = acc[u][c];
            if (quad == 0) {
                part_ml[base * 2] = run_max[u] == NEG_INF ? NEG_INF : run_max[u] * g.scale;
                part_ml[base * 2 + 1] = total;
            }
            continue;
        }
        const float inv = total > 0.f ? 1.f / total : 0.f;
        elem_t* o = out + ((size_t)(row_start[row] + q0 + u * g.tokens_per_tile + pair_token) * g.n_q + head) * D + 4 * quad;
#pragma unroll
        for (int c = 0; c < ND; ++c) {
            bf16x4 r4;
#pragma unroll
            for (int r = 0; r < 4; ++r) r4[r] = (bf16_t)(acc[u][c][r] * inv);
            *reinterpret_cast<bf16x4*>(o + 16 * c) = r4;
        }
    }
}
#else  // float32
// ------------------------------------------------------------------------------------------------
// Portions of prompts in float32: the same arrangement as the bfloat16 kernel above in its plainest form.  The four
// wavefronts of a workgroup take four consecutive tiles of 16 pairs of one request; each step's 16 keys and values
// are fetched from the pages once per workgroup (a step ahead, through registers into the other of two LDS buffers)
// and every wavefront reads its operands from there, so a key travels from the caches once for 64 pairs instead
// of once for 16.  Every step is masked; products are true 32-bit (16x16x4 MFMAs).
constexpr int TK_ROW = D * 4 + 16;                 // bytes of a key row in LDS (padded: the 16 rows of an operand read spread over the banks)
constexpr int TV_ROW = 16 * 4 + 16;                // bytes of a value row (one head dimension, 16 keys)
constexpr int TK_BYTES = 16 * TK_ROW, TV_BYTES = D * TV_ROW;
constexpr int TK_PIECES = 16 * (D / 4), TV_PIECES = D * 4;        // 16-byte pieces of a step: four dimensions of a key; four keys of a dimension
constexpr int TKP = (TK_PIECES + 255) / 256, TVP = (TV_PIECES + 255) / 256;

__global__ __launch_bounds__(256) void paged_attention_tile_kernel_f32(
    const float* __restrict__ q, long q_token_stride, float* __restrict__ out,
    const float* __restrict__ keys, const float* __restrict__ values,
    const int* __restrict__ table, int table_stride,
    const int* __restrict__ row_start, const int* __restrict__ row_len, const int* __restrict__ row_ctx,
    const Item* __restrict__ tiles, Geometry g) {
    __shared__ __attribute__((aligned(16))) unsigned char lds[2 * (TK_BYTES + TV_BYTES)];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int heads = g.n_kv * g.gtiles;
    const Item tile = tiles[blockIdx.x / heads];
    const int head_index = blockIdx.x % heads;
    const int kv_head = head_index / g.gtiles, gtile = head_index % g.gtiles;
    const int col = lane & 15, quad = lane >> 4;
    const int row = tile.row;
    const int n = row_len[row], first_pos = row_ctx[row] - n;
    const int q0 = tile.q0 + wave * g.tokens_per_tile;             // first token of this wavefront's tile
    const int pair_token = col / g.gheads, pair_head_in_group = gtile * g.gheads + col % g.gheads;
    const int head = kv_head * g.group + pair_head_in_group;
    const bool pair_valid = pair_token < g.tokens_per_tile && q0 + pair_token < n && pair_head_in_group < g.group;
    const int q_pos = pair_valid ? first_pos + q0 + pair_token : -1;
    const int* row_table = table + (size_t)row * table_stride;
    const int ps = g.page_size;
    const size_t kv_head_keys = (size_t)kv_head * ps * D, kv_head_values = (size_t)kv_head * D * ps;
    const size_t page_elems = (size_t)g.n_kv * ps * D;
    const int wave_tokens = max(0, min(g.tokens_per_tile, n - q0));
    const int wave_hi = wave_tokens > 0 ? first_pos + q0 + wave_tokens : 0;                  // keys this wavefront's pairs can see: [wave_lo, wave_hi)
    const int wave_lo = g.window > 0 ? max(0, first_pos + q0 - g.window + 1) : 0;

    f32x4 qf[NS];
#pragma unroll
    for (int s = 0; s < NS; ++s) {
        f32x4 x = {0.f, 0.f, 0.f, 0.f};
        if (pair_valid) x = *reinterpret_cast<const f32x4*>(q + (size_t)(row_start[row] + q0 + pair_token) * q_token_stride + (size_t)head * D + 16 * s + 4 * quad);
        qf[s] = x;
    }
    f32x4 acc[ND];
#pragma unroll
    for (int c = 0; c < ND; ++c) acc[c] = (f32x4){0.f, 0.f, 0.f, 0.f};
    float run_max = NEG_INF, run_sum = 0.f;

    const int k_begin = tile.k_begin, k_end = tile.k_end;
    int chunk = -1, pages_cur = 0, pages_next = 0;
    auto table_chunk = [&](int c) __attribute__((always_inline)) { return row_table[min(64 * c + lane, table_stride - 1)]; };
    auto enter_chunk = [&](int kt) __attribute__((always_inline)) {
        const int c = (int)__umulhi((unsigned)kt, g.page_magic) >> 6;
        if (c != chunk) {
            pages_cur = (chunk >= 0 && c == chunk + 1) ? pages_next : table_chunk(c);
            chunk = c;
            pages_next = table_chunk(c + 1);
        }
    };
    auto locate = [&](int key, int& slot) __attribute__((always_inline)) {
        const int block = (int)__umulhi((unsigned)key, g.page_magic);
        slot = key - block * ps;
        return (size_t)__shfl(pages_cur, block - 64 * chunk, 64) * page_elems;
    };
    struct Staged { f32x4 k[TKP], v[TVP]; };
    // Loads are unconditional: a piece whose keys lie outside the tile's range reads keys of the step that lie inside.
    auto issue_loads = [&](Staged& r, int kt) __attribute__((always_inline)) {
        enter_chunk(kt);
        const int lo = max(k_begin, kt), hi = min(k_end, kt + 16) - 1;
#pragma unroll
        for (int j = 0; j < TKP; ++j) {
            const int piece = min(tid + 256 * j, TK_PIECES - 1);
            int slot;
            const int key = min(max(kt + piece / (D / 4), lo), hi);
            const size_t page = locate(key, slot);
            r.k[j] = *reinterpret_cast<const f32x4*>(keys + page + kv_head_keys + (size_t)slot * D + 4 * (piece % (D / 4)));
        }
#pragma unroll
        for (int j = 0; j < TVP; ++j) {
            const int piece = min(tid + 256 * j, TV_PIECES - 1);
            int slot;
            const int key0 = min(max(kt + 4 * (piece & 3), lo & ~3), hi & ~3);
            const size_t page = locate(key0, slot);
            r.v[j] = *reinterpret_cast<const f32x4*>(values + page + kv_head_values + (size_t)(piece >> 2) * ps + slot);
        }
    };
    auto store_lds = [&](int buf, Staged& r, int kt) __attribute__((always_inline)) {
        unsigned char* kl = lds + buf * (TK_BYTES + TV_BYTES);
        unsigned char* vl = kl + TK_BYTES;
#pragma unroll
        for (int j = 0; j < TKP; ++j) {
            const int piece = tid + 256 * j;
            if (piece < TK_PIECES) *reinterpret_cast<f32x4*>(kl + (piece / (D / 4)) * TK_ROW + 16 * (piece % (D / 4))) = r.k[j];
        }
#pragma unroll
        for (int j = 0; j < TVP; ++j) {
            const int piece = tid + 256 * j;
            f32x4 four = r.v[j];
#pragma unroll
            for (int e = 0; e < 4; ++e) {               // keys outside the range may hold anything: keep them out of the sums
                const int kpos = kt + 4 * (piece & 3) + e;
                if (kpos < k_begin || kpos >= k_end) four[e] = 0.f;
            }
            if (piece < TV_PIECES) *reinterpret_cast<f32x4*>(vl + (piece >> 2) * TV_ROW + 16 * (piece & 3)) = four;
        }
    };
    auto compute = [&](int buf, int kt) __attribute__((always_inline)) {
        if (kt >= wave_hi || kt + 16 <= wave_lo) return;           // nothing for this wavefront's pairs in this step
        const unsigned char* kl = lds + buf * (TK_BYTES + TV_BYTES);
        const unsigned char* vl = kl + TK_BYTES;
        f32x4 s4 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int s = 0; s < NS; ++s) {
            const f32x4 kf = *reinterpret_cast<const f32x4*>(kl + col * TK_ROW + 64 * s + 16 * quad);
#pragma unroll
            for (int r = 0; r < 4; ++r) s4 = __builtin_amdgcn_mfma_f32_16x16x4f32(kf[r], qf[s][r], s4, 0, 0, 0);
        }
        float sv[4];
        float step_max = NEG_INF;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const int kpos = kt + 4 * quad + r;
            const bool seen = kpos >= k_begin && kpos < k_end && kpos <= q_pos && (g.window <= 0 || kpos > q_pos - g.window);
            sv[r] = seen ? s4[r] * g.scale : NEG_INF;
            step_max = fmaxf(step_max, sv[r]);
        }
        step_max = fmaxf(step_max, __shfl_xor(step_max, 16, 64));
        step_max = fmaxf(step_max, __shfl_xor(step_max, 32, 64));
        const float new_max = fmaxf(run_max, step_max);
        const float use_max = new_max == NEG_INF ? 0.f : new_max;
        const float alpha = expf(run_max - use_max);                 // exp(-inf) = 0 for the first keys
        run_max = new_max;
        run_sum *= alpha;
        float pv[4];
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            pv[r] = expf(sv[r] - use_max);
            run_sum += pv[r];
        }
#pragma unroll
        for (int c = 0; c < ND; ++c) {
            acc[c] *= alpha;
            const f32x4 vf = *reinterpret_cast<const f32x4*>(vl + (16 * c + col) * TV_ROW + 16 * quad);
#pragma unroll
            for (int r = 0; r < 4; ++r) acc[c] = __builtin_amdgcn_mfma_f32_16x16x4f32(vf[r], pv[r], acc[c], 0, 0, 0);
        }
    };

    if (k_begin < k_end) {
        Staged ahead;
        int kt = (k_begin / 16) * 16;
        const int last = ((k_end - 1) / 16) * 16;
        issue_loads(ahead, kt);
        store_lds(0, ahead, kt);
        __syncthreads();
        int buf = 0;
        while (true) {
            const bool more = kt + 16 <= last;
            if (more) issue_loads(ahead, kt + 16);                // under way while this step is multiplied
            compute(buf, kt);
            if (!more) break;
            store_lds(buf ^ 1, ahead, kt + 16);                   // the other buffer: everybody left it at the last barrier
            __syncthreads();
            buf ^= 1;
            kt += 16;
        }
    }
    run_sum += __shfl_xor(run_sum, 16, 64);
    run_sum += __shfl_xor(run_sum, 32, 64);
    if (!pair_valid) return;
    const float inv = run_sum > 0.f ? 1.f / run_sum : 0.f;
    float* o = out + ((size_t)(row_start[row] + q0 + pair_token) * g.n_q + head) * D + 4 * quad;
#pragma unroll
    for (int c = 0; c < ND; ++c) *reinterpret_cast<f32x4*>(o + 16 * c) = acc[c] * inv;
}
#endif  // LSA_BF16

// Merge the partial slots of a tile: out = sum_s w_s acc_s / sum_s w_s l_s, w_s = exp(m_s - max m).
struct Merge { int row, q0, first_slot, n_slots; };

constexpr int MERGE_WAVES = 4;         // at most; the launch brings as many as the merges' slots can use
constexpr int MERGE_MOST_SLOTS = 128;  // key ranges one tile may be split into (two slots' weights per lane of a wavefront)

__global__ __launch_bounds__(MERGE_WAVES * 64) void merge_kernel(
    elem_t* __restrict__ out, const int* __restrict__ row_start, const int* __restrict__ row_len,
    const Merge* __restrict__ merges, const float* __restrict__ part_acc, const float* __restrict__ part_ml, Geometry g) {
    // One block per (tile, KV head, pair).  First the slots' weights (a thread per slot), then the weighted sum:
    // with W wavefronts in the block, wavefront v takes slots v, v + W, ... (four loads in flight each, so 64 slots
    // are four trips to memory for four wavefronts, not sixteen), a lane two neighbouring output dimensions, and the
    // wavefronts' sums meet in LDS.
    constexpr int PAIRS = D / 2, PER_LANE = (PAIRS + 63) / 64;
    __shared__ float weight[MERGE_MOST_SLOTS];
    __shared__ float inv_total;
    __shared__ float2 wave_total[MERGE_WAVES - 1][PAIRS];
    const Merge m = merges[blockIdx.x];
    const int col = blockIdx.z;
    const int kv_head = blockIdx.y / g.gtiles, gtile = blockIdx.y % g.gtiles;
    const int pair_token = col / g.gheads, pair_head_in_group = gtile * g.gheads + col % g.gheads;
    if (pair_token >= g.tokens_per_tile || m.q0 + pair_token >= row_len[m.row] || pair_head_in_group >= g.group) return;
    const size_t stride = (size_t)gridDim.y * 16;                       // pairs per slot
    const size_t base = ((size_t)m.first_slot * gridDim.y + blockIdx.y) * 16 + col;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, waves = blockDim.x >> 6;
    if (wave == 0) {
        float mx[MERGE_MOST_SLOTS / 64], sum[MERGE_MOST_SLOTS / 64];
        float top = NEG_INF;
#pragma unroll
        for (int i = 0; i < MERGE_MOST_SLOTS / 64; ++i) {
            const int s = lane + 64 * i;
            mx[i] = NEG_INF;
            sum[i] = 0.f;
            if (s < m.n_slots) {
                mx[i] = part_ml[(base + s * stride) * 2];
                sum[i] = part_ml[(base + s * stride) * 2 + 1];
            }
            top = fmaxf(top, mx[i]);
        }
        top = wave_max(top);
        float weighted = 0.f;
#pragma unroll
        for (int i = 0; i < MERGE_MOST_SLOTS / 64; ++i) {
            const float w = mx[i] == NEG_INF ? 0.f : expf(mx[i] - top);
            weight[lane + 64 * i] = w;
            weighted += w * sum[i];
        }
        const float total = wave_sum(weighted);
        if (lane == 0) inv_total = total > 0.f ? 1.f / total : 0.f;
    }
    // The partial results do not depend on the weights: their first loads are issued before the barrier.
    const float* acc = part_acc + base * D;
    float2 total[PER_LANE];
#pragma unroll
    for (int i = 0; i < PER_LANE; ++i) total[i] = make_float2(0.f, 0.f);
    auto slot_values = [&](int s, int i) {
        const int pair = min(lane + 64 * i, PAIRS - 1);
        return *reinterpret_cast<const float2*>(acc + (size_t)min(s, m.n_slots - 1) * stride * D + 2 * pair);
    };
    float2 first[PER_LANE][4];
#pragma unroll
    for (int i = 0; i < PER_LANE; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) first[i][j] = slot_values(wave + waves * j, i);
    __syncthreads();
#pragma unroll
    for (int i = 0; i < PER_LANE; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int s = wave + waves * j;
            const float w = s < m.n_slots ? weight[s] : 0.f;
            total[i].x += w * first[i][j].x;
            total[i].y += w * first[i][j].y;
        }
    for (int s0 = wave + 4 * waves; s0 < m.n_slots; s0 += 4 * waves) {
#pragma unroll
        for (int i = 0; i < PER_LANE; ++i) {
            float2 v[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) v[j] = slot_values(s0 + waves * j, i);
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const int s = s0 + waves * j;
                const float w = s < m.n_slots ? weight[s] : 0.f;
                total[i].x += w * v[j].x;
                total[i].y += w * v[j].y;
            }
        }
    }
    if (wave) {
#pragma unroll
        for (int i = 0; i < PER_LANE; ++i)
            if (lane + 64 * i < PAIRS) wave_total[wave - 1][lane + 64 * i] = total[i];
    }
    __syncthreads();
    if (wave) return;
    const int head = kv_head * g.group + pair_head_in_group;
    elem_t* o = out + ((size_t)(row_start[m.row] + m.q0 + pair_token) * g.n_q + head) * D;
#pragma unroll
    for (int i = 0; i < PER_LANE; ++i) {
        const int pair = lane + 64 * i;
        if (pair >= PAIRS) continue;
        float2 sum = total[i];
#pragma unroll
        for (int v = 0; v < waves - 1; ++v) {
            sum.x += wave_total[v][pair].x;
            sum.y += wave_total[v][pair].y;
        }
        o[2 * pair] = (elem_t)(sum.x * inv_total);
        o[2 * pair + 1] = (elem_t)(sum.y * inv_total);
    }
}

LSA_EXPORT int lsa_paged_attention(
    const void* q, long q_token_stride, void* out, const void* keys, const void* values, const int* table, int table_stride,
    const int* row_start, const int* row_len, const int* row_ctx, const void* items, const int* item_slot, int n_items,
    const void* merges, int n_merges, int n_slots, float* part_acc, float* part_ml, const void* tiles, const void* tile_slots, int n_tiles,
    float scale,
    int window, int page_size, int n_q, int n_kv, int gheads, int tokens_per_tile, int gtiles,
    int decode_fusion, const float* q_weight, const float* k_weight, float norm_eps, const float* cos_sin, int tiles_per_workgroup,
    int merge_in_workgroup, int tile_halves, hipStream_t stream) {
    if (n_items <= 0 && n_tiles <= 0) return 0;
    // decode_fusion (see DecodeFusion::mode): the caller promises that every row of the step brings one token.
    DecodeFusion fusion = {q_weight, k_weight, cos_sin, norm_eps, decode_fusion};
    if (decode_fusion != 0 && decode_fusion != 1 && decode_fusion != 3) return -1;
    if (decode_fusion && (!LSA_BF16 || D % 64 != 0 || n_tiles > 0 || (q_weight == nullptr) != (k_weight == nullptr))) return -1;
    Geometry g;
    g.n_q = n_q; g.n_kv = n_kv; g.group = n_q / n_kv; g.gheads = gheads; g.tokens_per_tile = tokens_per_tile;
    g.gtiles = gtiles; g.page_size = page_size; g.window = window; g.scale = scale;
    g.page_magic = (unsigned)(((1ull << 32) + page_size - 1) / page_size);
    if (n_tiles > 0) {
#if LSA_BF16
        // The plan's entries of `tiles` span what a workgroup takes: 4 or 8 tiles.  A load brings 8 keys of a value row.
        if (tiles_per_workgroup != 4 && tiles_per_workgroup != 4 * MAX_SUB) return -1;
        if (page_size % 8 != 0) return -1;
        dim3 tgrid(n_tiles * n_kv * gtiles);
        if (tile_halves != 1 && tile_halves != MAX_HALVES) return -1;
#define LSA_LAUNCH_TILES(SUB, HALVES) paged_attention_tile_kernel<SUB, HALVES><<<tgrid, 256 * HALVES, 0, stream>>>( \
                (const elem_t*)q, q_token_stride, (elem_t*)out, (const elem_t*)keys, (const elem_t*)values, table, table_stride, \
                row_start, row_len, row_ctx, (const Item*)tiles, (const TileSlots*)tile_slots, part_acc, part_ml, g)
        if (tile_slots != nullptr && (part_acc == nullptr || part_ml == nullptr || n_merges <= 0)) return -1;
        if (tiles_per_workgroup == 4 && tile_halves == 1) LSA_LAUNCH_TILES(1, 1);
        else if (tiles_per_workgroup == 4) LSA_LAUNCH_TILES(1, MAX_HALVES);
        else if (tile_halves == 1) LSA_LAUNCH_TILES(MAX_SUB, 1);
        else LSA_LAUNCH_TILES(MAX_SUB, MAX_HALVES);
#undef LSA_LAUNCH_TILES
        const int terr = (int)hipGetLastError();
        if (terr) return terr;
#else
        if (tiles_per_workgroup != 4 || tile_halves != 1 || tile_slots != nullptr) return -1;      // the float32 kernel: four tiles, keys whole
        paged_attention_tile_kernel_f32<<<dim3(n_tiles * n_kv * gtiles), 256, 0, stream>>>(
            (const elem_t*)q, q_token_stride, (elem_t*)out, (const elem_t*)keys, (const elem_t*)values, table, table_stride,
            row_start, row_len, row_ctx, (const Item*)tiles, g);
        const int terr = (int)hipGetLastError();
        if (terr) return terr;
#endif
    }
    int err = 0;
    if (n_items > 0) {
        // merge_in_workgroup (0, 2 or 4 ranges a tile): items 4 i .. 4 i + 3 are the four key ranges of one tile, or the two
        // ranges of each of two tiles (some may be empty), no item has a slot, nothing is left to merge.
        if (merge_in_workgroup && ((merge_in_workgroup != 2 && merge_in_workgroup != 4) || n_items % 4 != 0 || n_merges != 0)) return -1;
        dim3 grid((n_items + 3) / 4, n_kv * gtiles);
#define LSA_LAUNCH_ITEMS(MODE, PLAIN) LSA_LAUNCH_ITEMS_MERGE(MODE, PLAIN, 0)
#define LSA_LAUNCH_ITEMS_MERGE(MODE, PLAIN, RANGES) paged_attention_kernel<MODE, PLAIN, RANGES><<<grid, 256, 0, stream>>>( \
            (const elem_t*)q, q_token_stride, (elem_t*)out, (const elem_t*)keys, (const elem_t*)values, table, table_stride, \
            row_start, row_len, row_ctx, (const Item*)items, item_slot, n_items, part_acc, part_ml, g, fusion)
#if LSA_BF16
        const bool plain = q_weight != nullptr && cos_sin != nullptr;
        if (merge_in_workgroup && decode_fusion && !plain) return -1;      // the caller asks lsa_attention_merges_in_workgroup first
        if (merge_in_workgroup == 4 && decode_fusion == 3) LSA_LAUNCH_ITEMS_MERGE(3, true, 4);
        else if (merge_in_workgroup == 4 && decode_fusion == 1) LSA_LAUNCH_ITEMS_MERGE(1, true, 4);
        else if (merge_in_workgroup == 4) LSA_LAUNCH_ITEMS_MERGE(0, false, 4);
        else if (merge_in_workgroup == 2 && decode_fusion == 3) LSA_LAUNCH_ITEMS_MERGE(3, true, 2);
        else if (merge_in_workgroup == 2 && decode_fusion == 1) LSA_LAUNCH_ITEMS_MERGE(1, true, 2);
        else if (merge_in_workgroup == 2) LSA_LAUNCH_ITEMS_MERGE(0, false, 2);
        else if (decode_fusion == 3 && plain) LSA_LAUNCH_ITEMS(3, true);
        else if (decode_fusion == 3) LSA_LAUNCH_ITEMS(3, false);
        else if (decode_fusion == 1 && plain) LSA_LAUNCH_ITEMS(1, true);
        else if (decode_fusion == 1) LSA_LAUNCH_ITEMS(1, false);
        else
#else
        if (merge_in_workgroup == 4) LSA_LAUNCH_ITEMS_MERGE(0, false, 4);
        else if (merge_in_workgroup == 2) LSA_LAUNCH_ITEMS_MERGE(0, false, 2);
        else
#endif
        LSA_LAUNCH_ITEMS(0, false);
#undef LSA_LAUNCH_ITEMS_MERGE
#undef LSA_LAUNCH_ITEMS
        err = (int)hipGetLastError();
    }
    if (err || n_merges <= 0) return err;
    dim3 mgrid(n_merges, n_kv * gtiles, 16);
    // A wavefront for every four slots of an average merge (the slots of a step's merges differ little).
    const int wanted_waves = (n_slots / n_merges + 3) / 4;
    const int merge_waves = wanted_waves < 1 ? 1 : wanted_waves > MERGE_WAVES ? MERGE_WAVES : wanted_waves;
    merge_kernel<<<mgrid, merge_waves * 64, 0, stream>>>((elem_t*)out, row_start, row_len, (const Merge*)merges, part_acc, part_ml, g);
    LSA_LAUNCH_CHECK();
}

// Most tiles of 16 pairs that one workgroup of the prompt-portion kernel takes (it also takes 4; the float32 kernel
// takes 4 only).  The bfloat16 kernel takes pages of a multiple of 8 keys only (lsa_attention_tile_page_multiple).
LSA_EXPORT int lsa_attention_tile_page_multiple() { return LSA_BF16 ? 8 : 4; }
LSA_EXPORT int lsa_attention_workgroup_tiles() {
#if LSA_BF16
    return 4 * MAX_SUB;
#else
    return 4;
#endif
}
// Halves that a workgroup of the prompt-portion kernel can split a tile's keys between (1: it cannot).
LSA_EXPORT int lsa_attention_tile_halves() {
#if LSA_BF16
    return MAX_HALVES;
#else
    return 1;
#endif
}
// Most key ranges a tile's keys may be split into (the merge takes no more slots per tile).
LSA_EXPORT int lsa_attention_most_splits() { return MERGE_MOST_SLOTS; }
// Most key ranges that the tiles of a workgroup of the prompt-portion kernel may share with other workgroups (1: none).
LSA_EXPORT int lsa_attention_tile_key_ranges() { return LSA_BF16 ? MERGE_MOST_SLOTS : 1; }
LSA_EXPORT int lsa_attention_head_dim() { return D; }
LSA_EXPORT int lsa_attention_is_bf16() { return LSA_BF16; }
