// gfx950 kernels of the permutohedral-lattice filter.
//
// This translation unit must be compiled with -ffp-contract=off: the integer results (nearest
// lattice point, rank permutation, vertex keys) are only equal to those of the reference CPU path
// (src/PermutohedralLatticeCPU.h:220-304 of the reference tree) if every float operation of the
// embedding is a single IEEE operation, and the three double-precision steps are kept in double.
//
// Data layout in HBM
//   cell_keys[n_cells]     u64  open-addressed hash cells holding packed vertex keys (all-ones = empty)
//   cell_vertex[n_cells]   i32  dense vertex index of the key in the same cell
//   vertex_keys[M]         u64  packed key of vertex v
//   neighbours[(pd+1)*M]   int2 per blur axis a and vertex v: indices of v's two neighbours or -1
//   values[M*vd]           f32  vertex values, two buffers (ping-pong across blur axes)
//   replay[(pd+1)*T] {i32, f32} [r][t]: vertex r of the point of thread t (hash cell until the
//                                first splat) and its barycentric weight
//
// Packed key.  Every coordinate of lattice vertex with remainder r is (pd+1)*q_i + r, so a key is
// (r, q_0..q_{pd-1}): r in bits 60..63, q_i biased into a field of B = min(16, 60/pd) bits.
#include <type_traits>

#include "pl_kernels.h"
#include "pl_device.h"

namespace plk {

namespace {

using namespace device;

// A vertex's row of values, moved as one vector when its size is a power of two
template <int VD, typename S = float>
struct alignas(VD == 3 ? sizeof(S) : sizeof(S) * VD) ValueRow {
    S c[VD];
};

template <int PD>
__device__ __forceinline__ void load_position(const float *positions, int n, float (&pos)[PD]) {
    const float *row = positions + (size_t)n * PD;
#pragma unroll
    for (int i = 0; i < PD; ++i) pos[i] = row[i];
}

// The feature vector from a positions array, or built on the fly exactly as k_positions builds it
// (reference: src/PermutohedralLatticeCPU.h:464-473): IEEE float division of the grid coordinate
// and of the reference channels.
template <int PD>
__device__ __forceinline__ void load_features(const PointFeatures &f, int n, float (&pos)[PD]) {
    if (f.positions) {
        load_position<PD>(f.positions, n, pos);
        return;
    }
    int rest = n;
#pragma unroll
    for (int i = PD - 1; i >= 0; --i) {
        if (i < f.n_spatial_dims) {
            const int next = rest / f.dims.v[i];
            pos[i] = (float)(rest - next * f.dims.v[i]) / f.spatial_std;
            rest = next;
        }
    }
    if (f.n_reference_channels > 0) {
        // (every channel is asked for at once, from an element that exists, and taken or not
        // afterwards: loads behind the condition would wait for one another)
        const float *row = f.reference + (size_t)n * f.n_reference_channels;
        float channel[PD];
#pragma unroll
        for (int i = 0; i < PD; ++i) {
            const int j = i - f.n_spatial_dims;
            channel[i] = row[j >= 0 && j < f.n_reference_channels ? j : 0];
        }
#pragma unroll
        for (int i = 0; i < PD; ++i)
            if (i >= f.n_spatial_dims) pos[i] = channel[i] / f.feature_std;
    }
}

// ------------------------------------------------------------------------------------------------
// Hash table
// ------------------------------------------------------------------------------------------------

__global__ __launch_bounds__(kBlock) void k_clear_table(uint64_t *cell_keys, uint32_t n_cells) {
    const uint32_t i = blockIdx.x * kBlock + threadIdx.x;
    if (i < n_cells) cell_keys[i] = kEmptyCell;
}

// ------------------------------------------------------------------------------------------------
// Wavefront reduction used by the splat
// ------------------------------------------------------------------------------------------------
// x + (x of another lane, by DPP control), zero where the source lane does not exist or the row is
// masked out
template <int CTRL, int ROW_MASK = 0xf>
__device__ __forceinline__ float add_from_lane(float x) {
    const int other = __builtin_amdgcn_update_dpp(0, __float_as_int(x), CTRL, ROW_MASK, 0xf, true);
    return x + __int_as_float(other);
}
constexpr int kDppQuadSwap1 = 0xB1;   // quad_perm:[1,0,3,2]
constexpr int kDppQuadSwap2 = 0x4E;   // quad_perm:[2,3,0,1]
constexpr int kDppRowShr2 = 0x112, kDppRowShr4 = 0x114, kDppRowShr8 = 0x118;

// Sum over the four rows (of 16 lanes) of the wavefront, lane by lane, delivered to every row.
// v_permlane16_swap exchanges the odd rows of its first operand with the even rows of its second:
// given x twice, the first result holds x's even rows in both rows of a pair and the second x's
// odd rows, so their sum is the pair's sum in either row; v_permlane32_swap does the same with the
// halves of the wavefront.  Both are gfx950 instructions.
__device__ __forceinline__ float add_rows(float x) {
    const unsigned u = __float_as_uint(x);
    const auto pair = __builtin_amdgcn_permlane16_swap(u, u, false, false);
    const float y = __uint_as_float(pair[0]) + __uint_as_float(pair[1]);
    const unsigned w = __float_as_uint(y);
    const auto half = __builtin_amdgcn_permlane32_swap(w, w, false, false);
    return __uint_as_float(half[0]) + __uint_as_float(half[1]);
}

// Sum over the lanes with `member` set of term[0..VD) (VD <= 4), delivered channel-wise to the
// last lanes of the wavefront: lane 64-P+i (P = 2 for VD == 2, else 4) returns the sum of channel
// channel_of_lane(i).  The terms are reduce-scattered inside each quad of lanes (a lane keeps one
// channel), then summed across the quads of a row and across the four rows.  All 64 lanes must
// call it.
template <int VD>
__device__ __forceinline__ int channel_of_lane(int lane) {
    return VD == 2 ? (lane & 1) : (((lane & 1) << 1) | ((lane >> 1) & 1));
}
// Which of its terms a lane keeps and which it hands to its neighbour in the first exchange
// depends only on the lane, not on the group being summed: sorted once per point.
struct QuadTerms {
    float keep_a, keep_b, send_a, send_b;
};
template <int VD>
__device__ __forceinline__ QuadTerms quad_terms(const float (&term)[4], int lane) {
    const bool bit0 = lane & 1;
    QuadTerms q;
    if (VD == 2) {
        q.keep_a = bit0 ? term[1] : term[0];
        q.send_a = bit0 ? term[0] : term[1];
        q.keep_b = q.send_b = 0.0f;
    } else {
        q.keep_a = bit0 ? term[2] : term[0];
        q.keep_b = bit0 ? term[3] : term[1];
        q.send_a = bit0 ? term[0] : term[2];
        q.send_b = bit0 ? term[1] : term[3];
    }
    return q;
}
template <int VD>
__device__ __forceinline__ float wave_sum_to_last_lanes(bool member, const QuadTerms &q, int lane) {
    float sum;
    if (VD == 2) {
        const float keep = member ? q.keep_a : 0.0f, send = member ? q.send_a : 0.0f;
        sum = keep + __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(send),
                                                                 kDppQuadSwap1, 0xf, 0xf, true));
        sum = add_from_lane<kDppRowShr2>(sum);
    } else {
        const bool bit1 = lane & 2;
        const float keep_a = member ? q.keep_a : 0.0f, keep_b = member ? q.keep_b : 0.0f;
        const float send_a = member ? q.send_a : 0.0f, send_b = member ? q.send_b : 0.0f;
        const float ya = keep_a + __int_as_float(__builtin_amdgcn_update_dpp(
                                      0, __float_as_int(send_a), kDppQuadSwap1, 0xf, 0xf, true));
        const float yb = keep_b + __int_as_float(__builtin_amdgcn_update_dpp(
                                      0, __float_as_int(send_b), kDppQuadSwap1, 0xf, 0xf, true));
        const float keep = bit1 ? yb : ya, send = bit1 ? ya : yb;
        sum = keep + __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(send),
                                                                 kDppQuadSwap2, 0xf, 0xf, true));
    }
    sum = add_from_lane<kDppRowShr4>(sum);
    sum = add_from_lane<kDppRowShr8>(sum);
    return add_rows(sum);
}

// ------------------------------------------------------------------------------------------------
// Stage 1+2: embed, simplex, insert
// ------------------------------------------------------------------------------------------------
// SPLAT_VD != 0 (2..4): the kernel also splats.  The sums of each group of equal keys go, by one
// atomic instruction per group, to the row of the key's CELL in cell_values (the vertices are not
// numbered yet); the numbering pass moves the rows into the dense value table.  One kernel then
// does the work of two, shares the deduplication between them and never reads the replay arrays.
// Address of a hash cell as the table's base plus a 32-bit byte offset (tables stay below 2^29
// cells): one address register per cell instead of two.
__device__ __forceinline__ uint64_t *cell_at(uint64_t *cell_keys, uint32_t cell) {
    return reinterpret_cast<uint64_t *>(reinterpret_cast<char *>(cell_keys) + (cell << 3));
}

// T = double (SPLAT_VD == 0 only): positions, scale factors and the weights written are those of
// `points64`; the replay rows then carry the cells only.
// WIDE: keys of two words (Key128) in cells of two words; one cell per probe step, plain hashing.
// A cell is claimed by swapping the first word in; its second word follows with a store, and a
// lane that finds the first word of its key with the second still missing looks again.
template <int PD, int SPLAT_VD, typename T = float, bool WIDE = false>
__global__ __launch_bounds__(kBlock) void k_build(PointFeatures features, PointMap map,
                                                   ScaleFactor scale, uint64_t *cell_keys,
                                                   uint32_t mask, Counters *counters,
                                                   ReplayEntry *__restrict__ replay,
                                                   int xcd_aware, const void *__restrict__ input_any,
                                                   int in_channels, void *cell_values_any,
                                                   CreatedLists created_lists,
                                                   Points64 points64, RegionSource region_source) {
    constexpr bool kDouble = sizeof(T) == sizeof(double);
    static_assert(!kDouble || SPLAT_VD == 0, "the fused splat is for float values");
    constexpr int D1 = PD + 1;
    const float *__restrict__ input = static_cast<const float *>(input_any);
    float *cell_values = static_cast<float *>(cell_values_any);
    __shared__ int group_created, waves_done;
    if (threadIdx.x == 0) {
        group_created = 0;
        waves_done = 0;
    }
    __syncthreads();
    const unsigned vblock = xcd_contiguous_block(blockIdx.x, gridDim.x, xcd_aware);
    const size_t t = (size_t)vblock * kBlock + threadIdx.x;   // slot in the replay arrays
    const size_t n_slots = (size_t)gridDim.x * kBlock;
    const int n = point_of_thread(map, vblock, threadIdx.x);
    const int lane = threadIdx.x & 63;
    const bool valid = n >= 0;

    Simplex<PD, T> s;
    if constexpr (kDouble) {
        double pos[PD];
#pragma unroll
        for (int i = 0; i < PD; ++i) pos[i] = valid ? points64.positions[(size_t)n * PD + i] : 0.0;
        enclosing_simplex<PD>(pos, points64.scale, s);
    } else {
        float pos[PD];
#pragma unroll
        for (int i = 0; i < PD; ++i) pos[i] = 0.0f;
        if (valid) load_features<PD>(features, n, pos);
        enclosing_simplex<PD>(pos, scale, s);
    }

    // The weights are wanted after the insertion only, and the compiler would carry the residuals
    // and ranks they come from (twice as many registers) across it instead: have them now.
#pragma unroll
    for (int r = 0; r < D1; ++r) asm volatile("" : "+v"(s.weight[r]));
    const bool in_range = WIDE ? simplex_in_short_range<PD>(s) : simplex_in_key_range<PD>(s);
    if (valid && !in_range) atomicOr(&counters->flags, kFlagKeyRange);
    const bool active = valid && in_range;

    // Wavefront-level deduplication: each distinct key of the wavefront is inserted by one lane
    // (the lowest that holds it) and its cell is broadcast to the others.  Only leaders touch the
    // table.
    using Key = std::conditional_t<WIDE, Key128, uint64_t>;
    Key key[D1];
    // (leader lanes are kept five to a register, six bits each: registers decide how many
    // wavefronts a CU holds)
    unsigned leaders[(D1 + 4) / 5] = {};
    auto leader_of = [&](int r) { return (int)((leaders[r / 5] >> (6 * (r % 5))) & 63u); };
    if constexpr (WIDE)
        wide_keys_of<PD>(s, key);
    else
        vertex_keys_of<PD>(s, key);
#pragma unroll
    for (int r = 0; r < D1; ++r)
        leaders[r / 5] |= (unsigned)wave_leader_of_equal(key[r], active, lane) << (6 * (r % 5));

    // Insertion of a lane's pd+1 keys proceeds in rounds over all of them at once, so that the
    // loads and compare-and-swaps of one round are in flight together: a round loads the current
    // cell of every unresolved key, swaps the key into the cells seen empty, and steps the
    // keys that met another key to their next cell.  Cells only ever change from empty to a key,
    // so a stale load can at worst report "empty" and the compare-and-swap returns the truth.
    const KeyRegions regions = key_regions(region_source);
    if (blockIdx.x == 0 && threadIdx.x == 0) {
        counters->region_lo = regions.lo;
        counters->region_per_unit = regions.per_unit;
    }
    uint32_t cell[D1];
    unsigned open = 0;      // bit r: this lane still has to place key r
    unsigned created = 0;   // bit r: this lane's swap made the vertex of rank r
#pragma unroll
    for (int r = 0; r < D1; ++r)
        if (active && leader_of(r) == lane) open |= 1u << r;
    bool any_open = open != 0;
    if constexpr (WIDE) {
        // Rounds as below.  Words are read past the first-level cache: a second word may arrive
        // while this lane waits for it.  A lane waits at most kWideWaits rounds in all for
        // second words (the owner stores it right behind its swap), then reports a full table.
        constexpr int kWideWaits = 1 << 16;
        uint64_t *words = cell_keys;   // cell c: words 2c (first) and 2c+1 (second)
        int waits = 0;
#pragma unroll
        for (int r = 0; r < D1; ++r) cell[r] = hash_key(key[r]) & mask;
        for (uint32_t probe = 0; any_open && probe <= mask + 2u;) {
            uint64_t first[D1], second[D1];
#pragma unroll
            for (int r = 0; r < D1; ++r) {
                if ((open >> r) & 1u) {
                    first[r] = __hip_atomic_load(words + 2 * (size_t)cell[r], __ATOMIC_RELAXED,
                                                 __HIP_MEMORY_SCOPE_AGENT);
                    second[r] = __hip_atomic_load(words + 2 * (size_t)cell[r] + 1, __ATOMIC_RELAXED,
                                                  __HIP_MEMORY_SCOPE_AGENT);
                }
            }
            bool swapped[D1];
#pragma unroll
            for (int r = 0; r < D1; ++r) {
                swapped[r] = false;
                if (((open >> r) & 1u) && first[r] == kEmptyCell) {
                    first[r] = atomicCAS((unsigned long long *)(words + 2 * (size_t)cell[r]),
                                         (unsigned long long)kEmptyCell, (unsigned long long)key[r].a);
                    swapped[r] = first[r] == kEmptyCell;
                    second[r] = kEmptyCell;   // (of a cell that another lane took meanwhile: look again)
                }
            }
            bool stepped = false, waited = false;
#pragma unroll
            for (int r = 0; r < D1; ++r) {
                if (!((open >> r) & 1u)) continue;
                if (swapped[r]) {
                    __hip_atomic_store(words + 2 * (size_t)cell[r] + 1, key[r].b, __ATOMIC_RELAXED,
                                       __HIP_MEMORY_SCOPE_AGENT);
                    created |= 1u << r;
                    open &= ~(1u << r);
                } else if (first[r] == key[r].a && second[r] == key[r].b) {
                    open &= ~(1u << r);           // already there
                } else if (first[r] == key[r].a && second[r] == kEmptyCell) {
                    waited = true;                // its second word is on its way, or it is our key's
                } else {
                    cell[r] = (cell[r] + 1u) & mask;
                    stepped = true;
                }
            }
            any_open = open != 0;
            if (stepped) ++probe;
            if (waited && ++waits > kWideWaits) break;
        }
    }
    uint64_t seen[D1];
    if constexpr (!WIDE) {
#pragma unroll
    for (int r = 0; r < D1; ++r) cell[r] = cell_of_key<PD>(key[r], mask, regions);
    for (uint32_t probe = 0; any_open && probe <= mask + 2u; ++probe) {
#pragma unroll
        for (int r = 0; r < D1; ++r)
            seen[r] = (open >> r) & 1u ? *cell_at(cell_keys, cell[r]) : key[r];
#pragma unroll
        for (int r = 0; r < D1; ++r)
            if (((open >> r) & 1u) && seen[r] == kEmptyCell)
                seen[r] = atomicCAS((unsigned long long *)cell_at(cell_keys, cell[r]),
                                    (unsigned long long)kEmptyCell, (unsigned long long)key[r]);
#pragma unroll
        for (int r = 0; r < D1; ++r) {
            if ((open >> r) & 1u) {
                if (seen[r] == kEmptyCell || seen[r] == key[r]) {
                    if (seen[r] == kEmptyCell) created |= 1u << r;
                    open &= ~(1u << r);           // swapped in, or already there
                } else {
                    cell[r] = next_cell(cell[r], probe, key[r], mask, regions);
                }
            }
        }
        any_open = open != 0;
    }
    }
    if (any_open) atomicOr(&counters->flags, kFlagTableFull);

    // The vertices this workgroup created (cell and key), as a list of its own, and how many:
    // the numbering pass gives the vertices dense numbers in the order of the workgroups, that
    // is, of the image tiles.  A wavefront draws its run of list entries with one LDS atomic; the
    // wavefront that finishes last knows the workgroup's total.  No barrier: the wavefronts of a
    // workgroup leave the insertion at very different times.
    {
        int offset[D1];
        int total = 0;
#pragma unroll
        for (int r = 0; r < D1; ++r) {
            const uint64_t b = wave_ballot((created >> r) & 1u);
            offset[r] = total + (int)__builtin_amdgcn_mbcnt_hi(
                                    (uint32_t)(b >> 32), __builtin_amdgcn_mbcnt_lo((uint32_t)b, 0u));
            total += __builtin_popcountll(b);
        }
        int base = 0;
        if (lane == 0 && total) base = atomicAdd(&group_created, total);
        base = __builtin_amdgcn_readfirstlane(base);
        const size_t list = (size_t)vblock * (size_t)created_lists.stride;
#pragma unroll
        for (int r = 0; r < D1; ++r) {
            if ((created >> r) & 1u) {
                if constexpr (WIDE) {
                    // (two entries per vertex: the key, then the cell)
                    uint4 *entry = created_lists.entries + list + 2 * (size_t)(base + offset[r]);
                    entry[0] = make_uint4((uint32_t)key[r].a, (uint32_t)(key[r].a >> 32),
                                          (uint32_t)key[r].b, (uint32_t)(key[r].b >> 32));
                    entry[1] = make_uint4(cell[r], 0u, 0u, 0u);
                } else {
                    created_lists.entries[list + base + offset[r]] =
                        make_uint4((uint32_t)key[r], (uint32_t)(key[r] >> 32), cell[r], 0u);
                }
            }
        }
        if (lane == 0 && atomicAdd(&waves_done, 1) == kBlock / 64 - 1) {
            const int sum = atomicAdd(&group_created, 0);
            created_lists.block_count[vblock] = sum;
            if (sum) atomicAdd(&created_lists.chunk_count[vblock / kBlocksPerChunk], sum);
        }
    }

    float val[4] = {0.0f, 0.0f, 0.0f, 0.0f};
    if (SPLAT_VD) {
#pragma unroll
        for (int j = 0; j < SPLAT_VD; ++j) val[j] = 1.0f;  // homogeneous channel when vd-1 are given
        if (valid) {
#pragma unroll
            for (int j = 0; j < SPLAT_VD; ++j)
                if (j < in_channels) val[j] = input[(size_t)n * in_channels + j];
        }
    }

#pragma unroll
    for (int r = 0; r < D1; ++r) {
        const int own = (open >> r) & 1u ? -1 : (int)cell[r];
        const int leader = leader_of(r);
        const int c = __shfl(own, leader);
        replay[(size_t)r * n_slots + t] = ReplayEntry{active ? c : -1, valid ? (float)s.weight[r] : 0.0f};
        if constexpr (kDouble) points64.weights[(size_t)r * n_slots + t] = valid ? s.weight[r] : 0.0;
        if (SPLAT_VD) {
            constexpr int VD = SPLAT_VD ? SPLAT_VD : 2;
            constexpr int P = VD == 2 ? 2 : 4;
            const float w = (float)s.weight[r];
            const float term[4] = {w * val[0], w * val[1], w * val[2], w * val[3]};
            const QuadTerms quad = quad_terms<VD>(term, lane);
            const uint64_t among = wave_ballot(active);
            uint64_t remaining = among;
            while (remaining) {
                const int first = __builtin_ctzll(remaining);
                const uint64_t group = lanes_equal(leader, first) & among;
                remaining &= ~group;
                const bool same = lane_in(group);
                const int group_cell = lane_value(own, first);
                const float sum = wave_sum_to_last_lanes<VD>(same, quad, lane);
                if (group_cell >= 0 && lane >= 64 - P && channel_of_lane<VD>(lane) < VD)
                    atomicAdd(cell_values + (size_t)group_cell * VD + channel_of_lane<VD>(lane), sum);
            }
        }
    }
}

// The same stage with the keys and sums of a whole workgroup merged in LDS before they go to the
// table: for an image tile of 16x16 pixels the four wavefronts hold about 165 (wavefront, vertex)
// pairs but only about 100 distinct vertices, and what limits the build is the number of requests
// to the L2 atomic unit (one per compare-and-swap, one per row of sums).  Each wavefront elects
// its leaders and sums its groups as above, but the leaders place their keys in a small hash table
// in LDS and the sums are added to the rows of the LDS slots; then every occupied slot is placed
// in the table in HBM by one thread, and its row goes out with one request.  A workgroup whose
// distinct keys do not fit the LDS table raises kFlagTileFull and the host repeats the build with
// k_build (and uses it for a while).  Three barriers; every thread reaches each of them.
static_assert(kTileSlots == 2 * kBlock, "a thread places at most two slots in the table");
constexpr int kTileProbeLimit = 48;

template <int PD, int SPLAT_VD, typename T = float>
__global__ __launch_bounds__(kBlock) void k_build_tile(PointFeatures features, PointMap map,
                                                        ScaleFactor scale, uint64_t *cell_keys,
                                                        uint32_t mask, Counters *counters,
                                                        ReplayEntry *__restrict__ replay,
                                                        int xcd_aware, const void *__restrict__ input_any,
                                                        int in_channels, void *cell_values_any,
                                                        CreatedLists created_lists,
                                                        Points64 points64, RegionSource region_source,
                                                        InBuildNumbering numbering) {
    constexpr bool kDouble = sizeof(T) == sizeof(double);
    constexpr int D1 = PD + 1;
    constexpr int VD = SPLAT_VD ? SPLAT_VD : 2;
    constexpr int P = (VD == 2 && !kDouble) ? 2 : 4;      // values per LDS row of sums
    const T *__restrict__ input = static_cast<const T *>(input_any);
    unsigned vblock;
    if (!block_of_points(map, xcd_aware, vblock)) {
        // (no points: nothing created, no rows of sums for the passes that walk the lists)
        if (threadIdx.x == 0) created_lists.block_count[vblock] = 0;
        return;
    }
    __shared__ uint64_t slot_key[kTileSlots];
    __shared__ int slot_cell[kTileSlots];
    __shared__ T slot_sum[SPLAT_VD ? kTileSlots * P : 1];
    // the slots in use, in the order their keys arrived: the last phases walk these, not all slots
    __shared__ unsigned short occupied[kTileSlots];
    __shared__ int n_occupied;
    // which of the vertices this workgroup created a slot's key is (kNotCreated: none of them)
    __shared__ unsigned short slot_rank[kTileSlots];
    constexpr unsigned short kNotCreated = 0xffffu;
    __shared__ int group_created;
    const int tid = threadIdx.x;
    for (int i = tid; i < kTileSlots; i += kBlock) slot_key[i] = kEmptyCell;
    if (SPLAT_VD)
        for (int i = tid; i < kTileSlots * P; i += kBlock) slot_sum[i] = (T)0;
    if (tid == 0) {
        n_occupied = 0;
        group_created = 0;
    }

    const size_t t = (size_t)vblock * kBlock + tid;   // slot in the replay arrays
    const size_t n_slots = (size_t)gridDim.x * kBlock;
    const int n = point_of_thread(map, vblock, tid);
    const int lane = tid & 63;
    const bool valid = n >= 0;

    Simplex<PD, T> s;
    if constexpr (kDouble) {
        double pos[PD];
#pragma unroll
        for (int i = 0; i < PD; ++i) pos[i] = valid ? points64.positions[(size_t)n * PD + i] : 0.0;
        enclosing_simplex<PD>(pos, points64.scale, s);
    } else {
        float pos[PD];
#pragma unroll
        for (int i = 0; i < PD; ++i) pos[i] = 0.0f;
        if (valid) load_features<PD>(features, n, pos);
        enclosing_simplex<PD>(pos, scale, s);
    }
#pragma unroll
    for (int r = 0; r < D1; ++r) asm volatile("" : "+v"(s.weight[r]));
    const bool in_range = simplex_in_key_range<PD>(s);
    if (valid && !in_range) atomicOr(&counters->flags, kFlagKeyRange);
    const bool active = valid && in_range;

    unsigned leaders[(D1 + 4) / 5] = {};
    auto leader_of = [&](int r) { return (int)((leaders[r / 5] >> (6 * (r % 5))) & 63u); };
    int slot[D1];           // the LDS slot of key r, at first in the lanes of the leaders only
    // Groups of a few lanes add their terms to the slot's row one by one; the tree that sums a
    // group costs the same for two lanes as for sixty-four, and half the groups have four or fewer.
    constexpr int kSmallGroup = SPLAT_VD ? 4 : 0;
    uint64_t small[D1];
    __syncthreads();        // the LDS table is empty
    {
        uint64_t key[D1];
        unsigned open = 0;
        vertex_keys_of<PD>(s, key);
#pragma unroll
        for (int r = 0; r < D1; ++r) {
            const int leader = wave_leader_of_equal(key[r], active, lane, kSmallGroup, small[r]);
            leaders[r / 5] |= (unsigned)leader << (6 * (r % 5));
            if (active && leader == lane) open |= 1u << r;
            static_assert(kTileSlots == 1 << (32 - kTileSlotShift), "the slot is the hash's high bits");
            slot[r] = (int)(hash_key(key[r]) >> kTileSlotShift);
        }
        bool any_open = open != 0;
        for (int probe = 0; any_open && probe < kTileProbeLimit; ++probe) {
#pragma unroll
            for (int r = 0; r < D1; ++r) {
                if ((open >> r) & 1u) {
                    const uint64_t seen =
                        atomicCAS((unsigned long long *)&slot_key[slot[r]],
                                  (unsigned long long)kEmptyCell, (unsigned long long)key[r]);
                    if (seen == kEmptyCell || seen == key[r]) {
                        open &= ~(1u << r);
                        // the slot was empty: it joins the list of slots in use
                        if (seen == kEmptyCell)
                            occupied[atomicAdd(&n_occupied, 1)] = (unsigned short)slot[r];
                    } else {
                        slot[r] = (slot[r] + 1) & (kTileSlots - 1);
                    }
                }
            }
            any_open = open != 0;
        }
        if (any_open) atomicOr(&counters->flags, kFlagTileFull);
#pragma unroll
        for (int r = 0; r < D1; ++r)
            if ((open >> r) & 1u) slot[r] = -1;
    }

    T val[4] = {(T)0, (T)0, (T)0, (T)0};
    if (SPLAT_VD) {
#pragma unroll
        for (int j = 0; j < SPLAT_VD; ++j) val[j] = (T)1;  // homogeneous channel when vd-1 are given
        if (valid) {
#pragma unroll
            for (int j = 0; j < SPLAT_VD; ++j)
                if (j < in_channels) val[j] = input[(size_t)n * in_channels + j];
        }
    }
#pragma unroll
    for (int r = 0; r < D1; ++r) {
        const int leader = leader_of(r);
        const int own = slot[r];
        slot[r] = active ? __shfl(own, leader) : -1;
        if (SPLAT_VD) {
            const T w = s.weight[r];
            const T term[4] = {w * val[0], w * val[1], w * val[2], w * val[3]};
            const uint64_t among = wave_ballot(active) & ~small[r];
            uint64_t remaining = among;
            if constexpr (kDouble) {
                while (remaining) {
                    const int first = __builtin_ctzll(remaining);
                    const uint64_t group = lanes_equal(leader, first) & among;
                    remaining &= ~group;
                    const int group_slot = lane_value(own, first);
                    const double sum = wave_sums_to_quads_f64(lane_in(group), term, lane);
                    if (group_slot >= 0 && lane < 4 && channel_of_quad_lane(lane) < VD)
                        atomicAdd(&slot_sum[group_slot * P + channel_of_quad_lane(lane)], sum);
                }
            } else {
                const QuadTerms quad = quad_terms<VD>(term, lane);
                // (one group per turn: two side by side, to overlap their chains of cross-lane
                // additions, cost more for the odd group out than they gain)
                while (remaining) {
                    const int first = __builtin_ctzll(remaining);
                    const uint64_t group = lanes_equal(leader, first) & among;
                    remaining &= ~group;
                    const bool same = lane_in(group);
                    const int group_slot = lane_value(own, first);
                    const float sum = wave_sum_to_last_lanes<VD>(same, quad, lane);
                    if (group_slot >= 0 && lane >= 64 - P && channel_of_lane<VD>(lane) < VD)
                        atomicAdd(&slot_sum[group_slot * P + channel_of_lane<VD>(lane)], sum);
                }
            }
            if (lane_in(small[r]) && slot[r] >= 0) {
#pragma unroll
                for (int j = 0; j < VD; ++j) atomicAdd(&slot_sum[slot[r] * P + j], term[j]);
            }
        }
    }
    __syncthreads();        // the keys and sums of all four wavefronts are in the LDS table

    // Every slot in use goes to the table in HBM: thread i takes the i-th of them (and the
    // (i + kBlock)-th when a tile has that many, in rounds over both as in k_build).  A tile of an
    // image has about a hundred, so two of the four wavefronts have nothing to do here.
    const KeyRegions regions = key_regions(region_source);
    if (blockIdx.x == 0 && tid == 0) {
        counters->region_lo = regions.lo;
        counters->region_per_unit = regions.per_unit;
    }
    const int n_in_use = n_occupied;
    // numbering.n_segments != 0: the workgroups number their vertices themselves; else they list
    // them for the numbering pass and add all their sums to the rows of the hash cells
    const bool numbers_here = numbering.n_segments != 0;
    auto place_in_table = [&](auto slots_per_thread) {
        constexpr int H = decltype(slots_per_thread)::value;
        // A round looks at the pair of cells a key has come to (one 16-byte load), takes the key's
        // cell if it is there, else swaps the key into the pair's first empty cell, else moves on
        // to the next pair.  A swap lost to another key looks at the same pair again: each turn
        // either moves on or sees a cell of the pair filled for good.
        uint64_t key[H];
        uint32_t cell[H], pair_index[H];
        ulonglong2 seen[H];
        unsigned open = 0, created = 0;
        int in_slot[H];
#pragma unroll
        for (int h = 0; h < H; ++h) {
            const bool has = tid + h * kBlock < n_in_use;
            in_slot[h] = has ? (int)occupied[tid + h * kBlock] : 0;
            key[h] = has ? slot_key[in_slot[h]] : kEmptyCell;
            if (has) open |= 1u << h;
            cell[h] = cell_of_key<PD>(key[h], mask, regions);
            pair_index[h] = 0;
        }
        bool any_open = open != 0;
        for (uint32_t turn = 0; any_open && turn <= 2u * mask + 8u; ++turn) {
#pragma unroll
            for (int h = 0; h < H; ++h)
                if ((open >> h) & 1u)
                    seen[h] = *reinterpret_cast<const ulonglong2 *>(cell_at(cell_keys, cell[h]));
            int target[H];
#pragma unroll
            for (int h = 0; h < H; ++h) {
                target[h] = -1;
                if ((open >> h) & 1u) {
                    if (seen[h].x == key[h]) {
                        open &= ~(1u << h);
                    } else if (seen[h].x == kEmptyCell) {
                        target[h] = 0;
                    } else if (seen[h].y == key[h]) {
                        cell[h] += 1u;
                        open &= ~(1u << h);
                    } else if (seen[h].y == kEmptyCell) {
                        target[h] = 1;
                    } else {
                        cell[h] = next_pair(cell[h], pair_index[h], key[h], mask, regions);
                        pair_index[h] += 1u;
                    }
                }
            }
            uint64_t found[H];
#pragma unroll
            for (int h = 0; h < H; ++h)
                if (target[h] >= 0)
                    found[h] = atomicCAS(
                        (unsigned long long *)cell_at(cell_keys, cell[h] + (uint32_t)target[h]),
                        (unsigned long long)kEmptyCell, (unsigned long long)key[h]);
#pragma unroll
            for (int h = 0; h < H; ++h) {
                if (target[h] >= 0 && (found[h] == kEmptyCell || found[h] == key[h])) {
                    if (found[h] == kEmptyCell) created |= 1u << h;
                    cell[h] += (uint32_t)target[h];
                    open &= ~(1u << h);
                }
            }
            any_open = open != 0;
        }
        if (any_open) atomicOr(&counters->flags, kFlagTableFull);
#pragma unroll
        for (int h = 0; h < H; ++h)
            if (tid + h * kBlock < n_in_use)
                slot_cell[in_slot[h]] = (open >> h) & 1u ? -1 : (int)cell[h];

        // the vertices this workgroup created, as in k_build
        int offset[H];
        int total = 0;
#pragma unroll
        for (int h = 0; h < H; ++h) {
            const uint64_t b = wave_ballot((created >> h) & 1u);
            offset[h] = total + (int)__builtin_amdgcn_mbcnt_hi(
                                    (uint32_t)(b >> 32), __builtin_amdgcn_mbcnt_lo((uint32_t)b, 0u));
            total += __builtin_popcountll(b);
        }
        int base = 0;
        if (lane == 0 && total) base = atomicAdd(&group_created, total);
        base = __builtin_amdgcn_readfirstlane(base);
#pragma unroll
        for (int h = 0; h < H; ++h)
            if (tid + h * kBlock < n_in_use)
                slot_rank[in_slot[h]] =
                    (created >> h) & 1u ? (unsigned short)(base + offset[h]) : kNotCreated;
        if (!numbers_here) {
            // (for the numbering pass: what this workgroup created, as in k_build)
            const size_t list = (size_t)vblock * (size_t)created_lists.stride;
#pragma unroll
            for (int h = 0; h < H; ++h) {
                if ((created >> h) & 1u) {
                    created_lists.entries[list + base + offset[h]] =
                        make_uint4((uint32_t)key[h], (uint32_t)(key[h] >> 32), cell[h], 0u);
                }
            }
        }
    };
    if ((tid & ~63) < n_in_use) {
        if (n_in_use <= kBlock)
            place_in_table(std::integral_constant<int, 1>{});
        else
            place_in_table(std::integral_constant<int, kTileSlots / kBlock>{});
    }
    __syncthreads();        // every slot's cell is known

    if (!numbers_here) {
        // The numbering pass follows: it needs the length of the workgroup's list, and moves the
        // rows of sums from the hash cells to the vertices.
        if (tid == 0) {
            const int sum = group_created;
            created_lists.block_count[vblock] = sum;
            if (sum) atomicAdd(&created_lists.chunk_count[vblock / kBlocksPerChunk], sum);
        }
        if (SPLAT_VD) {
            // rows of sums: P consecutive lanes per slot in use, one request per row
            T *cell_values = static_cast<T *>(cell_values_any);
            const int channel = tid % P;
            for (int i = tid / P; i < n_in_use; i += kBlock / P) {
                const int sl = (int)occupied[i];
                const int cell = slot_cell[sl];
                if (cell >= 0 && channel < VD)
                    atomicAdd(cell_values + (size_t)cell * VD + channel, slot_sum[sl * P + channel]);
            }
        }
#pragma unroll
        for (int r = 0; r < D1; ++r) {
            const int c = slot[r] >= 0 ? slot_cell[slot[r]] : -1;
            replay[(size_t)r * n_slots + t] = ReplayEntry{c, valid ? (float)s.weight[r] : 0.0f};
            if constexpr (kDouble) points64.weights[(size_t)r * n_slots + t] = valid ? s.weight[r] : 0.0;
        }
        return;
    }

    // Numbers for the vertices this workgroup created: a run of its segment's, drawn with one
    // atomic (the segment is the eighth of the image the workgroup lies in, which is the XCD it
    // runs on when the workgroups are dealt out that way; a small table has one segment).  The
    // atomic takes a microsecond or more to come back -- a segment's workgroups all add to one
    // address -- so only the first wavefront waits for it: the others end behind their replay rows
    // and leave their places to the wavefronts of the next workgroup.
    const unsigned stride = segment_stride((uint32_t)numbering.max_vertices, numbering.n_segments);
    unsigned segment = 0;
    if (numbering.n_segments >= (int)kXcds) {
        // the eighth of the image this workgroup lies in and, with sixty-four segments, which
        // eighth of that (vblock runs through an XCD's share of the workgroups in order)
        const unsigned parts = (unsigned)numbering.n_segments / kXcds;
        if (xcd_aware) {
            const unsigned nb = map.mode == 1 && *map.n_tiles < gridDim.x ? *map.n_tiles : gridDim.x;
            const unsigned xcd = blockIdx.x % kXcds;
            const unsigned share = nb / kXcds + (xcd < nb % kXcds ? 1u : 0u);
            const unsigned index = blockIdx.x / kXcds;
            segment = xcd * parts + (share ? (unsigned)(((size_t)index * parts) / share) : 0u);
        } else {
            segment = (unsigned)(((size_t)vblock * (size_t)numbering.n_segments) / gridDim.x);
        }
    }
    const unsigned count = (unsigned)group_created;
    unsigned first = 0;
    if (tid == 0 && count) first = atomicAdd(&counters->segment_count[segment].n, count);
#pragma unroll
    for (int r = 0; r < D1; ++r) {
        const int c = slot[r] >= 0 ? slot_cell[slot[r]] : -1;
        replay[(size_t)r * n_slots + t] = ReplayEntry{c, valid ? (float)s.weight[r] : 0.0f};
        if constexpr (kDouble) points64.weights[(size_t)r * n_slots + t] = valid ? s.weight[r] : 0.0;
    }
    if (blockIdx.x == 0 && tid < kMaxSegments) {
        counters->n_segments = numbering.n_segments;
        counters->segment_count[tid].n_segments = numbering.n_segments;
    }
    if (tid >= 64) return;

    // Per slot in use: a vertex this workgroup created gets its number, its entries in the
    // per-vertex tables and its row of the value table (the tile's sums, or zeros when the build
    // does not splat; other workgroups' sums for it are added by neighbours()); the sums for a
    // vertex that another workgroup created go to this workgroup's list.
    first = (unsigned)__builtin_amdgcn_readfirstlane((int)first);
    // (a run that leaves the segment: the host repeats the build with a larger table; what is
    // enqueued behind this build walks the segment's numbers, so those still get vertices)
    if (lane == 0 && first + count > stride) atomicOr(&counters->flags, kFlagTableFull);
    T *values = static_cast<T *>(numbering.values);
    const int numbers_from = (int)(segment * stride);
    uint4 *part = created_lists.entries + (size_t)vblock * (size_t)created_lists.stride;
    T *foreign_rows = reinterpret_cast<T *>(part);
    int *foreign_cells = reinterpret_cast<int *>(part + kTileSlots * (kDouble ? 2 : 1));
    int n_foreign = 0;
    for (int i0 = 0; i0 < n_in_use; i0 += 64) {
        const int i = i0 + lane;
        const bool has = i < n_in_use;
        const int sl = has ? (int)occupied[i] : 0;
        const int cell = has ? slot_cell[sl] : -1;
        const unsigned short rank = slot_rank[sl];
        const bool mine = cell >= 0 && rank != kNotCreated;
        const bool foreign = SPLAT_VD != 0 && cell >= 0 && rank == kNotCreated;
        T row[4] = {(T)0, (T)0, (T)0, (T)0};
        if (SPLAT_VD) {
#pragma unroll
            for (int j = 0; j < P; ++j) row[j] = slot_sum[sl * P + j];
        }
        if (mine) {
            // (a number beyond the segment is not given out: what runs until the host repeats
            // the build must find a valid one)
            const bool fits = first + rank < stride;
            const int v = fits ? numbers_from + (int)(first + rank) : 0;
            numbering.cell_vertex[cell] = v;
            if (fits) {
                numbering.vertex_keys[v] = slot_key[sl];
                numbering.vertex_cell[v] = cell;
#pragma unroll
                for (int a = 0; a < D1; ++a)
                    numbering.neighbours[(size_t)a * numbering.max_vertices + v] = make_int2(-1, -1);
                if (SPLAT_VD) {
                    if constexpr (VD == 4 || (VD == 2 && !kDouble)) {
                        reinterpret_cast<ValueRow<VD, T> *>(values)[v] =
                            *reinterpret_cast<const ValueRow<VD, T> *>(row);
                    } else {
#pragma unroll
                        for (int j = 0; j < VD; ++j) values[(size_t)v * VD + j] = row[j];
                    }
                } else {
                    float *words = static_cast<float *>(numbering.values);
                    for (int j = 0; j < numbering.value_words; ++j)
                        words[(size_t)v * numbering.value_words + j] = 0.0f;
                }
            }
        }
        if (SPLAT_VD) {
            const uint64_t b = wave_ballot(foreign);
            const int offset = n_foreign + (int)__builtin_amdgcn_mbcnt_hi(
                                               (uint32_t)(b >> 32), __builtin_amdgcn_mbcnt_lo((uint32_t)b, 0u));
            n_foreign += (int)__builtin_popcountll(b);
            if (foreign) {
                foreign_cells[offset] = cell;
#pragma unroll
                for (int j = 0; j < 4; ++j) foreign_rows[(size_t)offset * 4 + j] = row[j];
            }
        }
    }
    if (lane == 0) {
        created_lists.block_count[vblock] = n_foreign;
        // (how many such rows there are in all tells the host whether numbering here pays)
        if ((blockIdx.x / kXcds) % kForeignSampling == 0 && n_foreign)
            atomicAdd(&counters->foreign_rows_sampled.n, (unsigned)n_foreign);
    }
}

// Dense vertex numbering in the order of the build's workgroups, i.e. of the image tiles: the
// vertices a workgroup created follow those of the workgroups before it.  Vertices that are close
// in the lattice were created by the same or a neighbouring tile, so their numbers are close, and
// what the neighbour, blur and slice passes gather falls into few cache lines instead of one line
// per access.  One wavefront per workgroup of the build walks that workgroup's list.  Per vertex
// v: cell_vertex[cell] := v, vertex_keys[v], vertex_cell[v], the row of the value table (moved
// from cell_values, which the fused build+splat filled, or zeroed), and (-1, -1) for all its
// neighbour entries.  The last wavefront knows the total: it publishes it to the device counters
// and to host-visible memory and clears what the next build will count in.
// WIDE: the build had keys of two words: two entries per vertex (key, then cell), and
// vertex_keys holds two words per vertex.
template <int D1, bool WIDE = false>
__global__ __launch_bounds__(64) void k_number_vertices(CreatedLists lists, int *next_chunk_count,
                                                        unsigned n_chunks,
                                                        VertexTables vertices, float *values, int vd,
                                                        float *cell_values, Counters *counters,
                                                        Counters *next_counters,
                                                        HostReport host_report) {
    HostStatus *host_status = host_report.status;
    // (an XCD takes the lists of one contiguous range of tiles: their cells are in its part of the
    // table and their vertex numbers in one range)
    const unsigned b = xcd_contiguous_block(blockIdx.x, gridDim.x, 1);
    const int lane = threadIdx.x;
    const unsigned chunk = b / kBlocksPerChunk;
    const size_t list = (size_t)b * (size_t)lists.stride;
    // Everything the pass reads that does not depend on something else it reads is asked for at
    // once, without branches (an index out of range reads element 0 and is dropped afterwards):
    // the sums of the chunks before this workgroup's, the counts of the workgroups before it in
    // its chunk, its own count, and the first 64 entries of its list whether it has that many or
    // not (the list's memory is there).  With a load behind each condition the pass waited for
    // five memory round trips in a row; now for two, the entries and then their rows of sums.
    static_assert(kBlocksPerChunk == 64, "one lane per workgroup of the chunk");
    // (the sums of up to 512 chunks -- a volume of eight million voxels has that many -- in eight
    // loads per lane that are all in flight together)
    constexpr int kChunkLoads = 8;
    int part[kChunkLoads];
#pragma unroll
    for (int u = 0; u < kChunkLoads; ++u) {
        const unsigned i = (unsigned)lane + 64u * (unsigned)u;
        part[u] = lists.chunk_count[i < chunk ? i : 0];
    }
    const unsigned sibling = chunk * kBlocksPerChunk + lane;
    int sibling_count = lists.block_count[sibling < b ? sibling : b];
    const int count = lists.block_count[b];
    uint4 first_entry = lists.entries[list + (WIDE ? 2 * lane + 1 : lane)];
    asm volatile("" : "+v"(sibling_count), "+v"(first_entry.x), "+v"(first_entry.y), "+v"(first_entry.z));
#pragma unroll
    for (int u = 0; u < kChunkLoads; ++u) asm volatile("" : "+v"(part[u]));
    int before = 0;
#pragma unroll
    for (int u = 0; u < kChunkLoads; ++u)
        before += (unsigned)lane + 64u * (unsigned)u < chunk ? part[u] : 0;
    for (unsigned i = lane + 64 * kChunkLoads; i < chunk; i += 64) before += lists.chunk_count[i];
    before += sibling < b ? sibling_count : 0;
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) before += __shfl_xor(before, off);
    const int max_vertices = vertices.max_vertices;

    if (b == gridDim.x - 1) {
        if (lane == 0) {
            const uint32_t m = (uint32_t)(before + count);
            counters->vertices = m;
            counters->n_segments = 0;
            for (int k = 0; k < kMaxSegments; ++k) {
                counters->segment_count[k].n = m;
                counters->segment_count[k].n_segments = 0;
            }
            host_status->num_vertices = (int)m;
            host_status->flags = counters->flags | (m > (uint32_t)max_vertices ? kFlagTableFull : 0);
            host_status->max_segment = (int)m;
            host_status->n_segments = 0;
            host_status->foreign_rows = 0;
            __threadfence_system();
            __hip_atomic_store(&host_status->sequence, host_report.sequence, __ATOMIC_RELAXED,
                               __HIP_MEMORY_SCOPE_SYSTEM);
            reset_counters(next_counters);
        }
        for (unsigned i = lane; i < n_chunks; i += 64) next_chunk_count[i] = 0;
    }

    for (int i = lane; i < count; i += 64) {
        const uint4 entry =
            i < 64 ? first_entry : lists.entries[list + (WIDE ? 2 * (size_t)i + 1 : (size_t)i)];
        const int cell = WIDE ? (int)entry.x : (int)entry.z;
        const int v = before + i;
        if (v < max_vertices) {
            vertices.cell_vertex[cell] = v;
            if constexpr (WIDE)
                reinterpret_cast<uint4 *>(vertices.vertex_keys)[v] = lists.entries[list + 2 * (size_t)i];
            else
                vertices.vertex_keys[v] = ((uint64_t)entry.y << 32) | entry.x;
            vertices.vertex_cell[v] = cell;
            if (cell_values && vd == 4) {
                float4 *from = reinterpret_cast<float4 *>(cell_values) + cell;
                reinterpret_cast<float4 *>(values)[v] = *from;
                *from = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
            } else if (cell_values && vd == 8) {
                float4 *from = reinterpret_cast<float4 *>(cell_values) + 2 * (size_t)cell;
                float4 *to = reinterpret_cast<float4 *>(values) + 2 * (size_t)v;
                to[0] = from[0];
                to[1] = from[1];
                from[0] = from[1] = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
            } else if (cell_values && vd == 2) {
                float2 *from = reinterpret_cast<float2 *>(cell_values) + cell;
                reinterpret_cast<float2 *>(values)[v] = *from;
                *from = make_float2(0.0f, 0.0f);
            } else if (cell_values) {
                for (int j = 0; j < vd; ++j) {
                    values[(size_t)v * vd + j] = cell_values[(size_t)cell * vd + j];
                    cell_values[(size_t)cell * vd + j] = 0.0f;
                }
            } else {
                for (int j = 0; j < vd; ++j) values[(size_t)v * vd + j] = 0.0f;
            }
            // "no neighbour" everywhere; the neighbour pass fills in the ones that exist
            for (int a = 0; a < D1; ++a)
                vertices.neighbours[(size_t)a * max_vertices + v] = make_int2(-1, -1);
        } else {
            vertices.cell_vertex[cell] = 0;   // the host sees the count and repeats with a larger table
        }
    }
}

// ------------------------------------------------------------------------------------------------
// Neighbour table: along axis a the neighbours of key k are k + (1,..,1) - (pd+1) e_a and its
// mirror image (reference: src/PermutohedralLatticeCPU.h:381-388).  In (r, q) form the first is
// r+1 with q_a-1, or, when r = pd, r = 0 with every q but q_a one higher; axis pd is the implicit
// last coordinate, which no stored q belongs to.  out[a*max_vertices + v].
// A workgroup takes 256 consecutive vertices along one axis; the pd+1 workgroups of a run of
// vertices follow each other.  u is the + neighbour of v exactly when v is the - neighbour of u:
// one lookup fills out[a][v].x and out[a][u].y (all entries start as -1).
// ------------------------------------------------------------------------------------------------
// After a merging build that numbered its vertices and splatted, the launch also adds the rows of
// sums that the build's workgroups hold for vertices other workgroups created (ForeignRows) to the
// value table, now that every vertex has its number: its first foreign_blocks workgroups (a
// multiple of 8, or 0) take four workgroups' lists each, one per wavefront, a row per group of
// four lanes.  S: the value type.
template <typename S>
__device__ __forceinline__ void add_foreign_rows(const CreatedLists &lists, unsigned n_lists,
                                                 unsigned group, int vd,
                                                 const int *__restrict__ cell_vertex, S *values) {
    const unsigned list = group * (kBlock / 64) + (threadIdx.x >> 6);
    if (list >= n_lists) return;
    const int lane = threadIdx.x & 63;
    const int n = lists.block_count[list];
    const uint4 *part = lists.entries + (size_t)list * (size_t)lists.stride;
    const S *rows = reinterpret_cast<const S *>(part);
    const int *cells = reinterpret_cast<const int *>(part + kTileSlots * (sizeof(S) / sizeof(float)));
    const int channel = lane & 3;
    // (what bounds this is the atomic unit, a request per row: asking for all rows of the four
    // lists at once instead of sixteen rows at a time per list made it slower)
    for (int e = lane >> 2; e < n; e += 16) {
        const int v = cell_vertex[cells[e]];
        if (channel < vd) atomicAdd(values + (size_t)v * vd + channel, rows[(size_t)e * 4 + channel]);
    }
}

// WIDE: keys and cells of two words (see k_build), one cell per probe step, plain hashing.
template <int PD, bool WIDE = false>
__global__ __launch_bounds__(kBlock) void k_neighbours(VertexTables vertices,
                                                        const Counters *counters,
                                                        const uint64_t *__restrict__ cell_keys,
                                                        uint32_t mask, unsigned foreign_blocks,
                                                        CreatedLists lists, unsigned n_lists,
                                                        void *values, int vd, int values_are_double,
                                                        Counters *report, Counters *next_counters,
                                                        HostReport host_report) {
    constexpr int D1 = PD + 1;
    HostStatus *host_status = host_report.status;
    // After a merging build nothing has told the host yet how the build went: the segments' counts
    // are summed here, and what the next build will count in is cleared.
    // (by the first wavefront of the first workgroup that looks up neighbours, which starts with
    // the launch: a lane per segment)
    if (report && blockIdx.x == foreign_blocks && threadIdx.x < 64) {
        static_assert(kMaxSegments <= 64, "a lane per segment");
        const int n_segments = report->n_segments;
        const unsigned c = (int)threadIdx.x < n_segments ? report->segment_count[threadIdx.x].n : 0u;
        unsigned total = c, fullest = c;
#pragma unroll
        for (int off = 32; off >= 1; off >>= 1) {
            total += __shfl_xor(total, off);
            const unsigned other = __shfl_xor(fullest, off);
            fullest = other > fullest ? other : fullest;
        }
        if (threadIdx.x == 0) {
            report->vertices = total;
            host_status->num_vertices = (int)total;
            host_status->flags = report->flags;
            host_status->max_segment = (int)fullest;
            host_status->n_segments = n_segments;
            host_status->foreign_rows = (int)(report->foreign_rows_sampled.n * kForeignSampling);
            __threadfence_system();
            __hip_atomic_store(&host_status->sequence, host_report.sequence, __ATOMIC_RELAXED,
                               __HIP_MEMORY_SCOPE_SYSTEM);
            reset_counters(next_counters);
        }
    }
    if (blockIdx.x < foreign_blocks) {
        const unsigned group = xcd_contiguous_block(blockIdx.x, foreign_blocks, 1);
        if (values_are_double)
            add_foreign_rows(lists, n_lists, group, vd, vertices.cell_vertex, static_cast<double *>(values));
        else
            add_foreign_rows(lists, n_lists, group, vd, vertices.cell_vertex, static_cast<float *>(values));
        return;
    }
    const KeyRegions regions{counters->region_lo, counters->region_per_unit};
    const int max_vertices = vertices.max_vertices;
    SegmentWalk walk(counters, max_vertices, blockIdx.x - foreign_blocks, gridDim.x - foreign_blocks);
    unsigned ib;
    while (walk.next(1u, D1, ib)) {
    const int a = (int)(ib % D1);
    const unsigned i = (ib / D1) * kBlock + threadIdx.x;
    if (i >= walk.count) continue;
    const int v = (int)(walk.first + i);

    int q[PD], r;
    if constexpr (WIDE) {
        const ulonglong2 k = reinterpret_cast<const ulonglong2 *>(vertices.vertex_keys)[v];
        WideCodec<PD>::unpack(Key128{k.x, k.y}, q, r);
    } else {
        KeyCodec<PD>::unpack(vertices.vertex_keys[v], q, r);
    }
    int qp[PD];
    const bool wrap_up = (r == PD);
#pragma unroll
    for (int i = 0; i < PD; ++i) {
        const bool on_axis = (i == a);
        qp[i] = q[i] + (wrap_up ? (on_axis ? 0 : 1) : (on_axis ? -1 : 0));
    }
    int u = -1;
    if constexpr (WIDE) {
        const Key128 want = WideCodec<PD>::pack(qp, wrap_up ? 0 : r + 1);
        uint32_t h = hash_key(want) & mask;
        for (uint32_t index = 0; index <= mask; ++index) {
            const ulonglong2 cur = reinterpret_cast<const ulonglong2 *>(cell_keys)[h];
            if (cur.x == want.a && cur.y == want.b) {
                u = vertices.cell_vertex[h];
                break;
            }
            if (cur.x == kEmptyCell) break;
            h = (h + 1u) & mask;
        }
    }
    const uint64_t want = WIDE ? 0ull : KeyCodec<PD>::pack(qp, wrap_up ? 0 : r + 1);
    uint32_t h = WIDE ? 0u : cell_of_key<PD>(want, mask, regions);
    for (uint32_t index = 0; !WIDE && index <= (mask >> 1) + 1u; ++index) {
        const ulonglong2 cur = *reinterpret_cast<const ulonglong2 *>(cell_keys + h);
        if (cur.x == want || (cur.x != kEmptyCell && cur.y == want)) {
            u = vertices.cell_vertex[cur.x == want ? h : h + 1u];
            break;
        }
        if (cur.x == kEmptyCell || cur.y == kEmptyCell) break;
        h = next_pair(h, index, want, mask, regions);
    }
    if (u >= 0) {
        int *entries = reinterpret_cast<int *>(vertices.neighbours);
        entries[2 * ((size_t)a * max_vertices + v)] = u;          // out[a][v].x
        entries[2 * ((size_t)a * max_vertices + u) + 1] = v;      // out[a][u].y
    }
    }
}

__global__ __launch_bounds__(kBlock) void k_fill_zero(float *p, size_t n) {
    const size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x;
    if (i < n) p[i] = 0.0f;
}

// ------------------------------------------------------------------------------------------------
// Stage 3: splat
//
// What bounds it is the L2 atomic unit, which retires about 20 G requests per second on MI355X,
// where a request is what one instruction sends to one 64-byte line, however many lanes it
// carries.  So (a) the contributions of a wavefront to one vertex are summed before they leave
// the wavefront and (b) the sums go out with consecutive lanes on consecutive channels of the
// vertex, so that a vertex row costs one request and not vd.
// ------------------------------------------------------------------------------------------------

// vd <= 4: all in registers.  The group loop of the deduplication doubles as the reduction loop:
// for each distinct vertex of the wavefront the members' terms are reduce-scattered inside each
// quad of lanes (lane keeps one channel), summed across the quads of a row and across the four rows,
// and lanes 60..63 send the four channel sums of the vertex as one atomic instruction.
template <int VD, int D1>
__global__ __launch_bounds__(kBlock) void k_splat_dpp(PointMap map,
                                                       const float *__restrict__ input,
                                                       int in_channels, ReplayEntry *replay,
                                                       const int *__restrict__ cell_vertex,
                                                       float *values, int xcd_aware) {
    static_assert(VD >= 2 && VD <= 4, "register splat handles 2..4 channels");
    constexpr int P = VD == 2 ? 2 : 4;   // lanes per vertex row in the final atomic
    unsigned vblock;
    if (!block_of_points(map, xcd_aware, vblock)) return;
    const size_t t = (size_t)vblock * kBlock + threadIdx.x;
    const size_t T = (size_t)gridDim.x * kBlock;
    const int n = point_of_thread(map, vblock, threadIdx.x);
    const int lane = threadIdx.x & 63;
    const int my_channel = channel_of_lane<VD>(lane);

    float val[4] = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
    for (int j = 0; j < VD; ++j) val[j] = 1.0f;  // homogeneous channel when only vd-1 are given
    if (n >= 0) {
#pragma unroll
        for (int j = 0; j < VD; ++j)
            if (j < in_channels) val[j] = input[(size_t)n * in_channels + j];
    }

    // all rows of the point at once, so that their latencies overlap
    int vertex[D1];
    float weight[D1];
#pragma unroll
    for (int r = 0; r < D1; ++r) {
        const ReplayEntry e = replay[(size_t)r * T + t];
        vertex[r] = n >= 0 ? e.index : -1;
        weight[r] = e.weight;
    }
    if (cell_vertex) {
#pragma unroll
        for (int r = 0; r < D1; ++r)
            if (vertex[r] >= 0) vertex[r] = cell_vertex[vertex[r]];
#pragma unroll
        for (int r = 0; r < D1; ++r)
            if (n >= 0) replay[(size_t)r * T + t].index = vertex[r];
    }

#pragma unroll
    for (int r = 0; r < D1; ++r) {
        const int v = vertex[r];
        const float w = weight[r];
        const float term[4] = {w * val[0], w * val[1], w * val[2], w * val[3]};
        const QuadTerms quad = quad_terms<VD>(term, lane);
        uint64_t remaining = wave_ballot(v >= 0);
        while (remaining) {
            const int first = __builtin_ctzll(remaining);
            const int k = lane_value(v, first);
            const uint64_t group = lanes_equal(v, k);
            remaining &= ~group;
            const bool same = lane_in(group);
            const float sum = wave_sum_to_last_lanes<VD>(same, quad, lane);
            if (lane >= 64 - P && my_channel < VD)
                atomicAdd(values + (size_t)k * VD + my_channel, sum);
        }
    }
}

// Any vd: the same, four channels at a time.  The deduplication loop runs once per block of four
// channels (it is cheap next to the reduction), the replay rows stay in registers.
template <int D1>
__global__ __launch_bounds__(kBlock) void k_splat_dpp_blocks(int vd, PointMap map,
                                                              const float *__restrict__ input,
                                                              int in_channels, ReplayEntry *replay,
                                                              const int *__restrict__ cell_vertex,
                                                              float *values, int xcd_aware) {
    unsigned vblock;
    if (!block_of_points(map, xcd_aware, vblock)) return;
    const size_t t = (size_t)vblock * kBlock + threadIdx.x;
    const size_t T = (size_t)gridDim.x * kBlock;
    const int n = point_of_thread(map, vblock, threadIdx.x);
    const int lane = threadIdx.x & 63;
    const int my_channel = channel_of_lane<4>(lane);

    int vertex[D1];
    float weight[D1];
#pragma unroll
    for (int r = 0; r < D1; ++r) {
        const ReplayEntry e = replay[(size_t)r * T + t];
        vertex[r] = n >= 0 ? e.index : -1;
        weight[r] = e.weight;
    }
    if (cell_vertex) {
#pragma unroll
        for (int r = 0; r < D1; ++r)
            if (vertex[r] >= 0) vertex[r] = cell_vertex[vertex[r]];
#pragma unroll
        for (int r = 0; r < D1; ++r)
            if (n >= 0) replay[(size_t)r * T + t].index = vertex[r];
    }

    for (int first_channel = 0; first_channel < vd; first_channel += 4) {
        float val[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int c = first_channel + j;
            // channels past the input are the homogeneous one (1), past vd nothing
            val[j] = c >= vd ? 0.0f
                             : (c < in_channels ? (n >= 0 ? input[(size_t)n * in_channels + c] : 0.0f)
                                                : 1.0f);
        }
#pragma unroll
        for (int r = 0; r < D1; ++r) {
            const int v = vertex[r];
            const float w = weight[r];
            const float term[4] = {w * val[0], w * val[1], w * val[2], w * val[3]};
            const QuadTerms quad = quad_terms<4>(term, lane);
            uint64_t remaining = wave_ballot(v >= 0);
            while (remaining) {
                const int first = __builtin_ctzll(remaining);
                const int k = lane_value(v, first);
                const uint64_t group = lanes_equal(v, k);
                remaining &= ~group;
                const bool same = lane_in(group);
                const float sum = wave_sum_to_last_lanes<4>(same, quad, lane);
                if (lane >= 60 && first_channel + my_channel < vd)
                    atomicAdd(values + (size_t)k * vd + first_channel + my_channel, sum);
            }
        }
    }
}

// Many channels (vd > 4, input rows of up to 64 channels): the lanes of a wavefront turn from
// points into channels.  The wavefront first puts the input rows of its 64 points into LDS
// (coalesced: consecutive lanes read consecutive floats); then, per simplex corner and per group
// of points that share the vertex, lane c runs over the group's members, reads channel c of each
// member's row from LDS and accumulates weight * value (channels past the input are the
// homogeneous 1); one atomic instruction then adds the vd sums to the vertex row, consecutive
// lanes on consecutive floats.  Against four channels at a time with a reduction tree per group
// this is 1/6 of the instructions for vd = 22 and reads every input float from memory once.
template <int W>
__global__ __launch_bounds__(kBlock) void k_splat_channels(int d1, int vd, PointMap map,
                                                            const float *__restrict__ input,
                                                            int in_channels, ReplayEntry *replay,
                                                            const int *__restrict__ cell_vertex,
                                                            float *values, int xcd_aware) {
    extern __shared__ float rows[];   // [kBlock][in_channels]
    // workgroup (x, y): simplex corners 2y and 2y+1 of the points of block x.  With a few hundred
    // thousand points there are too few wavefronts to hide the latencies of this serial code
    // unless the corners are spread over several of them; each pays for putting the rows into LDS.
    constexpr int kCorners = 2;
    unsigned vblock;
    if (!block_of_points(map, xcd_aware, vblock)) return;
    const size_t t = (size_t)vblock * kBlock + threadIdx.x;
    const size_t T = (size_t)gridDim.x * kBlock;
    const int n = point_of_thread(map, vblock, threadIdx.x);
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    float *wave_rows = rows + (size_t)wave * 64 * in_channels;

    int vertex[kCorners];
    float weight[kCorners];
#pragma unroll
    for (int i = 0; i < kCorners; ++i) {
        const int r = blockIdx.y * kCorners + i;
        vertex[i] = -1;
        weight[i] = 0.0f;
        if (r < d1) {
            const ReplayEntry e = replay[(size_t)r * T + t];
            vertex[i] = n >= 0 ? e.index : -1;
            weight[i] = e.weight;
            if (cell_vertex) {
                if (vertex[i] >= 0) vertex[i] = cell_vertex[vertex[i]];
                if (n >= 0) replay[(size_t)r * T + t].index = vertex[i];
            }
        }
    }

    // element i of the wavefront's 64 rows belongs to point i / in_channels, channel i % in_channels
    // (eight loads asked for before the first is stored: a point without data reads point 0 and
    // stores zero, so that no load waits behind a branch)
    {
        int p = lane / in_channels, c = lane - p * in_channels;
        const int step_p = 64 / in_channels, step_c = 64 - step_p * in_channels;
        constexpr int kBatch = 8;
        for (int i0 = lane; i0 < 64 * in_channels; i0 += 64 * kBatch) {
            float x[kBatch];
            bool has[kBatch];
#pragma unroll
            for (int k = 0; k < kBatch; ++k) {
                const bool inside = i0 + 64 * k < 64 * in_channels;
                const int np = __shfl(n, inside ? p : 0);
                has[k] = inside && np >= 0;
                x[k] = input[(size_t)(has[k] ? np : 0) * in_channels + (has[k] ? c : 0)];
                p += step_p;
                c += step_c;
                if (c >= in_channels) {
                    c -= in_channels;
                    p += 1;
                }
            }
#pragma unroll
            for (int k = 0; k < kBatch; ++k) asm volatile("" : "+v"(x[k]));
#pragma unroll
            for (int k = 0; k < kBatch; ++k)
                if (i0 + 64 * k < 64 * in_channels) wave_rows[i0 + 64 * k] = has[k] ? x[k] : 0.0f;
        }
    }
    __syncthreads();

    // W lanes per member (W = 16, 32 or 64, at least vd unless vd > 64): G = 64 / W members of a
    // group are taken per step, member g by the lanes g*W .. g*W+W-1
    constexpr int G = 64 / W;
    const int sub = lane / W, c_in_w = lane % W;
#pragma unroll
    for (int i = 0; i < kCorners; ++i) {
        const int v = vertex[i];
        const float w = weight[i];
        uint64_t remaining = wave_ballot(v >= 0);
        while (remaining) {
            const int first = __builtin_ctzll(remaining);
            const int k = lane_value(v, first);
            const uint64_t group = lanes_equal(v, k);
            remaining &= ~group;
            for (int c0 = 0; c0 < vd; c0 += W) {
                const int c = c0 + c_in_w;
                float acc = 0.0f;
                uint64_t members = group;
                while (members) {
                    int m = first;
                    float wm = 0.0f;
#pragma unroll
                    for (int g = 0; g < G; ++g) {
                        const bool has = members != 0;
                        const int mg = has ? __builtin_ctzll(members) : first;
                        members &= members - 1;
                        const float wg =
                            __int_as_float(__builtin_amdgcn_readlane(__float_as_int(w), mg));
                        if (sub == g) {
                            m = mg;
                            wm = has ? wg : 0.0f;
                        }
                    }
                    const float x = c < in_channels ? wave_rows[m * in_channels + c] : 1.0f;
                    acc += wm * x;
                }
                if (G >= 4) acc += __shfl_xor(acc, 16);
                if (G >= 2) acc += __shfl_xor(acc, 32);
                if (sub == 0 && c < vd) atomicAdd(values + ((unsigned)k * (unsigned)vd + (unsigned)c), acc);
            }
        }
    }
}

// ------------------------------------------------------------------------------------------------
// Stage 4: blur along one axis (reference: src/PermutohedralLatticeCPU.h:403-405, evaluated in
// double and rounded once, as there).  The vertex count is read on the device.  The first blur
// after a build also empties the hash cells of its vertices (reset_cell_keys != nullptr), which
// leaves the table clean for the next build without a pass over all cells.
// ------------------------------------------------------------------------------------------------
__device__ __forceinline__ float blur_tap(float a, float self, float b) {
    return (float)(0.25 * (double)a + 0.5 * (double)self + 0.25 * (double)b);
}

// (S = double: the values of a lattice of doubles)
__device__ __forceinline__ double blur_tap(double a, double self, double b) {
    return 0.25 * a + 0.5 * self + 0.25 * b;
}

// Loads never depend on a branch: an absent neighbour (-1) reads vertex 0 and the value is then
// replaced by zero, so that all the loads of one level of the gather are in flight together
// (with a branch per neighbour each load is waited for before the next is asked for: thirteen
// round trips in a row for two axes instead of three).  The empty asm statements keep the
// compiler from moving the loads back under the conditions.
template <typename S, int N>
__device__ __forceinline__ void gather_elements(const S *__restrict__ src, int vd, int j,
                                                const int (&u)[N], S (&x)[N]) {
#pragma unroll
    for (int k = 0; k < N; ++k) x[k] = src[(size_t)(u[k] >= 0 ? u[k] : 0) * vd + j];
#pragma unroll
    for (int k = 0; k < N; ++k) asm volatile("" : "+v"(x[k]));
#pragma unroll
    for (int k = 0; k < N; ++k) x[k] = u[k] >= 0 ? x[k] : (S)0;
}

// The vertices whose values the taps along axis a, then axis b at vertex v combine (nine; -1
// where there is none: an absent b-neighbour stands for three zeros, whose tap is zero).
__device__ __forceinline__ void two_axis_sources(const int2 *__restrict__ nbr_a,
                                                 const int2 *__restrict__ nbr_b, int v,
                                                 int (&u)[9]) {
    const int2 nb = nbr_b[v];
    const int2 na_self = nbr_a[v];
    int2 na_x = nbr_a[nb.x >= 0 ? nb.x : 0];
    int2 na_y = nbr_a[nb.y >= 0 ? nb.y : 0];
    asm volatile("" : "+v"(na_x.x), "+v"(na_x.y), "+v"(na_y.x), "+v"(na_y.y));
    u[0] = nb.x >= 0 ? na_x.x : -1;
    u[1] = nb.x;
    u[2] = nb.x >= 0 ? na_x.y : -1;
    u[3] = na_self.x;
    u[4] = v;
    u[5] = na_self.y;
    u[6] = nb.y >= 0 ? na_y.x : -1;
    u[7] = nb.y;
    u[8] = nb.y >= 0 ? na_y.y : -1;
}

// one thread per (vertex, channel), any vd
template <typename S>
__global__ __launch_bounds__(kBlock) void k_blur_element(const Counters *counters, int max_vertices,
                                                          int vd, const S *__restrict__ src,
                                                          S *__restrict__ dst,
                                                          const int2 *__restrict__ nbr,
                                                          uint64_t *reset_cell_keys,
                                                          const int *__restrict__ vertex_cell) {
    SegmentWalk walk(counters, max_vertices, blockIdx.x, gridDim.x);
    unsigned eb;
    while (walk.next((unsigned)vd, 1u, eb)) {
        const size_t i = (size_t)eb * kBlock + threadIdx.x;
        if (i >= (size_t)walk.count * vd) continue;
        const size_t e = (size_t)walk.first * vd + i;
        const int v = (int)(e / (size_t)vd);
        const int j = (int)(e - (size_t)v * vd);
        const int2 nb = nbr[v];
        const int u[3] = {nb.x, v, nb.y};
        S x[3];
        gather_elements<S, 3>(src, vd, j, u, x);
        dst[e] = blur_tap(x[0], x[1], x[2]);
        if (reset_cell_keys && j == 0) reset_cell_keys[vertex_cell[v]] = kEmptyCell;
    }
}

// Two axes in one launch.  Every kernel boundary costs a cold L2 and a round of dependent loads,
// and a blur pass has almost no work, so axis a and then axis b are applied together: the value
// after axis a is evaluated (and rounded to the value type, as the separate pass would store it)
// at the vertex and at its two b-neighbours, then the b tap combines the three.  An absent
// b-neighbour contributes zero, whatever its own a-neighbours hold.  Same arithmetic, same results.
template <typename S>
__global__ __launch_bounds__(kBlock) void k_blur2_element(const Counters *counters, int max_vertices,
                                                           int vd, const S *__restrict__ src,
                                                           S *__restrict__ dst,
                                                           const int2 *__restrict__ nbr_a,
                                                           const int2 *__restrict__ nbr_b,
                                                           uint64_t *reset_cell_keys,
                                                           const int *__restrict__ vertex_cell) {
    SegmentWalk walk(counters, max_vertices, blockIdx.x, gridDim.x);
    unsigned eb;
    while (walk.next((unsigned)vd, 1u, eb)) {
        const size_t i = (size_t)eb * kBlock + threadIdx.x;
        if (i >= (size_t)walk.count * vd) continue;
        const size_t e = (size_t)walk.first * vd + i;
        const int v = (int)(e / (size_t)vd);
        const int j = (int)(e - (size_t)v * vd);
        int u[9];
        two_axis_sources(nbr_a, nbr_b, v, u);
        S x[9];
        gather_elements<S, 9>(src, vd, j, u, x);
        dst[e] = blur_tap(blur_tap(x[0], x[1], x[2]), blur_tap(x[3], x[4], x[5]),
                          blur_tap(x[6], x[7], x[8]));
        if (reset_cell_keys && j == 0) reset_cell_keys[vertex_cell[v]] = kEmptyCell;
    }
}

// For up to four channels: one thread per vertex, the whole row in one vector access.  With
// vertex numbers that follow the image the rows a thread gathers are near each other, and a
// quarter of the memory instructions moves the same bytes (34 -> 25 us for the three launches
// of pd = 5, vd = 4).  Same arithmetic per channel, same results.
template <int VD, typename S = float>
__device__ __forceinline__ ValueRow<VD, S> blur_rows(const ValueRow<VD, S> &a, const ValueRow<VD, S> &self,
                                                  const ValueRow<VD, S> &b) {
    ValueRow<VD, S> out;
#pragma unroll
    for (int j = 0; j < VD; ++j) out.c[j] = blur_tap(a.c[j], self.c[j], b.c[j]);
    return out;
}

// Loads never depend on a branch: an absent neighbour (-1) reads row 0 and its values are then
// replaced by zeros, so that all the loads of one level of the gather are in flight together
// (with a branch per neighbour each load is waited for before the next is asked for: thirteen
// round trips in a row for two axes instead of three).  The empty asm statements keep the
// compiler from moving the loads back under the conditions.
template <int VD, typename S, int N>
__device__ __forceinline__ void gather_rows(const ValueRow<VD, S> *__restrict__ src,
                                            const int (&u)[N], ValueRow<VD, S> (&row)[N]) {
#pragma unroll
    for (int k = 0; k < N; ++k) row[k] = src[u[k] >= 0 ? u[k] : 0];
#pragma unroll
    for (int k = 0; k < N; ++k) {
#pragma unroll
        for (int j = 0; j < VD; ++j) asm volatile("" : "+v"(row[k].c[j]));
    }
#pragma unroll
    for (int k = 0; k < N; ++k) {
#pragma unroll
        for (int j = 0; j < VD; ++j) row[k].c[j] = u[k] >= 0 ? row[k].c[j] : (S)0;
    }
}

template <int VD, typename S = float>
__global__ __launch_bounds__(kBlock) void k_blur_row(const Counters *counters, int max_vertices,
                                                      const ValueRow<VD, S> *__restrict__ src,
                                                      ValueRow<VD, S> *__restrict__ dst,
                                                      const int2 *__restrict__ nbr,
                                                      uint64_t *reset_cell_keys,
                                                      const int *__restrict__ vertex_cell) {
    SegmentWalk walk(counters, max_vertices, blockIdx.x, gridDim.x);
    unsigned vb;
    while (walk.next(1u, 1u, vb)) {
        const unsigned i = vb * kBlock + threadIdx.x;
        if (i >= walk.count) continue;
        const int v = (int)(walk.first + i);
        const int2 nb = nbr[v];
        const int u[3] = {nb.x, v, nb.y};
        ValueRow<VD, S> row[3];
        gather_rows<VD, S, 3>(src, u, row);
        dst[v] = blur_rows<VD, S>(row[0], row[1], row[2]);
        if (reset_cell_keys) reset_cell_keys[vertex_cell[v]] = kEmptyCell;
    }
}

template <int VD, typename S = float>
__global__ __launch_bounds__(kBlock) void k_blur2_row(const Counters *counters, int max_vertices,
                                                       const ValueRow<VD, S> *__restrict__ src,
                                                       ValueRow<VD, S> *__restrict__ dst,
                                                       const int2 *__restrict__ nbr_a,
                                                       const int2 *__restrict__ nbr_b,
                                                       uint64_t *reset_cell_keys,
                                                       const int *__restrict__ vertex_cell) {
    SegmentWalk walk(counters, max_vertices, blockIdx.x, gridDim.x);
    unsigned vb;
    while (walk.next(1u, 1u, vb)) {
        const unsigned i = vb * kBlock + threadIdx.x;
        if (i >= walk.count) continue;
        const int v = (int)(walk.first + i);
        // level 1: the vertex's neighbours along both axes; level 2: the a-neighbours of its
        // b-neighbours; level 3: nine rows
        int u[9];
        two_axis_sources(nbr_a, nbr_b, v, u);
        ValueRow<VD, S> row[9];
        gather_rows<VD, S, 9>(src, u, row);
        dst[v] = blur_rows<VD, S>(blur_rows<VD, S>(row[0], row[1], row[2]),
                                  blur_rows<VD, S>(row[3], row[4], row[5]),
                                  blur_rows<VD, S>(row[6], row[7], row[8]));
        if (reset_cell_keys) reset_cell_keys[vertex_cell[v]] = kEmptyCell;
    }
}

// Three axes in one launch: four levels of loads (1, 3, 9 neighbour pairs, 27 rows) instead of
// three launches' worth.  u[3i..3i+2] are the sources of the a-tap at the i-th of the nine
// vertices the b- and c-taps combine.
__device__ __forceinline__ void three_axis_sources(const int2 *__restrict__ nbr_a,
                                                   const int2 *__restrict__ nbr_b,
                                                   const int2 *__restrict__ nbr_c, int v,
                                                   int (&u)[27]) {
    const int2 nc = nbr_c[v];
    const int w[3] = {nc.x, v, nc.y};
    int2 nbw[3];
#pragma unroll
    for (int k = 0; k < 3; ++k) nbw[k] = nbr_b[w[k] >= 0 ? w[k] : 0];
#pragma unroll
    for (int k = 0; k < 3; ++k) asm volatile("" : "+v"(nbw[k].x), "+v"(nbw[k].y));
    int m[9];
#pragma unroll
    for (int k = 0; k < 3; ++k) {
        m[3 * k] = w[k] >= 0 ? nbw[k].x : -1;
        m[3 * k + 1] = w[k];
        m[3 * k + 2] = w[k] >= 0 ? nbw[k].y : -1;
    }
    int2 nam[9];
#pragma unroll
    for (int i = 0; i < 9; ++i) nam[i] = nbr_a[m[i] >= 0 ? m[i] : 0];
#pragma unroll
    for (int i = 0; i < 9; ++i) asm volatile("" : "+v"(nam[i].x), "+v"(nam[i].y));
#pragma unroll
    for (int i = 0; i < 9; ++i) {
        u[3 * i] = m[i] >= 0 ? nam[i].x : -1;
        u[3 * i + 1] = m[i];
        u[3 * i + 2] = m[i] >= 0 ? nam[i].y : -1;
    }
}

template <int VD, typename S = float>
__global__ __launch_bounds__(kBlock) void k_blur3_row(const Counters *counters, int max_vertices,
                                                       const ValueRow<VD, S> *__restrict__ src,
                                                       ValueRow<VD, S> *__restrict__ dst,
                                                       const int2 *__restrict__ nbr_a,
                                                       const int2 *__restrict__ nbr_b,
                                                       const int2 *__restrict__ nbr_c,
                                                       uint64_t *reset_cell_keys,
                                                       const int *__restrict__ vertex_cell) {
    SegmentWalk walk(counters, max_vertices, blockIdx.x, gridDim.x);
    unsigned vb;
    while (walk.next(1u, 1u, vb)) {
        const unsigned i = vb * kBlock + threadIdx.x;
        if (i >= walk.count) continue;
        const int v = (int)(walk.first + i);
        int u[27];
        three_axis_sources(nbr_a, nbr_b, nbr_c, v, u);
        ValueRow<VD, S> row[27];
        gather_rows<VD, S, 27>(src, u, row);
        ValueRow<VD, S> after_a[9];
#pragma unroll
        for (int i = 0; i < 9; ++i)
            after_a[i] = blur_rows<VD, S>(row[3 * i], row[3 * i + 1], row[3 * i + 2]);
        dst[v] = blur_rows<VD, S>(blur_rows<VD, S>(after_a[0], after_a[1], after_a[2]),
                                  blur_rows<VD, S>(after_a[3], after_a[4], after_a[5]),
                                  blur_rows<VD, S>(after_a[6], after_a[7], after_a[8]));
        if (reset_cell_keys) reset_cell_keys[vertex_cell[v]] = kEmptyCell;
    }
}

// ------------------------------------------------------------------------------------------------
// Stage 5: slice (reference: src/PermutohedralLatticeCPU.h:333-352)
// ------------------------------------------------------------------------------------------------
// cell_vertex != nullptr: the replay rows still hold hash cells (nothing has translated them yet)
template <int VD, int D1 = 0>
__global__ __launch_bounds__(kBlock) void k_slice_point(int d1, PointMap map,
                                                         const ReplayEntry *__restrict__ replay,
                                                         const int *__restrict__ cell_vertex,
                                                         const float *__restrict__ values,
                                                         float *__restrict__ output, int normalize) {
    // each XCD takes one contiguous range of the tiles: the value rows it gathers (vertex numbers
    // follow the tiles) are then in its own L2 and not in all eight
    unsigned vblock;
    if (!block_of_points(map, 1, vblock)) return;
    const size_t t = (size_t)vblock * kBlock + threadIdx.x;
    const size_t T = (size_t)gridDim.x * kBlock;
    const int n = point_of_thread(map, vblock, threadIdx.x);
    if (n < 0) return;
    float acc[VD];
#pragma unroll
    for (int j = 0; j < VD; ++j) acc[j] = 0.0f;
    if constexpr (D1 > 0) {
        // all replay rows, then all translations, then all value rows: three round trips to
        // memory instead of three per corner (what a point waits for when many workgroups queue
        // behind each other, as for a volume of millions of voxels)
        ReplayEntry e[D1];
        int v[D1];
#pragma unroll
        for (int r = 0; r < D1; ++r) e[r] = replay[(size_t)r * T + t];
#pragma unroll
        for (int r = 0; r < D1; ++r) {
            v[r] = e[r].index;
            if (cell_vertex && v[r] >= 0) v[r] = cell_vertex[v[r]];
        }
        ValueRow<VD> row[D1];
#pragma unroll
        for (int r = 0; r < D1; ++r)
            row[r] = reinterpret_cast<const ValueRow<VD> *>(values)[v[r] >= 0 ? v[r] : 0];
#pragma unroll
        for (int r = 0; r < D1; ++r) {
            if (v[r] < 0) continue;
#pragma unroll
            for (int j = 0; j < VD; ++j) acc[j] += e[r].weight * row[r].c[j];
        }
    } else {
        for (int r = 0; r < d1; ++r) {
            const ReplayEntry e = replay[(size_t)r * T + t];
            int v = e.index;
            if (v < 0) continue;
            if (cell_vertex) v = cell_vertex[v];
            const float w = e.weight;
            const float *src = values + (size_t)v * VD;
#pragma unroll
            for (int j = 0; j < VD; ++j) acc[j] += w * src[j];
        }
    }
    if (normalize) {
        const float scale = (float)(1.0 / (double)acc[VD - 1]);
#pragma unroll
        for (int j = 0; j < VD - 1; ++j) output[(size_t)n * (VD - 1) + j] = acc[j] * scale;
    } else {
#pragma unroll
        for (int j = 0; j < VD; ++j) output[(size_t)n * VD + j] = acc[j];
    }
}

// The same for rows of doubles (weights64[r*T+t]: the barycentric weights as doubles; the replay
// rows give the vertices).  Arithmetic as in k_slice_point_f64.
template <int VD, int D1>
__global__ __launch_bounds__(kBlock) void k_slice_rows_f64(PointMap map,
                                                            const ReplayEntry *__restrict__ replay,
                                                            const double *__restrict__ weights64,
                                                            const int *__restrict__ cell_vertex,
                                                            const double *__restrict__ values,
                                                            double *__restrict__ output,
                                                            int normalize) {
    unsigned vblock;
    if (!block_of_points(map, 1, vblock)) return;
    const size_t t = (size_t)vblock * kBlock + threadIdx.x;
    const size_t T = (size_t)gridDim.x * kBlock;
    const int n = point_of_thread(map, vblock, threadIdx.x);
    if (n < 0) return;
    int v[D1];
    double w[D1];
#pragma unroll
    for (int r = 0; r < D1; ++r) {
        v[r] = replay[(size_t)r * T + t].index;
        w[r] = weights64[(size_t)r * T + t];
    }
    if (cell_vertex) {
#pragma unroll
        for (int r = 0; r < D1; ++r)
            if (v[r] >= 0) v[r] = cell_vertex[v[r]];
    }
    ValueRow<VD, double> row[D1];
#pragma unroll
    for (int r = 0; r < D1; ++r)
        row[r] = reinterpret_cast<const ValueRow<VD, double> *>(values)[v[r] >= 0 ? v[r] : 0];
    double sum[VD];
#pragma unroll
    for (int j = 0; j < VD; ++j) sum[j] = 0.0;
#pragma unroll
    for (int r = 0; r < D1; ++r) {
        if (v[r] < 0) continue;
#pragma unroll
        for (int j = 0; j < VD; ++j) sum[j] += w[r] * row[r].c[j];
    }
    if (normalize) {
        const double scale = 1.0 / sum[VD - 1];
#pragma unroll
        for (int j = 0; j < VD - 1; ++j) output[(size_t)n * (VD - 1) + j] = sum[j] * scale;
    } else {
#pragma unroll
        for (int j = 0; j < VD; ++j) output[(size_t)n * VD + j] = sum[j];
    }
}

// Any vd: one thread per point and run of four channels.  The pd+1 replay rows, then the value
// rows, are all requested before the first is used (with a run-time loop the passes waited for
// two memory round trips per vertex, one after the other); the channels of a run share the index
// arithmetic and the replay loads.
constexpr int kSliceRun = 4;   // channels per thread of k_slice_channels (8: 10 % slower)
template <int D1>
__global__ __launch_bounds__(kBlock) void k_slice_channels(int vd, PointMap map, size_t T,
                                                            const ReplayEntry *__restrict__ replay,
                                                            const float *__restrict__ values,
                                                            float *__restrict__ output, int normalize) {
    // workgroup (x, y): items y*256 .. y*256+255 of the 256*runs (point, run of channels) pairs
    // of point block x
    const int out_ch = normalize ? vd - 1 : vd;
    const unsigned runs = (unsigned)(out_ch + kSliceRun - 1) / (unsigned)kSliceRun;
    const unsigned item = blockIdx.y * kBlock + threadIdx.x;
    const unsigned slot = item / runs;
    if (slot >= kBlock) return;
    const int j0 = kSliceRun * (int)(item - slot * runs);
    unsigned vblock;   // as in k_slice_point
    if (!block_of_points(map, 1, vblock)) return;
    const size_t t = (size_t)vblock * kBlock + slot;
    const int n = point_of_thread(map, vblock, slot);
    if (n < 0) return;
    ReplayEntry e[D1];
#pragma unroll
    for (int r = 0; r < D1; ++r) e[r] = replay[(size_t)r * T + t];
    float own[D1][kSliceRun], last[D1];
#pragma unroll
    for (int r = 0; r < D1; ++r) {
        const bool present = e[r].index >= 0;
        const float *src = values + (size_t)(present ? e[r].index : 0) * vd;
        // rows of an even number of floats start on 8-byte boundaries: loads of two floats; the
        // memory pipeline is bound by the number of requests here, not by bytes
#pragma unroll
        for (int i = 0; i < kSliceRun; i += 2) {
            if (present && (vd & 1) == 0 && j0 + i + 1 < vd) {
                const float2 x = *reinterpret_cast<const float2 *>(src + j0 + i);
                own[r][i] = x.x, own[r][i + 1] = x.y;
            } else {
                own[r][i] = (present && j0 + i < vd) ? src[j0 + i] : 0.0f;
                own[r][i + 1] = (present && j0 + i + 1 < vd) ? src[j0 + i + 1] : 0.0f;
            }
        }
        last[r] = present ? src[vd - 1] : 0.0f;
    }
    float acc[kSliceRun], hom = 0.0f;
#pragma unroll
    for (int i = 0; i < kSliceRun; ++i) acc[i] = 0.0f;
#pragma unroll
    for (int r = 0; r < D1; ++r) {
        if (e[r].index < 0) continue;
#pragma unroll
        for (int i = 0; i < kSliceRun; ++i) acc[i] += e[r].weight * own[r][i];
        hom += e[r].weight * last[r];
    }
    const float scale = normalize ? (float)(1.0 / (double)hom) : 1.0f;
#pragma unroll
    for (int i = 0; i < kSliceRun; ++i)
        if (j0 + i < out_ch)
            output[(size_t)n * out_ch + j0 + i] = normalize ? acc[i] * scale : acc[i];
}

// Nine to sixty-four channels: L lanes per point (4, 8 or 16), lane i on the channels 4i .. 4i+3.
// What bounds the slice of rows of many channels is the number of load instructions, not bytes
// (the memory pipeline looks at the 64 addresses of one for 16 cycles whatever their width): a
// lane reads its four channels of a vertex row with one 16-byte load (rows need only be aligned to
// four bytes for that), and the pd+1 replay rows of a point are read once, a corner per lane, and
// handed round.  The lane on the row's last channels reads the row's last four instead, so that
// no load leaves the row, and its sums are shifted back before they are stored.  Same sums in the
// same order as k_slice_channels.
struct alignas(4) FourFloats {
    float c[4];
};
constexpr int kSlicePoints = 2;   // points per group of L lanes (1: 2 % slower, 4: 4 %)
template <int D1, int L>
__global__ __launch_bounds__(kBlock) void k_slice_quads(int vd, PointMap map, size_t T,
                                                         const ReplayEntry *__restrict__ replay,
                                                         const float *__restrict__ values,
                                                         float *__restrict__ output, int normalize) {
    // workgroup (x, y): kSlicePoints * 256 / L points of point block x, each group of L lanes
    // kSlicePoints of them, with the loads of all in flight together (a point's loads alone
    // leave the lanes waiting: what bounds the pass is then how many points are in flight)
    constexpr int kGroups = kBlock / L;
    constexpr int P = kSlicePoints;
    constexpr int E = (D1 + L - 1) / L;     // replay rows a lane reads per point
    const int sub = threadIdx.x % L;
    unsigned vblock;   // as in k_slice_point
    if (!block_of_points(map, 1, vblock)) return;
    int n[P];
    ReplayEntry mine[P][E];
#pragma unroll
    for (int q = 0; q < P; ++q) {
        const unsigned slot = (blockIdx.y * P + q) * kGroups + threadIdx.x / L;
        const size_t t = (size_t)vblock * kBlock + slot;
        n[q] = point_of_thread(map, vblock, slot);   // (the same for all L lanes)
#pragma unroll
        for (int u = 0; u < E; ++u) {
            const int r = u * L + sub;
            mine[q][u] = replay[(size_t)(r < D1 ? r : 0) * T + t];
        }
    }
    const int c = 4 * sub;
    const int start = c < vd - 4 ? c : vd - 4;
    FourFloats x[P][D1];
    float w[P][D1];
#pragma unroll
    for (int q = 0; q < P; ++q) {
#pragma unroll
        for (int r = 0; r < D1; ++r) {
            const int index = __shfl(mine[q][r / L].index, r % L, L);
            w[q][r] = __shfl(mine[q][r / L].weight, r % L, L);
            const bool present = index >= 0 && n[q] >= 0;
            x[q][r] = *reinterpret_cast<const FourFloats *>(values + (size_t)(present ? index : 0) * vd +
                                                            start);
            if (!present) w[q][r] = 0.0f, x[q][r] = FourFloats{{0.0f, 0.0f, 0.0f, 0.0f}};
        }
    }
    // the homogeneous channel vd-1 is with the lane (vd-1)/4
    const int with = (vd - 1) / 4;
    const int with_start = 4 * with < vd - 4 ? 4 * with : vd - 4;
    const int at = vd - 1 - with_start;
    const int out_ch = normalize ? vd - 1 : vd;
    const int shift = c - start;
#pragma unroll
    for (int q = 0; q < P; ++q) {
        float acc[4] = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
        for (int r = 0; r < D1; ++r) {
#pragma unroll
            for (int j = 0; j < 4; ++j) acc[j] += w[q][r] * x[q][r].c[j];
        }
        const float own = at == 0 ? acc[0] : at == 1 ? acc[1] : at == 2 ? acc[2] : acc[3];
        const float hom = __shfl(own, with, L);
        if (n[q] < 0) continue;
        const float scale = normalize ? (float)(1.0 / (double)hom) : 1.0f;
        float *out = output + (size_t)n[q] * out_ch + c;
        if (shift == 0 && c + 4 <= out_ch) {
            FourFloats y;
#pragma unroll
            for (int j = 0; j < 4; ++j) y.c[j] = normalize ? acc[j] * scale : acc[j];
            *reinterpret_cast<FourFloats *>(out) = y;
        } else {
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                if (c + j < out_ch) {
                    const int i = shift + j;
                    const float v = i == 0 ? acc[0] : i == 1 ? acc[1] : i == 2 ? acc[2] : acc[3];
                    out[j] = normalize ? v * scale : v;
                }
            }
        }
    }
}

// ------------------------------------------------------------------------------------------------
// Debug exports and the feature builder
// ------------------------------------------------------------------------------------------------
template <int PD>
__global__ __launch_bounds__(kBlock) void k_debug_simplex(const float *__restrict__ positions, int N,
                                                           ScaleFactor scale, short *rem0, short *rank,
                                                           short *keys, float *barycentric) {
    constexpr int D1 = PD + 1;
    const int n = blockIdx.x * kBlock + threadIdx.x;
    if (n >= N) return;
    float pos[PD];
    load_position<PD>(positions, n, pos);
    Simplex<PD> s;
    enclosing_simplex<PD>(pos, scale, s);
#pragma unroll
    for (int i = 0; i < D1; ++i) {
        if (rem0) rem0[(size_t)n * D1 + i] = (short)(s.q[i] * D1);
        if (rank) rank[(size_t)n * D1 + i] = (short)s.rank[i];
        if (barycentric) barycentric[(size_t)n * D1 + i] = s.weight[i];
    }
    if (keys) {
#pragma unroll
        for (int r = 0; r < D1; ++r) {
            int q[PD];
            vertex_q<PD>(s, r, q);
#pragma unroll
            for (int i = 0; i < PD; ++i)
                keys[((size_t)n * D1 + r) * PD + i] = (short)(q[i] * D1 + r);
        }
    }
}

// The debug exports count the vertices densely, segment after segment (VertexNumbers).
template <int PD, bool WIDE>
__global__ __launch_bounds__(kBlock) void k_export_keys(const uint64_t *__restrict__ vertex_keys,
                                                         VertexNumbers numbers, short *keys) {
    const unsigned d = blockIdx.x * kBlock + threadIdx.x;
    if (d >= numbers.total) return;
    int q[PD], r;
    if constexpr (WIDE) {
        const ulonglong2 k = reinterpret_cast<const ulonglong2 *>(vertex_keys)[numbers.vertex_of(d)];
        WideCodec<PD>::unpack(Key128{k.x, k.y}, q, r);
    } else {
        KeyCodec<PD>::unpack(vertex_keys[numbers.vertex_of(d)], q, r);
    }
#pragma unroll
    for (int i = 0; i < PD; ++i) keys[(size_t)d * PD + i] = (short)(q[i] * (PD + 1) + r);
}

__global__ __launch_bounds__(kBlock) void k_export_values(const float *__restrict__ values, int words,
                                                           VertexNumbers numbers, float *out) {
    const size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x;
    if (i >= (size_t)numbers.total * words) return;
    const unsigned d = (unsigned)(i / words);
    out[i] = values[(size_t)numbers.vertex_of(d) * words + (i - (size_t)d * words)];
}

// replay arrays from thread order to point order: out[r*N + n]; cells are translated to vertex
// indices when cell_vertex != nullptr
__global__ __launch_bounds__(kBlock) void k_export_replay(int d1, PointMap map,
                                                           const ReplayEntry *__restrict__ replay,
                                                           const int *__restrict__ cell_vertex,
                                                           VertexNumbers numbers,
                                                           int *vertex, float *weight) {
    const size_t t = (size_t)blockIdx.x * kBlock + threadIdx.x;
    const size_t T = (size_t)gridDim.x * kBlock;
    const int n = point_of_thread(map, blockIdx.x, threadIdx.x);
    if (n < 0) return;
    for (int r = 0; r < d1; ++r) {
        const ReplayEntry e = replay[(size_t)r * T + t];
        if (vertex) {
            int v = e.index;
            if (cell_vertex && v >= 0) v = cell_vertex[v];
            vertex[(size_t)r * map.N + n] = v >= 0 ? (int)numbers.dense_of((unsigned)v) : v;
        }
        if (weight) weight[(size_t)r * map.N + n] = e.weight;
    }
}

// Is the list of points a row-major grid?  The feature builder of the reference puts the grid
// coordinates first (src/PermutohedralLatticeCPU.h:464-469), so in positions that describe an
// image feature 0 changes exactly every row length points, and feature 1 (the next slower
// coordinate of a volume) every P1 points.  Pass 1 finds the first change of each, pass 2 checks
// that the changes are exactly at the multiples of those periods.  The result only chooses the
// order in which points are worked on, so a wrong guess costs time, never correctness.
__global__ __launch_bounds__(kBlock) void k_first_changes(const float *__restrict__ positions, int N,
                                                           int pd, GridGuess *guess) {
    const int n = blockIdx.x * kBlock + threadIdx.x + 1;
    if (n >= N) return;
    const float *row = positions + (size_t)n * pd;
    if (row[0] != row[0 - pd]) atomicMin(&guess->period[0], n);
    if (pd >= 2 && row[1] != row[1 - pd]) atomicMin(&guess->period[1], n);
}

__global__ __launch_bounds__(kBlock) void k_check_periods(const float *__restrict__ positions, int N,
                                                           int pd, GridGuess *guess) {
    const int n = blockIdx.x * kBlock + threadIdx.x + 1;
    if (n >= N) return;
    const int p0 = guess->period[0], p1 = pd >= 2 ? guess->period[1] : 1;
    const float *row = positions + (size_t)n * pd;
    bool bad = (row[0] != row[0 - pd]) != (n % p0 == 0);
    if (pd >= 2) bad = bad || ((row[1] != row[1 - pd]) != (n % p1 == 0));
    if (bad) guess->mismatch = 1;
}

// reference: src/PermutohedralLatticeCPU.h:464-473 (IEEE float division, int -> float exact)
__global__ __launch_bounds__(kBlock) void k_positions(const float *__restrict__ reference,
                                                       float *__restrict__ positions, int N, int rc,
                                                       int nsd, SpatialDims dims, float spatial_std,
                                                       float feature_std) {
    const int n = blockIdx.x * kBlock + threadIdx.x;
    if (n >= N) return;
    const int pd = nsd + rc;
    float *row = positions + (size_t)n * pd;
    int stride = 1;
    for (int s = nsd - 1; s >= 0; --s) {
        const int coord = (n / stride) % dims.v[s];
        row[s] = (float)coord / spatial_std;
        stride *= dims.v[s];
    }
    for (int c = 0; c < rc; ++c) row[nsd + c] = reference[(size_t)n * rc + c] / feature_std;
}

}  // namespace

int key_field_bits(int pd) {
    if (pd < 1 || pd > kMaxPd) return 0;
    const int b = 60 / pd;
    return b > 16 ? 16 : b;
}

PointMap make_point_map(int N, int n_dims, const int *dims) {
    PointMap m{};
    m.N = N;
    m.mode = 0;
    m.dims[0] = m.dims[1] = 1;
    m.dims[2] = N;
    m.tiles[0] = m.tiles[1] = m.tiles[2] = 1;
    m.n_blocks = (unsigned)(((size_t)N + kBlock - 1) / kBlock);
    if (n_dims >= 2 && dims) {
        // fold every leading extent into the slowest one: (d_0 * ... * d_{k-3}, d_{k-2}, d_{k-1})
        long long lead = 1;
        for (int i = 0; i < n_dims - 2; ++i) lead *= dims[i];
        const int H = dims[n_dims - 2], W = dims[n_dims - 1];
        if (n_dims == 2 || lead == 1) {
            m.mode = 2;
            m.dims[0] = 1; m.dims[1] = H; m.dims[2] = W;
            m.tiles[0] = 1; m.tiles[1] = (H + 15) / 16; m.tiles[2] = (W + 15) / 16;
        } else {
            m.mode = 3;
            m.dims[0] = (int)lead; m.dims[1] = H; m.dims[2] = W;
            m.tiles[0] = (int)((lead + 3) / 4); m.tiles[1] = (H + 7) / 8; m.tiles[2] = (W + 7) / 8;
        }
        const size_t tiles = (size_t)m.tiles[0] * m.tiles[1] * m.tiles[2];
        // An extent much shorter than its tile edge (a grid of N x 2 points) would leave most
        // lanes of every tile without a point and multiply the per-point scratch: such points are
        // taken as a plain list.
        if (tiles > 2 * (((size_t)N + kBlock - 1) / kBlock)) {
            m.mode = 0;
            m.dims[0] = m.dims[1] = 1;
            m.dims[2] = N;
            m.tiles[0] = m.tiles[1] = m.tiles[2] = 1;
        } else {
            m.n_blocks = (unsigned)tiles;
        }
    }
    if (N == 0) m.n_blocks = 0;
    return m;
}

hipError_t clear_table(uint64_t *cell_keys, uint32_t n_cells, hipStream_t s) {
    hipLaunchKernelGGL(k_clear_table, dim3(blocks_for(n_cells)), dim3(kBlock), 0, s, cell_keys, n_cells);
    return hipGetLastError();
}

bool build_can_splat(int vd) { return vd >= 2 && vd <= 4; }

hipError_t build(int pd, const PointFeatures &features, const PointMap &map, const ScaleFactor &scale,
                 uint64_t *cell_keys, uint32_t n_cells, Counters *counters, ReplayEntry *replay,
                 int xcd_aware, int splat_vd, const float *input,
                 int in_channels, float *cell_values, const CreatedLists &created_lists,
                 const RegionSource &regions, const InBuildNumbering *numbering, bool wide_keys,
                 hipStream_t s) {
    if (map.n_blocks == 0) return hipSuccess;
    if (wide_keys && numbering) return hipErrorInvalidValue;
    const bool merge_in_workgroup = numbering != nullptr;
    // (only the merging kernel knows of workgroups without points, as an ordered list has them)
    if (map.mode == 1 && (!merge_in_workgroup || !map.order || !map.n_tiles)) return hipErrorInvalidValue;
    const InBuildNumbering in_build = numbering ? *numbering : InBuildNumbering{};
#define PLK_BUILD_ARGS                                                                             \
    dim3(map.n_blocks), dim3(kBlock), 0, s, features, map, scale, cell_keys, n_cells - 1u,         \
        counters, replay, xcd_aware, (const void *)input, in_channels, (void *)cell_values,        \
        created_lists, Points64{}, regions
#define PLK_BUILD(SPLAT_VD)                                                                        \
    if (merge_in_workgroup)                                                                        \
        PLK_DISPATCH_PD(pd, hipLaunchKernelGGL((k_build_tile<PD, SPLAT_VD>), PLK_BUILD_ARGS,       \
                                               in_build))                                          \
    else if (wide_keys)                                                                            \
        PLK_DISPATCH_WIDE_PD(pd, hipLaunchKernelGGL((k_build<PD, SPLAT_VD, float, true>),          \
                                                    PLK_BUILD_ARGS))                               \
    else                                                                                           \
        PLK_DISPATCH_PD(pd, hipLaunchKernelGGL((k_build<PD, SPLAT_VD>), PLK_BUILD_ARGS))
    switch (splat_vd) {
        case 0: PLK_BUILD(0); break;
        case 2: PLK_BUILD(2); break;
        case 3: PLK_BUILD(3); break;
        case 4: PLK_BUILD(4); break;
        default: return hipErrorInvalidValue;
    }
#undef PLK_BUILD
#undef PLK_BUILD_ARGS
    return hipGetLastError();
}

hipError_t build_f64(int pd, const Points64 &points, const PointMap &map, uint64_t *cell_keys,
                     uint32_t n_cells, Counters *counters, ReplayEntry *replay, int xcd_aware,
                     const CreatedLists &created_lists, const RegionSource &regions,
                     const InBuildNumbering *numbering, int splat_vd, const double *input,
                     int in_channels, double *cell_values, bool wide_keys, hipStream_t s) {
    if (map.n_blocks == 0) return hipSuccess;
    if (wide_keys && numbering) return hipErrorInvalidValue;
    const bool merge_in_workgroup = numbering != nullptr;
    if (map.mode == 1 && (!merge_in_workgroup || !map.order || !map.n_tiles)) return hipErrorInvalidValue;
    const InBuildNumbering in_build = numbering ? *numbering : InBuildNumbering{};
    if (splat_vd && !merge_in_workgroup) return hipErrorInvalidValue;
#define PLK_BUILD_ARGS                                                                             \
    dim3(map.n_blocks), dim3(kBlock), 0, s, PointFeatures{}, map, ScaleFactor{}, cell_keys,        \
        n_cells - 1u, counters, replay, xcd_aware, (const void *)input, in_channels,               \
        (void *)cell_values, created_lists, points, regions
#define PLK_BUILD(SPLAT_VD)                                                                        \
    PLK_DISPATCH_PD(pd, hipLaunchKernelGGL((k_build_tile<PD, SPLAT_VD, double>), PLK_BUILD_ARGS,  \
                                           in_build))
    if (merge_in_workgroup) {
        switch (splat_vd) {
            case 0: PLK_BUILD(0); break;
            case 2: PLK_BUILD(2); break;
            case 3: PLK_BUILD(3); break;
            case 4: PLK_BUILD(4); break;
            default: return hipErrorInvalidValue;
        }
    } else if (wide_keys) {
        PLK_DISPATCH_WIDE_PD(pd, hipLaunchKernelGGL((k_build<PD, 0, double, true>), PLK_BUILD_ARGS))
    } else {
        PLK_DISPATCH_PD(pd, hipLaunchKernelGGL((k_build<PD, 0, double>), PLK_BUILD_ARGS))
    }
#undef PLK_BUILD
#undef PLK_BUILD_ARGS
    return hipGetLastError();
}

hipError_t number_vertices(int pd, const PointMap &map, const CreatedLists &lists,
                           int *next_chunk_count, unsigned n_chunks, const VertexTables &vertices,
                           float *values,
                           int vd, float *cell_values, Counters *counters, Counters *next_counters,
                           HostReport host_report, bool wide_keys, hipStream_t s) {
    if (map.n_blocks == 0) return hipErrorInvalidValue;
    if (wide_keys) {
        PLK_DISPATCH_WIDE_PD(pd, hipLaunchKernelGGL((k_number_vertices<PD + 1, true>), dim3(map.n_blocks),
                                               dim3(64), 0, s, lists, next_chunk_count, n_chunks,
                                               vertices, values, vd, cell_values, counters,
                                               next_counters, host_report));
    } else {
        PLK_DISPATCH_PD(pd, hipLaunchKernelGGL((k_number_vertices<PD + 1>), dim3(map.n_blocks),
                                               dim3(64), 0, s, lists, next_chunk_count, n_chunks,
                                               vertices, values, vd, cell_values, counters,
                                               next_counters, host_report));
    }
    return hipGetLastError();
}

hipError_t neighbours(int pd, const VertexTables &vertices, const Counters *counters,
                      const uint64_t *cell_keys, uint32_t n_cells, int launch_vertices,
                      const CreatedLists *foreign_rows, unsigned n_lists, void *values, int vd,
                      bool values_are_double, Counters *report, Counters *next_counters,
                      HostReport host_report, bool wide_keys, hipStream_t s) {
    if (vertices.max_vertices <= 0) return hipErrorInvalidValue;
    const size_t items = (size_t)(pd + 1) * (size_t)launch_vertices;
    const unsigned foreign_blocks =
        foreign_rows ? (blocks_for(n_lists, kBlock / 64) + kXcds - 1u) / kXcds * kXcds : 0u;
#define PLK_NEIGHBOURS(WIDE, DISPATCH)                                                             \
    DISPATCH(pd, hipLaunchKernelGGL((k_neighbours<PD, WIDE>),                                      \
                                           dim3(foreign_blocks + vertex_blocks(items)),            \
                                           dim3(kBlock), 0, s, vertices, counters, cell_keys,      \
                                           n_cells - 1u, foreign_blocks,                           \
                                           foreign_rows ? *foreign_rows : CreatedLists{}, n_lists, \
                                           values, vd, values_are_double ? 1 : 0, report,          \
                                           next_counters, host_report))
    if (wide_keys) {
        PLK_NEIGHBOURS(true, PLK_DISPATCH_WIDE_PD);
    } else {
        PLK_NEIGHBOURS(false, PLK_DISPATCH_PD);
    }
#undef PLK_NEIGHBOURS
    return hipGetLastError();
}

hipError_t fill_zero(float *p, size_t n, hipStream_t s) {
    if (n == 0) return hipSuccess;
    hipLaunchKernelGGL(k_fill_zero, dim3(blocks_for(n)), dim3(kBlock), 0, s, p, n);
    return hipGetLastError();
}

hipError_t splat(int pd, int vd, const PointMap &map, const float *input, int in_channels,
                 ReplayEntry *replay, const int *cell_vertex, float *values,
                 int xcd_aware, hipStream_t s) {
    if (map.n_blocks == 0) return hipSuccess;
    const dim3 grid(map.n_blocks), block(kBlock);
#define PLK_SPLAT_DPP(VD)                                                                         \
    case VD:                                                                                      \
        PLK_DISPATCH_PD(pd, hipLaunchKernelGGL((k_splat_dpp<VD, PD + 1>), grid, block, 0, s, map, \
                                               input, in_channels, replay,                        \
                                               cell_vertex, values, xcd_aware));                  \
        break;
    switch (vd) {
        PLK_SPLAT_DPP(2) PLK_SPLAT_DPP(3) PLK_SPLAT_DPP(4)
        default:
            if (in_channels >= 1 && in_channels <= 64) {
                const size_t lds = sizeof(float) * kBlock * (size_t)in_channels;
                const dim3 grid2(map.n_blocks, (pd + 2) / 2);
                if (vd <= 16)
                    hipLaunchKernelGGL(k_splat_channels<16>, grid2, block, lds, s, pd + 1, vd, map, input,
                                       in_channels, replay, cell_vertex, values, xcd_aware);
                else if (vd <= 32)
                    hipLaunchKernelGGL(k_splat_channels<32>, grid2, block, lds, s, pd + 1, vd, map, input,
                                       in_channels, replay, cell_vertex, values, xcd_aware);
                else
                    hipLaunchKernelGGL(k_splat_channels<64>, grid2, block, lds, s, pd + 1, vd, map, input,
                                       in_channels, replay, cell_vertex, values, xcd_aware);
                break;
            }
            PLK_DISPATCH_PD(pd, hipLaunchKernelGGL(k_splat_dpp_blocks<PD + 1>, grid, block, 0, s, vd,
                                                   map, input, in_channels, replay,
                                                   cell_vertex, values, xcd_aware));
            break;
    }
#undef PLK_SPLAT_DPP
    return hipGetLastError();
}

hipError_t blur_axis(int vd, const Counters *counters, int max_vertices, const float *src, float *dst,
                     const int2 *nbr, uint64_t *reset_cell_keys, const int *vertex_cell,
                     int launch_vertices, hipStream_t s) {
    if (max_vertices <= 0) return hipSuccess;
#define PLK_BLUR_ROW(VD)                                                                          \
    case VD:                                                                                      \
        hipLaunchKernelGGL(k_blur_row<VD>, dim3(vertex_blocks((size_t)launch_vertices)),          \
                           dim3(kBlock), 0, s, counters, max_vertices,                            \
                           reinterpret_cast<const ValueRow<VD> *>(src),                           \
                           reinterpret_cast<ValueRow<VD> *>(dst), nbr, reset_cell_keys,           \
                           vertex_cell);                                                          \
        return hipGetLastError();
    switch (vd) {
        PLK_BLUR_ROW(2) PLK_BLUR_ROW(3) PLK_BLUR_ROW(4)
        default: break;
    }
#undef PLK_BLUR_ROW
    hipLaunchKernelGGL(k_blur_element<float>, dim3(vertex_blocks((size_t)launch_vertices * vd)), dim3(kBlock), 0, s,
                       counters, max_vertices, vd, src, dst, nbr, reset_cell_keys, vertex_cell);
    return hipGetLastError();
}

hipError_t blur_two_axes(int vd, const Counters *counters, int max_vertices, const float *src,
                         float *dst, const int2 *nbr_first, const int2 *nbr_second,
                         uint64_t *reset_cell_keys, const int *vertex_cell, int launch_vertices,
                         hipStream_t s) {
    if (max_vertices <= 0) return hipSuccess;
#define PLK_BLUR2_ROW(VD)                                                                         \
    case VD:                                                                                      \
        hipLaunchKernelGGL(k_blur2_row<VD>, dim3(vertex_blocks((size_t)launch_vertices)),         \
                           dim3(kBlock), 0, s, counters, max_vertices,                            \
                           reinterpret_cast<const ValueRow<VD> *>(src),                           \
                           reinterpret_cast<ValueRow<VD> *>(dst), nbr_first, nbr_second,          \
                           reset_cell_keys, vertex_cell);                                         \
        return hipGetLastError();
    switch (vd) {
        PLK_BLUR2_ROW(2) PLK_BLUR2_ROW(3) PLK_BLUR2_ROW(4)
        default: break;
    }
#undef PLK_BLUR2_ROW
    hipLaunchKernelGGL(k_blur2_element<float>, dim3(vertex_blocks((size_t)launch_vertices * vd)), dim3(kBlock), 0, s,
                       counters, max_vertices, vd, src, dst, nbr_first, nbr_second, reset_cell_keys,
                       vertex_cell);
    return hipGetLastError();
}

// The blur of a lattice of doubles: the same kernels over the value type.
hipError_t blur_axis_f64(int vd, const Counters *counters, int max_vertices, const double *src,
                              double *dst, const int2 *nbr, uint64_t *reset_cell_keys,
                              const int *vertex_cell, int launch_vertices, hipStream_t s) {
    if (max_vertices <= 0) return hipSuccess;
#define PLK_BLUR_ROW(VD)                                                                          \
    case VD:                                                                                      \
        hipLaunchKernelGGL((k_blur_row<VD, double>), dim3(vertex_blocks((size_t)launch_vertices)), \
                           dim3(kBlock), 0, s, counters, max_vertices,                            \
                           reinterpret_cast<const ValueRow<VD, double> *>(src),                   \
                           reinterpret_cast<ValueRow<VD, double> *>(dst), nbr, reset_cell_keys,   \
                           vertex_cell);                                                          \
        return hipGetLastError();
    switch (vd) {
        PLK_BLUR_ROW(2) PLK_BLUR_ROW(3) PLK_BLUR_ROW(4)
        default: break;
    }
#undef PLK_BLUR_ROW
    hipLaunchKernelGGL(k_blur_element<double>, dim3(vertex_blocks((size_t)launch_vertices * vd)),
                       dim3(kBlock), 0, s, counters, max_vertices, vd, src, dst, nbr,
                       reset_cell_keys, vertex_cell);
    return hipGetLastError();
}

hipError_t blur_two_axes_f64(int vd, const Counters *counters, int max_vertices,
                                  const double *src, double *dst, const int2 *nbr_first,
                                  const int2 *nbr_second, uint64_t *reset_cell_keys,
                                  const int *vertex_cell, int launch_vertices, hipStream_t s) {
    if (max_vertices <= 0) return hipSuccess;
#define PLK_BLUR2_ROW(VD)                                                                         \
    case VD:                                                                                      \
        hipLaunchKernelGGL((k_blur2_row<VD, double>), dim3(vertex_blocks((size_t)launch_vertices)), \
                           dim3(kBlock), 0, s, counters, max_vertices,                            \
                           reinterpret_cast<const ValueRow<VD, double> *>(src),                   \
                           reinterpret_cast<ValueRow<VD, double> *>(dst), nbr_first, nbr_second,  \
                           reset_cell_keys, vertex_cell);                                         \
        return hipGetLastError();
    switch (vd) {
        PLK_BLUR2_ROW(2) PLK_BLUR2_ROW(3) PLK_BLUR2_ROW(4)
        default: break;
    }
#undef PLK_BLUR2_ROW
    hipLaunchKernelGGL(k_blur2_element<double>, dim3(vertex_blocks((size_t)launch_vertices * vd)),
                       dim3(kBlock), 0, s, counters, max_vertices, vd, src, dst, nbr_first,
                       nbr_second, reset_cell_keys, vertex_cell);
    return hipGetLastError();
}

bool blur_can_take_three_axes(int vd) { return vd >= 2 && vd <= 4; }

template <typename S>
static hipError_t blur_three_axes_of(int vd, const Counters *counters, int max_vertices, const S *src,
                                     S *dst, const int2 *nbr_first, const int2 *nbr_second,
                                     const int2 *nbr_third, uint64_t *reset_cell_keys,
                                     const int *vertex_cell, int launch_vertices, hipStream_t s) {
    if (max_vertices <= 0) return hipSuccess;
#define PLK_BLUR3_ROW(VD)                                                                         \
    case VD:                                                                                      \
        hipLaunchKernelGGL((k_blur3_row<VD, S>), dim3(vertex_blocks((size_t)launch_vertices)),    \
                           dim3(kBlock), 0, s, counters, max_vertices,                            \
                           reinterpret_cast<const ValueRow<VD, S> *>(src),                        \
                           reinterpret_cast<ValueRow<VD, S> *>(dst), nbr_first, nbr_second,       \
                           nbr_third, reset_cell_keys, vertex_cell);                              \
        return hipGetLastError();
    switch (vd) {
        PLK_BLUR3_ROW(2) PLK_BLUR3_ROW(3) PLK_BLUR3_ROW(4)
        default: return hipErrorInvalidValue;
    }
#undef PLK_BLUR3_ROW
}
hipError_t blur_three_axes(int vd, const Counters *counters, int max_vertices, const float *src,
                           float *dst, const int2 *nbr_first, const int2 *nbr_second,
                           const int2 *nbr_third, uint64_t *reset_cell_keys, const int *vertex_cell,
                           int launch_vertices, hipStream_t s) {
    return blur_three_axes_of<float>(vd, counters, max_vertices, src, dst, nbr_first, nbr_second,
                                     nbr_third, reset_cell_keys, vertex_cell, launch_vertices, s);
}
hipError_t blur_three_axes_f64(int vd, const Counters *counters, int max_vertices, const double *src,
                               double *dst, const int2 *nbr_first, const int2 *nbr_second,
                               const int2 *nbr_third, uint64_t *reset_cell_keys,
                               const int *vertex_cell, int launch_vertices, hipStream_t s) {
    return blur_three_axes_of<double>(vd, counters, max_vertices, src, dst, nbr_first, nbr_second,
                                      nbr_third, reset_cell_keys, vertex_cell, launch_vertices, s);
}

hipError_t slice(int pd, int vd, const PointMap &map, const ReplayEntry *replay,
                 const int *cell_vertex, const float *values,
                 float *output, int normalize, hipStream_t s) {
    if (map.n_blocks == 0) return hipSuccess;
    const int d1 = pd + 1;
    const dim3 grid(map.n_blocks), block(kBlock);
    const size_t T = (size_t)map.n_blocks * kBlock;
#define PLK_SLICE(VD)                                                                          \
    case VD:                                                                                   \
        hipLaunchKernelGGL(k_slice_point<VD>, grid, block, 0, s, d1, map, replay,              \
                           cell_vertex, values, output, normalize);                            \
        break;
#define PLK_SLICE_ROWS(VD)                                                                     \
    case VD:                                                                                   \
        PLK_DISPATCH_PD(pd, hipLaunchKernelGGL((k_slice_point<VD, PD + 1>), grid, block, 0, s, \
                                               d1, map, replay, cell_vertex, values, output,   \
                                               normalize));                                    \
        break;
    switch (vd) {
        PLK_SLICE_ROWS(2) PLK_SLICE_ROWS(3) PLK_SLICE_ROWS(4)
        PLK_SLICE(5) PLK_SLICE(6) PLK_SLICE(7) PLK_SLICE(8)
        default: {
            const int out_ch = normalize ? vd - 1 : vd;
#define PLK_SLICE_QUADS(L)                                                                      \
    PLK_DISPATCH_PD(pd, hipLaunchKernelGGL((k_slice_quads<PD + 1, L>),                          \
                                           dim3(map.n_blocks, L / kSlicePoints),                \
                                           block, 0, s, vd, map, T, replay, values, output,     \
                                           normalize))
            if (vd <= 16) {
                PLK_SLICE_QUADS(4);
                break;
            } else if (vd <= 32) {
                PLK_SLICE_QUADS(8);
                break;
            } else if (vd <= 64) {
                PLK_SLICE_QUADS(16);
                break;
            }
#undef PLK_SLICE_QUADS
            PLK_DISPATCH_PD(pd, hipLaunchKernelGGL((k_slice_channels<PD + 1>),
                                                   dim3(map.n_blocks, (out_ch + kSliceRun - 1) / kSliceRun), block, 0, s,
                                                   vd, map, T, replay, values, output, normalize));
        } break;
    }
#undef PLK_SLICE
#undef PLK_SLICE_ROWS
    return hipGetLastError();
}

hipError_t slice_rows_f64(int pd, int vd, const PointMap &map, const ReplayEntry *replay,
                          const double *weights, const int *cell_vertex, const double *values,
                          double *output, int normalize, hipStream_t s) {
    if (map.n_blocks == 0) return hipSuccess;
    const dim3 grid(map.n_blocks), block(kBlock);
#define PLK_SLICE_ROWS(VD)                                                                     \
    case VD:                                                                                   \
        PLK_DISPATCH_PD(pd, hipLaunchKernelGGL((k_slice_rows_f64<VD, PD + 1>), grid, block, 0, \
                                               s, map, replay, weights, cell_vertex, values,   \
                                               output, normalize));                            \
        break;
    switch (vd) {
        PLK_SLICE_ROWS(2) PLK_SLICE_ROWS(3) PLK_SLICE_ROWS(4)
        default: return hipErrorInvalidValue;
    }
#undef PLK_SLICE_ROWS
    return hipGetLastError();
}

hipError_t debug_simplex(int pd, const float *positions, int N, const ScaleFactor &scale,
                         short *rem0, short *rank, short *keys, float *barycentric, hipStream_t s) {
    if (N <= 0) return hipSuccess;
    PLK_DISPATCH_PD(pd, hipLaunchKernelGGL(k_debug_simplex<PD>, dim3(blocks_for((size_t)N)),
                                           dim3(kBlock), 0, s, positions, N, scale, rem0, rank, keys,
                                           barycentric));
    return hipGetLastError();
}

hipError_t export_keys(int pd, const uint64_t *vertex_keys, const VertexNumbers &numbers, short *keys,
                       bool wide_keys, hipStream_t s) {
    const unsigned M = numbers.total;
    if (M == 0) return hipSuccess;
    if (wide_keys) {
        PLK_DISPATCH_WIDE_PD(pd, hipLaunchKernelGGL((k_export_keys<PD, true>), dim3(blocks_for((size_t)M)),
                                               dim3(kBlock), 0, s, vertex_keys, numbers, keys));
    } else {
        PLK_DISPATCH_PD(pd, hipLaunchKernelGGL((k_export_keys<PD, false>), dim3(blocks_for((size_t)M)),
                                               dim3(kBlock), 0, s, vertex_keys, numbers, keys));
    }
    return hipGetLastError();
}

hipError_t export_values(const float *values, int words, const VertexNumbers &numbers, float *out,
                         hipStream_t s) {
    const size_t n = (size_t)numbers.total * words;
    if (n == 0) return hipSuccess;
    hipLaunchKernelGGL(k_export_values, dim3(blocks_for(n)), dim3(kBlock), 0, s, values, words,
                       numbers, out);
    return hipGetLastError();
}

hipError_t export_replay(int pd, const PointMap &map, const ReplayEntry *replay,
                         const int *cell_vertex, const VertexNumbers &numbers, int *vertex,
                         float *weight, hipStream_t s) {
    if (map.n_blocks == 0) return hipSuccess;
    hipLaunchKernelGGL(k_export_replay, dim3(map.n_blocks), dim3(kBlock), 0, s, pd + 1, map,
                       replay, cell_vertex, numbers, vertex, weight);
    return hipGetLastError();
}

hipError_t guess_grid(const float *positions, int N, int pd, GridGuess *guess, hipStream_t s) {
    if (N < 2) return hipErrorInvalidValue;
    // *guess must hold {N, N} and 0 (set by the caller)
    hipLaunchKernelGGL(k_first_changes, dim3(blocks_for((size_t)N - 1)), dim3(kBlock), 0, s, positions,
                       N, pd, guess);
    hipLaunchKernelGGL(k_check_periods, dim3(blocks_for((size_t)N - 1)), dim3(kBlock), 0, s, positions,
                       N, pd, guess);
    return hipGetLastError();
}

hipError_t compute_positions(const float *reference, float *positions, int N, int n_ref_channels,
                             int n_spatial_dims, const SpatialDims &dims, float spatial_std,
                             float feature_std, hipStream_t s) {
    if (N <= 0) return hipSuccess;
    hipLaunchKernelGGL(k_positions, dim3(blocks_for((size_t)N)), dim3(kBlock), 0, s, reference,
                       positions, N, n_ref_channels, n_spatial_dims, dims, spatial_std, feature_std);
    return hipGetLastError();
}

}  // namespace plk
