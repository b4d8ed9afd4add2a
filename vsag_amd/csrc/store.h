// Device-resident code store: quantizer state + codes re-tiled for wave64 streaming.
//
// HBM layout.  Codes are grouped into tiles of 64.  A tile is G rows of 1 KiB; row j holds bytes
// [16j, 16j+16) of each of the 64 codes, lane-major, so one global_load_dwordx4 per lane reads a whole
// row fully coalesced and every lane ends up with the bytes of "its" code.  Only the leading
// payload_bytes of a reference code (the part the distance loop consumes) go into the tiles; trailing
// per-code scalars (norms, sums, RaBitQ factors) are kept as structure-of-arrays words in `meta`.
// A flat store maps tile t, lane l to inner id 64 t + l.  A posting-list store pads every list to whole
// tiles and keeps an explicit inner-id array in the same tile order.
#pragma once

#include <vector>

#include "common.h"

// A metadata word that is no field of the reference code but the sum of its payload bytes, formed when the code is
// re-tiled (sq8_uniform: the int8 matrix cores take code and query centred by 128, and putting the product right
// needs the plain sum of the code values next to the scalar the code carries).
constexpr uint32_t kMetaPayloadSum = 0xFFFFFFFFU;

struct vsag_amd_store {
    int kind = 0;
    int metric = 0;
    uint32_t dim = 0;
    int query_bits = 4;          // rabitq: 4 or 32
    uint32_t base_bits = 1;      // rabitq: bits per dimension of the base code (more than 1: fp32 queries only)

    uint32_t code_size = 0;      // bytes per code in the reference layout
    uint32_t payload_bytes = 0;  // leading bytes consumed by the distance loop
    uint32_t G = 0;              // 16-byte granules per code
    // The payload as planes: `planes` runs of plane_bytes source bytes, each padded to plane_granules granules in the
    // tiles (multi-bit rabitq: one run per bit plane; every other kind: one run, the whole payload).
    uint32_t planes = 1;
    uint32_t plane_bytes = 0;
    uint32_t plane_granules = 0;
    uint32_t dpad = 0;           // dims covered by G granules (per-dim tables are this long)
    // Scan settings of this store; the values below follow the process-wide ones (vsag_amd_set_scan_contraction /
    // vsag_amd_set_scan_tuning).
    int contraction_mode = -2;
    int tile_override = -1;
    int chunk_override = -1;

    uint32_t nmeta = 0;          // 4-byte metadata words per code
    uint32_t meta_offset[4] = {0, 0, 0, 0};  // byte offsets of those words in the reference code
                                             // (kMetaPayloadSum: no field of the code, see below)
    uint32_t meta_is_u64 = 0;    // bit m set: word m is a u64 in the reference code, kept as float
    bool stored_codes = false;   // appended codes come out of a serialized index: fp32 + cosine rows are unit already

    // quantizer state
    float* scale_dev = nullptr;  // sq8/sq4: diff[d]/levels, zero beyond dim
    float* lb_dev = nullptr;     // sq8/sq4: lower bound, zero beyond dim
    float* diff_dev = nullptr;   // sq8/sq4: diff (kept for encoders)
    float ulb = 0, udiff = 0, scalar_rate = 0;  // uniform kinds
    float* bounds_dev = nullptr;                // uniform kinds: {lb, diff}
    float* rotation_dev = nullptr;              // rabitq
    float* centroid_dev = nullptr;              // rabitq
    uint32_t pq_dim = 0;                        // pqfs: subspaces
    float* codebooks_dev = nullptr;             // pqfs: pq_dim x 16 x (dim / pq_dim)

    // codes
    uint4* tiles = nullptr;
    uint32_t* meta = nullptr;    // nmeta arrays of cap_tiles*64 words
    uint64_t cap_tiles = 0;
    uint64_t ntiles = 0;
    uint64_t n = 0;

    // posting lists (nlist == 0: flat store).  Every list owns a run of tiles with some room behind the tiles it
    // uses, so that codes can be appended in place; a list that outgrows its room moves all lists once.
    uint32_t nlist = 0;
    uint32_t* ids_dev = nullptr;         // inner id per tile slot, VSAG_AMD_INVALID_ID in padding
    uint32_t* list_tile_dev = nullptr;   // 2 * nlist: first tile of list l at [2 l], end of its used tiles at [2 l + 1]
    std::vector<uint32_t> list_sizes;    // codes per list
    uint32_t* list_sizes_dev = nullptr;  // the same on the device
    std::vector<uint32_t> list_begin;    // first tile per list
    std::vector<uint32_t> list_room;     // tiles of room per list
    uint32_t max_list_tiles = 0;         // used tiles of the longest list
    uint32_t* slot_of_id_dev = nullptr;  // tile slot of every inner id (the reference's location_map_, ivf.h:300-306)
    uint64_t slot_of_id_cap = 0;
    // use_residual (bucket_datacell.h:527-572,612-639): per slot -2 <c, decoded> - |c|^2 of its list's centroid c
    // (l2 only, else null) and the centroids the codes are residuals of.
    float* residual_bias_dev = nullptr;
    float* residual_centroids_dev = nullptr;  // nlist x dim, null: no residual
    float residual_cmax = 0.0F;               // the largest norm among those centroids (rounded up)

    // flat fp32 / sq8 stores: per slot |y|^2 and the largest |y| (float bits) of the code as the batched
    // contraction sees it, kept up to date by append
    // Flat stores the matrix cores pre-select on: the codes once more, a row per code (G granules in a run), for the
    // rescoring of scattered candidates -- one or two memory lines per candidate instead of one per granule.
    // With metadata words (nmeta > 0) a row is one granule longer: the code's words, so that a candidate is one run of
    // memory (row_granules = G or G + 1).
    uint4* rows = nullptr;
    uint32_t row_granules = 0;
    float* pf_term = nullptr;
    uint32_t* pf_ymax = nullptr;
    // 1-bit rabitq stores with 4-bit queries (l2 / ip, at most kRbMaxG granules, no residual), flat or lists: the code
    // bits once more as the fp4 operand of the matrix cores wants them (prefilter_rb.hip).  f4tiles[(tile G + g) 64 +
    // lane], lane = 32 h + r: dwords 4 g + h and 4 g + 2 + h of code r of the tile (x, y) and of code 32 + r (z, w),
    // each with bit 8 v + j of the code's dword moved to bit 4 j + v, so that ((w >> v) << 1) & 0x22222222 is register
    // v of the operand (elements 8 v .. 8 v + 7 as fp4 1.0 or 0).  f4const: per slot the three constants the pass
    // takes from a code's factors and two flags as the bits of w (1: the slot holds a code, 2: the code stands outside
    // the pass and is a candidate of every query).  f4group: per tile and group of sixteen codes (those whose verdicts
    // share a lane: 32 i + 8 gq + 4 h + j of group 2 i + h) the centre and half width of the first constant, the least
    // second, the centre and half width of the third, in two float4.  Flat stores keep all of it up to date in append;
    // posting lists renew it over all cap_tiles when codes are added (f4_slots = their room).
    uint4* f4tiles = nullptr;
    float4* f4const = nullptr;
    float4* f4group = nullptr;
    uint64_t f4_slots = 0;
    // sq8 / sq4 posting lists of at most 128 dimensions keep the same per-slot term (over all cap_tiles * 64 slots, renewed
    // when codes are added) for the int8 pass over lists; pf_term_slots = the slots pf_term has room for there.
    uint64_t pf_term_slots = 0;
};

namespace vsag_amd {

// Query-side table geometry of one store kind (what the prepare kernel writes per query).
constexpr uint32_t kRbMaxG = 8;  // granules per code (1024 dimensions) of the rabitq matrix-core pass
// Largest per-code factors the fp32 threshold of that pass takes (A_c, |B_c| of prefilter_rb.hip; codes beyond them stand
// outside the pass, as candidates of every query): the per-query slack there is sized for them.  The second grows with
// the square of the data's scale (norm x error factor / 2).
constexpr float kRbMaxA = 64.0F;
constexpr float kRbMaxB = 4096.0F;

struct QueryLayout {
    uint32_t qstride;  // 4-byte words per query in the main table
    uint32_t qmeta;    // floats per query in the scalar table
};

QueryLayout query_layout(const vsag_amd_store* s);
// Device bytes prepare_queries needs behind its `qcodes` pointer for nq queries: the encoded queries of the kinds
// that encode them, then whatever their encoders use as scratch.
size_t query_staging_bytes(const vsag_amd_store* s, uint64_t nq);
// The bits word of the rabitq entry points for a store: query bits plus 256 * base bits for multi-bit base codes.
inline int
rabitq_bits_word(const vsag_amd_store* s) {
    return s->query_bits | (s->base_bits > 1 ? static_cast<int>(s->base_bits) << 8 : 0);
}
int launch_code_terms(vsag_amd_store* s, uint64_t first, uint64_t count, hipStream_t st);

}  // namespace vsag_amd
