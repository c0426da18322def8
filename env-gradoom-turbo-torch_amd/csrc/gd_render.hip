// MI355X (gfx950) batched software renderer + observation pipeline.
//
// One frame for N lanes runs as a short chain of kernels on the caller's stream:
//
//   lane_setup      1 thread / lane           view basis, pitch centre, camera sector
//   lane_tables     1 thread / (lane, row)    per-lane distance bounds of every height level, plane rows, row slopes
//   wall_setup      1 wave-slot / (lane,wall) FWallCoords span+depths, span ownership bounds, the linedef's
//                                             entry in the candidate list of every column it can own, and the
//                                             nearest blocking hit of every column (64-bit atomicMin)
//   strip_key/order 1 thread / 64-col strip   longest strip first (counting sort on the blocking distance)
//   wall_select     1 wave / strip            portal traversal: which drawseg every column pass selects, one record each
//   wall_raster     1 wave / strip            the recorded passes drawn: projection, clips, tiers, planes, masked mid-textures
//   plane_shade     1 thread / 12 pixels      flat texel + light for every pixel a plane of the wall pass shows,
//                                             the wall tiers' palette indices
//   flat_list       128 threads / lane        per-pixel plane rays (fine point raster) for the listed gap pixels
//   flat_span_select, flat_tail, flat_span_finish
//                                             visplane repair of the rows where a gap pixel stayed unresolved
//   flat_shade      128 threads / lane        the gap pixels' flats
//   decal           320 threads / lane        bullet chips on the wall tiers they hit (frames that carry decals
//                                             also keep a per-pixel scene depth: wall_raster<true>, plane_shade<true>)
//   sprite_columns  320 threads / lane        billboards far -> near, opaque / additive / translucent
//   weapon_overlay, hud                       player weapon, muzzle flash and status bar patches
//   observe         1 thread / obs pixel      PLAYPAL + exact area pool + gray + 4-frame stack
//   expand_rgb      1 thread / pixel          PLAYPAL expansion for callers that want RGB24 frames
//
// All fixed-point arithmetic is int64 like the reference's Torch code; float32
// expressions are evaluated operation by operation (-ffp-contract=off) so that
// palette-index frames are bit-identical to the reference.  Citations name
// /root/reference/src/gradoom/engine.py unless stated otherwise.

#include <hip/hip_runtime.h>

#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstring>
#include <map>
#include <new>
#include <string>
#include <type_traits>
#include <vector>

#include "../../include/gradoom_amd.h"

namespace {

typedef long long i64;
typedef unsigned long long u64;

#define SW 320
#define VH 208
#define CAND_MAX 64          // candidate linedefs a screen column keeps in its own slots
// A column whose ray can reach more than CAND_MAX linedefs (a long corridor seen end on) gets a slot in the chunk's spill
// pool, where cand_spill_kernel lists all of them, up to SPILL_DEPTH.  The pool continues the candidate blocks with
// the same layout (entry k of a column lies k * 320 entries on), SPILL_DEPTH x 320 entries per pool block, so a
// spilled column differs from the others only in where its list starts and how long it may be.
#define SPILL_DEPTH 256
#define SPILL_SHIFT 12       // cand_count of a spilled column: entries | (pool slot + 1) << SPILL_SHIFT
static_assert(SPILL_DEPTH < (1 << SPILL_SHIFT), "a spilled column's count and its pool slot share a word");
#define SEG_COLS 64           // columns of a traversal segment; a wavefront takes 64 / SEG_COLS segments, of any lanes
#define SEGS_PER_LANE (SW / SEG_COLS)
#define GD_INF __builtin_inff()

// engine.py:42-51, 139-156
#define FIXED_UNIT 65536LL
#define UINT32_MASK 0xFFFFFFFFLL
#define FINE_ANGLES 8192
#define ANGLE_90 (1LL << 30)
#define FOCAL_X_FIXED (160LL * 65536LL)
#define Y_ASPECT_FIXED ((320LL * 65536LL * 240LL) / (200LL * 320LL))
#define FOCAL_Y_FIXED (160LL * Y_ASPECT_FIXED)
#define FLOOR_VISIBILITY_FIXED ((160LL * 65536LL * (8LL * 65536LL)) / FOCAL_Y_FIXED)
#define WALL_VISIBILITY_FIXED (((FOCAL_Y_FIXED * (320LL * 600LL) / (320LL * 240LL * 3LL)) * (8LL * 65536LL)) >> 16)
#define SPRITE_MIN_DEPTH_FIXED 8192LL

// candidate flags
#define CF_GEO 1
#define CF_PROJ 2
#define CF_LEDGE 4
#define CF_ALONG_HI 8   // along > 0.5: the ray is nearer the linedef's end vertex
#define CF_FF 16        // camera on the front side of the linedef (float32 test)
#define CF_MASKED 32    // candidate entries only: the side facing the camera carries a masked mid-texture

// wall record flags
#define WF_HC 1        // owns at least one column after every span test
#define WF_FF 2        // front facing (float32 test of engine.py:11376-11381)
#define WF_SUBPIXEL 4  // two-sided and at most one column wide (engine.py:11589-11591)
#define WF_ANYGEO 8    // some column ray hits the segment
#define WF_SPLIT 16    // projects through BSP fragments (engine.py:11472-11545, 12310-12380)

struct LaneCtx {
    float x, y, view_z, pitch_offset, fsin, fcos;
    i64 view_x_fixed, view_y_fixed, vsin, vcos, center_fixed, flash_light;
    i64 upper_clip, lower_clip;   // OWallMost's view-frustum slopes at the top and bottom row (engine.py:12402-12413)
    int sector;
    int last_ceiling_row;         // rows 0 .. last_ceiling_row of the view look at ceilings, the rest at floors (-1: all floors)
};

struct WallRec {   // one linedef seen from one lane
    int tx0, tx1, ty0, ty1;  // view-space endpoints, start then end (engine.py:11173-11205)
    i64 dl, dr;              // clipped endpoint depths (engine.py:10835-10852)
    i64 sl, sr;              // clipped half-open screen span (engine.py:10825-10868); a rejected
                             // linedef keeps whatever its projection produced, hence 64 bits
    short pl, pr;            // span used for ray ownership (engine.py:11347-11427), within [0, 320]
    int flags;
};

// What the selection half of a column pass hands to the drawing half (wall_select_kernel -> wall_raster_kernel): the
// drawseg the pass selected and, where a geometric portal path continues behind a projected solid
// (engine.py:12969-13069), that path.  `bits` holds the PB_* flags of the selection (they fit 16 bits).
struct __align__(16) PassRec {
    unsigned short wall, render_current, bits, ps_path;
    short ps_other;
    unsigned short spare;
    float distance;
};
#define PASS_MAX 255  // most column passes recorded per screen column (the count is a byte).  A chunk keeps room for as many as the
                      // map has sectors (a column runs at most that many passes), at least 16, at most PASS_MAX: Scratch::pass_slots.
                      // A column that needs more sets STATUS_PASS_OVERFLOW.

struct RecSpan {   // what a ray test of one linedef needs (eval_segment), kept for every linedef of the map; the full record
                   // above exists only for the linedefs the camera can see at all
    short pl, pr;
    int flags;
};

struct __align__(16) Cand {      // one linedef with a finite ray distance at one column, with the static
                   // linedef facts every scan needs packed in so that scans do no gathers
    unsigned short flags, wall;   // in this order: the entry's first word under its last is the key below
    short s0, s1;            // front / back sector (-1 = none)
    unsigned short v0, v1;   // vertex ids of start / end
    float dist;
};
// (distance, linedef, flags) of a candidate as one unsigned number.  Listed distances are positive, so their bit patterns
// order as they do: the smallest key is the nearest candidate, the lowest linedef on ties, which is how every scan of the
// traversal breaks them (no column lists a linedef twice).  CAND_KEY_NONE, greater than any entry's, stands for "none".
#define CAND_KEY_NONE 0x7F800000FFFFFFFFULL
__device__ __forceinline__ u64 cand_key(const Cand &q) { return ((u64)__float_as_uint(q.dist) << 32) | ((u64)q.wall << 16) | (u64)q.flags; }
__device__ __forceinline__ float cand_key_distance(u64 key) { return __uint_as_float((unsigned)(key >> 32)); }
__device__ __forceinline__ int cand_key_wall(u64 key) { return key == CAND_KEY_NONE ? 0x7fffffff : (int)((unsigned)key >> 16); }
__device__ __forceinline__ int cand_key_flags(u64 key) { return key == CAND_KEY_NONE ? 0 : (int)((unsigned)key & 0xFFFFu); }

struct Eval {      // distances/along/geometric/projected/left-edge of one linedef at one column;
                   // CF_ALONG_HI in flags carries (along > 0.5), the only use the traversal makes of along
    float dist;
    int flags;
};

struct DeviceMap {  // device copy of gd_map_desc (device pointers) + fixed tables
    gd_map_desc d;
    const i64 *fine_sine;     // [8192]
    const i64 *fine_tangent;  // [4096]
    const float *cosine_correction;  // [320] cos(native_ray_offsets), supplied by the host
    const float *inverse_cosine;     // [320] 1 / cosine_correction, correctly rounded
    float strip_reach_scale[SW / 64];// per 64-column strip: 1.001 / (its smallest cosine_correction), inf if not positive
    float strip_far_scale[SW / 64];  // per 64-column strip: 0.999 / (its largest cosine_correction), 0 if any is not positive
    float fine_inverse;              // 1 / fine_cell
    // Sectors grouped by plane level, floors (in floor_levels order) then ceilings: CSR over
    // floor_level_count + ceil_level_count rows into level_boxes, one padded bounding box
    // (x0, y0, x1, y1) per sector outside which no point tests inside that sector.
    const int *level_box_ofs;
    const float4 *level_boxes;
    // The coarse grid repacked for the crossing test of flat selection: per cell its item range, per
    // item one 16-byte record, per item edge a copy of the linedef's endpoints, so that a test is
    // three dependent loads (range, record, edges) instead of six.
    const int2 *cell_range;              // [cells] first item, one past the last
    const int4 *cell_item;               // [items] sector | GRID_ALWAYS_INSIDE, floor level index | ceiling level
                                         // index << 8 (or -1 when not recorded), first edge, one past the last
    const float4 *cell_edge;             // [item edges] x1, y1, x2, y2
    const int *wall_blocking_slot;       // [W] position of the linedef in blocking_walls, -1 when it does not block
    const unsigned int *sector_level;    // [S] index of the floor in floor_levels | index of the ceiling in ceil_levels << 16;
                                         // null when some sector's height is missing from the level lists
};

struct Overlays {   // device copy of gd_overlay_desc; count 0 = layer not loaded
    gd_overlay_desc d;
};

struct Scratch {    // per-chunk working memory, sized at create
    LaneCtx *ctx;          // [L]
    WallRec *rec;          // [L,W] written for the linedefs wall_setup_kernel does not cull; never read for the others
    RecSpan *span;         // [L,W] every linedef
    WallRec *frag_rec;     // [L,split_count,fragment_slots] FWallCoords of the BSP fragments of split linedefs
    float *scene_depth;    // [L,208,320] depth of the surface each pixel shows (engine.py:11553, 12700, 13411, 13740),
                           // kept only for frames that draw wall decals, else null
    Cand *cand;            // [L,CAND_MAX,320], then the spill pool [spill_slots / 320, SPILL_DEPTH, 320]
    int *cand_count;       // [L,320] entries listed (beyond CAND_MAX: the column wanted more than its own slots hold), or for
                           // a column with a pool slot: entries in the pool | (slot + 1) << SPILL_SHIFT
    int *spill_columns;    // [spill_slots] the columns (lane * 320 + column) that were given pool slots, in slot order
    int *spill_count;      // [1] columns that asked for a slot (cleared by lane_setup_kernel, counted by strip_key_kernel)
    unsigned spill_base;   // where the pool starts in `cand`, in entries
    int spill_slots;       // pool slots of this chunk (a multiple of 320)
    unsigned short *flat_sector;// [L,208,320]
    unsigned char *flat_flags;  // [L,208,320] bit0 unresolved
    int *flat_list;        // [L,FLAT_LIST_MAX] view pixels no wall tier, plane or masked texture covers: they show the
                           // flat pass's picture.  Listed by wall_raster_kernel, column by column.
    int *flat_list_count;  // [L] how many there are (more than FLAT_LIST_MAX: the lane is handled pixel by pixel)
    int *flat_tail;        // [L,2,320] per screen half and column: the sector of the first resolved pixel below the
                           // half's noted rows, -1 if the column was not looking for one or found none
    int *flat_span;        // [L,4] first / last row of the ceiling half, then of the floor half, that holds a shown
                           // pixel the flat pass could not resolve and whose repair reads its row (208, -1 = none):
                           // the rows the row repairs work on
    int *flat_rows;        // [L*208] the noted rows of every lane as one work list, entry = lane << 8 | row
    int *flat_row_count;   // [1] its length (cleared by lane_setup_kernel, filled by flat_rows_kernel)
    int *gap_columns;      // [L*2*320] the screen columns (of any lane, either half) that hold a shown pixel the flat pass
                           // could not resolve, as one work list: lane << 18 | half << 17 | topmost such row << 9 | column
    int *gap_column_count; // [1] its length (cleared by lane_setup_kernel, filled by flat_gap_column_kernel)
    int *flat_col_top;     // [L,2,320] per screen half and column: the topmost shown pixel the flat pass could not
                           // resolve (any value >= 208: none).  lane_tables_kernel sets "none", flat_gap_column_kernel
                           // lowers it while it selects the gap pixels.
    int pass_slots;        // passes a column can record in this chunk
    PassRec *pass_rec;     // [L,pass_slots,320] the drawsegs of each column's passes, in pass order
    float *pass_path_distance;  // [L,pass_slots,320] distance of the portal path of a pass that carries PB_PS_KEEPS (written for those only)
    unsigned char *pass_count;  // [L,320] passes recorded for the column: up to its last pass that draws or moves a clip
    unsigned int *meta;    // [L,208,320] filled | floor | plane_sector+1 | clip_wall+1
    float *clip_depth;     // [L,208,320]
    unsigned char *frame;  // [L,240,320] when the caller wants no indexed output
    u64 *block_hit;        // [L,320] nearest blocking linedef of the column ray: float bits of the distance << 32 |
                           // slot in blocking_walls, all ones when no ray hits (engine.py:10534-10557)
    int *lane_blends;      // [L] does some live billboard of the lane blend with the pixel below it (sprite_style other than -1)?
                           // lane_tables_kernel says; launch_chunk's two billboard launches split the lanes by it
    unsigned char *strip_key;  // [L*SEGS_PER_LANE] expected traversal length of each (lane, segment of SEG_COLS columns)
    int *strip_order;      // [L*SEGS_PER_LANE] segments, longest expected traversal first
    int *status;           // [1] sticky overflow flags
    float *level_reach;    // [L, floor levels + ceiling levels] lower bound of the distance from the
                           // camera to any point inside a sector with that plane level
    float *level_far;      // [L, floor levels + ceiling levels] upper bound of that distance
    unsigned int *level_masks;  // [L, LEVEL_BUCKETS, level_mask_words]: the plane levels a flat probe can reach at all, by
                                // bucket of the probe's distance scale (see level_bucket)
    i64 *level_plane;      // [L, floor levels + ceiling levels, 2] plane height (16.16) and its visibility factor
    i64 *row_slope;        // [L, 208] plane distance per unit of plane height on each view row
    i64 *step_scale;       // [L, 3, 2, 16] per log2 texture size (widths, then heights): the flat texture step per
                           // column, the fraction at screen column 0, the camera's offset
};
#define FLAT_LIST_MAX 1024 // listed gap pixels per lane (a gap is typically one column wide)
#define PLANE_LEVELS 32    // the per-lane plane tables of level lists up to this long (each) are staged in LDS by the
                           // shading kernels; longer lists are read where lane_tables_kernel left them

#define META_FILLED 0x80000000u   // an opaque wall tier owns the pixel; its palette index sits in the low byte of the
                                  // plane sector field (plane shading, which writes every other view pixel, stores it)
#define META_FLOOR 0x40000000u    // the owning plane is a floor
// which lanes a billboard or flat-shading launch takes (launch_chunk splits them by Scratch::lane_blends)
#define LANES_ALL 0
#define LANES_PLAIN 1
#define LANES_BLENDING 2
#define META_GAP_COVERED META_FLOOR   // in the word of a gap pixel (no tier, no plane, no masked texture: the bit above means nothing
                                  // there): a billboard was painted over it before the flat pass's pixels were, which flat_shade_kernel respects
#define META_MASKED 0x20000000u   // a masked mid-texture was drawn over the pixel
#define META_SECTOR_SHIFT 16
#define META_SECTOR_MASK 0x1FFFu  // plane sector + 1
#define META_WALL_MASK 0xFFFFu    // sprite-clip linedef + 1

#define STATUS_CAND_OVERFLOW 1
#define STATUS_PASS_OVERFLOW 2
#define SPAN_SELECT_BLOCKS 6144   // flat_span_select_kernel's grid: four times what 256 compute units hold at eight wavefronts per
                                  // SIMD, so that rows of unequal cost even out
#define STEP_TABLE 96   // int64 entries per lane of Scratch::step_scale

__device__ __forceinline__ i64 mul64(i64 a, i64 b) { return (i64)((u64)a * (u64)b); }
__device__ __forceinline__ i64 shl64(i64 a, int s) { return (i64)((u64)a << s); }
// a * b for a multiplier known to fit 32 unsigned bits: two 32-bit multiplies instead of three
__device__ __forceinline__ i64 mul64_u32(i64 a, unsigned b) { return (i64)((u64)a * (u64)b); }
// Bits 16..47 of a * b, all that `((a * b) >> 16) & 0xFFFFFFFF` ever looks at: the low words' full product, and of the
// two cross products only their low 16 bits, which 24-bit multiplies of the operands' low halves give at full rate.
__device__ __forceinline__ unsigned mul64_bits_16_47(i64 a, i64 b) {
    const unsigned al = (unsigned)a, ah = (unsigned)((u64)a >> 32), bl = (unsigned)b, bh = (unsigned)((u64)b >> 32);
    const u64 low = (u64)al * (u64)bl;
    const unsigned cross = __umul24(al & 0xFFFFu, bh & 0xFFFFu) + __umul24(ah & 0xFFFFu, bl & 0xFFFFu);
    return (unsigned)(low >> 16) + (cross << 16);
}
// C truncating division (engine.py:3115-3118).  gfx950 has no 64-bit integer divider; when both
// magnitudes are below 2^52 the quotient estimated in float64 is within one of the true quotient
// and one remainder check, also in float64, makes it exact.  Larger operands take the compiler's long division.
// The rare large-operand case is a compact shift-subtract loop rather than the compiler's
// unrolled long division, which would be replicated at every call site and push the kernels
// far past the instruction cache.
__device__ __forceinline__ u64 udiv_long(u64 n, u64 d) {
    u64 q = 0, r = 0;
#pragma unroll 1
    for (int i = 63; i >= 0; --i) {
        r = (r << 1) | ((n >> i) & 1);
        if (r >= d) { r -= d; q |= 1ULL << i; }
    }
    return q;
}
__device__ __forceinline__ i64 tdiv(i64 a, i64 b) {
    u64 ua = a < 0 ? (u64)0 - (u64)a : (u64)a;
    u64 ub = b < 0 ? (u64)0 - (u64)b : (u64)b;
    if (((ua | ub) >> 52) != 0 || ub == 0) {
        const u64 uq = ub == 0 ? 0 : udiv_long(ua, ub);
        return ((a < 0) != (b < 0)) ? -(i64)uq : (i64)uq;
    }
    // Both conversions are exact.  The rounded quotient, truncated, is the true quotient or one above it; the
    // remainder a - q * b is an integer below 2^53 in magnitude, so the fused multiply-add returns it exactly and its
    // sign tells which.  (The int64 product and compare this replaces cost three quarter-rate multiplies.)
    const double ad = fabs((double)a), bd = fabs((double)b);
    double q = trunc(ad / bd);
    const double r = __builtin_fma(-q, bd, ad);
    if (r < 0.0) q -= 1.0;
    else if (r >= bd) q += 1.0;
    if ((a < 0) != (b < 0)) q = -q;
    return (i64)q;
}
// Value of `v` in lane `lane` of the wavefront; `lane` must be the same in every active lane.
__device__ __forceinline__ int bcast(int v, int lane) { return __builtin_amdgcn_readlane(v, lane); }
__device__ __forceinline__ float bcast(float v, int lane) { return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), lane)); }
__device__ __forceinline__ i64 clampi(i64 v, i64 lo, i64 hi) { return v < lo ? lo : (v > hi ? hi : v); }
__device__ __forceinline__ i64 max64(i64 a, i64 b) { return a > b ? a : b; }
__device__ __forceinline__ i64 min64(i64 a, i64 b) { return a < b ? a : b; }
__device__ __forceinline__ i64 round_to_i64(float v) { return (i64)rintf(v); }
__device__ __forceinline__ i64 f64_to_i64(double v) {
    // Torch's CPU cast (x86 cvttsd2si): out of range or NaN -> INT64_MIN
    if (!(v >= -9223372036854775808.0 && v < 9223372036854775808.0)) return (i64)0x8000000000000000ULL;
    return (i64)v;
}
__device__ __forceinline__ int ilog2(int v) { return 31 - __clz(v); }
__device__ __forceinline__ bool finitef(float v) { return fabsf(v) < GD_INF; }
__device__ __forceinline__ float tolerance_of(float d) { return fmaxf(fabsf(d) / 128.0f, 4.0f); }

// ---------------------------------------------------------------------------------------------
// map relations (engine.py:399-484, 1578-1612), answered from vertex ids and the vertex CSR
// ---------------------------------------------------------------------------------------------
struct MapView {
    const gd_map_desc *m;
    __device__ int sec(int w, int side) const { return m->wall_sectors[2 * w + side]; }
    __device__ int vert(int w, int slot) const { return m->wall_vertex[2 * w + slot]; }
    __device__ bool one_sided(int w) const { return m->wall_sectors[2 * w + 1] < 0; }
    __device__ bool two_sided_distinct(int w) const { return sec(w, 0) >= 0 && sec(w, 1) >= 0 && sec(w, 0) != sec(w, 1); }
    __device__ bool same_pair(int a, int b) const {
        int a0 = sec(a, 0), a1 = sec(a, 1), b0 = sec(b, 0), b1 = sec(b, 1);
        return (a0 == b0 && a1 == b1) || (a0 == b1 && a1 == b0);
    }
    __device__ bool shares_any_endpoint(int a, int b) const {
        int a0 = vert(a, 0), a1 = vert(a, 1), b0 = vert(b, 0), b1 = vert(b, 1);
        return a0 == b0 || a0 == b1 || a1 == b0 || a1 == b1;
    }
    __device__ bool opposing(int a, int b) const {
        if (!same_pair(a, b) || sec(a, 1) < 0 || sec(b, 1) < 0 || shares_any_endpoint(a, b)) return false;
        const float *wa = m->walls + 4 * a, *wb = m->walls + 4 * b;
        float ax = wa[2] - wa[0], ay = wa[3] - wa[1], bx = wb[2] - wb[0], by = wb[3] - wb[1];
        float dot = ax * bx + ay * by;
        float cross = ax * by - ay * bx;
        return dot < 0 && fabsf(cross) < 1e-6f;
    }
    __device__ bool triangle_bridge(int vertex, int a, int b, int *index) const {
        *index = 0;
        if (!two_sided_distinct(a) || !two_sided_distinct(b)) return false;
        int a0 = sec(a, 0), a1 = sec(a, 1), b0 = sec(b, 0), b1 = sec(b, 1);
        int shared_count = (a0 == b0 || a0 == b1) + (a1 == b0 || a1 == b1);
        if (shared_count != 1) return false;
        int shared = (a0 == b0 || a0 == b1) ? a0 : a1;
        int pa = (a0 == shared) ? a1 : a0;
        int pb = (b0 == shared) ? b1 : b0;
        int found = -1, count = 0;
        for (int k = m->vertex_wall_ofs[vertex]; k < m->vertex_wall_ofs[vertex + 1]; ++k) {
            int w = m->vertex_wall_idx[k];
            if (w == a || w == b) continue;
            int s0 = sec(w, 0), s1 = sec(w, 1);
            if ((s0 == pa && s1 == pb) || (s0 == pb && s1 == pa)) { found = w; ++count; }
        }
        if (count != 1) return false;
        *index = found;
        return true;
    }
    __device__ bool portal_bridge(int slot, int path, int owner, int *index) const {
        *index = 0;
        if (owner == path) return false;
        int v = vert(path, slot);
        if (vert(owner, 0) != v && vert(owner, 1) != v) return false;
        return triangle_bridge(v, path, owner, index);
    }
    __device__ bool sector_bridge(int slot, int pending, int path, int *index) const {
        *index = 0;
        if (path == pending) return false;
        return triangle_bridge(vert(pending, slot), pending, path, index);
    }
};

#define LDS_SECTORS 512
#define LDS_TEXTURES 224   // textures whose size bits are staged in LDS (a multiple of 32); later ones read the global arrays
#define GRID_ALWAYS_INSIDE (1 << 30)   // grid item flag: the whole cell lies inside the sector

// Even-odd parity of one sector's edge sub-list around a point (engine.py:9598-9612, 10994-11015).
__device__ __forceinline__ bool inside_edges(const gd_map_desc *m, int e0, int e1, float px, float py) {
    int crossings = 0;
    for (int k = e0; k < e1; ++k) {
        const float4 e = *reinterpret_cast<const float4 *>(m->walls + 4 * m->grid_item_edges[k]);
        float dy = e.w - e.y;
        float safe_dy = fabsf(dy) < 1e-6f ? 1.0f : dy;
        bool crosses = (e.y > py) != (e.w > py);
        float crossing_x = e.x + (py - e.y) * (e.z - e.x) / safe_dy;
        crossings += (crosses && px < crossing_x) ? 1 : 0;
    }
    return crossings & 1;
}

// inside_edges over the repacked edge copies, two edges per step
__device__ __forceinline__ bool inside_edge_copies(const float4 *edges, int e0, int e1, float px, float py) {
    int crossings = 0;
    for (int k = e0; k < e1; k += 2) {
        const float4 a = edges[k], b = edges[k + 1 < e1 ? k + 1 : k];
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const float4 e = j == 0 ? a : b;
            float dy = e.w - e.y;
            float safe_dy = fabsf(dy) < 1e-6f ? 1.0f : dy;
            bool crosses = (e.y > py) != (e.w > py);
            float crossing_x = e.x + (py - e.y) * (e.z - e.x) / safe_dy;
            crossings += (k + j < e1 && crosses && px < crossing_x) ? 1 : 0;
        }
    }
    return crossings & 1;
}

// Cell of the point grid, or -1 when no sector can contain the point.
__device__ __forceinline__ int grid_cell_of(const gd_map_desc *m, float px, float py) {
    float fx = floorf((px - m->grid_min_x) / m->grid_cell);
    float fy = floorf((py - m->grid_min_y) / m->grid_cell);
    if (!(fy >= 0.0f) || !(fy < (float)m->grid_ny) || !(fx < (float)m->grid_nx)) return -1;
    int ix = fx < 0.0f ? 0 : (int)fx;   // column 0 also stands for everything left of the grid
    if (!(fx == fx)) return -1;
    return (int)fy * m->grid_nx + ix;
}

// Fine raster entries (top two bits): a decided sector, empty, or undecided with / without the
// masks of plane levels that can win in the cell.
#define FINE_KIND(v) ((unsigned)(v) >> 30)
#define FINE_DECIDED 0u
#define FINE_EMPTY 1u
#define FINE_MIXED 2u
#define FINE_UNKNOWN 3u
#define FINE_MASK_LEVELS 15
#define FLAT_BATCH 2       // plane levels probed together in flat_select
#define FLAT_BATCH_MASKED 3   // ... on maps with bit sets of reachable levels, where a batch holds levels that are looked at

// Fine raster lookup.  Points outside the raster (or not finite) report FINE_UNKNOWN with a
// negative cell, and the caller locates them with grid_cell_of.  The coarse cell of a point
// inside the raster is (iy >> 3) * grid_nx + (ix >> 3): grid_cell is 8 * fine_cell and both
// grids pad their cells far beyond the rounding of either index computation.
// (fx, fy) is the point in raster cell units; anything within a small fraction of a cell of the
// true position will do, because decided cells keep a margin of half a map unit.
__device__ __forceinline__ unsigned fine_lookup_cells(const gd_map_desc *m, float fx, float fy, int *coarse_cell) {
    int ix = (int)floorf(fx), iy = (int)floorf(fy);
    *coarse_cell = -1;
    if ((unsigned)ix >= (unsigned)m->fine_nx || (unsigned)iy >= (unsigned)m->fine_ny || !(fx == fx) || !(fy == fy)) return 0xC0000000u;
    *coarse_cell = (iy >> 3) * m->grid_nx + (ix >> 3);
    return m->fine_sector[iy * m->fine_nx + ix];
}
__device__ __forceinline__ unsigned fine_lookup(const gd_map_desc *m, float inv_cell, float px, float py, int *coarse_cell) {
    int ix = (int)floorf((px - m->grid_min_x) * inv_cell), iy = (int)floorf((py - m->grid_min_y) * inv_cell);
    *coarse_cell = -1;
    if ((unsigned)ix >= (unsigned)m->fine_nx || (unsigned)iy >= (unsigned)m->fine_ny || !(px == px) || !(py == py)) return 0xC0000000u;
    *coarse_cell = (iy >> 3) * m->grid_nx + (ix >> 3);
    return m->fine_sector[iy * m->fine_nx + ix];
}

// _sector_at (engine.py:9598-9617): first sector with odd parity, 0 when none
__device__ int sector_at(const gd_map_desc *m, float px, float py) {
    int cell;
    unsigned fine = fine_lookup(m, 1.0f / m->fine_cell, px, py, &cell);
    if (FINE_KIND(fine) == FINE_EMPTY) return 0;
    if (FINE_KIND(fine) == FINE_DECIDED) return (int)(fine & 0xFFFFu);
    if (cell < 0) cell = grid_cell_of(m, px, py);
    if (cell < 0) return 0;
    for (int it = m->grid_cell_ofs[cell]; it < m->grid_cell_ofs[cell + 1]; ++it) {
        int item = m->grid_item_sector[it];
        if ((item & GRID_ALWAYS_INSIDE) || inside_edges(m, m->grid_item_edge_ofs[it], m->grid_item_edge_ofs[it + 1], px, py))
            return item & ~GRID_ALWAYS_INSIDE;
    }
    return 0;
}

// A flat probe of plane level k lands at distance cd = h_k * g from the camera, h_k the level's plane height and
// g = 192 / |row - centre| / cos(column) the pixel's own scale, and can only hit a sector whose level is k if
// reach_k <= cd <= far_k (level_reach / level_far): that is, if g lies in [reach_k / h_k, far_k / h_k].  With a plane
// level per sector a pixel would test hundreds of such intervals to find the few that hold its g, so the lane keeps,
// for each of LEVEL_BUCKETS ranges of g (6.5 to the octave from g = 0.7 up, the first and last open-ended), a bit set
// of the levels whose interval reaches into the range, a bucket to spare on either side (far more than the rounding of
// the logarithm or of g can move anything).  A probe then visits only the levels of its bucket, in level order, and
// applies the exact test to those: the bit sets only spare it levels the exact test would reject as well.
#define LEVEL_BUCKETS 64
#define LEVEL_MASK_WORDS_MAX 32     // up to 1024 plane levels (floors and ceilings together); beyond that every level is visited,
#define LEVEL_MASK_MIN_LEVELS 64    // and so it is with few levels, where the bit sets cost more than they spare
__device__ __forceinline__ int level_mask_words(const gd_map_desc *m) {
    const int levels = m->floor_level_count + m->ceil_level_count;
    return levels > LEVEL_MASK_MIN_LEVELS && levels <= 32 * LEVEL_MASK_WORDS_MAX ? (levels + 31) / 32 : 0;
}
__device__ __forceinline__ int level_bucket(float g) {
    if (!(g > 0.0f)) return 0;
    const float b = floorf((__log2f(g) + 0.5f) * 6.5f);
    return b <= 0.0f ? 0 : (b >= (float)(LEVEL_BUCKETS - 1) ? LEVEL_BUCKETS - 1 : (int)b);
}

// Per-lane tables for the flat kernels, one block per lane (after lane_setup):
//  * per plane level, how far the camera is, at least, from every sector at that level: a flat
//    probe nearer than that cannot land in such a sector (engine.py:10981-11024 tests the point
//    against every sector; here the far ones are ruled out by their bounding boxes);
//  * per plane level, the fixed-point plane height and visibility factor (engine.py:10588-10600);
//  * per view row, the plane distance slope (engine.py:10917-10931);
//  * per log2 texture size, the per-column texture steps (engine.py:10895-10902).
// The last three only depend on (lane, level), (lane, row) and (lane, size), so dividing once
// here spares plane shading four 64-bit divisions per pixel.
__global__ void lane_tables_kernel(DeviceMap dm, gd_lanes_desc lanes, int lane_base, int lane_count, Scratch sc) {
    const int local = blockIdx.x;
    const int floors = dm.d.floor_level_count, levels = floors + dm.d.ceil_level_count;
    if (local >= lane_count) return;
    const LaneCtx &c = sc.ctx[local];
    // the lane's per-column lists start empty
    for (int x = threadIdx.x; x < SW; x += blockDim.x) { sc.cand_count[(size_t)local * SW + x] = 0; sc.block_hit[(size_t)local * SW + x] = ~0ULL; }
    // and no column holds an unresolved gap pixel yet
    for (int k = threadIdx.x; k < 2 * SW; k += blockDim.x) sc.flat_col_top[(size_t)local * 2 * SW + k] = VH;
    {   // does a live billboard of the lane blend with what lies under it?
        bool blends = false;
        if (lanes.sprite_style && lanes.sprite_alive)
            for (int k = threadIdx.x; k < lanes.sprite_slots; k += blockDim.x) {
                const size_t at = (size_t)(lane_base + local) * lanes.sprite_slots + k;
                blends |= lanes.sprite_alive[at] != 0 && lanes.sprite_style[at] != -1;
            }
        const int any = __syncthreads_or(blends ? 1 : 0);
        if (threadIdx.x == 0) sc.lane_blends[local] = any;
    }
    const float cx = lanes.x[lane_base + local], cy = lanes.y[lane_base + local];
    __shared__ unsigned int masks_lds[LEVEL_BUCKETS * LEVEL_MASK_WORDS_MAX];
    const int mask_words = level_mask_words(&dm.d);
    for (int k = threadIdx.x; k < LEVEL_BUCKETS * mask_words; k += blockDim.x) masks_lds[k] = 0u;
    __syncthreads();
    for (int l = threadIdx.x; l < levels; l += blockDim.x) {
        float reach = GD_INF, far = 0.0f;
        for (int k = dm.level_box_ofs[l]; k < dm.level_box_ofs[l + 1]; ++k) {
            const float4 box = dm.level_boxes[k];
            float dx = fmaxf(fmaxf(box.x - cx, cx - box.z), 0.0f), dy = fmaxf(fmaxf(box.y - cy, cy - box.w), 0.0f);
            reach = fminf(reach, sqrtf(dx * dx + dy * dy));
            dx = fmaxf(fabsf(box.x - cx), fabsf(box.z - cx)); dy = fmaxf(fabsf(box.y - cy), fabsf(box.w - cy));
            far = fmaxf(far, sqrtf(dx * dx + dy * dy));
        }
        // margin: the probe point is camera + unit ray * distance in float32, far inside 0.1%
        sc.level_reach[(size_t)local * levels + l] = reach * 0.999f - 0.5f;
        sc.level_far[(size_t)local * levels + l] = far * 1.001f + 0.5f;
        const float plane_height = l < floors ? (c.view_z - dm.d.floor_levels[l]) : (dm.d.ceil_levels[l - floors] - c.view_z);
        if (mask_words > 0 && plane_height > 0.0f && far >= reach) {      // a level at or beyond the eye shows no plane
            const float low = (reach * 0.999f - 0.5f) / plane_height, high = (far * 1.001f + 0.5f) / plane_height;
            const int first = max(level_bucket(low) - 1, 0), last = min(level_bucket(high) + 1, LEVEL_BUCKETS - 1);
            for (int b = first; b <= last; ++b) atomicOr(&masks_lds[b * mask_words + (l >> 5)], 1u << (l & 31));
        }
        const i64 plane_height_fixed = round_to_i64(plane_height * 65536.0f);
        sc.level_plane[((size_t)local * levels + l) * 2] = plane_height_fixed;
        sc.level_plane[((size_t)local * levels + l) * 2 + 1] = min64(tdiv(FLOOR_VISIBILITY_FIXED << 16, max64(plane_height_fixed, 1)), (1LL << 31) - 1);
    }
    __syncthreads();
    for (int k = threadIdx.x; k < LEVEL_BUCKETS * mask_words; k += blockDim.x) sc.level_masks[(size_t)local * LEVEL_BUCKETS * mask_words + k] = masks_lds[k];
    for (int py = threadIdx.x; py < VH; py += blockDim.x) {
        i64 center_row = c.center_fixed >> 16;
        i64 pixel_y_fixed = (i64)py * FIXED_UNIT;
        i64 den = (py < center_row) ? (c.center_fixed - pixel_y_fixed - FIXED_UNIT / 2) : (pixel_y_fixed - c.center_fixed + FIXED_UNIT / 2);
        den = max64(den, 1);
        bool overflow = den <= (FOCAL_Y_FIXED >> 15);
        i64 yslope = tdiv(FOCAL_Y_FIXED << 16, den);
        sc.row_slope[(size_t)local * VH + py] = overflow ? (1LL << 31) - 1 : yslope;
    }
    for (int k = threadIdx.x; k < 32; k += blockDim.x) {
        const i64 basis = k < 16 ? c.vsin : c.vcos;
        const i64 step = tdiv(shl64(basis, 32 - (k & 15)), FOCAL_X_FIXED);
        i64 *entry = sc.step_scale + (size_t)local * STEP_TABLE;
        entry[k] = step;
        // the texture fraction of screen column 0 (column px is (px - 159) steps from the view axis), and the
        // camera's own offset in the texture, for the same log2 size
        entry[32 + k] = (shl64(k < 16 ? c.vcos : -c.vsin, 32 - (k & 15)) >> 16) - mul64(SW / 2 - 1, step);
        entry[64 + k] = shl64(k < 16 ? c.view_x_fixed : -c.view_y_fixed, 32 - (k & 15)) >> 16;
    }
}

// ---------------------------------------------------------------------------------------------
// lane_setup: engine.py:10648-10658, 2122-2133, 9622-9631, 12384-12391, 9619
// ---------------------------------------------------------------------------------------------
__global__ void lane_setup_kernel(DeviceMap dm, gd_lanes_desc lanes, int lane_base, int lane_count, Scratch sc) {
    int local = blockIdx.x * blockDim.x + threadIdx.x;
    if (local >= lane_count) return;
    int n = lane_base + local;
    const float BAM_TO_RADIANS = (float)(2.0 * 3.14159265358979323846 / 4294967296.0);
    LaneCtx c;
    c.x = lanes.x[n]; c.y = lanes.y[n]; c.view_z = lanes.view_z[n];
    float angle = lanes.angle[n];
    i64 pitch_bam = lanes.pitch_bam[n];
    c.flash_light = lanes.flash_light ? lanes.flash_light[n] : 0;
    i64 retained_bam = lanes.angle_bam[n];
    float visible_angle = (float)retained_bam * BAM_TO_RADIANS;
    i64 angle_bam = retained_bam;
    if (angle != visible_angle) {
        float two_pi = (float)(2.0 * 3.14159265358979323846);
        float r = fmodf(angle, two_pi);
        if (r != 0.0f && (r < 0.0f)) r += two_pi;   // torch.remainder with a positive divisor
        angle_bam = round_to_i64(r / BAM_TO_RADIANS) & UINT32_MASK;
    }
    i64 xf = lanes.x_fixed[n], yf = lanes.y_fixed[n];
    float visible_x = (float)xf / 65536.0f, visible_y = (float)yf / 65536.0f;
    c.view_x_fixed = (c.x != visible_x) ? round_to_i64(c.x * 65536.0f) : xf;
    c.view_y_fixed = (c.y != visible_y) ? round_to_i64(c.y * 65536.0f) : yf;
    int fine = (int)((angle_bam >> 19) & (FINE_ANGLES - 1));
    c.vsin = dm.fine_sine[fine];
    c.vcos = dm.fine_sine[(fine + FINE_ANGLES / 4) & (FINE_ANGLES - 1)];
    c.fsin = (float)c.vsin / 65536.0f;
    c.fcos = (float)c.vcos / 65536.0f;
    i64 tangent_index = clampi((ANGLE_90 - pitch_bam) >> 19, 0, FINE_ANGLES / 2 - 1);
    i64 tangent = dm.fine_tangent[tangent_index];
    c.center_fixed = (i64)(VH / 2) * FIXED_UNIT + ((FOCAL_Y_FIXED * tangent) >> 16);
    c.upper_clip = tdiv(shl64(-c.center_fixed, 16), FOCAL_Y_FIXED);
    c.lower_clip = tdiv(shl64((i64)VH * FIXED_UNIT - c.center_fixed, 16), FOCAL_Y_FIXED);
    c.pitch_offset = (float)((tangent * 12582912LL) >> 16) / 65536.0f;
    c.sector = sector_at(&dm.d, c.x, c.y);
    c.last_ceiling_row = -1;
    for (int y = 0; y < VH; ++y) if (!(((float)y - (103.5f + c.pitch_offset)) > 0)) c.last_ceiling_row = y;   // flat_center()
    sc.ctx[local] = c;
    int *span = sc.flat_span + (size_t)local * 4;
    span[0] = VH; span[1] = -1; span[2] = VH; span[3] = -1;
    sc.flat_list_count[local] = 0;
    if (local == 0) { *sc.flat_row_count = 0; *sc.gap_column_count = 0; *sc.spill_count = 0; }
}

__device__ __forceinline__ void ray_direction(const LaneCtx &c, int x, float *rx, float *ry) {
    // engine.py:10660-10670
    float col = ((float)x - 160.0f) / 160.0f;
    *rx = c.fcos + c.fsin * col;
    *ry = c.fsin - c.fcos * col;
}

// distances / along / geometric / projected / left-edge of one linedef at one column
// (engine.py:11317-11331, 11440-11460)
__device__ __forceinline__ Eval eval_segment(const float4 wl, int rec_flags, int rec_pl, int rec_pr, bool os, const LaneCtx &c, int x, float rx, float ry) {
    float segx = wl.z - wl.x, segy = wl.w - wl.y;
    float offx = wl.x - c.x, offy = wl.y - c.y;
    float den = rx * segy - ry * segx;
    bool ok = fabsf(den) >= 1e-6f;
    float safe = ok ? den : 1.0f;
    float d = (offx * segy - offy * segx) / safe;
    float a = (offx * ry - offy * rx) / safe;
    bool g = ok && (d > 0) && (a >= 0) && (a <= 1);
    bool screen_valid = (rec_flags & WF_HC) && (x >= rec_pl) && (x < rec_pr);
    bool p = ok && (d > 0) && screen_valid;
    bool valid = os ? (p && (rec_flags & WF_FF)) : (g || p);
    Eval out;
    out.dist = valid ? d : GD_INF;
    out.flags = (g ? CF_GEO : 0) | (p ? CF_PROJ : 0) | ((x == rec_pl) ? CF_LEDGE : 0) | ((a > 0.5f) ? CF_ALONG_HI : 0) |
                ((rec_flags & WF_FF) ? CF_FF : 0);
    return out;
}

__device__ __forceinline__ Eval eval_wall(const gd_map_desc *m, const LaneCtx &c, const RecSpan *spans, int x, int w, float rx, float ry) {
    const float4 wl = *reinterpret_cast<const float4 *>(m->walls + 4 * w);
    const RecSpan r = spans[w];
    return eval_segment(wl, r.flags, r.pl, r.pr, m->wall_sectors[2 * w + 1] < 0, c, x, rx, ry);
}

// ---------------------------------------------------------------------------------------------
// wall_setup: engine.py:10747-10869 (FWallCoords) and the per-linedef half of 11304-11451
// ---------------------------------------------------------------------------------------------
// FWallCoords of one fixed-point segment seen from one lane (engine.py:10747-10869): view-space
// endpoints, clipped half-open screen span and clipped endpoint depths.
// `endpoint_quotient`, when asked for, receives tx * center / ty (ty == 0 counted as 1) of the linedef's two endpoints
// in map order: the projections below divide exactly these, whichever endpoint the facing puts first.
__device__ __forceinline__ void wall_coords(const LaneCtx &c, const int *wf, WallRec &r, i64 *endpoint_quotient = nullptr) {
    i64 rx0 = (i64)wf[0] - c.view_x_fixed, ry0 = (i64)wf[1] - c.view_y_fixed;
    i64 rx1 = (i64)wf[2] - c.view_x_fixed, ry1 = (i64)wf[3] - c.view_y_fixed;
    i64 tx0 = (rx0 * c.vsin - ry0 * c.vcos) >> 20, ty0 = (rx0 * c.vcos + ry0 * c.vsin) >> 20;
    i64 tx1v = (rx1 * c.vsin - ry1 * c.vcos) >> 20, ty1v = (rx1 * c.vcos + ry1 * c.vsin) >> 20;
    i64 vx = (i64)wf[2] - wf[0], vy = (i64)wf[3] - wf[1];
    i64 fx = c.view_x_fixed - wf[0], fy = c.view_y_fixed - wf[1];
    bool front = (vx * fy - vy * fx) < 0;
    i64 tx1 = front ? tx0 : tx1v, tx2 = front ? tx1v : tx0;
    i64 ty1 = front ? ty0 : ty1v, ty2 = front ? ty1v : ty0;
    const i64 center = 160 * FIXED_UNIT;
    const i64 quotient0 = tdiv(tx0 * center, ty0 == 0 ? 1 : ty0), quotient1 = tdiv(tx1v * center, ty1v == 0 ? 1 : ty1v);
    if (endpoint_quotient) { endpoint_quotient[0] = quotient0; endpoint_quotient[1] = quotient1; }
    i64 left_projected = ((center + (front ? quotient0 : quotient1)) >> 16) + (tx1 >= 0);
    if (tx1 >= 0) left_projected = min64(left_projected, SW);
    i64 right_projected = ((center + (front ? quotient1 : quotient0)) >> 16) + (tx2 >= 0);
    if (tx2 >= 0) right_projected = min64(right_projected, SW);
    i64 left_den = tx1 - tx2 - ty2 + ty1, right_den = ty2 - ty1 - tx2 + tx1;
    i64 safe_left_den = left_den == 0 ? 1 : left_den, safe_right_den = right_den == 0 ? 1 : right_den;
    bool left_inside = tx1 >= -ty1, right_inside = tx2 <= ty2;
    i64 sl = left_inside ? left_projected : 0;
    i64 sr = right_inside ? right_projected : SW;
    i64 dl = left_inside ? ty1 : ty1 + tdiv((ty2 - ty1) * (tx1 + ty1), safe_left_den);
    i64 dr = right_inside ? ty2 : ty1 + tdiv((ty2 - ty1) * (tx1 - ty1), safe_right_den);
    bool invalid_left = (left_inside ? ((tx1 > ty1) || (ty1 == 0)) : ((tx2 < -ty2) || (left_den == 0))) || (dl < 32);
    bool invalid_right = (right_inside ? ((tx2 < -ty2) || (ty2 == 0)) : ((tx1 > ty1) || (right_den == 0))) || (dr < 32);
    bool invalid = invalid_left || invalid_right || (sr <= sl);
    if (invalid) sr = sl;
    r.tx0 = (int)tx0; r.tx1 = (int)tx1v; r.ty0 = (int)ty0; r.ty1 = (int)ty1v;
    r.dl = dl; r.dr = dr; r.sl = sl; r.sr = sr;
}

// Every fragment of every split linedef of one lane (engine.py:11472-11500).
__global__ void fragment_setup_kernel(DeviceMap dm, int lane_count, Scratch sc) {
    const gd_map_desc *m = &dm.d;
    const int per_lane = m->split_count * m->fragment_slots;
    const int k = blockIdx.x * blockDim.x + threadIdx.x;
    const int local = blockIdx.y;
    if (local >= lane_count || k >= per_lane) return;
    WallRec r;
    wall_coords(sc.ctx[local], m->split_fragments_fixed + 4 * (size_t)k, r);
    r.pl = 0; r.pr = 0; r.flags = 0;
    sc.frag_rec[(size_t)local * per_lane + k] = r;
}

// A column that was offered more entries than its own slots hold asks for a slot in the spill pool.  With the pool
// used up the column keeps its first CAND_MAX entries and the renderer's status says so.
__device__ __forceinline__ void request_spill_slot(const Scratch &sc, int column) {
    const int slot = atomicAdd(sc.spill_count, 1);
    if (slot < sc.spill_slots) sc.spill_columns[slot] = column;
    else atomicOr(sc.status, STATUS_CAND_OVERFLOW);
}

// One thread owns one linedef for the per-linedef arithmetic.  The two per-column loops have
// wildly different trip counts per linedef (none for most, up to 320 for a few), so they are
// run by the whole wavefront together: the linedefs with a non-empty column range take turns,
// their parameters are broadcast from the owning lane, and the 64 lanes each take one column.
//
// Three quarters of a map's linedefs lie wholly behind the camera or wholly to one side of its view: no
// column ray can hit such a linedef and FWallCoords rejects it, so nothing of it is ever looked at beyond
// the ray-test facts of RecSpan (no owned span).  A block first sorts its SETUP_WALLS linedefs into those and the
// rest, and only the rest, packed into as few wavefronts as they fill, get the arithmetic below.
#define SETUP_WALLS 256
__global__ void __launch_bounds__(SETUP_WALLS) wall_setup_kernel(DeviceMap dm, int lane_count, Scratch sc) {
    const gd_map_desc *m = &dm.d;
    __shared__ int alive_list[SETUP_WALLS];
    __shared__ int alive_count;
    const int slot_in_wave = threadIdx.x & 63;
    const int local = blockIdx.y;
    if (local >= lane_count) return;          // uniform over the block
    const LaneCtx &c = sc.ctx[local];
    if (threadIdx.x == 0) alive_count = 0;
    __syncthreads();
    {
        const int w = blockIdx.x * SETUP_WALLS + threadIdx.x;
        if (w < m->wall_count) {
            const float4 wl = *reinterpret_cast<const float4 *>(m->walls + 4 * w);
            const float ax = wl.x - c.x, ay = wl.y - c.y, bx = wl.z - c.x, by = wl.w - c.y;
            // forward and rightward view coordinates of both endpoints; a column ray is forward + col * right, |col| <= 1
            const float f0 = ax * c.fcos + ay * c.fsin, r0 = ax * c.fsin - ay * c.fcos;
            const float f1 = bx * c.fcos + by * c.fsin, r1 = bx * c.fsin - by * c.fcos;
            // wholly in one of the half planes behind the camera, right of the right view edge, left of the left one (a map
            // unit to spare, far more than float32 and 16.16 coordinates can disagree): no ray reaches it, FWallCoords finds
            // no span.  Linedef 0 and the first blocking linedef stand in where a scan finds nothing, and are always kept.
            const bool unseen = (f0 < -1.0f && f1 < -1.0f) || (r0 > f0 + 1.0f && r1 > f1 + 1.0f) || (r0 < -f0 - 1.0f && r1 < -f1 - 1.0f);
            const bool kept = !unseen || w == 0 || (m->blocking_count > 0 && w == m->blocking_walls[0]);
            if (kept) {
                alive_list[atomicAdd(&alive_count, 1)] = w;
            } else {
                const float vfx = c.x - wl.x, vfy = c.y - wl.y;
                const bool ff = ((wl.z - wl.x) * vfy - (wl.w - wl.y) * vfx) < 0;
                RecSpan span;
                span.pl = 0; span.pr = 0;
                // an unseen linedef has an empty span (sr == sl), so a two-sided one counts as at most one column wide
                span.flags = (ff ? WF_FF : 0) | (m->wall_sectors[2 * w + 1] < 0 ? 0 : WF_SUBPIXEL) | (m->wall_split_slot[w] >= 0 ? WF_SPLIT : 0);
                sc.span[(size_t)local * m->wall_count + w] = span;
            }
        }
    }
    __syncthreads();
    const int alive = alive_count;
    if ((int)(threadIdx.x & ~63u) >= alive) return;   // whole wavefronts beyond the kept linedefs leave
    const bool live = (int)threadIdx.x < alive;  // dead lanes of the last wavefront still help with the column loops
    const int w = live ? alive_list[threadIdx.x] : 0;
    const int *wf = m->walls_fixed + 4 * w;
    WallRec r;
    i64 endpoint_quotient[2];
    wall_coords(c, wf, r, endpoint_quotient);
    const i64 tx0 = r.tx0, tx1v = r.tx1, ty0 = r.ty0, ty1v = r.ty1;
    const i64 sl = r.sl, sr = r.sr;
    const i64 center = 160 * FIXED_UNIT;

    // Ray x segment: first / last column whose ray hits the segment (engine.py:11323-11348).
    // A ray of column parameter col = (x-160)/160 is forward + col*right; an endpoint with view
    // coordinates (f, r) lies on it when r = col*f.  The float test below can only pass where the
    // two endpoints are not both clearly (> half a map unit) on one side of the ray, so for a
    // segment wholly in front of the camera only the columns between its endpoint columns
    // (padded) are examined; segments reaching behind the camera get the full scan.
    const float4 wl = *reinterpret_cast<const float4 *>(m->walls + 4 * w);
    float segx = wl.z - wl.x, segy = wl.w - wl.y;
    float offx = wl.x - c.x, offy = wl.y - c.y;
    int scan_lo = 0, scan_hi = SW - 1;
    {
        float e1x = offx + segx, e1y = offy + segy;
        float f0 = offx * c.fcos + offy * c.fsin, r0 = offx * c.fsin - offy * c.fcos;
        float f1 = e1x * c.fcos + e1y * c.fsin, r1 = e1x * c.fsin - e1y * c.fcos;
        if (f0 > 1.0f && f1 > 1.0f) {
            float c0 = r0 / f0, c1 = r1 / f1, p0 = 0.5f / f0, p1 = 0.5f / f1;
            float lo = fminf(c0 - p0, c1 - p1), hi = fmaxf(c0 + p0, c1 + p1);
            float xlo = floorf(160.0f + 160.0f * lo) - 1.0f, xhi = ceilf(160.0f + 160.0f * hi) + 1.0f;
            scan_lo = xlo < 0.0f ? 0 : (xlo > 320.0f ? 320 : (int)xlo);
            scan_hi = xhi > 319.0f ? 319 : (xhi < -1.0f ? -1 : (int)xhi);
        } else if (f0 < -1.0f && f1 < -1.0f) {
            scan_lo = 1; scan_hi = 0;   // wholly behind the camera: no ray reaches it
        }
    }
    if (!live) { scan_lo = 1; scan_hi = 0; }
    const int blocking_slot = dm.wall_blocking_slot[w];
    u64 *block_hits = sc.block_hit + (size_t)local * SW;
    int first = 0, last = SW - 1; bool any = false;
    float numer_d = offx * segy - offy * segx;
    // Most scan ranges are a few columns wide, so several linedefs share a turn (eight lanes each for eight of
    // them, sixteen for four, thirty-two for two); a wider range has the wavefront to itself.
    const int scan_width = scan_hi - scan_lo + 1;
    auto shared_scans = [&](bool member, int lanes_each) {
        const int group = slot_in_wave / lanes_each, group_lane = slot_in_wave - group * lanes_each;
        const int groups = 64 / lanes_each;
        const u64 group_mask = (lanes_each == 64 ? ~0ULL : ((1ULL << lanes_each) - 1)) << (group * lanes_each);
        for (u64 pending = __ballot(member); pending;) {
            int owners[8];
            int owner = -1;
#pragma unroll
            for (int k = 0; k < 8; ++k) {
                owners[k] = -1;
                if (k >= groups) continue;               // the same in every lane
                owners[k] = pending ? __ffsll((long long)pending) - 1 : -1;
                pending &= pending - 1;
                if (group == k) owner = owners[k];
            }
            const int source = owner < 0 ? 0 : owner;
            const float b_segx = __shfl(segx, source), b_segy = __shfl(segy, source);
            const float b_offx = __shfl(offx, source), b_offy = __shfl(offy, source), b_numer = __shfl(numer_d, source);
            const int b_lo = __shfl(scan_lo, source), b_hi = __shfl(scan_hi, source);
            const int b_block = __shfl(blocking_slot, source);
            const int x = b_lo + group_lane;
            float rx, ry; ray_direction(c, x, &rx, &ry);
            float den = rx * b_segy - ry * b_segx;
            bool ok = fabsf(den) >= 1e-6f;
            float safe = ok ? den : 1.0f;
            float d = b_numer / safe;
            float a = (b_offx * ry - b_offy * rx) / safe;
            bool g = owner >= 0 && x <= b_hi && ok && (d > 0) && (a >= 0) && (a <= 1);
            if (g && b_block >= 0) atomicMin(&block_hits[x], ((u64)__float_as_uint(d) << 32) | (u64)(unsigned)b_block);
            const u64 hits = __ballot(g) & group_mask;
            // every lane of a group holds its linedef's first / last hit column; the linedef's own lane fetches them
            const int group_first = hits ? b_lo + (__ffsll((long long)hits) - 1 - group * lanes_each) : SW;
            const int group_last = hits ? b_lo + (63 - __clzll((long long)hits) - group * lanes_each) : -1;
#pragma unroll
            for (int k = 0; k < 8; ++k) {
                if (k >= groups || owners[k] < 0) continue;   // the same in every lane
                const int k_first = bcast(group_first, k * lanes_each), k_last = bcast(group_last, k * lanes_each);
                if (slot_in_wave == owners[k] && k_last >= 0) { first = k_first; last = k_last; any = true; }
            }
        }
    };
    const bool scans = scan_lo <= scan_hi;
    shared_scans(scans && scan_width <= 8, 8);
    shared_scans(scans && scan_width > 8 && scan_width <= 16, 16);
    shared_scans(scans && scan_width > 16 && scan_width <= 32, 32);
    for (u64 pending = __ballot(scans && scan_width > 32); pending; pending &= pending - 1) {
        const int owner = __ffsll((long long)pending) - 1;
        const float b_segx = bcast(segx, owner), b_segy = bcast(segy, owner);
        const float b_offx = bcast(offx, owner), b_offy = bcast(offy, owner), b_numer = bcast(numer_d, owner);
        const int b_lo = bcast(scan_lo, owner), b_hi = bcast(scan_hi, owner);
        const int b_block = bcast(blocking_slot, owner);
        int hit_first = SW, hit_last = -1;
        for (int x0 = b_lo; x0 <= b_hi; x0 += 64) {
            const int x = x0 + slot_in_wave;
            float rx, ry; ray_direction(c, x, &rx, &ry);
            float den = rx * b_segy - ry * b_segx;
            bool ok = fabsf(den) >= 1e-6f;
            float safe = ok ? den : 1.0f;
            float d = b_numer / safe;
            float a = (b_offx * ry - b_offy * rx) / safe;
            bool g = x <= b_hi && ok && (d > 0) && (a >= 0) && (a <= 1);
            // the sprite pass wants the nearest blocking linedef each column ray hits, lowest slot on ties
            if (g && b_block >= 0) atomicMin(&block_hits[x], ((u64)__float_as_uint(d) << 32) | (u64)(unsigned)b_block);
            const u64 hits = __ballot(g);
            if (hits) {
                if (hit_last < 0) hit_first = x0 + __ffsll((long long)hits) - 1;
                hit_last = x0 + 63 - __clzll((long long)hits);
            }
        }
        if (slot_in_wave == owner && hit_last >= 0) { first = hit_first; last = hit_last; any = true; }
    }
    float vfx = c.x - wl.x, vfy = c.y - wl.y;
    bool ff = (segx * vfy - segy * vfx) < 0;
    i64 screen_left = first, screen_right = (i64)last + 1;
    bool hc = any;
    i64 ep_col[2]; bool ep_vis[2];
    i64 txe[2] = {tx0, tx1v}, tye[2] = {ty0, ty1v};
    for (int e = 0; e < 2; ++e) {
        i64 projected_fixed = center + endpoint_quotient[e];   // tx * center / ty, as wall_coords divided it
        ep_col[e] = (projected_fixed >> 16) + (txe[e] >= 0);
        ep_vis[e] = (tye[e] > 0) && (txe[e] >= -tye[e]) && (txe[e] <= tye[e]) && (ep_col[e] >= 0) && (ep_col[e] <= SW);
    }
    for (int e = 0; e < 2; ++e) {
        bool visible = ep_vis[e] && hc;
        bool owns_left = ff ? (e == 0) : (e == 1);
        if (visible && owns_left) screen_left = ep_col[e];
        if (visible && !owns_left) screen_right = ep_col[e];
    }
    if (ep_vis[0] && ep_vis[1]) {
        screen_left = ff ? ep_col[0] : ep_col[1];
        screen_right = ff ? ep_col[1] : ep_col[0];
        hc = screen_right > screen_left;
    }
    hc = hc && (sr > sl);
    const int s0 = m->wall_sectors[2 * w], s1 = m->wall_sectors[2 * w + 1];
    bool os = s1 < 0;
    r.pl = (short)screen_left; r.pr = (short)screen_right;
    r.flags = (hc ? WF_HC : 0) | (ff ? WF_FF : 0) | (((sr - sl <= 1) && !os) ? WF_SUBPIXEL : 0) | (any ? WF_ANYGEO : 0) |
              (m->wall_split_slot[w] >= 0 ? WF_SPLIT : 0);
    if (live) {
        sc.rec[(size_t)local * m->wall_count + w] = r;
        RecSpan span;
        span.pl = r.pl; span.pr = r.pr; span.flags = r.flags;
        sc.span[(size_t)local * m->wall_count + w] = span;
    }
    // Enter the linedef in the candidate list of every column where its distance can be
    // finite: its owned span (projected) and, for two-sided lines, the columns its rays hit
    // (engine.py:11446-11451).  List order is irrelevant: scans break ties on the linedef index.
    int a_lo = SW, a_hi = 0;
    if (hc && (!os || ff)) { a_lo = r.pl; a_hi = r.pr; }
    if (!os && any) { a_lo = a_lo < first ? a_lo : first; a_hi = a_hi > last + 1 ? a_hi : last + 1; }
    a_lo = a_lo < 0 ? 0 : a_lo; a_hi = a_hi > SW ? SW : a_hi;
    if (!live) { a_lo = SW; a_hi = 0; }
    Cand *list = sc.cand + (size_t)local * CAND_MAX * SW;
    int *counts = sc.cand_count + (size_t)local * SW;
    const int packed_sectors = (s0 & 0xFFFF) | (s1 << 16);
    const int packed_vertices = (int)(((unsigned)m->wall_vertex[2 * w] & 0xFFFFu) | ((unsigned)m->wall_vertex[2 * w + 1] << 16));
    const bool masked_side = !os && m->side_tex[(w * 2 + (ff ? 0 : 1)) * 3] >= 0;
    const int packed_span = (r.flags & 0xFF) | (os ? 0x100 : 0) | (masked_side ? 0x200 : 0);
    const int rec_pl = r.pl, rec_pr = r.pr;
    // Most linedefs cover a few columns only, so several of them share a turn: eight with eight lanes each, then
    // four with sixteen, then two with thirty-two; a wider one has the wavefront to itself.
    const bool listed = a_lo < a_hi;
    const bool narrow = listed && (a_hi - a_lo <= 32);
    auto shared_turns = [&](bool member, int lanes_each) {
        const int group = slot_in_wave / lanes_each, group_lane = slot_in_wave - group * lanes_each;
        const int groups = 64 / lanes_each;
        for (u64 pending = __ballot(member); pending;) {
            int owner = -1;
#pragma unroll
            for (int g = 0; g < 8; ++g) {
                if (g >= groups) break;                  // the same in every lane
                const int next = pending ? __ffsll((long long)pending) - 1 : -1;
                pending &= pending - 1;
                if (group == g) owner = next;
            }
            const int source = owner < 0 ? 0 : owner;
            float4 b_wl;
            b_wl.x = __shfl(wl.x, source); b_wl.y = __shfl(wl.y, source); b_wl.z = __shfl(wl.z, source); b_wl.w = __shfl(wl.w, source);
            const int b_span = __shfl(packed_span, source), b_pl = __shfl(rec_pl, source), b_pr = __shfl(rec_pr, source);
            const int b_sectors = __shfl(packed_sectors, source), b_vertices = __shfl(packed_vertices, source);
            const int b_lo = __shfl(a_lo, source), b_hi = __shfl(a_hi, source);
            const int b_wall = __shfl(w, source);
            const int x = b_lo + group_lane;
            if (owner < 0 || x >= b_hi) continue;
            float rx, ry; ray_direction(c, x, &rx, &ry);
            const Eval e = eval_segment(b_wl, b_span & 0xFF, b_pl, b_pr, (b_span & 0x100) != 0, c, x, rx, ry);
            if (!finitef(e.dist)) continue;
            const int slot = atomicAdd(&counts[x], 1);
            if (slot < CAND_MAX) {
                Cand entry;
                entry.wall = (unsigned short)b_wall;
                entry.s0 = (short)(b_sectors & 0xFFFF); entry.s1 = (short)(b_sectors >> 16);
                entry.v0 = (unsigned short)(b_vertices & 0xFFFF); entry.v1 = (unsigned short)((unsigned)b_vertices >> 16);
                entry.flags = (unsigned short)(e.flags | ((b_span & 0x200) ? CF_MASKED : 0));
                entry.dist = e.dist;
                list[(size_t)slot * SW + x] = entry;
            }   // else: the count says so, and the column is listed afresh in the spill pool (strip_key_kernel, cand_spill_kernel)
        }
    };
    shared_turns(listed && (a_hi - a_lo <= 8), 8);
    shared_turns(listed && (a_hi - a_lo > 8) && (a_hi - a_lo <= 16), 16);
    shared_turns(listed && (a_hi - a_lo > 16) && (a_hi - a_lo <= 32), 32);
    for (u64 pending = __ballot(listed && !narrow); pending; pending &= pending - 1) {
        const int owner = __ffsll((long long)pending) - 1;
        float4 b_wl;
        b_wl.x = bcast(wl.x, owner); b_wl.y = bcast(wl.y, owner); b_wl.z = bcast(wl.z, owner); b_wl.w = bcast(wl.w, owner);
        const int b_span = bcast(packed_span, owner), b_pl = bcast(rec_pl, owner), b_pr = bcast(rec_pr, owner);
        const int b_sectors = bcast(packed_sectors, owner), b_vertices = bcast(packed_vertices, owner);
        const int b_lo = bcast(a_lo, owner), b_hi = bcast(a_hi, owner);
        Cand entry;
        entry.wall = (unsigned short)bcast(w, owner);
        entry.s0 = (short)(b_sectors & 0xFFFF); entry.s1 = (short)(b_sectors >> 16);
        entry.v0 = (unsigned short)(b_vertices & 0xFFFF); entry.v1 = (unsigned short)((unsigned)b_vertices >> 16);
        for (int x = b_lo + slot_in_wave; x < b_hi; x += 64) {
            float rx, ry; ray_direction(c, x, &rx, &ry);
            Eval e = eval_segment(b_wl, b_span & 0xFF, b_pl, b_pr, (b_span & 0x100) != 0, c, x, rx, ry);
            if (finitef(e.dist)) {
                int slot = atomicAdd(&counts[x], 1);
                if (slot < CAND_MAX) {
                    entry.flags = (unsigned short)(e.flags | ((b_span & 0x200) ? CF_MASKED : 0));
                    entry.dist = e.dist;
                    list[(size_t)slot * SW + x] = entry;
                }
            }
        }
    }
}

// The candidate list of every column that was given a spill slot, written afresh into the pool: one wavefront per
// column tests the column's ray against every linedef of the map (eval_wall: the same test, on the same per-linedef
// facts, that entered the linedef in wall_setup_kernel) and keeps those with a finite distance, in linedef order.
// A fixed, small grid: the kernel is launched every frame and nearly always finds no column to do.
#define SPILL_BLOCKS 1024
__global__ void __launch_bounds__(64) cand_spill_kernel(DeviceMap dm, Scratch sc) {
    const gd_map_desc *m = &dm.d;
    const int wanted = *sc.spill_count;
    const int total = wanted < sc.spill_slots ? wanted : sc.spill_slots;
    const int walls = m->wall_count;
    for (int slot = blockIdx.x; slot < total; slot += gridDim.x) {
        const int column = sc.spill_columns[slot];
        const int local = column / SW, x = column - local * SW;
        const LaneCtx &c = sc.ctx[local];
        float rx, ry; ray_direction(c, x, &rx, &ry);
        const RecSpan *spans = sc.span + (size_t)local * walls;
        Cand *list = sc.cand + sc.spill_base + ((size_t)(slot / SW) * SPILL_DEPTH * SW + (size_t)(slot % SW));
        int listed = 0;
        for (int w0 = 0; w0 < walls; w0 += 64) {
            const int w = w0 + (int)threadIdx.x;
            bool keep = false;
            Cand entry;
            if (w < walls) {
                const Eval e = eval_wall(m, c, spans, x, w, rx, ry);
                keep = finitef(e.dist);
                const int s1 = m->wall_sectors[2 * w + 1];
                const bool front_facing = (spans[w].flags & WF_FF) != 0;
                const bool masked_side = s1 >= 0 && m->side_tex[(w * 2 + (front_facing ? 0 : 1)) * 3] >= 0;
                entry.wall = (unsigned short)w;
                entry.s0 = (short)m->wall_sectors[2 * w]; entry.s1 = (short)s1;
                entry.v0 = (unsigned short)m->wall_vertex[2 * w]; entry.v1 = (unsigned short)m->wall_vertex[2 * w + 1];
                entry.flags = (unsigned short)(e.flags | (masked_side ? CF_MASKED : 0));
                entry.dist = e.dist;
            }
            const u64 keeps = __ballot(keep);
            const int position = listed + __popcll(keeps & ((1ULL << threadIdx.x) - 1ULL));
            if (keep) {
                if (position < SPILL_DEPTH) list[(size_t)position * SW] = entry;
                else atomicOr(sc.status, STATUS_CAND_OVERFLOW);
            }
            listed += __popcll(keeps);
        }
        if (threadIdx.x == 0) sc.cand_count[column] = (listed < SPILL_DEPTH ? listed : SPILL_DEPTH) | ((slot + 1) << SPILL_SHIFT);
    }
}

// ---------------------------------------------------------------------------------------------
// flats: engine.py:10956-11171
// ---------------------------------------------------------------------------------------------
__device__ __forceinline__ float flat_center(const LaneCtx &c) { return 103.5f + c.pitch_offset; }

// Per pixel: nearest plane among all sectors (engine.py:10981-11024).  Sectors that share a
// plane height share the candidate point, and the distance grows with the plane height, so the
// levels are visited nearest first and the scan stops once a farther level cannot win.
//
// Does the point lie in some sector whose floor (ceiling) is at `level`?  The even-odd test of
// engine.py:10994-11015 over the sectors the point-location grid lists for the point's cell.
__device__ bool flat_level_hit(const DeviceMap &dm, bool is_floor, float level, float px, float py) {
    const gd_map_desc *m = &dm.d;
    int cell;
    const unsigned fine = fine_lookup(m, dm.fine_inverse, px, py, &cell);
    const unsigned kind = FINE_KIND(fine);
    if (kind == FINE_EMPTY) return false;
    if (kind == FINE_DECIDED) return m->sector_heights[2 * (int)(fine & 0xFFFFu) + (is_floor ? 0 : 1)] == level;
    if (cell < 0) cell = grid_cell_of(m, px, py);
    if (cell < 0) return false;
    const int2 range = dm.cell_range[cell];
    for (int it = range.x; it < range.y; ++it) {
        const int4 item = dm.cell_item[it];
        const int s = item.x & ~GRID_ALWAYS_INSIDE;
        if (m->sector_heights[2 * s + (is_floor ? 0 : 1)] != level) continue;
        if ((item.x & GRID_ALWAYS_INSIDE) || inside_edge_copies(dm.cell_edge, item.z, item.w, px, py)) return true;
    }
    return false;
}
//
// Does the flat ray of one pixel resolve at all, i.e. does the probe point of some plane level lie in a
// sector of that level (engine.py:10981-11024)?  `plane` is the sector whose plane the wall pass shows at the
// pixel: its own level nearly always answers yes at once.
__device__ bool flat_ray_resolves(const DeviceMap &dm, const LaneCtx &c, float rc, float rs, float cc, int y, int plane) {
    const gd_map_desc *m = &dm.d;
    const float delta = (float)y - flat_center(c);
    const bool is_floor = delta > 0;
    const float denom = fmaxf(fabsf(delta), 0.5f);
    const float *levels = is_floor ? m->floor_levels : m->ceil_levels;
    const int level_count = is_floor ? m->floor_level_count : m->ceil_level_count;
    const float own = m->sector_heights[2 * plane + (is_floor ? 0 : 1)];
    for (int k = -1; k < level_count; ++k) {
        const float level = k < 0 ? own : levels[k];
        if (k >= 0 && level == own) continue;
        const float height = is_floor ? (c.view_z - level) : (level - c.view_z);
        if (!(height > 0)) continue;
        const float cd = (height * 192.0f / denom) / cc;
        if (!(finitef(cd) && cd > 0)) continue;
        if (flat_level_hit(dm, is_floor, level, c.x + rc * cd, c.y + rs * cd)) return true;
    }
    return false;
}
//
// flat_select_pixel is called by whole wavefronts whose 64 lanes look at 64 pixels of ONE row of one lane's
// screen (wanted or not: every lane takes part in the level broadcasts); it returns the sector, -1 if no
// level's probe point lies in a sector of that level.
// MASKS: the map has enough plane levels for the per-bucket bit sets (level_mask_words() > 0).
template <bool MASKS>
__device__ __forceinline__ int flat_select_pixel(const DeviceMap &dm, const Scratch &sc, const gd_lanes_desc &lanes, int local, int n,
                                                 int x, int y, bool wanted) {
    const gd_map_desc *m = &dm.d;
    const LaneCtx &c = sc.ctx[local];
    const float delta = (float)y - flat_center(c);
    const bool is_floor = delta > 0;
    float denom = fmaxf(fabsf(delta), 0.5f);
    float cc = dm.cosine_correction[x];
    float rc = lanes.ray_cos[(size_t)n * SW + x], rs = lanes.ray_sin[(size_t)n * SW + x];
    // A wavefront covers 64 pixels of one row (320 = 5 * 64), so the plane side and everything
    // that depends only on (row, level) is the same in all its lanes.
    const bool floor_uniform = __builtin_amdgcn_readfirstlane((int)is_floor) != 0;
    const float *levels = floor_uniform ? m->floor_levels : m->ceil_levels;
    const int level_count = floor_uniform ? m->floor_level_count : m->ceil_level_count;
    const int mask_shift = floor_uniform ? 0 : FINE_MASK_LEVELS;
    const int index_shift = floor_uniform ? 16 : 20;
    const float *reach = sc.level_reach + (size_t)local * (m->floor_level_count + m->ceil_level_count) + (floor_uniform ? 0 : m->floor_level_count);
    const float *far = sc.level_far + (size_t)local * (m->floor_level_count + m->ceil_level_count) + (floor_uniform ? 0 : m->floor_level_count);
    // cd = perpendicular / cc below is the hot division.  With y = RN(1 / cc), q = RN(p * y) is within
    // one ulp of p / cc, and RN(q + RN(p - cc * q) * y) is then the correctly rounded quotient
    // (Markstein's theorem; the inner product is exact in an FMA) as long as nothing over- or
    // underflows, which the range tests on both operands ensure.
    const float inv_cc = dm.inverse_cosine[x];
    const bool cc_plain = cc >= 0.5f && cc <= 1.0f;
    const float inv_fine = dm.fine_inverse;       // a reciprocal is fine here: see fine_lookup_cells
    // the probe point camera + ray * cd in raster cell units, as one multiply-add per axis
    const float cell_x0 = (c.x - m->grid_min_x) * inv_fine, cell_y0 = (c.y - m->grid_min_y) * inv_fine;
    const float cell_dx = rc * inv_fine, cell_dy = rs * inv_fine;
    const int slot_in_wave = threadIdx.x & 63;
    // cd <= perpendicular / (smallest cc of the wavefront): with it a level whose every sector is
    // farther than that from the camera is dropped for the whole wavefront at once
    const float reach_scale = dm.strip_reach_scale[__builtin_amdgcn_readfirstlane(x >> 6)];
    // and cd >= perpendicular / (largest cc of the wavefront): a level whose every sector ends nearer than that
    const float far_scale = dm.strip_far_scale[__builtin_amdgcn_readfirstlane(x >> 6)];
    float best = GD_INF; int best_sector = -1;
    const bool camera_in_grid = grid_cell_of(m, c.x, c.y) >= 0;
    bool done = !wanted;
    // The levels some pixel of the wavefront can reach at all (level_bucket): the bit sets of the buckets its 64 scales
    // fall into, joined; lane j holds word j.  Levels outside them are skipped by the whole wavefront at once.
    const int mask_words = MASKS ? level_mask_words(m) : 0;
    constexpr int BATCH = MASKS ? FLAT_BATCH_MASKED : FLAT_BATCH;
    unsigned int joined_word = 0u;
    if (MASKS) {
        const int bucket = level_bucket((192.0f / denom) / cc);
        int lowest = bucket, highest = bucket;
#pragma unroll
        for (int step = 1; step < 64; step <<= 1) { lowest = min(lowest, __shfl_xor(lowest, step)); highest = max(highest, __shfl_xor(highest, step)); }
        const unsigned int *masks = sc.level_masks + (size_t)local * LEVEL_BUCKETS * mask_words;
        if (slot_in_wave < mask_words) for (int b = lowest; b <= highest; ++b) joined_word |= masks[b * mask_words + slot_in_wave];
    }
    const int first_bit = floor_uniform ? 0 : m->floor_level_count;
    for (int base = 0; base < level_count; base += 64) {
        if (__ballot(!done) == 0) break;   // every lane takes part in the level broadcasts below, wanted or not
        u64 chunk_levels = ~0ULL;          // bit k: level base + k is worth a look
        if (MASKS) {
            const int at = first_bit + base, word = at >> 5, shift = at & 31;
            const u64 w0 = (unsigned)bcast((int)joined_word, word), w1 = (unsigned)bcast((int)joined_word, (word + 1) & 63), w2 = (unsigned)bcast((int)joined_word, (word + 2) & 63);
            chunk_levels = ((w0 | (w1 << 32)) >> shift) | (shift ? w2 << (64 - shift) : 0ULL);   // lanes past the last word hold zeros
            if (chunk_levels == 0ULL) continue;    // the same in every lane
        }
        // lane k works out level base+k: its height and perpendicular distance (one division for
        // the wavefront instead of one per level per lane); a level the plane cannot show gets -1
        const int mine = base + slot_in_wave;
        const float my_level = mine < level_count ? levels[mine] : 0.0f;
        const float my_reach = mine < level_count ? reach[mine] : 0.0f;
        const float my_far = mine < level_count ? far[mine] : GD_INF;
        const float my_height = floor_uniform ? (c.view_z - my_level) : (my_level - c.view_z);
        const float my_perpendicular = (mine < level_count && my_height > 0) ? my_height * 192.0f / denom : -1.0f;
        const int chunk = level_count - base < 64 ? level_count - base : 64;
        // Levels are taken BATCH at a time: first the probe points and raster loads of the whole
        // batch (independent, so their memory latencies overlap), then the decisions in level order.
        // A load for a level past the one that ends the scan is wasted, never wrong.
        // Only the levels whose bit is set are walked (with bit sets: the few that some pixel here can reach), so a
        // batch holds BATCH levels that are looked at, not BATCH list positions.  `rest` is the same in every lane.
        if (chunk < 64) chunk_levels &= (1ULL << chunk) - 1ULL;
        u64 rest = ((u64)(unsigned)__builtin_amdgcn_readfirstlane((int)(chunk_levels >> 32)) << 32) | (u64)(unsigned)__builtin_amdgcn_readfirstlane((int)chunk_levels);
        while (rest != 0ULL) {
            if (__ballot(!done) == 0) break;
            float cdv[BATCH];
            unsigned finev[BATCH];
            int cellv[BATCH];
            int kv[BATCH];
#pragma unroll
            for (int j = 0; j < BATCH; ++j) {
                kv[j] = rest ? __ffsll((long long)rest) - 1 : -1;
                rest &= rest - 1ULL;
            }
#pragma unroll
            for (int j = 0; j < BATCH; ++j) {
                const int k = kv[j];
                cdv[j] = -1.0f; finev[j] = 0x40000000u; cellv[j] = -1;
                if (k < 0) continue;                             // the same in every lane
                const float perpendicular = bcast(my_perpendicular, k);
                const float nearest = bcast(my_reach, k);
                if (!(perpendicular > 0)) continue;              // the same in every lane
                if (perpendicular * reach_scale < nearest) continue;   // the same in every lane: no lane can reach the level
                if (perpendicular * far_scale > bcast(my_far, k)) continue;   // the same in every lane: every lane looks past the level
                float cd;
                if (cc_plain && perpendicular >= 1e-18f && perpendicular <= 1e18f) {
                    const float q = perpendicular * inv_cc;
                    cd = __builtin_fmaf(__builtin_fmaf(-cc, q, perpendicular), inv_cc, q);
                } else {
                    cd = perpendicular / cc;
                }
                cdv[j] = cd;
                if (done || !(finitef(cd) && cd > 0) || cd > best || cd < nearest) continue;   // cd < nearest: every sector at this level is farther away
                finev[j] = fine_lookup_cells(m, __builtin_fmaf(cd, cell_dx, cell_x0), __builtin_fmaf(cd, cell_dy, cell_y0), &cellv[j]);
            }
#pragma unroll
            for (int j = 0; j < BATCH; ++j) {
                const int k = kv[j];
                if (k < 0 || done) continue;
                const float cd = cdv[j];
                if (!(finitef(cd) && cd > 0)) continue;
                if (cd > best) { done = true; continue; }        // later levels are at least this far
                const unsigned fine = finev[j];
                const unsigned kind = FINE_KIND(fine);
                if (kind == FINE_EMPTY) continue;                // also levels skipped above
                const float level = bcast(my_level, k);
                if (kind == FINE_DECIDED) {
                    const int s = (int)(fine & 0xFFFFu);
                    const unsigned listed = (fine >> index_shift) & 15u;   // the sector's level index, 15 = not recorded
                    bool same_level = listed == (unsigned)(base + k);
                    if (listed == 15u) same_level = m->sector_heights[2 * s + (floor_uniform ? 0 : 1)] == level;
                    if (same_level && (cd < best || (cd == best && s < best_sector))) { best = cd; best_sector = s; }
                    continue;
                }
                if (kind == FINE_MIXED && !((fine >> (mask_shift + base + k)) & 1u)) continue;   // no sector here has this level
                const float px = c.x + rc * cd, py = c.y + rs * cd;
                int cell = cellv[j];
                if (cell < 0) cell = grid_cell_of(m, px, py);
                // Outside the grid (above, below or right of every linedef) no sector holds the point.  Seen from a
                // camera inside that convex region, the probe points of the levels still to come lie farther
                // along the same ray, which has left the region for good.
                if (cell < 0) { done = camera_in_grid; continue; }
                const int2 range = dm.cell_range[cell];
                for (int it = range.x; it < range.y; ++it) {
                    const int4 item = dm.cell_item[it];
                    const int s = item.x & ~GRID_ALWAYS_INSIDE;
                    const bool same_level = item.y >= 0 ? ((floor_uniform ? (item.y & 0xFFFF) : (item.y >> 16)) == base + k)
                                                        : (m->sector_heights[2 * s + (floor_uniform ? 0 : 1)] == level);
                    if (!same_level) continue;
                    if (cd < best || (cd == best && s < best_sector)) {
                        if ((item.x & GRID_ALWAYS_INSIDE) || inside_edge_copies(dm.cell_edge, item.z, item.w, px, py)) { best = cd; best_sector = s; }
                    }
                }
            }
        }
    }
    return best_sector;
}

// One pixel's flat ray on its own (flat_select_pixel shares work between the 64 pixels of a row): the sector of
// the nearest plane level whose probe point lies in a sector of that level, -1 if there is none
// (engine.py:10981-11024).
// The plane levels of the map and, per lane and level, bounds of the distance from the camera to the sectors of that
// level: floors first, then ceilings, in all three lists.  A pixel's scan reads them level after level, each read
// waiting for the one before (the scan may end at any level), so a block that works on one lane copies them to LDS
// first: with a plane level per sector (several hundred) the scans otherwise spend their time waiting for device memory.
#define FLAT_LDS_LEVELS (32 * LEVEL_MASK_WORDS_MAX)
struct LevelLists { const float *level, *reach, *far; const unsigned int *masks; int floors, ceilings, mask_words; };
struct LevelLds { float lists[3 * FLAT_LDS_LEVELS]; };
__device__ __forceinline__ LevelLists stage_level_lists(const DeviceMap &dm, const Scratch &sc, int local, LevelLds *lds) {
    const gd_map_desc *m = &dm.d;
    LevelLists lists;
    lists.floors = m->floor_level_count; lists.ceilings = m->ceil_level_count;
    lists.mask_words = level_mask_words(m);
    const int total = lists.floors + lists.ceilings;
    const float *reach = sc.level_reach + (size_t)local * total, *far = sc.level_far + (size_t)local * total;
    if (total > FLAT_LDS_LEVELS) {        // read where they are; `level` then only serves the floors (see flat_probe_pixel)
        lists.level = nullptr; lists.reach = reach; lists.far = far; lists.masks = nullptr;   // more levels than the bit sets cover
        return lists;
    }
    for (int k = threadIdx.x; k < total; k += blockDim.x) {
        lds->lists[k] = k < lists.floors ? m->floor_levels[k] : m->ceil_levels[k - lists.floors];
        lds->lists[FLAT_LDS_LEVELS + k] = reach[k];
        lds->lists[2 * FLAT_LDS_LEVELS + k] = far[k];
    }
    const unsigned int *masks = sc.level_masks + (size_t)local * LEVEL_BUCKETS * lists.mask_words;
    lists.level = lds->lists; lists.reach = lds->lists + FLAT_LDS_LEVELS; lists.far = lds->lists + 2 * FLAT_LDS_LEVELS;
    lists.masks = masks;   // one row of a few words per pixel: read where it is
    return lists;   // the caller synchronises the block before the first scan
}

__device__ int flat_probe_pixel(const DeviceMap &dm, const Scratch &sc, const LevelLists &lists, int local, float rc, float rs, float cc, int y) {
    const LaneCtx &c = sc.ctx[local];
    const gd_map_desc *m = &dm.d;
    const float delta = (float)y - flat_center(c);
    const bool is_floor = delta > 0;
    const float denom = fmaxf(fabsf(delta), 0.5f);
    const int first = is_floor ? 0 : lists.floors;
    const float *levels = lists.level ? lists.level + first : (is_floor ? m->floor_levels : m->ceil_levels);
    const int level_count = is_floor ? lists.floors : lists.ceilings;
    const float *reach = lists.reach + first, *far = lists.far + first;
    float best = GD_INF; int best_sector = -1;
    const bool camera_in_grid = grid_cell_of(m, c.x, c.y) >= 0;
    // one level of the scan; true ends it
    auto visit = [&](int k) -> bool {
        const float level = levels[k];
        const float height = is_floor ? (c.view_z - level) : (level - c.view_z);
        if (!(height > 0)) return false;
        const float cd = (height * 192.0f / denom) / cc;
        if (!(finitef(cd) && cd > 0)) return false;
        if (cd > best) return true;                                 // later levels are at least this far
        if (cd < reach[k] || cd > far[k]) return false;            // no sector of this level lies at that distance
        const float px = c.x + rc * cd, py = c.y + rs * cd;
        int cell;
        const unsigned fine = fine_lookup(m, dm.fine_inverse, px, py, &cell);
        const unsigned kind = FINE_KIND(fine);
        if (kind == FINE_EMPTY) return false;
        if (kind == FINE_DECIDED) {
            const int s = (int)(fine & 0xFFFFu);
            if (m->sector_heights[2 * s + (is_floor ? 0 : 1)] == level && (cd < best || (cd == best && s < best_sector))) { best = cd; best_sector = s; }
            return false;
        }
        if (cell < 0) cell = grid_cell_of(m, px, py);
        if (cell < 0) return camera_in_grid;   // outside the grid no sector holds the point; seen from inside it, the ray has left that convex region for good
        const int2 range = dm.cell_range[cell];
        for (int it = range.x; it < range.y; ++it) {
            const int4 item = dm.cell_item[it];
            const int s = item.x & ~GRID_ALWAYS_INSIDE;
            if (m->sector_heights[2 * s + (is_floor ? 0 : 1)] != level) continue;
            if (cd < best || (cd == best && s < best_sector)) {
                if ((item.x & GRID_ALWAYS_INSIDE) || inside_edge_copies(dm.cell_edge, item.z, item.w, px, py)) { best = cd; best_sector = s; }
            }
        }
        return false;
    };
    // With bit sets: only the levels whose distance bounds can hold a probe of this pixel's scale at all (level_bucket),
    // in level order; bits [first, end) of the bucket's row are this half's levels.  Without: every level.
    const bool masked = lists.mask_words > 0 && lists.masks;
    const unsigned int *row = masked ? lists.masks + level_bucket((192.0f / denom) / cc) * lists.mask_words : nullptr;
    const int end = first + level_count;
    int word = (first >> 5) - 1, k = -1;
    unsigned int bits = 0u;
    for (;;) {
        if (masked) {
            while (!bits && word < ((end - 1) >> 5)) {
                ++word;
                bits = row[word];
                if (word == first >> 5) bits &= ~0u << (first & 31);
                if (word == (end - 1) >> 5 && (end & 31)) bits &= (1u << (end & 31)) - 1u;
            }
            if (!bits) break;
            k = (word << 5) + __ffs((int)bits) - 1 - first;
            bits &= bits - 1;
        } else if (++k >= level_count) {
            break;
        }
        if (visit(k)) break;
    }
    return best_sector;
}

// The flat pass runs after the walls and only where its result can matter.  A pixel a wall tier filled never
// shows it; a pixel a plane of the wall pass claimed only asks whether the flat ray resolved at all, and only
// where a sprite stands behind the plane with no sprite clip recorded, which the sprite pass finds out for
// itself (flat_ray_resolves); the few pixels left (columns whose traversal left a gap) show the flat pass's
// picture.  wall_raster_kernel lists those.  flat_gap_column_kernel, one block per lane, first selects them, one
// thread per listed pixel, and notes per screen half and column the topmost one that stayed unresolved.
//
// Then the vertical repair (engine.py:11026-11083) of the listed pixels, column by column.  An unresolved pixel takes
// the sector of the next resolved pixel below it in its half of the screen; when that sector is not the camera's,
// the pixel is its own left and right anchor in the horizontal repair (engine.py:11085-11135), which then leaves
// it as it is: such a pixel is settled here and its row needs no further work.  Only the rows of the others (no
// resolved pixel below, or the camera's own sector) are noted for the row kernels (flat_span_select_kernel,
// flat_tail_kernel, flat_span_finish_kernel).  A wavefront takes one column that holds an unresolved listed pixel
// after another, its lanes probing 64 rows of the column at a time, from the bottom of the half up to the column's
// topmost unresolved listed pixel.
// GAP_THREADS: three wavefronts a lane.  Most lanes have a few dozen listed pixels and one or two columns to repair, and a
// launch lasts as many rounds of blocks as the chip needs to hold them all: with five wavefronts a block (one thread a
// column) it took 0.05 ms longer, with one or two the lanes with many columns hold it up.
#define GAP_THREADS 192
__global__ void __launch_bounds__(GAP_THREADS) __attribute__((amdgpu_waves_per_eu(8, 8))) flat_gap_column_kernel(DeviceMap dm, gd_lanes_desc lanes, int lane_base, int lane_count, Scratch sc) {
    const int local = blockIdx.x;
    if (local >= lane_count) return;
    const int listed = sc.flat_list_count[local];
    if (listed == 0) return;                         // the same in every thread: a lane without gap pixels has no flat pass
    const LaneCtx &c = sc.ctx[local];
    const int n = lane_base + local;
    const int lane_id = threadIdx.x & 63;
    int *span = sc.flat_span + (size_t)local * 4;
    const int last_ceiling_row = c.last_ceiling_row;
    const unsigned int *meta = sc.meta + (size_t)local * VH * SW;
    __shared__ LevelLds level_lds;
    const LevelLists lists = stage_level_lists(dm, sc, local, &level_lds);
    __syncthreads();
    if (listed > FLAT_LIST_MAX) {
        // too many to list (a camera outside the map, say): every row of both halves is selected and repaired
        if (threadIdx.x == 0) {
            if (last_ceiling_row >= 0) { span[0] = 0; span[1] = last_ceiling_row; }
            if (last_ceiling_row + 1 < VH) { span[2] = last_ceiling_row + 1; span[3] = VH - 1; }
        }
    } else {
        for (int slot = threadIdx.x; slot < listed; slot += blockDim.x) {
            const int pixel = sc.flat_list[(size_t)local * FLAT_LIST_MAX + slot];
            const int y = pixel / SW, x = pixel - y * SW;
            const int s = flat_probe_pixel(dm, sc, lists, local, lanes.ray_cos[(size_t)n * SW + x], lanes.ray_sin[(size_t)n * SW + x], dm.cosine_correction[x], y);
            const size_t i = (size_t)local * VH * SW + pixel;
            sc.flat_sector[i] = (unsigned short)(s < 0 ? c.sector : s);
            sc.flat_flags[i] = s < 0 ? 1 : 0;
            if (s < 0) {
                const bool floor_row = ((float)y - flat_center(c)) > 0;
                atomicMin(&sc.flat_col_top[((size_t)local * 2 + (floor_row ? 1 : 0)) * SW + x], y);
            }
        }
    }
    __threadfence_block();   // what the selection wrote (column tops, row ranges) is read below by other threads of the block
    __syncthreads();
    // the lane's columns with work, both halves together, join one work list that flat_gap_repair_kernel deals out to
    // wavefronts evenly, whichever lanes they come from
    __shared__ int column_list[2 * SW];
    __shared__ int column_count, list_base;
    if (threadIdx.x == 0) column_count = 0;
    __syncthreads();
    for (int half = 0; half < 2; ++half) for (int x = threadIdx.x; x < SW; x += blockDim.x) {
        int *top_at = sc.flat_col_top + ((size_t)local * 2 + half) * SW + x;
        const int top = __hip_atomic_load(top_at, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);   // where the atomics above wrote, not a cached copy
        if (top < VH) {
            column_list[atomicAdd(&column_count, 1)] = x | (top << 9) | (half << 17) | (local << 18);
        }
    }
    __syncthreads();
    const int columns = column_count;
    if (columns == 0) return;                        // the same in every thread
    if (threadIdx.x == 0) list_base = atomicAdd(sc.gap_column_count, columns);
    __syncthreads();
    for (int k = threadIdx.x; k < columns; k += blockDim.x) sc.gap_columns[list_base + k] = column_list[k];
}

// The vertical repair (engine.py:11026-11083) of the listed gap pixels, column by column: one work-group per listed column
// (flat_gap_column_kernel's work list), one wavefront per chunk of 64 rows between the column's topmost unresolved listed
// pixel and the bottom of its half, all chunks probed at once.  What a chunk needs from the chunks below it (the sector of
// the next resolved pixel down) goes through LDS once every chunk has probed: a column lasts as long as its slowest
// pixel's walk over the plane levels, not as long as one such walk per chunk.
#define GAP_REPAIR_BLOCKS 8192
#define GAP_REPAIR_CHUNKS ((VH + 63) / 64)
__global__ void __launch_bounds__(64 * GAP_REPAIR_CHUNKS) __attribute__((amdgpu_waves_per_eu(8, 8))) flat_gap_repair_kernel(DeviceMap dm, gd_lanes_desc lanes, int lane_base, Scratch sc) {
    __shared__ LevelLds level_lds;
    __shared__ int chunk_found[GAP_REPAIR_CHUNKS], chunk_sector[GAP_REPAIR_CHUNKS];
    const int total = *sc.gap_column_count;
    const int lane_id = threadIdx.x & 63, chunk = threadIdx.x >> 6;
    int staged = -1;
    LevelLists lists;
    for (int entry = blockIdx.x; entry < total; entry += gridDim.x) {
        const int packed = sc.gap_columns[entry];
        const int x = packed & 511, first = (packed >> 9) & 255, half = (packed >> 17) & 1, local = packed >> 18;
        __syncthreads();         // nobody reads the previous column's chunk results or the previous lane's lists any more
        if (local != staged) {   // the same in every thread
            lists = stage_level_lists(dm, sc, local, &level_lds);
            staged = local;
        }
        __syncthreads();
        const LaneCtx &c = sc.ctx[local];
        const int n = lane_base + local;
        int *span = sc.flat_span + (size_t)local * 4;
        const unsigned int *meta = sc.meta + (size_t)local * VH * SW;
        const int half_end = half ? VH - 1 : c.last_ceiling_row;
        const float rc = lanes.ray_cos[(size_t)n * SW + x], rs = lanes.ray_sin[(size_t)n * SW + x], cc = dm.cosine_correction[x];
        const int chunks = (half_end - first) / 64 + 1;   // at most GAP_REPAIR_CHUNKS
        const int y = first + chunk * 64 + lane_id;
        const bool live = chunk < chunks && y <= half_end;
        const int s = live ? flat_probe_pixel(dm, sc, lists, local, rc, rs, cc, y) : -1;
        const u64 resolved = __ballot(live && s >= 0);
        const int first_sector = __shfl(s, resolved ? __ffsll((long long)resolved) - 1 : 0);
        if (lane_id == 0) { chunk_found[chunk] = resolved != 0; chunk_sector[chunk] = first_sector; }
        __syncthreads();
        // the next resolved pixel below: in this chunk, else the topmost one of the nearest chunk below that has any
        bool below_found = false; int below_sector = 0;
        for (int lower_chunk = chunk + 1; lower_chunk < chunks && !below_found; ++lower_chunk)
            if (chunk_found[lower_chunk]) { below_found = true; below_sector = chunk_sector[lower_chunk]; }
        const u64 lower = resolved & ~((2ULL << lane_id) - 1);   // resolved rows of this chunk below this one (none for lane 63)
        const int from = lower ? __ffsll((long long)lower) - 1 : lane_id;
        const int taken = __shfl(s, from);
        const bool found = lower ? true : below_found;
        const int sector = lower ? taken : below_sector;
        if (live && s < 0) {
            const size_t i = (size_t)y * SW + x;
            const unsigned int word = meta[i];
            const bool listed = !(word & (META_FILLED | META_MASKED)) && ((word >> META_SECTOR_SHIFT) & META_SECTOR_MASK) == 0;
            if (listed) {
                if (found && sector != c.sector) {
                    sc.flat_sector[(size_t)local * VH * SW + i] = (unsigned short)sector;
                    sc.flat_flags[(size_t)local * VH * SW + i] = (unsigned char)(1 | 2 | 4 | 8);
                } else {
                    atomicMin(&span[half ? 2 : 0], y);
                    atomicMax(&span[half ? 3 : 1], y);
                }
            }
        }
    }
}

// The lanes' row ranges are final once every listed column is repaired: their rows join the work list that
// flat_span_select_kernel deals out evenly, whichever lanes they come from.  One wavefront per lane.
__global__ void __launch_bounds__(64) flat_rows_kernel(int lane_count, Scratch sc) {
    const int local = blockIdx.x;
    if (local >= lane_count) return;
    const int *span = sc.flat_span + (size_t)local * 4;
    const int lo0 = span[0], hi0 = span[1], lo1 = span[2], hi1 = span[3];
    const int rows0 = hi0 < lo0 ? 0 : hi0 - lo0 + 1, rows1 = hi1 < lo1 ? 0 : hi1 - lo1 + 1;
    if (rows0 + rows1 == 0) return;                  // the same in every thread
    int list_base = 0;
    if (threadIdx.x == 0) list_base = atomicAdd(sc.flat_row_count, rows0 + rows1);
    list_base = __shfl(list_base, 0);
    for (int r = threadIdx.x; r < rows0 + rows1; r += blockDim.x)
        sc.flat_rows[list_base + r] = (local << 8) | (r < rows0 ? lo0 + r : lo1 + (r - rows0));
}

// Small per-sector / per-texture tables staged in LDS by the kernels whose inner loops chase
// them (a dependent global gather costs ~500 cycles, an LDS read ~60).  Sectors or textures
// beyond the staged count fall back to the global arrays.
struct Tables {
    const gd_map_desc *m;
    const float4 *sector;          // floor, ceiling, light, bits(floor_tex | ceil_tex << 16)
    const unsigned char *tex_bits; // floor(log2 width) | floor(log2 height) << 4
    const unsigned int *tex_odd;   // bit t: the width of texture t is no power of two
    int sector_cached, tex_cached;
    __device__ __forceinline__ float floor_h(int s) const { return s < sector_cached ? sector[s].x : m->sector_heights[2 * s]; }
    __device__ __forceinline__ float ceil_h(int s) const { return s < sector_cached ? sector[s].y : m->sector_heights[2 * s + 1]; }
    __device__ __forceinline__ float light(int s) const { return s < sector_cached ? sector[s].z : m->sector_lights[s]; }
    __device__ __forceinline__ int floor_tex(int s) const { return s < sector_cached ? (int)(__float_as_uint(sector[s].w) & 0xFFFFu) : m->sector_floor_tex[s]; }
    __device__ __forceinline__ int ceil_tex(int s) const { return s < sector_cached ? (int)(__float_as_uint(sector[s].w) >> 16) : m->sector_ceil_tex[s]; }
    __device__ __forceinline__ int width_bits(int t) const { return t < tex_cached ? (tex_bits[t] & 15) : ilog2(m->tex_w[t]); }
    __device__ __forceinline__ int height_bits(int t) const { return t < tex_cached ? (tex_bits[t] >> 4) : ilog2(m->tex_h[t]); }
    // Texture column of a wall: torch.remainder(u, width) (engine.py:12792-12798).  Widths are powers of two
    // on most maps, where the remainder is a mask; WAD textures of other widths take the division.
    __device__ __forceinline__ i64 wrap_column(int t, i64 u) const {
        const bool odd = t < tex_cached ? ((tex_odd[t >> 5] >> (t & 31)) & 1u) != 0 : (m->tex_w[t] & (m->tex_w[t] - 1)) != 0;
        if (!odd) return u & (i64)((1 << width_bits(t)) - 1);
        const i64 width = m->tex_w[t];
        const i64 r = u - tdiv(u, width) * width;
        return r < 0 ? r + width : r;
    }
};

// Cooperative fill of the LDS tables by the whole block (call before a __syncthreads()).
struct TexLds { unsigned char bits[LDS_TEXTURES]; unsigned int odd[LDS_TEXTURES / 32]; };   // 252 bytes: plane_shade_kernel's LDS budget is exact
__device__ __forceinline__ void stage_tables(const gd_map_desc *m, float4 *sector_lds, TexLds *tex_lds, Tables &tb) {
    int sectors = m->sector_count < LDS_SECTORS ? m->sector_count : LDS_SECTORS;
    int textures = m->texture_count < LDS_TEXTURES ? m->texture_count : LDS_TEXTURES;
    for (int s = threadIdx.x; s < sectors; s += blockDim.x) {
        float4 v;
        v.x = m->sector_heights[2 * s]; v.y = m->sector_heights[2 * s + 1]; v.z = m->sector_lights[s];
        v.w = __uint_as_float(((unsigned)m->sector_floor_tex[s] & 0xFFFFu) | ((unsigned)m->sector_ceil_tex[s] << 16));
        sector_lds[s] = v;
    }
    for (int t = threadIdx.x; t < textures; t += blockDim.x) tex_lds->bits[t] = (unsigned char)(ilog2(m->tex_w[t]) | (ilog2(m->tex_h[t]) << 4));
    for (int k = threadIdx.x; k < LDS_TEXTURES / 32; k += blockDim.x) {
        unsigned int odd = 0;
        for (int t = 32 * k; t < 32 * k + 32 && t < textures; ++t) odd |= (m->tex_w[t] & (m->tex_w[t] - 1)) ? 1u << (t & 31) : 0u;
        tex_lds->odd[k] = odd;
    }
    tb.m = m; tb.sector = sector_lds; tb.tex_bits = tex_lds->bits; tb.tex_odd = tex_lds->odd; tb.sector_cached = sectors; tb.tex_cached = textures;
}

// engine.py:10879-10954
__device__ __forceinline__ void flat_texture_coordinates(const Tables &tb, const LaneCtx &c, int texture_id, float plane_height, int px, int py, i64 *u, i64 *v) {
    int width_bits = tb.width_bits(texture_id);
    int height_bits = tb.height_bits(texture_id);
    i64 xscale = shl64(1, 32 - width_bits), yscale = shl64(1, 32 - height_bits);
    i64 xstep_scale = tdiv(mul64(xscale, c.vsin), FOCAL_X_FIXED);
    i64 ystep_scale = tdiv(mul64(yscale, c.vcos), FOCAL_X_FIXED);
    i64 flat_column = (i64)px - (SW / 2 - 1);
    i64 basexfrac = (mul64(xscale, c.vcos) >> 16) + mul64(flat_column, xstep_scale);
    i64 baseyfrac = (mul64(yscale, -c.vsin) >> 16) + mul64(flat_column, ystep_scale);
    i64 pviewx = mul64(xscale, c.view_x_fixed) >> 16;
    i64 pviewy = mul64(yscale, -c.view_y_fixed) >> 16;
    i64 center_row = c.center_fixed >> 16;
    i64 pixel_y_fixed = (i64)py * FIXED_UNIT;
    i64 den = (py < center_row) ? (c.center_fixed - pixel_y_fixed - FIXED_UNIT / 2) : (pixel_y_fixed - c.center_fixed + FIXED_UNIT / 2);
    den = max64(den, 1);
    bool overflow = den <= (FOCAL_Y_FIXED >> 15);
    i64 yslope = tdiv(FOCAL_Y_FIXED << 16, den);
    if (overflow) yslope = (1LL << 31) - 1;
    i64 plane_height_fixed = round_to_i64(plane_height * 65536.0f);
    i64 distance = mul64(plane_height_fixed, yslope) >> 16;
    i64 xfrac = ((mul64(distance, basexfrac) >> 16) + pviewx) & UINT32_MASK;
    i64 yfrac = ((mul64(distance, baseyfrac) >> 16) + pviewy) & UINT32_MASK;
    *u = xfrac >> (32 - width_bits);
    *v = yfrac >> (32 - height_bits);
}

// engine.py:10588-10616
__device__ __forceinline__ unsigned char plane_colormap(const unsigned char *colormap, const LaneCtx &c, unsigned char index, float light, float plane_height, int py) {
    i64 plane_height_fixed = round_to_i64(plane_height * 65536.0f);
    i64 glob = min64(tdiv(FLOOR_VISIBILITY_FIXED << 16, max64(plane_height_fixed, 1)), (1LL << 31) - 1);
    i64 row = c.center_fixed - (i64)py * FIXED_UNIT;
    if (row < 0) row = -row;
    i64 visibility = min64(mul64(glob, row) >> 16, 24 * FIXED_UNIT);
    i64 plane_shade = 64 * FIXED_UNIT - ((i64)light + 12) * (FIXED_UNIT / 4);
    i64 shade = clampi((plane_shade - visibility) >> 16, 0, 31);
    return colormap[shade * 256 + index];
}

__device__ __forceinline__ unsigned char flat_pixel(const Tables &tb, const unsigned char *colormap, const LaneCtx &c, int sector, bool is_floor, int px, int py) {
    const gd_map_desc *m = tb.m;
    float plane_height = is_floor ? (c.view_z - tb.floor_h(sector)) : (tb.ceil_h(sector) - c.view_z);
    int texture = is_floor ? tb.floor_tex(sector) : tb.ceil_tex(sector);
    i64 u, v;
    flat_texture_coordinates(tb, c, texture, plane_height, px, py, &u, &v);
    unsigned char index = m->tex_atlas[((size_t)texture * m->tex_max_h + v) * m->tex_max_w + u];
    float light = tb.light(sector) + (float)(c.flash_light * 16);
    return plane_colormap(colormap, c, index, light, plane_height, py);
}

// flat_pixel with every division looked up: the lane's per-level, per-row and per-size tables
// hold exactly the quotients flat_texture_coordinates and plane_colormap would compute, and a
// product with a power-of-two texture scale is a shift.
struct LaneTables {
    const i64 *level_plane;   // this lane's [levels][2]
    const i64 *step_scale;    // this lane's [3][2][16]
    int floors;
};
// Returns the texel's offset in the texture atlas and the colormap row, so that a caller can
// have several texel loads in flight before it needs any of them.
__device__ __forceinline__ size_t flat_sample_tabled(const Tables &tb, const LaneCtx &c, const LaneTables &lt,
                                                     i64 yslope, int level_index, int sector, bool is_floor, int px, int py, int *colormap_row) {
    const gd_map_desc *m = tb.m;
    const int texture = is_floor ? tb.floor_tex(sector) : tb.ceil_tex(sector);
    const int width_bits = tb.width_bits(texture), height_bits = tb.height_bits(texture);
    const i64 *plane = lt.level_plane + 2 * (is_floor ? level_index : lt.floors + level_index);
    const i64 plane_height_fixed = plane[0], glob = plane[1];
    // The same integers as flat_texture_coordinates, with narrower multiplies: base + (px - 159) * step is
    // (base - 159 * step) + px * step; the row slope and the visibility factor are below 2^31 and not negative
    // (lane_tables_kernel clamps both); of distance * basefrac only bits 16..47 reach the texel coordinate.
    const i64 xstep_scale = lt.step_scale[width_bits], ystep_scale = lt.step_scale[16 + height_bits];
    const i64 basexfrac = lt.step_scale[32 + width_bits] + mul64_u32(xstep_scale, (unsigned)px);
    const i64 baseyfrac = lt.step_scale[48 + height_bits] + mul64_u32(ystep_scale, (unsigned)px);
    const unsigned pviewx = (unsigned)lt.step_scale[64 + width_bits], pviewy = (unsigned)lt.step_scale[80 + height_bits];
    const i64 distance = mul64_u32(plane_height_fixed, (unsigned)yslope) >> 16;
    const unsigned xfrac = mul64_bits_16_47(distance, basexfrac) + pviewx;
    const unsigned yfrac = mul64_bits_16_47(distance, baseyfrac) + pviewy;
    const unsigned u = (xfrac >> (31 - width_bits)) >> 1, v = (yfrac >> (31 - height_bits)) >> 1;   // two shifts: a size of one shifts by 32
    const float light = tb.light(sector) + (float)(c.flash_light * 16);
    i64 row = c.center_fixed - (i64)py * FIXED_UNIT;
    if (row < 0) row = -row;
    const i64 visibility = min64(mul64_u32(row, (unsigned)glob) >> 16, 24 * FIXED_UNIT);
    const i64 plane_shade = 64 * FIXED_UNIT - ((i64)light + 12) * (FIXED_UNIT / 4);
    *colormap_row = (int)clampi((plane_shade - visibility) >> 16, 0, 31);
    return (size_t)(((unsigned)texture * (unsigned)m->tex_max_h + v) * (unsigned)m->tex_max_w + u);   // the atlas is below 4 GiB (checked at create)
}

// flat_sample_tabled for a run of neighbouring pixels of one row that show the same plane: what depends on the row and the
// plane is worked out once (plane_span), each pixel then costs two 64-bit additions and two products (plane_span_texel).
// The same integers: base + px * step is (base + px0 * step) + k * step in 64-bit arithmetic.
struct PlaneSpan {
    i64 distance, xfrac_base, yfrac_base, xstep, ystep;
    unsigned pviewx, pviewy, texture_row0, atlas_width;
    int width_shift, height_shift, colormap_row;
};
__device__ __forceinline__ PlaneSpan plane_span(const Tables &tb, const LaneCtx &c, const LaneTables &lt, i64 yslope, int level_index, int sector,
                                                bool is_floor, int px0, int py) {
    const gd_map_desc *m = tb.m;
    PlaneSpan s;
    const int texture = is_floor ? tb.floor_tex(sector) : tb.ceil_tex(sector);
    const int width_bits = tb.width_bits(texture), height_bits = tb.height_bits(texture);
    const i64 *plane = lt.level_plane + 2 * (is_floor ? level_index : lt.floors + level_index);
    const i64 plane_height_fixed = plane[0], glob = plane[1];
    s.xstep = lt.step_scale[width_bits]; s.ystep = lt.step_scale[16 + height_bits];
    s.xfrac_base = lt.step_scale[32 + width_bits] + mul64_u32(s.xstep, (unsigned)px0);
    s.yfrac_base = lt.step_scale[48 + height_bits] + mul64_u32(s.ystep, (unsigned)px0);
    s.pviewx = (unsigned)lt.step_scale[64 + width_bits]; s.pviewy = (unsigned)lt.step_scale[80 + height_bits];
    s.distance = mul64_u32(plane_height_fixed, (unsigned)yslope) >> 16;
    s.width_shift = 31 - width_bits; s.height_shift = 31 - height_bits;
    const float light = tb.light(sector) + (float)(c.flash_light * 16);
    i64 row = c.center_fixed - (i64)py * FIXED_UNIT;
    if (row < 0) row = -row;
    const i64 visibility = min64(mul64_u32(row, (unsigned)glob) >> 16, 24 * FIXED_UNIT);
    const i64 plane_shade = 64 * FIXED_UNIT - ((i64)light + 12) * (FIXED_UNIT / 4);
    s.colormap_row = (int)clampi((plane_shade - visibility) >> 16, 0, 31);
    s.texture_row0 = (unsigned)texture * (unsigned)m->tex_max_h; s.atlas_width = (unsigned)m->tex_max_w;
    return s;
}
__device__ __forceinline__ unsigned plane_span_texel(const PlaneSpan &s, int k) {   // pixel px0 + k
    const unsigned xfrac = mul64_bits_16_47(s.distance, s.xfrac_base + mul64_u32(s.xstep, (unsigned)k)) + s.pviewx;
    const unsigned yfrac = mul64_bits_16_47(s.distance, s.yfrac_base + mul64_u32(s.ystep, (unsigned)k)) + s.pviewy;
    const unsigned u = (xfrac >> s.width_shift) >> 1, v = (yfrac >> s.height_shift) >> 1;   // two shifts: a size of one shifts by 32
    return (s.texture_row0 + v) * s.atlas_width + u;   // the atlas is below 4 GiB (checked at create)
}

// Visplane repair (engine.py:11026-11135) of the row ranges flat_select_kernel noted, one block per lane, one
// wavefront per 64 columns.  Every pixel of those rows is selected first (the repairs read whole rows and
// columns).  Vertical: an unresolved pixel takes the sector of the next resolved pixel below it in its half of
// the screen; rows below the noted range are selected one at a time until every column that still looks for
// one has found it.  Horizontal: an unresolved pixel between a left and a right anchor of one sector takes
// that sector.  Pixels outside the noted rows need none of this: no shown pixel there is unresolved, and
// resolved pixels are never repaired.
// Every pixel of the noted rows: the blocks take the rows of the work list in turn, so that lanes with many rows
// and lanes with none load the chip alike.  One block per row at a time, one wavefront per 64 columns.
template <bool MASKS>
__global__ void __launch_bounds__(SW) __attribute__((amdgpu_waves_per_eu(8, 8))) flat_span_select_kernel(DeviceMap dm, gd_lanes_desc lanes, int lane_base, int lane_count, Scratch sc) {
    const int total = *sc.flat_row_count;
    const int x = threadIdx.x;
    for (int entry = blockIdx.x; entry < total; entry += gridDim.x) {
        const int packed = sc.flat_rows[entry];
        const int local = packed >> 8, y = packed & 255;
        const int s = flat_select_pixel<MASKS>(dm, sc, lanes, local, lane_base + local, x, y, true);
        const size_t i = (size_t)local * VH * SW + (size_t)y * SW + x;
        sc.flat_sector[i] = (unsigned short)(s < 0 ? sc.ctx[local].sector : s);
        sc.flat_flags[i] = s < 0 ? 1 : 0;
    }
}

// A column whose pixel in the last noted row of a half is unresolved looks further down for a resolved one
// (engine.py:11026-11083).  One block per (lane, 64-column strip); its tail_rows() wavefronts select that many rows
// at a time, while any of the strip's columns is still looking.  Eight rows a step suit maps with few plane levels, where
// a resolved row is usually near; with a level per sector a search runs further and sixteen are quicker.
constexpr int tail_rows(bool masks) { return masks ? 16 : 8; }
template <bool MASKS>
__global__ void __launch_bounds__(64 * tail_rows(MASKS)) flat_tail_kernel(DeviceMap dm, gd_lanes_desc lanes, int lane_base, int lane_count, Scratch sc) {
    constexpr int TAIL_ROWS = tail_rows(MASKS);
    __shared__ int found_lds[TAIL_ROWS][64];
    const int local = blockIdx.y;
    if (local >= lane_count) return;
    const int *span = sc.flat_span + (size_t)local * 4;
    const int lo[2] = {span[0], span[2]}, hi[2] = {span[1], span[3]};
    if (hi[0] < lo[0] && hi[1] < lo[1]) return;      // the same in every thread
    const int n = lane_base + local;
    const int slot = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int x = blockIdx.x * 64 + slot;
    const int last_ceiling_row = sc.ctx[local].last_ceiling_row;
    for (int half = 0; half < 2; ++half) {
        if (hi[half] < lo[half]) continue;           // the same in every thread
        const int half_end = half ? VH - 1 : last_ceiling_row;
        bool looking = sc.flat_flags[(size_t)local * VH * SW + (size_t)hi[half] * SW + x] & 1;
        int found = -1;
        for (int y0 = hi[half] + 1; y0 <= half_end; y0 += TAIL_ROWS) {
            if (!__syncthreads_or(looking)) break;   // also keeps the rows of the previous step apart from this one's
            const int y = y0 + wave;
            int s = -1;
            if (y <= half_end) s = flat_select_pixel<MASKS>(dm, sc, lanes, local, n, x, y, looking);   // the same in a whole wavefront
            found_lds[wave][slot] = s;
            __syncthreads();
            if (looking) {
                for (int j = 0; j < TAIL_ROWS; ++j) {
                    const int below = found_lds[j][slot];
                    if (below >= 0) { looking = false; found = below; break; }
                }
            }
        }
        __syncthreads();
        if (wave == 0) sc.flat_tail[((size_t)local * 2 + half) * SW + x] = found;
    }
}

__global__ void __launch_bounds__(SW) flat_span_finish_kernel(DeviceMap dm, gd_lanes_desc lanes, int lane_base, int lane_count, Scratch sc) {
    const int local = blockIdx.x;
    if (local >= lane_count) return;
    const int *span = sc.flat_span + (size_t)local * 4;
    const int lo[2] = {span[0], span[2]}, hi[2] = {span[1], span[3]};
    if (hi[0] < lo[0] && hi[1] < lo[1]) return;      // the same in every thread
    const LaneCtx c = sc.ctx[local];
    const int n = lane_base + local;
    unsigned short *sector = sc.flat_sector + (size_t)local * VH * SW;
    unsigned char *flags = sc.flat_flags + (size_t)local * VH * SW;
    const int x = threadIdx.x;
    const int last_ceiling_row = c.last_ceiling_row;
    // --- vertical (engine.py:11026-11083): floors and ceilings alike look downwards, within their own half
    for (int half = 0; half < 2; ++half) {
        if (hi[half] < lo[half]) continue;           // the same in every thread
        const int half_end = half ? VH - 1 : last_ceiling_row;
        // what flat_tail_kernel found below the range for a column whose pixel in the range's last row is unresolved
        const int below = sc.flat_tail[((size_t)local * 2 + half) * SW + x];
        bool found = below >= 0;
        int span_sector = found ? below : 0;
        // eight rows at a time, their loads first: a column's rows are its own, so no store of the loop touches them
        for (int y0 = hi[half]; y0 >= lo[half]; y0 -= 8) {
            unsigned char row_flags[8]; unsigned short row_sector[8];
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const int y = y0 - j < lo[half] ? lo[half] : y0 - j;
                row_flags[j] = flags[(size_t)y * SW + x]; row_sector[j] = sector[(size_t)y * SW + x];
            }
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const int y = y0 - j;
                if (y < lo[half]) break;
                const size_t i = (size_t)y * SW + x;
                if (!(row_flags[j] & 1)) { found = true; span_sector = row_sector[j]; }
                else if (found) {
                    sector[i] = (unsigned short)span_sector;
                    // bit1: vertical span; bit2: its sector differs from the camera's (anchor)
                    flags[i] = (unsigned char)(1 | 2 | ((span_sector != c.sector) ? 4 : 0));
                }
            }
        }
    }
    __syncthreads();
    // --- horizontal (engine.py:11085-11135): between a left and a right anchor of one sector
    {
        const int lane_id = threadIdx.x & 63;
        const int wave = threadIdx.x >> 6;
        const int rows0 = hi[0] < lo[0] ? 0 : hi[0] - lo[0] + 1, rows1 = hi[1] < lo[1] ? 0 : hi[1] - lo[1] + 1;
        for (int r = wave; r < rows0 + rows1; r += SW / 64) {
            const int y = r < rows0 ? lo[0] + r : lo[1] + (r - rows0);
            unsigned short *row_sector = sector + (size_t)y * SW;
            unsigned char *row_flags = flags + (size_t)y * SW;
            u64 anchors[5];
            unsigned char f[5];
#pragma unroll
            for (int k = 0; k < 5; ++k) f[k] = row_flags[k * 64 + lane_id];
#pragma unroll
            for (int k = 0; k < 5; ++k) {
                bool anchor = !(f[k] & 1) || (f[k] & 4);
                anchors[k] = __ballot(anchor);
            }
            for (int k = 0; k < 5; ++k) {
                if (!(f[k] & 1)) continue;
                int col = k * 64 + lane_id;
                // nearest anchor at or left of col
                int left = -1;
                u64 below = anchors[k] & ((lane_id == 63) ? ~0ULL : ((1ULL << (lane_id + 1)) - 1));
                if (below) left = k * 64 + 63 - __clzll(below);
                else for (int j = k - 1; j >= 0 && left < 0; --j) if (anchors[j]) left = j * 64 + 63 - __clzll(anchors[j]);
                int right = SW;
                u64 above = anchors[k] & ~((1ULL << lane_id) - 1);
                if (above) right = k * 64 + __ffsll((long long)above) - 1;
                else for (int j = k + 1; j < 5 && right >= SW; ++j) if (anchors[j]) right = j * 64 + __ffsll((long long)anchors[j]) - 1;
                if (left >= 0 && right < SW) {
                    int ls = row_sector[left], rs_ = row_sector[right];
                    // anchors are never rewritten by this pass, so reading them while other
                    // lanes write their own unresolved pixels is race free
                    if (ls == rs_) { row_sector[col] = (unsigned short)ls; row_flags[col] = (unsigned char)(f[k] | 8); }
                }
            }
        }
    }
}

// ---------------------------------------------------------------------------------------------
// walls: engine.py:11462-13745
// ---------------------------------------------------------------------------------------------
#define CAND_BATCH 8
#define SELECT_STAGED_STRIPS 512   // wall_select_kernel's launch for the longest strips: how many strips,
#define SELECT_STAGED_PARTS 4      // and over how many wavefronts each is shared out
#define WALL_ROWS 8          // rows painted / clipped per step of the wall traversal
struct ColumnCtx {
    const Tables *tb;
    const gd_map_desc *m;
    MapView mv;
    const LaneCtx *c;
    const WallRec *recs;  // the chunk's [L,W] records, with rec_base = lane * W
    const RecSpan *spans; // the chunk's [L,W] ray-test facts of every linedef
    const WallRec *frags; // this lane's [split_count, fragment_slots] fragment records
    const Cand *list;     // the chunk's candidate blocks; entry k of this column sits list_column + k * 320 * 16 bytes in
    unsigned rec_base, list_column;
    int count;
    int x;
    float rx, ry;
    // wall_select_kernel's staged launch: this column's list copied to LDS (entry k at staged + k * 256 bytes: a row of
    // the wavefront's 16 columns), unused everywhere else.  (One or the other for a whole kernel: a choice per load would become one flat
    // load of a selected address.)
    typedef __attribute__((address_space(3))) const char LdsByte;
    LdsByte *staged;
    bool use_staged = false;
    __device__ __forceinline__ const WallRec &rec(int w) const { return recs[rec_base + (unsigned)w]; }
    // Where the list of column `x` of the chunk's lane `local` starts and how many entries it has: the column's own
    // slots, or its slot in the spill pool.
    __device__ __forceinline__ void set_list(const Scratch &sc, int local, int column) {
        list = sc.cand;
        const int listed = sc.cand_count[(size_t)local * SW + column];
        const unsigned spill = (unsigned)listed >> SPILL_SHIFT;
        if (spill) {
            const unsigned slot = spill - 1;
            list_column = (sc.spill_base + (slot / SW) * (unsigned)(SPILL_DEPTH * SW) + slot % SW) * 16u;
            count = listed & ((1 << SPILL_SHIFT) - 1);
        } else {
            list_column = ((unsigned)local * (CAND_MAX * SW) + (unsigned)column) * 16u;
            count = listed < CAND_MAX ? listed : CAND_MAX;
        }
    }
    __device__ __forceinline__ Cand cand(int k) const {
        typedef unsigned int Words4 __attribute__((ext_vector_type(4)));
        typedef __attribute__((address_space(3))) const Words4 LdsEntry;
        union { uint4 raw; Words4 words; Cand c; } u;
        if (use_staged) u.words = *(LdsEntry *)(staged + (unsigned)k * (64 / SELECT_STAGED_PARTS * 16u));   // all of the list is there
        else u.raw = *reinterpret_cast<const uint4 *>(reinterpret_cast<const char *>(list) + (list_column + (unsigned)k * (SW * 16u)));   // one 16-byte load
        return u.c;
    }
    // Entries k0 .. k0+CAND_BATCH-1 of this column's list, loaded together so that their memory
    // latencies overlap; slots past the end repeat the last entry (callers skip them).
    __device__ __forceinline__ void cand_batch(int k0, Cand (&out)[CAND_BATCH]) const {
#pragma unroll
        for (int j = 0; j < CAND_BATCH; ++j) out[j] = cand(k0 + j < count ? k0 + j : count - 1);
    }
    // The next CAND_BATCH entries named by the bits of `rest` (list positions, ascending), loaded together;
    // slot j is absent where at[j] < 0.
    __device__ __forceinline__ void cand_batch_of(u64 &rest, Cand (&out)[CAND_BATCH], int (&at)[CAND_BATCH]) const {
#pragma unroll
        for (int j = 0; j < CAND_BATCH; ++j) {
            at[j] = rest ? __ffsll((long long)rest) - 1 : -1;
            rest &= rest - 1;
        }
#pragma unroll
        for (int j = 0; j < CAND_BATCH; ++j) out[j] = cand(at[j] < 0 ? 0 : at[j]);
    }
    __device__ Eval eval(int w) const { return eval_wall(m, *c, spans + rec_base, x, w, rx, ry); }
};

// The projection fragment of a linedef at one column (engine.py:11511-11529, 12324-12376): the first
// present fragment whose half-open span holds the column.  A linedef that was never split is its own
// fragment.  `has` is false where no fragment holds the column (OWallMost then falls back to the whole
// linedef, engine.py:12598-12604); `lights` tells whether wallscan light interpolates over the fragment,
// which only linedefs with several fragments do (engine.py:11530-11545).
struct FragmentChoice {
    const WallRec *rec;
    bool has, lights;
};
// SPLIT is false for maps without split linedefs, whose kernels then carry none of the search.
template <bool SPLIT>
__device__ __forceinline__ FragmentChoice choose_fragment(const gd_map_desc *m, const WallRec *frags, const WallRec &whole, int w, int x) {
    FragmentChoice f;
    f.rec = &whole; f.lights = false;
    f.has = (whole.sr > whole.sl) && (x >= whole.sl) && (x < whole.sr);
    if (SPLIT && (whole.flags & WF_SPLIT)) {
        const int F = m->fragment_slots, row = m->wall_split_slot[w];
        int count = 0;
        f.has = false;
        for (int k = 0; k < F; ++k) {
            if (!m->split_fragment_mask[row * F + k]) continue;
            ++count;
            const WallRec &g = frags[row * F + k];
            if (!f.has && (g.sr > g.sl) && (x >= g.sl) && (x < g.sr)) { f.rec = &g; f.has = true; }
        }
        f.lights = f.has && count > 1;
        if (!f.has) f.rec = &whole;
    }
    return f;
}

// engine.py:11217-11291 for one endpoint order, evaluated at one column
__device__ i64 wall_visibility(const WallRec &r, int side, int x) {
    i64 tx1 = side ? r.tx1 : r.tx0, tx2 = side ? r.tx0 : r.tx1;
    i64 ty1 = side ? r.ty1 : r.ty0, ty2 = side ? r.ty0 : r.ty1;
    const i64 center = 160 * FIXED_UNIT;
    i64 safe_ty1 = ty1 == 0 ? 1 : ty1, safe_ty2 = ty2 == 0 ? 1 : ty2;
    i64 left_projected = ((center + tdiv(tx1 * center, safe_ty1)) >> 16) + (tx1 >= 0);
    i64 right_projected = ((center + tdiv(tx2 * center, safe_ty2)) >> 16) + (tx2 >= 0);
    i64 left_den = tx1 - tx2 - ty2 + ty1, right_den = ty2 - ty1 - tx2 + tx1;
    i64 safe_left_den = left_den == 0 ? 1 : left_den, safe_right_den = right_den == 0 ? 1 : right_den;
    bool left_inside = tx1 >= -ty1, right_inside = tx2 <= ty2;
    i64 wsl = left_inside ? left_projected : 0;
    i64 wsr = right_inside ? right_projected : SW;
    i64 wdl = left_inside ? ty1 : ty1 + tdiv((ty2 - ty1) * (tx1 + ty1), safe_left_den);
    i64 wdr = right_inside ? ty2 : ty1 + tdiv((ty2 - ty1) * (tx1 - ty1), safe_right_den);
    i64 light_left = tdiv(WALL_VISIBILITY_FIXED << 12, max64(wdl, 1));
    i64 light_right = tdiv(WALL_VISIBILITY_FIXED << 12, max64(wdr, 1));
    i64 light_step = tdiv(light_right - light_left, max64(wsr - wsl, 1));
    return light_left + ((i64)x - wsl) * light_step;
}

// engine.py:10672-10739 (PrepWall) for one (linedef, column)
__device__ void texture_mapping(const gd_map_desc *m, const WallRec &r, int w, int x, i64 *hoff, i64 *vstep) {
    const float wall_map_scale = (float)((320 * 200.0 / 320.0 / 240) * 64.0 / (320 / 2.0));
    i64 tx1 = r.tx0, tx2 = r.tx1, ty1 = r.ty0, ty2 = r.ty1;
    double u_over_z_origin = (double)((float)tx1 * 160.0f);
    float u_over_z_step_f = -(float)ty1;
    double u_over_z_step = (double)u_over_z_step_f;
    double inv_z_origin = (double)((float)(tx1 - tx2) * 160.0f);
    float inv_z_step_float = (float)(ty2 - ty1);
    double inv_z_step = (double)inv_z_step_float;
    double depth_scale = (double)(inv_z_step_float * wall_map_scale);
    double depth_origin = (double)(-u_over_z_step_f * wall_map_scale);
    double repeat = (double)round_to_i64(m->wall_len[w] * 65536.0f);
    double column = (double)x - 160.0;
    double top = u_over_z_origin + u_over_z_step * column;
    double bottom = inv_z_origin + inv_z_step * column;
    double safe_bottom = bottom == 0 ? 1.0 : bottom;
    double fraction = top / safe_bottom;
    *hoff = f64_to_i64(floor(fraction * repeat + 0.5));
    *vstep = f64_to_i64(floor(fraction * depth_scale + depth_origin + 0.5));
}

// engine.py:12294-12605 (OWallMost) for one column
__device__ __forceinline__ float project(const LaneCtx &c, const WallRec &g, const FragmentChoice &fragment, float world_z, int x) {
    i64 whole_sl = g.sl, whole_sr = g.sr;
    i64 whole_dl = max64(g.dl, 1), whole_dr = max64(g.dr, 1);
    const bool has_fragment = fragment.has;
    const WallRec &f = *fragment.rec;
    i64 screen_left = f.sl, screen_right = f.sr, depth_left = max64(f.dl, 1), depth_right = max64(f.dr, 1);
    i64 relative_z_fixed = round_to_i64((world_z - c.view_z) * 65536.0f);
    i64 pz = -(relative_z_fixed >> 4);
    i64 center_fixed = c.center_fixed;
    i64 px = x;
    if (!has_fragment) {
        i64 original_span = max64(whole_sr - whole_sl, 1);
        i64 opl = tdiv(mul64(pz, FOCAL_Y_FIXED), whole_dl);
        i64 opr = tdiv(mul64(pz, FOCAL_Y_FIXED), whole_dr);
        i64 ostep = tdiv(opr - opl, original_span);
        return (float)clampi((center_fixed + opl + mul64(px - whole_sl, ostep)) >> 16, 0, VH);
    }
    const i64 upper_clip = c.upper_clip, lower_clip = c.lower_clip;
    i64 upper_left = mul64(upper_clip, depth_left) >> 16, upper_right = mul64(upper_clip, depth_right) >> 16;
    i64 lower_left = mul64(lower_clip, depth_left) >> 16, lower_right = mul64(lower_clip, depth_right) >> 16;
    bool above_left = pz < upper_left, above_right = pz < upper_right;
    bool below_left = pz > lower_left, below_right = pz > lower_right;
    bool entirely_above = above_left && above_right, entirely_below = below_left && below_right;
    i64 clipped_left = screen_left, clipped_right = screen_right;
    i64 clipped_dl = depth_left, clipped_dr = depth_right;
    bool outside_top = false, outside_bottom = false;
    bool crosses_top = above_left != above_right;
    if (crosses_top) {
        i64 safe_upper_delta = (upper_right != upper_left) ? (upper_right - upper_left) : 1;
        i64 top_fraction = tdiv(shl64(pz - upper_left, 30), safe_upper_delta);
        i64 top_depth = depth_left + (mul64(depth_right - depth_left, top_fraction) >> 30);
        i64 top_cross = screen_left + tdiv(mul64(mul64(depth_right, top_fraction) >> 30, screen_right - screen_left), max64(top_depth, 1));
        if (above_right && (screen_left <= top_cross)) { clipped_right = top_cross; clipped_dr = top_depth; }
        outside_top |= above_right && (screen_right > top_cross) && (px >= top_cross) && (px < screen_right);
        if (above_left && (top_cross <= screen_right)) { clipped_left = top_cross; clipped_dl = top_depth; }
        outside_top |= above_left && (top_cross > screen_left) && (px >= screen_left) && (px < top_cross);
    }
    bool crosses_bottom = below_left != below_right;
    if (crosses_bottom) {
        i64 safe_lower_delta = (lower_right != lower_left) ? (lower_right - lower_left) : 1;
        i64 bottom_fraction = tdiv(shl64(pz - lower_left, 30), safe_lower_delta);
        i64 bottom_depth = depth_left + (mul64(depth_right - depth_left, bottom_fraction) >> 30);
        i64 bottom_cross = screen_left + tdiv(mul64(mul64(depth_right, bottom_fraction) >> 30, screen_right - screen_left), max64(bottom_depth, 1));
        if (below_right && (screen_left <= bottom_cross)) { clipped_right = bottom_cross; clipped_dr = bottom_depth; }
        outside_bottom |= below_right && (screen_right > bottom_cross) && (px >= bottom_cross) && (px < screen_right);
        if (below_left && (bottom_cross <= screen_right)) { clipped_left = bottom_cross; clipped_dl = bottom_depth; }
        outside_bottom |= below_left && (bottom_cross > screen_left) && (px >= screen_left) && (px < bottom_cross);
    }
    i64 projected_left = tdiv(mul64(pz, FOCAL_Y_FIXED), max64(clipped_dl, 1));
    i64 projected_right = tdiv(mul64(pz, FOCAL_Y_FIXED), max64(clipped_dr, 1));
    i64 span = max64(clipped_right - clipped_left, 1);
    i64 projected_step = tdiv(projected_right - projected_left, span);
    i64 projected = clampi((center_fixed + projected_left + mul64(px - clipped_left, projected_step)) >> 16, 0, VH);
    bool collapsed = (clipped_right == clipped_left) && (px == clipped_left) && !(entirely_above || entirely_below);
    if (entirely_above || (outside_top && !collapsed)) projected = 0;
    else if (entirely_below || (outside_bottom && !collapsed)) projected = VH;
    return (float)projected;
}

// engine.py:10630-10640
__device__ __forceinline__ i64 wall_shade(float light, i64 visibility) {
    i64 shade = 64 * FIXED_UNIT - ((i64)light + 12) * (FIXED_UNIT / 4);
    return clampi((shade - min64(visibility, 24 * FIXED_UNIT)) >> 16, 0, 31);
}

// engine.py:11596-11730 for one (column, linedef)
__device__ __forceinline__ void endpoint_owner(const ColumnCtx &cc, int w, const Eval &cw, int *owner_index, float *owner_distance) {
    const gd_map_desc *m = cc.m;
    const int K = m->neighbor_slots;
    const bool subpixel = cc.spans[cc.rec_base + (unsigned)w].flags & WF_SUBPIXEL;
    float tol_w = tolerance_of(cw.dist);
    // the owner only matters for a linedef that does not own this column itself (engine.py:11716)
    if (cw.flags & CF_PROJ) { *owner_index = w; *owner_distance = cw.dist; return; }
    bool uses_start = !(cw.flags & CF_ALONG_HI);
    int index; float distance; bool valid;
    if (m->direct_neighbors) {
        // {start neighbour, end neighbour, start slot | end slot << 8 | has start << 16 | has end << 17}
        const int4 nb = *reinterpret_cast<const int4 *>(m->direct_neighbor_table + 4 * w);
        int ss = nb.z & 0xFF, es = (nb.z >> 8) & 0xFF; bool hs = (nb.z >> 16) & 1, he = (nb.z >> 17) & 1;
        int rslot = uses_start ? ss : es, oslot = uses_start ? es : ss;
        bool rexists = uses_start ? hs : he, oexists = uses_start ? he : hs;
        int rn = uses_start ? nb.x : nb.y, on = uses_start ? nb.y : nb.x;
        Eval r = cc.eval(rn);
        bool r_owns = rexists && (r.flags & CF_PROJ) && (r.flags & CF_LEDGE);
        Eval o = (on == rn) ? r : cc.eval(on);
        bool o_owns = subpixel && oexists && (o.flags & CF_PROJ) && (o.flags & CF_LEDGE) && (fabsf(o.dist - cw.dist) <= tol_w);
        bool use_o = o_owns && (!r_owns || (o.dist < r.dist) || ((o.dist == r.dist) && (oslot < rslot)));
        index = use_o ? on : rn;
        distance = use_o ? o.dist : r.dist;
        valid = r_owns || o_owns;
    } else {
        float best = GD_INF; int best_slot = 0;
        for (int k = 0; k < K; ++k) {
            int n = m->endpoint_neighbors[w * K + k];
            bool st = m->endpoint_neighbor_starts[w * K + k], en = m->endpoint_neighbor_ends[w * K + k];
            Eval nb = cc.eval(n);
            bool ray_nb = uses_start ? st : en;
            bool selected = ray_nb || (subpixel && (st || en) && (fabsf(nb.dist - cw.dist) <= tol_w));
            float v = ((nb.flags & CF_PROJ) && (nb.flags & CF_LEDGE) && selected) ? nb.dist : GD_INF;
            if (v < best) { best = v; best_slot = k; }
        }
        index = m->endpoint_neighbors[w * K + best_slot];
        distance = best;
        valid = finitef(best);
    }
    bool has = !(cw.flags & CF_PROJ) && valid;
    *owner_index = has ? index : w;
    *owner_distance = has ? distance : cw.dist;
}


struct ColumnState {   // engine.py:11561-11580, 11735-11762
    int current_sector;
    float ceiling_clip, floor_clip;
    float masked_ceiling_clip, masked_floor_clip, masked_distance;
    int masked_wall;
    float previous_distance;
    int pend_po_vertex, pend_ep_vertex, pend_ep_wall, pend_eb_index, pend_pb_index, pend_pb_sector;
    float pend_pb_exit;
    int flags;  // bit0 pend_po_boundary, bit1 pend_ep_boundary, bit2 pend_eb_boundary, bit3 pend_pb
};
#define ST_PO 1
#define ST_EP 2
#define ST_EB 4
#define ST_PB 8

__device__ __forceinline__ bool same_state(const ColumnState &a, const ColumnState &b) {
    return a.current_sector == b.current_sector && a.ceiling_clip == b.ceiling_clip && a.floor_clip == b.floor_clip &&
           a.masked_ceiling_clip == b.masked_ceiling_clip && a.masked_floor_clip == b.masked_floor_clip &&
           a.masked_distance == b.masked_distance && a.masked_wall == b.masked_wall &&
           a.previous_distance == b.previous_distance && a.pend_po_vertex == b.pend_po_vertex &&
           a.pend_ep_vertex == b.pend_ep_vertex && a.pend_ep_wall == b.pend_ep_wall && a.pend_eb_index == b.pend_eb_index &&
           a.pend_pb_index == b.pend_pb_index && a.pend_pb_sector == b.pend_pb_sector && a.pend_pb_exit == b.pend_pb_exit &&
           a.flags == b.flags;
}

struct PassColumn {
    int wall, side, render_current, other_sector;
    float distance;
    i64 visibility;
    float view_floor, view_ceiling, other_floor, other_ceiling;
    float clipped_top, clipped_bottom, clipped_upper_bottom, clipped_lower_top;
    int side_tex[3];
    int ps_path_index, ps_other, no_path_other, sel_vertex, fb_idx;
    float ps_path_distance, no_path_distance;
    int bits;
    // what the drawing half adds (pass_geometry, pass_clip)
    int render_other;       // the sector behind the drawn side, -1 for none
    float one_top, one_bottom, lower_top, upper_bottom;              // the four heights' projected rows, not yet clipped
    float path_top, path_bottom, path_lower_top, path_upper_bottom;  // the same of the portal path of a PB_PS_KEEPS pass
    i64 u_base, swall;      // texture column before wrapping, texture step (engine.py:12762-12807)
    float offset_y;         // the side's vertical texture offset
    float fake_contrast;    // +16 on vertical linedefs, -16 on horizontal ones (engine.py:12853-12861)
};
#define PB_VALID 0x1
#define PB_RASTER 0x2
#define PB_ONE_SIDED 0x4
#define PB_TIER0 0x8
#define PB_TIER1 0x10
#define PB_TIER2 0x20
#define PB_MARK_CEILING 0x40
#define PB_MARK_FLOOR 0x80
#define PB_PS_KEEPS 0x100
#define PB_NO_KEEPS 0x200
#define PB_GEOMETRIC 0x400
#define PB_REPLACE_NP 0x800
#define PB_PS_FROM_FRONT 0x1000
#define PB_CONTINUES_PO 0x2000
#define PB_FORWARD_BRIDGE 0x4000
#define PB_FINAL_ALONG_HI 0x8000

// (distance, linedef) lexicographic minimum: what torch.min(dim) returns on ascending indices
__device__ __forceinline__ void take_min(float v, int w, float &best, int &best_w) {
    if (v < best || (v == best && w < best_w && finitef(v))) { best = v; best_w = w; }
}

// engine.py:12240-12620, 12762-12861, 12969-13010: what one column draws of the drawseg a pass selected, as far as it
// depends on the selection alone (r.wall, r.render_current, r.ps_path_index, r.ps_other, PB_RASTER / PB_ONE_SIDED /
// PB_PS_KEEPS / PB_PS_FROM_FRONT in r.bits) and not on the column's clips: the side and sectors drawn from, the wallscan
// light, the four heights' projected rows, the texture column and step, and the projected rows of a portal path behind a
// projected solid.  Every division of the drawing half is in here.
template <bool SPLIT>
__device__ __forceinline__ void pass_geometry(const ColumnCtx &cc, PassColumn &r) {
    const gd_map_desc *m = cc.m;
    const MapView &mv = cc.mv;
    const LaneCtx &L = *cc.c;
    const int x = cc.x, wi = r.wall, render_current = r.render_current;
    const bool one_sided = r.bits & PB_ONE_SIDED;
    // h. sides (engine.py:12240-12292)
    const int front = mv.sec(wi, 0), back = mv.sec(wi, 1);
    const bool render_from_front = render_current == front;
    const int render_other = render_from_front ? back : front;
    const int side = render_from_front ? 0 : 1;
    const int safe_other = render_other < 0 ? 0 : render_other;
    r.side = side; r.render_other = render_other;
    const WallRec &wr = cc.rec(wi);
    const FragmentChoice wr_fragment = choose_fragment<SPLIT>(m, cc.frags, wr, wi, x);
    r.visibility = wall_visibility(wr_fragment.lights ? *wr_fragment.rec : wr, side, x);
    const float view_floor = m->sector_heights[2 * render_current], view_ceiling = m->sector_heights[2 * render_current + 1];
    const float other_floor = m->sector_heights[2 * safe_other], other_ceiling = m->sector_heights[2 * safe_other + 1];
    for (int t = 0; t < 3; ++t) r.side_tex[t] = m->side_tex[(wi * 2 + side) * 3 + t];
    // j. projection (engine.py:12607-12620): one copy of the projection code, four heights; the back sector's two only
    // matter across a two-sided linedef (every use of them is behind !one_sided)
    r.one_top = 0; r.one_bottom = 0; r.lower_top = 0; r.upper_bottom = 0;
    const int heights = one_sided ? 2 : 4;
#pragma unroll 1
    for (int k = 0; k < heights; ++k) {
        float z = k == 0 ? view_ceiling : (k == 1 ? view_floor : (k == 2 ? other_floor : other_ceiling));
        float v = project(L, wr, wr_fragment, z, x);
        if (k == 0) r.one_top = v; else if (k == 1) r.one_bottom = v; else if (k == 2) r.lower_top = v; else r.upper_bottom = v;
    }
    // texture column and step (engine.py:12762-12807), fake contrast (engine.py:12853-12861): only tiers use them
    r.u_base = 0; r.swall = 0; r.offset_y = 0.0f; r.fake_contrast = 0.0f;
    if (r.bits & PB_RASTER) {
        const float *toff = m->side_off + (wi * 2 + side) * 2;
        i64 h, swall;
        texture_mapping(m, wr, wi, x, &h, &swall);
        i64 repeat = round_to_i64(m->wall_len[wi] * 65536.0f);
        if (side != 0) h = repeat - h;
        if (wr.sl > 0 && h < 0) h = 0;
        if (h >= repeat) h = repeat - 1;
        i64 offx_fixed = round_to_i64(toff[0] * 65536.0f);
        r.u_base = (h + offx_fixed) >> 16;
        r.swall = swall;
        r.offset_y = toff[1];
        const float4 wl = *reinterpret_cast<const float4 *>(m->walls + 4 * wi);
        bool horizontal = fabsf(wl.w - wl.y) < 1e-6f, vertical = fabsf(wl.z - wl.x) < 1e-6f;
        r.fake_contrast = vertical ? 16.0f : (horizontal ? -16.0f : 0.0f);
    }
    // the portal path behind a projected solid (engine.py:12969-13010): the view sector's two heights and the path's other
    // sector's two, projected through the path linedef
    r.path_top = 0; r.path_bottom = 0; r.path_lower_top = 0; r.path_upper_bottom = 0;
    if (r.bits & PB_PS_KEEPS) {
        const int path = r.ps_path_index;
        const WallRec &pr = cc.rec(path);
        const FragmentChoice pr_fragment = choose_fragment<SPLIT>(m, cc.frags, pr, path, x);
        const int path_safe_other = r.ps_other < 0 ? 0 : r.ps_other;
        const float pof = m->sector_heights[2 * path_safe_other], poc = m->sector_heights[2 * path_safe_other + 1];
#pragma unroll 1
        for (int k = 0; k < 4; ++k) {
            float z = k == 0 ? view_ceiling : (k == 1 ? view_floor : (k == 2 ? pof : poc));
            float v = project(L, pr, pr_fragment, z, x);
            if (k == 0) r.path_top = v; else if (k == 1) r.path_bottom = v; else if (k == 2) r.path_lower_top = v; else r.path_upper_bottom = v;
        }
    }
}

// engine.py:12607-12636: the projected rows of pass_geometry against the column's clips, the plane marks and the tiers.
// r.side and r.render_other come from pass_geometry.
__device__ __forceinline__ void pass_clip(const ColumnCtx &cc, float ceiling_clip, float floor_clip, PassColumn &r) {
    const Tables &tb = *cc.tb;
    const int render_current = r.render_current;
    const int safe_other = r.render_other < 0 ? 0 : r.render_other;
    const bool raster_valid = r.bits & PB_RASTER, one_sided = r.bits & PB_ONE_SIDED;
    r.view_floor = tb.floor_h(render_current); r.view_ceiling = tb.ceil_h(render_current);
    r.other_floor = tb.floor_h(safe_other); r.other_ceiling = tb.ceil_h(safe_other);
    r.clipped_top = fmaxf(r.one_top, ceiling_clip);
    r.clipped_bottom = fminf(r.one_bottom, floor_clip);
    r.clipped_upper_bottom = fmaxf(fminf(r.upper_bottom, floor_clip), r.clipped_top);
    r.clipped_lower_top = fminf(fmaxf(r.lower_top, ceiling_clip), r.clipped_bottom);
    // k. plane marks (engine.py:12621-12636)
    bool light_differs = tb.light(render_current) != tb.light(safe_other);
    bool mark_ceiling = one_sided || (r.view_ceiling != r.other_ceiling) || (tb.ceil_tex(render_current) != tb.ceil_tex(safe_other)) || light_differs;
    bool mark_floor = one_sided || (r.view_floor != r.other_floor) || (tb.floor_tex(render_current) != tb.floor_tex(safe_other)) || light_differs;
    bool tier0 = one_sided && raster_valid && (r.side_tex[0] >= 0) && (r.clipped_top < r.clipped_bottom);
    bool tier1 = !one_sided && raster_valid && (r.view_floor < r.other_floor) && (r.side_tex[1] >= 0) && (r.clipped_lower_top < r.clipped_bottom);
    bool tier2 = !one_sided && raster_valid && (r.view_ceiling > r.other_ceiling) && (r.side_tex[2] >= 0) && (r.clipped_top < r.clipped_upper_bottom);
    r.bits |= (tier0 ? PB_TIER0 : 0) | (tier1 ? PB_TIER1 : 0) | (tier2 ? PB_TIER2 : 0) | (mark_ceiling ? PB_MARK_CEILING : 0) | (mark_floor ? PB_MARK_FLOOR : 0);
}

// engine.py:11769-12239: selection of the pass's drawseg for one column
template <bool SPLIT>
__device__ __forceinline__ void pass_select(const ColumnCtx &cc, const ColumnState &c, bool boundary_has_po, PassColumn &r) {
    const gd_map_desc *m = cc.m;
    const MapView &mv = cc.mv;
    const int x = cc.x;
    const int cs = c.current_sector;
    const int cur = cs < 0 ? 0 : cs;
    const float prev = c.previous_distance;
    const float prev_eps = prev + 1e-3f;
    auto incident = [&](int w) { return mv.sec(w, 0) == cur || mv.sec(w, 1) == cur; };
    auto incident_c = [&](const Cand &q) { return q.s0 == cur || q.s1 == cur; };
    // a. nearest incident linedef beyond previous_distance (engine.py:11769-11780)
    float distance = GD_INF; int wi = 0x7fffffff;
    Eval cwi;
    // List positions of the candidates incident to the current sector and beyond previous_distance: the later
    // scans of this pass ask for both (and more), so they only visit these.  Without a current sector: all.
    // Bit b stands for the positions b, b + 64, b + 128, ... of a list longer than 64 (a spilled column's): the later
    // scans test every candidate they visit again, so a bit that also names candidates outside the set costs a look.
    u64 incident_beyond = cc.count >= 64 ? ~0ULL : ((1ULL << cc.count) - 1);
    if (cs >= 0) {
        incident_beyond = 0;
        // b. equal-depth solid (engine.py:11784-11807): the nearest one-sided candidate replaces
        // the selection when it lies within 1e-3 of the nearest candidate, found in the same scan.
        u64 nearest = CAND_KEY_NONE, nearest_solid = CAND_KEY_NONE;
        for (int k0 = 0; k0 < cc.count; k0 += CAND_BATCH) {
            Cand batch[CAND_BATCH];
            cc.cand_batch(k0, batch);
            unsigned batch_bits = 0u;
#pragma unroll
            for (int j = 0; j < CAND_BATCH; ++j) {
                const Cand q = batch[j];
                const bool hit = k0 + j < cc.count && incident_c(q) && q.dist > prev;
                batch_bits |= hit ? 1u << j : 0u;
                const u64 key = hit ? cand_key(q) : CAND_KEY_NONE;
                nearest = key < nearest ? key : nearest;
                const u64 solid_key = q.s1 < 0 ? key : CAND_KEY_NONE;
                nearest_solid = solid_key < nearest_solid ? solid_key : nearest_solid;
            }
            incident_beyond |= (u64)batch_bits << (k0 & 63);
        }
        const float sd = cand_key_distance(nearest_solid);
        if (finitef(sd) && (fabsf(sd - cand_key_distance(nearest)) <= 1e-3f)) nearest = nearest_solid;
        distance = cand_key_distance(nearest); wi = cand_key_wall(nearest);
        cwi.dist = distance; cwi.flags = cand_key_flags(nearest);
    }
    if (!finitef(distance)) { wi = 0; cwi = cc.eval(0); }
    // c. selected endpoint (engine.py:11815-11871)
    bool sel_start = !(cwi.flags & CF_ALONG_HI);
    int sel_vertex = mv.vert(wi, sel_start ? 0 : 1);
    auto shares_sel_c = [&](const Cand &q) { return (int)q.v0 == sel_vertex || (int)q.v1 == sel_vertex; };
    bool continues_po_boundary = (c.flags & ST_PO) && (sel_vertex == c.pend_po_vertex);
    bool continues_ep_boundary = (c.flags & ST_EP) && (sel_vertex == c.pend_ep_vertex);
    int sel_slot = sel_start ? 0 : 1;
    // the forward bridge only matters while an endpoint-projected boundary continues
    int fb_idx = 0;
    bool pend_ep_has_forward_bridge = false;
    if (continues_ep_boundary && mv.portal_bridge(sel_slot, wi, c.pend_ep_wall, &fb_idx))
        pend_ep_has_forward_bridge = cc.eval(fb_idx).dist > distance + 1e-3f;
    bool completes_pending_endpoint_bridge = (c.flags & ST_EB) && (wi == c.pend_eb_index);
    bool sel_is_proj = cwi.flags & CF_PROJ;
    bool sel_excl_right = cc.rec(wi).sr == x;
    // d. projected solid owner (engine.py:11872-11954)
    float ps_path_distance = distance; int ps_path_index = wi;
    bool ps_path_geo = cwi.flags & CF_GEO;
    float psd = GD_INF; int psi = 0x7fffffff; int psi_flags = 0;
    if (!sel_is_proj) {
        auto solid_owner = [&](const Cand &q) {
            bool owner = incident_c(q) && (q.s1 < 0) && (q.flags & CF_PROJ) && (q.flags & CF_LEDGE) && shares_sel_c(q) && (q.dist > prev_eps);
            if (owner && (q.dist < psd || (q.dist == psd && (int)q.wall < psi))) { psd = q.dist; psi = q.wall; psi_flags = q.flags; }
        };
        for (u64 rest = incident_beyond; rest;) {
            Cand batch[CAND_BATCH]; int at[CAND_BATCH];
            cc.cand_batch_of(rest, batch, at);
#pragma unroll
            for (int j = 0; j < CAND_BATCH; ++j) {
                if (at[j] < 0) continue;
                solid_owner(batch[j]);
            }
        }
        for (int k = 64; k < cc.count; ++k)   // a spilled column's further entries
            if ((incident_beyond >> (k & 63)) & 1ULL) solid_owner(cc.cand(k));
        if (sel_excl_right) {
            const int *ofs = sel_start ? m->solid_bridge_start_ofs : m->solid_bridge_end_ofs;
            const int *idx = sel_start ? m->solid_bridge_start_idx : m->solid_bridge_end_idx;
            float sbd = GD_INF; int sbi = 0; int sbi_flags = 0;
            for (int k = ofs[wi]; k < ofs[wi + 1]; ++k) {
                int b = idx[k];
                if (!(incident(b) && mv.one_sided(b))) continue;
                Eval q = cc.eval(b);
                bool owner = (q.flags & CF_PROJ) && (q.flags & CF_LEDGE) && (q.dist > prev_eps);
                float v = owner ? q.dist : GD_INF;
                if (v < sbd) { sbd = v; sbi = b; sbi_flags = q.flags; }   // list is ascending: first slot wins ties
            }
            if (sbd < psd) { psd = sbd; psi = sbi; psi_flags = sbi_flags; }
        }
    }
    bool has_ps = finitef(psd);
    if (has_ps) { distance = psd; wi = psi; cwi.dist = psd; cwi.flags = psi_flags; }
    // e. endpoint owner (engine.py:11960-12001)
    int eo_idx; float eo_dist;
    endpoint_owner(cc, wi, cwi, &eo_idx, &eo_dist);
    bool eo_path_geo = cwi.flags & CF_GEO;
    bool replace_eo = (eo_idx != wi) && (eo_dist > prev_eps);
    if (replace_eo) { distance = eo_dist; wi = eo_idx; cwi = cc.eval(wi); }
    int no_path_index = wi; float no_path_distance = distance;
    bool no_path_geo = replace_eo ? eo_path_geo : (bool)(cwi.flags & CF_GEO);
    bool no_from_front = cs == mv.sec(no_path_index, 0);
    int no_path_other = no_from_front ? mv.sec(no_path_index, 1) : mv.sec(no_path_index, 0);
    // f. near projected owner (engine.py:12002-12179)
    bool so_is_proj = cwi.flags & CF_PROJ;
    const WallRec &so_rec = cc.rec(wi);
    bool so_excl_right = so_rec.sr == x;
    i64 so_span = so_rec.sr - so_rec.sl;
    bool so_short = m->wall_len[wi] <= 32.0f;
    float npd = GD_INF; int npi = 0x7fffffff; int npi_flags = 0;
    const int so_s0 = mv.sec(wi, 0), so_s1 = mv.sec(wi, 1);
    if (!so_is_proj) {
        auto near_owner = [&](const Cand &q) {
            int w = q.wall;
            if (!(incident_c(q) && (q.s1 >= 0) && (q.flags & CF_PROJ) && (q.dist > prev_eps))) return;
            bool le = q.flags & CF_LEDGE;
            bool same_pair = (q.s0 == so_s0 && q.s1 == so_s1) || (q.s0 == so_s1 && q.s1 == so_s0);
            bool close = (same_pair || (le && so_excl_right && ((so_span <= 2) || (shares_sel_c(q) && so_short)))) &&
                         (fabsf(q.dist - distance) <= tolerance_of(q.dist));
            bool topo = false;
            if (!close && le && so_excl_right && so_span <= 2) { int dummy; topo = mv.sector_bridge((q.flags & CF_ALONG_HI) ? 1 : 0, w, no_path_index, &dummy); }
            if ((close || topo) && (q.dist < npd || (q.dist == npd && w < npi))) { npd = q.dist; npi = w; npi_flags = q.flags; }
        };
        for (u64 rest = incident_beyond; rest;) {
            Cand batch[CAND_BATCH]; int at[CAND_BATCH];
            cc.cand_batch_of(rest, batch, at);
#pragma unroll
            for (int j = 0; j < CAND_BATCH; ++j) {
                if (at[j] < 0) continue;
                near_owner(batch[j]);
            }
        }
        for (int k = 64; k < cc.count; ++k)   // a spilled column's further entries
            if ((incident_beyond >> (k & 63)) & 1ULL) near_owner(cc.cand(k));
    }
    int pe_wall = c.pend_ep_wall;
    int pe_s0 = mv.sec(pe_wall, 0), pe_s1 = mv.sec(pe_wall, 1);
    bool pe_from_current = cs == pe_s0;
    bool pe_incident = pe_from_current || (cs == pe_s1);
    int pe_other = pe_from_current ? pe_s1 : pe_s0;
    bool use_psb = false; int psb_idx = 0;
    if ((c.flags & ST_EP) && pe_incident && (pe_other >= 0) && (no_path_other >= 0) && no_path_geo && !so_is_proj && so_excl_right &&
        (cc.rec(pe_wall).sr - cc.rec(pe_wall).sl <= 1)) {
        int pe_slot = (c.pend_ep_vertex == mv.vert(pe_wall, 1)) ? 1 : 0;
        bool psb_exists = mv.sector_bridge(pe_slot, pe_wall, no_path_index, &psb_idx);
        if (psb_exists) {
            int b0 = mv.sec(psb_idx, 0), b1 = mv.sec(psb_idx, 1);
            bool matches = (b0 == pe_other && b1 == no_path_other) || (b1 == pe_other && b0 == no_path_other);
            Eval qb = cc.eval(psb_idx);
            float pe_tol = tolerance_of(cc.eval(pe_wall).dist);
            bool psb = matches && (qb.flags & CF_PROJ) && (qb.flags & CF_LEDGE) && (qb.dist > prev - pe_tol) && (qb.dist < no_path_distance);
            if (psb && qb.dist < npd) { use_psb = true; npd = qb.dist; npi = psb_idx; npi_flags = qb.flags; }
        }
    }
    bool replace_np = finitef(npd);
    if (replace_np) { distance = npd; wi = npi; cwi.dist = npd; cwi.flags = npi_flags; }
    bool final_proj = cwi.flags & CF_PROJ, final_geo = cwi.flags & CF_GEO;
    bool completes_poab = (c.flags & ST_EP) && final_proj && !final_geo && mv.opposing(pe_wall, wi);
    // g. validity (engine.py:12197-12239)
    bool valid = finitef(distance);
    bool excl_only = !so_is_proj && so_excl_right && !replace_np && (so_span <= 2) && !boundary_has_po;
    bool raster_valid = valid && !excl_only && !continues_po_boundary &&
                        !((pend_ep_has_forward_bridge || completes_pending_endpoint_bridge) && !sel_is_proj && sel_excl_right && !replace_np);
    bool geometric_intersection = replace_np ? no_path_geo : (replace_eo ? eo_path_geo : final_geo);
    bool no_keeps = replace_np && no_path_geo && (no_path_other >= 0);
    // h. sides (engine.py:12240-12292)
    int front = mv.sec(wi, 0), back = mv.sec(wi, 1);
    bool from_front = cs == front;
    int other_sector = from_front ? back : front;
    int render_current = use_psb ? pe_other : (completes_poab ? other_sector : cur);
    bool render_from_front = render_current == front;
    int render_other = render_from_front ? back : front;
    int side = render_from_front ? 0 : 1;
    bool ps_from_front = cs == mv.sec(ps_path_index, 0);
    int ps_other = ps_from_front ? mv.sec(ps_path_index, 1) : mv.sec(ps_path_index, 0);
    bool ps_keeps = has_ps && ps_path_geo && (ps_other >= 0);
    bool one_sided = other_sector < 0;

    r.wall = wi; r.side = side; r.render_current = render_current; r.other_sector = other_sector;
    r.distance = distance;
    r.ps_path_index = ps_path_index; r.ps_other = ps_other; r.no_path_other = no_path_other; r.sel_vertex = sel_vertex; r.fb_idx = fb_idx;
    r.ps_path_distance = ps_path_distance; r.no_path_distance = no_path_distance;
    r.bits = (valid ? PB_VALID : 0) | (raster_valid ? PB_RASTER : 0) | (one_sided ? PB_ONE_SIDED : 0) |
             (ps_keeps ? PB_PS_KEEPS : 0) | (no_keeps ? PB_NO_KEEPS : 0) | (geometric_intersection ? PB_GEOMETRIC : 0) |
             (replace_np ? PB_REPLACE_NP : 0) | (ps_from_front ? PB_PS_FROM_FRONT : 0) | (continues_po_boundary ? PB_CONTINUES_PO : 0) |
             (pend_ep_has_forward_bridge ? PB_FORWARD_BRIDGE : 0) | ((cwi.flags & CF_ALONG_HI) ? PB_FINAL_ALONG_HI : 0);
}

// The per-pixel planes of a chunk of lanes and one column's place in them.  The wavefronts of the traversal hold columns of
// several lanes, so the planes' base pointers are the same for all of them and each column keeps byte offsets: a chunk
// is at most 4096 lanes, which keeps every offset below 4 GiB.
struct PixelBuffers {
    unsigned char *frame;   // [L][240][320] or null
    unsigned int *meta;     // [L][208][320]
    float *clip_depth;      // [L][208][320], only meaningful where the meta word names a clip linedef
    float *scene_depth;     // [L][208][320] or null
    unsigned word_column;   // byte offset of (lane, row 0, column) in the four-byte planes
    unsigned frame_column;  // and in the frame
    __device__ __forceinline__ unsigned int &m(int y) const { return *reinterpret_cast<unsigned int *>(reinterpret_cast<char *>(meta) + (word_column + (unsigned)y * (SW * 4u))); }
    __device__ __forceinline__ float &d(int y) const { return *reinterpret_cast<float *>(reinterpret_cast<char *>(clip_depth) + (word_column + (unsigned)y * (SW * 4u))); }
    __device__ __forceinline__ float &s(int y) const { return *reinterpret_cast<float *>(reinterpret_cast<char *>(scene_depth) + (word_column + (unsigned)y * (SW * 4u))); }
    __device__ __forceinline__ unsigned char &f(int y) const { return frame[frame_column + (unsigned)y * (unsigned)SW]; }
};

// Silhouette bookkeeping: every row >= bot_row holds a clip depth <= bot_depth, every row
// < top_row holds a clip depth <= top_depth.  Clip depths only ever decrease, so a silhouette
// at a depth not below the bound cannot change those rows and they need not be visited.
struct SilhouetteBounds {
    int bot_row, top_row;
    float bot_depth, top_depth;
};

// Rows [first, last) of one column take `distance` / `wall` as their sprite clip where it is nearer
// than what they hold.  WALL_ROWS rows at a time, loads first, so the rows' memory latencies overlap.
__device__ __forceinline__ void clip_rows(PixelBuffers &pb, int x, int first, int last, float distance, int wall) {
    // one batch ahead: the next rows are asked for before this batch's stores (the rows of two batches are distinct)
    auto load_rows = [&](int y0, float (&held)[WALL_ROWS], unsigned int (&meta)[WALL_ROWS]) {
#pragma unroll
        for (int j = 0; j < WALL_ROWS; ++j) {
            const int y = y0 + j < last ? y0 + j : last - 1;
            held[j] = pb.d(y); meta[j] = pb.m(y);
        }
    };
    float held[WALL_ROWS]; unsigned int meta[WALL_ROWS];
    if (first < last) load_rows(first, held, meta);
    for (int y0 = first; y0 < last; y0 += WALL_ROWS) {
        float next_held[WALL_ROWS]; unsigned int next_meta[WALL_ROWS];
#pragma unroll
        for (int j = 0; j < WALL_ROWS; ++j) { next_held[j] = 0.0f; next_meta[j] = 0u; }
        if (y0 + WALL_ROWS < last) load_rows(y0 + WALL_ROWS, next_held, next_meta);
#pragma unroll
        for (int j = 0; j < WALL_ROWS; ++j) {
            const float depth = (meta[j] & META_WALL_MASK) ? held[j] : GD_INF;   // no clip recorded yet: infinite
            if (y0 + j >= last || !(distance < depth)) continue;
            pb.d(y0 + j) = distance; pb.m(y0 + j) = (meta[j] & ~META_WALL_MASK) | (unsigned)(wall + 1);
        }
#pragma unroll
        for (int j = 0; j < WALL_ROWS; ++j) { held[j] = next_held[j]; meta[j] = next_meta[j]; }
    }
}

// `done_from` / `done_to`: rows [done_from, done_to) already carry this silhouette (pass_paint wrote it with
// the rows the pass took out of a window nothing had touched); an empty range otherwise.
__device__ __forceinline__ void apply_silhouette(PixelBuffers &pb, SilhouetteBounds &sb, int x, bool bottom, bool top, float floor_clip, float ceiling_clip, float distance, int wall,
                                                 int done_from, int done_to) {
    if (bottom) {
        int first = floor_clip <= 0.0f ? 0 : (floor_clip >= (float)VH ? VH : (int)floor_clip);   // clips hold integers
        int last = (distance >= sb.bot_depth) ? (sb.bot_row < VH ? sb.bot_row : VH) : VH;
        clip_rows(pb, x, (done_to > first && done_from <= first) ? done_to : first, last, distance, wall);
        sb.bot_row = first < sb.bot_row ? first : sb.bot_row;
        sb.bot_depth = fmaxf(sb.bot_depth, distance);
    }
    if (top) {
        int end = ceiling_clip <= 0.0f ? 0 : (ceiling_clip >= (float)VH ? VH : (int)ceiling_clip);
        int start = (distance >= sb.top_depth) ? (sb.top_row > 0 ? sb.top_row : 0) : 0;
        clip_rows(pb, x, start, (done_from < end && done_to >= end) ? done_from : end, distance, wall);
        sb.top_row = end > sb.top_row ? end : sb.top_row;
        sb.top_depth = fmaxf(sb.top_depth, distance);
    }
}

// May pass_paint write a two-sided pass's sprite silhouettes along with the rows the pass takes out of an untouched
// window?  Only while its lower and upper tier do not overlap on screen.
__device__ __forceinline__ bool silhouette_folds(const PassColumn &r) {
    const bool lower_on = r.view_floor < r.other_floor, upper_on = r.view_ceiling > r.other_ceiling;
    return !(lower_on && upper_on && r.clipped_lower_top < r.clipped_upper_bottom);
}

// The meta plane is never cleared between frames.  Instead the traversal keeps every row of its column that lies
// outside the open window [ceiling_clip, floor_clip) written (with a claim, a tier, or an explicit zero), reads no row
// inside the window until a one-sided drawseg has painted all of it, and zeroes what is left of the window when the
// column ends.  Rows that received such a zero are the only ones that can end up without an owner: the column keeps
// their range and lists the ownerless ones as gap pixels for the flat pass.
struct GapRange {
    // Four row numbers (0..VH, VH < 256) in one register: the traversal holds them for the whole column.
    //   bits 0-7 lo, 8-15 hi: rows [lo, hi) hold every zero this column wrote
    //   bits 16-23 filled_lo, 24-31 filled_hi: rows [filled_lo, filled_hi) are known to hold wall tier pixels
    //   (the one-sided drawseg's own)
    unsigned int rows;
    __device__ __forceinline__ int lo() const { return (int)(rows & 255u); }
    __device__ __forceinline__ int hi() const { return (int)((rows >> 8) & 255u); }
    __device__ __forceinline__ int filled_lo() const { return (int)((rows >> 16) & 255u); }
    __device__ __forceinline__ int filled_hi() const { return (int)(rows >> 24); }
    __device__ __forceinline__ void reset() { rows = (unsigned)VH; }
    __device__ __forceinline__ void set_zeroed(int lo, int hi) { rows = (rows & 0xffff0000u) | (unsigned)lo | ((unsigned)hi << 8); }
    __device__ __forceinline__ void set_filled(int lo, int hi) { rows = (rows & 0x0000ffffu) | ((unsigned)lo << 16) | ((unsigned)hi << 24); }
};
static_assert(VH < 256, "GapRange packs row numbers into bytes");
__device__ __forceinline__ void zero_rows(PixelBuffers &pb, GapRange &gaps, int x, int first, int last) {
    first = first < 0 ? 0 : first; last = last > VH ? VH : last;
    if (first >= last) return;
    for (int y = first; y < last; ++y) pb.m(y) = 0u;
    gaps.set_zeroed(min(first, gaps.lo()), max(last, gaps.hi()));
}

// Exchanges inside the aligned groups of four lanes (DPP quads): the value of the group's first lane, and the
// conjunction, the largest and the smallest of the four.  All four lanes must be executing.
template <int PATTERN> __device__ __forceinline__ int quad_move(int v) { return __builtin_amdgcn_mov_dpp(v, PATTERN, 0xF, 0xF, true); }
__device__ __forceinline__ int quad_first(int v) { return quad_move<0x00>(v); }                 // lanes 0,0,0,0
__device__ __forceinline__ int quad_and(int v) { v &= quad_move<0xB1>(v); return v & quad_move<0x4E>(v); }   // lanes 1,0,3,2 then 2,3,0,1
__device__ __forceinline__ float quad_max(float v) {
    v = fmaxf(v, __int_as_float(quad_move<0xB1>(__float_as_int(v))));
    return fmaxf(v, __int_as_float(quad_move<0x4E>(__float_as_int(v))));
}
__device__ __forceinline__ float quad_min(float v) {
    v = fminf(v, __int_as_float(quad_move<0xB1>(__float_as_int(v))));
    return fminf(v, __int_as_float(quad_move<0x4E>(__float_as_int(v))));
}

// Smallest / largest of a small value (0..255) over the lanes that execute the call, found by ballots: usable inside
// divergent code, where a lane exchange would read lanes that are switched off.  The result is uniform.
__device__ __forceinline__ int wave_min_byte(int v) {
    u64 candidates = __ballot(true);
    int result = 0;
#pragma unroll
    for (int bit = 7; bit >= 0; --bit) {
        const u64 clear = __ballot(!((v >> bit) & 1)) & candidates;
        if (clear) candidates = clear; else result |= 1 << bit;
    }
    return result;
}
__device__ __forceinline__ int wave_max_byte(int v) { return 255 - wave_min_byte(255 - v); }

// engine.py:12637-12884
// `window_dirty` says whether some pixel inside the open window [ceiling_clip, floor_clip) may
// already be filled, plane-owned or carry a sprite-clip depth.  A two-sided drawseg only writes
// rows that its own clip update then removes from the window, so the window stays untouched
// until a one-sided drawseg (which leaves the clips alone) has painted; until then painting
// needs no reads and visits only the rows it writes.
template <bool DEPTH>
__device__ __forceinline__ void pass_paint(const ColumnCtx &cc, const ColumnState &c, const PassColumn &r, PixelBuffers &pb,
                           const bool group_valid[3], const float group_bottom[3], i64 first_group_visibility,
                           const unsigned char *colormap, bool &window_dirty, GapRange &gaps) {
    if (!(r.bits & PB_RASTER)) return;
    const gd_map_desc *m = cc.m;
    const LaneCtx &L = *cc.c;
    const int x = cc.x, wi = r.wall, side = r.side;
    const bool one_sided = r.bits & PB_ONE_SIDED;
    const float ceiling_plane_bottom = fminf(r.clipped_top, c.floor_clip);
    const float floor_plane_top = fmaxf(r.clipped_bottom, c.ceiling_clip);
    const i64 u_base = r.u_base, swall = r.swall;
    const Tables &tb = *cc.tb;
    float light = (tb.light(r.render_current) + (float)(L.flash_light * 16)) + r.fake_contrast;
    const i64 shade_own = wall_shade(light, r.visibility);
    const i64 shade_group = wall_shade(light, first_group_visibility);
    // every span of this pass lies inside the open window [ceiling_clip, floor_clip)
    int y0 = c.ceiling_clip <= 0.0f ? 0 : (int)c.ceiling_clip;
    int y1 = c.floor_clip >= (float)VH ? VH : (int)c.floor_clip;
    const bool lower_on = !one_sided && (r.view_floor < r.other_floor);
    const bool upper_on = !one_sided && (r.view_ceiling > r.other_ceiling);
    if (!window_dirty) {
        // clips and projections hold integers in [0, 208]
        const unsigned claim = (unsigned)(r.render_current + 1) << META_SECTOR_SHIFT;
        // The sprite silhouettes of a two-sided drawseg (engine.py:12943-12964) give every row that this pass
        // takes out of the window the pass's own (distance, linedef) as sprite clip.  Those rows are untouched
        // so far, so what this pass writes there carries the clip along and pass_advance need not revisit them:
        // tier rows hold it anyway, plane rows get it with their claim, rows left bare get it alone.
        // (Not where the lower and the upper tier overlap, a closed door say: a row of both that the lower tier
        // leaves undrawn for want of a texture would be missed.  silhouette_folds() is asked here and there.)
        const bool masked_texture = r.side_tex[0] >= 0;
        const bool folds = !one_sided && silhouette_folds(r);
        const bool sil_bottom = folds && ((r.view_floor > r.other_floor) || (L.view_z < r.other_floor) || masked_texture);
        const bool sil_top = folds && ((r.view_ceiling < r.other_ceiling) || (L.view_z > r.other_ceiling) || masked_texture);
        const unsigned clip_word = (unsigned)(wi + 1);
        int ceiling_rows_end = 0; bool ceiling_claims = false;
        {
            const bool claims = r.bits & PB_MARK_CEILING;
            const bool bare = !claims && sil_top && upper_on && (r.side_tex[2] >= 0);   // the upper tier lowers the clip past these rows
            // The wavefront walks the rows together, each column writing where its own range has the row: neighbouring
            // columns then store to neighbouring words, where loops that start at each column's own first row would
            // scatter every store over as many rows as the edges' slopes spread them.
            const bool writes = claims || bare;
            const int first = writes ? (y0 < 0 ? 0 : y0) : VH, last = writes ? min((int)ceiling_plane_bottom, VH) : 0;
            const unsigned word = (claims ? claim : 0u) | (sil_top ? clip_word : 0u);
            for (int y = wave_min_byte(first), wave_last = wave_max_byte(last); y < wave_last; ++y) {
                if (y < first || y >= last) continue;
                pb.m(y) = word;
                if (sil_top) pb.d(y) = r.distance;
                ceiling_rows_end = last; ceiling_claims = claims;
        }
            ceiling_rows_end = last; ceiling_claims = claims;
        }
        {
            const bool claims = r.bits & PB_MARK_FLOOR;
            const bool bare = !claims && sil_bottom && lower_on && (r.side_tex[1] >= 0);   // the lower tier raises the clip past these rows
            const bool writes = claims || bare;
            const int first = writes ? max((int)floor_plane_top, 0) : VH, last = writes ? y1 : 0;
            const unsigned word = (claims ? (claim | META_FLOOR) : 0u) | (sil_bottom ? clip_word : 0u);
            for (int y = wave_min_byte(min(first, VH)), wave_last = wave_max_byte(last); y < wave_last; ++y) {
                if (y < first || y >= last) continue;
                pb.m(y) = word;
                if (sil_bottom) pb.d(y) = r.distance;
            }
            // A sector whose ceiling lies below its floor: the rows from its floor's row down to its ceiling's row
            // belong to both runs.  There the floor's claim has the say, the ceiling's stands where the floor makes none,
            // and the clip is recorded if either silhouette asks for it.
            if (__any(first < ceiling_rows_end)) {
                const int both_end = min(last, ceiling_rows_end);
                const unsigned both = (claims ? (claim | META_FLOOR) : (ceiling_claims ? claim : 0u)) | ((sil_top || sil_bottom) ? clip_word : 0u);
                for (int y = first; y < both_end; ++y) {
                    pb.m(y) = both;
                    if (sil_top || sil_bottom) pb.d(y) = r.distance;
                }
            }
        }
        // Rows that leave the window without being written: those the upper tier covers but that belong to a lower
        // tier without a texture (the lower tier has the say there), and a one-sided drawseg's own rows when it has none.
        if (lower_on && upper_on && r.side_tex[1] < 0 && r.side_tex[2] >= 0)
            zero_rows(pb, gaps, x, max((int)r.clipped_top, (int)r.clipped_lower_top), min((int)r.clipped_upper_bottom, (int)r.clipped_bottom));
        if (one_sided && r.side_tex[0] < 0) zero_rows(pb, gaps, x, max((int)r.clipped_top, y0), min((int)r.clipped_bottom, y1));
        int t0 = VH, t1 = 0;
        if (one_sided) { t0 = (int)r.clipped_top; t1 = (int)r.clipped_bottom; }
        if (lower_on) { t0 = min(t0, (int)r.clipped_lower_top); t1 = max(t1, (int)r.clipped_bottom); }
        if (upper_on) { t0 = min(t0, (int)r.clipped_top); t1 = max(t1, (int)r.clipped_upper_bottom); }
        // The texture row of screen row y is bits 32-height_bits .. 31 of
        //   fraction(y) = (texture_mid << (16 - height_bits)) + ((step * (y * 65536 + 65536 - center)) >> 16).
        // step * y * 65536 has no low 16 bits, so it shifts out of the floor unchanged, and only the low 32 bits of
        // the sum are looked at: they advance by the low 32 bits of step per row, whatever the 64-bit terms wrap to.
        const float toff_y = r.offset_y * 65536.0f;
        const unsigned atlas_w = (unsigned)m->tex_max_w;
        const int side_tex0 = r.side_tex[0], side_tex1 = r.side_tex[1], side_tex2 = r.side_tex[2];
        const bool tiers_overlap = lower_on && upper_on && r.clipped_lower_top < r.clipped_upper_bottom;
        if (!tiers_overlap) {
            // The usual case: the rows of a tier are one run, [top, bottom) of a one-sided drawseg, or the upper tier
            // above the lower one.  Each run is painted by a loop that knows its texture, so a row costs an add, a
            // shift, a texel, a colormap entry and the stores.  WALL_ROWS rows at a time, one batch ahead: the texels
            // of the next batch are asked for before the rows of this one are stored, so that a step waits for memory
            // once, not for its stores and then for its loads.
            auto paint_run = [&](int first, int last, int texture, float origin, bool has_tail, float tail_from) {
                if (texture < 0 || first >= last) return;
                const int bits = tb.height_bits(texture);
                const i64 step64 = mul64(swall, shl64(1, 14 - bits));
                const i64 base = shl64(round_to_i64((origin - L.view_z) * 65536.0f + toff_y), 16 - bits);
                const unsigned shift = (unsigned)(31 - bits);   // a one-row texture (bits == 0) must shift everything out: two shifts
                const unsigned step = (unsigned)step64;
                unsigned frac = (unsigned)(base + (mul64(step64, FIXED_UNIT - L.center_fixed) >> 16)) + step * (unsigned)first;
                const unsigned char *column = m->tex_atlas + ((size_t)texture * m->tex_max_h * m->tex_max_w + (size_t)tb.wrap_column(texture, u_base));
                // rows from tail_row on take the group's shade: (float)y >= tail_from, which no row meets if that is not a number
                const int tail_row = !has_tail || !(tail_from < (float)VH) ? VH : (tail_from <= 0.0f ? 0 : (int)ceilf(tail_from));
                const unsigned meta_word = META_FILLED | (unsigned)(wi + 1);
                auto load_rows = [&](int yb, unsigned char (&texel)[WALL_ROWS]) {
#pragma unroll
                    for (int j = 0; j < WALL_ROWS; ++j) {
                        texel[j] = 0;
                        if (yb + j < last) texel[j] = column[__umul24((frac >> shift) >> 1, atlas_w)];
                        frac += step;
                    }
                };
                unsigned char texel[WALL_ROWS];
                load_rows(first, texel);
                for (int yb = first; yb < last; yb += WALL_ROWS) {
                    unsigned char next_texel[WALL_ROWS];
#pragma unroll
                    for (int j = 0; j < WALL_ROWS; ++j) next_texel[j] = 0;
                    if (yb + WALL_ROWS < last) load_rows(yb + WALL_ROWS, next_texel);
#pragma unroll
                    for (int j = 0; j < WALL_ROWS; ++j) {
                        const int y = yb + j;
                        if (y >= last) break;
                        const unsigned colour = colormap[(y >= tail_row ? shade_group : shade_own) * 256 + texel[j]];
                        pb.d(y) = r.distance;
                        if (DEPTH) pb.s(y) = r.distance;
                        pb.m(y) = meta_word | (colour << META_SECTOR_SHIFT);
                    }
#pragma unroll
                    for (int j = 0; j < WALL_ROWS; ++j) texel[j] = next_texel[j];
                }
            };
            // first run: a one-sided drawseg's rows, or the upper tier; second run: the lower tier
            const bool first_run = one_sided || upper_on;
            paint_run(first_run ? (int)r.clipped_top : 0, first_run ? (int)(one_sided ? r.clipped_bottom : r.clipped_upper_bottom) : 0,
                      one_sided ? side_tex0 : side_tex2, one_sided ? r.view_ceiling : r.other_ceiling,
                      one_sided ? group_valid[0] : group_valid[2], one_sided ? group_bottom[0] : group_bottom[2]);
            paint_run(lower_on ? (int)r.clipped_lower_top : 0, lower_on ? (int)r.clipped_bottom : 0, side_tex1, r.other_floor,
                      group_valid[1], group_bottom[1]);
        } else {
            // The lower and the upper tier share rows (a closed door, say): the lower tier has the say there, row by row.
                int tier_tex[3]; unsigned tier_frac[3], tier_step[3], tier_shift[3]; size_t tier_texel[3];
            const float tier_origin[3] = {r.view_ceiling, r.other_floor, r.other_ceiling};
#pragma unroll
            for (int t = 0; t < 3; ++t) {
                tier_tex[t] = r.side_tex[t];
                const int id = tier_tex[t] < 0 ? 0 : tier_tex[t];
                const int bits = tb.height_bits(id);
                const i64 step = mul64(swall, shl64(1, 14 - bits));
                const i64 base = shl64(round_to_i64((tier_origin[t] - L.view_z) * 65536.0f + toff_y), 16 - bits);
                tier_shift[t] = (unsigned)(31 - bits);   // a one-row texture (bits == 0) must shift everything out: two shifts
                tier_step[t] = (unsigned)step;
                tier_frac[t] = (unsigned)(base + (mul64(step, FIXED_UNIT - L.center_fixed) >> 16)) + (unsigned)step * (unsigned)t0;
                tier_texel[t] = (size_t)id * m->tex_max_h * m->tex_max_w + (size_t)tb.wrap_column(id, u_base);
            }
            // WALL_ROWS rows at a time, one batch ahead: the texels of the next batch are asked for before the rows of
            // this one are stored, so that a step waits for memory once, not for its stores and then for its loads
            auto load_rows = [&](int yb, unsigned char (&texel)[WALL_ROWS], unsigned &draw, unsigned &tail) {
                draw = 0; tail = 0;
#pragma unroll
                for (int j = 0; j < WALL_ROWS; ++j) {
                    const int y = yb + j;
                    const float py = (float)y;
                    const bool one_span = one_sided && (py >= r.clipped_top) && (py < r.clipped_bottom);
                    const bool lower_span = lower_on && (py >= r.clipped_lower_top) && (py < r.clipped_bottom);
                    const bool upper_span = upper_on && (py >= r.clipped_top) && (py < r.clipped_upper_bottom);
                    const int t = one_span ? 0 : (lower_span ? 1 : 2);
                    const bool draws = y < t1 && (one_span || lower_span || upper_span) && tier_tex[t] >= 0;
                    if (draws) draw |= 1u << j;
                    // rows that both tiers cover take the group's shade if either tier's common bottom has been passed
                    if ((one_span && group_valid[0] && py >= group_bottom[0]) || (lower_span && group_valid[1] && py >= group_bottom[1]) ||
                        (upper_span && group_valid[2] && py >= group_bottom[2])) tail |= 1u << j;
                    texel[j] = 0;
                    if (draws) {
                        const unsigned tv = (tier_frac[t] >> tier_shift[t]) >> 1;
                        texel[j] = m->tex_atlas[tier_texel[t] + __umul24(tv, atlas_w)];
                    }
#pragma unroll
                    for (int k = 0; k < 3; ++k) tier_frac[k] += tier_step[k];
                }
            };
            unsigned char texel[WALL_ROWS]; unsigned draw = 0, tail = 0;
            if (t0 < t1) load_rows(t0, texel, draw, tail);
            for (int yb = t0; yb < t1; yb += WALL_ROWS) {
                unsigned char next_texel[WALL_ROWS]; unsigned next_draw = 0, next_tail = 0;
#pragma unroll
                for (int j = 0; j < WALL_ROWS; ++j) next_texel[j] = 0;
                if (yb + WALL_ROWS < t1) load_rows(yb + WALL_ROWS, next_texel, next_draw, next_tail);
#pragma unroll
                for (int j = 0; j < WALL_ROWS; ++j) {
                    if (!(draw & (1u << j))) continue;
                    const unsigned colour = colormap[((tail & (1u << j)) ? shade_group : shade_own) * 256 + texel[j]];
                    pb.d(yb + j) = r.distance;
                    if (DEPTH) pb.s(yb + j) = r.distance;
                    pb.m(yb + j) = META_FILLED | (colour << META_SECTOR_SHIFT) | (unsigned)(wi + 1);
                }
#pragma unroll
                for (int j = 0; j < WALL_ROWS; ++j) texel[j] = next_texel[j];
                draw = next_draw; tail = next_tail;
            }
        }
        if (one_sided) {
            window_dirty = true;
            if (r.side_tex[0] >= 0 && t0 < t1) gaps.set_filled(max(t0, 0), min(t1, VH));   // every row of [t0, t1) was drawn just now
        }
        return;
    }
    // A one-sided drawseg has painted this window.  Every row of it has been written since (GapRange), so what a later pass
    // can still change is narrow: a tier pixel where no tier was drawn yet, which can only lie in this pass's own tier rows
    // and outside the rows that drawseg filled, and a plane claim on a row nobody owns, which can only be one of the rows
    // this column had to zero.  Only those rows are visited (usually none).  Few columns come here (one pass in 300 on the
    // 4000-linedef map) but every eighth wavefront pass has one, so the loop is kept plain and light on registers.
    int lo = VH, hi = 0;
    if (one_sided) { lo = (int)r.clipped_top; hi = (int)r.clipped_bottom; }
    if (lower_on) { lo = min(lo, (int)r.clipped_lower_top); hi = max(hi, (int)r.clipped_bottom); }
    if (upper_on) { lo = min(lo, (int)r.clipped_top); hi = max(hi, (int)r.clipped_upper_bottom); }
    if (gaps.lo() < gaps.hi()) { lo = min(lo, gaps.lo()); hi = max(hi, gaps.hi()); }
    lo = max(lo, y0); hi = min(hi, y1);
    const int filled_lo = gaps.filled_lo(), filled_hi = gaps.filled_hi();
    // copies taken by value: a choice between members of `r` made per row would be a choice between addresses and
    // would keep the whole record in private memory
    const int side_tex0 = r.side_tex[0], side_tex1 = r.side_tex[1], side_tex2 = r.side_tex[2];
    const float origin0 = r.view_ceiling, origin1 = r.other_floor, origin2 = r.other_ceiling;
    const bool tail0 = group_valid[0], tail1 = group_valid[1], tail2 = group_valid[2];
    const float tail_row0 = group_bottom[0], tail_row1 = group_bottom[1], tail_row2 = group_bottom[2];
    for (int y = lo; y < hi; ++y) {
        if (y >= filled_lo && y < filled_hi) { y = filled_hi - 1; continue; }   // tier pixels already: nothing to add
        const float py = (float)y;
        unsigned int meta = pb.m(y);
        bool ceiling_span = (r.bits & PB_MARK_CEILING) && (py >= c.ceiling_clip) && (py < ceiling_plane_bottom);
        bool floor_span = (r.bits & PB_MARK_FLOOR) && (py >= floor_plane_top) && (py < c.floor_clip);
        bool meta_dirty = false;
        if (!(meta & META_FILLED) && ((meta >> META_SECTOR_SHIFT) & META_SECTOR_MASK) == 0 && (ceiling_span || floor_span)) {
            meta |= ((unsigned)(r.render_current + 1) << META_SECTOR_SHIFT) | (floor_span ? META_FLOOR : 0);
            meta_dirty = true;
        }
        bool one_span = one_sided && (py >= r.clipped_top) && (py < r.clipped_bottom);
        bool lower_span = lower_on && (py >= r.clipped_lower_top) && (py < r.clipped_bottom);
        bool upper_span = upper_on && (py >= r.clipped_top) && (py < r.clipped_upper_bottom);
        if (one_span || lower_span || upper_span) {
            int texture_id = one_span ? side_tex0 : (lower_span ? side_tex1 : side_tex2);
            if (texture_id >= 0 && !(meta & META_FILLED)) {
                bool bottom_tail = (one_span && tail0 && py >= tail_row0) ||
                                   (lower_span && tail1 && py >= tail_row1) ||
                                   (upper_span && tail2 && py >= tail_row2);
                i64 tu = tb.wrap_column(texture_id, u_base);
                float origin_z = one_span ? origin0 : (lower_span ? origin1 : origin2);
                int height_bits = tb.height_bits(texture_id);
                i64 vertical_step = mul64(swall, shl64(1, 14 - height_bits));
                i64 screen_delta = (i64)y * FIXED_UNIT - L.center_fixed + FIXED_UNIT;
                i64 texture_mid = round_to_i64((origin_z - L.view_z) * 65536.0f + r.offset_y * 65536.0f);
                i64 fraction = shl64(texture_mid, 16 - height_bits) + (mul64(vertical_step, screen_delta) >> 16);
                i64 tv = (fraction & UINT32_MASK) >> (32 - height_bits);
                unsigned char texel = m->tex_atlas[((size_t)texture_id * m->tex_max_h + tv) * m->tex_max_w + tu];
                const unsigned colour = colormap[(bottom_tail ? shade_group : shade_own) * 256 + texel];
                if (DEPTH) pb.s(y) = r.distance;
                const float held = (meta & META_WALL_MASK) ? pb.d(y) : GD_INF;   // no clip recorded yet
                if (r.distance < held) { pb.d(y) = r.distance; meta = (meta & ~META_WALL_MASK) | (unsigned)(wi + 1); }
                meta = (meta & ~(META_SECTOR_MASK << META_SECTOR_SHIFT)) | (colour << META_SECTOR_SHIFT) | META_FILLED;
                meta_dirty = true;
            }
        }
        if (meta_dirty) pb.m(y) = meta;
    }
}

// engine.py:12885-13371.  PART: ADVANCE_ALL, or only the column's clips, masked-drawseg snapshot and sprite silhouettes
// (ADVANCE_CLIPS: what needs the projected rows and touches pixels), or only the traversal state (ADVANCE_STATE: next
// sector, previous distance, pending boundaries; it reads neither rows nor clips).
#define ADVANCE_ALL 0
#define ADVANCE_STATE 1
#define ADVANCE_CLIPS 2
template <bool SPLIT, int PART>
__device__ __forceinline__ bool pass_advance(const ColumnCtx &cc, ColumnState &c, const PassColumn &r, PixelBuffers &pb, SilhouetteBounds &sb, bool window_untouched, GapRange &gaps) {
    const gd_map_desc *m = cc.m;
    const MapView &mv = cc.mv;
    const LaneCtx &L = *cc.c;
    const ColumnState before = c;
    const int x = cc.x;
    const int cs = c.current_sector;
    const int cur = cs < 0 ? 0 : cs;
    const int wi = r.wall;
    const float distance = r.distance;
    const bool valid = r.bits & PB_VALID, raster_valid = r.bits & PB_RASTER, one_sided = r.bits & PB_ONE_SIDED;
    auto incident = [&](int w) { return mv.sec(w, 0) == cur || mv.sec(w, 1) == cur; };
  if (PART != ADVANCE_STATE) {
    // o. clip updates (engine.py:12888-12913)
    bool draws_upper = (r.view_ceiling > r.other_ceiling) && (r.side_tex[2] >= 0);
    if (raster_valid && !one_sided && (draws_upper || (r.bits & PB_MARK_CEILING))) c.ceiling_clip = draws_upper ? r.clipped_upper_bottom : r.clipped_top;
    bool draws_lower = (r.view_floor < r.other_floor) && (r.side_tex[1] >= 0);
    if (raster_valid && !one_sided && (draws_lower || (r.bits & PB_MARK_FLOOR))) c.floor_clip = draws_lower ? r.clipped_lower_top : r.clipped_bottom;
    // p. masked drawseg snapshot (engine.py:12914-12939)
    if (raster_valid && !one_sided && (r.side_tex[0] >= 0) && (distance < c.masked_distance)) {
        c.masked_ceiling_clip = c.ceiling_clip; c.masked_floor_clip = c.floor_clip; c.masked_distance = distance; c.masked_wall = wi;
    }
    // q. sprite silhouettes (engine.py:12943-12964)
    if (raster_valid && !one_sided) {
        bool masked_texture = r.side_tex[0] >= 0;
        bool bottom_sil = (r.view_floor > r.other_floor) || (L.view_z < r.other_floor) || masked_texture;
        bool top_sil = (r.view_ceiling < r.other_ceiling) || (L.view_z > r.other_ceiling) || masked_texture;
        // pass_paint, finding the window untouched, has written the silhouette into the rows that this pass took out
        // of it: [new floor clip, old floor clip) at the bottom, [old ceiling clip, new ceiling clip) at the top
        auto row_of = [](float clip) { return clip <= 0.0f ? 0 : (clip >= (float)VH ? VH : (int)clip); };
        const int old_floor = row_of(before.floor_clip), old_ceiling = row_of(before.ceiling_clip);
        if (window_untouched && silhouette_folds(r)) {
            // one call per side: the rows already done differ.  pass_paint stays inside the old window, and a sector whose
            // ceiling lies below its floor can carry a clip past the window's other end: then the rows beyond that end
            // are not done, and the range is cut there (apply_silhouette then takes no short cut and visits them all).
            apply_silhouette(pb, sb, x, bottom_sil, false, c.floor_clip, c.ceiling_clip, distance, wi, max(row_of(c.floor_clip), old_ceiling), old_floor);
            apply_silhouette(pb, sb, x, false, top_sil, c.floor_clip, c.ceiling_clip, distance, wi, old_ceiling, min(row_of(c.ceiling_clip), old_floor));
        } else {
            apply_silhouette(pb, sb, x, bottom_sil, top_sil, c.floor_clip, c.ceiling_clip, distance, wi, 0, 0);
        }
    }
    // r. clips of the geometric portal behind a projected solid (engine.py:12969-13069)
    if (r.bits & PB_PS_KEEPS) {
        int path = r.ps_path_index;
        int path_safe_other = r.ps_other < 0 ? 0 : r.ps_other;
        const Tables &tb = *cc.tb;
        float pof = tb.floor_h(path_safe_other), poc = tb.ceil_h(path_safe_other);
        int pside = (r.bits & PB_PS_FROM_FRONT) ? 0 : 1;
        const int *ptex = m->side_tex + (path * 2 + pside) * 3;
        const float path_top = r.path_top, path_bottom = r.path_bottom, path_lower_top = r.path_lower_top, path_upper_bottom = r.path_upper_bottom;
        float pct = fmaxf(path_top, c.ceiling_clip);
        float pcb = fminf(path_bottom, c.floor_clip);
        float pcub = fmaxf(fminf(path_upper_bottom, c.floor_clip), pct);
        float pclt = fminf(fmaxf(path_lower_top, c.ceiling_clip), pcb);
        bool light_differs = tb.light(r.render_current) != tb.light(path_safe_other);
        bool p_draws_upper = (r.view_ceiling > poc) && (ptex[2] >= 0);
        bool p_marks_ceiling = (r.view_ceiling != poc) || (tb.ceil_tex(r.render_current) != tb.ceil_tex(path_safe_other)) || light_differs;
        bool p_draws_lower = (r.view_floor < pof) && (ptex[1] >= 0);
        bool p_marks_floor = (r.view_floor != pof) || (tb.floor_tex(r.render_current) != tb.floor_tex(path_safe_other)) || light_differs;
        float new_ceiling = c.ceiling_clip, new_floor = c.floor_clip;
        if (p_draws_upper || p_marks_ceiling) new_ceiling = p_draws_upper ? pcub : pct;
        if (p_draws_lower || p_marks_floor) new_floor = p_draws_lower ? pclt : pcb;
        if (window_untouched) {
            // These clips move without anything being painted or claimed: the rows they take out of an untouched
            // window would leave it unwritten.  They show the flat pass's picture.
            auto row_of = [](float clip) { return clip <= 0.0f ? 0 : (clip >= (float)VH ? VH : (int)clip); };
            const int window_top = row_of(c.ceiling_clip), window_bottom = row_of(c.floor_clip);
            zero_rows(pb, gaps, x, window_top, min(row_of(new_ceiling), window_bottom));
            zero_rows(pb, gaps, x, max(row_of(new_floor), window_top), window_bottom);
        }
        c.ceiling_clip = new_ceiling; c.floor_clip = new_floor;
        bool pmasked = ptex[0] >= 0;
        bool pbottom = (r.view_floor > pof) || (L.view_z < pof) || pmasked;
        bool ptop = (r.view_ceiling < poc) || (L.view_z > poc) || pmasked;
        apply_silhouette(pb, sb, x, pbottom, ptop, c.floor_clip, c.ceiling_clip, r.ps_path_distance, path, 0, 0);
    }
  }
    if (PART == ADVANCE_CLIPS) return false;
    // s. next sector (engine.py:13070-13241)
    const float prior = before.previous_distance;
    const float prior_eps = prior + 1e-3f;
    const bool geometric_intersection = r.bits & PB_GEOMETRIC;
    bool endpoint_only_portal = valid && !one_sided && !geometric_intersection;
    const int other_sector = r.other_sector;
    float pd = prior;
    int next_sector = -1;
    bool endpoint_portal_bridge = false;
    int ppb_idx = 0, gp_other = -1; float gpd = GD_INF;
    if (endpoint_only_portal) {
        const float dist_eps = distance + 1e-3f;
        float cnd = GD_INF, ond = GD_INF; int cni = 0x7fffffff, oni = 0x7fffffff;
        float csd = GD_INF, osd = GD_INF;
        int gpi = 0x7fffffff; bool gp_along_hi = false;
        const int v0 = mv.vert(wi, 0), v1 = mv.vert(wi, 1);
        for (int k0 = 0; k0 < cc.count; k0 += CAND_BATCH) {
            Cand batch[CAND_BATCH];
            cc.cand_batch(k0, batch);
#pragma unroll
            for (int j = 0; j < CAND_BATCH; ++j) {
                if (k0 + j >= cc.count) continue;
                const Cand q = batch[j];
                int w = q.wall; float d = q.dist;
                bool os = q.s1 < 0;
                bool inc = (q.s0 == cur || q.s1 == cur), oinc = (q.s0 == other_sector || q.s1 == other_sector);
                bool future = ((q.flags & CF_GEO) || os) && (d > dist_eps);
                if (future) {
                    if (inc) take_min(d, w, cnd, cni);
                    if (oinc) take_min(d, w, ond, oni);
                }
                bool shares_endpoint = (int)q.v0 == v0 || (int)q.v0 == v1 || (int)q.v1 == v0 || (int)q.v1 == v1;
                bool shared_solid = os && (shares_endpoint || (q.flags & CF_LEDGE)) && (d > prior_eps) && (d <= dist_eps);
                if (shared_solid) {
                    if (inc && d < csd) csd = d;
                    if (oinc && d < osd) osd = d;
                }
                bool sgp = (q.flags & CF_GEO) && inc && shares_endpoint && !os && (d > prior_eps) && (fabsf(d - distance) <= (1.0f / 16.0f));
                if (sgp && (d < gpd || (d == gpd && w < gpi))) { gpd = d; gpi = w; gp_along_hi = (q.flags & CF_ALONG_HI) != 0; }
            }
        }
        if (!finitef(cnd)) cni = 0;
        if (!finitef(ond)) oni = 0;
        bool enters_tied_strip = finitef(cnd) && (cni == oni) && mv.opposing(wi, cni);
        bool enters_other = (other_sector >= 0) && ((ond < cnd) || enters_tied_strip);
        bool enters_shared = (other_sector >= 0) && (osd < csd);
        bool uses_geometric_path = false;
        if (finitef(gpd)) {
            bool gp_from_front = cs == mv.sec(gpi, 0);
            gp_other = gp_from_front ? mv.sec(gpi, 1) : mv.sec(gpi, 0);
            uses_geometric_path = gp_other >= 0;
            if (uses_geometric_path) {
                int pb_slot = gp_along_hi ? 1 : 0;
                bool ppb_exists = mv.portal_bridge(pb_slot, gpi, wi, &ppb_idx);
                if (ppb_exists) {
                    Eval qb = cc.eval(ppb_idx);
                    endpoint_portal_bridge = (qb.flags & CF_PROJ) && (qb.flags & CF_LEDGE) && (qb.dist > prior_eps) && (fabsf(qb.dist - gpd) <= tolerance_of(gpd));
                }
            }
        }
        // t. previous_distance (engine.py:13242-13262)
        if (r.bits & PB_NO_KEEPS) pd = r.no_path_distance;
        else if (r.bits & PB_PS_KEEPS) pd = r.ps_path_distance;
        else if (enters_shared && (osd < distance)) pd = prior;
        else if (uses_geometric_path) pd = gpd;
        else pd = distance;
        if (r.bits & PB_NO_KEEPS) next_sector = r.no_path_other;
        else if (r.bits & PB_PS_KEEPS) next_sector = r.ps_other;
        else if (uses_geometric_path) next_sector = gp_other;
        else if (enters_other || enters_shared) next_sector = other_sector;
        else next_sector = cs;
    } else {
        if (valid) {
            if (r.bits & PB_NO_KEEPS) pd = r.no_path_distance;
            else if (r.bits & PB_PS_KEEPS) pd = r.ps_path_distance;
            else pd = distance;
        }
        if (r.bits & PB_NO_KEEPS) next_sector = r.no_path_other;
        else if (r.bits & PB_PS_KEEPS) next_sector = r.ps_other;
        else if (valid && !one_sided && geometric_intersection) next_sector = other_sector;
        else next_sector = -1;
    }
    bool completes_pending_portal_bridge = valid && (before.flags & ST_PB) && (wi == before.pend_pb_index);
    if (valid && endpoint_portal_bridge) pd = prior;
    if (valid && completes_pending_portal_bridge) pd = fmaxf(distance, before.pend_pb_exit);
    c.previous_distance = pd;
    // carried state (engine.py:13276-13313, 13355-13371)
    bool starts_po = r.bits & PB_REPLACE_NP;
    if (starts_po) c.pend_po_vertex = r.sel_vertex;
    bool po = starts_po || ((before.flags & ST_PO) && (r.bits & PB_CONTINUES_PO));
    if (endpoint_only_portal) {
        c.pend_ep_vertex = mv.vert(wi, (r.bits & PB_FINAL_ALONG_HI) ? 1 : 0);
        c.pend_ep_wall = wi;
    }
    if (r.bits & PB_FORWARD_BRIDGE) c.pend_eb_index = r.fb_idx;
    if (endpoint_portal_bridge) next_sector = other_sector;
    if (completes_pending_portal_bridge) next_sector = before.pend_pb_sector;
    if (endpoint_portal_bridge) { c.pend_pb_index = ppb_idx; c.pend_pb_sector = gp_other; c.pend_pb_exit = gpd; }
    c.flags = (po ? ST_PO : 0) | (endpoint_only_portal ? ST_EP : 0) | ((r.bits & PB_FORWARD_BRIDGE) ? ST_EB : 0) | (endpoint_portal_bridge ? ST_PB : 0);
    c.current_sector = next_sector;
    return !same_state(before, c);
}

// engine.py:13424-13744 for one column
template <bool DEPTH, bool SPLIT>
__device__ __forceinline__ void masked_midtexture(const ColumnCtx &cc, const ColumnState &c, PixelBuffers &pb, const unsigned char *colormap) {
    const gd_map_desc *m = cc.m;
    const MapView &mv = cc.mv;
    const LaneCtx &L = *cc.c;
    const int x = cc.x;
    float md = GD_INF; int mw = 0x7fffffff; int mside = 0; int cand_flags = 0;
    for (int k0 = 0; k0 < cc.count; k0 += CAND_BATCH) {
        Cand batch[CAND_BATCH];
        cc.cand_batch(k0, batch);
#pragma unroll
        for (int j = 0; j < CAND_BATCH; ++j) {
            if (k0 + j >= cc.count) continue;
            const Cand q = batch[j];
            int w = q.wall;
            if (!(q.flags & CF_PROJ) || (q.s1 < 0)) continue;
            int sidew = (q.flags & CF_FF) ? 0 : 1;   // engine.py:13436-13444, the float32 facing test
            if (!(q.flags & CF_MASKED)) continue;     // no mid-texture on that side
            if (q.dist < md || (q.dist == md && w < mw)) { md = q.dist; mw = w; mside = sidew; cand_flags = q.flags; }
        }
    }
    if (!finitef(md)) return;
    int texture_id = m->side_tex[(mw * 2 + mside) * 3];
    if (texture_id < 0) texture_id = 0;
    bool left_edge = cand_flags & CF_LEDGE;
    bool has_saved = c.masked_wall == mw;
    if (!(has_saved || left_edge)) return;
    const WallRec &wr = cc.rec(mw);
    const FragmentChoice wr_fragment = choose_fragment<SPLIT>(m, cc.frags, wr, mw, x);
    int front_sector = mv.sec(mw, 0), back_sector = mv.sec(mw, 1) < 0 ? 0 : mv.sec(mw, 1);
    int light_sector = mside == 0 ? front_sector : back_sector;
    const Tables &tb = *cc.tb;
    float world_top = fminf(tb.ceil_h(front_sector), tb.ceil_h(back_sector));
    const int th = m->tex_h[texture_id];   // the texture's own height, whatever its row mask (engine.py:13480-13483)
    float owall_top = 0, owall_bottom = 0;
#pragma unroll 1
    for (int k = 0; k < 2; ++k) {
        float v = project(L, wr, wr_fragment, k == 0 ? world_top : world_top - (float)th, x);
        if (k == 0) owall_top = v; else owall_bottom = v;
    }
    float mceil = fmaxf(owall_top, has_saved ? c.masked_ceiling_clip : 0.0f);
    float mfloor = fminf(owall_bottom, has_saved ? c.masked_floor_clip : (float)VH);
    const float *toff = m->side_off + (mw * 2 + mside) * 2;
    i64 h, swall_cur;
    texture_mapping(m, wr, mw, x, &h, &swall_cur);
    i64 repeat = round_to_i64(m->wall_len[mw] * 65536.0f);
    if (mside != 0) h = repeat - h;
    i64 msl = wr.sl, msr = wr.sr;
    if (msl > 0 && h < 0) h = 0;
    if (h >= repeat) h = repeat - 1;
    i64 offx = round_to_i64(toff[0] * 65536.0f);
    i64 mu = tb.wrap_column(texture_id, (h + offx) >> 16);
    int height_bits = ilog2(th);
    i64 vertical_step = mul64(swall_cur, shl64(1, 14 - height_bits));
    i64 center_fixed = L.center_fixed;
    i64 texture_mid = round_to_i64((world_top - L.view_z) * 65536.0f + toff[1] * 65536.0f);
    int safe_left = (int)clampi(msl, 0, SW - 1), safe_last = (int)clampi(msr - 1, 0, SW - 1);
    i64 dummy_h, start_swall = 0, end_swall = 0;
#pragma unroll 1
    for (int k = 0; k < 2; ++k) {
        i64 sw;
        texture_mapping(m, wr, mw, k == 0 ? safe_left : safe_last, &dummy_h, &sw);
        if (k == 0) start_swall = sw; else end_swall = sw;
    }
    auto iscale_of = [](i64 swall) {
        i64 s = mul64(swall, FIXED_UNIT) >> 18;
        if (s >= 0 && s < 3) return (i64)3;
        if (s > -3 && s < 0) return (i64)-3;
        return s;
    };
    i64 start_scale = tdiv(1LL << 32, iscale_of(start_swall)), end_scale = tdiv(1LL << 32, iscale_of(end_swall));
    i64 scale_step = tdiv(end_scale - start_scale, max64(msr - msl, 1));
    i64 sprite_scale = start_scale + mul64(scale_step, (i64)x - msl);
    i64 top_screen = center_fixed - (mul64(texture_mid, sprite_scale) >> 16);
    i64 post_top = top_screen >> 16;
    i64 post_bottom = ((top_screen + mul64(sprite_scale, th) - FIXED_UNIT) >> 16) + 1;
    i64 clipped_top = max64(post_top, (i64)mceil);
    i64 clipped_bottom = min64(post_bottom, (i64)mfloor);
    i64 dc_iscale = mul64(swall_cur, FIXED_UNIT) >> 18;
    bool initial_post = clipped_top < clipped_bottom;
    i64 frac_start = texture_mid + mul64(clipped_top, dc_iscale) - (mul64(center_fixed - FIXED_UNIT, dc_iscale) >> 16);
    i64 frac_end = frac_start + mul64(clipped_bottom - clipped_top - 1, dc_iscale);
    bool extends = initial_post && ((float)clipped_bottom < mfloor) && (frac_end < (i64)th * FIXED_UNIT - dc_iscale);
    clipped_bottom += extends ? 1 : 0;
    const float4 wl = *reinterpret_cast<const float4 *>(m->walls + 4 * mw);
    bool horizontal = fabsf(wl.w - wl.y) < 1e-6f, vertical = fabsf(wl.z - wl.x) < 1e-6f;
    float contrast = vertical ? 16.0f : (horizontal ? -16.0f : 0.0f);
    float light = (tb.light(light_sector) + (float)(L.flash_light * 16)) + contrast;
    i64 shade = wall_shade(light, wall_visibility(wr_fragment.lights ? *wr_fragment.rec : wr, mside, x));
    int y0 = (int)clampi(clipped_top, 0, VH), y1 = (int)clampi(clipped_bottom, 0, VH);
    // WALL_ROWS rows at a time: texels and meta words are asked for together, then the stores
    // as in pass_paint: only the low 32 bits of the row fraction matter, and they advance by the step's low 32 bits
    const unsigned row_step = (unsigned)vertical_step;
    const unsigned row_base = (unsigned)(shl64(texture_mid, 16 - height_bits) + (mul64(vertical_step, FIXED_UNIT - center_fixed) >> 16));
    const size_t texel_base = (size_t)texture_id * m->tex_max_h * m->tex_max_w + (size_t)mu;
    const unsigned atlas_w = (unsigned)m->tex_max_w;
    for (int yb = y0; yb < y1; yb += WALL_ROWS) {
        unsigned char texel[WALL_ROWS]; unsigned int word[WALL_ROWS];
#pragma unroll
        for (int j = 0; j < WALL_ROWS; ++j) {
            const int y = yb + j < y1 ? yb + j : y1 - 1;
            const unsigned fraction = row_base + row_step * (unsigned)y;
            const unsigned mv_ = (fraction >> (31 - height_bits)) >> 1;
            texel[j] = m->tex_atlas[texel_base + __umul24(mv_, atlas_w)];
            word[j] = pb.m(y);
        }
#pragma unroll
        for (int j = 0; j < WALL_ROWS; ++j) {
            const int y = yb + j;
            if (y >= y1) continue;
            // the texel goes to the frame where there is one; otherwise it waits in the sprite clip plane, which nothing
            // reads any more once a column's traversal is over, for the kernel that assembles the frame
            const unsigned char colour = colormap[shade * 256 + texel[j]];
            if (pb.frame) pb.f(y) = colour;
            else pb.d(y) = __uint_as_float((unsigned)colour);
            pb.m(y) = word[j] | META_MASKED;
            if (DEPTH) pb.s(y) = md;
        }
    }
}

// How long a column's traversal runs is set by the portals it crosses: the two-sided linedefs its ray hits before the
// nearest blocking one.  Columns differ by a factor of ten, a wavefront runs as long as its longest column, and a launch
// ends with its longest wavefront.  So the screen is cut into segments of SEG_COLS columns, a wavefront takes
// 64 / SEG_COLS segments of about the same length (whatever lanes they belong to), and the longest go first.  The length
// is taken to be the longest candidate list of the segment, which wall_setup_kernel has counted anyway: walking the lists
// to count the portals proper orders the segments a little better (the traversal gains 0.04 ms on the 4000-linedef map)
// but the walk costs 0.11 ms.  strip_key_kernel takes the maxima, strip_order_kernel sorts them (one block, counting sort).
// Narrow segments waste fewer column passes (on the 4000-linedef map 69 % of the passes a wavefront runs are useful with
// whole 64-column strips, 80 % with two sorted 32-column segments, 89 % with four of 16), but unrelated segments share no
// linedefs, branches or row ranges, and a pass costs what the union of its columns' paths costs: measured, the traversal
// takes 3.86 ms with 64 or 32 columns a segment, 4.06 ms with 16 and 4.23 ms with 8.  Hence whole strips.
__global__ void __launch_bounds__(256) strip_key_kernel(int lane_count, Scratch sc) {
    const int strip = blockIdx.x * 4 + (threadIdx.x >> 6);
    const int local = strip / (SW / 64);
    if (local >= lane_count) return;
    const int x = (strip - local * (SW / 64)) * 64 + (threadIdx.x & 63);
    int length = sc.cand_count[(size_t)local * SW + x];
    if (length > CAND_MAX) { request_spill_slot(sc, local * SW + x); length = CAND_MAX; }   // cand_spill_kernel runs next
#pragma unroll
    for (int step = 1; step < SEG_COLS; step <<= 1) length = max(length, __shfl_xor(length, step));
    if ((x & (SEG_COLS - 1)) == 0) sc.strip_key[local * SEGS_PER_LANE + x / SEG_COLS] = (unsigned char)length;   // at most CAND_MAX
}

__global__ void __launch_bounds__(1024) strip_order_kernel(int strips, Scratch sc) {
    __shared__ int histogram[CAND_MAX + 1], position[CAND_MAX + 1];
    for (int k = threadIdx.x; k <= CAND_MAX; k += blockDim.x) histogram[k] = 0;
    __syncthreads();
    for (int s = threadIdx.x; s < strips; s += blockDim.x) atomicAdd(&histogram[sc.strip_key[s]], 1);
    __syncthreads();
    if (threadIdx.x == 0) {
        int running = 0;
        for (int k = CAND_MAX; k >= 0; --k) { position[k] = running; running += histogram[k]; }
    }
    __syncthreads();
    for (int s = threadIdx.x; s < strips; s += blockDim.x) sc.strip_order[atomicAdd(&position[sc.strip_key[s]], 1)] = s;
}

// The traversal in two kernels.  Which drawseg a column pass selects, and where the column goes next, depends on the map,
// the camera and the column's ray alone, never on projected rows or clips: wall_select_kernel runs that half
// (pass_select without the projection, pass_advance's state part) and records one PassRec per pass; wall_raster_kernel
// runs the other half over the records (pass_geometry, pass_clip, pass_paint, pass_advance's clip part, the masked mid-texture).
// Each half is lighter in registers and in code than the two together, so more of its wavefronts share a SIMD and
// its pass loop fits the instruction cache.  Same segment order and one wavefront per segment in both.
#define SELECT_STRIPS_PER_GROUP 1
// The kernel lasts as long as its longest strips: on the 4000-linedef map the 256 longest of 20,480 take 0.94 ms with the
// chip to themselves, all of them together 1.22 ms, all but the 4096 longest 0.53 ms.  Such a strip's wavefront is held
// up by its candidate scans (the longest lists, read from device memory beside 20,000 other wavefronts) and by running,
// pass after pass, every rule that any of its 64 columns takes.  So the SELECT_STAGED_STRIPS longest strips (they lead
// the order) go to a launch of their own (STAGED): a strip is shared out over SELECT_STAGED_PARTS wavefronts of 16 columns
// each, which first copy their columns' lists to LDS (16 KB a wavefront) and scan them there.  It runs beside the
// launch for all other strips: 1.22 -> 0.99 ms.  (Measured: 256 to 1024 strips, 1, 2, 4 or 8 parts; lists left in device
// memory: no gain.)
static_assert(SEG_COLS == 64 && SELECT_STRIPS_PER_GROUP == 1, "wall_select_kernel's staged launch: parts of one whole strip per work-group");
template <bool SPLIT, bool STAGED>
__global__ void __launch_bounds__(64 * SELECT_STRIPS_PER_GROUP) wall_select_kernel(DeviceMap dm, int lane_count, Scratch sc, int staged_slots) {
    const gd_map_desc *m = &dm.d;
    __shared__ LaneCtx lane_ctxs[SELECT_STRIPS_PER_GROUP][64 / SEG_COLS];
    constexpr int PARTS = STAGED ? SELECT_STAGED_PARTS : 1, PART_COLS = 64 / PARTS;
    __shared__ uint4 staged_entries[STAGED ? CAND_MAX * PART_COLS : 1];   // [CAND_MAX][PART_COLS] in the staged launch
    const int wave_in_group = threadIdx.x >> 6;
    const int lane_id = threadIdx.x & 63;
    const int segment_in_wave = lane_id / SEG_COLS;
    const int segment_slot = (blockIdx.x / PARTS * SELECT_STRIPS_PER_GROUP + wave_in_group) * (64 / SEG_COLS) + segment_in_wave;
    const int part = blockIdx.x % PARTS;
    const bool live = segment_slot < (STAGED ? staged_slots : lane_count * SEGS_PER_LANE);
    const int segment = live ? sc.strip_order[segment_slot] : 0;
    const int local = segment / SEGS_PER_LANE;
    if ((lane_id & (SEG_COLS - 1)) == 0 && live) lane_ctxs[wave_in_group][segment_in_wave] = sc.ctx[local];
    __syncthreads();
    if (!live) return;
    const LaneCtx &lane_ctx = lane_ctxs[wave_in_group][segment_in_wave];
    // A strip with a column in the spill pool (more entries than the LDS copy holds) is left to the other launch, which
    // covers the staged launch's slots as well and otherwise leaves them alone.  Both ask all 64 columns of the strip.
    const int strip_x = (segment - local * SEGS_PER_LANE) * SEG_COLS;
    const bool long_lists = __ballot(((unsigned)sc.cand_count[(size_t)local * SW + strip_x + lane_id] >> SPILL_SHIFT) != 0) != 0;
    if (STAGED ? long_lists : (segment_slot < staged_slots && !long_lists)) return;   // the same in the whole wavefront
    if (lane_id >= PART_COLS) return;
    const int x = strip_x + part * PART_COLS + lane_id;
    ColumnCtx cc;
    cc.tb = nullptr; cc.m = m; cc.mv.m = m; cc.c = &lane_ctx;
    cc.recs = sc.rec; cc.spans = sc.span;
    cc.rec_base = (unsigned)local * (unsigned)m->wall_count;
    cc.frags = sc.frag_rec + (size_t)local * m->split_count * m->fragment_slots;
    cc.set_list(sc, local, x);
    cc.x = x;
    ray_direction(lane_ctx, x, &cc.rx, &cc.ry);
    if (STAGED) {
        // every lane copies its own column's entries and reads only those: no barrier
        char *mine = reinterpret_cast<char *>(staged_entries) + lane_id * 16;
        const int depth = cc.count;
        for (int k0 = 0; k0 < depth; k0 += CAND_BATCH) {
            Cand batch[CAND_BATCH];
            cc.cand_batch(k0, batch);
#pragma unroll
            for (int j = 0; j < CAND_BATCH; ++j) {
                union { uint4 raw; Cand c; } u;
                u.c = batch[j];
                if (k0 + j < depth) *reinterpret_cast<uint4 *>(mine + (k0 + j) * (PART_COLS * 16)) = u.raw;
            }
        }
        cc.staged = (ColumnCtx::LdsByte *)mine;
        cc.use_staged = true;
    }
    ColumnState st;
    st.current_sector = lane_ctx.sector;
    st.ceiling_clip = 0.0f; st.floor_clip = (float)VH;
    st.masked_ceiling_clip = 0.0f; st.masked_floor_clip = (float)VH; st.masked_distance = GD_INF; st.masked_wall = -1;
    st.previous_distance = 0.0f;
    st.pend_po_vertex = -1; st.pend_ep_vertex = -1; st.pend_ep_wall = 0; st.pend_eb_index = 0;
    st.pend_pb_index = 0; st.pend_pb_sector = -1; st.pend_pb_exit = 0.0f; st.flags = 0;
    bool boundary_has_po = false;
    for (int k = 0; k < cc.count; ++k) if (cc.cand(k).flags & CF_LEDGE) { boundary_has_po = true; break; }
    PassRec *records = sc.pass_rec + ((size_t)local * sc.pass_slots * SW + x);
    float *path_distances = sc.pass_path_distance + ((size_t)local * sc.pass_slots * SW + x);
    PixelBuffers no_pixels; SilhouetteBounds no_bounds; GapRange no_gaps;   // the state part of pass_advance touches none of them
    PassColumn pc;
    bool done = false;
    int recorded = 0;
    const int sectors = m->sector_count;
    for (int pass = 0; pass < sectors; ++pass) {
        if (!done) {
            pass_select<SPLIT>(cc, st, boundary_has_po, pc);
            if (pc.bits & (PB_RASTER | PB_PS_KEEPS)) {
                if (pass < sc.pass_slots) {
                    PassRec rec;
                    rec.wall = (unsigned short)pc.wall; rec.render_current = (unsigned short)pc.render_current;
                    rec.bits = (unsigned short)pc.bits; rec.ps_path = (unsigned short)pc.ps_path_index;
                    rec.ps_other = (short)pc.ps_other; rec.spare = 0; rec.distance = pc.distance;
                    // passes between two recorded ones keep whatever the slot held: the drawing half skips them by their bits
                    for (int skipped = recorded; skipped < pass; ++skipped) records[(size_t)skipped * SW].bits = 0;
                    records[(size_t)pass * SW] = rec;
                    if (pc.bits & PB_PS_KEEPS) path_distances[(size_t)pass * SW] = pc.ps_path_distance;
                    recorded = pass + 1;
                } else {
                    atomicOr(sc.status, STATUS_PASS_OVERFLOW);
                }
            }
            const bool changed = pass_advance<SPLIT, ADVANCE_STATE>(cc, st, pc, no_pixels, no_bounds, false, no_gaps);
            // A pass that found nothing and changed nothing repeats identically for ever.
            if (!(pc.bits & PB_VALID) && !changed) done = true;
        }
        if (__ballot(!done) == 0) break;
    }
    sc.pass_count[(size_t)local * SW + x] = (unsigned char)recorded;
}

// One wavefront per 64 / SEG_COLS segments.  Segments share nothing but read-only tables; a work-group of the drawing
// half is WALL_STRIPS_PER_GROUP wavefronts (neighbours in the longest-first order) only so that the LDS copies of
// those tables, 16.7 KB, are held once per group rather than once per wavefront (a CU has 160 KB of LDS and room for
// sixteen of these wavefronts at 128 registers).  After the staging barrier the wavefronts never meet again.
#define WALL_STRIPS_PER_GROUP 2
// DEPTH: also keep the depth of every wall pixel (frames that draw decals).  SPLIT: the map has linedefs with
// BSP projection fragments.
template <bool DEPTH, bool SPLIT>
__global__ void __launch_bounds__(64 * WALL_STRIPS_PER_GROUP) __attribute__((amdgpu_waves_per_eu(4, 4))) wall_raster_kernel(DeviceMap dm, int lane_count, Scratch sc, unsigned char *frame_base, size_t frame_stride) {
    const gd_map_desc *m = &dm.d;
    __shared__ LaneCtx lane_ctxs[WALL_STRIPS_PER_GROUP][64 / SEG_COLS];
    __shared__ unsigned char colormap_lds[32 * 256];   // shade rows 0..31 are the only ones indexed
    __shared__ float4 sector_lds[LDS_SECTORS];
    __shared__ TexLds tex_lds;
    const int wave_in_group = threadIdx.x >> 6;
    const int lane_id = threadIdx.x & 63;
    const int segment_in_wave = lane_id / SEG_COLS;
    const int segment_slot = (blockIdx.x * WALL_STRIPS_PER_GROUP + wave_in_group) * (64 / SEG_COLS) + segment_in_wave;
    const bool live = segment_slot < lane_count * SEGS_PER_LANE;
    const int segment = live ? sc.strip_order[segment_slot] : 0;
    const int local = segment / SEGS_PER_LANE;
    Tables tb;
    stage_tables(m, sector_lds, &tex_lds, tb);
    if ((lane_id & (SEG_COLS - 1)) == 0 && live) lane_ctxs[wave_in_group][segment_in_wave] = sc.ctx[local];
    for (int k = threadIdx.x; k < 32 * 256 / 4; k += blockDim.x) reinterpret_cast<unsigned int *>(colormap_lds)[k] = reinterpret_cast<const unsigned int *>(m->colormap)[k];
    __syncthreads();
    if (!live) return;   // whole segments: the groups of four columns that exchange values below live or leave together
    const LaneCtx &lane_ctx = lane_ctxs[wave_in_group][segment_in_wave];
    const int x = (segment - local * SEGS_PER_LANE) * SEG_COLS + (lane_id & (SEG_COLS - 1));
    bool window_dirty = false;
    GapRange gaps; gaps.reset();
    ColumnCtx cc;
    cc.tb = &tb; cc.m = m; cc.mv.m = m; cc.c = &lane_ctx;
    cc.recs = sc.rec; cc.spans = sc.span;
    cc.rec_base = (unsigned)local * (unsigned)m->wall_count;
    cc.frags = sc.frag_rec + (size_t)local * m->split_count * m->fragment_slots;
    cc.set_list(sc, local, x);
    cc.x = x;
    ray_direction(lane_ctx, x, &cc.rx, &cc.ry);
    PixelBuffers pb;
    pb.frame = frame_base;
    pb.meta = sc.meta; pb.clip_depth = sc.clip_depth;
    pb.scene_depth = DEPTH ? sc.scene_depth : nullptr;
    pb.word_column = ((unsigned)local * (VH * SW) + (unsigned)x) * 4u;
    pb.frame_column = (unsigned)local * (unsigned)frame_stride + (unsigned)x;
    // the meta plane arrives with whatever the last frame left: see GapRange for how every row gets written
    ColumnState st;   // only the clips and the masked-drawseg snapshot live here; the traversal state stayed in wall_select_kernel
    st.current_sector = -1;
    st.ceiling_clip = 0.0f; st.floor_clip = (float)VH;
    st.masked_ceiling_clip = 0.0f; st.masked_floor_clip = (float)VH; st.masked_distance = GD_INF; st.masked_wall = -1;
    st.previous_distance = 0.0f;
    st.pend_po_vertex = -1; st.pend_ep_vertex = -1; st.pend_ep_wall = 0; st.pend_eb_index = 0;
    st.pend_pb_index = 0; st.pend_pb_sector = -1; st.pend_pb_exit = 0.0f; st.flags = 0;
    SilhouetteBounds sb; sb.bot_row = VH; sb.top_row = 0; sb.bot_depth = -GD_INF; sb.top_depth = -GD_INF;
    const int passes = sc.pass_count[(size_t)local * SW + x];
    const PassRec *records = sc.pass_rec + ((size_t)local * sc.pass_slots * SW + x);
    const float *path_distances = sc.pass_path_distance + ((size_t)local * sc.pass_slots * SW + x);
    PassColumn pc;
    pc.wall = 0; pc.side = 0; pc.bits = 0; pc.visibility = 0;
    pc.clipped_top = 0.0f; pc.clipped_bottom = 0.0f; pc.clipped_upper_bottom = 0.0f; pc.clipped_lower_top = 0.0f;
    for (int pass = 0; __ballot(pass < passes) != 0; ++pass) {
        const bool mine = pass < passes;
        bool draws = false;
        if (mine) {
            const PassRec rec = records[(size_t)pass * SW];
            draws = (rec.bits & (PB_RASTER | PB_PS_KEEPS)) != 0;
            pc.bits = draws ? (int)rec.bits : 0;
            if (draws) {
                pc.wall = rec.wall; pc.render_current = rec.render_current; pc.distance = rec.distance;
                pc.ps_path_index = rec.ps_path; pc.ps_other = rec.ps_other;
                pc.ps_path_distance = (rec.bits & PB_PS_KEEPS) ? path_distances[(size_t)pass * SW] : 0.0f;
                pass_geometry<SPLIT>(cc, pc);
                pass_clip(cc, st.ceiling_clip, st.floor_clip, pc);
            }
        } else {
            pc.bits = 0;   // a finished column draws no tier: its group of four has no common tail
        }
        // 4-column wallscan groups (engine.py:12688-12761): the aligned group of four columns agrees on its drawseg, on
        // which tiers all four draw and on the rows all four share.  The four lanes of a group are one DPP quad, so every
        // exchange is a vector move with a lane pattern (no trip through the LDS crossbar), and the minima, maxima and
        // conjunctions take two steps each.  Every lane of the wavefront is active here.
        const int w0 = quad_first(pc.wall), s0 = quad_first(pc.side);
        const int GROUP_AGREES = 0x1;   // takes PB_VALID's place in the word that is and-ed over the group
        const int agreed = quad_and((pc.bits & (PB_TIER0 | PB_TIER1 | PB_TIER2)) | ((pc.wall == w0 && pc.side == s0) ? GROUP_AGREES : 0));
        const bool same_group = (agreed & GROUP_AGREES) != 0;
        // a value that is not a number never becomes a common top or bottom (std::max(-inf, nan) is -inf)
        const float shared_top = fmaxf(-GD_INF, quad_max(pc.clipped_top)), shared_lower_top = fmaxf(-GD_INF, quad_max(pc.clipped_lower_top));
        const float shared_bottom = fminf(GD_INF, quad_min(pc.clipped_bottom)), shared_upper_bottom = fminf(GD_INF, quad_min(pc.clipped_upper_bottom));
        const float common_bottom[3] = {shared_bottom, shared_bottom, shared_upper_bottom};
        const i64 first_group_visibility = ((i64)quad_first((int)(pc.visibility >> 32)) << 32) | (i64)(unsigned)quad_first((int)(pc.visibility & 0xFFFFFFFFLL));
        bool group_valid[3];
        group_valid[0] = same_group && (agreed & PB_TIER0) && (shared_top < shared_bottom);
        group_valid[1] = same_group && (agreed & PB_TIER1) && (shared_lower_top < shared_bottom);
        group_valid[2] = same_group && (agreed & PB_TIER2) && (shared_top < shared_upper_bottom);
        if (draws) {
            pass_paint<DEPTH>(cc, st, pc, pb, group_valid, common_bottom, first_group_visibility, colormap_lds, window_dirty, gaps);
            pass_advance<SPLIT, ADVANCE_CLIPS>(cc, st, pc, pb, sb, !window_dirty, gaps);
        }
    }
    // what is left of a window no one-sided drawseg closed shows the flat pass's picture
    if (!window_dirty) zero_rows(pb, gaps, x, st.ceiling_clip <= 0.0f ? 0 : (int)st.ceiling_clip, st.floor_clip >= (float)VH ? VH : (int)st.floor_clip);
    masked_midtexture<DEPTH, SPLIT>(cc, st, pb, colormap_lds);
    // The view pixels no wall tier, plane or masked texture covers: the flat pass selects them (flat_gap_column_kernel) and
    // flat_shade_kernel paints them.  More than the list holds: the lane is handled pixel by pixel.
    for (int y = gaps.lo(), gap_end = gaps.hi(); y < gap_end; ++y) {
        const unsigned int word = pb.m(y);
        if ((word & (META_FILLED | META_MASKED)) || ((word >> META_SECTOR_SHIFT) & META_SECTOR_MASK) != 0) continue;
        const int slot = atomicAdd(&sc.flat_list_count[local], 1);
        if (slot < FLAT_LIST_MAX) sc.flat_list[(size_t)local * FLAT_LIST_MAX + slot] = y * SW + x;
    }
}

// ---------------------------------------------------------------------------------------------
// plane shading, one thread per view pixel.  A pixel no wall tier owns shows a flat: the
// visplane the wall traversal marked for it (engine.py:13372-13405) or, where no drawseg marked
// one, the sector the per-pixel plane rays selected (engine.py:11145-11163).  Doing both here
// shades every pixel once, in a kernel light enough to run at full occupancy.
// ---------------------------------------------------------------------------------------------
#define SHADE_RUN 4      // neighbouring pixels of a row per thread
#define SHADE_TILES 13   // tiles (256 runs) per block: 65 tiles per view = 5 blocks per lane (each block stages the tables once)
#define SHADE_GROUP 1    // tiles per step
static_assert(SW % SHADE_RUN == 0 && SHADE_RUN == 4, "plane_shade_kernel: a run is one 16-byte load of per-pixel words and one 4-byte store");
// DEPTH: also keep the depth of every pixel no wall tier covers (frames that draw decals).  STAGED: the lane's plane table
// is short enough for LDS (the kernel then reads it with LDS instructions; a pointer that may be either costs more).
template <bool DEPTH, bool STAGED>
// Eight wavefronts per SIMD.  The kernel runs beside the flat pass (launch_chunk) and the billboards follow it on the same
// stream: the sooner it is done, the sooner they are (with the billboards still after the flat pass, five wavefronts per
// SIMD and two tiles per step were better: the flat pass's kernels found more room beside it).
__global__ void __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(8, 8))) plane_shade_kernel(DeviceMap dm, int lane_count, Scratch sc, unsigned char *frame_base, size_t frame_stride) {
    const gd_map_desc *m = &dm.d;
    __shared__ float4 sector_lds[LDS_SECTORS];
    __shared__ unsigned int sector_level_lds[LDS_SECTORS];
    __shared__ TexLds tex_lds;
    __shared__ unsigned char colormap_lds[32 * 256];
    __shared__ i64 level_plane_lds[2 * PLANE_LEVELS * 2];
    __shared__ i64 step_scale_lds[STEP_TABLE];
    const int local = blockIdx.y;
    if (local >= lane_count) return;     // uniform over the block
    Tables tb;
    stage_tables(m, sector_lds, &tex_lds, tb);
    for (int k = threadIdx.x; k < 32 * 256 / 4; k += blockDim.x) reinterpret_cast<unsigned int *>(colormap_lds)[k] = reinterpret_cast<const unsigned int *>(m->colormap)[k];
    const int floors = m->floor_level_count, levels = floors + m->ceil_level_count;
    const bool tabled = dm.sector_level != nullptr;
    const bool levels_staged = STAGED;
    if (tabled) {
        for (int s = threadIdx.x; s < tb.sector_cached; s += blockDim.x) sector_level_lds[s] = dm.sector_level[s];
        if (levels_staged) for (int k = threadIdx.x; k < 2 * levels; k += blockDim.x) level_plane_lds[k] = sc.level_plane[(size_t)local * levels * 2 + k];
        if (threadIdx.x < STEP_TABLE) step_scale_lds[threadIdx.x] = sc.step_scale[(size_t)local * STEP_TABLE + threadIdx.x];
    }
    __syncthreads();
    LaneTables lt; lt.step_scale = step_scale_lds; lt.floors = floors;
    if (STAGED) lt.level_plane = level_plane_lds;
    else lt.level_plane = sc.level_plane + (size_t)local * levels * 2;
    const LaneCtx &c = sc.ctx[local];
    unsigned char *frame = frame_base + (size_t)local * frame_stride;
    const bool frame_aligned = (reinterpret_cast<size_t>(frame) & 3) == 0;
    const uint4 *meta_groups = reinterpret_cast<const uint4 *>(sc.meta + (size_t)local * VH * SW);
    // A thread takes SHADE_RUN neighbouring pixels of a row (a row is a whole number of runs): their per-pixel words arrive
    // in one load, pixels that show the same plane share everything but two products, and the run's bytes leave in
    // one store.  SHADE_GROUP runs, a tile apart, per step, each stage's loads issued together.
    for (int tile0 = 0; tile0 < SHADE_TILES; tile0 += SHADE_GROUP) {
        unsigned int meta[SHADE_GROUP][SHADE_RUN];
        int first_pixel[SHADE_GROUP];
#pragma unroll
        for (int g = 0; g < SHADE_GROUP; ++g) {
            const int run = (blockIdx.x * SHADE_TILES + tile0 + g) * 256 + threadIdx.x;
            const bool valid = tile0 + g < SHADE_TILES && run < VH * SW / SHADE_RUN;
            first_pixel[g] = valid ? run * SHADE_RUN : -1;
            const uint4 words = meta_groups[valid ? run : 0];
            meta[g][0] = words.x; meta[g][1] = words.y; meta[g][2] = words.z; meta[g][3] = words.w;
            if (valid && run < (GD_SCREEN_HEIGHT - VH) * SW / SHADE_RUN) {   // the empty status bar, rows 208..239
                unsigned char *bar = frame + (size_t)VH * SW + (size_t)run * SHADE_RUN;
                if (frame_aligned) *reinterpret_cast<unsigned int *>(bar) = 0u;
                else for (int k = 0; k < SHADE_RUN; ++k) bar[k] = 0;
            }
        }
        int colormap_row[SHADE_GROUP][SHADE_RUN]; unsigned char texel[SHADE_GROUP][SHADE_RUN];
        unsigned int shades[SHADE_GROUP];   // bit k: pixel k of the run shows a visplane's flat
#pragma unroll
        for (int g = 0; g < SHADE_GROUP; ++g) {
            shades[g] = 0;
            const int pixel0 = first_pixel[g] < 0 ? 0 : first_pixel[g];
            const int y = pixel0 / SW, x0 = pixel0 - y * SW;
            // what names a pixel's plane in its word: the sector and which of its two planes
            const unsigned int PLANE_KEY = (META_SECTOR_MASK << META_SECTOR_SHIFT) | META_FLOOR;
            int leader = -1;
#pragma unroll
            for (int k = 0; k < SHADE_RUN; ++k) {
                const int ps = (int)((meta[g][k] >> META_SECTOR_SHIFT) & META_SECTOR_MASK) - 1;
                texel[g][k] = 0; colormap_row[g][k] = 0;
                if (tabled && first_pixel[g] >= 0 && ps >= 0 && !(meta[g][k] & (META_FILLED | META_MASKED))) {
                    shades[g] |= 1u << k;
                    if (leader < 0) leader = k;
                }
            }
            if (leader < 0) continue;
            const i64 yslope = sc.row_slope[(size_t)local * VH + y];
            unsigned int leader_word = meta[g][0];
#pragma unroll
            for (int k = 1; k < SHADE_RUN; ++k) if (leader == k) leader_word = meta[g][k];
            auto span_of = [&](unsigned int word) {
                const int sector = (int)((word >> META_SECTOR_SHIFT) & META_SECTOR_MASK) - 1;
                const bool is_floor = (word & META_FLOOR) != 0;
                const unsigned int pair = sector < tb.sector_cached ? sector_level_lds[sector] : dm.sector_level[sector];
                return plane_span(tb, c, lt, yslope, is_floor ? (pair & 0xFFFF) : (pair >> 16), sector, is_floor, x0, y);
            };
            const PlaneSpan shared = span_of(leader_word);
#pragma unroll
            for (int k = 0; k < SHADE_RUN; ++k) {
                if (!(shades[g] & (1u << k))) continue;
                if (((meta[g][k] ^ leader_word) & PLANE_KEY) == 0) {
                    colormap_row[g][k] = shared.colormap_row;
                    texel[g][k] = m->tex_atlas[plane_span_texel(shared, k)];
                } else {   // another plane starts inside the run
                    const PlaneSpan own = span_of(meta[g][k]);
                    colormap_row[g][k] = own.colormap_row;
                    texel[g][k] = m->tex_atlas[plane_span_texel(own, k)];
                }
            }
        }
#pragma unroll
        for (int g = 0; g < SHADE_GROUP; ++g) {
            if (first_pixel[g] < 0) continue;
            const int y = first_pixel[g] / SW, x0 = first_pixel[g] - y * SW;
            unsigned int colours = 0, written = 0;   // bit k of `written`: this kernel decides pixel k
#pragma unroll
            for (int k = 0; k < SHADE_RUN; ++k) {
                const unsigned int word = meta[g][k];
                const int ps = (int)((word >> META_SECTOR_SHIFT) & META_SECTOR_MASK) - 1;
                unsigned int colour = 0; bool writes = false;
                if (word & META_FILLED) {   // a wall tier's pixel, unless a masked texture went over it
                    colour = (word >> META_SECTOR_SHIFT) & 0xFFu; writes = !(word & META_MASKED);
                } else if (ps >= 0) {
                    // (neither tier nor plane: the flat pass's picture shows there, unless a masked texture covers it;
                    // flat_shade_kernel paints the pixel once that pass has run)
                    const bool is_floor = (word & META_FLOOR) != 0;
                    if (shades[g] & (1u << k)) { colour = colormap_lds[colormap_row[g][k] * 256 + texel[g][k]]; writes = true; }
                    else if (!(word & META_MASKED)) { colour = flat_pixel(tb, colormap_lds, c, ps, is_floor, x0 + k, y); writes = true; }
                    if (DEPTH && !(word & META_MASKED)) {   // exact plane depth (engine.py:13406-13416)
                        const float flat_center_px = (103.0f + c.pitch_offset) + 0.5f;
                        const float plane_height = is_floor ? (c.view_z - tb.floor_h(ps)) : (tb.ceil_h(ps) - c.view_z);
                        sc.scene_depth[(size_t)local * VH * SW + first_pixel[g] + k] = plane_height * 192.0f / fmaxf(fabsf((float)y - flat_center_px), 0.5f);
                    }
                }
                colours |= colour << (8 * k);
                if (writes) written |= 1u << k;
            }
            unsigned char *out = frame + first_pixel[g];
            if (written == (1u << SHADE_RUN) - 1 && frame_aligned) {
                *reinterpret_cast<unsigned int *>(out) = colours;
            } else {   // some pixel of the run is the flat pass's or a masked texture's: byte by byte
#pragma unroll
                for (int k = 0; k < SHADE_RUN; ++k) if (written & (1u << k)) out[k] = (unsigned char)(colours >> (8 * k));
            }
        }
    }
}

// The listed gap pixels, painted with the flat the flat pass settled on (engine.py:11145-11163); frames that
// draw decals also keep the depth that pass leaves there (engine.py:11140-11166).
__device__ void flat_shade_pixel(const DeviceMap &dm, const Scratch &sc, const LaneCtx &c, int local, int pixel, unsigned char *frame) {
    const gd_map_desc *m = &dm.d;
    Tables tb; tb.m = m; tb.sector = nullptr; tb.tex_bits = nullptr; tb.tex_odd = nullptr; tb.sector_cached = 0; tb.tex_cached = 0;
    const int y = pixel / SW, x = pixel - y * SW;
    const size_t i = (size_t)local * VH * SW + pixel;
    const int s = sc.flat_sector[i];
    const float delta = (float)y - flat_center(c);
    frame[pixel] = flat_pixel(tb, m->colormap, c, s, delta > 0, x, y);
    if (sc.scene_depth) {
        const unsigned char flags = sc.flat_flags[i];
        const float plane_height = delta > 0 ? (c.view_z - tb.floor_h(s)) : (tb.ceil_h(s) - c.view_z);
        const float perpendicular = plane_height * 192.0f / fmaxf(fabsf(delta), 0.5f);
        const float cosine = dm.cosine_correction[x];
        float depth;
        if (flags & (2 | 8)) depth = perpendicular;             // repaired: its visplane's depth
        else if (flags & 1) depth = GD_INF;                    // no sector found along the ray
        else depth = (perpendicular / cosine) * cosine;        // ray distance of the hit, corrected back
        sc.scene_depth[i] = depth;
    }
}

// lane_pick: LANES_ALL, or one half of launch_chunk's split: LANES_PLAIN for the lanes whose billboards were painted first and
// marked the gap pixels they took, LANES_BLENDING for the others, whose billboards come after this.
__global__ void __launch_bounds__(128) flat_shade_kernel(DeviceMap dm, int lane_count, Scratch sc, unsigned char *frame_base, size_t frame_stride, int lane_pick) {
    const int local = blockIdx.x;
    if (local >= lane_count) return;
    if (lane_pick != LANES_ALL && (sc.lane_blends[local] != 0) != (lane_pick == LANES_BLENDING)) return;   // the same in the whole block
    const bool after_billboards = lane_pick == LANES_PLAIN;
    const int listed = sc.flat_list_count[local];
    const LaneCtx &c = sc.ctx[local];
    unsigned char *frame = frame_base + (size_t)local * frame_stride;
    if (listed <= FLAT_LIST_MAX) {
        for (int slot = threadIdx.x; slot < listed; slot += blockDim.x) {
            const int pixel = sc.flat_list[(size_t)local * FLAT_LIST_MAX + slot];
            if (after_billboards && (sc.meta[(size_t)local * VH * SW + pixel] & META_GAP_COVERED)) continue;
            flat_shade_pixel(dm, sc, c, local, pixel, frame);
        }
        return;
    }
    // a lane with more gap pixels than the list holds: every pixel is looked at
    for (int pixel = threadIdx.x; pixel < VH * SW; pixel += blockDim.x) {
        const unsigned int meta = sc.meta[(size_t)local * VH * SW + pixel];
        if (!(meta & (META_FILLED | META_MASKED)) && ((meta >> META_SECTOR_SHIFT) & META_SECTOR_MASK) == 0 && !(after_billboards && (meta & META_GAP_COVERED)))
            flat_shade_pixel(dm, sc, c, local, pixel, frame);
    }
}

// ---------------------------------------------------------------------------------------------
// sprites: engine.py:10534-10557 (blocking raycast) and 14684-14947
// ---------------------------------------------------------------------------------------------
#define SPRITE_ROWS 4   // rows of a sprite column in flight together
// Columns per block.  A block lasts as long as its slowest column, so many small blocks pack the chip better than a few
// wide ones, until the staging each block repeats for itself outweighs that; each lists only the billboards that reach its
// own columns.  Measured on 4096 lanes with 128 billboards each, columns x row parts: 128x1 0.70 ms, 128x2 0.55, 64x2 0.49,
// 64x4 0.51, 32x2 0.59, 32x4 0.45.
#define SPRITE_COLUMNS 32
struct SpriteRec {
    float x, y, depth, light;
    i64 depth_fixed, left, right, hstep, yscale, top_fixed, fraction_base, iscale;
    int id, flags;   // bit0 alive, bit1 fullbright, bits 8..15 style (signed: -1 opaque, -2 translucent, >= 0 additive),
                     // bits 16..23 / 24..31 first / one past the last screen row the patch can reach
};

// A frame some kernel paints into: all of a lane's 320x240 frame in device memory, or the rows a work-group keeps in LDS.
struct GlobalFrame {
    unsigned char *base;     // row 0, column 0 of the lane's frame
    __device__ __forceinline__ unsigned char *at(int y, int x) const { return base + (size_t)y * SW + x; }
};

// The billboards of one lane, worked out once per work-group (engine.py:14684-14760): `sp[a]` for every slot, and in
// `on_screen` the slots that can reach columns [x_first, x_end) at all (alive, in front, some column between left and
// right): the per-column loops only walk these.  Their order in the list is irrelevant, ties go by slot number.
__device__ __forceinline__ void stage_sprites(const DeviceMap &dm, const gd_lanes_desc &lanes, int n, const LaneCtx &L, int x_first, int x_end,
                                              int row_first, int row_end, SpriteRec *sp, unsigned short *on_screen, int *on_screen_count) {
    const gd_map_desc *m = &dm.d;
    const int A = lanes.sprite_slots;
    for (int a = threadIdx.x; a < A; a += blockDim.x) {
        SpriteRec s;
        size_t k = (size_t)n * A + a;
        s.x = lanes.sprite_x[k]; s.y = lanes.sprite_y[k];
        float z = lanes.sprite_z[k];
        s.depth = lanes.sprite_depth[k]; s.id = lanes.sprite_id[k];
        const bool known_patch = s.id >= 0 && s.id < m->sprite_count;   // an unknown patch id is never drawn
        if (!known_patch) s.id = 0;
        s.flags = ((lanes.sprite_alive[k] && known_patch) ? 1 : 0) | ((lanes.sprite_fullbright && lanes.sprite_fullbright[k]) ? 2 : 0);
        s.flags |= ((lanes.sprite_style ? (int)lanes.sprite_style[k] : -1) & 0xFF) << 8;
        i64 ax = round_to_i64(s.x * 65536.0f), ay = round_to_i64(s.y * 65536.0f);
        i64 rx = ax - L.view_x_fixed, ry = ay - L.view_y_fixed;
        s.depth_fixed = (rx * L.vcos + ry * L.vsin) >> 20;
        i64 side_fixed = (rx * L.vsin - ry * L.vcos) >> 16;
        i64 xscale = tdiv(FOCAL_X_FIXED << 12, max64(s.depth_fixed, SPRITE_MIN_DEPTH_FIXED));
        i64 left_fixed = side_fixed - (i64)m->spr_left[s.id] * FIXED_UNIT;
        s.left = SW / 2 + (mul64(left_fixed, xscale) >> 32);
        i64 right_fixed = left_fixed + (i64)m->spr_w[s.id] * FIXED_UNIT;
        s.right = SW / 2 + (mul64(right_fixed, xscale) >> 32);
        s.hstep = tdiv((i64)m->spr_w[s.id] << 16, max64(s.right - s.left, 1));
        s.yscale = tdiv(FOCAL_Y_FIXED << 12, max64(s.depth_fixed, SPRITE_MIN_DEPTH_FIXED));
        const i64 texmid = (i64)m->spr_top[s.id] * FIXED_UNIT - round_to_i64((L.view_z - z) * 65536.0f);
        s.top_fixed = L.center_fixed - (mul64(texmid, s.yscale) >> 16);
        s.iscale = tdiv(UINT32_MASK, max64(s.yscale, 1));
        // Screen row y shows source row (fraction_base + y * iscale) >> 16 (engine.py:14830-14846).  The rows whose source
        // row can fall inside the patch: a bracket from two divisions, a row too wide on either side; the exact test
        // stays per row.
        s.fraction_base = texmid - (mul64(L.center_fixed - FIXED_UNIT, s.iscale) >> 16);
        int y_lo = 0, y_hi = VH;
        if (s.iscale > 0) {
            y_lo = (int)clampi(tdiv(-s.fraction_base, s.iscale) - 1, 0, VH);
            y_hi = (int)clampi(tdiv(((i64)m->spr_h[s.id] << 16) - s.fraction_base, s.iscale) + 2, 0, VH);
        }
        s.flags |= (int)(((unsigned)y_lo << 16) | ((unsigned)y_hi << 24));
        const bool reaches = (s.flags & 1) && (s.depth > 0) && (s.right > x_first) && (s.left < x_end) && (s.right > s.left) &&
                             y_hi > row_first && y_lo < row_end;
        s.light = reaches ? m->sector_lights[sector_at(m, s.x, s.y)] : 0.0f;
        sp[a] = s;
        if (reaches) on_screen[atomicAdd(on_screen_count, 1)] = (unsigned short)a;
    }
}

// The billboards that can show in column x at all (alive, in front, horizontally covering it and not hidden by the
// column's blocking linedef), as a bit set over `on_screen` (sprite_slots <= 512): the painter's loop runs once per
// drawn billboard and would otherwise test every slot each time.  engine.py:10534-10557, 14762-14800
struct SpriteCover { u64 bits[8]; };
__device__ __forceinline__ SpriteCover sprite_cover(const DeviceMap &dm, const Scratch &sc, int local, const SpriteRec *sp,
                                                    const unsigned short *on_screen, int listed, int x) {
    const gd_map_desc *m = &dm.d;
    const WallRec *recs = sc.rec + (size_t)local * m->wall_count;
    // nearest blocking linedef of this column (engine.py:10534-10557), gathered by wall_setup
    const u64 hit = sc.block_hit[(size_t)local * SW + x];
    float best = hit == ~0ULL ? GD_INF : __uint_as_float((unsigned)(hit >> 32));
    int slot = finitef(best) ? (int)(hit & 0xFFFFFFFFu) : 0;
    float wall_distance = fminf(fmaxf(best, 1.0f), 4096.0f);
    int bw = m->blocking_count ? m->blocking_walls[slot] : 0;
    const WallRec &bg = recs[bw];
    i64 bnear = min64(bg.dl, bg.dr), bfar = max64(bg.dl, bg.dr);
    const float4 bl = *reinterpret_cast<const float4 *>(m->walls + 4 * bw);
    float bdx = bl.z - bl.x, bdy = bl.w - bl.y;
    bool owns = (x >= bg.sl) && (x < bg.sr);
    SpriteCover cover;
#pragma unroll
    for (int word = 0; word < 8; ++word) {
        cover.bits[word] = 0;
        if (word * 64 >= listed) continue;     // the same in every thread
        u64 bits = 0;
        const int end = listed - word * 64 < 64 ? listed - word * 64 : 64;
        for (int b = 0; b < end; ++b) {
            const SpriteRec &s = sp[on_screen[word * 64 + b]];
            if (!((x >= s.left) && (x < s.right))) continue;
            bool ray_visible = s.depth < wall_distance;
            if (!ray_visible) {
                float bside = bdx * (s.y - bl.y) - bdy * (s.x - bl.x);
                bool behind = (bnear > s.depth_fixed) || ((bfar > s.depth_fixed) && (bside <= 0));
                ray_visible = !owns || behind;
            }
            if (ray_visible) bits |= 1ULL << b;
        }
        cover.bits[word] = bits;
    }
    return cover;
}

// Every billboard of `cover` in column x, rows [row_first, row_end), far -> near (engine.py:14762-14947).
template <typename Frame>
__device__ __forceinline__ void sprite_paint(const DeviceMap &dm, const gd_lanes_desc &lanes, const Scratch &sc, int local, int n, const LaneCtx &L,
                                             const SpriteRec *sp, const unsigned short *on_screen, const SpriteCover &cover, int x, int row_first,
                                             int row_end, const Frame &frame, bool mark_gaps = false) {
    const gd_map_desc *m = &dm.d;
    const int A = lanes.sprite_slots;
    const WallRec *recs = sc.rec + (size_t)local * m->wall_count;
    unsigned int *meta = sc.meta + (size_t)local * VH * SW;
    int clip_wall = -1; i64 clip_near = 0, clip_far = 0; float4 clip_line = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
    // painter's order far -> near: repeatedly take the farthest candidate nearer than the last one
    float last_depth = GD_INF; int last_slot = A;
    for (;;) {
        float pick_depth = -GD_INF; int pick = -1;
#pragma unroll
        for (int word = 0; word < 8; ++word) {
            for (u64 bits = cover.bits[word]; bits; bits &= bits - 1) {
                const int a = on_screen[word * 64 + __ffsll((long long)bits) - 1];
                const float depth = sp[a].depth;
                // strictly before (last_depth, last_slot) in (depth, slot) order
                if (!(depth < last_depth || (depth == last_depth && a < last_slot))) continue;
                if (depth > pick_depth || (depth == pick_depth && a > pick)) { pick_depth = depth; pick = a; }
            }
        }
        if (pick < 0) break;
        last_depth = pick_depth; last_slot = pick;
        const SpriteRec &s = sp[pick];
        int width = m->spr_w[s.id], height = m->spr_h[s.id];
        i64 su = mul64((i64)x - s.left, s.hstep) >> 16;
        if (!(su >= 0 && su < width)) continue;
        const int style = (int)(signed char)(s.flags >> 8);
        float light = s.light + (float)(L.flash_light * 16);
        if (s.flags & 2) light = 255.0f;
        float base_shade = 61.0f - light / 4.0f;
        // engine.py:10583 divides a Python number by a tensor, which Torch evaluates as reciprocal(distance) * 1280
        // (Tensor.__rtruediv__): two roundings, not one division
        float visibility = fminf((1.0f / fmaxf(s.depth, 1.0f)) * 1280.0f, 24.0f);
        i64 shade = clampi((i64)floorf(base_shade - visibility), 0, 31);
        const i64 fraction_base = s.fraction_base;
        const int y_lo = max((int)((unsigned)s.flags >> 16) & 255, row_first), y_hi = min((int)((unsigned)s.flags >> 24), row_end);
        // SPRITE_ROWS rows per step, each stage's loads issued together so that their latencies overlap
        for (int yb = y_lo; yb < y_hi; yb += SPRITE_ROWS) {
            i64 sv[SPRITE_ROWS]; bool live[SPRITE_ROWS]; unsigned int row_meta[SPRITE_ROWS];
#pragma unroll
            for (int j = 0; j < SPRITE_ROWS; ++j) {
                const int y = yb + j;
                sv[j] = (fraction_base + mul64((i64)y, s.iscale)) >> 16;
                live[j] = y < y_hi && sv[j] >= 0 && sv[j] < height;
                const size_t i = (size_t)(y < VH ? y : VH - 1) * SW + x;
                row_meta[j] = meta[i];
            }
            // the patch texels do not wait for the clip test: asked for now, they arrive with the meta words
            unsigned char opaque[SPRITE_ROWS], post_top[SPRITE_ROWS], texel[SPRITE_ROWS];
#pragma unroll
            for (int j = 0; j < SPRITE_ROWS; ++j) {
                opaque[j] = 0; post_top[j] = 0; texel[j] = 0;
                if (!live[j]) continue;
                const size_t t = ((size_t)s.id * m->spr_max_h + sv[j]) * m->spr_max_w + su;
                opaque[j] = m->spr_opaque[t]; post_top[j] = m->spr_post_top[t]; texel[j] = m->spr_atlas[t];
            }
#pragma unroll
            for (int j = 0; j < SPRITE_ROWS; ++j) {
                if (!live[j]) continue;
                const int cw = (int)(row_meta[j] & META_WALL_MASK) - 1;
                bool visible;
                if (cw >= 0) {
                    // runs of rows share their clip linedef: its depths and line are kept from row to row
                    if (cw != clip_wall) {
                        const WallRec &cg = recs[cw];
                        clip_near = min64(cg.dl, cg.dr); clip_far = max64(cg.dl, cg.dr);
                        clip_line = *reinterpret_cast<const float4 *>(m->walls + 4 * cw);
                        clip_wall = cw;
                    }
                    float side = (clip_line.z - clip_line.x) * (s.y - clip_line.y) - (clip_line.w - clip_line.y) * (s.x - clip_line.x);
                    visible = (clip_near > s.depth_fixed) || ((clip_far > s.depth_fixed) && (side <= 0));
                } else {
                    visible = s.depth < GD_INF;   // no clip linedef: the clip depth is infinite
                    // No clip recorded, but a plane of the wall pass shows here: where the flat ray did not
                    // resolve, the plane's own depth clips sprites (engine.py:13417-13422).  Only a sprite
                    // standing behind the plane needs to know.
                    const int plane = (int)((row_meta[j] >> META_SECTOR_SHIFT) & META_SECTOR_MASK) - 1;
                    if (visible && plane >= 0 && !(row_meta[j] & META_FILLED)) {
                        const int y = yb + j;
                        const bool plane_floor = (row_meta[j] & META_FLOOR) != 0;
                        const float plane_height = plane_floor ? (L.view_z - m->sector_heights[2 * plane]) : (m->sector_heights[2 * plane + 1] - L.view_z);
                        const float plane_depth = plane_height * 192.0f / fmaxf(fabsf((float)y - ((103.0f + L.pitch_offset) + 0.5f)), 0.5f);
                        if (!(s.depth < plane_depth))
                            visible = flat_ray_resolves(dm, L, lanes.ray_cos[(size_t)n * SW + x], lanes.ray_sin[(size_t)n * SW + x],
                                                        dm.cosine_correction[x], y, plane);
                    }
                }
                live[j] = visible;
            }
#pragma unroll
            for (int j = 0; j < SPRITE_ROWS; ++j) {
                if (!live[j] || !opaque[j]) continue;
                const int y = yb + j;
                i64 post_screen_top = (s.top_fixed + mul64(s.yscale, post_top[j])) >> 16;
                if ((i64)y < post_screen_top) continue;
                // engine.py:14914-14939: opaque, additive table or translucent table over the pixel below
                unsigned char lit = m->colormap[shade * 256 + texel[j]];
                unsigned char *pixel = frame.at(y, x);
                if (style == -2) lit = m->translucent_lut[(size_t)*pixel * 256 + lit];
                else if (style >= 0) lit = m->additive_luts[((size_t)(style > 1 ? 1 : style) * 256 + *pixel) * 256 + lit];
                *pixel = lit;
                // painted ahead of the flat pass's pixels (launch_chunk): a gap pixel says that it is taken
                if (mark_gaps && !(row_meta[j] & (META_FILLED | META_MASKED)) && ((row_meta[j] >> META_SECTOR_SHIFT) & META_SECTOR_MASK) == 0)
                    meta[(size_t)y * SW + x] = row_meta[j] | META_GAP_COVERED;
            }
        }
    }
}

template <typename Frame>
__device__ __forceinline__ void sprite_column(const DeviceMap &dm, const gd_lanes_desc &lanes, const Scratch &sc, int local, int n, const LaneCtx &L,
                                              const SpriteRec *sp, const unsigned short *on_screen, int listed, int x, int row_first, int row_end,
                                              const Frame &frame) {
    const SpriteCover cover = sprite_cover(dm, sc, local, sp, on_screen, listed, x);
    sprite_paint(dm, lanes, sc, local, n, L, sp, on_screen, cover, x, row_first, row_end, frame);
}

// Each column's rows are shared out among SPRITE_ROW_PARTS threads (a column's time is a chain of memory round trips,
// one row batch after another); the first of them finds the column's billboards and leaves the set in LDS for the others.
#define SPRITE_ROW_PARTS 4
static_assert(VH % (SPRITE_ROW_PARTS * SPRITE_ROWS) == 0, "sprite_columns_kernel: row parts hold whole row batches");
__global__ void __launch_bounds__(SPRITE_COLUMNS * SPRITE_ROW_PARTS) __attribute__((amdgpu_waves_per_eu(4, 4))) sprite_columns_kernel(DeviceMap dm, gd_lanes_desc lanes, int lane_base, int lane_count, Scratch sc,
                                                            unsigned char *frame_base, size_t frame_stride, int lane_pick) {
    extern __shared__ unsigned char shared_raw[];
    SpriteRec *sp = reinterpret_cast<SpriteRec *>(shared_raw);
    const int local = blockIdx.y;
    if (local >= lane_count) return;
    // lane_pick: LANES_ALL, or one half of launch_chunk's split: LANES_PLAIN (lanes whose billboards all simply cover what is
    // under them: painted early, marking the gap pixels they take) or LANES_BLENDING (the others, after the flat pass)
    if (lane_pick != LANES_ALL && (sc.lane_blends[local] != 0) != (lane_pick == LANES_BLENDING)) return;   // the same in the whole block
    const bool mark_gaps = lane_pick == LANES_PLAIN;
    const int n = lane_base + local;
    const int A = lanes.sprite_slots;
    const int x_first = blockIdx.x * SPRITE_COLUMNS, x_end = x_first + SPRITE_COLUMNS < SW ? x_first + SPRITE_COLUMNS : SW;
    unsigned short *on_screen = reinterpret_cast<unsigned short *>(sp + A);
    __shared__ int on_screen_count;
    if (threadIdx.x == 0) on_screen_count = 0;
    __syncthreads();
    const LaneCtx L = sc.ctx[local];
    stage_sprites(dm, lanes, n, L, x_first, x_end, 0, VH, sp, on_screen, &on_screen_count);
    __syncthreads();
    const int column = threadIdx.x % SPRITE_COLUMNS, part = threadIdx.x / SPRITE_COLUMNS;
    const int x = x_first + column;
    const int listed = on_screen_count;
    if (listed == 0) return;                       // the same in the whole block
    __shared__ u64 cover_bits[8][SPRITE_COLUMNS];
    SpriteCover cover;
    if (part == 0 && x < x_end) {
        cover = sprite_cover(dm, sc, local, sp, on_screen, listed, x);
#pragma unroll
        for (int word = 0; word < 8; ++word) if (word * 64 < listed) cover_bits[word][column] = cover.bits[word];
    }
    __syncthreads();
    if (x >= x_end) return;
#pragma unroll
    for (int word = 0; word < 8; ++word) cover.bits[word] = word * 64 < listed ? cover_bits[word][column] : 0;
    GlobalFrame frame; frame.base = frame_base + (size_t)local * frame_stride;
    sprite_paint(dm, lanes, sc, local, n, L, sp, on_screen, cover, x, part * (VH / SPRITE_ROW_PARTS), (part + 1) * (VH / SPRITE_ROW_PARTS), frame, mark_gaps);
}

// ---------------------------------------------------------------------------------------------
// wall decals: engine.py:13747-13991, drawn after the walls and before the sprites
// ---------------------------------------------------------------------------------------------
// One thread per screen column; a lane's decals are painted oldest first, each only where the scene
// depth is the decal's own ray distance (which ties it to the wall tier it sits on).
__global__ void __launch_bounds__(SW) decal_kernel(DeviceMap dm, Overlays ov, gd_lanes_desc lanes, int lane_base, int lane_count, Scratch sc,
                                                   unsigned char *frame_base, size_t frame_stride) {
    const gd_map_desc *m = &dm.d;
    const gd_overlay_desc &o = ov.d;
    const int local = blockIdx.x;
    if (local >= lane_count) return;
    const int n = lane_base + local;
    const int x = threadIdx.x;
    const LaneCtx &L = sc.ctx[local];
    const int D = lanes.decal_slots;
    const int width = o.decal_max_w;
    const float center = 104.0f + L.pitch_offset;
    unsigned char *frame = frame_base + (size_t)local * frame_stride;
    const float *scene_depth = sc.scene_depth + (size_t)local * VH * SW;
    float rx, ry; ray_direction(L, x, &rx, &ry);
    for (int k = 0; k < D; ++k) {
        const int *state = lanes.decal_state + ((size_t)n * D + k) * 3;
        const float *geom = lanes.decal_geom + ((size_t)n * D + k) * 4;
        if (!state[2]) continue;
        const int wall_index = (int)clampi(state[0], 0, m->wall_count - 1);
        const int style = state[1];
        const int variant = style % 5;
        const bool flip_x = (style / 5) % 2, flip_y = (style / 10) % 2;
        const int side = style / 20;
        const float along_wall = geom[0], impact_z = geom[1], tangent_x = geom[2], tangent_y = geom[3];
        const float4 wl = *reinterpret_cast<const float4 *>(m->walls + 4 * wall_index);
        const float wvx = wl.z - wl.x, wvy = wl.w - wl.y;
        const float viewer_cross = wvx * (L.y - wl.y) - wvy * (L.x - wl.x);
        if ((viewer_cross > 0 ? 1 : 0) != side) continue;
        const float impact_x = wl.x + along_wall * wvx, impact_y = wl.y + along_wall * wvy;
        const float left_offset = (float)o.decal_left[variant];
        const float back = left_offset * 0.5f, forth = ((float)width - left_offset) * 0.5f;
        const float left_x = impact_x - tangent_x * back, left_y = impact_y - tangent_y * back;
        const float right_x = impact_x + tangent_x * forth, right_y = impact_y + tangent_y * forth;
        const float seg_x = right_x - left_x, seg_y = right_y - left_y;
        // FWallCoords::Init on the two fixed-point endpoints (engine.py:13836-13887)
        const i64 lx = round_to_i64(left_x * 65536.0f) - L.view_x_fixed, ly = round_to_i64(left_y * 65536.0f) - L.view_y_fixed;
        const i64 qx = round_to_i64(right_x * 65536.0f) - L.view_x_fixed, qy = round_to_i64(right_y * 65536.0f) - L.view_y_fixed;
        const i64 tx1 = (lx * L.vsin - ly * L.vcos) >> 20, ty1 = (lx * L.vcos + ly * L.vsin) >> 20;
        const i64 tx2 = (qx * L.vsin - qy * L.vcos) >> 20, ty2 = (qx * L.vcos + qy * L.vsin) >> 20;
        const i64 center_fixed = 160 * FIXED_UNIT;
        const i64 projected_left = ((center_fixed + tdiv(tx1 * center_fixed, ty1 == 0 ? 1 : ty1)) >> 16) + (tx1 >= 0);
        const i64 projected_right = ((center_fixed + tdiv(tx2 * center_fixed, ty2 == 0 ? 1 : ty2)) >> 16) + (tx2 >= 0);
        const i64 left_den = tx1 - tx2 - ty2 + ty1, right_den = ty2 - ty1 - tx2 + tx1;
        const bool left_inside = (tx1 >= -ty1) && (tx1 <= ty1) && (ty1 != 0);
        const bool right_inside = (tx2 <= ty2) && (tx2 >= -ty2) && (ty2 != 0);
        const bool left_clipped = (tx1 < -ty1) && (tx2 >= -ty2) && (left_den != 0);
        const bool right_clipped = (tx2 > ty2) && (tx1 <= ty1) && (right_den != 0);
        const i64 screen_left = left_inside ? clampi(projected_left, 0, SW) : 0;
        const i64 screen_right = right_inside ? clampi(projected_right, 0, SW) : SW;
        if (!((left_inside || left_clipped) && (right_inside || right_clipped) && (screen_right > screen_left))) continue;
        if (!(x >= screen_left && x < screen_right)) continue;
        const float off_x = left_x - L.x, off_y = left_y - L.y;
        const float den = rx * seg_y - ry * seg_x;
        if (!(fabsf(den) >= 1e-6f)) continue;
        const float distance = (off_x * seg_y - off_y * seg_x) / den;
        const float decal_along = (off_x * ry - off_y * rx) / den;
        if (!(distance > 0)) continue;
        i64 tu = clampi((i64)floorf(decal_along * (float)width), 0, width - 1);
        if (flip_x) tu = width - 1 - tu;
        const float safe_distance = fmaxf(distance, 1e-6f);
        // engine.py:13909 divides a Python number by a tensor: reciprocal(distance) * 96 in Torch (Tensor.__rtruediv__)
        const float vertical_scale = (1.0f / safe_distance) * 96.0f;
        const float top = center - ((impact_z + (float)o.decal_top[variant] * 0.5f) - L.view_z) * 192.0f / safe_distance;
        int sector = m->wall_sectors[2 * wall_index + (side > 1 ? 1 : side)];
        if (sector < 0) sector = 0;
        const bool horizontal = fabsf(wvy) < 1e-6f, vertical = fabsf(wvx) < 1e-6f;
        float light = m->sector_lights[sector] + (vertical ? 16.0f : (horizontal ? -16.0f : 0.0f));
        light = light + (float)(L.flash_light * 16);
        const i64 depth_fixed = round_to_i64(safe_distance * 4096.0f);
        const i64 shade = wall_shade(light, tdiv(WALL_VISIBILITY_FIXED << 12, max64(depth_fixed, 1)));
        const int height = o.decal_h[variant];
        // rows whose source row floor((y - top) / vertical_scale) can fall inside the patch, a row wider
        // on either side; the exact test stays per row
        int y_lo = (int)fminf(fmaxf(floorf(top) - 1.0f, 0.0f), (float)VH);
        int y_hi = (int)fminf(fmaxf(ceilf(top + (float)height * vertical_scale) + 2.0f, 0.0f), (float)VH);
        for (int y = y_lo; y < y_hi; ++y) {
            i64 tv = (i64)floorf(((float)y - top) / vertical_scale);
            if (!(tv >= 0 && tv < height)) continue;
            if (flip_y) tv = height - 1 - tv;
            const size_t i = (size_t)y * SW + x;
            if (!(fabsf(scene_depth[i] - distance) <= 1e-3f)) continue;
            const unsigned char source = o.decal_atlas[((size_t)variant * o.decal_max_h + tv) * o.decal_max_w + tu];
            if (source == 0) continue;
            const unsigned char opacity = o.decal_opacity_lut[shade * 256 + source];
            frame[i] = o.decal_black_lut[(size_t)opacity * 256 + frame[i]];
        }
    }
}

// ---------------------------------------------------------------------------------------------
// overlay layers drawn after the sprites
// ---------------------------------------------------------------------------------------------
// One psprite patch over one pixel (engine.py:14997-15049, _triton_kernels.py:2611-2634).
__device__ __forceinline__ bool psprite_texel(const gd_overlay_desc &o, i64 patch, i64 horizontal_fixed, i64 vertical_fixed, int px, int py, unsigned char *value) {
    if (patch < 0 || patch >= o.weapon_patch_count) return false;
    const i64 width = o.weapon_w[patch], height = o.weapon_h[patch];
    const i64 screen_left = (horizontal_fixed - (i64)o.weapon_left[patch] * FIXED_UNIT) >> 16;
    const i64 source_x = (i64)px - screen_left;
    // BASEYCENTER 100, weapon top 32 + 0x6000/65536, reciprocal of the 240/200 vertical scale
    const i64 weapon_top_fixed = 32 * FIXED_UNIT + 0x6000;
    const i64 texture_mid = 100 * FIXED_UNIT - weapon_top_fixed - vertical_fixed + (i64)o.weapon_top[patch] * FIXED_UNIT;
    const i64 y_scale = ((i64)GD_SCREEN_HEIGHT * FIXED_UNIT) / 200;
    const i64 y_iscale = UINT32_MASK / y_scale;
    const i64 source_y = (texture_mid + ((i64)py - (VH / 2 - 1)) * y_iscale) >> 16;
    if (source_x < 0 || source_x >= width || source_y < 0 || source_y >= height) return false;
    if (source_x >= o.weapon_max_w || source_y >= o.weapon_max_h) return false;   // sizes beyond the atlas: malformed patch
    const size_t t = ((size_t)patch * o.weapon_max_h + (size_t)source_y) * o.weapon_max_w + (size_t)source_x;
    if (!o.weapon_opaque[t]) return false;
    *value = o.weapon_atlas[t];
    return true;
}

// _native_render_weapon (engine.py:15051-15110): the weapon patch, then its muzzle flash on top
__global__ void __launch_bounds__(256) weapon_overlay_kernel(Overlays ov, const int64_t *weapon_state, int lane_base, int lane_count,
                                                             unsigned char *frame_base, size_t frame_stride) {
    const int local = blockIdx.y;
    const int pixel = blockIdx.x * blockDim.x + threadIdx.x;
    if (local >= lane_count || pixel >= VH * SW) return;
    const int64_t *state = weapon_state + (size_t)(lane_base + local) * 5;
    if (state[4] == 0) return;                    // player dead: no psprite
    const int py = pixel / SW, px = pixel - py * SW;
    unsigned char value;
    bool drawn = psprite_texel(ov.d, state[0], state[2], state[3], px, py, &value);
    unsigned char flash;
    if (state[1] >= 0 && psprite_texel(ov.d, state[1], state[2], state[3], px, py, &flash)) { value = flash; drawn = true; }
    if (drawn) frame_base[(size_t)local * frame_stride + pixel] = value;
}

// _native_render_hud (engine.py:15153-15267): the status bar is a short list of patches drawn in
// order, later ones over earlier ones.  One block per lane: thread 0 writes the list, then every
// thread resolves its pixels by walking the list backwards to the first opaque texel.
#define HUD_ROWS (GD_SCREEN_HEIGHT - VH)
#define HUD_LIST_MAX 48
struct HudEntry { int patch, x, y; };

// _native_draw_hud_number (engine.py:15186-15207); note that the glyph offsets are applied here and
// again by the patch draw, as in the reference
__device__ void hud_number(const gd_overlay_desc &o, HudEntry *list, int *count, int value, int right, int y, bool small) {
    value = value < -99 ? -99 : (value > 999 ? 999 : value);
    const int digit_width = small ? 4 : 14, base = small ? 28 : 2;
    const bool negative = value < 0;
    int magnitude = negative ? -value : value;
    int digits[3], length = 0;
    do { digits[length++] = magnitude % 10; magnitude /= 10; } while (magnitude > 0);
    int x = right - (length + (negative ? 1 : 0)) * digit_width;
    if (negative) x += digit_width;               // the sign takes a cell and draws nothing
    for (int k = length - 1; k >= 0; --k) {
        const int patch = base + digits[k];
        if (patch < o.hud_patch_count && *count < HUD_LIST_MAX) {
            HudEntry e; e.patch = patch; e.x = x - o.hud_left[patch]; e.y = y - o.hud_top[patch];
            list[(*count)++] = e;
        }
        x += digit_width;
    }
}

// The status bar's patches in drawing order (engine.py:15232-15267), written by one thread.
__device__ int build_hud_list(const gd_overlay_desc &o, const int *state, HudEntry *list) {
    int count = 0;
    auto patch_at = [&](int patch, int x, int y) {
        if (patch >= 0 && patch < o.hud_patch_count && count < HUD_LIST_MAX) { HudEntry e; e.patch = patch; e.x = x; e.y = y; list[count++] = e; }
    };
    patch_at(0, 0, 0);
    patch_at(1, 104, 0);
    hud_number(o, list, &count, state[0], 44, 3, false);
    hud_number(o, list, &count, state[1], 90, 3, false);
    patch_at(12, 90, 3);
    hud_number(o, list, &count, state[2], 221, 3, false);
    patch_at(12, 221, 3);
    patch_at(state[3], 143, 0);
    const int arms_x[6] = {111, 123, 135, 111, 123, 135}, arms_y[6] = {4, 4, 4, 14, 14, 14};
    for (int k = 0; k < 6; ++k) {
        const bool owned = k < 5 && ((state[4] >> k) & 1);
        patch_at(owned ? 30 + k : 38 + k, arms_x[k], arms_y[k]);
    }
    const int maximum[4] = {200, 50, 50, 300};
    for (int row = 0; row < 4; ++row) {
        hud_number(o, list, &count, state[5 + row], 288, 5 + row * 6, true);
        hud_number(o, list, &count, maximum[row], 314, 5 + row * 6, true);
    }
    return count;
}

// One pixel of the status bar (cx, cy relative to row 208): the last listed patch with an opaque texel there.
__device__ __forceinline__ unsigned char hud_pixel(const gd_overlay_desc &o, const HudEntry *list, int count, int cx, int cy) {
    for (int k = count - 1; k >= 0; --k) {
        const HudEntry e = list[k];
        // _native_draw_hud_patch (engine.py:15153-15184): position minus the patch's own offsets, clipped
        const int sx = cx - (e.x - o.hud_left[e.patch]), sy = cy - (e.y - o.hud_top[e.patch]);
        if (sx < 0 || sy < 0 || sx >= o.hud_w[e.patch] || sy >= o.hud_h[e.patch] || sx >= o.hud_max_w || sy >= o.hud_max_h) continue;
        const size_t t = ((size_t)e.patch * o.hud_max_h + sy) * o.hud_max_w + sx;
        if (o.hud_opaque[t]) return o.hud_atlas[t];
    }
    return 0;
}

__global__ void __launch_bounds__(256) hud_kernel(Overlays ov, const int *hud_state, int lane_base, int lane_count,
                                                  unsigned char *frame_base, size_t frame_stride) {
    const gd_overlay_desc &o = ov.d;
    __shared__ HudEntry list[HUD_LIST_MAX];
    __shared__ int list_count;
    const int local = blockIdx.x;
    if (local >= lane_count) return;
    if (threadIdx.x == 0) list_count = build_hud_list(o, hud_state + (size_t)(lane_base + local) * 9, list);
    __syncthreads();
    unsigned char *bar = frame_base + (size_t)local * frame_stride + (size_t)VH * SW;
    for (int p = threadIdx.x; p < HUD_ROWS * SW; p += blockDim.x) bar[p] = hud_pixel(o, list, list_count, p % SW, p / SW);
}

// ---------------------------------------------------------------------------------------------
// observation: _triton_kernels.py:120-177 + engine.py:9545-9548 / 2443-2450
// ---------------------------------------------------------------------------------------------
// One PLAYPAL channel after the pickup (gold) and damage (red) screen blends, evaluated in float32 one
// operation at a time and truncated to a byte (engine.py:15385-15397).
__device__ __forceinline__ unsigned char blended_channel(unsigned char value, int channel, float bonus, float flash) {
    const float gold = channel == 0 ? 215.0f : (channel == 1 ? 186.0f : 69.0f);
    const float red = channel == 0 ? 255.0f : 0.0f;
    float v = (float)value * (1.0f - bonus) + gold * bonus;
    v = v * (1.0f - flash) + red * flash;
    return (unsigned char)fminf(fmaxf(v, 0.0f), 255.0f);
}

// `blend` points at the first lane's (bonus, damage) alphas, or is null for plain PLAYPAL colours.
__device__ __forceinline__ void stage_palette(unsigned char *pal, const unsigned char *playpal, const float *blend, int lane) {
    if (blend) {
        const float bonus = blend[2 * lane], flash = blend[2 * lane + 1];
        for (int k = threadIdx.x; k < 768; k += blockDim.x) pal[k] = blended_channel(playpal[k], k % 3, bonus, flash);
    } else {
        for (int k = threadIdx.x; k < 768; k += blockDim.x) pal[k] = playpal[k];
    }
    __syncthreads();
}

// The frame stack of one lane, four pixels (one word per stacked observation) at a time: what the stack holds after
// this call goes to `stack` (when it changes) and to the caller's copy, which is laid out either like the stack
// ([4][84][84]) or with the four stacked values of a pixel next to each other ([84][84][4]).
// `kept` holds the stack's words as they were (unused for a lane that resets).  env.py:678-688, engine.py:15447-15450
__device__ __forceinline__ void store_stack_word(unsigned char *stack_lane, unsigned char *copy_lane, bool copy_hwc, bool aligned, size_t word,
                                                 const unsigned int (&kept)[GD_FRAME_STACK], unsigned int grays, bool resets, int stack_mode) {
    const size_t plane = (size_t)GD_OBS_SIZE * GD_OBS_SIZE;   // bytes per stacked observation
    auto store = [&](unsigned char *p, unsigned int v) {
        if (aligned) *reinterpret_cast<unsigned int *>(p) = v;
        else for (int k = 0; k < 4; ++k) p[k] = (unsigned char)(v >> (8 * k));
    };
    const bool steps = !resets && stack_mode == GD_STACK_STEP;
    unsigned int next[GD_FRAME_STACK];
#pragma unroll
    for (int k = 0; k < GD_FRAME_STACK; ++k) next[k] = resets ? grays : (steps ? (k + 1 < GD_FRAME_STACK ? kept[k + 1] : grays) : kept[k]);
    if (resets || steps) {
#pragma unroll
        for (int k = 0; k < GD_FRAME_STACK; ++k) store(stack_lane + k * plane + word * 4, next[k]);
    }
    if (!copy_lane) return;
    if (!copy_hwc) {
#pragma unroll
        for (int k = 0; k < GD_FRAME_STACK; ++k) store(copy_lane + k * plane + word * 4, next[k]);
        return;
    }
    static_assert(GD_FRAME_STACK == 4, "the interleaved copy packs the four stacked values of a pixel into one word");
#pragma unroll
    for (int j = 0; j < 4; ++j) {   // pixel j of the word
        const unsigned int v = ((next[0] >> (8 * j)) & 255u) | (((next[1] >> (8 * j)) & 255u) << 8) |
                               (((next[2] >> (8 * j)) & 255u) << 16) | (((next[3] >> (8 * j)) & 255u) << 24);
        store(copy_lane + (word * 4 + j) * GD_FRAME_STACK, v);
    }
}

// One block per lane and OBS_BLOCK_ROWS = 7 observation rows, which pool exactly OBS_SOURCE_ROWS = 20 frame rows
// (84 observation rows x 240 / 84 frame rows each).  An observation pixel covers 240/84 frame rows and 320/84 frame
// columns; its weights (y_overlap * x_overlap) // 48 are exactly (y_overlap / 12) * (x_overlap / 4), since row
// overlaps are multiples of 12 and column overlaps multiples of 4 (84 = 12 * 7 = 4 * 21, 240 = 12 * 20, 320 = 4 * 80):
// the weighted sum factors into a pass along the rows and one down the columns, all in integers.  The first pass
// looks every frame pixel's colour up once per observation column it touches (five taps per frame row and
// observation column), the second adds four row sums per observation pixel: 10,752 palette taps per block where a
// pixel-by-pixel pooling takes 11,760, and a tap is a byte load, a palette load and three dot products.
#define OBS_BLOCK_ROWS 7
#define OBS_SOURCE_ROWS (OBS_BLOCK_ROWS * GD_SCREEN_HEIGHT / GD_OBS_SIZE)
static_assert(GD_OBS_SIZE % OBS_BLOCK_ROWS == 0 && OBS_SOURCE_ROWS * GD_OBS_SIZE == OBS_BLOCK_ROWS * GD_SCREEN_HEIGHT, "observe_kernel: seven rows pool twenty");
static_assert((OBS_BLOCK_ROWS * GD_OBS_SIZE) % 4 == 0 && 3 * GD_OBS_SIZE <= 256, "observe_kernel: whole words, three rows of threads");
__global__ void __launch_bounds__(256) observe_kernel(const unsigned char *indexed, size_t lane_stride, int source_rows, const unsigned char *playpal,
                               int lane_count, unsigned char *obs, unsigned char *frames, const unsigned char *reset_mask, int stack_mode,
                               unsigned char *final_frames, bool final_hwc, const float *blend) {
    __shared__ unsigned int pal[256];   // PLAYPAL after the lane's screen blend, one word per colour (red | green << 8 | blue << 16)
    __shared__ unsigned int tile[OBS_SOURCE_ROWS * (SW / 4)];
    __shared__ unsigned int along_rg[OBS_SOURCE_ROWS * GD_OBS_SIZE];      // per frame row and observation column: red | green << 16 summed along the row
    __shared__ unsigned short along_b[OBS_SOURCE_ROWS * GD_OBS_SIZE];     // and blue (each at most 80 * 255)
    __shared__ unsigned int gray_words[OBS_BLOCK_ROWS * GD_OBS_SIZE / 4];
    int n = blockIdx.y;
    if (n >= lane_count) return;                   // the same in the whole block
    const unsigned char *src = indexed + (size_t)n * lane_stride;
    const int first_row = blockIdx.x * OBS_BLOCK_ROWS;
    const int tile_first = blockIdx.x * OBS_SOURCE_ROWS;
    // Everything the block reads from memory is asked for up front (palette entry, tile words, the stack words
    // that the roll keeps), so that the block waits for memory once.
    const size_t F = (size_t)GD_OBS_SIZE * GD_OBS_SIZE / 4;     // words per observation
    const size_t word = (size_t)first_row * GD_OBS_SIZE / 4 + threadIdx.x;
    const bool rolls = threadIdx.x < OBS_BLOCK_ROWS * GD_OBS_SIZE / 4;
    const bool stack_aligned = ((reinterpret_cast<size_t>(frames) | reinterpret_cast<size_t>(final_frames)) & 3) == 0;
    unsigned char *stack_bytes = frames ? frames + ((size_t)n * GD_FRAME_STACK * F + word) * 4 : nullptr;
    auto load_word = [](const unsigned char *p, bool aligned) -> unsigned int {
        if (aligned) return *reinterpret_cast<const unsigned int *>(p);
        return (unsigned)p[0] | ((unsigned)p[1] << 8) | ((unsigned)p[2] << 16) | ((unsigned)p[3] << 24);
    };
    const bool resets = reset_mask && reset_mask[n];
    unsigned int kept[GD_FRAME_STACK];
    for (int k = 0; k < GD_FRAME_STACK; ++k) kept[k] = (rolls && frames && !resets) ? load_word(stack_bytes + k * F * 4, stack_aligned) : 0u;
    {
        const int k = threadIdx.x;   // 256 threads, 256 colours
        unsigned int r = playpal[3 * k], g = playpal[3 * k + 1], b = playpal[3 * k + 2];
        if (blend) {
            const float bonus = blend[2 * n], flash = blend[2 * n + 1];
            r = blended_channel((unsigned char)r, 0, bonus, flash); g = blended_channel((unsigned char)g, 1, bonus, flash); b = blended_channel((unsigned char)b, 2, bonus, flash);
        }
        pal[k] = r | (g << 8) | (b << 16);
    }
    {
        const bool aligned = (reinterpret_cast<size_t>(src) & 3) == 0;
        for (int k = threadIdx.x; k < OBS_SOURCE_ROWS * (SW / 4); k += blockDim.x) {
            const int r = k / (SW / 4), c = k - r * (SW / 4);
            tile[k] = load_word(src + (size_t)min(tile_first + r, source_rows - 1) * SW + 4 * c, aligned);   // rows past the source weigh nothing below
        }
    }
    __syncthreads();
    // three rows of 84 threads: thread (slot, ox) takes observation column ox of every third row
    const int slot = min((int)threadIdx.x / GD_OBS_SIZE, 2), ox = min((int)threadIdx.x - slot * GD_OBS_SIZE, GD_OBS_SIZE - 1);
    const bool works = threadIdx.x < 3 * GD_OBS_SIZE;
    const unsigned char *staged = reinterpret_cast<const unsigned char *>(tile);
    {
        // along the rows: up to five frame columns overlap an observation column, by multiples of 4 out of 84
        const int x_start = ox * 320, x_end = x_start + 320, first_x = x_start / 84;
        unsigned int weight_r[5], weight_g[5], weight_b[5]; int column[5];
#pragma unroll
        for (int sx = 0; sx < 5; ++sx) {
            const int source_x = first_x + sx;
            const int over = min(x_end, (source_x + 1) * 84) - max(x_start, source_x * 84);
            const unsigned int weight = (source_x >= SW || over <= 0) ? 0u : (unsigned)over >> 2;
            // a colour word times a weight in byte 0, 1 or 2 is that channel times the weight (a four-byte dot product)
            weight_r[sx] = weight; weight_g[sx] = weight << 8; weight_b[sx] = weight << 16;
            column[sx] = min(source_x, SW - 1);
        }
        for (int sy = slot; sy < OBS_SOURCE_ROWS && works; sy += 3) {
            unsigned int rs = 0, gs = 0, bs = 0;
            if (tile_first + sy < source_rows) {
                unsigned int colour[5];
#pragma unroll
                for (int sx = 0; sx < 5; ++sx) colour[sx] = pal[staged[sy * SW + column[sx]]];
#pragma unroll
                for (int sx = 0; sx < 5; ++sx) {
                    rs = __builtin_amdgcn_udot4(colour[sx], weight_r[sx], rs, false);
                    gs = __builtin_amdgcn_udot4(colour[sx], weight_g[sx], gs, false);
                    bs = __builtin_amdgcn_udot4(colour[sx], weight_b[sx], bs, false);
                }
            }
            along_rg[sy * GD_OBS_SIZE + ox] = rs | (gs << 16);
            along_b[sy * GD_OBS_SIZE + ox] = (unsigned short)bs;
        }
    }
    __syncthreads();
    // down the columns: up to four frame rows overlap an observation row, by multiples of 12 out of 84
    for (int row_in_block = slot; row_in_block < OBS_BLOCK_ROWS && works; row_in_block += 3) {
        const int y_start = row_in_block * 240, y_end = y_start + 240, first_y = y_start / 84;   // relative to the block's first frame row
        unsigned int rs = 0, gs = 0, bs = 0;
#pragma unroll
        for (int sy = 0; sy < 4; ++sy) {
            const int source_y = first_y + sy;
            const int over = min(y_end, (source_y + 1) * 84) - max(y_start, source_y * 84);
            const unsigned int weight = (source_y >= OBS_SOURCE_ROWS || over <= 0) ? 0u : (unsigned)over / 12u;
            const int at = min(source_y, OBS_SOURCE_ROWS - 1) * GD_OBS_SIZE + ox;
            const unsigned int rg = along_rg[at];
            rs += __umul24(rg & 0xFFFFu, weight); gs += __umul24(rg >> 16, weight); bs += __umul24(along_b[at], weight);
        }
        const unsigned int r = (rs + 800u) / 1600u, g = (gs + 800u) / 1600u, b = (bs + 800u) / 1600u;
        reinterpret_cast<unsigned char *>(gray_words)[row_in_block * GD_OBS_SIZE + ox] = (unsigned char)((r * 77u + g * 150u + b * 29u + 128u) >> 8);
    }
    __syncthreads();
    // The block's pixels are contiguous in the observation; they go out, and the stack is rolled, a word (four
    // pixels) per thread.
    if (!rolls) return;
    const unsigned int grays = gray_words[threadIdx.x];
    if (obs) {
        unsigned char *out = obs + ((size_t)n * F + word) * 4;
        if ((reinterpret_cast<size_t>(obs) & 3) == 0) *reinterpret_cast<unsigned int *>(out) = grays;
        else for (int k = 0; k < 4; ++k) out[k] = (unsigned char)(grays >> (8 * k));
    }
    // a stack is [4][84][84] bytes, so word access only needs the tensors themselves word aligned
    if (frames) store_stack_word(frames + (size_t)n * GD_FRAME_STACK * F * 4, final_frames ? final_frames + (size_t)n * GD_FRAME_STACK * F * 4 : nullptr,
                                 final_hwc, stack_aligned, word, kept, grays, resets, stack_mode);
}

// engine.py:15381-15384
// A block of 256 pixels never straddles two lanes when lane_pixels is a multiple of 256 (240 x 320 is).
__global__ void expand_rgb_kernel(const unsigned char *indexed, const unsigned char *playpal, size_t pixels, unsigned char *rgb,
                                  const float *blend, size_t lane_pixels) {
    __shared__ unsigned char pal[768];
    stage_palette(pal, playpal, blend, blend ? (int)(((size_t)blockIdx.x * blockDim.x) / lane_pixels) : 0);
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= pixels) return;
    int p = indexed[i] * 3;
    rgb[i * 3] = pal[p]; rgb[i * 3 + 1] = pal[p + 1]; rgb[i * 3 + 2] = pal[p + 2];
}

// ---------------------------------------------------------------------------------------------
// finish: everything after the wall traversal and the flat selection, for one band of one lane's frame at a time,
// with the band held in LDS from the first shaded pixel to the pooled observation: plane and tier pixels
// (engine.py:13372-13405), the flat pass's pixels where nothing else shows (engine.py:11145-11163), billboards
// (engine.py:14762-14947), weapon and status bar (engine.py:15051-15110, 15232-15267), PLAYPAL expansion
// (engine.py:15381-15398), area pooling and the frame stack (_triton_kernels.py:120-177, engine.py:9545-9548).
// The 320x240 frame only goes to device memory when the caller asks for it.
// ---------------------------------------------------------------------------------------------
// A band is 80 frame rows: 28 observation rows pool exactly those (84 observation rows x 240 / 84 source rows each).
#define BAND_ROWS 80
#define BAND_COUNT (GD_SCREEN_HEIGHT / BAND_ROWS)
#define BAND_OBS_ROWS (BAND_ROWS * GD_OBS_SIZE / GD_SCREEN_HEIGHT)
#define BAND_THREADS 512   // sixteen wavefronts a compute unit when two work-groups share it: four per SIMD, none left over
static_assert(BAND_COUNT * BAND_ROWS == GD_SCREEN_HEIGHT && BAND_OBS_ROWS * BAND_COUNT == GD_OBS_SIZE, "bands tile the frame and the observation");
static_assert(BAND_THREADS >= SW && (BAND_OBS_ROWS * GD_OBS_SIZE) % 4 == 0, "band_finish_kernel: thread layout");

struct BandFrame {   // the rows [row0, row0 + BAND_ROWS) of a lane's frame, in LDS
    unsigned char *rows;
    int row0;
    __device__ __forceinline__ unsigned char *at(int y, int x) const { return rows + (y - row0) * SW + x; }
};

struct FinishOut {   // device pointers of the chunk's first lane; null = not wanted
    unsigned char *indexed, *rgb, *obs, *frames, *final_frames;
    const unsigned char *reset_mask;
    const float *blend;
    int stack_mode, source_rows;
    bool final_hwc;
};

__global__ void __launch_bounds__(BAND_THREADS) __attribute__((amdgpu_waves_per_eu(4, 4))) band_finish_kernel(DeviceMap dm, Overlays ov, gd_lanes_desc lanes, int lane_base, int lane_count, Scratch sc, FinishOut out) {
    extern __shared__ unsigned char shared_raw[];                // billboard records, when there are too many to reuse the tables' LDS
    __shared__ unsigned int band_words[BAND_ROWS * SW / 4];
    // the sector table and the colormap serve the shading phase only; the billboard records take their place afterwards
    __shared__ struct { float4 sector[LDS_SECTORS]; unsigned char colormap[32 * 256]; } shading_lds;
    float4 *sector_lds = shading_lds.sector;
    unsigned char *colormap_lds = shading_lds.colormap;
    __shared__ unsigned int sector_level_lds[LDS_SECTORS];
    __shared__ TexLds tex_lds;
    __shared__ i64 level_plane_lds[2 * PLANE_LEVELS * 2];
    __shared__ i64 step_scale_lds[STEP_TABLE];
    __shared__ unsigned int pal[256];                            // PLAYPAL after the lane's screen blend: red | green << 8 | blue << 16
    __shared__ unsigned int gray_words[BAND_OBS_ROWS * GD_OBS_SIZE / 4];
    __shared__ HudEntry hud_list[HUD_LIST_MAX];
    __shared__ int hud_count, on_screen_count;
    const gd_map_desc *m = &dm.d;
    const int band = blockIdx.x, local = blockIdx.y;
    if (local >= lane_count) return;     // uniform over the block
    const int n = lane_base + local;
    const int tid = threadIdx.x;
    const int row0 = band * BAND_ROWS;
    const int view_rows = row0 >= VH ? 0 : (row0 + BAND_ROWS <= VH ? BAND_ROWS : VH - row0);   // the rest are status bar rows
    unsigned char *band_bytes = reinterpret_cast<unsigned char *>(band_words);
    BandFrame frame; frame.rows = band_bytes; frame.row0 = row0;
    Tables tb;
    stage_tables(m, sector_lds, &tex_lds, tb);
    for (int k = tid; k < 32 * 256 / 4; k += BAND_THREADS) reinterpret_cast<unsigned int *>(colormap_lds)[k] = reinterpret_cast<const unsigned int *>(m->colormap)[k];
    const int floors = m->floor_level_count, levels = floors + m->ceil_level_count;
    const bool tabled = dm.sector_level != nullptr;
    const bool levels_staged = levels <= 2 * PLANE_LEVELS;
    if (tabled) {
        for (int s = tid; s < tb.sector_cached; s += BAND_THREADS) sector_level_lds[s] = dm.sector_level[s];
        if (levels_staged) for (int k = tid; k < 2 * levels; k += BAND_THREADS) level_plane_lds[k] = sc.level_plane[(size_t)local * levels * 2 + k];
        if (tid < STEP_TABLE) step_scale_lds[tid] = sc.step_scale[(size_t)local * STEP_TABLE + tid];
    }
    if (tid < 256) {
        unsigned int r = m->playpal[3 * tid], g = m->playpal[3 * tid + 1], b = m->playpal[3 * tid + 2];
        if (out.blend) {
            const float bonus = out.blend[2 * local], flash = out.blend[2 * local + 1];
            r = blended_channel((unsigned char)r, 0, bonus, flash); g = blended_channel((unsigned char)g, 1, bonus, flash); b = blended_channel((unsigned char)b, 2, bonus, flash);
        }
        pal[tid] = r | (g << 8) | (b << 16);
    }
    if (tid == 0) {
        on_screen_count = 0;
        hud_count = (view_rows < BAND_ROWS && lanes.hud_state && ov.d.hud_patch_count > 0) ? build_hud_list(ov.d, lanes.hud_state + (size_t)n * 9, hud_list) : 0;
    }
    __syncthreads();
    const LaneCtx L = sc.ctx[local];
    LaneTables lt; lt.step_scale = step_scale_lds; lt.floors = floors;
    lt.level_plane = levels_staged ? level_plane_lds : sc.level_plane + (size_t)local * levels * 2;
    // --- the status bar rows of this band (engine.py:15232-15267); empty without status bar patches
    for (int p = tid; p < (BAND_ROWS - view_rows) * SW; p += BAND_THREADS)
        band_bytes[view_rows * SW + p] = hud_count > 0 ? hud_pixel(ov.d, hud_list, hud_count, p % SW, row0 + view_rows + p / SW - VH) : (unsigned char)0;
    // --- every view pixel of the band once: a wall tier's palette index, a visplane's flat, a masked mid-texture's texel, or
    // the flat pass's pick.  A wavefront takes a row at a time, its lanes the row's five groups of 64 columns: what depends
    // on the row alone is worked out once per row, and each stage's loads are issued together.
    const size_t lane_pixels = (size_t)local * VH * SW;
    const int wave = tid >> 6, lane_id = tid & 63;
    constexpr int ROW_GROUPS = SW / 64;
    for (int py = wave; py < view_rows; py += BAND_THREADS / 64) {
        const int y = row0 + py;
        const size_t row_at = lane_pixels + (size_t)y * SW;
        const i64 yslope = sc.row_slope[(size_t)local * VH + y];
        unsigned int meta[ROW_GROUPS];
#pragma unroll
        for (int j = 0; j < ROW_GROUPS; ++j) meta[j] = sc.meta[row_at + j * 64 + lane_id];
        int colormap_row[ROW_GROUPS]; unsigned char texel[ROW_GROUPS];
        bool shade[ROW_GROUPS];
#pragma unroll
        for (int j = 0; j < ROW_GROUPS; ++j) {
            const int ps = (int)((meta[j] >> META_SECTOR_SHIFT) & META_SECTOR_MASK) - 1;
            shade[j] = tabled && ps >= 0 && !(meta[j] & (META_FILLED | META_MASKED));
            texel[j] = 0; colormap_row[j] = 0;
            if (!shade[j]) continue;
            const bool is_floor = (meta[j] & META_FLOOR) != 0;
            const unsigned int pair = ps < tb.sector_cached ? sector_level_lds[ps] : dm.sector_level[ps];
            const size_t texel_at = flat_sample_tabled(tb, L, lt, yslope, is_floor ? (pair & 0xFFFF) : (pair >> 16), ps, is_floor, j * 64 + lane_id, y, &colormap_row[j]);
            texel[j] = m->tex_atlas[texel_at];
        }
#pragma unroll
        for (int j = 0; j < ROW_GROUPS; ++j) {
            const int x = j * 64 + lane_id;
            const int ps = (int)((meta[j] >> META_SECTOR_SHIFT) & META_SECTOR_MASK) - 1;
            unsigned char colour;
            if (meta[j] & META_MASKED) colour = (unsigned char)__float_as_uint(sc.clip_depth[row_at + x]);   // left there by masked_midtexture
            else if (meta[j] & META_FILLED) colour = (unsigned char)(meta[j] >> META_SECTOR_SHIFT);
            else if (shade[j]) colour = colormap_lds[colormap_row[j] * 256 + texel[j]];
            else if (ps >= 0) colour = flat_pixel(tb, colormap_lds, L, ps, (meta[j] & META_FLOOR) != 0, x, y);
            else colour = flat_pixel(tb, colormap_lds, L, sc.flat_sector[row_at + x], ((float)y - flat_center(L)) > 0, x, y);   // the flat pass's picture
            band_bytes[py * SW + x] = colour;
        }
    }
    // --- billboards, one thread per screen column
    if (lanes.sprite_slots > 0 && lanes.sprite_x && view_rows > 0) {
        __syncthreads();                  // every shaded pixel is in place, and the shading tables are free
        const bool fits = (size_t)lanes.sprite_slots * (sizeof(SpriteRec) + sizeof(unsigned short)) <= sizeof(shading_lds);
        SpriteRec *sp = reinterpret_cast<SpriteRec *>(fits ? reinterpret_cast<unsigned char *>(&shading_lds) : shared_raw);
        unsigned short *on_screen = reinterpret_cast<unsigned short *>(sp + lanes.sprite_slots);
        stage_sprites(dm, lanes, n, L, 0, SW, row0, row0 + view_rows, sp, on_screen, &on_screen_count);
        __syncthreads();
        if (tid < SW && on_screen_count > 0) sprite_column(dm, lanes, sc, local, n, L, sp, on_screen, on_screen_count, tid, row0, row0 + view_rows, frame);
    }
    __syncthreads();
    // --- the player's weapon and its muzzle flash (engine.py:15051-15110)
    if (lanes.weapon_state && ov.d.weapon_patch_count > 0) {
        const int64_t *state = lanes.weapon_state + (size_t)n * 5;
        if (state[4] != 0) {
            for (int p = tid; p < view_rows * SW; p += BAND_THREADS) {
                const int py = p / SW, px = p - py * SW;
                unsigned char value;
                bool drawn = psprite_texel(ov.d, state[0], state[2], state[3], px, row0 + py, &value);
                unsigned char flash;
                if (state[1] >= 0 && psprite_texel(ov.d, state[1], state[2], state[3], px, row0 + py, &flash)) { value = flash; drawn = true; }
                if (drawn) band_bytes[p] = value;
            }
        }
        __syncthreads();
    }
    // --- what the caller asked for
    if (out.indexed) {
        uint4 *rows = reinterpret_cast<uint4 *>(out.indexed + ((size_t)local * GD_SCREEN_HEIGHT + row0) * SW);
        const bool aligned = (reinterpret_cast<size_t>(out.indexed) & 15) == 0;
        if (aligned) {
            for (int k = tid; k < BAND_ROWS * SW / 16; k += BAND_THREADS) rows[k] = reinterpret_cast<const uint4 *>(band_words)[k];
        } else {
            unsigned char *bytes = out.indexed + ((size_t)local * GD_SCREEN_HEIGHT + row0) * SW;
            for (int k = tid; k < BAND_ROWS * SW; k += BAND_THREADS) bytes[k] = band_bytes[k];
        }
    }
    if (out.rgb) {   // four pixels, twelve bytes, three words per step
        unsigned char *rows = out.rgb + ((size_t)local * GD_SCREEN_HEIGHT + row0) * SW * 3;
        const bool aligned = (reinterpret_cast<size_t>(out.rgb) & 3) == 0;
        for (int k = tid; k < BAND_ROWS * SW / 4; k += BAND_THREADS) {
            const unsigned int four = band_words[k];
            const unsigned int c0 = pal[four & 0xFFu], c1 = pal[(four >> 8) & 0xFFu], c2 = pal[(four >> 16) & 0xFFu], c3 = pal[four >> 24];
            const unsigned int w0 = c0 | (c1 << 24), w1 = (c1 >> 8) | (c2 << 16), w2 = (c2 >> 16) | (c3 << 8);
            if (aligned) {
                unsigned int *words = reinterpret_cast<unsigned int *>(rows) + 3 * k;
                words[0] = w0; words[1] = w1; words[2] = w2;
            } else {
                unsigned char *bytes = rows + 12 * k;
                for (int q = 0; q < 4; ++q) { bytes[q] = (unsigned char)(w0 >> (8 * q)); bytes[4 + q] = (unsigned char)(w1 >> (8 * q)); bytes[8 + q] = (unsigned char)(w2 >> (8 * q)); }
            }
        }
    }
    if (!out.obs && !out.frames) return;
    // --- the band's observation rows, pooled from LDS (_triton_kernels.py:120-177).  An observation pixel covers 240/84 source
    // rows and 320/84 source columns; its weights (y_overlap * x_overlap) // 48 are exactly (y_overlap / 12) * (x_overlap / 4),
    // since row overlaps are multiples of 12 and column overlaps multiples of 4 (84 = 12 * 7 = 4 * 21, 240 = 12 * 20,
    // 320 = 4 * 80): the weighted sum factors into a pass along the rows and one down the columns, all in integers.
    // Seven observation rows pool exactly twenty source rows; rows at or past source_rows are black.
    constexpr int OBS_GROUP = 7, SRC_GROUP = OBS_GROUP * GD_SCREEN_HEIGHT / GD_OBS_SIZE;   // 7 and 20
    static_assert(BAND_OBS_ROWS % OBS_GROUP == 0 && SRC_GROUP * GD_OBS_SIZE == OBS_GROUP * GD_SCREEN_HEIGHT, "observation rows group by seven");
    // per source row and observation column: the three channel sums along the row, 16 bits each (at most 80 * 255)
    unsigned short *along = reinterpret_cast<unsigned short *>(&shading_lds);
    static_assert(sizeof(shading_lds) >= (size_t)SRC_GROUP * GD_OBS_SIZE * 3 * sizeof(unsigned short), "row sums fit the shading tables' LDS");
    const int first_obs_row = band * BAND_OBS_ROWS;
    for (int group = 0; group < BAND_OBS_ROWS / OBS_GROUP; ++group) {
        __syncthreads();   // the billboard records (first round) or the last group's row sums are no longer needed
        for (int q = tid; q < SRC_GROUP * GD_OBS_SIZE; q += BAND_THREADS) {
            const int sy = q / GD_OBS_SIZE, ox = q - sy * GD_OBS_SIZE;
            const int band_row = group * SRC_GROUP + sy;
            const unsigned char *row = band_bytes + band_row * SW;
            const int x_start = ox * 320, x_end = x_start + 320, first_x = x_start / 84;
            unsigned int rs = 0, gs = 0, bs = 0;
            if (row0 + band_row < out.source_rows) {
#pragma unroll
                for (int sx = 0; sx < 5; ++sx) {
                    const int source_x = first_x + sx;
                    const int over = min(x_end, (source_x + 1) * 84) - max(x_start, source_x * 84);
                    const unsigned weight = (source_x >= SW || over <= 0) ? 0u : (unsigned)over >> 2;
                    const unsigned int colour = pal[row[min(source_x, SW - 1)]];
                    rs += __umul24(colour & 0xFFu, weight); gs += __umul24((colour >> 8) & 0xFFu, weight); bs += __umul24(colour >> 16, weight);
                }
            }
            along[3 * q] = (unsigned short)rs; along[3 * q + 1] = (unsigned short)gs; along[3 * q + 2] = (unsigned short)bs;
        }
        __syncthreads();
        for (int q = tid; q < OBS_GROUP * GD_OBS_SIZE; q += BAND_THREADS) {
            const int row_in_group = q / GD_OBS_SIZE, ox = q - row_in_group * GD_OBS_SIZE;
            const int y_start = row_in_group * 240, y_end = y_start + 240, first_y = y_start / 84;   // relative to the group's first source row
            unsigned int rs = 0, gs = 0, bs = 0;
#pragma unroll
            for (int sy = 0; sy < 4; ++sy) {
                const int source_y = first_y + sy;
                const int over = min(y_end, (source_y + 1) * 84) - max(y_start, source_y * 84);
                const unsigned weight = (source_y >= SRC_GROUP || over <= 0) ? 0u : (unsigned)over / 12u;
                const unsigned short *sums = along + 3 * (min(source_y, SRC_GROUP - 1) * GD_OBS_SIZE + ox);
                rs += __umul24(sums[0], weight); gs += __umul24(sums[1], weight); bs += __umul24(sums[2], weight);
            }
            const unsigned r = (rs + 800u) / 1600u, g = (gs + 800u) / 1600u, b = (bs + 800u) / 1600u;
            reinterpret_cast<unsigned char *>(gray_words)[group * OBS_GROUP * GD_OBS_SIZE + q] = (unsigned char)((r * 77u + g * 150u + b * 29u + 128u) >> 8);
        }
    }
    __syncthreads();
    // the band's pixels are contiguous in the observation; they go out, and the stack is rolled, a word (four pixels) per thread
    const size_t F = (size_t)GD_OBS_SIZE * GD_OBS_SIZE / 4;     // words per observation
    const bool stack_aligned = ((reinterpret_cast<size_t>(out.frames) | reinterpret_cast<size_t>(out.final_frames)) & 3) == 0;
    const bool resets = out.reset_mask && out.reset_mask[local];
    auto load_word = [](const unsigned char *p, bool aligned) -> unsigned int {
        if (aligned) return *reinterpret_cast<const unsigned int *>(p);
        return (unsigned)p[0] | ((unsigned)p[1] << 8) | ((unsigned)p[2] << 16) | ((unsigned)p[3] << 24);
    };
    auto store_word = [](unsigned char *p, unsigned int v, bool aligned) {
        if (aligned) *reinterpret_cast<unsigned int *>(p) = v;
        else for (int k = 0; k < 4; ++k) p[k] = (unsigned char)(v >> (8 * k));
    };
    for (int k = tid; k < BAND_OBS_ROWS * GD_OBS_SIZE / 4; k += BAND_THREADS) {
        const size_t word = (size_t)first_obs_row * GD_OBS_SIZE / 4 + k;
        const unsigned int grays = gray_words[k];
        if (out.obs) store_word(out.obs + ((size_t)local * F + word) * 4, grays, (reinterpret_cast<size_t>(out.obs) & 3) == 0);
        if (!out.frames) continue;
        unsigned char *stack_lane = out.frames + (size_t)local * GD_FRAME_STACK * F * 4;
        unsigned int kept[GD_FRAME_STACK];
        // a lane that steps drops its oldest observation; it is only read for a copy of a stack that stays as it is
        const bool reads = !resets, reads_oldest = reads && out.stack_mode != GD_STACK_STEP && out.final_frames;
        for (int f = 0; f < GD_FRAME_STACK; ++f)
            kept[f] = (reads && (f > 0 || reads_oldest)) ? load_word(stack_lane + (size_t)f * F * 4 + word * 4, stack_aligned) : 0u;
        store_stack_word(stack_lane, out.final_frames ? out.final_frames + (size_t)local * GD_FRAME_STACK * F * 4 : nullptr, out.final_hwc,
                         stack_aligned, word, kept, grays, resets, out.stack_mode);
    }
}

// ---------------------------------------------------------------------------------------------
// actor packing: engine.py:14328-14682 with the sprite-id helpers of 14011-14136 and 14258-14317
// ---------------------------------------------------------------------------------------------
// Index of the animation frame showing after `elapsed` tics: the number of frames whose running end has
// passed, held on the last one (engine.py:14084-14091, 14117-14122).
__device__ __forceinline__ int frame_after(i64 elapsed, const int64_t *durations, int frames, i64 count) {
    i64 end = 0; int frame = 0;
    for (int k = 0; k < frames; ++k) { end += durations[k]; frame += elapsed >= end ? 1 : 0; }
    const i64 last = count - 1;
    return (int)(frame < last ? frame : last);
}

__device__ __forceinline__ i64 clamp_type(i64 v, i64 hi) { return v < 0 ? 0 : (v > hi ? hi : v); }

__device__ __forceinline__ i64 explosion_patch(const gd_actor_desc &a, i64 kind, i64 remaining) {
    kind = clamp_type(kind, 2);
    const int F = a.explosion_frames;
    const i64 elapsed = a.projectile_explosion_total_tics[kind] - remaining;
    const int frame = frame_after(elapsed, a.projectile_explosion_frame_durations + kind * F, F, a.projectile_explosion_frame_counts[kind]);
    return a.raw_projectile_explosion_sprite_ids[kind * F + frame];
}

__global__ void __launch_bounds__(64) pack_actors_kernel(gd_actor_desc a, int width) {
    const int slot = blockIdx.x * blockDim.x + threadIdx.x;
    const int n = blockIdx.y;
    if (slot >= width || n >= a.lane_count) return;
    float x = 0, y = 0, z = 0; i64 patch = 0; bool alive = false, bright = false; int style = -1;
    int k = slot;
    const int Se = a.enemy_slots, Sd = a.doll_count, Sp = a.player_projectile_slots, Sq = a.enemy_projectile_slots;
    if (k < Se) {                                   // monsters (engine.py:14011-14077, 14125-14136)
        const size_t i = (size_t)n * Se + k;
        x = a.enemy_x[i]; y = a.enemy_y[i]; z = a.enemy_z[i]; alive = a.enemy_alive[i] != 0;
        const i64 kind = clamp_type(a.enemy_type[i], 5);
        const int facing = a.enemy_rotation[i];
        const int tics = a.enemy_animation_tics[i];
        int walking = (tics / a.enemy_walk_frame_tics[kind]) % 4;
        int idling = (tics / a.enemy_idle_frame_tics[kind]) % 2;
        if (kind == 2) idling = 0;
        if (a.enemy_target_slot[i] < -1) walking = idling;
        const int phase = a.enemy_attack_phase[i], cooldown = a.enemy_cooldown[i];
        const bool recovering = cooldown > a.enemy_attack_recovery[kind] / 2;
        const bool hitscanner = kind == 0 || kind == 1, melee = kind == 4 || kind == 5;
        int attacking = 0;
        if (hitscanner && phase == 2) attacking = recovering ? 1 : 0;
        if (melee && phase == 1) attacking = cooldown <= 8 ? 1 : 0;
        if (melee && phase == 2) attacking = 2;
        if (kind == 3 && (phase == 4 || phase == 2)) attacking = 1;
        if (kind == 3 && phase == 3) attacking = 2;
        patch = phase > 0 ? a.enemy_attack_sprite_ids[(kind * a.attack_frames + attacking) * 8 + facing]
                          : a.enemy_walk_sprite_ids[(kind * 4 + walking) * 8 + facing];
        if (a.enemy_pain_tics[i] > 0) patch = a.enemy_pain_sprite_ids[kind * 8 + facing];
        bright = (kind == 1 && phase == 2 && recovering) || (kind == 3 && (phase == 2 || phase == 3));
    } else if ((k -= Se) < Sd) {                    // the other players' start dolls (engine.py:14345-14379)
        x = a.doll_x[k]; y = a.doll_y[k]; z = a.doll_z[k]; alive = a.player_dead[n] == 0;
        patch = a.enemy_walk_sprite_ids[(2 * 4 + 0) * 8 + a.doll_rotation[(size_t)n * Sd + k]];
    } else if ((k -= Sd) < Se) {                    // corpses (engine.py:14079-14106)
        const size_t i = (size_t)n * Se + k;
        x = a.enemy_x[i]; y = a.enemy_y[i]; z = a.enemy_z[i]; alive = a.enemy_death_tics[i] > 0;
        const i64 kind = clamp_type(a.enemy_death_type[i], 5);
        const i64 elapsed = a.enemy_death_elapsed[i];
        if (a.enemy_death_extreme[i]) {
            const int F = a.xdeath_frames;
            patch = a.enemy_xdeath_sprite_ids[kind * F + frame_after(elapsed, a.enemy_xdeath_frame_durations + kind * F, F, a.enemy_xdeath_frame_counts[kind])];
        } else {
            const int F = a.death_frames;
            patch = a.enemy_death_sprite_ids[kind * F + frame_after(elapsed, a.enemy_death_frame_durations + kind * F, F, a.enemy_death_frame_counts[kind])];
        }
    } else if ((k -= Se) < Sp) {                    // rockets and plasma balls in flight (engine.py:14410-14460)
        const size_t i = (size_t)n * Sp + k;
        x = a.projectile_x[i]; y = a.projectile_y[i]; z = a.projectile_z[i]; alive = a.projectile_alive[i] != 0;
        const i64 shot = clamp_type(a.projectile_type[i], 1);
        const int frame = shot == 1 ? (a.projectile_age[i] / 6) % 2 : 0;
        patch = a.raw_projectile_flight_sprite_ids[(shot * 2 + frame) * 8 + a.projectile_rotation[i]];
        bright = alive; style = shot == 1 ? 0 : -1;
    } else if ((k -= Sp) < Sq) {                    // monster fireballs in flight (engine.py:14462-14510)
        const size_t i = (size_t)n * Sq + k;
        x = a.enemy_projectile_x[i]; y = a.enemy_projectile_y[i]; z = a.enemy_projectile_z[i]; alive = a.enemy_projectile_alive[i] != 0;
        const int frame = (a.enemy_projectile_age[i] / 4) % 2;
        patch = a.raw_projectile_flight_sprite_ids[(2 * 2 + frame) * 8 + a.enemy_projectile_rotation[i]];
        bright = alive; style = 1;
    } else if ((k -= Sq) < Sp) {                    // the player's explosions (engine.py:14512-14541)
        const size_t i = (size_t)n * Sp + k;
        x = a.projectile_x[i]; y = a.projectile_y[i]; z = a.projectile_z[i]; alive = a.projectile_impact_tics[i] > 0;
        patch = explosion_patch(a, a.projectile_impact_type[i], a.projectile_impact_tics[i]);
        bright = alive; style = a.projectile_impact_type[i] == 1 ? 0 : -1;
    } else if ((k -= Sp) < Sq) {                    // fireball explosions (engine.py:14543-14573)
        const size_t i = (size_t)n * Sq + k;
        x = a.enemy_projectile_x[i]; y = a.enemy_projectile_y[i]; z = a.enemy_projectile_z[i]; alive = a.enemy_projectile_impact_tics[i] > 0;
        patch = explosion_patch(a, 2, a.enemy_projectile_impact_tics[i]);
        bright = alive; style = 1;
    } else if ((k -= Sq) < a.fog_slots) {           // teleport fog: 12 frames of 6 tics out of 72 (engine.py:14577-14595)
        const size_t i = (size_t)n * a.fog_slots + k;
        x = a.teleport_fog_x[i]; y = a.teleport_fog_y[i]; z = a.teleport_fog_z[i];
        const int tics = a.teleport_fog_tics[i];
        alive = tics > 0;
        const int elapsed = 72 - tics;
        int frame = elapsed >= 0 ? elapsed / 6 : -((-elapsed + 5) / 6);   // floor division, like Torch's //
        if (frame > 11) frame = 11;
        if (frame < 0) frame += 12;                                      // a negative index counts from the end
        patch = a.raw_teleport_fog_sprite_ids[frame];
        bright = alive; style = 1;
    } else if ((k -= a.fog_slots) < a.puff_slots) { // bullet puffs: 4 frames of 4 tics (engine.py:14597-14630)
        const size_t i = (size_t)n * a.puff_slots + k;
        x = a.hitscan_puff_x[i]; y = a.hitscan_puff_y[i]; z = a.hitscan_puff_z[i];
        const int tics = a.hitscan_puff_tics[i];
        alive = tics > 0;
        const int frame = tics > 12 ? 0 : (tics > 8 ? 1 : (tics > 4 ? 2 : 3));
        patch = a.raw_bullet_puff_sprite_ids[frame];
        bright = frame == 0; style = -2;
    } else if ((k -= a.puff_slots) < a.item_count) {   // map items (engine.py:14258-14317, 14632-14655)
        const size_t i = (size_t)n * a.item_count + k;
        x = a.item_x[k]; y = a.item_y[k]; z = a.item_z[k]; alive = a.item_available[i] != 0;
        const i64 kind = a.item_types[k];
        const i64 elapsed = (i64)a.episode_time[n] + (6 - (i64)a.item_animation_initial_tics[i]);
        const i64 sixth = elapsed >= 0 ? elapsed / 6 : -((-elapsed + 5) / 6);
        const int phase = (int)(((sixth % 6) + 6) % 6);
        const int swing = phase == 0 ? -1 : (phase <= 3 ? phase - 1 : 5 - phase);   // A, then B C D C B
        patch = a.item_raw_visual_types[k];
        if (kind == 2014 && swing >= 0) patch = a.raw_item_animation_sprite_ids[swing];
        if (kind == 2015 && swing >= 0) patch = a.raw_item_animation_sprite_ids[3 + swing];
        const bool green = kind == 2018 && (((elapsed % 13) + 13) % 13) >= 6;
        const bool blue = kind == 2019 && (((elapsed % 12) + 12) % 12) >= 6;
        if (green) patch = a.raw_item_animation_sprite_ids[6];
        if (blue) patch = a.raw_item_animation_sprite_ids[7];
        bright = green || blue;
    } else {                                        // what monsters drop (engine.py:14657-14682)
        k -= a.item_count;
        const size_t i = (size_t)n * a.drop_slots + k;
        x = a.drop_x[i]; y = a.drop_y[i]; z = a.drop_z[i];
        const i64 kind = a.drop_type[i];
        alive = kind >= 0 && a.drop_spawned[i] != 0;
        patch = a.raw_static_sprite_ids[kind == 2002 ? 14 : (kind == 2007 ? 6 : 12)];
    }
    const size_t out = (size_t)n * width + slot;
    a.sprite_x[out] = x; a.sprite_y[out] = y; a.sprite_z[out] = z;
    a.sprite_id[out] = (int)patch;
    a.sprite_alive[out] = alive ? 1 : 0; a.sprite_fullbright[out] = bright ? 1 : 0; a.sprite_style[out] = (signed char)style;
}

// ---------------------------------------------------------------------------------------------
// host side
// ---------------------------------------------------------------------------------------------
thread_local std::string g_error;

int fail(int code, const std::string &message) { g_error = message; return code; }

// gd_pack_weapon: one thread per lane.  Which patch the player's weapon shows and where (engine.py:14949-14967,
// 15051-15092): the frame table is indexed by weapon, by a parity that alternates with every shot (an idling chainsaw
// alternates every four tics instead) and by the tics left of the weapon's state; a weapon being lowered or raised sits
// six map pixels lower per tic, as does one raised at the start of an episode; a ready weapon sways with the player's bob
// along a circle of the fine sine table that advances 128 steps a tic.
__global__ void __launch_bounds__(64) pack_weapon_kernel(gd_weapon_desc d) {
    const int lane = blockIdx.x * blockDim.x + threadIdx.x;
    if (lane >= d.lane_count) return;
    const i64 slots = d.cooldown_slots;
    const i64 weapon = clampi(d.active_weapon[lane], 0, 7);
    const i64 state_tics = d.weapon_state_cooldown[lane];
    const i64 tic = clampi(state_tics, 0, slots - 1);
    i64 parity = d.weapon_fire_count[lane] % 2;
    if (parity < 0) parity += 2;                    // torch.remainder: the sign of the divisor
    if (weapon == 1 && tic == 0) parity = (max64(d.weapon_ready_tics[lane] - 1, 0) / 4) % 2;
    const i64 entry = (weapon * 2 + parity) * slots + tic;
    const i64 switching = d.pending_weapon[lane] >= 0;
    const i64 raising = d.weapon_raise_cooldown[lane];
    i64 lowered = switching ? clampi(16 - d.weapon_lower_cooldown[lane], 0, 16) : raising;      // engine.py:111 (16 tics to lower)
    const i64 time = d.episode_time[lane];
    lowered = max64(lowered, clampi(14 - (time - 1), 0, 14));                                   // engine.py:114 (14 tics to raise at spawn)
    const bool steady = state_tics <= 0 && raising <= 0 && !switching;
    const i64 swing = mul64(time, 128) & (FINE_ANGLES - 1);
    const i64 bob = d.player_bob_fixed[lane];
    const i64 sway_x = steady ? mul64(bob, d.fine_sine[(swing + FINE_ANGLES / 4) & (FINE_ANGLES - 1)]) >> 16 : 0;
    const i64 sway_y = steady ? mul64(bob, d.fine_sine[swing & (FINE_ANGLES / 2 - 1)]) >> 16 : 0;
    int64_t *out = d.weapon_state + (size_t)lane * 5;
    out[0] = d.weapon_frame_ids[entry];
    out[1] = d.weapon_flash_ids[entry];
    out[2] = sway_x;
    out[3] = mul64(lowered, 6 * FIXED_UNIT) + sway_y;
    out[4] = d.player_dead[lane] ? 0 : 1;
    if (d.flash_light) d.flash_light[lane] = d.weapon_flash_lights[entry];
}

#define HIP_TRY(expr)                                                                          \
    do {                                                                                       \
        hipError_t e_ = (expr);                                                                \
        if (e_ != hipSuccess) return fail(GD_E_HIP, std::string(#expr) + ": " + hipGetErrorString(e_)); \
    } while (0)

// A descriptor filled in against another version of the header is refused before any of its fields is trusted.
#define SIZE_CHECK(ptr, type)                                                                  \
    do {                                                                                       \
        if ((ptr)->struct_size != sizeof(type))                                                \
            return fail(GD_E_ARG, #type ".struct_size is " + std::to_string((ptr)->struct_size) + ", this library expects " + \
                                      std::to_string(sizeof(type)) + ": the caller was built against another gradoom_amd.h"); \
    } while (0)

}  // namespace

// Every kernel of a frame runs on the caller's stream.  (Cutting a batch into chunks or halves pipelined over
// more streams measured no faster: the kernels already fill the machine.)
struct gd_renderer {
    DeviceMap dm;
    Scratch sc;
    int chunk_lanes;
    int assembly;                            // GD_ASSEMBLY_*: how frames are put together after the walls (see launch_chunk)
    unsigned char *scratch_block;            // the one allocation `sc` is laid out in (null for a renderer made for 0 lanes)
    size_t scratch_bytes;
    std::vector<void *> allocations;
    hipEvent_t events[16];
    bool events_ready;
    // The flat pass (short kernels that leave most of the chip idle) runs beside the plane shading on a stream of the
    // renderer's own: forked from the caller's stream after the walls, joined before the billboards.
    hipStream_t side_stream;
    hipEvent_t fork_event, join_event;
    bool side_ready;
    Overlays overlays;                       // device pointers, counts 0 until gd_renderer_set_overlays
    std::vector<void *> overlay_allocations;
};

namespace {

// Working memory of callers that may not allocate (gd_render_static): one array per device, held until the
// process ends.  In host code the array's name only stands for the symbol; its address on the current
// device comes from hipGetSymbolAddress, once per device.
#define STATIC_SCRATCH_BYTES ((size_t)GD_STATIC_SCRATCH_MIB << 20)
#define STATIC_SCRATCH_DEVICES 64
}  // namespace
static __device__ __align__(256) unsigned char scratch[STATIC_SCRATCH_BYTES];
namespace {
unsigned char *g_static_scratch[STATIC_SCRATCH_DEVICES];

int static_scratch_address(unsigned char **out) {
    int device = 0;
    HIP_TRY(hipGetDevice(&device));
    if (device < 0 || device >= STATIC_SCRATCH_DEVICES) return fail(GD_E_ARG, "device ordinal beyond the static working memory table");
    if (!g_static_scratch[device]) {
        unsigned char *ptr = nullptr;
        HIP_TRY(hipGetSymbolAddress(reinterpret_cast<void **>(&ptr), HIP_SYMBOL(scratch)));
        if (!ptr) return fail(GD_E_HIP, "hipGetSymbolAddress returned no address for the static working memory");
        g_static_scratch[device] = ptr;
    }
    if (out) *out = g_static_scratch[device];
    return GD_OK;
}

__global__ void fill_words_kernel(unsigned int *words, size_t count, unsigned int value) {
    for (size_t k = (size_t)blockIdx.x * blockDim.x + threadIdx.x; k < count; k += (size_t)gridDim.x * blockDim.x) words[k] = value;
}

// Blocks of the spill pool (320 columns each, 1.25 MiB) for a chunk of `lanes` lanes: every column of up to eight
// lanes, one column in 32 of a large chunk (160 MiB at 4096 lanes).  The static working memory has room for one.
size_t spill_pool_blocks(int lanes) {
    const int share = lanes / 32 > 8 ? lanes / 32 : 8;
    return (size_t)(lanes < share ? lanes : share);
}
#define STATIC_SPILL_BLOCKS 1

// Lay the per-chunk buffers of `sc` out in one block of device memory for `L` lanes of map `h` (every buffer
// 256-byte aligned) and return the bytes the layout takes; with a null `base` nothing is assigned and the call
// only measures.  `status` is not part of the block: the renderer keeps it.  `depth`: also the scene depth plane
// of frames that draw decals.
size_t carve_scratch(Scratch &sc, unsigned char *base, size_t L, const gd_map_desc &h, bool depth, size_t spill_blocks) {
    // `depth`: frames that draw decals also need a scene depth plane
    size_t used = 0;
    auto take = [&](auto **field, size_t count) {
        typedef typename std::remove_reference<decltype(**field)>::type T;
        used = (used + 255) & ~(size_t)255;
        if (base) *field = reinterpret_cast<T *>(base + used);
        used += (count ? count : 1) * sizeof(T);
    };
    const size_t W = h.wall_count, PX = (size_t)VH * SW, levels = (size_t)(h.floor_level_count + h.ceil_level_count);
    take(&sc.ctx, L);
    take(&sc.rec, L * W);
    take(&sc.span, L * W);
    take(&sc.frag_rec, L * (size_t)(h.split_count > 0 ? h.split_count * h.fragment_slots : 1));
    take(&sc.cand, L * CAND_MAX * SW + spill_blocks * SPILL_DEPTH * SW);   // byte offsets into it are 32 bits wide: L <= 4096, spill_blocks <= 512
    sc.spill_base = (unsigned)(L * CAND_MAX * SW); sc.spill_slots = (int)(spill_blocks * SW);
    take(&sc.cand_count, L * SW);
    take(&sc.spill_columns, spill_blocks * SW);
    take(&sc.spill_count, 1);
    take(&sc.flat_sector, L * PX);
    take(&sc.flat_flags, L * PX);
    take(&sc.flat_span, L * 4);
    take(&sc.flat_tail, L * 2 * SW);
    take(&sc.flat_rows, L * (size_t)VH);
    take(&sc.flat_row_count, 1);
    take(&sc.gap_columns, L * 2 * SW);
    take(&sc.gap_column_count, 1);
    take(&sc.flat_col_top, L * 2 * SW);
    take(&sc.flat_list, L * FLAT_LIST_MAX);
    take(&sc.flat_list_count, L);
    sc.pass_slots = h.sector_count < 16 ? 16 : (h.sector_count > PASS_MAX ? PASS_MAX : h.sector_count);
    take(&sc.pass_rec, L * (size_t)sc.pass_slots * SW);
    take(&sc.pass_path_distance, L * (size_t)sc.pass_slots * SW);
    take(&sc.pass_count, L * SW);
    take(&sc.meta, L * PX);
    take(&sc.clip_depth, L * PX);
    take(&sc.level_reach, L * levels);
    take(&sc.level_far, L * levels);
    take(&sc.level_masks, L * LEVEL_BUCKETS * (size_t)(levels <= 32 * LEVEL_MASK_WORDS_MAX ? (levels + 31) / 32 : 1));
    take(&sc.level_plane, L * levels * 2);
    take(&sc.row_slope, L * (size_t)VH);
    take(&sc.step_scale, L * STEP_TABLE);
    take(&sc.block_hit, L * SW);
    take(&sc.lane_blends, L);
    take(&sc.strip_key, L * SEGS_PER_LANE);
    take(&sc.strip_order, L * SEGS_PER_LANE);
    if (depth) take(&sc.scene_depth, L * PX);
    take(&sc.frame, L * (size_t)GD_SCREEN_HEIGHT * SW);   // where a frame is put together kernel by kernel when the caller takes none
    return (used + 255) & ~(size_t)255;
}

template <typename T>
int upload(gd_renderer *r, const T *host, size_t count, const T **device) {
    if (count == 0) count = 1;
    void *ptr = nullptr;
    HIP_TRY(hipMalloc(&ptr, count * sizeof(T)));
    r->allocations.push_back(ptr);
    if (host) HIP_TRY(hipMemcpy(ptr, host, count * sizeof(T), hipMemcpyHostToDevice));
    else HIP_TRY(hipMemset(ptr, 0, count * sizeof(T)));
    *device = static_cast<const T *>(ptr);
    return GD_OK;
}

template <typename T>
int scratch_alloc(gd_renderer *r, size_t count, T **device) {
    void *ptr = nullptr;
    HIP_TRY(hipMalloc(&ptr, (count ? count : 1) * sizeof(T)));
    r->allocations.push_back(ptr);
    *device = static_cast<T *>(ptr);
    return GD_OK;
}

// Bounding boxes of the sectors, grouped by plane level (floors first).  The box of a sector is
// that of its edges padded by half a map unit; the even-odd test of engine.py:9598-9617 counts
// edges to the right of the point, so a sector whose boundary is not a set of closed loops can
// also test inside anywhere to the left of its edges and its box is open on that side.
void build_level_boxes(const gd_map_desc *h, std::vector<int> &ofs, std::vector<float4> &boxes) {
    const int S = h->sector_count;
    std::vector<float4> sector_box(S);
    std::vector<char> has_box(S, 0);
    for (int s = 0; s < S; ++s) {
        float x0 = GD_INF, y0 = GD_INF, x1 = -GD_INF, y1 = -GD_INF;
        std::map<std::pair<float, float>, int> degree;
        for (int k = h->sector_edge_ofs[s]; k < h->sector_edge_ofs[s + 1]; ++k) {
            const float *w = h->walls + 4 * h->sector_edge_idx[k];
            for (int e = 0; e < 2; ++e) {
                float x = w[2 * e] + 0.0f, y = w[2 * e + 1] + 0.0f;
                x0 = std::fmin(x0, x); x1 = std::fmax(x1, x); y0 = std::fmin(y0, y); y1 = std::fmax(y1, y);
                ++degree[std::make_pair(x, y)];
            }
            has_box[s] = 1;
        }
        bool closed = true;
        for (const auto &entry : degree) closed = closed && (entry.second % 2 == 0);
        if (!closed) x0 = -GD_INF;
        sector_box[s] = make_float4(x0 - 0.5f, y0 - 0.5f, x1 + 0.5f, y1 + 0.5f);
    }
    ofs.assign(1, 0);
    for (int side = 0; side < 2; ++side) {
        const float *levels = side == 0 ? h->floor_levels : h->ceil_levels;
        const int count = side == 0 ? h->floor_level_count : h->ceil_level_count;
        for (int l = 0; l < count; ++l) {
            for (int s = 0; s < S; ++s)
                if (has_box[s] && h->sector_heights[2 * s + side] == levels[l]) boxes.push_back(sector_box[s]);
            ofs.push_back((int)boxes.size());
        }
    }
}

void build_fine_tables(std::vector<i64> &sine, std::vector<i64> &tangent) {
    // engine.py:309-328
    const double PI = 3.14159265358979323846;
    sine.assign(FINE_ANGLES, 0);
    tangent.assign(FINE_ANGLES / 2, 0);
    const int quarter = FINE_ANGLES / 4;
    for (int i = 0; i < quarter; ++i) sine[i] = (i64)std::trunc(std::sin((double)i * (2.0 * PI / FINE_ANGLES)) * 65536.0);
    for (int i = 0; i < quarter; ++i) sine[quarter + i] = sine[quarter - 1 - i];
    for (int i = 0; i < 2 * quarter; ++i) sine[2 * quarter + i] = -sine[i];
    sine[quarter] = 65536;
    sine[3 * quarter] = -65536;
    for (int i = 0; i < FINE_ANGLES / 2; ++i) {
        double phase = ((double)i - FINE_ANGLES / 4) * (2.0 * PI / FINE_ANGLES);
        if (i == 0) phase += PI / FINE_ANGLES;
        tangent[i] = (i64)std::trunc(std::tan(phase) * 65536.0 + 0.5);
    }
}

// Host-side check of a map descriptor before anything is uploaded: every index a kernel follows must land inside
// its table (a bad one would be a wild device read), and inputs the renderer does not reproduce are refused.
int validate_map(const gd_map_desc *h) {
    const int W = h->wall_count, S = h->sector_count, V = h->vertex_count, T = h->texture_count, K = h->neighbor_slots;
    const void *const needed[] = {h->walls, h->walls_fixed, h->wall_sectors, h->wall_vertex, h->side_tex, h->side_off, h->wall_len,
                                  h->direct_neighbor_table, h->solid_bridge_start_ofs, h->solid_bridge_end_ofs, h->vertex_wall_ofs,
                                  h->sector_wall_ofs, h->sector_edge_ofs, h->grid_cell_ofs, h->grid_item_edge_ofs, h->floor_levels,
                                  h->ceil_levels, h->sector_heights, h->sector_lights, h->sector_floor_tex, h->sector_ceil_tex,
                                  h->tex_atlas, h->tex_w, h->tex_h, h->playpal, h->colormap};
    for (const void *p : needed) if (!p) return fail(GD_E_ARG, "gd_map_desc holds a null table");
    if (V <= 0 || T <= 0 || K < 0 || h->tex_max_h <= 0 || h->tex_max_w <= 0 || h->blocking_count < 0 || h->sprite_count < 0 ||
        h->floor_level_count <= 0 || h->ceil_level_count <= 0 || h->grid_nx <= 0 || h->grid_ny <= 0)
        return fail(GD_E_ARG, "gd_map_desc holds a count out of range");
    if (K > 0 && (!h->endpoint_neighbors || !h->endpoint_neighbor_starts || !h->endpoint_neighbor_ends)) return fail(GD_E_ARG, "missing endpoint neighbour tables");
    if (h->blocking_count > 0 && !h->blocking_walls) return fail(GD_E_ARG, "missing blocking_walls");
    if (h->sprite_count > 0 && (!h->spr_atlas || !h->spr_opaque || !h->spr_post_top || !h->spr_w || !h->spr_h || !h->spr_left || !h->spr_top))
        return fail(GD_E_ARG, "missing sprite patch tables");
    for (int s = 0; s < S; ++s) {
        const float floor_z = h->sector_heights[2 * s], ceiling_z = h->sector_heights[2 * s + 1];
        if (!(floor_z == floor_z) || !(ceiling_z == ceiling_z)) return fail(GD_E_ARG, "sector_heights holds a NaN");
        if (h->sector_floor_tex[s] < 0 || h->sector_floor_tex[s] >= T || h->sector_ceil_tex[s] < 0 || h->sector_ceil_tex[s] >= T)
            return fail(GD_E_ARG, "a sector's flat names a texture out of range");
    }
    for (int t = 0; t < T; ++t)
        if (h->tex_w[t] <= 0 || h->tex_w[t] > h->tex_max_w || h->tex_h[t] <= 0 || h->tex_h[t] > h->tex_max_h || h->tex_w[t] > 32768 || h->tex_h[t] > 32768)
            return fail(GD_E_ARG, "a texture size lies outside 1..32768 or outside the atlas");
    for (int p = 0; p < h->sprite_count; ++p)
        if (h->spr_w[p] < 0 || h->spr_w[p] > h->spr_max_w || h->spr_h[p] < 0 || h->spr_h[p] > h->spr_max_h)
            return fail(GD_E_ARG, "a sprite patch is larger than its atlas");
    for (int w = 0; w < W; ++w) {
        const int front = h->wall_sectors[2 * w], back = h->wall_sectors[2 * w + 1];
        if (front < 0 || front >= S || back < -1 || back >= S) return fail(GD_E_ARG, "wall_sectors names a sector out of range");
        for (int e = 0; e < 2; ++e) if (h->wall_vertex[2 * w + e] < 0 || h->wall_vertex[2 * w + e] >= V) return fail(GD_E_ARG, "wall_vertex names a vertex out of range");
        for (int k = 0; k < 6; ++k) if (h->side_tex[6 * w + k] < -1 || h->side_tex[6 * w + k] >= T) return fail(GD_E_ARG, "side_tex names a texture out of range");
        for (int k = 0; k < K; ++k) if (h->endpoint_neighbors[(size_t)w * K + k] < 0 || h->endpoint_neighbors[(size_t)w * K + k] >= W) return fail(GD_E_ARG, "endpoint_neighbors names a linedef out of range");
        for (int k = 0; k < 2; ++k) if (h->direct_neighbor_table[4 * w + k] < 0 || h->direct_neighbor_table[4 * w + k] >= W) return fail(GD_E_ARG, "direct_neighbor_table names a linedef out of range");
    }
    struct Csr { const int *ofs, *idx; int rows, limit; const char *name; };
    const Csr lists[] = {{h->solid_bridge_start_ofs, h->solid_bridge_start_idx, W, W, "solid_bridge_start"}, {h->solid_bridge_end_ofs, h->solid_bridge_end_idx, W, W, "solid_bridge_end"},
                         {h->vertex_wall_ofs, h->vertex_wall_idx, V, W, "vertex_wall"}, {h->sector_wall_ofs, h->sector_wall_idx, S, W, "sector_wall"},
                         {h->sector_edge_ofs, h->sector_edge_idx, S, W, "sector_edge"}};
    for (const Csr &c : lists) {
        if (c.ofs[0] != 0) return fail(GD_E_ARG, std::string(c.name) + "_ofs must start at 0");
        for (int r = 0; r < c.rows; ++r) if (c.ofs[r + 1] < c.ofs[r]) return fail(GD_E_ARG, std::string(c.name) + "_ofs must not decrease");
        if (c.ofs[c.rows] > 0 && !c.idx) return fail(GD_E_ARG, std::string(c.name) + "_idx is missing");
        for (int k = 0; k < c.ofs[c.rows]; ++k) if (c.idx[k] < 0 || c.idx[k] >= c.limit) return fail(GD_E_ARG, std::string(c.name) + "_idx names a linedef out of range");
    }
    const size_t cells = (size_t)h->grid_nx * h->grid_ny;
    if (h->grid_cell_ofs[0] != 0) return fail(GD_E_ARG, "grid_cell_ofs must start at 0");
    for (size_t c = 0; c < cells; ++c) if (h->grid_cell_ofs[c + 1] < h->grid_cell_ofs[c]) return fail(GD_E_ARG, "grid_cell_ofs must not decrease");
    const int items = h->grid_cell_ofs[cells];
    if (items > 0 && (!h->grid_item_sector || (h->grid_item_edge_ofs[items] > 0 && !h->grid_item_edges))) return fail(GD_E_ARG, "missing grid item tables");
    if (h->grid_item_edge_ofs[0] != 0) return fail(GD_E_ARG, "grid_item_edge_ofs must start at 0");
    for (int it = 0; it < items; ++it) if (h->grid_item_edge_ofs[it + 1] < h->grid_item_edge_ofs[it]) return fail(GD_E_ARG, "grid_item_edge_ofs must not decrease");
    const size_t fine_cells = (size_t)h->fine_nx * h->fine_ny;
    for (size_t k = 0; k < fine_cells; ++k)
        if (FINE_KIND(h->fine_sector[k]) == FINE_DECIDED && (int)(h->fine_sector[k] & 0xFFFFu) >= S) return fail(GD_E_ARG, "fine_sector names a sector out of range");
    return GD_OK;
}

const int STAGE_COUNT = 9;

int launch_chunk(gd_renderer *r, const Scratch &chunk_scratch, const gd_lanes_desc *lanes, const gd_frame_out *out, int base, int count, hipStream_t stream, bool timed) {
    const gd_map_desc &m = r->dm.d;
    Scratch sc = chunk_scratch;
    if (out->final_frames && !out->frames) return fail(GD_E_ARG, "final_frames needs frames");
    if (out->final_frames_layout != GD_LAYOUT_CHW && out->final_frames_layout != GD_LAYOUT_HWC) return fail(GD_E_ARG, "unknown final_frames_layout");
    const size_t frame_stride = (size_t)GD_SCREEN_HEIGHT * SW;
    const size_t F = (size_t)GD_OBS_SIZE * GD_OBS_SIZE;
    const int source_rows = out->obs_source_rows == GD_SCREEN_HEIGHT ? GD_SCREEN_HEIGHT : VH;
    int stage = 0;
    auto mark = [&]() { if (timed) (void)hipEventRecord(r->events[stage], stream); ++stage; };
    // After the walls and the flat selection a frame is put together in one of two ways.  Kernel by kernel through a
    // 320x240 frame in device memory (shade, paint the flat pass's pixels, decals, billboards, overlays, then pool the
    // observation from it), the caller's `indexed` or the working memory's own: the faster way on this chip (its kernels
    // run at full occupancy), and the only one for frames that draw wall decals, which need a per-pixel scene depth.  Or
    // band by band in LDS (band_finish_kernel), the frame never reaching device memory: a fifth less traffic in the
    // assembly for a caller that only wants observations, at nine tenths of the speed; chosen with gd_renderer_set_assembly.
    const bool decals = lanes->decal_slots > 0 && lanes->decal_state && lanes->decal_geom && r->overlays.d.decal_variant_count > 0;
    if (!decals) sc.scene_depth = nullptr;
    if (decals && (!sc.scene_depth || !sc.frame)) return fail(GD_E_ARG, "decal working memory missing");
    const bool fused = !decals && (r->assembly == GD_ASSEMBLY_FUSED || (r->assembly == GD_ASSEMBLY_AUTO && !out->indexed && !sc.frame));
    unsigned char *frame_base = nullptr;
    if (!fused) {
        frame_base = out->indexed ? out->indexed + (size_t)base * frame_stride : sc.frame;
        if (!frame_base) return fail(GD_E_ARG, "assembling the frame kernel by kernel needs an indexed output");
    }
    mark();
    hipLaunchKernelGGL(lane_setup_kernel, dim3((count + 63) / 64), dim3(64), 0, stream, r->dm, *lanes, base, count, sc);
    hipLaunchKernelGGL(lane_tables_kernel, dim3(count), dim3(256), 0, stream, r->dm, *lanes, base, count, sc);
    hipLaunchKernelGGL(wall_setup_kernel, dim3((m.wall_count + SETUP_WALLS - 1) / SETUP_WALLS, count), dim3(SETUP_WALLS), 0, stream, r->dm, count, sc);
    if (m.split_count > 0)
        hipLaunchKernelGGL(fragment_setup_kernel, dim3((m.split_count * m.fragment_slots + 63) / 64, count), dim3(64), 0, stream, r->dm, count, sc);
    hipLaunchKernelGGL(strip_key_kernel, dim3((count * (SW / 64) + 3) / 4), dim3(256), 0, stream, count, sc);
    if (sc.spill_slots > 0)
        hipLaunchKernelGGL(cand_spill_kernel, dim3(sc.spill_slots < SPILL_BLOCKS ? sc.spill_slots : SPILL_BLOCKS), dim3(64), 0, stream, r->dm, sc);
    hipLaunchKernelGGL(strip_order_kernel, dim3(1), dim3(1024), 0, stream, count * SEGS_PER_LANE, sc);
    mark();
    {
        const int wavefronts = (count * SEGS_PER_LANE + 64 / SEG_COLS - 1) / (64 / SEG_COLS);
        const bool split = m.split_count > 0;
        const dim3 select_block(64 * SELECT_STRIPS_PER_GROUP);
        // The longest strips here with their lists in LDS, the others on the side stream, both at once.  This way round: the
        // side stream starts a few microseconds behind, time enough for the staged launch's work-groups to be placed;
        // started together, the other launch's 20,000 take every wavefront slot first and the strips that decide how long
        // the pair lasts begin last.
        const int strips = count * SEGS_PER_LANE;
        const int staged_strips = r->side_ready ? (strips < SELECT_STAGED_STRIPS ? strips : SELECT_STAGED_STRIPS) : 0;
        auto select_kernel = split ? wall_select_kernel<true, false> : wall_select_kernel<false, false>;
        if (staged_strips > 0) {
            HIP_TRY(hipEventRecord(r->fork_event, stream));
            HIP_TRY(hipStreamWaitEvent(r->side_stream, r->fork_event, 0));
            auto staged_kernel = split ? wall_select_kernel<true, true> : wall_select_kernel<false, true>;
            hipLaunchKernelGGL(staged_kernel, dim3(staged_strips * SELECT_STAGED_PARTS), select_block, 0, stream, r->dm, count, sc, staged_strips);
            hipLaunchKernelGGL(select_kernel, dim3(strips), select_block, 0, r->side_stream, r->dm, count, sc, staged_strips);
            HIP_TRY(hipEventRecord(r->join_event, r->side_stream));
            HIP_TRY(hipStreamWaitEvent(stream, r->join_event, 0));
        } else {
            hipLaunchKernelGGL(select_kernel, dim3(strips), select_block, 0, stream, r->dm, count, sc, 0);
        }
        mark();
        const dim3 grid((wavefronts + WALL_STRIPS_PER_GROUP - 1) / WALL_STRIPS_PER_GROUP), block(64 * WALL_STRIPS_PER_GROUP);
        auto kernel = decals ? (split ? wall_raster_kernel<true, true> : wall_raster_kernel<true, false>)
                             : (split ? wall_raster_kernel<false, true> : wall_raster_kernel<false, false>);
        hipLaunchKernelGGL(kernel, grid, block, 0, stream, r->dm, count, sc, frame_base, frame_stride);
    }
    mark();
    // The plane shading and the flat pass do not depend on each other: the first reads the per-pixel words and writes the
    // pixels some drawseg owns, the second reads the same words and writes its own planes and, at the end, the pixels no
    // drawseg owns.  The flat pass is a chain of short kernels that wait more than they compute; it stays on the
    // caller's stream, where its first kernel starts the moment the traversal ends, and the shading goes to the renderer's
    // side stream, a few microseconds behind (the other way round the shading takes every compute unit before the first
    // block of the flat pass is placed).  (Not when stages are being timed.)
    const bool beside = !fused && !timed && r->side_ready;
    hipStream_t shade_stream = stream;
    if (beside) {
        HIP_TRY(hipEventRecord(r->fork_event, stream));
        HIP_TRY(hipStreamWaitEvent(r->side_stream, r->fork_event, 0));
        shade_stream = r->side_stream;
    }
    // timed (and so serial): shading, then the flat pass, each between its own marks
    auto shade_planes = [&]() {
        if (fused) return;
        const dim3 grid(((VH * SW / SHADE_RUN + 255) / 256 + SHADE_TILES - 1) / SHADE_TILES, count);
        const bool staged = m.floor_level_count + m.ceil_level_count <= 2 * PLANE_LEVELS;
        auto kernel = decals ? (staged ? plane_shade_kernel<true, true> : plane_shade_kernel<true, false>)
                             : (staged ? plane_shade_kernel<false, true> : plane_shade_kernel<false, false>);
        hipLaunchKernelGGL(kernel, grid, dim3(256), 0, shade_stream, r->dm, count, sc, frame_base, frame_stride);
    };
    if (!beside) shade_planes();
    mark();
    // the flat pass, where the walls left it something to decide
    hipLaunchKernelGGL(flat_gap_column_kernel, dim3(count), dim3(GAP_THREADS), 0, stream, r->dm, *lanes, base, count, sc);
    hipLaunchKernelGGL(flat_gap_repair_kernel, dim3(GAP_REPAIR_BLOCKS), dim3(64 * GAP_REPAIR_CHUNKS), 0, stream, r->dm, *lanes, base, sc);
    hipLaunchKernelGGL(flat_rows_kernel, dim3(count), dim3(64), 0, stream, count, sc);
    const int plane_levels = m.floor_level_count + m.ceil_level_count;
    const bool level_masks = plane_levels > LEVEL_MASK_MIN_LEVELS && plane_levels <= 32 * LEVEL_MASK_WORDS_MAX;   // level_mask_words() > 0
    hipLaunchKernelGGL(level_masks ? flat_span_select_kernel<true> : flat_span_select_kernel<false>, dim3(SPAN_SELECT_BLOCKS), dim3(SW), 0, stream, r->dm, *lanes, base, count, sc);
    mark();
    hipLaunchKernelGGL(level_masks ? flat_tail_kernel<true> : flat_tail_kernel<false>, dim3(SW / 64, count), dim3(64 * tail_rows(level_masks)), 0, stream, r->dm, *lanes, base, count, sc);
    hipLaunchKernelGGL(flat_span_finish_kernel, dim3(count), dim3(SW), 0, stream, r->dm, *lanes, base, count, sc);
    // Billboards that simply cover what lies under them need not wait for the flat pass's pixels: the lanes that hold no other
    // kind (lane_blends, decided on the device) have theirs painted right after the shading, on the side stream, where they
    // mark the gap pixels they take; the flat pass's pixels of those lanes are painted after the join, around the marks.  The
    // flat chain, which waits for memory most of its time, then has the billboards beside it as well as the shading.  Lanes
    // with a billboard that blends with the pixel below (sprite_style) keep the order flat pass, then billboards; so do
    // frames with decals, which go between the two.
    const bool has_billboards = lanes->sprite_slots > 0 && lanes->sprite_x;
    const bool billboards_split = beside && has_billboards && !decals;
    const bool may_blend = lanes->sprite_style != nullptr;   // without styles no lane blends: the launches for such lanes are left out
    auto paint_billboards = [&](hipStream_t on, int lane_pick) {
        const size_t shared = (size_t)lanes->sprite_slots * (sizeof(SpriteRec) + sizeof(unsigned short));
        hipLaunchKernelGGL(sprite_columns_kernel, dim3((SW + SPRITE_COLUMNS - 1) / SPRITE_COLUMNS, count), dim3(SPRITE_COLUMNS * SPRITE_ROW_PARTS), shared, on, r->dm, *lanes, base, count, sc, frame_base, frame_stride, lane_pick);
    };
    if (!fused && !(billboards_split && !may_blend)) hipLaunchKernelGGL(flat_shade_kernel, dim3(count), dim3(128), 0, stream, r->dm, count, sc, frame_base, frame_stride, billboards_split ? LANES_BLENDING : LANES_ALL);
    if (beside) {
        shade_planes();
        if (billboards_split) paint_billboards(r->side_stream, LANES_PLAIN);
        HIP_TRY(hipEventRecord(r->join_event, r->side_stream));
        HIP_TRY(hipStreamWaitEvent(stream, r->join_event, 0));
        if (billboards_split) hipLaunchKernelGGL(flat_shade_kernel, dim3(count), dim3(128), 0, stream, r->dm, count, sc, frame_base, frame_stride, LANES_PLAIN);
    }
    mark();
    const float *blend = lanes->screen_blend ? lanes->screen_blend + 2 * (size_t)base : nullptr;
    if (fused) {
        FinishOut finish;
        finish.indexed = out->indexed ? out->indexed + (size_t)base * frame_stride : nullptr;
        finish.rgb = out->rgb ? out->rgb + (size_t)base * frame_stride * 3 : nullptr;
        finish.obs = out->obs ? out->obs + (size_t)base * F : nullptr;
        finish.frames = out->frames ? out->frames + (size_t)base * GD_FRAME_STACK * F : nullptr;
        finish.final_frames = out->final_frames ? out->final_frames + (size_t)base * GD_FRAME_STACK * F : nullptr;
        finish.reset_mask = out->reset_mask ? out->reset_mask + base : nullptr;
        finish.blend = blend;
        finish.stack_mode = out->stack_mode;
        finish.final_hwc = out->final_frames_layout == GD_LAYOUT_HWC;
        finish.source_rows = source_rows;
        const bool sprites = lanes->sprite_slots > 0 && lanes->sprite_x;
        size_t shared = sprites ? (size_t)lanes->sprite_slots * (sizeof(SpriteRec) + sizeof(unsigned short)) : 0;
        if (shared <= (size_t)LDS_SECTORS * sizeof(float4) + 32 * 256) shared = 0;   // the records reuse the shading tables' LDS
        hipLaunchKernelGGL(band_finish_kernel, dim3(BAND_COUNT, count), dim3(BAND_THREADS), shared, stream, r->dm, r->overlays, *lanes, base, count, sc, finish);
        mark();
        mark();
        HIP_TRY(hipGetLastError());
        return GD_OK;
    }
    if (decals)
        hipLaunchKernelGGL(decal_kernel, dim3(count), dim3(SW), 0, stream, r->dm, r->overlays, *lanes, base, count, sc, frame_base, frame_stride);
    if (has_billboards && !(billboards_split && !may_blend)) paint_billboards(stream, billboards_split ? LANES_BLENDING : LANES_ALL);
    if (lanes->weapon_state && r->overlays.d.weapon_patch_count > 0)
        hipLaunchKernelGGL(weapon_overlay_kernel, dim3((VH * SW + 255) / 256, count), dim3(256), 0, stream, r->overlays, lanes->weapon_state, base, count,
                           frame_base, frame_stride);
    if (lanes->hud_state && r->overlays.d.hud_patch_count > 0)
        hipLaunchKernelGGL(hud_kernel, dim3(count), dim3(256), 0, stream, r->overlays, lanes->hud_state, base, count, frame_base, frame_stride);
    mark();
    if (out->obs || out->frames) {
        hipLaunchKernelGGL(observe_kernel, dim3(GD_OBS_SIZE / OBS_BLOCK_ROWS, count), dim3(256), 0, stream,
                           frame_base, frame_stride, source_rows, m.playpal, count, out->obs ? out->obs + (size_t)base * F : nullptr,
                           out->frames ? out->frames + (size_t)base * GD_FRAME_STACK * F : nullptr,
                           out->reset_mask ? out->reset_mask + base : nullptr, out->stack_mode,
                           out->final_frames ? out->final_frames + (size_t)base * GD_FRAME_STACK * F : nullptr,
                           out->final_frames_layout == GD_LAYOUT_HWC, blend);
    }
    if (out->rgb) {
        size_t pixels = (size_t)count * frame_stride;
        static_assert((GD_SCREEN_HEIGHT * SW) % 256 == 0, "expand_rgb_kernel: one lane per block");
        hipLaunchKernelGGL(expand_rgb_kernel, dim3((unsigned)((pixels + 255) / 256)), dim3(256), 0, stream, frame_base, m.playpal, pixels,
                           out->rgb + (size_t)base * frame_stride * 3, blend, (size_t)GD_SCREEN_HEIGHT * SW);
    }
    mark();
    HIP_TRY(hipGetLastError());
    return GD_OK;
}

}  // namespace

extern "C" {

const char *gd_version(void) { return "gradoom_amd 0.2.0 (gfx950)"; }
uint32_t gd_abi_version(void) { return GD_ABI_VERSION; }
const char *gd_last_error(void) { return g_error.c_str(); }

int gd_renderer_create(const gd_map_desc *h, const float *cosine_correction, int32_t max_lanes, gd_renderer **out) {
    if (!h || !out || !cosine_correction) return fail(GD_E_ARG, "null argument");
    SIZE_CHECK(h, gd_map_desc);
    if (max_lanes < 0) return fail(GD_E_ARG, "max_lanes must not be negative");
    if (h->wall_count <= 0 || h->sector_count <= 0) return fail(GD_E_ARG, "empty map");
    if (h->wall_count >= 65535) return fail(GD_E_ARG, "at most 65534 linedefs");
    if (h->sector_count >= 8191) return fail(GD_E_ARG, "at most 8190 sectors");
    if (h->vertex_count >= 65536) return fail(GD_E_ARG, "at most 65535 distinct vertices");
    if (h->fine_nx <= 0 || h->fine_ny <= 0 || !(h->fine_cell > 0.0f) || !h->fine_sector) return fail(GD_E_ARG, "missing fine point-location raster");
    if (h->grid_cell != 8.0f * h->fine_cell || (h->fine_nx + 7) / 8 > h->grid_nx || (h->fine_ny + 7) / 8 > h->grid_ny)
        return fail(GD_E_ARG, "grid_cell must be 8 * fine_cell and the coarse grid must cover the fine raster");
    if (h->fragment_slots < 1 || h->split_count < 0 || h->split_count > h->wall_count || !h->wall_split_slot ||
        (h->split_count > 0 && (!h->split_fragments_fixed || !h->split_fragment_mask)))
        return fail(GD_E_ARG, "invalid projection fragment tables");
    for (int w = 0; w < h->wall_count; ++w)
        if (h->wall_split_slot[w] < -1 || h->wall_split_slot[w] >= h->split_count)
            return fail(GD_E_ARG, "wall_split_slot names a row outside the fragment tables");
    if (!h->additive_luts || !h->translucent_lut) return fail(GD_E_ARG, "missing sprite blend tables");
    if ((unsigned long long)h->texture_count * (unsigned long long)h->tex_max_h * (unsigned long long)h->tex_max_w >= (1ULL << 32))
        return fail(GD_E_ARG, "the texture atlas must stay below 4 GiB");
    if (int bad = validate_map(h)) return bad;
    gd_renderer *r = new (std::nothrow) gd_renderer();
    if (!r) return fail(GD_E_ARG, "out of host memory");
    r->events_ready = false;
    r->side_ready = false;
    r->scratch_block = nullptr; r->scratch_bytes = 0;
    r->assembly = GD_ASSEMBLY_AUTO;
    std::memset(&r->sc, 0, sizeof(r->sc));
    std::memset(&r->overlays, 0, sizeof(r->overlays));
    r->dm.d = *h;
    gd_map_desc &d = r->dm.d;
    const size_t W = h->wall_count, S = h->sector_count, V = h->vertex_count, K = h->neighbor_slots;
    int rc = GD_OK;
#define UP(field, count) if (rc == GD_OK) rc = upload(r, h->field, (size_t)(count), &d.field)
    UP(walls, W * 4); UP(walls_fixed, W * 4); UP(wall_sectors, W * 2); UP(wall_vertex, W * 2);
    UP(side_tex, W * 6); UP(side_off, W * 4); UP(wall_len, W);
    UP(endpoint_neighbors, W * K); UP(endpoint_neighbor_starts, W * K); UP(endpoint_neighbor_ends, W * K);
    UP(direct_neighbor_table, W * 4);
    UP(solid_bridge_start_ofs, W + 1); UP(solid_bridge_start_idx, h->solid_bridge_start_ofs[W]);
    UP(solid_bridge_end_ofs, W + 1); UP(solid_bridge_end_idx, h->solid_bridge_end_ofs[W]);
    UP(vertex_wall_ofs, V + 1); UP(vertex_wall_idx, h->vertex_wall_ofs[V]);
    UP(sector_wall_ofs, S + 1); UP(sector_wall_idx, h->sector_wall_ofs[S]);
    UP(sector_edge_ofs, S + 1); UP(sector_edge_idx, h->sector_edge_ofs[S]);
    UP(blocking_walls, h->blocking_count);
    {
        const size_t fragments = (size_t)(h->split_count > 0 ? h->split_count : 1) * h->fragment_slots;
        UP(wall_split_slot, W);
        if (h->split_count > 0) { UP(split_fragments_fixed, fragments * 4); UP(split_fragment_mask, fragments); }
        else { d.split_fragments_fixed = nullptr; d.split_fragment_mask = nullptr; }
    }
    const size_t cells = (size_t)h->grid_nx * h->grid_ny;
    const size_t items = h->grid_cell_ofs[cells];
    UP(grid_cell_ofs, cells + 1); UP(grid_item_sector, items); UP(grid_item_edge_ofs, items + 1);
    UP(grid_item_edges, h->grid_item_edge_ofs[items]);
    UP(fine_sector, (size_t)h->fine_nx * h->fine_ny);
    UP(floor_levels, h->floor_level_count); UP(ceil_levels, h->ceil_level_count);
    UP(sector_heights, S * 2); UP(sector_lights, S); UP(sector_floor_tex, S); UP(sector_ceil_tex, S);
    const size_t texels = (size_t)h->texture_count * h->tex_max_h * h->tex_max_w;
    UP(tex_atlas, texels); UP(tex_w, h->texture_count); UP(tex_h, h->texture_count);
    UP(playpal, 768); UP(colormap, 34 * 256);
    const size_t sprels = (size_t)h->sprite_count * h->spr_max_h * h->spr_max_w;
    UP(spr_atlas, sprels); UP(spr_opaque, sprels); UP(spr_post_top, sprels);
    UP(spr_w, h->sprite_count); UP(spr_h, h->sprite_count); UP(spr_left, h->sprite_count); UP(spr_top, h->sprite_count);
    UP(additive_luts, 2 * 256 * 256); UP(translucent_lut, 256 * 256);
#undef UP
    std::vector<i64> sine, tangent;
    build_fine_tables(sine, tangent);
    if (rc == GD_OK) rc = upload(r, sine.data(), sine.size(), &r->dm.fine_sine);
    if (rc == GD_OK) rc = upload(r, tangent.data(), tangent.size(), &r->dm.fine_tangent);
    if (rc == GD_OK) rc = upload(r, cosine_correction, (size_t)SW, &r->dm.cosine_correction);
    {
        std::vector<float> inverse(SW);
        for (int x = 0; x < SW; ++x) inverse[x] = 1.0f / cosine_correction[x];   // IEEE division, as on the device
        if (rc == GD_OK) rc = upload(r, inverse.data(), inverse.size(), &r->dm.inverse_cosine);
        for (int strip = 0; strip < SW / 64; ++strip) {
            float smallest = cosine_correction[strip * 64];
            for (int x = strip * 64; x < strip * 64 + 64; ++x) smallest = std::fmin(smallest, cosine_correction[x]);
            r->dm.strip_reach_scale[strip] = smallest > 0.0f ? 1.001f / smallest : GD_INF;
            float largest = cosine_correction[strip * 64];
            for (int x = strip * 64; x < strip * 64 + 64; ++x) largest = std::fmax(largest, cosine_correction[x]);
            r->dm.strip_far_scale[strip] = smallest > 0.0f && std::isfinite(largest) ? 0.999f / largest : 0.0f;
        }
        r->dm.fine_inverse = 1.0f / h->fine_cell;
    }
    {
        std::vector<int> box_ofs;
        std::vector<float4> boxes;
        build_level_boxes(h, box_ofs, boxes);
        if (rc == GD_OK) rc = upload(r, box_ofs.data(), box_ofs.size(), &r->dm.level_box_ofs);
        if (rc == GD_OK) rc = upload(r, boxes.data(), boxes.size(), &r->dm.level_boxes);
        std::vector<int> blocking_slot(W, -1);
        for (int b = 0; b < h->blocking_count; ++b) {
            const int w = h->blocking_walls[b];
            if (w < 0 || (size_t)w >= W) { if (rc == GD_OK) rc = fail(GD_E_ARG, "blocking_walls holds a linedef index out of range"); continue; }
            if (blocking_slot[w] < 0) blocking_slot[w] = b;   // the first slot wins ties, like the scan it replaces
        }
        if (rc == GD_OK) rc = upload(r, blocking_slot.data(), blocking_slot.size(), &r->dm.wall_blocking_slot);
        r->dm.sector_level = nullptr;
        std::vector<unsigned int> pairs(S, 0);
        bool listed = h->floor_level_count <= 65535 && h->ceil_level_count <= 65535;
        if (listed) {
            for (size_t s = 0; s < S; ++s) {
                int fi = -1, ci = -1;
                for (int l = 0; l < h->floor_level_count; ++l) if (h->floor_levels[l] == h->sector_heights[2 * s]) fi = l;
                for (int l = 0; l < h->ceil_level_count; ++l) if (h->ceil_levels[l] == h->sector_heights[2 * s + 1]) ci = l;
                listed = listed && fi >= 0 && ci >= 0;
                pairs[s] = ((unsigned)fi & 0xFFFFu) | (((unsigned)ci & 0xFFFFu) << 16);
            }
            // a sector whose height is missing from the level lists keeps the per-pixel divisions
            if (listed && rc == GD_OK) rc = upload(r, pairs.data(), pairs.size(), &r->dm.sector_level);
        }
        std::vector<int2> cell_range(cells);
        std::vector<int4> cell_item(items);
        std::vector<float4> cell_edge;
        for (size_t c = 0; c < cells; ++c) cell_range[c] = make_int2(h->grid_cell_ofs[c], h->grid_cell_ofs[c + 1]);
        for (size_t it = 0; it < items; ++it) {
            const int entry = h->grid_item_sector[it];
            const size_t s = (size_t)(entry & ~GRID_ALWAYS_INSIDE);
            if (s >= S) { if (rc == GD_OK) rc = fail(GD_E_ARG, "grid_item_sector holds a sector index out of range"); continue; }
            const int first = (int)cell_edge.size();
            for (int k = h->grid_item_edge_ofs[it]; k < h->grid_item_edge_ofs[it + 1]; ++k) {
                const int w = h->grid_item_edges[k];
                if (w < 0 || (size_t)w >= W) { if (rc == GD_OK) rc = fail(GD_E_ARG, "grid_item_edges holds a linedef index out of range"); continue; }
                cell_edge.push_back(make_float4(h->walls[4 * w], h->walls[4 * w + 1], h->walls[4 * w + 2], h->walls[4 * w + 3]));
            }
            // .y: the sector's level indices (as in sector_level), or negative: compare heights (also when the ceiling
            // index would reach the sign bit)
            cell_item[it] = make_int4(entry, listed ? (int)pairs[s] : -1, first, (int)cell_edge.size());
        }
        if (rc == GD_OK) rc = upload(r, cell_range.data(), cell_range.size(), &r->dm.cell_range);
        if (rc == GD_OK) rc = upload(r, cell_item.data(), cell_item.size(), &r->dm.cell_item);
        if (rc == GD_OK) rc = upload(r, cell_edge.data(), cell_edge.size(), &r->dm.cell_edge);
    }
    // Working memory for one chunk of lanes; larger batches are rendered chunk by chunk.  A renderer made for no
    // lanes holds the map only and renders through gd_render_static.
    const int chunk = max_lanes < 4096 ? max_lanes : 4096;
    r->chunk_lanes = chunk;
    Scratch &sc = r->sc;
    if (rc == GD_OK && chunk > 0) {
        unsigned char *block = nullptr;
        const size_t bytes = carve_scratch(sc, nullptr, (size_t)chunk, *h, false, spill_pool_blocks(chunk));
        rc = scratch_alloc(r, bytes, &block);
        if (rc == GD_OK) {
            carve_scratch(sc, block, (size_t)chunk, *h, false, spill_pool_blocks(chunk));
            r->scratch_block = block; r->scratch_bytes = bytes;
        }
    }
    if (rc == GD_OK) rc = scratch_alloc(r, 1, &sc.status);
    if (rc == GD_OK && hipMemset(sc.status, 0, sizeof(int)) != hipSuccess) rc = fail(GD_E_HIP, "hipMemset status");
    if (rc == GD_OK) rc = static_scratch_address(nullptr);   // looked up once per device, outside any stream capture
    if (rc == GD_OK) {
        for (int i = 0; i < 16; ++i) if (hipEventCreate(&r->events[i]) != hipSuccess) rc = fail(GD_E_HIP, "hipEventCreate");
        r->events_ready = rc == GD_OK;
    }
    if (rc == GD_OK) {
        // default priority, like the caller's stream; no implicit synchronisation with the null stream
        if (hipStreamCreateWithFlags(&r->side_stream, hipStreamNonBlocking) != hipSuccess) rc = fail(GD_E_HIP, "hipStreamCreateWithFlags");
        else if (hipEventCreateWithFlags(&r->fork_event, hipEventDisableTiming) != hipSuccess) { (void)hipStreamDestroy(r->side_stream); rc = fail(GD_E_HIP, "hipEventCreateWithFlags"); }
        else if (hipEventCreateWithFlags(&r->join_event, hipEventDisableTiming) != hipSuccess) {
            (void)hipEventDestroy(r->fork_event); (void)hipStreamDestroy(r->side_stream); rc = fail(GD_E_HIP, "hipEventCreateWithFlags");
        } else r->side_ready = true;
    }
    if (rc != GD_OK) { std::string keep = g_error; gd_renderer_destroy(r); g_error = keep; return rc; }
    *out = r;
    return GD_OK;
}

void gd_renderer_destroy(gd_renderer *r) {
    if (!r) return;
    for (void *ptr : r->allocations) (void)hipFree(ptr);
    for (void *ptr : r->overlay_allocations) (void)hipFree(ptr);
    if (r->events_ready) for (int i = 0; i < 16; ++i) (void)hipEventDestroy(r->events[i]);
    if (r->side_ready) { (void)hipEventDestroy(r->fork_event); (void)hipEventDestroy(r->join_event); (void)hipStreamDestroy(r->side_stream); }
    delete r;
}

static int check_render_args(gd_renderer *r, const gd_lanes_desc *lanes, const gd_frame_out *out) {
    if (!r || !lanes || !out) return fail(GD_E_ARG, "null argument");
    SIZE_CHECK(lanes, gd_lanes_desc);
    SIZE_CHECK(out, gd_frame_out);
    if (out->obs_source_rows != 0 && out->obs_source_rows != VH && out->obs_source_rows != GD_SCREEN_HEIGHT)
        return fail(GD_E_ARG, "obs_source_rows must be 208 (or 0) or 240");
    if (lanes->lane_count < 0) return fail(GD_E_ARG, "negative lane count");
    // an empty batch is a call that does nothing: its tensors hold no element and may have no address
    if (lanes->lane_count > 0 && (!lanes->x || !lanes->y || !lanes->angle || !lanes->view_z || !lanes->x_fixed || !lanes->y_fixed ||
                                  !lanes->angle_bam || !lanes->pitch_bam || !lanes->ray_cos || !lanes->ray_sin))
        return fail(GD_E_ARG, "missing lane tensor");
    if (out->stack_mode != GD_STACK_STEP && out->stack_mode != GD_STACK_RESET) return fail(GD_E_ARG, "unknown stack_mode");
    if (lanes->sprite_slots < 0 || lanes->sprite_slots > 512) return fail(GD_E_ARG, "sprite_slots must be in [0, 512]");
    if (lanes->decal_slots < 0) return fail(GD_E_ARG, "negative decal_slots");
    if (lanes->decal_slots > 0 && (lanes->decal_state != nullptr) != (lanes->decal_geom != nullptr))
        return fail(GD_E_ARG, "decal_state and decal_geom go together");
    if (lanes->sprite_slots > 0 && lanes->sprite_x &&
        (!lanes->sprite_y || !lanes->sprite_z || !lanes->sprite_depth || !lanes->sprite_id || !lanes->sprite_alive))
        return fail(GD_E_ARG, "missing sprite tensor");
    return GD_OK;
}

int gd_render(gd_renderer *r, const gd_lanes_desc *lanes, const gd_frame_out *out, void *stream) {
    int rc = check_render_args(r, lanes, out);
    if (rc != GD_OK) return rc;
    if (r->chunk_lanes <= 0) return fail(GD_E_ARG, "this renderer was created for 0 lanes and holds no working memory: use gd_render_static");
    hipStream_t caller = static_cast<hipStream_t>(stream);
    for (int base = 0; base < lanes->lane_count; base += r->chunk_lanes) {
        int count = lanes->lane_count - base < r->chunk_lanes ? lanes->lane_count - base : r->chunk_lanes;
        rc = launch_chunk(r, r->sc, lanes, out, base, count, caller, false);
        if (rc != GD_OK) return rc;
    }
    return GD_OK;
}

int gd_render_static(gd_renderer *r, const gd_lanes_desc *lanes, const gd_frame_out *out, void *stream) {
    int rc = check_render_args(r, lanes, out);
    if (rc != GD_OK) return rc;
    unsigned char *block = nullptr;
    rc = static_scratch_address(&block);
    if (rc != GD_OK) return rc;
    const gd_map_desc &m = r->dm.d;
    const bool decals = lanes->decal_slots > 0 && lanes->decal_state && lanes->decal_geom && r->overlays.d.decal_variant_count > 0;
    Scratch sc = r->sc;   // keeps the renderer's status word
    const size_t one = carve_scratch(sc, nullptr, 1, m, decals, STATIC_SPILL_BLOCKS), two = carve_scratch(sc, nullptr, 2, m, decals, STATIC_SPILL_BLOCKS);
    if (one > STATIC_SCRATCH_BYTES)
        return fail(GD_E_ARG, "map too large for gd_render_static: one lane needs " + std::to_string(one) + " bytes of working memory, the static block holds " +
                                  std::to_string(STATIC_SCRATCH_BYTES));
    // the layout grows by a fixed amount per lane, up to the padding between its buffers
    size_t fit = 1 + (STATIC_SCRATCH_BYTES - one) / (two - one);
    while (fit > 1 && carve_scratch(sc, nullptr, fit, m, decals, STATIC_SPILL_BLOCKS) > STATIC_SCRATCH_BYTES) --fit;
    const int chunk = fit > 4096 ? 4096 : (int)fit;
    if (lanes->lane_count > GD_STATIC_MAX_LANES)
        return fail(GD_E_ARG, "gd_render_static renders at most " + std::to_string(GD_STATIC_MAX_LANES) + " lanes per call");
    carve_scratch(sc, block, (size_t)chunk, m, decals, STATIC_SPILL_BLOCKS);
    hipStream_t caller = static_cast<hipStream_t>(stream);
    // the block keeps whatever the last call left: the kernels expect nothing of it
    for (int base = 0; base < lanes->lane_count; base += chunk) {
        const int count = lanes->lane_count - base < chunk ? lanes->lane_count - base : chunk;
        rc = launch_chunk(r, sc, lanes, out, base, count, caller, false);
        if (rc != GD_OK) return rc;
    }
    return GD_OK;
}

int gd_render_timed(gd_renderer *r, const gd_lanes_desc *lanes, const gd_frame_out *out, void *stream, int32_t launches, float *ms, int32_t stage_count) {
    int rc = check_render_args(r, lanes, out);
    if (rc != GD_OK) return rc;
    if (r->chunk_lanes <= 0) return fail(GD_E_ARG, "this renderer was created for 0 lanes and holds no working memory");
    if (!ms || stage_count < STAGE_COUNT - 1 || launches <= 0) return fail(GD_E_ARG, "ms must hold 8 stage times");
    for (int s = 0; s < stage_count; ++s) ms[s] = 0.0f;
    hipStream_t st = static_cast<hipStream_t>(stream);
    for (int it = 0; it < launches; ++it) {
        for (int base = 0; base < lanes->lane_count; base += r->chunk_lanes) {
            int count = lanes->lane_count - base < r->chunk_lanes ? lanes->lane_count - base : r->chunk_lanes;
            rc = launch_chunk(r, r->sc, lanes, out, base, count, st, true);
            if (rc != GD_OK) return rc;
            HIP_TRY(hipEventSynchronize(r->events[STAGE_COUNT - 1]));
            for (int s = 0; s + 1 < STAGE_COUNT; ++s) {
                float t = 0.0f;
                HIP_TRY(hipEventElapsedTime(&t, r->events[s], r->events[s + 1]));
                ms[s] += t;
            }
        }
    }
    for (int s = 0; s + 1 < STAGE_COUNT; ++s) ms[s] /= (float)launches;
    return GD_OK;
}

/* Sticky status bits of the renderer (synchronises the device): bit0 = a column had more than
   CAND_MAX candidate linedefs and its list was truncated. Replaces nothing in the reference. */
int gd_renderer_status(gd_renderer *r, int32_t *status) {
    if (!r || !status) return fail(GD_E_ARG, "null argument");
    int value = 0;
    HIP_TRY(hipMemcpy(&value, r->sc.status, sizeof(int), hipMemcpyDeviceToHost));
    *status = value;
    return GD_OK;
}

/* Fill the renderer's working memory with one byte value.
   Frames must not depend on what that memory held; this lets a caller check it.  Replaces nothing in the reference. */
int gd_renderer_scribble(gd_renderer *r, int32_t value, void *stream) {
    if (!r) return fail(GD_E_ARG, "null argument");
    if (!r->scratch_block) return GD_OK;
    hipStream_t st = static_cast<hipStream_t>(stream);
    const unsigned int byte = (unsigned int)value & 0xFFu, word = byte * 0x01010101u;
    hipLaunchKernelGGL(fill_words_kernel, dim3(4096), dim3(256), 0, st, reinterpret_cast<unsigned int *>(r->scratch_block), r->scratch_bytes / 4, word);
    HIP_TRY(hipGetLastError());
    return GD_OK;
}

int gd_renderer_set_assembly(gd_renderer *r, int32_t assembly) {
    if (!r) return fail(GD_E_ARG, "null argument");
    if (assembly != GD_ASSEMBLY_AUTO && assembly != GD_ASSEMBLY_FUSED && assembly != GD_ASSEMBLY_SEPARATE) return fail(GD_E_ARG, "unknown assembly");
    r->assembly = assembly;
    return GD_OK;
}

int gd_renderer_set_overlays(gd_renderer *r, const gd_overlay_desc *h) {
    if (!r || !h) return fail(GD_E_ARG, "null argument");
    SIZE_CHECK(h, gd_overlay_desc);
    if (h->weapon_patch_count < 0 || h->hud_patch_count < 0 || h->weapon_max_h < 0 || h->weapon_max_w < 0 || h->hud_max_h < 0 || h->hud_max_w < 0)
        return fail(GD_E_ARG, "negative overlay size");
    if (h->weapon_patch_count > 0 && (!h->weapon_atlas || !h->weapon_opaque || !h->weapon_w || !h->weapon_h || !h->weapon_left || !h->weapon_top))
        return fail(GD_E_ARG, "missing weapon patch array");
    if (h->decal_variant_count != 0 &&
        (h->decal_variant_count != 5 || h->decal_max_h <= 0 || h->decal_max_w <= 0 || h->decal_black_rows <= 0 || !h->decal_atlas ||
         !h->decal_h || !h->decal_left || !h->decal_top || !h->decal_opacity_lut || !h->decal_black_lut))
        return fail(GD_E_ARG, "decal patches need 5 variants, their sizes and both tables");
    if (h->decal_variant_count == 5) {
        for (int v = 0; v < 5; ++v)
            if (h->decal_h[v] < 0 || h->decal_h[v] > h->decal_max_h) return fail(GD_E_ARG, "decal height outside the atlas");
        for (int k = 0; k < 32 * 256; ++k)
            if (h->decal_opacity_lut[k] >= h->decal_black_rows) return fail(GD_E_ARG, "decal_opacity_lut names a row outside decal_black_lut");
    }
    if (h->hud_patch_count > 0 && (!h->hud_atlas || !h->hud_opaque || !h->hud_w || !h->hud_h || !h->hud_left || !h->hud_top))
        return fail(GD_E_ARG, "missing status bar patch array");
    HIP_TRY(hipDeviceSynchronize());              // no frame may still be reading the old patches
    for (void *ptr : r->overlay_allocations) (void)hipFree(ptr);
    r->overlay_allocations.clear();
    std::memset(&r->overlays, 0, sizeof(r->overlays));
    gd_overlay_desc d = *h;
    auto copy = [&](const void *host, size_t bytes, const void **device) -> int {
        void *ptr = nullptr;
        HIP_TRY(hipMalloc(&ptr, bytes ? bytes : 1));
        r->overlay_allocations.push_back(ptr);
        if (bytes) HIP_TRY(hipMemcpy(ptr, host, bytes, hipMemcpyHostToDevice));
        *device = ptr;
        return GD_OK;
    };
    int rc = GD_OK;
    const size_t wp = h->weapon_patch_count, wt = wp * h->weapon_max_h * h->weapon_max_w;
    const size_t hp = h->hud_patch_count, ht = hp * h->hud_max_h * h->hud_max_w;
#define OV(field, bytes) if (rc == GD_OK) rc = copy(h->field, (bytes), reinterpret_cast<const void **>(&d.field))
    OV(weapon_atlas, wt); OV(weapon_opaque, wt); OV(weapon_w, wp * 4); OV(weapon_h, wp * 4); OV(weapon_left, wp * 4); OV(weapon_top, wp * 4);
    OV(hud_atlas, ht); OV(hud_opaque, ht); OV(hud_w, hp * 4); OV(hud_h, hp * 4); OV(hud_left, hp * 4); OV(hud_top, hp * 4);
    r->sc.scene_depth = nullptr;
    if (h->decal_variant_count == 5) {
        OV(decal_atlas, (size_t)5 * h->decal_max_h * h->decal_max_w); OV(decal_h, 5 * 4); OV(decal_left, 5 * 4); OV(decal_top, 5 * 4);
        OV(decal_opacity_lut, 32 * 256); OV(decal_black_lut, (size_t)h->decal_black_rows * 256);
        if (rc == GD_OK) {   // the depth buffer decals test against, for one chunk of lanes
            void *ptr = nullptr;
            if (hipMalloc(&ptr, (size_t)(r->chunk_lanes > 0 ? r->chunk_lanes : 1) * VH * SW * sizeof(float)) != hipSuccess) rc = fail(GD_E_HIP, "out of device memory for the decal depth buffer");
            else { r->overlay_allocations.push_back(ptr); r->sc.scene_depth = static_cast<float *>(ptr); }
        }
    }
#undef OV
    if (rc != GD_OK) {
        for (void *ptr : r->overlay_allocations) (void)hipFree(ptr);
        r->overlay_allocations.clear();
        r->sc.scene_depth = nullptr;
        return rc;
    }
    r->overlays.d = d;
    return GD_OK;
}

int gd_renderer_set_sector_lights(gd_renderer *r, const float *lights, void *stream) {
    if (!r || !lights) return fail(GD_E_ARG, "null argument");
    HIP_TRY(hipMemcpyAsync(const_cast<float *>(r->dm.d.sector_lights), lights, (size_t)r->dm.d.sector_count * sizeof(float),
                           hipMemcpyDeviceToDevice, static_cast<hipStream_t>(stream)));
    return GD_OK;
}


int gd_observe(const uint8_t *indexed, int32_t source_rows, const uint8_t *playpal, int32_t lane_count,
               uint8_t *obs, uint8_t *frames, const uint8_t *reset_mask, int32_t stack_mode, void *stream) {
    if (stack_mode != GD_STACK_STEP && stack_mode != GD_STACK_RESET) return fail(GD_E_ARG, "unknown stack_mode");
    if (source_rows != 208 && source_rows != 240) return fail(GD_E_ARG, "indexed must have 208 or 240 rows");
    if (lane_count < 0) return fail(GD_E_ARG, "negative lane count");
    if (lane_count == 0) return GD_OK;    // an empty batch: its tensors may have no address
    if (!indexed || !playpal) return fail(GD_E_ARG, "null argument");
    if (!obs && !frames) return GD_OK;
    for (int base = 0; base < lane_count; base += 32768) {
        int count = lane_count - base < 32768 ? lane_count - base : 32768;
        const size_t F = (size_t)GD_OBS_SIZE * GD_OBS_SIZE;
        hipLaunchKernelGGL(observe_kernel, dim3(GD_OBS_SIZE / OBS_BLOCK_ROWS, count), dim3(256), 0, static_cast<hipStream_t>(stream),
                           indexed + (size_t)base * source_rows * SW, (size_t)source_rows * SW, source_rows, playpal, count,
                           obs ? obs + (size_t)base * F : nullptr, frames ? frames + (size_t)base * GD_FRAME_STACK * F : nullptr,
                           reset_mask ? reset_mask + base : nullptr, stack_mode, nullptr, false, nullptr);
    }
    HIP_TRY(hipGetLastError());
    return GD_OK;
}

int gd_expand_rgb24(const uint8_t *indexed, int32_t rows, const uint8_t *playpal, int32_t lane_count, uint8_t *rgb, void *stream) {
    if (rows <= 0 || lane_count < 0) return fail(GD_E_ARG, "bad shape");
    size_t pixels = (size_t)lane_count * rows * SW;
    if (pixels == 0) return GD_OK;        // an empty batch: its tensors may have no address
    if (!indexed || !playpal || !rgb) return fail(GD_E_ARG, "null argument");
    const size_t step = (size_t)1 << 30;
    for (size_t base = 0; base < pixels; base += step) {
        size_t count = pixels - base < step ? pixels - base : step;
        hipLaunchKernelGGL(expand_rgb_kernel, dim3((unsigned)((count + 255) / 256)), dim3(256), 0, static_cast<hipStream_t>(stream),
                           indexed + base, playpal, count, rgb + base * 3, nullptr, (size_t)1);
    }
    HIP_TRY(hipGetLastError());
    return GD_OK;
}

int gd_pack_actors(const gd_actor_desc *a, void *stream) {
    if (!a) return fail(GD_E_ARG, "null argument");
    SIZE_CHECK(a, gd_actor_desc);
    const int32_t counts[] = {a->lane_count, a->enemy_slots, a->doll_count, a->player_projectile_slots, a->enemy_projectile_slots,
                              a->fog_slots, a->puff_slots, a->item_count, a->drop_slots};
    for (int32_t v : counts) if (v < 0) return fail(GD_E_ARG, "negative count");
    if (a->attack_frames < 3 || a->death_frames < 1 || a->xdeath_frames < 1 || a->explosion_frames < 1)
        return fail(GD_E_ARG, "animation tables need at least 3 attack frames and 1 frame of every other kind");
    // every pointer of the descriptor sits between the scalars and the end of the struct
    const void *const *first = reinterpret_cast<const void *const *>(&a->enemy_x);
    const void *const *last = reinterpret_cast<const void *const *>(&a->sprite_style);
    for (const void *const *p = first; p <= last; ++p) {
        const bool doll = p >= reinterpret_cast<const void *const *>(&a->doll_x) && p <= reinterpret_cast<const void *const *>(&a->doll_rotation);
        const bool item = p >= reinterpret_cast<const void *const *>(&a->item_x) && p <= reinterpret_cast<const void *const *>(&a->item_animation_initial_tics);
        if (!*p && !(doll && a->doll_count == 0) && !(item && a->item_count == 0)) return fail(GD_E_ARG, "null tensor in gd_actor_desc");
    }
    const long long width = 2LL * a->enemy_slots + a->doll_count + 2LL * a->player_projectile_slots + 2LL * a->enemy_projectile_slots +
                            a->fog_slots + a->puff_slots + a->item_count + a->drop_slots;
    if (a->lane_count == 0 || width == 0) return GD_OK;
    if (width > 65535 * 64LL || a->lane_count > 65535) return fail(GD_E_ARG, "too many slots or lanes for one launch");
    hipLaunchKernelGGL(pack_actors_kernel, dim3((unsigned)((width + 63) / 64), (unsigned)a->lane_count), dim3(64), 0,
                       static_cast<hipStream_t>(stream), *a, (int)width);
    HIP_TRY(hipGetLastError());
    return GD_OK;
}

int gd_pack_weapon(const gd_weapon_desc *w, void *stream) {
    if (!w) return fail(GD_E_ARG, "null argument");
    SIZE_CHECK(w, gd_weapon_desc);
    if (w->lane_count < 0 || w->cooldown_slots <= 0) return fail(GD_E_ARG, "gd_weapon_desc holds a count out of range");
    const void *const needed[] = {w->active_weapon, w->weapon_state_cooldown, w->weapon_fire_count, w->weapon_ready_tics, w->weapon_lower_cooldown,
                                  w->weapon_raise_cooldown, w->pending_weapon, w->episode_time, w->player_bob_fixed, w->player_dead,
                                  w->weapon_frame_ids, w->weapon_flash_ids, w->fine_sine, w->weapon_state};
    for (const void *p : needed) if (!p) return fail(GD_E_ARG, "null tensor in gd_weapon_desc");
    if (w->flash_light && !w->weapon_flash_lights) return fail(GD_E_ARG, "flash_light needs weapon_flash_lights");
    if (w->lane_count == 0) return GD_OK;
    hipLaunchKernelGGL(pack_weapon_kernel, dim3((unsigned)((w->lane_count + 63) / 64)), dim3(64), 0, static_cast<hipStream_t>(stream), *w);
    HIP_TRY(hipGetLastError());
    return GD_OK;
}

}  // extern "C"
