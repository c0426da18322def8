// CPU oracle: a scalar, literal restatement of the reference's Torch "reference"
// render path and observation pipeline, one lane at a time.
//
// TEST INFRASTRUCTURE ONLY.  Only tests/, __graft_entry__.smoke() and the
// cpu_baseline leg of bench.py may load this library; the shipped HIP path never
// links, loads or calls it.
//
// Every function cites the lines of /root/reference/src/gradoom/engine.py it
// follows.  Dense [N,320,W] tensor expressions of the reference become loops
// over linedefs for one (lane, column); `torch.min(dim)` becomes a scan that
// keeps the FIRST minimal index; int64 arithmetic wraps like Torch's; float32
// expressions are evaluated one rounded operation at a time (compile with
// -ffp-contract=off).
//
// Pinned against golden vectors produced by the reference itself on seeded
// synthetic maps (tests/golden/*.npz); functions without such a pin are listed
// in the header of each section as "parity unpinned".
//
// Linedefs may carry BSP projection fragments (engine.py:745-767, 11472-11545) and textures may have
// any size: wall columns wrap modulo the width, rows and flats modulo 2^floor(log2(size))
// (engine.py:10888, 12792-12843), both as in the reference and both covered by golden cases.

#include "../include/gradoom_amd.h"

#include <algorithm>
#include <chrono>
#include <cstdio>
#include <cstdlib>
#include <cmath>
#include <cstdint>
#include <cstring>
#include <limits>
#include <mutex>
#include <string>
#include <thread>
#include <vector>

namespace {

typedef int64_t i64;
typedef uint64_t u64;

const float INF = std::numeric_limits<float>::infinity();
const int SW = GD_SCREEN_WIDTH;   // 320
const int VH = GD_VIEW_HEIGHT;    // 208

// engine.py:42-51, 139-156
const i64 FIXED_UNIT = 1 << 16;
const i64 UINT32_MASK = (i64(1) << 32) - 1;
const int FINE_ANGLES = 8192;
const i64 ANGLE_90 = i64(1) << 30;
const int ANGLE_TO_FINE_SHIFT = 19;
const i64 FOCAL_X_FIXED = 160 * FIXED_UNIT;
const i64 Y_ASPECT_FIXED = (i64(320) * FIXED_UNIT * 240) / (200 * 320);
const i64 FOCAL_Y_FIXED = 160 * Y_ASPECT_FIXED;
const i64 FLOOR_VISIBILITY_FIXED = (160 * FIXED_UNIT * (8 * FIXED_UNIT)) / FOCAL_Y_FIXED;
const i64 WALL_VISIBILITY_FIXED = ((FOCAL_Y_FIXED * (320 * 600) / (320 * 240 * 3)) * (8 * FIXED_UNIT)) >> 16;
const i64 SPRITE_MIN_DEPTH_FIXED = 2048 * 4;
const float SHARED_ENDPOINT_DEPTH_TOLERANCE = 1.0f / 16.0f;
const float PROJECTED_OWNER_MAX_WALL_LENGTH = 32.0f;
const float BAM_TO_RADIANS = float(2.0 * M_PI / 4294967296.0);

i64 g_fine_sine[FINE_ANGLES];
i64 g_fine_tangent[FINE_ANGLES / 2];
std::once_flag g_tables_once;

// engine.py:309-328 (ZDoom R_InitTables)
void fill_tables() {
    const int quarter = FINE_ANGLES / 4;
    for (int i = 0; i < quarter; ++i) {
        double phase = double(i) * (2.0 * M_PI / FINE_ANGLES);
        g_fine_sine[i] = (i64)std::trunc(std::sin(phase) * double(FIXED_UNIT));
    }
    for (int i = 0; i < quarter; ++i) g_fine_sine[quarter + i] = g_fine_sine[quarter - 1 - i];
    for (int i = 0; i < 2 * quarter; ++i) g_fine_sine[2 * quarter + i] = -g_fine_sine[i];
    g_fine_sine[quarter] = FIXED_UNIT;
    g_fine_sine[3 * quarter] = -FIXED_UNIT;
    const int half = FINE_ANGLES / 2;
    for (int i = 0; i < half; ++i) {
        double phase = (double(i) - FINE_ANGLES / 4) * (2.0 * M_PI / FINE_ANGLES);
        if (i == 0) phase += M_PI / FINE_ANGLES;
        g_fine_tangent[i] = (i64)std::trunc(std::tan(phase) * double(FIXED_UNIT) + 0.5);
    }
}
void build_tables() { std::call_once(g_tables_once, fill_tables); }

inline i64 mul64(i64 a, i64 b) { return (i64)((u64)a * (u64)b); }
inline i64 shl64(i64 a, int s) { return (i64)((u64)a << s); }
inline i64 tdiv(i64 a, i64 b) { return a / b; }  // engine.py:3115-3118, C truncation
inline i64 clampi(i64 v, i64 lo, i64 hi) { return v < lo ? lo : (v > hi ? hi : v); }
inline i64 round_to_i64(float v) { return (i64)std::nearbyintf(v); }  // torch.round(...).to(int64)
inline i64 f64_to_i64(double v) {
    // x86 cvttsd2si semantics, which Torch's CPU cast inherits: out of range -> INT64_MIN
    if (!(v >= -9223372036854775808.0 && v < 9223372036854775808.0)) return std::numeric_limits<i64>::min();
    return (i64)v;
}
inline int ilog2(int v) { int b = 0; while ((1 << (b + 1)) <= v) ++b; return b; }

// Rule coverage counters (how often each ownership rule fired), reported through gdo_coverage.
enum {
    COV_PASSES, COV_VALID, COV_EQUAL_DEPTH_SOLID, COV_PROJECTED_SOLID, COV_SOLID_BRIDGE, COV_ENDPOINT_OWNER, COV_NEAR_PROJECTED,
    COV_TOPOLOGICAL_OWNER, COV_SECTOR_BRIDGE, COV_OPPOSING_BOUNDARY, COV_EXCLUDED_RIGHT_EDGE, COV_CONTINUES_OWNER_BOUNDARY,
    COV_FORWARD_BRIDGE, COV_COMPLETES_ENDPOINT_BRIDGE, COV_ENDPOINT_ONLY_PORTAL, COV_TIED_STRIP, COV_ENTERS_OTHER, COV_ENTERS_SHARED,
    COV_GEOMETRIC_PATH, COV_PORTAL_BRIDGE, COV_COMPLETES_PORTAL_BRIDGE, COV_PS_KEEPS_PATH, COV_NO_KEEPS_PATH, COV_BOTTOM_TAIL,
    COV_MASKED_COLUMN, COV_MASKED_EXTENDS, COV_DEAD_COLUMN_REVIVED, COV_COUNT
};
thread_local long long g_coverage[COV_COUNT];   // per thread: lanes may be rendered by several threads at once
#define COVER(name, cond) do { if (cond) ++g_coverage[name]; } while (0)

struct Lane {
    float x, y, angle, view_z;
    i64 view_x_fixed, view_y_fixed, angle_bam, pitch_bam, flash_light;
    int fine;
    i64 vsin, vcos;        // fixed
    float fsin, fcos;      // float (engine.py:2167-2179)
    i64 center_fixed;      // (104<<16) + pitch offset (engine.py:12384-12391)
    float pitch_offset;    // engine.py:9622-9631
    int sector;
};

struct WallGeom {  // FWallCoords of one linedef for one lane (engine.py:10747-10869)
    i64 sl, sr, dl, dr;
};

struct WallVis {   // wallscan light interpolation, per side (engine.py:11217-11291)
    i64 light_left, light_step, screen_left;
};

struct Oracle {
    const gd_map_desc *m;
    int W, S;
    std::vector<uint8_t> one_sided;
    std::vector<i64> wall_len_fixed;
    // direct endpoint neighbours (engine.py:1548-1577)
    std::vector<int> start_nb, end_nb, start_slot, end_slot;
    std::vector<uint8_t> has_start, has_end;

    // per-lane
    Lane L;
    std::vector<WallGeom> geom;
    std::vector<WallVis> vis;      // [W][2]
    std::vector<i64> tx, ty;       // [W][2] view coordinates (engine.py:11173-11205)
    // BSP projection fragments of split linedefs (engine.py:11472-11545): FWallCoords and wallscan light
    std::vector<WallGeom> frag_geom;  // [SP][F]
    std::vector<WallVis> frag_vis;    // [SP][F][2]
    std::vector<uint8_t> front_facing_f32;  // engine.py:11376-11381
    std::vector<float> dist, along;        // [320][W]
    std::vector<uint8_t> geo, proj, ledge; // [320][W]
    std::vector<i64> hoff, vstep;          // [320][W] PrepWall
    std::vector<uint8_t> subpixel_two_sided;
    float dirx[SW], diry[SW];

    // per-lane pixel buffers [VH][SW]
    std::vector<uint8_t> frame, filled, plane_is_floor;
    std::vector<int> plane_sector, sprite_clip_wall, flat_sector;
    std::vector<float> surface_depth, scene_surface_depth, scene_depth, sprite_clip_depth;

    std::string error;

    explicit Oracle(const gd_map_desc *map) : m(map), W(map->wall_count), S(map->sector_count) {
        build_tables();
        one_sided.resize(W);
        wall_len_fixed.resize(W);
        for (int w = 0; w < W; ++w) {
            one_sided[w] = m->wall_sectors[2 * w + 1] < 0;
            wall_len_fixed[w] = round_to_i64(m->wall_len[w] * float(FIXED_UNIT));
        }
        const int K = m->neighbor_slots;
        start_nb.resize(W); end_nb.resize(W); start_slot.resize(W); end_slot.resize(W);
        has_start.resize(W); has_end.resize(W);
        for (int w = 0; w < W; ++w) {
            int ss = 0, es = 0, sc = 0, ec = 0;
            for (int k = K - 1; k >= 0; --k) {
                if (m->endpoint_neighbor_starts[w * K + k]) { ss = k; ++sc; }
                if (m->endpoint_neighbor_ends[w * K + k]) { es = k; ++ec; }
            }
            start_slot[w] = ss; end_slot[w] = es;
            start_nb[w] = m->endpoint_neighbors[w * K + ss];
            end_nb[w] = m->endpoint_neighbors[w * K + es];
            has_start[w] = sc > 0; has_end[w] = ec > 0;
        }
        geom.resize(W); vis.resize(2 * W); tx.resize(2 * W); ty.resize(2 * W);
        frag_geom.resize(size_t(m->split_count) * m->fragment_slots);
        frag_vis.resize(2 * size_t(m->split_count) * m->fragment_slots);
        front_facing_f32.resize(W); subpixel_two_sided.resize(W);
        dist.resize(size_t(SW) * W); along.resize(size_t(SW) * W);
        geo.resize(size_t(SW) * W); proj.resize(size_t(SW) * W); ledge.resize(size_t(SW) * W);
        hoff.resize(size_t(SW) * W); vstep.resize(size_t(SW) * W);
        const size_t px = size_t(VH) * SW;
        frame.resize(px); filled.resize(px); plane_is_floor.resize(px);
        plane_sector.resize(px); sprite_clip_wall.resize(px); flat_sector.resize(px);
        surface_depth.resize(px); scene_surface_depth.resize(px); scene_depth.resize(px);
        sprite_clip_depth.resize(px);
    }

    // ------------------------------------------------------------------ map relations
    int sec(int w, int side) const { return m->wall_sectors[2 * w + side]; }
    int vert(int w, int slot) const { return m->wall_vertex[2 * w + slot]; }
    bool two_sided_distinct(int w) const { return sec(w, 0) >= 0 && sec(w, 1) >= 0 && sec(w, 0) != sec(w, 1); }
    // engine.py:1597-1604
    bool same_pair(int a, int b) const {
        return (sec(a, 0) == sec(b, 0) && sec(a, 1) == sec(b, 1)) || (sec(a, 0) == sec(b, 1) && sec(a, 1) == sec(b, 0));
    }
    bool shares_any_endpoint(int a, int b) const {
        return vert(a, 0) == vert(b, 0) || vert(a, 0) == vert(b, 1) || vert(a, 1) == vert(b, 0) || vert(a, 1) == vert(b, 1);
    }
    // engine.py:1587-1612
    bool opposing(int a, int b) const {
        if (!same_pair(a, b) || sec(a, 1) < 0 || sec(b, 1) < 0 || shares_any_endpoint(a, b)) return false;
        const float *wa = m->walls + 4 * a, *wb = m->walls + 4 * b;
        float ax = wa[2] - wa[0], ay = wa[3] - wa[1], bx = wb[2] - wb[0], by = wb[3] - wb[1];
        float dot = ax * bx + ay * by;
        float cross = ax * by - ay * bx;
        return dot < 0 && std::fabs(cross) < 1e-6f;
    }
    // Shared tail of engine.py:399-440 and 443-484: the unique linedef at `vertex`
    // (other than a, b) whose sector set equals (pair(a) | pair(b)) - (pair(a) & pair(b)).
    bool triangle_bridge(int vertex, int a, int b, int *index) const {
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
    // _native_projected_portal_bridge_{indices,mask}[slot, path, owner] (engine.py:399-440)
    bool portal_bridge(int slot, int path, int owner, int *index) const {
        *index = 0;
        if (owner == path) return false;
        int v = vert(path, slot);
        if (vert(owner, 0) != v && vert(owner, 1) != v) return false;
        return triangle_bridge(v, path, owner, index);
    }
    // _native_projected_sector_bridge_{indices,mask}[slot, pending, path] (engine.py:443-484)
    bool sector_bridge(int slot, int pending, int path, int *index) const {
        *index = 0;
        if (path == pending) return false;
        return triangle_bridge(vert(pending, slot), pending, path, index);
    }

    // ------------------------------------------------------------------ lane setup
    // engine.py:10648-10658, 2122-2133, 9622-9631, 12384-12391
    void setup_lane(const gd_lanes_desc *lanes, int n) {
        L.x = lanes->x[n]; L.y = lanes->y[n]; L.angle = lanes->angle[n]; L.view_z = lanes->view_z[n];
        L.pitch_bam = lanes->pitch_bam[n];
        L.flash_light = lanes->flash_light ? lanes->flash_light[n] : 0;
        i64 retained_bam = lanes->angle_bam[n];
        float visible_angle = float(retained_bam) * BAM_TO_RADIANS;
        if (L.angle != visible_angle) {
            float two_pi = float(2.0 * M_PI);
            float r = std::fmod(L.angle, two_pi);
            if (r != 0 && ((r < 0) != (two_pi < 0))) r += two_pi;  // torch.remainder
            L.angle_bam = round_to_i64(r / BAM_TO_RADIANS) & UINT32_MASK;
        } else {
            L.angle_bam = retained_bam;
        }
        float visible_x = float(lanes->x_fixed[n]) / float(FIXED_UNIT);
        float visible_y = float(lanes->y_fixed[n]) / float(FIXED_UNIT);
        L.view_x_fixed = (L.x != visible_x) ? round_to_i64(L.x * float(FIXED_UNIT)) : lanes->x_fixed[n];
        L.view_y_fixed = (L.y != visible_y) ? round_to_i64(L.y * float(FIXED_UNIT)) : lanes->y_fixed[n];
        L.fine = int((L.angle_bam >> ANGLE_TO_FINE_SHIFT) & (FINE_ANGLES - 1));
        L.vsin = g_fine_sine[L.fine];
        L.vcos = g_fine_sine[(L.fine + FINE_ANGLES / 4) & (FINE_ANGLES - 1)];
        L.fsin = float(L.vsin) / float(FIXED_UNIT);
        L.fcos = float(L.vcos) / float(FIXED_UNIT);
        i64 tangent_index = clampi((ANGLE_90 - L.pitch_bam) >> ANGLE_TO_FINE_SHIFT, 0, FINE_ANGLES / 2 - 1);
        i64 tangent = g_fine_tangent[tangent_index];
        L.center_fixed = i64(VH / 2) * FIXED_UNIT + ((FOCAL_Y_FIXED * tangent) >> 16);
        // _pitch_projection_offset(192.0): round(192*65536) = 12582912
        i64 focal_fixed = 12582912;
        L.pitch_offset = float((tangent * focal_fixed) >> 16) / float(FIXED_UNIT);
        // engine.py:10660-10670
        for (int x = 0; x < SW; ++x) {
            float c = (float(x) - 160.0f) / 160.0f;
            dirx[x] = L.fcos + L.fsin * c;
            diry[x] = L.fsin - L.fcos * c;
        }
        L.sector = sector_at(L.x, L.y);
    }

    // engine.py:9598-9617 (_sector_at): first sector with odd crossing parity, 0 if none
    int sector_at(float px, float py) const {
        for (int s = 0; s < S; ++s) {
            int crossings = 0;
            for (int k = m->sector_edge_ofs[s]; k < m->sector_edge_ofs[s + 1]; ++k) {
                const float *e = m->walls + 4 * m->sector_edge_idx[k];
                float x1 = e[0], y1 = e[1], x2 = e[2], y2 = e[3];
                bool crosses = (y1 > py) != (y2 > py);
                float dy = y2 - y1;
                float safe_dy = std::fabs(dy) < 1e-6f ? 1.0f : dy;
                float crossing_x = x1 + (py - y1) * (x2 - x1) / safe_dy;
                if (crosses && px < crossing_x) ++crossings;
            }
            if (crossings & 1) return s;
        }
        return 0;
    }

    // engine.py:10747-10869 for one linedef (whole-linedef fragment)
    void wall_geometry(int w) { geom[w] = wall_coords(m->walls_fixed + 4 * w, &tx[2 * w], &ty[2 * w]); }

    // engine.py:11472-11500: the same for every fragment of the split linedefs
    void fragment_geometry() {
        const int F = m->fragment_slots;
        for (int k = 0; k < m->split_count * F; ++k) {
            i64 ftx[2], fty[2];
            frag_geom[k] = wall_coords(m->split_fragments_fixed + 4 * size_t(k), ftx, fty);
            frag_vis[2 * k] = wall_visibility_side(ftx[0], ftx[1], fty[0], fty[1]);
            frag_vis[2 * k + 1] = wall_visibility_side(ftx[1], ftx[0], fty[1], fty[0]);
        }
    }

    // engine.py:11511-11529 / 12324-12333: the first present fragment whose half-open span holds the
    // column; -1 if none.  *fragments receives how many fragments the linedef has.
    int owning_fragment(int w, int x, int *fragments) const {
        const int F = m->fragment_slots, row = m->wall_split_slot[w];
        int owner = -1, count = 0;
        for (int k = 0; k < F; ++k) {
            if (!m->split_fragment_mask[row * F + k]) continue;
            ++count;
            const WallGeom &g = frag_geom[size_t(row) * F + k];
            if (owner < 0 && (g.sr > g.sl) && (x >= g.sl) && (x < g.sr)) owner = row * F + k;
        }
        *fragments = count;
        return owner;
    }

    WallGeom wall_coords(const int32_t *wf, i64 *tx_out, i64 *ty_out) const {
        i64 rx0 = wf[0] - L.view_x_fixed, ry0 = wf[1] - L.view_y_fixed;
        i64 rx1 = wf[2] - L.view_x_fixed, ry1 = wf[3] - L.view_y_fixed;
        i64 tx0 = (rx0 * L.vsin - ry0 * L.vcos) >> 20, ty0 = (rx0 * L.vcos + ry0 * L.vsin) >> 20;
        i64 tx1v = (rx1 * L.vsin - ry1 * L.vcos) >> 20, ty1v = (rx1 * L.vcos + ry1 * L.vsin) >> 20;
        tx_out[0] = tx0; tx_out[1] = tx1v; ty_out[0] = ty0; ty_out[1] = ty1v;
        i64 vx = i64(wf[2]) - wf[0], vy = i64(wf[3]) - wf[1];
        i64 fx = L.view_x_fixed - wf[0], fy = L.view_y_fixed - wf[1];
        bool front = (vx * fy - vy * fx) < 0;
        i64 tx1 = front ? tx0 : tx1v, tx2 = front ? tx1v : tx0;
        i64 ty1 = front ? ty0 : ty1v, ty2 = front ? ty1v : ty0;
        const i64 center = 160 * FIXED_UNIT;
        i64 safe_ty1 = ty1 == 0 ? 1 : ty1, safe_ty2 = ty2 == 0 ? 1 : ty2;
        i64 left_projected = (center + tdiv(tx1 * center, safe_ty1)) >> 16;
        left_projected += (tx1 >= 0);
        if (tx1 >= 0) left_projected = std::min<i64>(left_projected, SW);
        i64 right_projected = (center + tdiv(tx2 * center, safe_ty2)) >> 16;
        right_projected += (tx2 >= 0);
        if (tx2 >= 0) right_projected = std::min<i64>(right_projected, SW);
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
        return WallGeom{sl, sr, dl, dr};
    }

    // engine.py:11217-11291 for one endpoint order
    WallVis wall_visibility_side(i64 tx1, i64 tx2, i64 ty1, i64 ty2) const {
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
        i64 light_left = tdiv(WALL_VISIBILITY_FIXED << 12, std::max<i64>(wdl, 1));
        i64 light_right = tdiv(WALL_VISIBILITY_FIXED << 12, std::max<i64>(wdr, 1));
        i64 light_step = tdiv(light_right - light_left, std::max<i64>(wsr - wsl, 1));
        return WallVis{light_left, light_step, wsl};
    }
    i64 visibility_at(int w, int side, int x) const {
        const WallVis *chosen = &vis[2 * w + side];
        if (m->wall_split_slot[w] >= 0) {   // engine.py:11530-11545: only linedefs with several fragments
            int fragments, owner = owning_fragment(w, x, &fragments);
            if (owner >= 0 && fragments > 1) chosen = &frag_vis[2 * size_t(owner) + side];
        }
        const WallVis &v = *chosen;
        return v.light_left + (i64(x) - v.screen_left) * v.light_step;
    }

    // engine.py:11304-11460 (+ 11472-11493, 11589-11595) for the whole lane
    void portal_intersections() {
        std::vector<int> first_col(W, 0), last_col(W, 0);
        std::vector<uint8_t> has_columns(W, 0), den_ok(size_t(SW) * W);
        for (int w = 0; w < W; ++w) {
            const float *wl = m->walls + 4 * w;
            float sx = wl[0], sy = wl[1];
            float segx = wl[2] - sx, segy = wl[3] - sy;
            float offx = sx - L.x, offy = sy - L.y;
            bool any = false; int first = 0, last = 0;
            for (int x = 0; x < SW; ++x) {
                float rx = dirx[x], ry = diry[x];
                float den = rx * segy - ry * segx;
                float safe = std::fabs(den) < 1e-6f ? 1.0f : den;
                float d = (offx * segy - offy * segx) / safe;
                float a = (offx * ry - offy * rx) / safe;
                bool ok = std::fabs(den) >= 1e-6f;
                bool g = ok && (d > 0) && (a >= 0) && (a <= 1);
                size_t i = size_t(x) * W + w;
                dist[i] = d; along[i] = a; geo[i] = g; den_ok[i] = ok;
                if (g) { if (!any) first = x; last = x; any = true; }
            }
            has_columns[w] = any;
            // argmax of an all-false row is 0: first=0, last=319-0
            first_col[w] = any ? first : 0;
            last_col[w] = any ? last : SW - 1;
            float vfx = L.x - sx, vfy = L.y - sy;
            front_facing_f32[w] = (segx * vfy - segy * vfx) < 0;
        }
        const i64 center = 160 * FIXED_UNIT;
        for (int w = 0; w < W; ++w) {
            i64 screen_left = first_col[w], screen_right = last_col[w] + 1;
            bool hc = has_columns[w];
            i64 ep_col[2]; bool ep_vis[2];
            for (int e = 0; e < 2; ++e) {
                i64 txe = tx[2 * w + e], tye = ty[2 * w + e];
                i64 safe_ty = tye == 0 ? 1 : tye;
                i64 projected_fixed = center + tdiv(txe * center, safe_ty);
                ep_col[e] = (projected_fixed >> 16) + (txe >= 0);
                ep_vis[e] = (tye > 0) && (txe >= -tye) && (txe <= tye) && (ep_col[e] >= 0) && (ep_col[e] <= SW);
            }
            bool ff = front_facing_f32[w];
            for (int e = 0; e < 2; ++e) {
                bool visible = ep_vis[e] && hc;
                bool owns_left = ff ? (e == 0) : (e == 1);
                if (visible && owns_left) screen_left = ep_col[e];
                if (visible && !owns_left) screen_right = ep_col[e];
            }
            i64 ord_col0 = ff ? ep_col[0] : ep_col[1], ord_col1 = ff ? ep_col[1] : ep_col[0];
            bool exact = ep_vis[0] && ep_vis[1];
            if (exact) { screen_left = ord_col0; screen_right = ord_col1; hc = screen_right > screen_left; }
            hc = hc && (geom[w].sr > geom[w].sl);
            bool os = one_sided[w];
            for (int x = 0; x < SW; ++x) {
                size_t i = size_t(x) * W + w;
                bool screen_valid = hc && (x >= screen_left) && (x < screen_right);
                bool p = den_ok[i] && (dist[i] > 0) && screen_valid;
                bool valid = os ? (p && ff) : (geo[i] || p);
                proj[i] = p;
                ledge[i] = (x == screen_left);
                if (!valid) dist[i] = INF;
                float a = along[i];
                along[i] = a < 0 ? 0.0f : (a > 1 ? 1.0f : a);  // NaN passes through like clamp
            }
            subpixel_two_sided[w] = (geom[w].sr - geom[w].sl <= 1) && !os;
        }
    }

    // engine.py:10672-10739 (PrepWall) for the whole lane
    void texture_mapping() {
        // inverse_vertical_aspect = 320*200/320/240 ; wall_map_scale = that*64/160 (Python floats)
        const double inverse_vertical_aspect = 320 * 200.0 / 320.0 / 240;
        const double wall_map_scale_d = inverse_vertical_aspect * 64.0 / (320 / 2.0);
        const float wall_map_scale = float(wall_map_scale_d);
        for (int w = 0; w < W; ++w) {
            i64 tx1 = tx[2 * w], tx2 = tx[2 * w + 1], ty1 = ty[2 * w], ty2 = ty[2 * w + 1];
            double u_over_z_origin = double(float(tx1) * 160.0f);
            float u_over_z_step_f = -float(ty1);
            double u_over_z_step = double(u_over_z_step_f);
            double inv_z_origin = double(float(tx1 - tx2) * 160.0f);
            float inv_z_step_float = float(ty2 - ty1);
            double inv_z_step = double(inv_z_step_float);
            double depth_scale = double(inv_z_step_float * wall_map_scale);
            double depth_origin = double(-float(u_over_z_step) * wall_map_scale);
            double repeat = double(wall_len_fixed[w]);
            for (int x = 0; x < SW; ++x) {
                double column = double(x) - 160.0;
                double top = u_over_z_origin + u_over_z_step * column;
                double bottom = inv_z_origin + inv_z_step * column;
                double safe_bottom = bottom == 0 ? 1.0 : bottom;
                double fraction = top / safe_bottom;
                size_t i = size_t(x) * W + w;
                hoff[i] = f64_to_i64(std::floor(fraction * repeat + 0.5));
                vstep[i] = f64_to_i64(std::floor(fraction * depth_scale + depth_origin + 0.5));
            }
        }
    }

    // ------------------------------------------------------------------ flats
    // engine.py:10879-10954 for one pixel
    void flat_texture_coordinates(int texture_id, float plane_height, int px, int py, i64 *u, i64 *v) const {
        int width_bits = ilog2(m->tex_w[texture_id]);
        int height_bits = ilog2(m->tex_h[texture_id]);
        i64 xscale = shl64(1, 32 - width_bits), yscale = shl64(1, 32 - height_bits);
        i64 fine_sine = L.vsin, fine_cosine = L.vcos;
        i64 xstep_scale = tdiv(mul64(xscale, fine_sine), FOCAL_X_FIXED);
        i64 ystep_scale = tdiv(mul64(yscale, fine_cosine), FOCAL_X_FIXED);
        i64 flat_column = i64(px) - (SW / 2 - 1);
        i64 basexfrac = (mul64(xscale, fine_cosine) >> 16) + mul64(flat_column, xstep_scale);
        i64 baseyfrac = (mul64(yscale, -fine_sine) >> 16) + mul64(flat_column, ystep_scale);
        i64 pviewx = mul64(xscale, L.view_x_fixed) >> 16;
        i64 pviewy = mul64(yscale, -L.view_y_fixed) >> 16;
        i64 center_row = L.center_fixed >> 16;
        i64 pixel_y_fixed = i64(py) * FIXED_UNIT;
        i64 den = (py < center_row) ? (L.center_fixed - pixel_y_fixed - FIXED_UNIT / 2)
                                    : (pixel_y_fixed - L.center_fixed + FIXED_UNIT / 2);
        den = std::max<i64>(den, 1);
        bool overflow = den <= (FOCAL_Y_FIXED >> 15);
        i64 yslope = tdiv(FOCAL_Y_FIXED << 16, den);
        if (overflow) yslope = (i64(1) << 31) - 1;
        i64 plane_height_fixed = round_to_i64(plane_height * float(FIXED_UNIT));
        i64 distance = mul64(plane_height_fixed, yslope) >> 16;
        i64 xfrac = ((mul64(distance, basexfrac) >> 16) + pviewx) & UINT32_MASK;
        i64 yfrac = ((mul64(distance, baseyfrac) >> 16) + pviewy) & UINT32_MASK;
        *u = xfrac >> (32 - width_bits);
        *v = yfrac >> (32 - height_bits);
    }
    // engine.py:10588-10616 for one pixel
    uint8_t plane_colormap(uint8_t index, float light, float plane_height, int py) const {
        i64 plane_height_fixed = round_to_i64(plane_height * float(FIXED_UNIT));
        i64 glob = std::min<i64>(tdiv(FLOOR_VISIBILITY_FIXED << 16, std::max<i64>(plane_height_fixed, 1)), (i64(1) << 31) - 1);
        i64 row = std::llabs(L.center_fixed - i64(py) * FIXED_UNIT);
        i64 visibility = std::min<i64>(mul64(glob, row) >> 16, 24 * FIXED_UNIT);
        i64 plane_shade = 64 * FIXED_UNIT - (i64(light) + 12) * (FIXED_UNIT / 4);
        i64 shade = clampi((plane_shade - visibility) >> 16, 0, 31);
        return m->colormap[shade * 256 + index];
    }
    uint8_t flat_pixel(int sector, bool is_floor, int px, int py) const {
        float plane_height = is_floor ? (L.view_z - m->sector_heights[2 * sector]) : (m->sector_heights[2 * sector + 1] - L.view_z);
        int texture = is_floor ? m->sector_floor_tex[sector] : m->sector_ceil_tex[sector];
        i64 u, v;
        flat_texture_coordinates(texture, plane_height, px, py, &u, &v);
        uint8_t index = m->tex_atlas[(size_t(texture) * m->tex_max_h + v) * m->tex_max_w + u];
        float light = m->sector_lights[sector] + float(L.flash_light * 16);
        return plane_colormap(index, light, plane_height, py);
    }

    // engine.py:10956-11171
    void render_flats(const float *ray_cos, const float *ray_sin, const float *cosine_correction) {
        const float focal_length = 192.0f;  // 320/2*1.2
        float center = 103.5f + L.pitch_offset;  // 208/2 - 0.5 + offset, evaluated in float32 by Torch
        std::vector<float> ray_distance(size_t(VH) * SW, INF);
        std::vector<uint8_t> floor_px(VH);
        std::vector<float> denom(VH);
        for (int y = 0; y < VH; ++y) {
            float delta = float(y) - center;
            floor_px[y] = delta > 0;
            denom[y] = std::max(std::fabs(delta), 0.5f);
        }
        for (size_t i = 0; i < size_t(VH) * SW; ++i) flat_sector[i] = L.sector;
        for (int s = 0; s < S; ++s) {
            float floor_height = L.view_z - m->sector_heights[2 * s];
            float ceiling_height = m->sector_heights[2 * s + 1] - L.view_z;
            int e0 = m->sector_edge_ofs[s], e1 = m->sector_edge_ofs[s + 1];
            for (int y = 0; y < VH; ++y) {
                float plane_height = floor_px[y] ? floor_height : ceiling_height;
                float perpendicular = plane_height * focal_length / denom[y];
                for (int x = 0; x < SW; ++x) {
                    float cd = perpendicular / cosine_correction[x];
                    float cx = L.x + ray_cos[x] * cd;
                    float cy = L.y + ray_sin[x] * cd;
                    int crossings = 0;
                    for (int k = e0; k < e1; ++k) {
                        const float *e = m->walls + 4 * m->sector_edge_idx[k];
                        float x1 = e[0], y1 = e[1], x2 = e[2], y2 = e[3];
                        float dy = y2 - y1;
                        float safe_dy = std::fabs(dy) < 1e-6f ? 1.0f : dy;
                        bool crosses = (y1 > cy) != (y2 > cy);
                        float crossing_x = x1 + (cy - y1) * (x2 - x1) / safe_dy;
                        if (crosses && cx < crossing_x) ++crossings;
                    }
                    size_t i = size_t(y) * SW + x;
                    bool nearer = (crossings & 1) && (plane_height > 0) && std::isfinite(cd) && (cd > 0) && (cd < ray_distance[i]);
                    if (nearer) { flat_sector[i] = s; ray_distance[i] = cd; }
                }
            }
        }
        // vertical repair (engine.py:11026-11083)
        std::vector<uint8_t> unresolved(size_t(VH) * SW), vspan(size_t(VH) * SW, 0), hspan(size_t(VH) * SW, 0);
        std::vector<int> vspan_sector(size_t(VH) * SW, 0);
        for (size_t i = 0; i < size_t(VH) * SW; ++i) unresolved[i] = !std::isfinite(ray_distance[i]);
        for (int x = 0; x < SW; ++x) {
            // floors: next resolved floor row at or below; sectors are read BEFORE this repair writes
            std::vector<int> snapshot(VH);
            for (int y = 0; y < VH; ++y) snapshot[y] = flat_sector[size_t(y) * SW + x];
            int next = VH;
            std::vector<int> next_floor(VH), next_ceiling(VH);
            for (int y = VH - 1; y >= 0; --y) {
                size_t i = size_t(y) * SW + x;
                if (!unresolved[i] && floor_px[y]) next = y;
                next_floor[y] = next;
            }
            std::vector<uint8_t> vfloor(VH, 0);
            std::vector<int> floor_span_sector(VH, 0);
            for (int y = 0; y < VH; ++y) {
                size_t i = size_t(y) * SW + x;
                floor_span_sector[y] = snapshot[std::min(next_floor[y], VH - 1)];
                vfloor[y] = unresolved[i] && floor_px[y] && next_floor[y] < VH;
                if (vfloor[y]) flat_sector[i] = floor_span_sector[y];
            }
            // ceilings read the sectors AFTER the floor repair (engine.py:11074)
            for (int y = 0; y < VH; ++y) snapshot[y] = flat_sector[size_t(y) * SW + x];
            next = VH;
            for (int y = VH - 1; y >= 0; --y) {
                size_t i = size_t(y) * SW + x;
                if (!unresolved[i] && !floor_px[y]) next = y;
                next_ceiling[y] = next;
            }
            for (int y = 0; y < VH; ++y) {
                size_t i = size_t(y) * SW + x;
                int ceiling_span_sector = snapshot[std::min(next_ceiling[y], VH - 1)];
                bool vceil = unresolved[i] && !floor_px[y] && next_ceiling[y] < VH;
                if (vceil) flat_sector[i] = ceiling_span_sector;
                vspan[i] = vfloor[y] || vceil;
                vspan_sector[i] = vfloor[y] ? floor_span_sector[y] : ceiling_span_sector;
            }
        }
        // horizontal repair (engine.py:11085-11135)
        for (int y = 0; y < VH; ++y) {
            std::vector<int> left_anchor(SW), right_anchor(SW), row_sector(SW);
            std::vector<uint8_t> anchor(SW);
            for (int x = 0; x < SW; ++x) {
                size_t i = size_t(y) * SW + x;
                bool vertical_anchor = vspan[i] && (vspan_sector[i] != L.sector);
                anchor[x] = !unresolved[i] || vertical_anchor;
                row_sector[x] = flat_sector[i];
            }
            int run = -1;
            for (int x = 0; x < SW; ++x) { if (anchor[x]) run = x; left_anchor[x] = run; }
            run = SW;
            for (int x = SW - 1; x >= 0; --x) { if (anchor[x]) run = x; right_anchor[x] = run; }
            for (int x = 0; x < SW; ++x) {
                size_t i = size_t(y) * SW + x;
                int ls = row_sector[std::max(left_anchor[x], 0)];
                int rs = row_sector[std::min(right_anchor[x], SW - 1)];
                bool h = unresolved[i] && left_anchor[x] >= 0 && right_anchor[x] < SW && ls == rs;
                if (h) flat_sector[i] = ls;
                hspan[i] = h;
            }
        }
        for (int y = 0; y < VH; ++y) {
            for (int x = 0; x < SW; ++x) {
                size_t i = size_t(y) * SW + x;
                surface_depth[i] = unresolved[i] ? INF : ray_distance[i] * cosine_correction[x];
                int s = flat_sector[i];
                bool is_floor = floor_px[y];
                frame[i] = flat_pixel(s, is_floor, x, y);
                float plane_height = is_floor ? (L.view_z - m->sector_heights[2 * s]) : (m->sector_heights[2 * s + 1] - L.view_z);
                float visplane_depth = plane_height * focal_length / denom[y];
                scene_surface_depth[i] = (vspan[i] || hspan[i]) ? visplane_depth : surface_depth[i];
            }
        }
    }

    // ------------------------------------------------------------------ walls
    // engine.py:11596-11730 for one (column, linedef)
    void endpoint_owner(int x, int w, int *owner_index, float *owner_distance) const {
        const float *D = &dist[size_t(x) * W];
        const float *AL = &along[size_t(x) * W];
        const uint8_t *P = &proj[size_t(x) * W];
        const uint8_t *LE = &ledge[size_t(x) * W];
        float tol_w = std::max(std::fabs(D[w]) / 128.0f, 4.0f);
        int index; float distance; bool valid;
        if (m->direct_neighbors) {
            bool uses_start = AL[w] <= 0.5f;
            int rn = uses_start ? start_nb[w] : end_nb[w];
            int rslot = uses_start ? start_slot[w] : end_slot[w];
            bool rexists = uses_start ? has_start[w] : has_end[w];
            float rd = D[rn];
            bool r_owns = rexists && P[rn] && LE[rn];
            int on = uses_start ? end_nb[w] : start_nb[w];
            int oslot = uses_start ? end_slot[w] : start_slot[w];
            bool oexists = uses_start ? has_end[w] : has_start[w];
            float od = D[on];
            bool o_owns = subpixel_two_sided[w] && oexists && P[on] && LE[on] && (std::fabs(od - D[w]) <= tol_w);
            bool use_o = o_owns && (!r_owns || (od < rd) || ((od == rd) && (oslot < rslot)));
            index = use_o ? on : rn;
            distance = use_o ? od : rd;
            valid = r_owns || o_owns;
        } else {
            const int K = m->neighbor_slots;
            bool uses_start = AL[w] <= 0.5f;
            float best = INF; int best_slot = 0;
            for (int k = 0; k < K; ++k) {
                int n = m->endpoint_neighbors[w * K + k];
                bool st = m->endpoint_neighbor_starts[w * K + k], en = m->endpoint_neighbor_ends[w * K + k];
                bool ray_nb = uses_start ? st : en;
                bool selected = ray_nb || (subpixel_two_sided[w] && (st || en) && (std::fabs(D[n] - D[w]) <= tol_w));
                float v = (P[n] && LE[n] && selected) ? D[n] : INF;
                if (v < best) { best = v; best_slot = k; }
            }
            index = m->endpoint_neighbors[w * K + best_slot];
            distance = best;
            valid = std::isfinite(best);
        }
        bool has = !P[w] && valid;
        *owner_index = has ? index : w;
        *owner_distance = has ? distance : D[w];
    }

    // engine.py:12294-12605 (OWallMost) for one column
    float project(float world_z, int w, int x) const {
        const WallGeom &g = geom[w];
        i64 whole_sl = g.sl, whole_sr = g.sr;
        i64 whole_dl = std::max<i64>(g.dl, 1), whole_dr = std::max<i64>(g.dr, 1);
        bool has_fragment = (g.sr > g.sl) && (x >= g.sl) && (x < g.sr);
        // argmax over an all-false fragment axis still selects fragment 0, but every use of the
        // selection is then overridden by the whole-linedef projection (engine.py:12598-12604)
        i64 screen_left = g.sl, screen_right = g.sr, depth_left = whole_dl, depth_right = whole_dr;
        if (m->wall_split_slot[w] >= 0) {
            int fragments, owner = owning_fragment(w, x, &fragments);
            has_fragment = owner >= 0;
            if (has_fragment) {
                const WallGeom &f = frag_geom[owner];
                screen_left = f.sl; screen_right = f.sr;
                depth_left = std::max<i64>(f.dl, 1); depth_right = std::max<i64>(f.dr, 1);
            }
        }
        i64 relative_z_fixed = round_to_i64((world_z - L.view_z) * float(FIXED_UNIT));
        i64 pz = -(relative_z_fixed >> 4);
        i64 center_fixed = L.center_fixed;
        i64 px = x;
        i64 original_span = std::max<i64>(whole_sr - whole_sl, 1);
        i64 opl = tdiv(mul64(pz, FOCAL_Y_FIXED), whole_dl);
        i64 opr = tdiv(mul64(pz, FOCAL_Y_FIXED), whole_dr);
        i64 ostep = tdiv(opr - opl, original_span);
        i64 original_projected = clampi((center_fixed + opl + mul64(px - whole_sl, ostep)) >> 16, 0, VH);
        i64 upper_clip = tdiv(shl64(-center_fixed, 16), FOCAL_Y_FIXED);
        i64 lower_clip = tdiv(shl64(i64(VH) * FIXED_UNIT - center_fixed, 16), FOCAL_Y_FIXED);
        i64 upper_left = mul64(upper_clip, depth_left) >> 16, upper_right = mul64(upper_clip, depth_right) >> 16;
        i64 lower_left = mul64(lower_clip, depth_left) >> 16, lower_right = mul64(lower_clip, depth_right) >> 16;
        bool above_left = pz < upper_left, above_right = pz < upper_right;
        bool below_left = pz > lower_left, below_right = pz > lower_right;
        bool entirely_above = above_left && above_right, entirely_below = below_left && below_right;
        i64 clipped_left = screen_left, clipped_right = screen_right;
        i64 clipped_dl = depth_left, clipped_dr = depth_right;
        bool outside_top = false, outside_bottom = false;

        bool crosses_top = above_left != above_right;
        i64 safe_upper_delta = (upper_right != upper_left) ? (upper_right - upper_left) : 1;
        i64 top_fraction = tdiv(shl64(pz - upper_left, 30), safe_upper_delta);
        i64 top_depth = depth_left + (mul64(depth_right - depth_left, top_fraction) >> 30);
        i64 top_cross = screen_left + tdiv(mul64(mul64(depth_right, top_fraction) >> 30, screen_right - screen_left), std::max<i64>(top_depth, 1));
        bool clip_top_right = crosses_top && above_right && (screen_left <= top_cross);
        if (clip_top_right) { clipped_right = top_cross; clipped_dr = top_depth; }
        outside_top |= crosses_top && above_right && (screen_right > top_cross) && (px >= top_cross) && (px < screen_right);
        bool clip_top_left = crosses_top && above_left && (top_cross <= screen_right);
        if (clip_top_left) { clipped_left = top_cross; clipped_dl = top_depth; }
        outside_top |= crosses_top && above_left && (top_cross > screen_left) && (px >= screen_left) && (px < top_cross);

        bool crosses_bottom = below_left != below_right;
        i64 safe_lower_delta = (lower_right != lower_left) ? (lower_right - lower_left) : 1;
        i64 bottom_fraction = tdiv(shl64(pz - lower_left, 30), safe_lower_delta);
        i64 bottom_depth = depth_left + (mul64(depth_right - depth_left, bottom_fraction) >> 30);
        i64 bottom_cross = screen_left + tdiv(mul64(mul64(depth_right, bottom_fraction) >> 30, screen_right - screen_left), std::max<i64>(bottom_depth, 1));
        bool clip_bottom_right = crosses_bottom && below_right && (screen_left <= bottom_cross);
        if (clip_bottom_right) { clipped_right = bottom_cross; clipped_dr = bottom_depth; }
        outside_bottom |= crosses_bottom && below_right && (screen_right > bottom_cross) && (px >= bottom_cross) && (px < screen_right);
        bool clip_bottom_left = crosses_bottom && below_left && (bottom_cross <= screen_right);
        if (clip_bottom_left) { clipped_left = bottom_cross; clipped_dl = bottom_depth; }
        outside_bottom |= crosses_bottom && below_left && (bottom_cross > screen_left) && (px >= screen_left) && (px < bottom_cross);

        i64 projected_left = tdiv(mul64(pz, FOCAL_Y_FIXED), std::max<i64>(clipped_dl, 1));
        i64 projected_right = tdiv(mul64(pz, FOCAL_Y_FIXED), std::max<i64>(clipped_dr, 1));
        i64 span = std::max<i64>(clipped_right - clipped_left, 1);
        i64 projected_step = tdiv(projected_right - projected_left, span);
        i64 projected = center_fixed + projected_left + mul64(px - clipped_left, projected_step);
        projected = clampi(projected >> 16, 0, VH);
        bool collapsed = (clipped_right == clipped_left) && (px == clipped_left) && !(entirely_above || entirely_below);
        if (entirely_above || (outside_top && !collapsed)) projected = 0;
        else if (entirely_below || (outside_bottom && !collapsed)) projected = VH;
        if (!has_fragment) projected = original_projected;
        return float(projected);
    }

    // engine.py:10630-10640
    static i64 wall_shade(float light, i64 visibility) {
        i64 shade = 64 * FIXED_UNIT - (i64(light) + 12) * (FIXED_UNIT / 4);
        return clampi((shade - std::min<i64>(visibility, 24 * FIXED_UNIT)) >> 16, 0, 31);
    }

    struct ColumnState {  // engine.py:11561-11580, 11735-11762
        int current_sector;
        float ceiling_clip, floor_clip;
        float masked_ceiling_clip, masked_floor_clip, masked_distance;
        int masked_wall;
        float previous_distance;
        bool pend_po_boundary; int pend_po_vertex;
        bool pend_ep_boundary; int pend_ep_vertex; int pend_ep_wall;
        bool pend_eb_boundary; int pend_eb_index;
        bool pend_pb; int pend_pb_index; int pend_pb_sector; float pend_pb_exit;
    };

    struct PassColumn {  // values of one pass that painting and the 4-column rule need
        bool valid, raster_valid, one_sided;
        int wall, side, render_current, other_sector, safe_other;
        float distance;
        i64 visibility;
        float view_floor, view_ceiling, other_floor, other_ceiling;
        float clipped_top, clipped_bottom, clipped_upper_bottom, clipped_lower_top;
        int side_tex[3];
        bool tier_column[3];
        bool mark_ceiling, mark_floor;
        // carried to the post-paint phase
        bool has_ps, ps_keeps, no_keeps, geometric_intersection, replace_np;
        int ps_path_index; float ps_path_distance; int ps_other; bool ps_from_front;
        int no_path_other; float no_path_distance;
        bool starts_po_boundary, continues_po_boundary;
        int sel_vertex;
        bool pend_ep_has_forward_bridge; int fb_idx;
    };

    // engine.py:11768-13371, plus exact planes 13372-13422 and masked mid-textures 13424-13744
    void render_portal_walls() {
        const size_t PX = size_t(VH) * SW;
        std::fill(filled.begin(), filled.end(), 0);
        std::fill(plane_sector.begin(), plane_sector.end(), -1);
        std::fill(plane_is_floor.begin(), plane_is_floor.end(), 0);
        for (size_t i = 0; i < PX; ++i) scene_depth[i] = scene_surface_depth[i];
        std::fill(sprite_clip_depth.begin(), sprite_clip_depth.end(), INF);
        std::fill(sprite_clip_wall.begin(), sprite_clip_wall.end(), -1);
        std::vector<ColumnState> st(SW);
        std::vector<uint8_t> boundary_has_projected_owner(SW, 0);
        for (int x = 0; x < SW; ++x) {
            ColumnState &c = st[x];
            c.current_sector = L.sector;
            c.ceiling_clip = 0.0f; c.floor_clip = float(VH);
            c.masked_ceiling_clip = 0.0f; c.masked_floor_clip = float(VH); c.masked_distance = INF; c.masked_wall = -1;
            c.previous_distance = 0.0f;
            c.pend_po_boundary = false; c.pend_po_vertex = -1;
            c.pend_ep_boundary = false; c.pend_ep_vertex = -1; c.pend_ep_wall = 0;
            c.pend_eb_boundary = false; c.pend_eb_index = 0;
            c.pend_pb = false; c.pend_pb_index = 0; c.pend_pb_sector = -1; c.pend_pb_exit = 0.0f;
            const float *D = &dist[size_t(x) * W]; const uint8_t *LE = &ledge[size_t(x) * W];
            for (int w = 0; w < W; ++w) if (LE[w] && std::isfinite(D[w])) { boundary_has_projected_owner[x] = 1; break; }
        }
        std::vector<PassColumn> pc(SW);
        for (int pass = 0; pass < S; ++pass) {
            bool any_valid = false;
            for (int x = 0; x < SW; ++x) { pass_select(x, st[x], boundary_has_projected_owner[x], pc[x]); any_valid |= pc[x].valid; }
            for (int x = 0; x < SW; ++x) pass_paint(x, st[x], pc);
            bool changed = false;
            for (int x = 0; x < SW; ++x) changed |= pass_advance(x, st[x], pc[x]);
            // A pass in which no column found a wall and no carried state changed is a fixed
            // point of the reference loop: every later pass repeats it exactly.
            if (!any_valid && !changed) break;
        }
        exact_planes();
        masked_midtextures(st);
    }

    void pass_select(int x, const ColumnState &c, bool boundary_has_po, PassColumn &r) const {
        const float *D = &dist[size_t(x) * W];
        const float *AL = &along[size_t(x) * W];
        const uint8_t *G = &geo[size_t(x) * W];
        const uint8_t *P = &proj[size_t(x) * W];
        const uint8_t *LE = &ledge[size_t(x) * W];
        const int cs = c.current_sector;
        const int cur = std::max(cs, 0);
        const float prev = c.previous_distance;
        const float prev_eps = prev + 1e-3f;
        auto incident = [&](int w) { return sec(w, 0) == cur || sec(w, 1) == cur; };

        // a. nearest incident wall beyond previous_distance (engine.py:11769-11780)
        float distance = INF; int wi = 0;
        for (int w = 0; w < W; ++w) {
            float v = (incident(w) && cs >= 0 && D[w] > prev) ? D[w] : INF;
            if (v < distance) { distance = v; wi = w; }
        }
        // b. equal-depth solid (engine.py:11784-11807)
        {
            float sd = INF; int swi = 0;
            for (int w = 0; w < W; ++w) {
                float v = (incident(w) && cs >= 0 && D[w] > prev) ? D[w] : INF;
                bool eds = one_sided[w] && std::isfinite(v) && (std::fabs(v - distance) <= 1e-3f);
                float vv = eds ? v : INF;
                if (vv < sd) { sd = vv; swi = w; }
            }
            COVER(COV_EQUAL_DEPTH_SOLID, std::isfinite(sd) && swi != wi);
        if (std::isfinite(sd)) { distance = sd; wi = swi; }
        }
        // c. selected endpoint (engine.py:11815-11871)
        float sel_along = AL[wi];
        bool sel_start = sel_along <= 0.5f;
        int sel_vertex = vert(wi, sel_start ? 0 : 1);
        auto shares_sel = [&](int w) { return vert(w, 0) == sel_vertex || vert(w, 1) == sel_vertex; };
        bool continues_po_boundary = c.pend_po_boundary && (sel_vertex == c.pend_po_vertex);
        bool continues_ep_boundary = c.pend_ep_boundary && (sel_vertex == c.pend_ep_vertex);
        int sel_slot = sel_along > 0.5f ? 1 : 0;
        int fb_idx; bool fb_exists = portal_bridge(sel_slot, wi, c.pend_ep_wall, &fb_idx);
        bool pend_ep_has_forward_bridge = continues_ep_boundary && fb_exists && (D[fb_idx] > distance + 1e-3f);
        bool completes_pending_endpoint_bridge = c.pend_eb_boundary && (wi == c.pend_eb_index);
        bool sel_is_proj = P[wi];
        bool sel_excl_right = geom[wi].sr == x;
        // d. projected solid owner (engine.py:11872-11954)
        float ps_path_distance = distance; int ps_path_index = wi;
        float psd = INF; int psi = 0;
        for (int w = 0; w < W; ++w) {
            bool owner = incident(w) && one_sided[w] && P[w] && LE[w] && shares_sel(w) && !sel_is_proj && (D[w] > prev_eps);
            float v = owner ? D[w] : INF;
            if (v < psd) { psd = v; psi = w; }
        }
        {
            const int32_t *ofs = sel_start ? m->solid_bridge_start_ofs : m->solid_bridge_end_ofs;
            const int32_t *idx = sel_start ? m->solid_bridge_start_idx : m->solid_bridge_end_idx;
            float sbd = INF; int sbi = wi;
            bool first = true;
            for (int k = ofs[wi]; k < ofs[wi + 1]; ++k) {
                int b = idx[k];
                if (first) { sbi = b; first = false; }
                bool owner = sel_excl_right && incident(b) && one_sided[b] && P[b] && LE[b] && !sel_is_proj && (D[b] > prev_eps);
                float v = owner ? D[b] : INF;
                if (v < sbd) { sbd = v; sbi = b; }
            }
            COVER(COV_SOLID_BRIDGE, sbd < psd);
            if (sbd < psd) { psd = sbd; psi = sbi; }
        }
        bool has_ps = std::isfinite(psd);
        COVER(COV_PROJECTED_SOLID, has_ps);
        if (has_ps) { distance = psd; wi = psi; }
        // e. endpoint owner (engine.py:11960-12001)
        int eo_idx; float eo_dist;
        endpoint_owner(x, wi, &eo_idx, &eo_dist);
        bool eo_path_geo = G[wi];
        bool replace_eo = (eo_idx != wi) && (eo_dist > prev_eps);
        COVER(COV_ENDPOINT_OWNER, replace_eo);
        if (replace_eo) { distance = eo_dist; wi = eo_idx; }
        int no_path_index = wi; float no_path_distance = distance;
        bool no_path_geo = replace_eo ? eo_path_geo : (bool)G[wi];
        bool no_from_front = cs == sec(no_path_index, 0);
        int no_path_other = no_from_front ? sec(no_path_index, 1) : sec(no_path_index, 0);
        // f. near projected owner (engine.py:12002-12179)
        bool so_is_proj = P[wi];
        bool so_excl_right = geom[wi].sr == x;
        i64 so_span = geom[wi].sr - geom[wi].sl;
        bool so_short = m->wall_len[wi] <= PROJECTED_OWNER_MAX_WALL_LENGTH;
        float npd = INF; int npi = 0;
        for (int w = 0; w < W; ++w) {
            if (!(incident(w) && !one_sided[w] && P[w] && !so_is_proj && (D[w] > prev_eps))) continue;
            bool close = ((same_pair(wi, w) || (LE[w] && so_excl_right && ((so_span <= 2) || (shares_sel(w) && so_short)))) &&
                          (std::fabs(D[w] - distance) <= std::max(std::fabs(D[w]) / 128.0f, 4.0f)));
            bool topo = false;
            if (!close && LE[w] && so_excl_right && so_span <= 2) {
                int dummy; topo = sector_bridge(AL[w] > 0.5f ? 1 : 0, w, no_path_index, &dummy);
            }
            if (!(close || topo)) continue;
            COVER(COV_TOPOLOGICAL_OWNER, topo);
            if (D[w] < npd) { npd = D[w]; npi = w; }
        }
        int pe_s0 = sec(c.pend_ep_wall, 0), pe_s1 = sec(c.pend_ep_wall, 1);
        bool pe_from_current = cs == pe_s0;
        bool pe_incident = pe_from_current || (cs == pe_s1);
        int pe_other = pe_from_current ? pe_s1 : pe_s0;
        int pe_slot = (c.pend_ep_vertex == vert(c.pend_ep_wall, 1)) ? 1 : 0;
        int psb_idx; bool psb_exists = sector_bridge(pe_slot, c.pend_ep_wall, no_path_index, &psb_idx);
        int b0 = sec(psb_idx, 0), b1 = sec(psb_idx, 1);
        bool psb_matches = (b0 == pe_other && b1 == no_path_other) || (b1 == pe_other && b0 == no_path_other);
        float psb_dist = D[psb_idx];
        float pe_tol = std::max(std::fabs(D[c.pend_ep_wall]) / 128.0f, 4.0f);
        bool psb = c.pend_ep_boundary && pe_incident && (pe_other >= 0) && (no_path_other >= 0) &&
                   (geom[c.pend_ep_wall].sr - geom[c.pend_ep_wall].sl <= 1) && no_path_geo && !so_is_proj && so_excl_right &&
                   psb_exists && psb_matches && P[psb_idx] && LE[psb_idx] && (psb_dist > prev - pe_tol) && (psb_dist < no_path_distance);
        if (!psb) psb_dist = INF;
        bool use_psb = psb_dist < npd;
        if (use_psb) { npd = psb_dist; npi = psb_idx; }
        bool replace_np = std::isfinite(npd);
        COVER(COV_SECTOR_BRIDGE, use_psb);
        COVER(COV_NEAR_PROJECTED, replace_np);
        if (replace_np) { distance = npd; wi = npi; }
        bool final_proj = P[wi], final_geo = G[wi];
        bool completes_poab = c.pend_ep_boundary && opposing(c.pend_ep_wall, wi) && final_proj && !final_geo;
        // g. validity (engine.py:12197-12239)
        bool valid = std::isfinite(distance);
        bool excl_only = !so_is_proj && so_excl_right && !replace_np && (so_span <= 2) && !boundary_has_po;
        bool raster_valid = valid && !excl_only && !continues_po_boundary &&
                            !((pend_ep_has_forward_bridge || completes_pending_endpoint_bridge) && !sel_is_proj && sel_excl_right && !replace_np);
        bool geometric_intersection = replace_np ? no_path_geo : (replace_eo ? eo_path_geo : (bool)G[wi]);
        bool no_keeps = replace_np && no_path_geo && (no_path_other >= 0);
        ++g_coverage[COV_PASSES];
        COVER(COV_VALID, valid);
        COVER(COV_DEAD_COLUMN_REVIVED, valid && cs < 0);
        COVER(COV_OPPOSING_BOUNDARY, completes_poab);
        COVER(COV_EXCLUDED_RIGHT_EDGE, valid && excl_only);
        COVER(COV_CONTINUES_OWNER_BOUNDARY, valid && continues_po_boundary);
        COVER(COV_FORWARD_BRIDGE, pend_ep_has_forward_bridge);
        COVER(COV_COMPLETES_ENDPOINT_BRIDGE, valid && completes_pending_endpoint_bridge);
        COVER(COV_NO_KEEPS_PATH, no_keeps);
        // h. sides (engine.py:12240-12292)
        int front = sec(wi, 0), back = sec(wi, 1);
        bool from_front = cs == front;
        int other_sector = from_front ? back : front;
        int render_current = use_psb ? pe_other : (completes_poab ? other_sector : cur);
        bool render_from_front = render_current == front;
        int render_other = render_from_front ? back : front;
        int side = render_from_front ? 0 : 1;
        bool ps_from_front = cs == sec(ps_path_index, 0);
        int ps_other = ps_from_front ? sec(ps_path_index, 1) : sec(ps_path_index, 0);
        bool ps_keeps = has_ps && G[ps_path_index] && (ps_other >= 0);
        COVER(COV_PS_KEEPS_PATH, ps_keeps);
        int safe_other = std::max(render_other, 0);

        r.valid = valid; r.raster_valid = raster_valid; r.one_sided = other_sector < 0;
        r.wall = wi; r.side = side; r.render_current = render_current; r.other_sector = other_sector; r.safe_other = safe_other;
        r.distance = distance;
        r.visibility = visibility_at(wi, side, x);
        r.view_floor = m->sector_heights[2 * render_current]; r.view_ceiling = m->sector_heights[2 * render_current + 1];
        r.other_floor = m->sector_heights[2 * safe_other]; r.other_ceiling = m->sector_heights[2 * safe_other + 1];
        for (int t = 0; t < 3; ++t) r.side_tex[t] = m->side_tex[(wi * 2 + side) * 3 + t];
        // j. projection and clipping (engine.py:12607-12620)
        float one_top = project(r.view_ceiling, wi, x), one_bottom = project(r.view_floor, wi, x);
        float lower_top = project(r.other_floor, wi, x), upper_bottom = project(r.other_ceiling, wi, x);
        r.clipped_top = std::max(one_top, c.ceiling_clip);
        r.clipped_bottom = std::min(one_bottom, c.floor_clip);
        r.clipped_upper_bottom = std::max(std::min(upper_bottom, c.floor_clip), r.clipped_top);
        r.clipped_lower_top = std::min(std::max(lower_top, c.ceiling_clip), r.clipped_bottom);
        // k. plane marks (engine.py:12621-12636)
        bool light_differs = m->sector_lights[render_current] != m->sector_lights[safe_other];
        r.mark_ceiling = r.one_sided || (r.view_ceiling != r.other_ceiling) ||
                         (m->sector_ceil_tex[render_current] != m->sector_ceil_tex[safe_other]) || light_differs;
        r.mark_floor = r.one_sided || (r.view_floor != r.other_floor) ||
                       (m->sector_floor_tex[render_current] != m->sector_floor_tex[safe_other]) || light_differs;
        // m. tier columns (engine.py:12720-12738)
        r.tier_column[0] = r.one_sided && raster_valid && (r.side_tex[0] >= 0) && (r.clipped_top < r.clipped_bottom);
        r.tier_column[1] = !r.one_sided && raster_valid && (r.view_floor < r.other_floor) && (r.side_tex[1] >= 0) && (r.clipped_lower_top < r.clipped_bottom);
        r.tier_column[2] = !r.one_sided && raster_valid && (r.view_ceiling > r.other_ceiling) && (r.side_tex[2] >= 0) && (r.clipped_top < r.clipped_upper_bottom);
        r.has_ps = has_ps; r.ps_keeps = ps_keeps; r.no_keeps = no_keeps; r.geometric_intersection = geometric_intersection;
        r.replace_np = replace_np;
        r.ps_path_index = ps_path_index; r.ps_path_distance = ps_path_distance; r.ps_other = ps_other; r.ps_from_front = ps_from_front;
        r.no_path_other = no_path_other; r.no_path_distance = no_path_distance;
        r.starts_po_boundary = replace_np; r.continues_po_boundary = continues_po_boundary;
        r.sel_vertex = sel_vertex;
        r.pend_ep_has_forward_bridge = pend_ep_has_forward_bridge; r.fb_idx = fb_idx;
    }

    // engine.py:12637-12884: plane marks, tier spans, 4-column bottom tail, texturing
    void pass_paint(int x, const ColumnState &c, const std::vector<PassColumn> &pc) {
        const PassColumn &r = pc[x];
        if (!r.raster_valid) return;  // every span below is gated by raster_valid
        // bottom-tail rule over the aligned group of four columns (engine.py:12688-12761)
        const int g0 = x & ~3;
        bool same_group = true;
        for (int k = 0; k < 4; ++k) same_group &= (pc[g0 + k].wall == pc[g0].wall) && (pc[g0 + k].side == pc[g0].side);
        i64 first_group_visibility = pc[g0].visibility;
        bool group_valid[3]; float group_bottom[3];
        for (int t = 0; t < 3; ++t) {
            bool all = true; float common_top = -INF, common_bottom = INF;
            for (int k = 0; k < 4; ++k) {
                const PassColumn &q = pc[g0 + k];
                float top = (t == 1) ? q.clipped_lower_top : q.clipped_top;
                float bottom = (t == 2) ? q.clipped_upper_bottom : q.clipped_bottom;
                all &= q.tier_column[t];
                common_top = std::max(common_top, top);
                common_bottom = std::min(common_bottom, bottom);
            }
            group_valid[t] = same_group && all && (common_top < common_bottom);
            group_bottom[t] = common_bottom;
        }
        const int wi = r.wall, side = r.side;
        const float ceiling_plane_bottom = std::min(r.clipped_top, c.floor_clip);
        const float floor_plane_top = std::max(r.clipped_bottom, c.ceiling_clip);
        // horizontal texture coordinate (engine.py:12765-12798)
        const float *toff = m->side_off + (wi * 2 + side) * 2;
        i64 h = hoff[size_t(x) * W + wi];
        i64 repeat = wall_len_fixed[wi];
        if (side != 0) h = repeat - h;
        if (geom[wi].sl > 0 && h < 0) h = 0;
        if (h >= repeat) h = repeat - 1;
        i64 offx_fixed = round_to_i64(toff[0] * float(FIXED_UNIT));
        i64 u_base = (h + offx_fixed) >> 16;
        i64 swall = vstep[size_t(x) * W + wi];
        const float *wl = m->walls + 4 * wi;
        bool horizontal = std::fabs(wl[3] - wl[1]) < 1e-6f, vertical = std::fabs(wl[2] - wl[0]) < 1e-6f;
        float fake_contrast = vertical ? 16.0f : (horizontal ? -16.0f : 0.0f);
        float light = (m->sector_lights[r.render_current] + float(L.flash_light * 16)) + fake_contrast;
        for (int y = 0; y < VH; ++y) {
            const float py = float(y);
            const size_t i = size_t(y) * SW + x;
            bool ceiling_span = r.mark_ceiling && (py >= c.ceiling_clip) && (py < ceiling_plane_bottom);
            bool floor_span = r.mark_floor && (py >= floor_plane_top) && (py < c.floor_clip);
            if (plane_sector[i] < 0 && (ceiling_span || floor_span)) {
                plane_sector[i] = r.render_current;
                if (floor_span) plane_is_floor[i] = 1;
            }
            bool one_span = r.one_sided && (py >= r.clipped_top) && (py < r.clipped_bottom);
            bool lower_span = !r.one_sided && (r.view_floor < r.other_floor) && (py >= r.clipped_lower_top) && (py < r.clipped_bottom);
            bool upper_span = !r.one_sided && (r.view_ceiling > r.other_ceiling) && (py >= r.clipped_top) && (py < r.clipped_upper_bottom);
            if (!(one_span || lower_span || upper_span)) continue;
            int texture_id = one_span ? r.side_tex[0] : (lower_span ? r.side_tex[1] : r.side_tex[2]);
            if (texture_id < 0 || filled[i]) continue;
            bool bottom_tail = (one_span && group_valid[0] && py >= group_bottom[0]) ||
                               (lower_span && group_valid[1] && py >= group_bottom[1]) ||
                               (upper_span && group_valid[2] && py >= group_bottom[2]);
            int tw = m->tex_w[texture_id], th = m->tex_h[texture_id];
            i64 tu = ((u_base % tw) + tw) % tw;  // torch.remainder
            float origin_z = one_span ? r.view_ceiling : (lower_span ? r.other_floor : r.other_ceiling);
            int height_bits = ilog2(th);
            i64 vertical_step = mul64(swall, shl64(1, 14 - height_bits));
            i64 screen_delta = i64(y) * FIXED_UNIT - L.center_fixed + FIXED_UNIT;
            i64 texture_mid = round_to_i64((origin_z - L.view_z) * float(FIXED_UNIT) + toff[1] * float(FIXED_UNIT));
            i64 fraction = shl64(texture_mid, 16 - height_bits) + (mul64(vertical_step, screen_delta) >> 16);
            i64 tv = (fraction & UINT32_MASK) >> (32 - height_bits);
            uint8_t texel = m->tex_atlas[(size_t(texture_id) * m->tex_max_h + tv) * m->tex_max_w + tu];
            COVER(COV_BOTTOM_TAIL, bottom_tail && first_group_visibility != r.visibility);
            i64 shade = wall_shade(light, bottom_tail ? first_group_visibility : r.visibility);
            frame[i] = m->colormap[shade * 256 + texel];
            scene_depth[i] = r.distance;
            if (r.distance < sprite_clip_depth[i]) { sprite_clip_depth[i] = r.distance; sprite_clip_wall[i] = wi; }
            filled[i] = 1;
        }
    }

    // engine.py:12885-13371: clip updates, masked drawseg, silhouettes, next sector, carried state
    bool pass_advance(int x, ColumnState &c, const PassColumn &r) {
        const ColumnState before = c;
        const float *D = &dist[size_t(x) * W];
        const float *AL = &along[size_t(x) * W];
        const uint8_t *G = &geo[size_t(x) * W];
        const uint8_t *P = &proj[size_t(x) * W];
        const uint8_t *LE = &ledge[size_t(x) * W];
        const int cs = c.current_sector;
        const int cur = std::max(cs, 0);
        const int wi = r.wall;
        const float distance = r.distance;
        auto incident = [&](int w) { return sec(w, 0) == cur || sec(w, 1) == cur; };
        // o. clip updates (engine.py:12888-12913)
        bool draws_upper = (r.view_ceiling > r.other_ceiling) && (r.side_tex[2] >= 0);
        if (r.raster_valid && !r.one_sided && (draws_upper || r.mark_ceiling))
            c.ceiling_clip = draws_upper ? r.clipped_upper_bottom : r.clipped_top;
        bool draws_lower = (r.view_floor < r.other_floor) && (r.side_tex[1] >= 0);
        if (r.raster_valid && !r.one_sided && (draws_lower || r.mark_floor))
            c.floor_clip = draws_lower ? r.clipped_lower_top : r.clipped_bottom;
        // p. masked drawseg snapshot (engine.py:12914-12939)
        if (r.raster_valid && !r.one_sided && (r.side_tex[0] >= 0) && (distance < c.masked_distance)) {
            c.masked_ceiling_clip = c.ceiling_clip; c.masked_floor_clip = c.floor_clip;
            c.masked_distance = distance; c.masked_wall = wi;
        }
        // q. sprite silhouettes (engine.py:12943-12964)
        {
            bool masked_texture = r.side_tex[0] >= 0;
            bool bottom_sil = !r.one_sided && ((r.view_floor > r.other_floor) || (L.view_z < r.other_floor) || masked_texture);
            bool top_sil = !r.one_sided && ((r.view_ceiling < r.other_ceiling) || (L.view_z > r.other_ceiling) || masked_texture);
            if (r.raster_valid && (bottom_sil || top_sil)) {
                for (int y = 0; y < VH; ++y) {
                    float py = float(y);
                    bool span = (bottom_sil && py >= c.floor_clip) || (top_sil && py < c.ceiling_clip);
                    size_t i = size_t(y) * SW + x;
                    if (span && distance < sprite_clip_depth[i]) { sprite_clip_depth[i] = distance; sprite_clip_wall[i] = wi; }
                }
            }
        }
        // r. clips of the geometric portal behind a projected solid (engine.py:12969-13069)
        {
            int path = r.ps_path_index;
            int path_safe_other = std::max(r.ps_other, 0);
            float pof = m->sector_heights[2 * path_safe_other], poc = m->sector_heights[2 * path_safe_other + 1];
            int pside = r.ps_from_front ? 0 : 1;
            const int32_t *ptex = m->side_tex + (path * 2 + pside) * 3;
            if (r.ps_keeps) {
                float path_top = project(r.view_ceiling, path, x), path_bottom = project(r.view_floor, path, x);
                float path_lower_top = project(pof, path, x), path_upper_bottom = project(poc, path, x);
                float pct = std::max(path_top, c.ceiling_clip);
                float pcb = std::min(path_bottom, c.floor_clip);
                float pcub = std::max(std::min(path_upper_bottom, c.floor_clip), pct);
                float pclt = std::min(std::max(path_lower_top, c.ceiling_clip), pcb);
                bool light_differs = m->sector_lights[r.render_current] != m->sector_lights[path_safe_other];
                bool p_draws_upper = (r.view_ceiling > poc) && (ptex[2] >= 0);
                bool p_marks_ceiling = (r.view_ceiling != poc) || (m->sector_ceil_tex[r.render_current] != m->sector_ceil_tex[path_safe_other]) || light_differs;
                bool p_draws_lower = (r.view_floor < pof) && (ptex[1] >= 0);
                bool p_marks_floor = (r.view_floor != pof) || (m->sector_floor_tex[r.render_current] != m->sector_floor_tex[path_safe_other]) || light_differs;
                // both updates read the clips as they stood after step o (engine.py:12987-12996)
                float new_ceiling = c.ceiling_clip, new_floor = c.floor_clip;
                if (p_draws_upper || p_marks_ceiling) new_ceiling = p_draws_upper ? pcub : pct;
                if (p_draws_lower || p_marks_floor) new_floor = p_draws_lower ? pclt : pcb;
                c.ceiling_clip = new_ceiling; c.floor_clip = new_floor;
                bool pmasked = ptex[0] >= 0;
                bool pbottom = (r.view_floor > pof) || (L.view_z < pof) || pmasked;
                bool ptop = (r.view_ceiling < poc) || (L.view_z > poc) || pmasked;
                for (int y = 0; y < VH; ++y) {
                    float py = float(y);
                    bool span = (pbottom && py >= c.floor_clip) || (ptop && py < c.ceiling_clip);
                    size_t i = size_t(y) * SW + x;
                    if (span && r.ps_path_distance < sprite_clip_depth[i]) { sprite_clip_depth[i] = r.ps_path_distance; sprite_clip_wall[i] = path; }
                }
            }
        }
        // s. next sector (engine.py:13070-13241)
        const float prior = c.previous_distance;
        const float prior_eps = prior + 1e-3f;
        bool endpoint_only_portal = r.valid && !r.one_sided && !r.geometric_intersection;
        const int other_sector = r.other_sector;
        auto other_incident = [&](int w) { return sec(w, 0) == other_sector || sec(w, 1) == other_sector; };
        const float dist_eps = distance + 1e-3f;
        float cnd = INF, ond = INF; int cni = 0, oni = 0;
        float csd = INF, osd = INF;
        float gpd = INF; int gpi = 0;
        const int v0 = vert(wi, 0), v1 = vert(wi, 1);
        for (int w = 0; w < W; ++w) {
            float d = D[w];
            bool future = (G[w] || (one_sided[w] && std::isfinite(d))) && (d > dist_eps);
            bool inc = incident(w), oinc = other_incident(w);
            if (future) {
                if (inc && d < cnd) { cnd = d; cni = w; }
                if (oinc && d < ond) { ond = d; oni = w; }
            }
            bool shares_endpoint = vert(w, 0) == v0 || vert(w, 0) == v1 || vert(w, 1) == v0 || vert(w, 1) == v1;
            bool shared_solid = std::isfinite(d) && one_sided[w] && (shares_endpoint || LE[w]) && (d > prior_eps) && (d <= dist_eps);
            if (shared_solid) {
                if (inc && d < csd) csd = d;
                if (oinc && d < osd) osd = d;
            }
            bool sgp = G[w] && inc && shares_endpoint && !one_sided[w] && (d > prior_eps) && (std::fabs(d - distance) <= SHARED_ENDPOINT_DEPTH_TOLERANCE);
            if (sgp && d < gpd) { gpd = d; gpi = w; }
        }
        bool enters_tied_strip = endpoint_only_portal && std::isfinite(cnd) && (cni == oni) && opposing(wi, cni);
        bool enters_other = endpoint_only_portal && (other_sector >= 0) && ((ond < cnd) || enters_tied_strip);
        bool enters_shared = endpoint_only_portal && (other_sector >= 0) && (osd < csd);
        bool gp_from_front = cs == sec(gpi, 0);
        int gp_other = gp_from_front ? sec(gpi, 1) : sec(gpi, 0);
        bool uses_geometric_path = endpoint_only_portal && std::isfinite(gpd) && (gp_other >= 0);
        int pb_slot = AL[gpi] > 0.5f ? 1 : 0;
        int ppb_idx; bool ppb_exists = portal_bridge(pb_slot, gpi, wi, &ppb_idx);
        float ppb_dist = D[ppb_idx];
        float gp_tol = std::max(std::fabs(D[gpi]) / 128.0f, 4.0f);
        bool endpoint_portal_bridge = uses_geometric_path && ppb_exists && P[ppb_idx] && LE[ppb_idx] && (ppb_dist > prior_eps) &&
                                      (std::fabs(ppb_dist - gpd) <= gp_tol);
        bool completes_pending_portal_bridge = r.valid && c.pend_pb && (wi == c.pend_pb_index);
        COVER(COV_ENDPOINT_ONLY_PORTAL, endpoint_only_portal);
        COVER(COV_TIED_STRIP, enters_tied_strip);
        COVER(COV_ENTERS_OTHER, enters_other);
        COVER(COV_ENTERS_SHARED, enters_shared);
        COVER(COV_GEOMETRIC_PATH, uses_geometric_path);
        COVER(COV_PORTAL_BRIDGE, endpoint_portal_bridge);
        COVER(COV_COMPLETES_PORTAL_BRIDGE, completes_pending_portal_bridge);
        // t. previous_distance (engine.py:13242-13275)
        float pd = prior;
        if (r.valid) {
            if (r.no_keeps) pd = r.no_path_distance;
            else if (r.ps_keeps) pd = r.ps_path_distance;
            else if (enters_shared && (osd < distance)) pd = prior;
            else if (uses_geometric_path) pd = gpd;
            else pd = distance;
        }
        if (r.valid && endpoint_portal_bridge) pd = prior;
        if (r.valid && completes_pending_portal_bridge) pd = std::max(distance, c.pend_pb_exit);
        c.previous_distance = pd;
        // carried state (engine.py:13276-13313)
        if (r.starts_po_boundary) c.pend_po_vertex = r.sel_vertex;
        c.pend_po_boundary = r.starts_po_boundary || (c.pend_po_boundary && r.continues_po_boundary);
        int ep_vertex = vert(wi, AL[wi] <= 0.5f ? 0 : 1);
        if (endpoint_only_portal) { c.pend_ep_vertex = ep_vertex; c.pend_ep_wall = wi; }
        c.pend_ep_boundary = endpoint_only_portal;
        if (r.pend_ep_has_forward_bridge) c.pend_eb_index = r.fb_idx;
        c.pend_eb_boundary = r.pend_ep_has_forward_bridge;
        // next sector (engine.py:13314-13350)
        int next_sector;
        if (r.no_keeps) next_sector = r.no_path_other;
        else if (r.ps_keeps) next_sector = r.ps_other;
        else if (uses_geometric_path) next_sector = gp_other;
        else if (r.valid && !r.one_sided && (r.geometric_intersection || enters_other || enters_shared)) next_sector = other_sector;
        else if (endpoint_only_portal) next_sector = cs;
        else next_sector = -1;
        if (endpoint_portal_bridge) next_sector = other_sector;
        if (completes_pending_portal_bridge) next_sector = c.pend_pb_sector;
        // engine.py:13355-13371
        if (endpoint_portal_bridge) { c.pend_pb_index = ppb_idx; c.pend_pb_sector = gp_other; c.pend_pb_exit = gpd; }
        c.pend_pb = endpoint_portal_bridge;
        c.current_sector = next_sector;
        return std::memcmp(&before, &c, sizeof(ColumnState)) != 0;
    }

    // engine.py:13372-13422
    void exact_planes() {
        const float focal_length = 192.0f;
        float center = 103.0f + L.pitch_offset;   // 208/2 - 1 + offset
        float flat_center = center + 0.5f;
        for (int y = 0; y < VH; ++y) {
            float plane_denominator = std::max(std::fabs(float(y) - flat_center), 0.5f);
            for (int x = 0; x < SW; ++x) {
                size_t i = size_t(y) * SW + x;
                if (!(plane_sector[i] >= 0 && !filled[i])) continue;
                int s = plane_sector[i];
                bool is_floor = plane_is_floor[i];
                frame[i] = flat_pixel(s, is_floor, x, y);
                float plane_height = is_floor ? (L.view_z - m->sector_heights[2 * s]) : (m->sector_heights[2 * s + 1] - L.view_z);
                scene_depth[i] = plane_height * focal_length / plane_denominator;
                if (std::isinf(surface_depth[i]) && std::isinf(sprite_clip_depth[i])) sprite_clip_depth[i] = scene_depth[i];
            }
        }
    }

    // engine.py:13424-13744
    void masked_midtextures(const std::vector<ColumnState> &st) {
        std::vector<int> masked_side(W), masked_tex(W);
        for (int w = 0; w < W; ++w) {
            const float *wl = m->walls + 4 * w;
            float vx = wl[2] - wl[0], vy = wl[3] - wl[1];
            float fx = L.x - wl[0], fy = L.y - wl[1];
            bool from_front = (vx * fy - vy * fx) < 0;
            masked_side[w] = from_front ? 0 : 1;
            masked_tex[w] = m->side_tex[(w * 2 + masked_side[w]) * 3 + 0];
        }
        for (int x = 0; x < SW; ++x) {
            const float *D = &dist[size_t(x) * W];
            const uint8_t *P = &proj[size_t(x) * W];
            const uint8_t *LE = &ledge[size_t(x) * W];
            float md = INF; int mw = 0;
            for (int w = 0; w < W; ++w) {
                bool cand = P[w] && !one_sided[w] && masked_tex[w] >= 0;
                float v = cand ? D[w] : INF;
                if (v < md) { md = v; mw = w; }
            }
            if (!std::isfinite(md)) continue;  // masked_valid gates the only writes
            const ColumnState &c = st[x];
            int mside = masked_side[mw];
            int texture_id = std::max(masked_tex[mw], 0);
            int front_sector = sec(mw, 0), back_sector = std::max(sec(mw, 1), 0);
            int light_sector = mside == 0 ? front_sector : back_sector;
            float world_top = std::min(m->sector_heights[2 * front_sector + 1], m->sector_heights[2 * back_sector + 1]);
            int tw = m->tex_w[texture_id], th = m->tex_h[texture_id];
            float owall_top = project(world_top, mw, x);
            float owall_bottom = project(world_top - float(th), mw, x);
            bool left_edge = LE[mw];
            bool has_saved = c.masked_wall == mw;
            float mceil = std::max(owall_top, has_saved ? c.masked_ceiling_clip : 0.0f);
            float mfloor = std::min(owall_bottom, has_saved ? c.masked_floor_clip : float(VH));
            const float *toff = m->side_off + (mw * 2 + mside) * 2;
            i64 h = hoff[size_t(x) * W + mw];
            i64 repeat = wall_len_fixed[mw];
            if (mside != 0) h = repeat - h;
            i64 msl = geom[mw].sl, msr = geom[mw].sr;
            if (msl > 0 && h < 0) h = 0;
            if (h >= repeat) h = repeat - 1;
            i64 offx = round_to_i64(toff[0] * float(FIXED_UNIT));
            i64 ub = (h + offx) >> 16;
            i64 mu = ((ub % tw) + tw) % tw;
            int height_bits = ilog2(th);
            i64 swall_cur = vstep[size_t(x) * W + mw];
            i64 vertical_step = mul64(swall_cur, shl64(1, 14 - height_bits));
            i64 center_fixed = L.center_fixed;
            i64 texture_mid = round_to_i64((world_top - L.view_z) * float(FIXED_UNIT) + toff[1] * float(FIXED_UNIT));
            i64 safe_left = clampi(msl, 0, SW - 1), safe_last = clampi(msr - 1, 0, SW - 1);
            i64 start_swall = vstep[size_t(safe_left) * W + mw], end_swall = vstep[size_t(safe_last) * W + mw];
            auto iscale_of = [](i64 swall) {
                i64 s = mul64(swall, FIXED_UNIT) >> 18;
                if (s >= 0 && s < 3) return i64(3);
                if (s > -3 && s < 0) return i64(-3);
                return s;
            };
            i64 start_iscale = iscale_of(start_swall), end_iscale = iscale_of(end_swall);
            i64 start_scale = tdiv(i64(1) << 32, start_iscale), end_scale = tdiv(i64(1) << 32, end_iscale);
            i64 screen_span = std::max<i64>(msr - msl, 1);
            i64 scale_step = tdiv(end_scale - start_scale, screen_span);
            i64 sprite_scale = start_scale + mul64(scale_step, i64(x) - msl);
            i64 top_screen = center_fixed - (mul64(texture_mid, sprite_scale) >> 16);
            i64 post_top = top_screen >> 16;
            i64 post_bottom = ((top_screen + mul64(sprite_scale, th) - FIXED_UNIT) >> 16) + 1;
            i64 clipped_top = std::max<i64>(post_top, (i64)mceil);
            i64 clipped_bottom = std::min<i64>(post_bottom, (i64)mfloor);
            i64 dc_iscale = mul64(swall_cur, FIXED_UNIT) >> 18;
            bool initial_post = clipped_top < clipped_bottom;
            i64 frac_start = texture_mid + mul64(clipped_top, dc_iscale) - (mul64(center_fixed - FIXED_UNIT, dc_iscale) >> 16);
            i64 frac_end = frac_start + mul64(clipped_bottom - clipped_top - 1, dc_iscale);
            bool extends = initial_post && (float(clipped_bottom) < mfloor) && (frac_end < i64(th) * FIXED_UNIT - dc_iscale);
            clipped_bottom += extends;
            if (!(has_saved || left_edge)) continue;
            ++g_coverage[COV_MASKED_COLUMN];
            COVER(COV_MASKED_EXTENDS, extends);
            const float *wl = m->walls + 4 * mw;
            bool horizontal = std::fabs(wl[3] - wl[1]) < 1e-6f, vertical = std::fabs(wl[2] - wl[0]) < 1e-6f;
            float contrast = vertical ? 16.0f : (horizontal ? -16.0f : 0.0f);
            float light = (m->sector_lights[light_sector] + float(L.flash_light * 16)) + contrast;
            i64 visibility = visibility_at(mw, mside, x);
            i64 shade = wall_shade(light, visibility);
            for (int y = 0; y < VH; ++y) {
                float py = float(y);
                if (!(py >= float(clipped_top) && py < float(clipped_bottom))) continue;
                i64 screen_delta = i64(y) * FIXED_UNIT - center_fixed + FIXED_UNIT;
                i64 fraction = shl64(texture_mid, 16 - height_bits) + (mul64(vertical_step, screen_delta) >> 16);
                i64 mv = (fraction & UINT32_MASK) >> (32 - height_bits);
                uint8_t texel = m->tex_atlas[(size_t(texture_id) * m->tex_max_h + mv) * m->tex_max_w + mu];
                size_t i = size_t(y) * SW + x;
                frame[i] = m->colormap[shade * 256 + texel];
                scene_depth[i] = md;
            }
        }
    }

    // ------------------------------------------------------------------ sprites
    // engine.py:10534-10557
    void blocking_raycast(float *wall_distance, int *blocking_wall) const {
        for (int x = 0; x < SW; ++x) {
            float best = INF; int slot = 0;
            for (int b = 0; b < m->blocking_count; ++b) {
                const float *wl = m->walls + 4 * m->blocking_walls[b];
                float sx = wl[0], sy = wl[1];
                float segx = wl[2] - sx, segy = wl[3] - sy;
                float offx = sx - L.x, offy = sy - L.y;
                float rx = dirx[x], ry = diry[x];
                float den = rx * segy - ry * segx;
                float safe = std::fabs(den) < 1e-6f ? 1.0f : den;
                float d = (offx * segy - offy * segx) / safe;
                float a = (offx * ry - offy * rx) / safe;
                bool valid = (std::fabs(den) >= 1e-6f) && (d > 0) && (a >= 0) && (a <= 1);
                float v = valid ? d : INF;
                if (v < best) { best = v; slot = b; }
            }
            wall_distance[x] = std::min(std::max(best, 1.0f), 4096.0f);
            blocking_wall[x] = m->blocking_count ? m->blocking_walls[slot] : 0;
        }
    }

    // engine.py:14684-14947 on an already packed sprite list
    void render_sprites(const gd_lanes_desc *lanes, int n) {
        const int A = lanes->sprite_slots;
        if (A <= 0 || !lanes->sprite_x) return;
        std::vector<float> wall_distance(SW); std::vector<int> blocking_wall(SW);
        blocking_raycast(wall_distance.data(), blocking_wall.data());
        struct Spr {
            float x, y, z, depth; int id; bool alive, fullbright; int style;
            i64 depth_fixed, left, right, hstep, yscale, top_fixed, texmid, iscale; float light;
        };
        std::vector<Spr> sp(A);
        for (int a = 0; a < A; ++a) {
            Spr &s = sp[a];
            size_t k = size_t(n) * A + a;
            s.x = lanes->sprite_x[k]; s.y = lanes->sprite_y[k]; s.z = lanes->sprite_z[k];
            s.depth = lanes->sprite_depth[k]; s.id = lanes->sprite_id[k];
            s.alive = lanes->sprite_alive[k]; s.fullbright = lanes->sprite_fullbright ? lanes->sprite_fullbright[k] : 0;
            s.style = lanes->sprite_style ? lanes->sprite_style[k] : -1;
            // engine.py:14174-14198
            i64 ax = round_to_i64(s.x * float(FIXED_UNIT)), ay = round_to_i64(s.y * float(FIXED_UNIT));
            i64 rx = ax - L.view_x_fixed, ry = ay - L.view_y_fixed;
            s.depth_fixed = (rx * L.vcos + ry * L.vsin) >> 20;
            i64 side_fixed = (rx * L.vsin - ry * L.vcos) >> 16;
            // engine.py:14138-14172
            i64 xscale = tdiv(FOCAL_X_FIXED << 12, std::max<i64>(s.depth_fixed, SPRITE_MIN_DEPTH_FIXED));
            i64 left_fixed = side_fixed - i64(m->spr_left[s.id]) * FIXED_UNIT;
            s.left = SW / 2 + (mul64(left_fixed, xscale) >> 32);
            i64 right_fixed = left_fixed + i64(m->spr_w[s.id]) * FIXED_UNIT;
            s.right = SW / 2 + (mul64(right_fixed, xscale) >> 32);
            i64 span = std::max<i64>(s.right - s.left, 1);
            s.hstep = tdiv(i64(m->spr_w[s.id]) << 16, span);
            // engine.py:14200-14228
            s.yscale = tdiv(FOCAL_Y_FIXED << 12, std::max<i64>(s.depth_fixed, SPRITE_MIN_DEPTH_FIXED));
            s.texmid = i64(m->spr_top[s.id]) * FIXED_UNIT - round_to_i64((L.view_z - s.z) * float(FIXED_UNIT));
            s.top_fixed = L.center_fixed - (mul64(s.texmid, s.yscale) >> 16);
            s.iscale = tdiv(UINT32_MASK, std::max<i64>(s.yscale, 1));
            s.light = m->sector_lights[sector_at(s.x, s.y)];
        }
        std::vector<int> order(A);
        for (int x = 0; x < SW; ++x) {
            // column candidates (engine.py:14694-14768)
            int count = 0;
            int bw = blocking_wall[x];
            const WallGeom &bg = geom[bw];
            i64 bnear = std::min(bg.dl, bg.dr), bfar = std::max(bg.dl, bg.dr);
            const float *bl = m->walls + 4 * bw;
            float bdx = bl[2] - bl[0], bdy = bl[3] - bl[1];
            bool owns = (x >= bg.sl) && (x < bg.sr);
            for (int a = 0; a < A; ++a) {
                const Spr &s = sp[a];
                bool ray_visible = s.depth < wall_distance[x];
                float bside = bdx * (s.y - bl[1]) - bdy * (s.x - bl[0]);
                bool behind = (bnear > s.depth_fixed) || ((bfar > s.depth_fixed) && (bside <= 0));
                ray_visible = ray_visible || !owns || behind;
                bool inside = (x >= s.left) && (x < s.right);
                if (inside && s.alive && (s.depth > 0) && ray_visible) order[count++] = a;
            }
            if (!count) continue;
            // topk(largest=False, sorted=True): ascending depth.  Among exactly equal depths the reference's order is
            // whatever torch.topk's partial sort leaves (it varies from column to column of one frame); here, and in the
            // HIP path, equal depths keep slot order.
            std::stable_sort(order.begin(), order.begin() + count, [&](int a, int b) { return sp[a].depth < sp[b].depth; });
            for (int layer = count - 1; layer >= 0; --layer) {
                const Spr &s = sp[order[layer]];
                int width = m->spr_w[s.id], height = m->spr_h[s.id];
                i64 su = mul64(i64(x) - s.left, s.hstep) >> 16;
                if (!(su >= 0 && su < width)) continue;
                float light = s.light + float(L.flash_light * 16);
                if (s.fullbright) light = 255.0f;
                // engine.py:10576-10586 (float shade)
                float base_shade = 61.0f - light / 4.0f;
                // `1280.0 / distance` divides a Python number by a tensor: Torch evaluates it as reciprocal(distance) * 1280
                // (Tensor.__rtruediv__), two roundings, not one division
                float visibility = std::min((1.0f / std::max(s.depth, 1.0f)) * 1280.0f, 24.0f);
                i64 shade = clampi((i64)std::floor(base_shade - visibility), 0, 31);
                for (int y = 0; y < VH; ++y) {
                    size_t i = size_t(y) * SW + x;
                    i64 fraction = s.texmid + mul64(i64(y), s.iscale) - (mul64(L.center_fixed - FIXED_UNIT, s.iscale) >> 16);
                    i64 sv = fraction >> 16;
                    if (!(sv >= 0 && sv < height)) continue;
                    bool visible;
                    int cw = sprite_clip_wall[i];
                    if (cw >= 0) {
                        const WallGeom &cg = geom[cw];
                        i64 cnear = std::min(cg.dl, cg.dr), cfar = std::max(cg.dl, cg.dr);
                        const float *cl = m->walls + 4 * cw;
                        float cdx = cl[2] - cl[0], cdy = cl[3] - cl[1];
                        float side = cdx * (s.y - cl[1]) - cdy * (s.x - cl[0]);
                        visible = (cnear > s.depth_fixed) || ((cfar > s.depth_fixed) && (side <= 0));
                    } else {
                        visible = s.depth < sprite_clip_depth[i];
                    }
                    if (!visible) continue;
                    size_t t = (size_t(s.id) * m->spr_max_h + sv) * m->spr_max_w + su;
                    if (!m->spr_opaque[t]) continue;
                    i64 post_screen_top = (s.top_fixed + mul64(s.yscale, m->spr_post_top[t])) >> 16;
                    if (i64(y) < post_screen_top) continue;
                    // engine.py:14914-14939: opaque, additive table or translucent table over the pixel below
                    uint8_t lit = m->colormap[shade * 256 + m->spr_atlas[t]];
                    if (s.style == -2) lit = m->translucent_lut[size_t(frame[i]) * 256 + lit];
                    else if (s.style >= 0) lit = m->additive_luts[(size_t(s.style > 1 ? 1 : s.style) * 256 + frame[i]) * 256 + lit];
                    frame[i] = lit;
                }
            }
        }
    }
};

// _native_render_hitscan_decals (engine.py:13747-13991) for one lane: decals in paint order over the
// wall pass's picture, each drawn only where the scene depth is the decal's own ray distance.
void render_decals(Oracle &o, const gd_overlay_desc &ov, const gd_lanes_desc *lanes, int n) {
    const gd_map_desc *m = o.m;
    const Lane &L = o.L;
    const int D = lanes->decal_slots;
    const float focal_length = 192.0f;
    const float center = 104.0f + L.pitch_offset;
    const int width = ov.decal_max_w;
    for (int k = 0; k < D; ++k) {
        const int32_t *state = lanes->decal_state + (size_t(n) * D + k) * 3;
        const float *geom = lanes->decal_geom + (size_t(n) * D + k) * 4;
        const bool alive = state[2] != 0;
        const int wall_index = int(clampi(state[0], 0, o.W - 1));
        const int style = state[1];
        const int variant = style % 5;
        const bool flip_x = (style / 5) % 2, flip_y = (style / 10) % 2;
        const int side = style / 20;
        const float along_wall = geom[0], impact_z = geom[1], tangent_x = geom[2], tangent_y = geom[3];
        const float *wl = m->walls + 4 * wall_index;
        const float wvx = wl[2] - wl[0], wvy = wl[3] - wl[1];
        const float impact_x = wl[0] + along_wall * wvx, impact_y = wl[1] + along_wall * wvy;
        const float left_offset = float(ov.decal_left[variant]);
        const float back = left_offset * 0.5f, forth = (float(width) - left_offset) * 0.5f;
        const float left_x = impact_x - tangent_x * back, left_y = impact_y - tangent_y * back;
        const float right_x = impact_x + tangent_x * forth, right_y = impact_y + tangent_y * forth;
        const float seg_x = right_x - left_x, seg_y = right_y - left_y;
        // FWallCoords::Init on the two fixed-point endpoints (engine.py:13836-13887)
        i64 ex[2] = {round_to_i64(left_x * float(FIXED_UNIT)), round_to_i64(right_x * float(FIXED_UNIT))};
        i64 ey[2] = {round_to_i64(left_y * float(FIXED_UNIT)), round_to_i64(right_y * float(FIXED_UNIT))};
        i64 tx[2], ty[2];
        for (int e = 0; e < 2; ++e) {
            i64 rx = ex[e] - L.view_x_fixed, ry = ey[e] - L.view_y_fixed;
            tx[e] = (rx * L.vsin - ry * L.vcos) >> 20;
            ty[e] = (rx * L.vcos + ry * L.vsin) >> 20;
        }
        const i64 tx1 = tx[0], tx2 = tx[1], ty1 = ty[0], ty2 = ty[1];
        const i64 center_fixed = 160 * FIXED_UNIT;
        i64 projected_left = ((center_fixed + tdiv(tx1 * center_fixed, ty1 == 0 ? 1 : ty1)) >> 16) + (tx1 >= 0);
        i64 projected_right = ((center_fixed + tdiv(tx2 * center_fixed, ty2 == 0 ? 1 : ty2)) >> 16) + (tx2 >= 0);
        i64 left_den = tx1 - tx2 - ty2 + ty1, right_den = ty2 - ty1 - tx2 + tx1;
        bool left_inside = (tx1 >= -ty1) && (tx1 <= ty1) && (ty1 != 0);
        bool right_inside = (tx2 <= ty2) && (tx2 >= -ty2) && (ty2 != 0);
        bool left_clipped = (tx1 < -ty1) && (tx2 >= -ty2) && (left_den != 0);
        bool right_clipped = (tx2 > ty2) && (tx1 <= ty1) && (right_den != 0);
        i64 screen_left = left_inside ? clampi(projected_left, 0, SW) : 0;
        i64 screen_right = right_inside ? clampi(projected_right, 0, SW) : SW;
        bool projected = alive && (left_inside || left_clipped) && (right_inside || right_clipped) && (screen_right > screen_left);
        float viewer_cross = wvx * (L.y - wl[1]) - wvy * (L.x - wl[0]);
        bool side_visible = (viewer_cross > 0 ? 1 : 0) == side;
        int sector = m->wall_sectors[2 * wall_index + (side < 0 ? 0 : (side > 1 ? 1 : side))];
        if (sector < 0) sector = 0;
        bool horizontal = std::fabs(wvy) < 1e-6f, vertical = std::fabs(wvx) < 1e-6f;
        float light = m->sector_lights[sector] + (vertical ? 16.0f : (horizontal ? -16.0f : 0.0f));
        light = light + float(L.flash_light * 16);
        const int height = ov.decal_h[variant];
        const float top_offset = float(ov.decal_top[variant]);
        if (!(projected && side_visible)) continue;
        for (int x = 0; x < SW; ++x) {
            float col = (float(x) - 160.0f) / 160.0f;
            float rx = L.fcos + L.fsin * col, ry = L.fsin - L.fcos * col;
            float off_x = left_x - L.x, off_y = left_y - L.y;
            float den = rx * seg_y - ry * seg_x;
            float safe = std::fabs(den) < 1e-6f ? 1.0f : den;
            float distance = (off_x * seg_y - off_y * seg_x) / safe;
            float decal_along = (off_x * ry - off_y * rx) / safe;
            bool inside_column = (x >= screen_left) && (x < screen_right) && (std::fabs(den) >= 1e-6f) && (distance > 0);
            if (!inside_column) continue;
            i64 tu = clampi(i64(std::floor(decal_along * float(width))), 0, width - 1);
            if (flip_x) tu = width - 1 - tu;
            float safe_distance = std::max(distance, 1e-6f);
            // `focal_length * _BULLET_DECAL_SCALE / distance` divides a Python number by a tensor, which Torch evaluates as
            // reciprocal(distance) * 96 (Tensor.__rtruediv__): two roundings, not one division
            float vertical_scale = (1.0f / safe_distance) * 96.0f;
            float top = center - ((impact_z + top_offset * 0.5f) - L.view_z) * focal_length / safe_distance;
            i64 depth_fixed = round_to_i64(safe_distance * 4096.0f);
            i64 visibility = tdiv(WALL_VISIBILITY_FIXED << 12, std::max<i64>(depth_fixed, 1));
            i64 shade = Oracle::wall_shade(light, visibility);
            for (int y = 0; y < VH; ++y) {
                i64 tv = i64(std::floor((float(y) - top) / vertical_scale));
                if (!(tv >= 0 && tv < height)) continue;
                if (flip_y) tv = height - 1 - tv;
                size_t i = size_t(y) * SW + x;
                if (!(std::fabs(o.scene_depth[i] - distance) <= 1e-3f)) continue;
                uint8_t source = ov.decal_atlas[(size_t(variant) * ov.decal_max_h + tv) * ov.decal_max_w + tu];
                if (source == 0) continue;
                uint8_t opacity = ov.decal_opacity_lut[shade * 256 + source];
                o.frame[i] = ov.decal_black_lut[size_t(opacity) * 256 + o.frame[i]];
            }
        }
    }
}

// _policy_area_grayscale_kernel (_triton_kernels.py:120-177) for one lane
// engine.py:15385-15397: PLAYPAL after the pickup (gold) and damage (red) screen blends, float32 op by op
void blended_palette(const uint8_t *playpal, const float *blend, uint8_t *out) {
    static const float gold[3] = {215.0f, 186.0f, 69.0f}, red[3] = {255.0f, 0.0f, 0.0f};
    for (int k = 0; k < 768; ++k) {
        if (!blend) { out[k] = playpal[k]; continue; }
        float v = float(playpal[k]) * (1.0f - blend[0]) + gold[k % 3] * blend[0];
        v = v * (1.0f - blend[1]) + red[k % 3] * blend[1];
        float clamped = std::min(std::max(v, 0.0f), 255.0f);
        out[k] = uint8_t(clamped);
    }
}

void observe_lane(const uint8_t *indexed, int source_rows, const uint8_t *playpal, uint8_t *obs) {
    for (int oy = 0; oy < GD_OBS_SIZE; ++oy) {
        for (int ox = 0; ox < GD_OBS_SIZE; ++ox) {
            int y_start = oy * 240, y_end = (oy + 1) * 240, x_start = ox * 320, x_end = (ox + 1) * 320;
            int rs = 0, gs = 0, bs = 0;
            for (int sy = 0; sy < 5; ++sy) {   // SAMPLE_BLOCK=32 -> rows 0..6, cols 0..4; overlap masks the rest
                int source_y = y_start / 84 + sy;
                int y_overlap = std::min(y_end, (source_y + 1) * 84) - std::max(y_start, source_y * 84);
                if (source_y >= source_rows || y_overlap <= 0) continue;
                for (int sx = 0; sx < 5; ++sx) {
                    int source_x = x_start / 84 + sx;
                    int x_overlap = std::min(x_end, (source_x + 1) * 84) - std::max(x_start, source_x * 84);
                    if (source_x >= 320 || x_overlap <= 0) continue;
                    int weight = (y_overlap * x_overlap) / 48;
                    int p = indexed[source_y * 320 + source_x];
                    rs += playpal[p * 3] * weight; gs += playpal[p * 3 + 1] * weight; bs += playpal[p * 3 + 2] * weight;
                }
            }
            int r = (rs + 800) / 1600, g = (gs + 800) / 1600, b = (bs + 800) / 1600;
            obs[oy * GD_OBS_SIZE + ox] = (uint8_t)((r * 77 + g * 150 + b * 29 + 128) / 256);
        }
    }
}

// engine.py:9545-9548 (roll + append) and engine.py:2443-2450 (reset fill)
void stack_lane(const uint8_t *obs, uint8_t *frames, bool reset, int stack_mode) {
    const size_t F = size_t(GD_OBS_SIZE) * GD_OBS_SIZE;
    if (reset) {
        for (int k = 0; k < GD_FRAME_STACK; ++k) std::memcpy(frames + k * F, obs, F);
    } else if (stack_mode == GD_STACK_STEP) {
        std::memmove(frames, frames + F, (GD_FRAME_STACK - 1) * F);
        std::memcpy(frames + (GD_FRAME_STACK - 1) * F, obs, F);
    }
}

thread_local std::string g_error;

}  // namespace

extern "C" {

const char *gdo_last_error(void) { return g_error.c_str(); }

// Debug taps (host pointers, any may be null), all for lane `debug_lane`.
typedef struct gdo_debug {
    int32_t debug_lane;
    uint8_t *flats_frame;        // [208,320] output of _native_render_flats
    float *surface_depth;        // [208,320]
    float *scene_surface_depth;  // [208,320]
    float *distances;            // [320,W]
    float *along;                // [320,W]
    uint8_t *geometric, *projected, *left_edge;  // [320,W]
    int64_t *geometry;           // [W,4] screen_left, screen_right, depth_left, depth_right
    int64_t *horizontal_offset;  // [320,W]
    int64_t *vertical_step;      // [320,W]
    int64_t *visibility;         // [320,W,2]
    float *scene_depth;          // [208,320]
    float *sprite_clip_depth;    // [208,320]
    int32_t *sprite_clip_wall;   // [208,320]
    int32_t *sector;             // [N] current sector of every lane
    uint8_t *walls_frame;        // [208,320] frame after walls/planes/masked, before sprites
} gdo_debug;

// ---------------------------------------------------------------------------------------------
// Overlay layers: weapon psprite (engine.py:14997-15110) and status bar (engine.py:15153-15267),
// restated as the reference's CPU path does them: whole-patch composites in draw order.
// ---------------------------------------------------------------------------------------------
static gd_overlay_desc g_overlays;
static bool g_overlays_set = false;

int gdo_set_overlays(const gd_overlay_desc *overlays) {
    g_overlays_set = overlays != nullptr;
    if (overlays) g_overlays = *overlays;     // host pointers, kept by the caller
    return GD_OK;
}

// _native_composite_weapon_patch (engine.py:14997-15049) over the 320x208 view of one lane
static void composite_weapon_patch(uint8_t *view, int64_t patch, int64_t horizontal_fixed, int64_t vertical_fixed, bool visible) {
    const gd_overlay_desc &o = g_overlays;
    if (!visible) return;
    const int64_t FIXED = 65536;
    const int64_t width = o.weapon_w[patch], height = o.weapon_h[patch];
    const int64_t left_offset = o.weapon_left[patch], top_offset = o.weapon_top[patch];
    const int64_t screen_left = (horizontal_fixed - left_offset * FIXED) >> 16;
    const int64_t weapon_top_fixed = 32 * FIXED + 0x6000;
    const int64_t texture_mid_fixed = 100 * FIXED - weapon_top_fixed - vertical_fixed + top_offset * FIXED;
    const int64_t psprite_y_scale_fixed = int64_t(GD_SCREEN_HEIGHT) * FIXED / 200;
    const int64_t psprite_y_iscale_fixed = int64_t(0xFFFFFFFFLL) / psprite_y_scale_fixed;
    for (int y = 0; y < VH; ++y) {
        const int64_t screen_delta = int64_t(y) - (VH / 2 - 1);
        const int64_t source_y = (texture_mid_fixed + screen_delta * psprite_y_iscale_fixed) >> 16;
        for (int x = 0; x < SW; ++x) {
            const int64_t source_x = int64_t(x) - screen_left;
            const bool inside = source_x >= 0 && source_x < width && source_y >= 0 && source_y < height;
            if (!inside) continue;
            const int64_t cx = std::min<int64_t>(std::max<int64_t>(source_x, 0), o.weapon_max_w - 1);
            const int64_t cy = std::min<int64_t>(std::max<int64_t>(source_y, 0), o.weapon_max_h - 1);
            const size_t t = (size_t(patch) * o.weapon_max_h + size_t(cy)) * o.weapon_max_w + size_t(cx);
            if (o.weapon_opaque[t]) view[size_t(y) * SW + x] = o.weapon_atlas[t];
        }
    }
}

// _native_draw_hud_patch (engine.py:15153-15184) on a [32,320] canvas
static void draw_hud_patch(uint8_t *canvas, int patch, int x, int y) {
    const gd_overlay_desc &o = g_overlays;
    const int rows = GD_SCREEN_HEIGHT - VH;
    x -= o.hud_left[patch];
    y -= o.hud_top[patch];
    const int width = o.hud_w[patch], height = o.hud_h[patch];
    if (width <= 0 || height <= 0) return;
    const int source_x = std::max(-x, 0), source_y = std::max(-y, 0);
    const int target_x = std::max(x, 0), target_y = std::max(y, 0);
    const int copy_width = std::min(width - source_x, SW - target_x);
    const int copy_height = std::min(height - source_y, rows - target_y);
    if (copy_width <= 0 || copy_height <= 0) return;
    for (int r = 0; r < copy_height; ++r) for (int c = 0; c < copy_width; ++c) {
        const size_t t = (size_t(patch) * o.hud_max_h + size_t(source_y + r)) * o.hud_max_w + size_t(source_x + c);
        if (o.hud_opaque[t]) canvas[size_t(target_y + r) * SW + target_x + c] = o.hud_atlas[t];
    }
}

// _native_draw_hud_number (engine.py:15186-15207)
static void draw_hud_number(uint8_t *canvas, int value, int right, int y, bool small) {
    const gd_overlay_desc &o = g_overlays;
    char text[16];
    std::snprintf(text, sizeof(text), "%d", std::max(-99, std::min(value, 999)));
    const int digit_width = small ? 4 : 14, base = small ? 28 : 2;
    int x = right - int(std::strlen(text)) * digit_width;
    for (const char *c = text; *c; ++c) {
        if (*c == '-') { x += digit_width; continue; }
        const int patch = base + (*c - '0');
        const int glyph_x = x - o.hud_left[patch], glyph_y = y - o.hud_top[patch];
        draw_hud_patch(canvas, patch, glyph_x, glyph_y);
        x += digit_width;
    }
}

// _native_render_hud (engine.py:15232-15267) for one lane; `state` as gd_lanes_desc.hud_state
static void render_hud(uint8_t *canvas, const int32_t *state) {
    draw_hud_patch(canvas, 0, 0, 0);
    draw_hud_patch(canvas, 1, 104, 0);
    draw_hud_number(canvas, state[0], 44, 3, false);
    draw_hud_number(canvas, state[1], 90, 3, false);
    draw_hud_patch(canvas, 12, 90, 3);
    draw_hud_number(canvas, state[2], 221, 3, false);
    draw_hud_patch(canvas, 12, 221, 3);
    draw_hud_patch(canvas, state[3], 143, 0);
    const int positions[6][2] = {{111, 4}, {123, 4}, {135, 4}, {111, 14}, {123, 14}, {135, 14}};
    for (int weapon_index = 0; weapon_index < 6; ++weapon_index) {
        const bool owned = weapon_index < 5 && ((state[4] >> weapon_index) & 1);
        draw_hud_patch(canvas, owned ? 28 + weapon_index + 2 : 38 + weapon_index, positions[weapon_index][0], positions[weapon_index][1]);
    }
    const int maximum[4] = {200, 50, 50, 300};
    for (int row = 0; row < 4; ++row) {
        const int y = 5 + row * 6;
        draw_hud_number(canvas, state[5 + row], 288, y, true);
        draw_hud_number(canvas, maximum[row], 314, y, true);
    }
}

// Full frame for lanes [lane_begin, lane_end): indexed, obs, stack, rgb as in gd_render.
int gdo_render(const gd_map_desc *map, const gd_lanes_desc *lanes, const gd_frame_out *out,
               int32_t lane_begin, int32_t lane_end, const float *cosine_correction, const gdo_debug *dbg) {
    if (!map || !lanes || !out || !cosine_correction) { g_error = "null argument"; return GD_E_ARG; }
    if (map->struct_size != sizeof(gd_map_desc) || lanes->struct_size != sizeof(gd_lanes_desc) || out->struct_size != sizeof(gd_frame_out)) {
        g_error = "a descriptor's struct_size does not match this build of the header";
        return GD_E_ARG;
    }
    if (out->obs_source_rows != 0 && out->obs_source_rows != VH && out->obs_source_rows != GD_SCREEN_HEIGHT) { g_error = "obs_source_rows"; return GD_E_ARG; }
    const int source_rows = out->obs_source_rows == GD_SCREEN_HEIGHT ? GD_SCREEN_HEIGHT : VH;
    Oracle o(map);
    const size_t W = map->wall_count;
    std::vector<uint8_t> obs(size_t(GD_OBS_SIZE) * GD_OBS_SIZE);
    std::vector<uint8_t> full(size_t(GD_SCREEN_HEIGHT) * SW);
    const bool profile = std::getenv("GDO_PROFILE") != nullptr;
    double t_setup = 0, t_flats = 0, t_walls = 0, t_sprites = 0, t_obs = 0;
    auto now = [] { return std::chrono::duration<double>(std::chrono::steady_clock::now().time_since_epoch()).count(); };
    for (int n = lane_begin; n < lane_end; ++n) {
        double t0 = now();
        o.setup_lane(lanes, n);
        for (int w = 0; w < o.W; ++w) {
            o.wall_geometry(w);
            o.vis[2 * w] = o.wall_visibility_side(o.tx[2 * w], o.tx[2 * w + 1], o.ty[2 * w], o.ty[2 * w + 1]);
            o.vis[2 * w + 1] = o.wall_visibility_side(o.tx[2 * w + 1], o.tx[2 * w], o.ty[2 * w + 1], o.ty[2 * w]);
        }
        o.fragment_geometry();
        o.portal_intersections();
        o.texture_mapping();
        double t1 = now();
        o.render_flats(lanes->ray_cos + size_t(n) * SW, lanes->ray_sin + size_t(n) * SW, cosine_correction);
        double t2 = now();
        const bool tap = dbg && dbg->debug_lane == n;
        if (dbg && dbg->sector) dbg->sector[n] = o.L.sector;
        if (tap) {
            const size_t PX = size_t(VH) * SW;
            if (dbg->flats_frame) std::memcpy(dbg->flats_frame, o.frame.data(), PX);
            if (dbg->surface_depth) std::memcpy(dbg->surface_depth, o.surface_depth.data(), PX * 4);
            if (dbg->scene_surface_depth) std::memcpy(dbg->scene_surface_depth, o.scene_surface_depth.data(), PX * 4);
            if (dbg->distances) std::memcpy(dbg->distances, o.dist.data(), SW * W * 4);
            if (dbg->along) std::memcpy(dbg->along, o.along.data(), SW * W * 4);
            if (dbg->geometric) std::memcpy(dbg->geometric, o.geo.data(), SW * W);
            if (dbg->projected) std::memcpy(dbg->projected, o.proj.data(), SW * W);
            if (dbg->left_edge) std::memcpy(dbg->left_edge, o.ledge.data(), SW * W);
            if (dbg->geometry) for (size_t w = 0; w < W; ++w) {
                dbg->geometry[4 * w] = o.geom[w].sl; dbg->geometry[4 * w + 1] = o.geom[w].sr;
                dbg->geometry[4 * w + 2] = o.geom[w].dl; dbg->geometry[4 * w + 3] = o.geom[w].dr;
            }
            if (dbg->horizontal_offset) std::memcpy(dbg->horizontal_offset, o.hoff.data(), SW * W * 8);
            if (dbg->vertical_step) std::memcpy(dbg->vertical_step, o.vstep.data(), SW * W * 8);
            if (dbg->visibility) for (int x = 0; x < SW; ++x) for (size_t w = 0; w < W; ++w) for (int s = 0; s < 2; ++s)
                {   // the tap is _native_portal_intersections' own tensor, before fragments replace split linedefs
                    const WallVis &v = o.vis[2 * w + s];
                    dbg->visibility[(size_t(x) * W + w) * 2 + s] = v.light_left + (i64(x) - v.screen_left) * v.light_step;
                }
        }
        double t3 = now();
        o.render_portal_walls();
        double t4 = now();
        if (tap) {
            const size_t PX = size_t(VH) * SW;
            if (dbg->scene_depth) std::memcpy(dbg->scene_depth, o.scene_depth.data(), PX * 4);
            if (dbg->sprite_clip_depth) std::memcpy(dbg->sprite_clip_depth, o.sprite_clip_depth.data(), PX * 4);
            if (dbg->sprite_clip_wall) std::memcpy(dbg->sprite_clip_wall, o.sprite_clip_wall.data(), PX * 4);
            if (dbg->walls_frame) std::memcpy(dbg->walls_frame, o.frame.data(), PX);
        }
        double t5 = now();
        if (g_overlays_set && g_overlays.decal_variant_count > 0 && lanes->decal_slots > 0 && lanes->decal_state && lanes->decal_geom)
            render_decals(o, g_overlays, lanes, n);
        o.render_sprites(lanes, n);
        double t6 = now();
        t_setup += t1 - t0; t_flats += t2 - t1; t_walls += t4 - t3; t_sprites += t6 - t5;
        std::memcpy(full.data(), o.frame.data(), size_t(VH) * SW);
        std::memset(full.data() + size_t(VH) * SW, 0, size_t(GD_SCREEN_HEIGHT - VH) * SW);
        if (g_overlays_set && lanes->weapon_state && g_overlays.weapon_patch_count > 0) {
            const int64_t *state = lanes->weapon_state + size_t(n) * 5;
            composite_weapon_patch(full.data(), state[0], state[2], state[3], state[4] != 0);
            composite_weapon_patch(full.data(), std::max<int64_t>(state[1], 0), state[2], state[3], state[4] != 0 && state[1] >= 0);
        }
        if (g_overlays_set && lanes->hud_state && g_overlays.hud_patch_count > 0)
            render_hud(full.data() + size_t(VH) * SW, lanes->hud_state + size_t(n) * 9);
        if (out->indexed) std::memcpy(out->indexed + size_t(n) * full.size(), full.data(), full.size());
        uint8_t palette[768];
        blended_palette(map->playpal, lanes->screen_blend ? lanes->screen_blend + 2 * size_t(n) : nullptr, palette);
        if (out->obs || out->frames) {
            observe_lane(full.data(), source_rows, palette, obs.data());  // 208: HUD rows masked black (engine.py:15444-15450)
            if (out->obs) std::memcpy(out->obs + size_t(n) * obs.size(), obs.data(), obs.size());
            if (out->frames) stack_lane(obs.data(), out->frames + size_t(n) * GD_FRAME_STACK * obs.size(), out->reset_mask && out->reset_mask[n], out->stack_mode);
        }
        if (out->rgb) {
            uint8_t *rgb = out->rgb + size_t(n) * full.size() * 3;
            for (size_t i = 0; i < full.size(); ++i) for (int c = 0; c < 3; ++c) rgb[i * 3 + c] = palette[full[i] * 3 + c];
        }
    }
    if (profile) std::fprintf(stderr, "oracle lanes %d: setup %.3fs flats %.3fs walls %.3fs sprites %.3fs\n", lane_end - lane_begin, t_setup, t_flats, t_walls, t_sprites);
    return GD_OK;
}

// gdo_render with the lanes dealt out to `threads` host threads (lanes are independent; every thread renders a
// contiguous share into its own rows of the outputs).  Debug taps are not available here.  The CPU baseline of the
// benchmark: the same scalar restatement on all the host's cores.
int gdo_render_parallel(const gd_map_desc *map, const gd_lanes_desc *lanes, const gd_frame_out *out,
                        int32_t lane_begin, int32_t lane_end, const float *cosine_correction, int32_t threads) {
    if (threads < 1 || lane_end < lane_begin) { g_error = "bad thread count or lane range"; return GD_E_ARG; }
    const int total = lane_end - lane_begin;
    if (threads > total) threads = total > 0 ? total : 1;
    std::vector<int> codes(threads, GD_OK);
    std::vector<std::string> errors(threads);
    std::vector<std::thread> pool;
    for (int t = 0; t < threads; ++t) {
        const int first = lane_begin + (int)((long long)total * t / threads), last = lane_begin + (int)((long long)total * (t + 1) / threads);
        pool.emplace_back([=, &codes, &errors] {
            codes[t] = gdo_render(map, lanes, out, first, last, cosine_correction, nullptr);
            if (codes[t] != GD_OK) errors[t] = g_error;
        });
    }
    for (std::thread &worker : pool) worker.join();
    for (int t = 0; t < threads; ++t) if (codes[t] != GD_OK) { g_error = errors[t]; return codes[t]; }
    return GD_OK;
}

int gdo_observe(const uint8_t *indexed, int32_t source_rows, const uint8_t *playpal, int32_t lane_count,
                uint8_t *obs, uint8_t *frames, const uint8_t *reset_mask, int32_t stack_mode) {
    if (!indexed || !playpal || (source_rows != 208 && source_rows != 240)) { g_error = "bad argument"; return GD_E_ARG; }
    std::vector<uint8_t> one(size_t(GD_OBS_SIZE) * GD_OBS_SIZE);
    for (int n = 0; n < lane_count; ++n) {
        observe_lane(indexed + size_t(n) * source_rows * SW, source_rows, playpal, one.data());
        if (obs) std::memcpy(obs + size_t(n) * one.size(), one.data(), one.size());
        if (frames) stack_lane(one.data(), frames + size_t(n) * GD_FRAME_STACK * one.size(), reset_mask && reset_mask[n], stack_mode);
    }
    return GD_OK;
}

// Dense forms of the pair/bridge relations the reference precomputes (engine.py:399-484, 1597-1612),
// evaluated through the same on-the-fly functions the render loop uses. Arrays are [W,W] / [2,W,W].
void gdo_relation_tables(const gd_map_desc *map, uint8_t *same_pair, uint8_t *opposing, int64_t *portal_bridge_index,
                         uint8_t *portal_bridge_mask, int64_t *sector_bridge_index, uint8_t *sector_bridge_mask) {
    Oracle o(map);
    const size_t W = map->wall_count;
    for (size_t a = 0; a < W; ++a) for (size_t b = 0; b < W; ++b) {
        same_pair[a * W + b] = o.same_pair(int(a), int(b));
        opposing[a * W + b] = o.opposing(int(a), int(b));
        for (int slot = 0; slot < 2; ++slot) {
            int index;
            portal_bridge_mask[(slot * W + a) * W + b] = o.portal_bridge(slot, int(a), int(b), &index);
            portal_bridge_index[(slot * W + a) * W + b] = index;
            sector_bridge_mask[(slot * W + a) * W + b] = o.sector_bridge(slot, int(a), int(b), &index);
            sector_bridge_index[(slot * W + a) * W + b] = index;
        }
    }
}

// Copies the rule-coverage counters (COV_COUNT values) and optionally clears them.
int gdo_coverage(long long *out, int capacity, int reset) {
    int n = capacity < COV_COUNT ? capacity : COV_COUNT;
    for (int i = 0; i < n; ++i) out[i] = g_coverage[i];
    if (reset) std::memset(g_coverage, 0, sizeof(g_coverage));
    return COV_COUNT;
}

void gdo_fine_tables(int64_t *fine_sine, int64_t *fine_tangent) {
    build_tables();
    std::memcpy(fine_sine, g_fine_sine, sizeof(g_fine_sine));
    std::memcpy(fine_tangent, g_fine_tangent, sizeof(g_fine_tangent));
}

}  // extern "C"
