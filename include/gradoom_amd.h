/*
 * gradoom_amd.h - C ABI of the MI355X (gfx950) batched software renderer and
 * observation pipeline that replaces the reference's Torch "reference" render
 * path behind GraDoomVecEnv (reset_device / step_and_reset_device / render).
 *
 * Every pointer in gd_map_desc / gd_lanes_desc / gd_frame_out is a DEVICE
 * pointer when passed to the gd_* entry points of libgradoom_amd.so, and a
 * HOST pointer when the same structs are handed to the CPU oracle
 * (liboracle.so, test infrastructure only).  The structs themselves live in
 * host memory.  Entry points return 0 on success or a negative GD_E_* code;
 * gd_last_error() returns a message for the calling thread.
 *
 * Host threads: the library takes no locks.  Calls that use the same renderer,
 * and gd_render_static calls on the same GPU (its first call on a device looks
 * up that device's working array), must come from one host thread at a time;
 * calls on different renderers are independent.
 *
 * Names follow the reference's domain: lanes (batched environments), linedefs
 * ("walls"), sectors, flats, visplanes, drawsegs, sprites, PLAYPAL, COLORMAP.
 */
#ifndef GRADOOM_AMD_H
#define GRADOOM_AMD_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define GD_SCREEN_WIDTH 320
#define GD_VIEW_HEIGHT 208   /* world view rows; rows 208..239 are the status bar */
#define GD_SCREEN_HEIGHT 240
#define GD_OBS_SIZE 84
#define GD_FRAME_STACK 4

/* gd_frame_out.stack_mode */
#define GD_STACK_STEP 0   /* every lane: roll by one, append (engine.py:9545-9548); lanes with reset_mask set: 4 copies */
#define GD_STACK_RESET 1  /* lanes with reset_mask set: 4 copies (engine.py:2443-2450); other lanes untouched */

/* gd_frame_out.final_frames_layout: how final_frames is laid out (obs_layout of env.py:351, 678-680) */
#define GD_LAYOUT_CHW 0   /* [N,4,84,84], like frames */
#define GD_LAYOUT_HWC 1   /* [N,84,84,4]: what frames.permute(0, 2, 3, 1) reads, made contiguous */

/*
 * Layout version of the structs below.  Every descriptor also starts with its own sizeof, which each entry
 * point checks: a caller built against another header gets GD_E_ARG instead of a wild read.
 */
#define GD_ABI_VERSION 4

#define GD_OK 0
#define GD_E_ARG (-1)       /* bad argument: null pointer, negative count, size over a limit */
#define GD_E_HIP (-2)       /* a HIP runtime call failed */
#define GD_E_UNSUPPORTED (-3) /* reserved: a map feature this build does not implement (none at present) */

/*
 * Immutable map, atlases and look-up tables.
 * Mirrors the tensors of DeviceScenario (reference src/gradoom/engine.py:607-719)
 * that the native render path reads, plus compact forms of the derived tables
 * the reference builds in DeviceScenario.from_host (engine.py:721-849) and in
 * TorchDeathmatchEngine.__init__ (engine.py:1527-1634).  The reference's dense
 * [W,W] and [2,W,W] pair/bridge tables are replaced by a vertex -> linedef CSR
 * from which the same answers are derived on the fly.
 */
typedef struct gd_map_desc {
    uint32_t struct_size;    /* sizeof(gd_map_desc) of the header the caller was built with */
    int32_t wall_count;      /* W linedefs */
    int32_t sector_count;    /* S */
    int32_t vertex_count;    /* V distinct endpoints (exact float32 equality) */
    int32_t texture_count;   /* T */
    int32_t tex_max_h, tex_max_w;
    int32_t sprite_count;    /* P raw sprite patches */
    int32_t spr_max_h, spr_max_w;
    int32_t blocking_count;  /* B one-sided / blocking linedefs */
    int32_t neighbor_slots;  /* K columns of endpoint_neighbors */
    int32_t direct_neighbors;/* 1: every linedef has <=1 start and <=1 end neighbour (engine.py:1558) */
    int32_t floor_level_count, ceil_level_count; /* distinct plane heights */
    int32_t grid_nx, grid_ny;/* point-location grid (cells of grid_cell map units) */
    int32_t fine_nx, fine_ny;/* fine point-location raster (cells of fine_cell map units, same origin) */
    int32_t fragment_slots;  /* F >= 1 projection fragments per split linedef (engine.py:620-621) */
    int32_t split_count;     /* SP linedefs whose projection fragments differ from the linedef itself */
    float grid_min_x, grid_min_y, grid_cell, fine_cell;

    const float *walls;              /* [W,4] x1,y1,x2,y2 (portal_walls) */
    const int32_t *walls_fixed;      /* [W,4] rint(walls*65536) (engine.py:10876) */
    const int32_t *wall_sectors;     /* [W,2] front, back (-1 = one-sided) */
    const int32_t *wall_vertex;      /* [W,2] vertex id of start, end */
    const int32_t *side_tex;         /* [W,2,3] middle,bottom,top texture id or -1 */
    const float *side_off;           /* [W,2,2] x,y texture offsets */
    const float *wall_len;           /* [W] floor(len+0.5) (engine.py:737-743) */
    const int32_t *endpoint_neighbors;      /* [W,K] (engine.py:833-849), self where unused */
    const uint8_t *endpoint_neighbor_starts;/* [W,K] */
    const uint8_t *endpoint_neighbor_ends;  /* [W,K] */
    const int32_t *direct_neighbor_table;   /* [W,4] engine.py:1558-1575 packed: start neighbour, end neighbour,
                                               start slot | end slot<<8 | has start<<16 | has end<<17, 0 */
    const int32_t *solid_bridge_start_ofs;  /* [W+1] CSR of engine.py:802-830 */
    const int32_t *solid_bridge_start_idx;
    const int32_t *solid_bridge_end_ofs;    /* [W+1] */
    const int32_t *solid_bridge_end_idx;
    const int32_t *vertex_wall_ofs;  /* [V+1] CSR vertex -> linedefs touching it, ascending */
    const int32_t *vertex_wall_idx;
    const int32_t *sector_wall_ofs;  /* [S+1] CSR sector -> linedefs with that sector on either side */
    const int32_t *sector_wall_idx;
    const int32_t *sector_edge_ofs;  /* [S+1] CSR rows of sector_edge_mask (scenario.py:906-916) */
    const int32_t *sector_edge_idx;
    const int32_t *blocking_walls;   /* [B] linedef index of each blocking segment, ascending */
    /* BSP fragments of split linedefs (scenario.py:420-454, portal_projection_fragments_fixed / _mask):
       OWallMost projects with the fragment that owns the column (engine.py:12310-12380) and wallscan
       light interpolates over it when the linedef has more than one (engine.py:11495-11545). */
    const int32_t *wall_split_slot;      /* [W] row of the linedef in the two tables below, -1 = not split */
    const int32_t *split_fragments_fixed;/* [SP,F,4] 16.16 x1,y1,x2,y2 */
    const uint8_t *split_fragment_mask;  /* [SP,F] 1 = fragment present */
    /* Point-location grid: the even-odd polygon tests of engine.py:9598-9617 and
       10994-11015 restricted, per cell, to the sectors and edges that can count there. */
    const int32_t *grid_cell_ofs;    /* [nx*ny+1] -> items */
    const int32_t *grid_item_sector; /* [items] ascending sector id within a cell; bit 30 set = the whole
                                        cell lies inside that sector (no edge list, no crossing test) */
    const int32_t *grid_item_edge_ofs;/* [items+1] -> grid_item_edges */
    const int32_t *grid_item_edges;  /* linedef ids */
    const uint32_t *fine_sector;     /* [fine_ny*fine_nx] bits 31..30: 0 = bits 0..15 name the one sector that
                                        contains the whole cell, bits 16..19 / 20..23 its index in floor_levels /
                                        ceil_levels (15 = not recorded); 1 = outside every sector; 2 = undecided
                                        (run the crossing test), bits 0..14 / 15..29 flag the floor_levels /
                                        ceil_levels entries that can win in the cell; 3 = undecided, levels
                                        unknown.  grid_cell must be 8 * fine_cell. */
    const float *floor_levels;       /* [floor_level_count] distinct floor heights, descending */
    const float *ceil_levels;        /* [ceil_level_count] distinct ceiling heights, ascending */

    const float *sector_heights;     /* [S,2] floor, ceiling */
    const float *sector_lights;      /* [S] */
    const int32_t *sector_floor_tex; /* [S] */
    const int32_t *sector_ceil_tex;  /* [S] */

    const uint8_t *tex_atlas;        /* [T,tex_max_h,tex_max_w] palette indices */
    const int32_t *tex_w;            /* [T] power of two */
    const int32_t *tex_h;            /* [T] power of two */
    const uint8_t *playpal;          /* [256,3] */
    const uint8_t *colormap;         /* [34,256] */

    const uint8_t *spr_atlas;        /* [P,spr_max_h,spr_max_w] */
    const uint8_t *spr_opaque;       /* [P,spr_max_h,spr_max_w] 0/1 */
    const uint8_t *spr_post_top;     /* [P,spr_max_h,spr_max_w] first row of the opaque run (engine.py:14230) */
    const int32_t *spr_w, *spr_h, *spr_left, *spr_top; /* [P] */
    /* Blend tables of styled sprites (engine.py:14920-14939): [style][pixel under the sprite][lit texel]. */
    const uint8_t *additive_luts;    /* [2,256,256] projectile_additive_luts */
    const uint8_t *translucent_lut;  /* [256,256] sprite_translucent_lut */
} gd_map_desc;

/*
 * Per-lane camera and sprite list for one frame.
 * x,y,angle,view_z and the retained fixed-point twins are the engine tensors
 * of the same names (engine.py:1669, 10648-10687).  ray_cos/ray_sin are
 * cos/sin(angle + native_ray_offsets) (engine.py:10966-10974) and sprite_depth
 * is dist*cos(wrap(atan2 - angle)) (engine.py:14684-14688): the host computes
 * these float32 transcendentals with the same Torch ops the reference uses so
 * the kernels only do +,-,*,/ and comparisons.
 */
typedef struct gd_lanes_desc {
    uint32_t struct_size;    /* sizeof(gd_lanes_desc) of the header the caller was built with */
    int32_t lane_count;       /* N; 0 is allowed: the call checks its arguments and does nothing */
    int32_t sprite_slots;     /* A sprites per lane (0 = none) */
    int32_t decal_slots;      /* D packed wall decals per lane (0 = none) */
    const float *x, *y;       /* [N] */
    const float *angle;       /* [N] radians */
    const float *view_z;      /* [N] */
    const int64_t *x_fixed, *y_fixed; /* [N] retained 16.16 */
    const int64_t *angle_bam; /* [N] retained unsigned 32-bit BAM */
    const int64_t *pitch_bam; /* [N] */
    const int64_t *flash_light; /* [N] extralight steps (x16) */
    const float *ray_cos, *ray_sin; /* [N,320] */
    const float *sprite_x, *sprite_y, *sprite_z; /* [N,A] */
    const float *sprite_depth;       /* [N,A] */
    const int32_t *sprite_id;        /* [N,A] */
    const uint8_t *sprite_alive;     /* [N,A] */
    const uint8_t *sprite_fullbright;/* [N,A] */
    /* Overlay layers, drawn after the sprites when the renderer holds overlay patches
       (gd_renderer_set_overlays); either pointer may be null to skip that layer. */
    const int64_t *weapon_state;    /* [N,5] psprite of engine.py:15051-15110: patch id, muzzle flash patch id
                                       (-1 = none), horizontal offset (bob) 16.16, vertical offset 16.16,
                                       visible (0/1) */
    const int32_t *hud_state;       /* [N,9] status bar of engine.py:15232-15267: ready ammo, health, armor,
                                       face patch id, owned weapon bits (bit k = weapon k+1, k < 5),
                                       four ammo counts */
    /* Wall decals in paint order, oldest first (_native_render_hitscan_decals, engine.py:13747-13991; the
       host sorts the active slots by serial, engine.py:13756-13776).  Drawn after the walls and before the
       sprites when the renderer holds decal patches. */
    const int32_t *decal_state;     /* [N,D,3] linedef index, style (variant + 5*flip_x + 10*flip_y + 20*side), alive */
    const float *decal_geom;        /* [N,D,4] along the linedef 0..1, impact height, and the linedef's direction
                                       on the decal's side quantised through the fine sine table: cos, sin
                                       (engine.py:13822-13829) */
    const float *screen_blend;      /* [N,2] or NULL (no blend): bonus alpha min(bonus_count*8, 128)/255 and damage
                                       alpha damage_to_alpha[clamp(damage_count, 0, 113)]/255; PLAYPAL colours are
                                       mixed with gold and then red before the RGB24 frame and the observation
                                       (_native_indexed_to_rgb with render_screen_flashes, engine.py:15381-15398) */
    const int8_t *sprite_style;     /* [N,A] or NULL (all -1): -1 opaque, -2 translucent_lut, s >= 0
                                       additive_luts[min(s, 1)] (actor_additive_style, engine.py:14343-14682) */
} gd_lanes_desc;

/*
 * Weapon psprite and status bar patches (HOST pointers; gd_renderer_set_overlays
 * uploads them).  Replaces map.native_weapon_patch_* (engine.py:14997-15049,
 * _triton_kernels.py:2571-2670) and map.hud_patch_* (engine.py:15153-15267).
 * Patch atlases are [patches, max_h, max_w] with per-patch sizes and offsets.
 * Status bar patch numbering follows the reference: 0 bar, 1 arms panel,
 * 2..11 big digits, 12 percent sign, 13.. faces, 28..37 small digits,
 * 30..35 owned weapon numbers, 38..43 missing weapon numbers (engine.py:15186-15259).
 */
typedef struct gd_overlay_desc {
    uint32_t struct_size;    /* sizeof(gd_overlay_desc) of the header the caller was built with */
    int32_t weapon_patch_count, weapon_max_h, weapon_max_w;
    int32_t hud_patch_count, hud_max_h, hud_max_w;
    const uint8_t *weapon_atlas;    /* [Pw,Hw,Ww] palette indices */
    const uint8_t *weapon_opaque;   /* [Pw,Hw,Ww] 0/1 */
    const int32_t *weapon_w, *weapon_h, *weapon_left, *weapon_top; /* [Pw] */
    const uint8_t *hud_atlas;       /* [Ph,Hh,Wh] */
    const uint8_t *hud_opaque;      /* [Ph,Hh,Wh] */
    const int32_t *hud_w, *hud_h, *hud_left, *hud_top;             /* [Ph] */
    /* Bullet chip decals (map.bullet_decal_*, engine.py:690-695, 1038-1070); decal_variant_count 0 = none.
       The reference indexes variants with style % 5, so a non-empty set has exactly 5. */
    int32_t decal_variant_count, decal_max_h, decal_max_w, decal_black_rows;
    const uint8_t *decal_atlas;        /* [5,Hd,Wd] 0 = transparent; every variant is Wd wide */
    const int32_t *decal_h, *decal_left, *decal_top; /* [5] */
    const uint8_t *decal_opacity_lut;  /* [32,256] colormap row x atlas value -> row of decal_black_lut */
    const uint8_t *decal_black_lut;    /* [decal_black_rows,256] opacity x pixel under the decal -> pixel */
} gd_overlay_desc;

/* Output buffers; any pointer may be null to skip that product. */
typedef struct gd_frame_out {
    uint32_t struct_size;    /* sizeof(gd_frame_out) of the header the caller was built with */
    uint8_t *indexed;   /* [N,240,320] palette indices; rows 208..239 = 0 (empty status bar) */
    uint8_t *obs;       /* [N,84,84] grayscale policy frame (HUD rows masked black) */
    uint8_t *frames;    /* [N,4,84,84] stack, oldest first: rolled by one and obs appended */
    const uint8_t *reset_mask; /* [N] or null: lanes whose stack is filled with 4 copies instead */
    uint8_t *rgb;       /* [N,240,320,3] PLAYPAL expansion of `indexed` */
    uint8_t *final_frames; /* [N,4,84,84] or null: also receives every lane's stack as this call leaves it,
                              the clone step_and_reset_device hands out as final_observations
                              (env.py:915-917), written by the same kernel instead of a second pass */
    int32_t stack_mode; /* GD_STACK_STEP or GD_STACK_RESET */
    int32_t obs_source_rows; /* rows of the frame the observation pools: 208 (or 0) = the world view, status bar rows
                                black (render_reference_frame with mask_hud, engine.py:15444-15450); 240 = the status bar
                                too, as the reference does when the environment is made with obs_crop=None
                                (env.py:441, engine.py:15440) */
    int32_t final_frames_layout; /* GD_LAYOUT_CHW or GD_LAYOUT_HWC.  With it final_frames doubles as the observation copy
                                    the host API hands out (obs_copy "copy" / "safe_view", env.py:678-688): the caller
                                    passes the buffer it would have copied into and no copy kernel runs */
} gd_frame_out;

typedef struct gd_renderer gd_renderer;

/* library identification; replaces nothing in the reference */
const char *gd_version(void);
uint32_t gd_abi_version(void);   /* GD_ABI_VERSION of the header the library was built with */
const char *gd_last_error(void);

/*
 * Upload an immutable map (HOST pointers in `host_map`) to the current HIP
 * device and allocate working memory for batches of up to `max_lanes` lanes
 * (larger batches are rendered in chunks; 0 = none, for gd_render_static only).  `cosine_correction` is a host
 * array of 320 floats, cos(native_ray_offsets) (engine.py:10967), computed by
 * the caller with Torch like every other float32 transcendental input.
 * Replaces DeviceScenario.from_host + the engine ctor precompute
 * (engine.py:721-1476, 1527-1634).
 */
int gd_renderer_create(const gd_map_desc *host_map, const float *cosine_correction, int32_t max_lanes, gd_renderer **out);
void gd_renderer_destroy(gd_renderer *r);

/*
 * Render one frame for every lane on `stream` (a hipStream_t, may be null).
 * All gd_lanes_desc / gd_frame_out pointers are device pointers.
 * Replaces TorchDeathmatchEngine._render_native_indexed_frame (engine.py:15338-15379)
 * + render_reference_frame (engine.py:15436-15451) + _finish_observation
 * (engine.py:9545-9548) / the reset stack fill (engine.py:2443-2450)
 * + _native_indexed_to_rgb (engine.py:15381-15398, flashes off).
 * No allocation, no host synchronisation.
 */
int gd_render(gd_renderer *r, const gd_lanes_desc *lanes, const gd_frame_out *out, void *stream);

/*
 * gd_render for callers that cannot allocate device memory (code under HIP graph capture, tight
 * serving loops, harnesses that forbid hipMalloc).  It has no counterpart in the reference.  The
 * working memory comes from one fixed array of GD_STATIC_SCRATCH_MIB MiB that the library holds on every
 * GPU it runs on, so `r` may be a renderer created with max_lanes 0 (the map only).  Lanes are rendered
 * in as many chunks as the array needs; GD_E_ARG when one lane of the map alone does not fit, or
 * for more than GD_STATIC_MAX_LANES lanes.  Calls no hipMalloc / hipFree.  Every call on a GPU uses that
 * GPU's one array: calls that overlap on one GPU (two streams, two threads) race.
 */
#define GD_STATIC_SCRATCH_MIB 64
#define GD_STATIC_MAX_LANES 65536
int gd_render_static(gd_renderer *r, const gd_lanes_desc *lanes, const gd_frame_out *out, void *stream);

/*
 * Sticky status bits (synchronises the device).  bit0: some screen column had
 * more candidate linedefs than the library keeps and was truncated - the frame
 * of that lane is not trustworthy.  A column keeps 64 in its own slots; one
 * that sees more moves to a spill pool (up to 256 per column; every column of
 * up to 8 lanes, one column in 32 of a 4096-lane chunk, 320 columns in
 * gd_render_static).  bit1: a column drew more than 255 passes.
 * Replaces nothing in the reference.
 */
int gd_renderer_status(gd_renderer *r, int32_t *status);

/*
 * How a frame is put together once the walls are traversed.  GD_ASSEMBLY_SEPARATE: kernel by kernel through a
 * 320x240 frame in device memory, gd_frame_out.indexed or, when the caller takes none, a frame of the working memory's
 * own.  GD_ASSEMBLY_FUSED: band by band in LDS, where shading, billboards, overlays, PLAYPAL expansion, pooling and the
 * stack update all happen; the frame only goes to device memory if the caller asks for it (observations only: no
 * 320x240 frame is ever written: a fifth less device-memory traffic in the assembly, nine tenths of the speed).
 * GD_ASSEMBLY_AUTO (the default): separate, the faster of the two on MI355X.  Frames that draw wall decals are always
 * assembled separately.  Both give the same bytes.  Replaces nothing in the reference.
 */
#define GD_ASSEMBLY_AUTO 0
#define GD_ASSEMBLY_FUSED 1
#define GD_ASSEMBLY_SEPARATE 2
int gd_renderer_set_assembly(gd_renderer *r, int32_t assembly);

/*
 * Fill the renderer's working memory with one byte value, asynchronously on `stream` (diagnostic: the frames
 * that follow must not depend on what the memory held before).  Replaces nothing in the reference.
 */
int gd_renderer_scribble(gd_renderer *r, int32_t value, void *stream);

/*
 * Replace the map-wide sector light levels (device pointer to S floats) for the frames
 * that follow on `stream`; the copy is asynchronous.  The reference keeps one
 * sector_lights tensor per map (engine.py:640, 1277-1279); this is how a caller
 * animates it (light flicker) between frames.
 */
int gd_renderer_set_sector_lights(gd_renderer *r, const float *lights, void *stream);

/*
 * Upload (or replace) the weapon and status bar patches.  With them a gd_render call
 * whose lanes carry weapon_state draws the psprite and its muzzle flash over the view
 * after the sprites (_native_render_weapon, engine.py:15051-15110, fixed-point path), and
 * one whose lanes carry hud_state draws the status bar into rows 208..239
 * (_native_render_hud, engine.py:15232-15267); without them those rows stay 0.
 * Synchronises the device; call it between frames.
 */
int gd_renderer_set_overlays(gd_renderer *r, const gd_overlay_desc *overlays);

/*
 * Observation pipeline alone on an existing indexed frame.
 * Replaces policy_area_grayscale (_triton_kernels.py:120-203) fused with the
 * frame-stack update (engine.py:9545-9548, 2443-2450).
 * indexed: [N,source_rows,320] with source_rows 208 or 240; rows >= source_rows are black.
 */
int gd_observe(const uint8_t *indexed, int32_t source_rows, const uint8_t *playpal, int32_t lane_count,
               uint8_t *obs, uint8_t *frames, const uint8_t *reset_mask, int32_t stack_mode, void *stream);

/* PLAYPAL expansion [N,rows,320] -> [N,rows,320,3]; replaces engine.py:15381-15384. */
int gd_expand_rgb24(const uint8_t *indexed, int32_t rows, const uint8_t *playpal, int32_t lane_count,
                    uint8_t *rgb, void *stream);

/*
 * Gameplay state -> packed billboard list, one thread per (lane, slot), nothing trimmed, no host round trip.
 * Replaces the list building at the head of _native_render_sprites (engine.py:14328-14682) with its helpers
 * _native_enemy_sprite_ids, _native_enemy_death_sprite_ids, _native_projectile_explosion_sprite_ids,
 * _native_enemy_fullbright and _native_item_sprite_ids (engine.py:14011-14136, 14258-14317): the same kinds of
 * actor in the same order, every slot kept and unused ones marked dead instead of the per-kind nonzero() trims
 * (list order breaks ties between equally distant sprites and is unchanged by trimming).  All pointers are
 * DEVICE pointers to the engine's own tensors (bool tensors as bytes); fields are the engine / map attributes of
 * the same names.  The *_rotation arrays are _doom_sprite_rotation (engine.py:13994-14009) of the camera-to-actor
 * angle and the actor's heading, which the host evaluates with the reference's own float32 Torch ops (atan2).
 * Output width A = 2 * enemy_slots + doll_count + 2 * player_projectile_slots + 2 * enemy_projectile_slots +
 * fog_slots + puff_slots + item_count + drop_slots, in the order: monsters, dolls, corpses, player projectiles in
 * flight, fireballs in flight, player explosions, fireball explosions, teleport fog, bullet puffs, map items,
 * drops.  Returns GD_E_ARG for a null pointer or a negative count.
 */
typedef struct gd_actor_desc {
    uint32_t struct_size;    /* sizeof(gd_actor_desc) of the header the caller was built with */
    int32_t lane_count, enemy_slots, doll_count, player_projectile_slots, enemy_projectile_slots, fog_slots, puff_slots,
        item_count, drop_slots, attack_frames, death_frames, xdeath_frames, explosion_frames;
    const float *enemy_x;  /* [N,Se] */
    const float *enemy_y;
    const float *enemy_z;
    const uint8_t *enemy_alive;  /* bool */
    const int64_t *enemy_type;
    const uint8_t *enemy_rotation;  /* 0..7, see above */
    const int32_t *enemy_animation_tics;
    const int64_t *enemy_target_slot;
    const int32_t *enemy_attack_phase;
    const int32_t *enemy_cooldown;
    const int32_t *enemy_pain_tics;
    const int32_t *enemy_death_tics;
    const int64_t *enemy_death_type;
    const int32_t *enemy_death_elapsed;
    const uint8_t *enemy_death_extreme;  /* bool */
    const float *doll_x;  /* [Sd] player_starts[:-1] */
    const float *doll_y;
    const float *doll_z;  /* _player_start_z[:-1] */
    const uint8_t *doll_rotation;  /* [N,Sd] */
    const uint8_t *player_dead;  /* [N] bool */
    const float *projectile_x;  /* [N,Sp] */
    const float *projectile_y;
    const float *projectile_z;
    const uint8_t *projectile_alive;  /* bool */
    const int64_t *projectile_type;
    const int32_t *projectile_age;
    const uint8_t *projectile_rotation;
    const int64_t *projectile_impact_type;
    const int32_t *projectile_impact_tics;
    const float *enemy_projectile_x;  /* [N,Sq] */
    const float *enemy_projectile_y;
    const float *enemy_projectile_z;
    const uint8_t *enemy_projectile_alive;  /* bool */
    const int32_t *enemy_projectile_age;
    const uint8_t *enemy_projectile_rotation;
    const int32_t *enemy_projectile_impact_tics;
    const float *teleport_fog_x;  /* [N,Sg] */
    const float *teleport_fog_y;
    const float *teleport_fog_z;
    const int32_t *teleport_fog_tics;
    const float *hitscan_puff_x;  /* [N,Sf] */
    const float *hitscan_puff_y;
    const float *hitscan_puff_z;
    const int32_t *hitscan_puff_tics;
    const float *item_x;  /* [Si] item_spawns[:,0] */
    const float *item_y;  /* item_spawns[:,1] */
    const float *item_z;  /* _item_z */
    const int64_t *item_types;  /* [Si] */
    const int64_t *item_raw_visual_types;  /* [Si] */
    const uint8_t *item_available;  /* [N,Si] bool */
    const int32_t *item_animation_initial_tics;  /* [N,Si] */
    const int32_t *episode_time;  /* [N] */
    const float *drop_x;  /* [N,Sr] */
    const float *drop_y;
    const float *drop_z;
    const int64_t *drop_type;
    const uint8_t *drop_spawned;  /* bool */
    const int32_t *enemy_walk_frame_tics;  /* [6] */
    const int32_t *enemy_idle_frame_tics;  /* [6] */
    const int32_t *enemy_attack_recovery;  /* [6] */
    const int64_t *enemy_walk_sprite_ids;  /* [6,4,8] */
    const int64_t *enemy_attack_sprite_ids;  /* [6,attack_frames,8] */
    const int64_t *enemy_pain_sprite_ids;  /* [6,8] */
    const int64_t *enemy_death_sprite_ids;  /* [6,death_frames] */
    const int64_t *enemy_death_frame_durations;  /* [6,death_frames] */
    const int64_t *enemy_death_frame_counts;  /* [6] */
    const int64_t *enemy_xdeath_sprite_ids;  /* [6,xdeath_frames] */
    const int64_t *enemy_xdeath_frame_durations;  /* [6,xdeath_frames] */
    const int64_t *enemy_xdeath_frame_counts;  /* [6] */
    const int64_t *projectile_explosion_total_tics;  /* [3] */
    const int64_t *projectile_explosion_frame_durations;  /* [3,explosion_frames] */
    const int64_t *projectile_explosion_frame_counts;  /* [3] */
    const int64_t *raw_projectile_explosion_sprite_ids;  /* [3,explosion_frames] */
    const int64_t *raw_projectile_flight_sprite_ids;  /* [3,2,8] */
    const int64_t *raw_teleport_fog_sprite_ids;  /* [12] */
    const int64_t *raw_bullet_puff_sprite_ids;  /* [4] */
    const int64_t *raw_static_sprite_ids;  /* [>=15] */
    const int64_t *raw_item_animation_sprite_ids;  /* [8] */
    /* outputs, [N,A] each: the sprite_* fields of gd_lanes_desc */
    float *sprite_x;
    float *sprite_y;
    float *sprite_z;
    int32_t *sprite_id;
    uint8_t *sprite_alive;
    uint8_t *sprite_fullbright;
    int8_t *sprite_style;
} gd_actor_desc;

int gd_pack_actors(const gd_actor_desc *actors, void *stream);

/*
 * The five weapon_state words of every lane (gd_lanes_desc.weapon_state) and the muzzle flash's extra light
 * (gd_lanes_desc.flash_light), from the gameplay tensors, in one kernel with no host synchronisation.
 * Replaces the per-lane part of the reference's weapon layer: frame / flash selection
 * (engine.py:14949-14967 _native_weapon_frame_selection) and the raise / lower / bob offsets of
 * engine.py:15051-15092 (_native_render_weapon).  Every input is an int64 device array of lane_count entries (the engine's
 * attributes of the same names; active_weapon is engine._active_weapon(), player_bob_fixed engine._player_bob_fixed),
 * player_dead a bool array; the three tables are the map's native_weapon_frame_ids / _flash_ids / _flash_lights
 * [8, 2, cooldown_slots] as int64, fine_sine the 8192-entry 16.16 sine table (engine.py:309-321).
 * weapon_state receives [lane_count, 5]: patch id, flash patch id (-1: none), horizontal and vertical offset (16.16),
 * visible.  flash_light (may be null) receives the flash's extra light level.  Returns GD_E_ARG for a null pointer or
 * a count out of range.
 */
typedef struct gd_weapon_desc {
    uint32_t struct_size;    /* sizeof(gd_weapon_desc) of the header the caller was built with */
    int32_t lane_count, cooldown_slots;
    const int64_t *active_weapon;
    const int64_t *weapon_state_cooldown;
    const int64_t *weapon_fire_count;
    const int64_t *weapon_ready_tics;
    const int64_t *weapon_lower_cooldown;
    const int64_t *weapon_raise_cooldown;
    const int64_t *pending_weapon;
    const int64_t *episode_time;
    const int64_t *player_bob_fixed;
    const uint8_t *player_dead;
    const int64_t *weapon_frame_ids;
    const int64_t *weapon_flash_ids;
    const int64_t *weapon_flash_lights;   /* may be null when flash_light is */
    const int64_t *fine_sine;
    int64_t *weapon_state;
    int64_t *flash_light;
} gd_weapon_desc;

int gd_pack_weapon(const gd_weapon_desc *weapon, void *stream);

/*
 * Time `launches` back-to-back gd_render launches with HIP events on `stream`
 * and return the average milliseconds per launch of each kernel stage in
 * ms[0..stage_count).  Measurement helper for the benchmark; replaces nothing.
 */
int gd_render_timed(gd_renderer *r, const gd_lanes_desc *lanes, const gd_frame_out *out, void *stream,
                    int32_t launches, float *ms, int32_t stage_count);

#ifdef __cplusplus
}
#endif
#endif /* GRADOOM_AMD_H */
