// Front-to-back alpha compositing for camera pixels and lidar points on gfx950.
//
// One workgroup per (sensor, tile); one lane per pixel / point.  A tile's depth-sorted
// Gaussian list is streamed through LDS in batches of one Gaussian per lane: the batch is
// gathered once (coalesced over the id list, 16-byte records in LDS; for cameras the colours
// too, for lidars the many features only of the Gaussians a wavefront composites) and then
// every wavefront tests 64 Gaussians at a time against its footprint and walks the survivors,
// reading LDS at a wave-uniform address, which the LDS serves as a broadcast without bank
// conflicts.  A 16x16 camera tile is four wavefronts of 8x8 pixels, a 64x4 lidar tile four
// of 16x4 points; a wavefront leaves the batch loop as soon as its 64 pixels are saturated
// and the workgroup stops fetching batches once all of its pixels are.  With 32 or 33
// channels the lidar kernel accumulates 32 of them on the matrix cores.
//
// Compositing rules follow gsplat/cuda/csrc/rasterization.cu:1360-1518 (pixels) and
// :2021-2219 (points) of the reference: alpha = min(0.999, o * exp(-sigma)); a Gaussian is
// skipped when sigma < 0 or alpha < 1/255; a pixel stops, without taking the Gaussian,
// when its transmittance would fall to 1e-4 or below.
//
// Channels: the kernels are compiled for CH accumulators per lane and take the real
// channel count, stride and offset at run time, so any channel count is rendered without
// host-side padding (wide inputs in passes of up to 32 channels).
#include "raster_common.h"
#include "sh_eval.h"

#include <type_traits>

namespace {

struct PixelArgs {
    uint32_t C;
    int64_t n_isects;
    uint32_t color_stride; // channels of the colour tensor
    uint32_t ch_offset;    // first channel of this pass
    uint32_t n_ch;         // channels of this pass (<= CH)
    const float *means2d, *conics, *colors, *opacities, *pix_vels, *rs_time, *backgrounds;
    uint32_t W, H, tile_size, tile_w, tile_h;
    const int32_t *tile_offsets, *flatten_ids;
    float *render_colors, *render_alphas;
    int32_t *last_ids;
    int write_aux; // first pass also writes alphas and last ids
    int32_t *tile_batches; // optional diagnostic: list entries each tile's workgroup staged
    int64_t *tile_cycles;  // optional diagnostic: shader clock cycles each tile's workgroup ran for
    unsigned long long *lane_stats; // STATS kernels only: kLaneStats counters, see the entry point
    // SHC kernels: channels 0-2 are the view-dependent colours of the Gaussians, evaluated from
    // their spherical-harmonic coefficients for the entries a tile stages (`colors` is unused);
    // channel 3, if rendered, is sh_depths[id].  Dense rows [C, N]: id = camera * sh_N + Gaussian;
    // packed rows: sh_gaussian_ids[id] (not null) is the Gaussian.
    // sh_cache: a float4 per row, NaN before the launch; the first workgroups to stage a row
    // leave its colour there for the later ones.
    const float *sh_means, *sh_viewmats, *sh_coeffs, *sh_depths;
    const int64_t *sh_gaussian_ids;
    float *sh_cache;
    uint32_t sh_N, sh_K, sh_degree;
    int sh_per_sensor; // coefficient rows: 1 = one per (camera, Gaussian), 0 = one per Gaussian
};

constexpr int kLaneStats = 8;

// PPL pixels per lane.  With PPL == 2 (tiles whose side is a multiple of 8 and that make whole
// wavefronts that way) a wavefront covers 8 columns x 16 rows, lane (lx, ly) the pixels (lx, ly)
// and (lx, ly + 8): every staged value read from LDS and every scalar instruction of the loop
// then serves two pixels.  A wavefront's LDS reads are broadcasts of 16 bytes to 64 lanes, which
// the LDS delivers at 128 bytes per clock: with one pixel per lane the three reads of a
// (wavefront, Gaussian) iteration keep the LDS of a compute unit as busy as the iteration's
// vector instructions keep a SIMD, and four SIMDs share that LDS.
//
// Per batch of the tile's list the workgroup stages, for every Gaussian, the six coefficients
// of its exponent polynomial (raster_common.h), what the footprint test needs and its colours.
// Every wavefront then tests 64 staged Gaussians at a time against its footprint, copies the
// survivors' records in list order into a private strip of LDS (its own writes and reads: no
// barrier) and walks that strip: sequential addresses, no lane-mask bookkeeping per Gaussian.
// LAST: the index of the last entry a pixel composited is kept and written (what the backward
// pass starts from); without it (last_ids null: calls that take no gradient) the loop is two
// instructions per survivor shorter.
template <int CH, int PPL, bool STATS = false, bool SHC = false, bool LAST = true>
// (Two pixels per lane: at most 512 lanes per tile.  The narrow two-pixel kernels are held to the
// 80 registers of six resident wavefronts per SIMD, which they exceeded by two: 0.116 -> 0.110 ms
// for the 1080p frame.)
__global__ void __launch_bounds__(PPL == 2 ? 512 : 1024)
    __attribute__((amdgpu_waves_per_eu(CH <= 5 && PPL == 2 ? 6 : 1, CH <= 5 && PPL == 2 ? 6 : 8)))
rasterize_to_pixels_fwd_kernel(PixelArgs a) {
    const long long t_begin = a.tile_cycles != nullptr ? clock64() : 0;
    extern __shared__ float4 lds4[];
    const uint32_t block_size = blockDim.x;
    const uint32_t batch = block_size; // list entries staged at a time, one per lane
    constexpr bool COPY = CH <= 4;           // survivors carry their colours along
    constexpr int RECORD = 2 + (CH + 3) / 4; // float4 per staged Gaussian
    constexpr int LIST = COPY ? 3 : 2;       // float4 per survivor
    float4 *s_rec = lds4;

    const uint32_t tiles_per_cam = a.tile_w * a.tile_h;
    const uint32_t unit = blockIdx.x;
    const uint32_t cam = unit / tiles_per_cam;
    const uint32_t tile_id = unit % tiles_per_cam;
    const uint32_t tile_y = tile_id / a.tile_w, tile_x = tile_id % a.tile_w;
    const uint32_t tr = threadIdx.x;
    const uint32_t lane = tr & (SPLATAD_WAVE - 1), wave = tr / SPLATAD_WAVE;
    float4 *s_list = lds4 + (size_t)RECORD * batch + (size_t)wave * SPLATAD_WAVE * LIST;

    const TileFrame frame = tile_frame(tile_x, tile_y, a.tile_size, a.rs_time[cam], a.H);
    uint32_t pi[PPL], pj;
    if (PPL == 2) {
        const uint32_t waves_per_row = a.tile_size / 8;
        const uint32_t lx = (wave % waves_per_row) * 8 + (lane & 7);
        const uint32_t ly = (wave / waves_per_row) * 16 + (lane >> 3);
        pj = tile_x * a.tile_size + lx;
#pragma unroll
        for (int p = 0; p < PPL; ++p) pi[p] = tile_y * a.tile_size + ly + 8 * p;
    } else {
        uint32_t lx, ly;
        pixel_of_lane(a.tile_size, tr, lx, ly);
        pj = tile_x * a.tile_size + lx;
        pi[0] = tile_y * a.tile_size + ly;
    }
    PixelConstants pc[PPL];
    bool inside[PPL];
    uint64_t alive_bits[PPL]; // lanes still compositing, as lane masks (scalar logic below)
    float y_lo = 0.f, y_hi = 0.f;
#pragma unroll
    for (int p = 0; p < PPL; ++p) {
        pc[p].init((float)pj + 0.5f, (float)pi[p] + 0.5f, frame);
        inside[p] = pi[p] < a.H && pj < a.W;
        alive_bits[p] = wave_ballot(inside[p]);
        y_lo = p == 0 ? pc[p].Y : fminf(y_lo, pc[p].Y);
        y_hi = p == 0 ? pc[p].Y : fmaxf(y_hi, pc[p].Y);
    }
    WaveBox box; // footprint of this wavefront (all 64 lanes exist in whole wavefronts)
    box.init(pc[0].X, pc[0].X, y_lo, y_hi, block_size % SPLATAD_WAVE == 0);

    const int32_t *offs = a.tile_offsets + (size_t)cam * tiles_per_cam;
    const int32_t range_start = offs[tile_id];
    const int32_t range_end = (cam == a.C - 1 && tile_id == tiles_per_cam - 1)
                                  ? (int32_t)a.n_isects
                                  : offs[tile_id + 1];
    const uint32_t num_batches = (uint32_t)(range_end - range_start + batch - 1) / batch;

    float T[PPL], out[PPL][CH];
    uint32_t cur_idx[PPL];
#pragma unroll
    for (int p = 0; p < PPL; ++p) {
        T[p] = 1.0f;
        cur_idx[p] = 0;
#pragma unroll
        for (int k = 0; k < CH; ++k) out[p][k] = 0.f;
    }

    // One Gaussian of the survivor strip for all pixels of the lane.  GENERAL: some Gaussian of
    // the strip needs the 0.999 clamp or the sigma < 0 rule (see pixel_polynomial).
    uint32_t st_iter = 0, st_take = 0, st_alive = 0, st_idle = 0, st_tested = 0, st_kept = 0, st_valid = 0;
    struct Survivor { float4 pa, pb, col; };
    // the three reads of a strip entry are requested together, ahead of their use
    auto fetch = [&](uint32_t k) {
        Survivor s;
        s.pa = s_list[LIST * k];
        s.pb = s_list[LIST * k + 1]; // {cXY, cYY, list position (bits), L or +inf}
        s.col = COPY ? s_list[LIST * k + 2] : make_float4(0.f, 0.f, 0.f, 0.f);
        return s;
    };
    auto composite = [&](Survivor &s, uint32_t batch_start, auto general) {
        constexpr bool GENERAL = decltype(general)::value;
        const float4 pa = s.pa, pb = s.pb;
        const float *col;
        if (COPY) {
            // the colours are in registers before the lanes part ways (the compiler would
            // otherwise read them behind each pixel's decision and wait for the LDS there)
            asm volatile("" : "+v"(s.col.x), "+v"(s.col.y), "+v"(s.col.z), "+v"(s.col.w));
            col = reinterpret_cast<const float *>(&s.col);
        } else {
            const uint32_t slot = __float_as_uint(pb.z) - batch_start;
            col = reinterpret_cast<const float *>(s_rec + (size_t)RECORD * slot + 2);
        }
        uint64_t any_alive = 0, any_take = 0;
#pragma unroll
        for (int p = 0; p < PPL; ++p) {
            const float e = pixel_exponent(pa, pb.x, pb.y, pc[p]);
            float alpha = __builtin_amdgcn_exp2f(e);
            if (GENERAL) alpha = fminf(0.999f, alpha);
            const float next_T = transmittance_behind(T[p], alpha);
            // same decisions as: skip if sigma < 0 or alpha < 1/255; stop if next_T <= 1e-4
            uint64_t valid_bits = alive_bits[p] & wave_ballot(!(alpha < 1.f / 255.f));
            if (GENERAL) valid_bits &= wave_ballot(!(e > pb.w));
            const uint64_t stop_bits = valid_bits & wave_ballot(next_T <= 1e-4f);
            const uint64_t take_bits = valid_bits & ~stop_bits;
            if (STATS) {
                st_alive += (uint32_t)__popcll(alive_bits[p]);
                st_valid += (uint32_t)__popcll(valid_bits);
                st_take += (uint32_t)__popcll(take_bits);
                any_take |= take_bits;
            }
            alive_bits[p] &= ~stop_bits;
            any_alive |= alive_bits[p];
            if (wave_lanes(take_bits)) {
                const float weight = alpha * T[p];
#pragma unroll
                for (int c = 0; c < CH; ++c) out[p][c] = fmaf(col[c], weight, out[p][c]);
                T[p] = next_T;
                if (LAST) cur_idx[p] = __float_as_uint(pb.z);
            }
        }
        if (STATS) { st_iter += 1; st_idle += any_take == 0 ? 1u : 0u; }
        return any_alive;
    };
    // walks the n survivors of the strip, two per trip so that the second one's reads are in
    // flight while the first is composited; returns the lanes still alive
    auto walk = [&](uint32_t n, uint32_t batch_start, uint64_t any_alive, auto general) {
        uint32_t k = 0;
        for (; k + 1 < n; k += 2) {
            Survivor s0 = fetch(k), s1 = fetch(k + 1);
            any_alive = composite(s0, batch_start, general);
            if (any_alive == 0) return any_alive;
            any_alive = composite(s1, batch_start, general);
            if (any_alive == 0) return any_alive;
        }
        if (k < n) {
            Survivor s0 = fetch(k);
            any_alive = composite(s0, batch_start, general);
        }
        return any_alive;
    };

    // Staging reads.  Every load is unconditional (entries beyond the list repeat its last one,
    // channels beyond the pass its last one), so that all of them are in flight together: two
    // dependent round trips to memory per batch (id, then the Gaussian), hidden by the other
    // workgroups of the compute unit.  (Requesting the next batch before compositing the current
    // one costs 15 registers, one resident wavefront per SIMD with them, and was slower.)
    struct Staged { float2 xy, vel; float cn[3], opac, col[CH]; };
    float sensor_x = 0.f, sensor_y = 0.f, sensor_z = 0.f;
    if (SHC) sensor_position(a.sh_viewmats + (size_t)cam * 16, sensor_x, sensor_y, sensor_z);
    auto id_of = [&](uint32_t b) -> int32_t {
        const uint32_t idx = min((uint32_t)range_start + batch * b + tr, (uint32_t)range_end - 1u);
        return b < num_batches ? a.flatten_ids[idx] : 0;
    };
    auto gather = [&](int32_t g) {
        Staged s;
        s.xy = reinterpret_cast<const float2 *>(a.means2d)[g];
        s.vel = reinterpret_cast<const float2 *>(a.pix_vels)[g];
        const float *c3 = a.conics + (size_t)g * 3;
        s.cn[0] = c3[0]; s.cn[1] = c3[1]; s.cn[2] = c3[2];
        s.opac = a.opacities[g];
        if (SHC) return s; // the colours are staged by stage_sh_color
        const float *c = a.colors + (size_t)g * a.color_stride + a.ch_offset;
#pragma unroll
        for (int k = 0; k < CH; ++k) s.col[k] = STATS ? 0.f : c[min((uint32_t)k, a.n_ch - 1u)]; // STATS: no colours
        return s;
    };
    // SHC: the colour of row g, what sh_fwd_kernel<true> writes for it, by the same instructions.
    // A row's colour is evaluated by the first workgroups that stage it and left in sh_cache for
    // the others (a Gaussian is listed by every tile it touches), on purpose without any
    // ordering: a word of a row only ever changes from the NaN the cache was filled with to its
    // colour, so another workgroup sees each word either as NaN -- then it evaluates the colour
    // itself, to the same value -- or as the colour; how soon it sees the colour is left to the
    // caches (the dies' L2 caches do not see one another's lines before the kernel ends, so each
    // die evaluates the rows its tiles stage).  A row is read once, by one aligned 16-byte load
    // whose four words are pinned in registers before their first use (an empty asm statement
    // takes and returns them, so the compiler can neither read the row a second time later nor
    // assume anything about the values), and written by one aligned 16-byte store; the
    // hardware moves a word whole, so a read sees each word before or after its one change.
    // Measured alternatives: relaxed atomic accesses word by word (four requests per row
    // instead of one) cost this kernel 8 %, volatile accesses and atomic accesses of device
    // scope go to memory every time and made it three to four times slower.
    struct Cached { float r, g, b, depth; };
    auto cached_color = [&](int32_t g) { // requested together with the rest of the Gaussian
        const float4 row = reinterpret_cast<const float4 *>(a.sh_cache)[g];
        return Cached{row.x, row.y, row.z, row.w};
    };
    auto stage_sh_color = [&](int32_t g, const Cached &c) {
        float cr = c.r, cg = c.g, cb = c.b, cd = c.depth; // the depth channel rides along
        asm volatile("" : "+v"(cr), "+v"(cg), "+v"(cb), "+v"(cd)); // the row as it was read, once (see above)
        const bool missing = !(cr == cr) || !(cg == cg) || !(cb == cb) || (CH > 3 && !(cd == cd));
        if (wave_ballot(missing) != 0) { // uniform
            if (missing) {
                const uint32_t gauss =
                    a.sh_gaussian_ids ? (uint32_t)a.sh_gaussian_ids[g] : (uint32_t)g - cam * a.sh_N;
                const float *m = a.sh_means + (size_t)gauss * 3;
                const float dx = m[0] - sensor_x, dy = m[1] - sensor_y, dz = m[2] - sensor_z;
                const size_t row = a.sh_per_sensor ? (size_t)cam * a.sh_N + gauss : (size_t)gauss;
                float r = 0.f, gr = 0.f, bl = 0.f;
                sh_color_by_band(a.sh_degree, a.sh_coeffs + row * a.sh_K * 3, dx, dy, dz, r, gr, bl);
                cr = fmaxf(r + 0.5f, 0.f);
                cg = fmaxf(gr + 0.5f, 0.f);
                cb = fmaxf(bl + 0.5f, 0.f);
                cd = CH > 3 ? a.sh_depths[g] : 0.f;
                reinterpret_cast<float4 *>(a.sh_cache)[g] = make_float4(cr, cg, cb, cd);
            }
        }
        float *col = reinterpret_cast<float *>(s_rec + RECORD * tr + 2);
        col[0] = cr;
        col[1 % CH] = cg;
        col[2 % CH] = cb;
        if (CH > 3) col[3 % CH] = cd;
    };
    uint32_t batches_done = 0;
    for (uint32_t b = 0; b < num_batches; ++b) {
        // also orders the previous batch's LDS reads before this batch's writes
        bool lane_alive = false;
#pragma unroll
        for (int p = 0; p < PPL; ++p) lane_alive = lane_alive || wave_lanes(alive_bits[p]);
        if (__syncthreads_count(!lane_alive) >= (int)block_size) break;
        batches_done = b + 1;

        const uint32_t batch_start = (uint32_t)range_start + batch * b;
        {
            const int32_t g = id_of(b);
            Cached cached = {};
            if (SHC) cached = cached_color(g);
            const Staged staged = gather(g);
            float4 pa, pb;
            pixel_polynomial(frame, staged.xy, staged.vel, staged.cn[0], staged.cn[1], staged.cn[2], staged.opac,
                             pa, pb);
            s_rec[RECORD * tr] = pa;
            s_rec[RECORD * tr + 1] = pb;
            // (the colour last: where it has to be evaluated, nothing else of the Gaussian is in
            // registers beside a band's coefficients)
            if (SHC) stage_sh_color(g, cached);
            if (!SHC) {
#pragma unroll
                for (int k = 0; k < CH; ++k)
                    reinterpret_cast<float *>(s_rec + RECORD * tr + 2)[k] = (uint32_t)k < a.n_ch ? staged.col[k] : 0.f;
            }
        }
        __syncthreads();

        const uint32_t batch_size = min(batch, (uint32_t)range_end - batch_start);
        uint64_t any_alive = 0;
#pragma unroll
        for (int p = 0; p < PPL; ++p) any_alive |= alive_bits[p];
        for (uint32_t base = 0; base < batch_size && any_alive != 0; base += SPLATAD_WAVE) {
            // lanes test 64 Gaussians against the wavefront's footprint ...
            const uint32_t slot = base + lane;
            bool keep = slot < batch_size;
            float4 pa = make_float4(0.f, 0.f, 0.f, 0.f), pb = pa;
            if (keep) {
                pa = s_rec[RECORD * slot];
                pb = s_rec[RECORD * slot + 1];
                keep = box.may_touch(pa, pb);
            }
            const uint64_t todo = wave_ballot(keep);
            const uint32_t n = (uint32_t)__popcll(todo);
            if (STATS) {
                st_tested += min(batch_size - base, (uint32_t)SPLATAD_WAVE);
                st_kept += n;
            }
            if (n == 0) continue; // uniform
            const bool general = wave_ballot(keep && !(pb.z == pb.z)) != 0; // uniform
            // ... and copy the survivors into the wavefront's strip, in list order
            if (keep) {
                const uint32_t pos = (uint32_t)__popcll(todo & ((1ull << lane) - 1ull));
                s_list[LIST * pos] = pa;
                // .w: what the sigma < 0 rule compares with in a strip that needs it (for a plain
                // Gaussian pb.w is the peak's row, not a bound)
                s_list[LIST * pos + 1] = make_float4(pb.x, pb.y, __uint_as_float(batch_start + slot),
                                                     pb.z == pb.z ? INFINITY : pb.w);
                if (COPY) s_list[LIST * pos + 2] = s_rec[RECORD * slot + 2];
            }
            // the strip is written and read by this wavefront only, whose LDS accesses execute in
            // order; the fence keeps the compiler from moving the reads above the writes
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
            if (!general) any_alive = walk(n, batch_start, any_alive, std::false_type{});
            else any_alive = walk(n, batch_start, any_alive, std::true_type{});
            // the next round overwrites the strip: its reads above are done (same wavefront)
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
        }
    }

    if (a.tile_batches != nullptr && a.write_aux && tr == 0)
        a.tile_batches[unit] = (int32_t)min(batches_done * batch, (uint32_t)(range_end - range_start));
    if (a.tile_cycles != nullptr && a.write_aux && tr == 0) a.tile_cycles[unit] = clock64() - t_begin;
    if (STATS) {
        if (lane == 0) {
            const uint32_t v[kLaneStats] = {st_iter, st_take, st_alive, st_idle, st_tested, st_kept, 0u, st_valid};
            for (int k = 0; k < kLaneStats; ++k)
                if (k != 6) atomicAdd(a.lane_stats + k, (unsigned long long)v[k]);
            if (blockIdx.x == 0 && tr == 0) a.lane_stats[6] = (unsigned long long)PPL;
        }
        return;
    }
#pragma unroll
    for (int p = 0; p < PPL; ++p) {
        if (!inside[p]) continue;
        const size_t pix = ((size_t)cam * a.H + pi[p]) * a.W + pj;
        float *dst = a.render_colors + pix * a.color_stride + a.ch_offset;
        const float *bg = a.backgrounds ? a.backgrounds + (size_t)cam * a.color_stride + a.ch_offset : nullptr;
#pragma unroll
        for (int k = 0; k < CH; ++k)
            if ((uint32_t)k < a.n_ch) dst[k] = bg ? out[p][k] + T[p] * bg[k] : out[p][k];
        if (a.write_aux) {
            a.render_alphas[pix] = 1.0f - T[p];
            if (LAST) a.last_ids[pix] = (int32_t)cur_idx[p];
        }
    }
}

struct PointArgs {
    uint32_t C;
    int64_t n_isects;
    uint32_t color_stride, ch_offset, n_ch;
    // With range_channel given, `colors` has rows of feat_stride = color_stride - 1 values and
    // channel depth_idx (the last one) is range_channel[id]; otherwise feat_stride ==
    // color_stride.
    uint32_t feat_stride;
    const float *range_channel;
    const float *means2d, *conics, *colors, *opacities, *pix_vels, *depth_comps, *backgrounds,
        *raster_pts;
    uint32_t W, H, tile_width, tile_height, grid_w, grid_h;
    int compute_alpha_sum;
    float threshold;
    const int32_t *tile_offsets, *flatten_ids;
    uint32_t depth_idx;
    float *render_colors, *render_alphas, *alpha_sum;
    int32_t *last_ids;
    float *median_depths;
    int write_aux;
    int32_t *tile_batches; // optional diagnostic, as in PixelArgs
    int64_t *tile_cycles;  // optional diagnostic, as in PixelArgs
};

// MATRIX (CH = 32 or 33, every channel in use, whole wavefronts): the first 32 channels are
// accumulated by the matrix cores.  Compositing a Gaussian adds the outer product of 64 weights
// (one per point) and its features to the wavefront's accumulators; two Gaussians at a time
// that is C[64 x 32] += W[64 x 2] F[2 x 32], two v_mfma_f32_32x32x2_f32 (one per 32 points).
// The weights of a pair are brought into the A layout (lanes 0-31: first Gaussian, lanes 32-63:
// second; points 0-31 for the first instruction, 32-63 for the second) by one
// v_permlane32_swap; the features are loaded in the B layout (lane = feature) with one
// coalesced 128-byte load per Gaussian.  This takes 32 of the about 65 vector instructions of a
// composited Gaussian off the vector ALUs, which bound this kernel.  The accumulators live in
// the D layout (lane = feature, register = point) until the end, when every half wavefront
// stores the 32 features of a point with one 128-byte store.
typedef float floatx16 __attribute__((ext_vector_type(16)));

// Four wavefronts per SIMD: the 1024 tiles of a 128 x 2048 sweep then run in one round.
template <int CH, bool MATRIX>
__global__ void __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(4)))
rasterize_to_points_fwd_kernel(PointArgs a) {
    const long long t_begin = a.tile_cycles != nullptr ? clock64() : 0;
    static_assert(!MATRIX || CH == 32 || CH == 33, "the matrix path accumulates 32 channels (+1)");
    extern __shared__ float4 lds4[];
    __shared__ uint32_t s_ref_thread;
    __shared__ float s_ref[2];
    const uint32_t block_size = blockDim.x * blockDim.y;
    // Staged per Gaussian: {u_az, u_el, v_az, v_el} (u relative to the tile's reference point),
    // {A, B, C, L} as in the pixel kernel, and the Gaussian's id.  That is all the footprint test
    // and the alpha need.  A lidar point is a sample, not an area: of the Gaussians in a tile's
    // list only a few per cent reach alpha >= 1/255 at any of a wavefront's points, so the rest
    // of a Gaussian (its CH features, the range velocity, the depth compensation) is read from
    // global memory by the wavefronts that composite it, one word per lane.
    constexpr int RECORD = 2; // float4 per Gaussian
    float4 *s_rec = lds4;
    int32_t *s_gid = reinterpret_cast<int32_t *>(lds4 + (size_t)RECORD * blockDim.x * blockDim.y);
    // per wavefront: {position in the batch, id} of the staged Gaussians that pass its footprint test
    uint2 *s_surv = reinterpret_cast<uint2 *>(s_gid + block_size) +
                    (size_t)((threadIdx.y * blockDim.x + threadIdx.x) / SPLATAD_WAVE) * block_size;

    const uint32_t tiles_per_cam = a.grid_w * a.grid_h;
    const uint32_t cam = blockIdx.x / tiles_per_cam;
    const uint32_t tile_id = blockIdx.x % tiles_per_cam;
    const uint32_t tr = threadIdx.y * blockDim.x + threadIdx.x;
    const uint32_t lane = tr & (SPLATAD_WAVE - 1);
    uint32_t lx, ly;
    point_of_lane(a.tile_width, a.tile_height, tr, lx, ly);
    const uint32_t i = (tile_id / a.grid_w) * a.tile_height + ly;
    const uint32_t j = (tile_id % a.grid_w) * a.tile_width + lx;

    // the workgroup is padded to whole wavefronts (the payload words below need every lane of a
    // wavefront to exist); lanes beyond the tile own no point
    const bool in_image = (tr < a.tile_width * a.tile_height && i < a.H && j < a.W);
    const size_t pix = in_image ? ((size_t)cam * a.H + i) * a.W + j : 0;
    float px = 0.f, py = 0.f, pz = 0.f, roll = 0.f;
    if (in_image) {
        const float4 p = reinterpret_cast<const float4 *>(a.raster_pts)[pix];
        px = p.x; py = p.y; pz = p.z; roll = p.w;
    }
    const bool inside = in_image && pz > 0.f;
    uint64_t alive_bits = wave_ballot(inside); // lanes still compositing, as in the pixel kernel

    // reference point of the tile: its first valid point
    if (tr == 0) s_ref_thread = 0xFFFFFFFFu;
    __syncthreads();
    if (inside) atomicMin(&s_ref_thread, tr);
    __syncthreads();
    if (tr == s_ref_thread) { s_ref[0] = px; s_ref[1] = py; }
    __syncthreads();
    const bool any_point = s_ref_thread != 0xFFFFFFFFu; // uniform
    const float ref_x = any_point ? s_ref[0] : 0.f, ref_y = any_point ? s_ref[1] : 0.f;
    const float rx = angle_difference(px, ref_x), ry = angle_difference(py, ref_y);

    const int32_t *offs = a.tile_offsets + (size_t)cam * tiles_per_cam;
    const int32_t range_start = offs[tile_id];
    const int32_t range_end = (cam == a.C - 1 && tile_id == tiles_per_cam - 1)
                                  ? (int32_t)a.n_isects
                                  : offs[tile_id + 1];
    const uint32_t num_batches =
        any_point ? (uint32_t)(range_end - range_start + block_size - 1) / block_size : 0u;
    const bool has_depth = a.depth_idx >= a.ch_offset && a.depth_idx < a.ch_offset + a.n_ch;

    // footprint of this wavefront over its valid lanes
    WavePointCull cull;
    cull.init(inside, rx, ry, roll, block_size % SPLATAD_WAVE == 0);

    float T = 1.0f, asum = 0.f, median = 0.f, depth_extra = 0.f;
    uint32_t cur_idx = 0;
    constexpr int NOUT = MATRIX ? CH - 32 : CH; // channels accumulated by the vector ALUs
    float out[NOUT > 0 ? NOUT : 1];
#pragma unroll
    for (int k = 0; k < NOUT; ++k) out[k] = 0.f;
    floatx16 acc_lo = {0}, acc_hi = {0};     // points 0-31 and 32-63 of the wavefront, D layout
    bool pair_open = false;                  // uniform: a Gaussian waits for its partner
    float pair_weight = 0.f, pair_feature = 0.f;
    // w0, w1: the weights of two Gaussians (lane = point); p0, p1: their payload words, the
    // features in lanes 0-31
    auto add_pair = [&](float w0, float w1, float p0, float p1) {
        const auto sw = __builtin_amdgcn_permlane32_swap(__float_as_uint(w0), __float_as_uint(w1), false, false);
        const auto sf = __builtin_amdgcn_permlane32_swap(__float_as_uint(p0), __float_as_uint(p1), false, false);
        const float f = __uint_as_float(sf[0]); // lanes 0-31: features of the first, 32-63: of the second
        acc_lo = __builtin_amdgcn_mfma_f32_32x32x2f32(__uint_as_float(sw[0]), f, acc_lo, 0, 0, 0);
        acc_hi = __builtin_amdgcn_mfma_f32_32x32x2f32(__uint_as_float(sw[1]), f, acc_hi, 0, 0, 0);
    };

    // One load per Gaussian brings everything compositing needs beyond the staged record, each
    // lane its own word: lanes 0-32 the features of this pass (for the matrix path lanes 0-31
    // are the B layout), lanes 33-36 the range velocity, the two depth compensations and the
    // range.  payload_at + id * payload_step is the lane's address; lanes without a word of
    // their own repeat a neighbour's.
    const uint32_t payload_ch = lane >= 36 ? a.depth_idx : a.ch_offset + min(lane, a.n_ch - 1u);
    const float *payload_at = a.colors + payload_ch;
    uint32_t payload_step = a.feat_stride;
    if (a.range_channel != nullptr && payload_ch == a.depth_idx) { payload_at = a.range_channel; payload_step = 1; }
    if (lane == 33) { payload_at = a.pix_vels + 2; payload_step = 3; }
    if (lane == 34 || lane == 35) { payload_at = a.depth_comps + (lane - 34); payload_step = 2; }

    // A tile's list is long (thousands of Gaussians) and a compute unit holds few of these
    // workgroups, so nothing but the workgroup itself can hide the two dependent memory round
    // trips of a batch (id, then the Gaussian): the values of the next batch are requested
    // before the current batch is worked on, the ids one batch earlier still.
    struct Fetched { float2 xy; float vx, vy, cn[3], opac; };
    auto id_of = [&](uint32_t b) -> int32_t { // Gaussian this lane stages in batch b, or -1
        const uint32_t idx = (uint32_t)range_start + block_size * b + tr;
        return (b < num_batches && idx < (uint32_t)range_end) ? a.flatten_ids[idx] : -1;
    };
    auto fetch = [&](int32_t g) -> Fetched {
        Fetched f = {};
        if (g >= 0) {
            f.xy = reinterpret_cast<const float2 *>(a.means2d)[g];
            const float *v = a.pix_vels + (size_t)g * 3;
            f.vx = v[0]; f.vy = v[1];
            const float *cn = a.conics + (size_t)g * 3;
            f.cn[0] = cn[0]; f.cn[1] = cn[1]; f.cn[2] = cn[2];
            f.opac = a.opacities[g];
        }
        return f;
    };
    int32_t g_now = id_of(0), g_ahead = id_of(1);
    Fetched now = fetch(g_now);

    uint32_t batches_done = 0;
    for (uint32_t b = 0; b < num_batches; ++b) {
        // also orders the previous batch's LDS reads before this batch's writes
        if (__syncthreads_count(!wave_lanes(alive_bits)) >= (int)block_size) break;
        batches_done = b + 1;
        const uint32_t batch_start = (uint32_t)range_start + block_size * b;
        if (g_now >= 0) {
            float4 *rec = s_rec + RECORD * tr;
            rec[0] = make_float4(angle_difference(now.xy.x, ref_x), angle_difference(now.xy.y, ref_y), now.vx, now.vy);
            rec[1] = staged_exponent(now.cn[0], now.cn[1], now.cn[2], now.opac);
            s_gid[tr] = g_now;
        }
        g_now = g_ahead;
        now = fetch(g_now);
        g_ahead = id_of(b + 2);
        __syncthreads();

        const uint32_t batch_size = min(block_size, (uint32_t)range_end - batch_start);
        // The footprint test runs over the whole batch first, 64 staged Gaussians per round; a
        // survivor's position in the batch and its id go to a list that belongs to the wavefront.
        uint32_t n_surv = 0; // uniform
        for (uint32_t base = 0; base < batch_size && alive_bits != 0; base += SPLATAD_WAVE) {
            bool keep = base + lane < batch_size, unfolded_ok = true;
            if (keep) keep = cull.may_touch(s_rec[RECORD * (base + lane)], s_rec[RECORD * (base + lane) + 1], unfolded_ok);
            const uint64_t kept = wave_ballot(keep);
            if (keep)
                s_surv[n_surv + (uint32_t)__popcll(kept & ((1ull << lane) - 1ull))] =
                    make_uint2((base + lane) | (unfolded_ok ? 0u : 0x80000000u), (uint32_t)s_gid[base + lane]);
            n_surv += (uint32_t)__popcll(kept);
        }
        // the list is written and read by the same wavefront, whose LDS operations complete in
        // order; the fences keep the compiler from moving the reads above the writes
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        // The survivors are composited four at a time.  What a Gaussian needs beyond its staged
        // record comes from global memory, a wait ten times longer than the work on the
        // Gaussian: a group's words are requested before the group ahead of it is composited
        // (two groups in two sets of registers, taking turns), so that the wait overlaps that
        // work.  Slots beyond the last survivor repeat it.
        constexpr int K = 4;
        struct Group {
            uint32_t ts[K]; // position in the batch, bit 31: the offset needs folding (uniform)
            float pay[K];
        };
        auto request = [&](Group &g, uint32_t first) {
#pragma unroll
            for (int k = 0; k < K; ++k) {
                const uint2 e = s_surv[min(first + (uint32_t)k, n_surv - 1u)];
                g.ts[k] = (uint32_t)__builtin_amdgcn_readfirstlane((int)e.x);
                g.pay[k] = payload_at[(size_t)(uint32_t)__builtin_amdgcn_readfirstlane((int)e.y) * payload_step];
            }
        };
        auto composite = [&](const Group &g, uint32_t count) {
            float4 uvs[K], cons[K];
#pragma unroll
            for (int k = 0; k < K; ++k) {
                uvs[k] = s_rec[RECORD * (g.ts[k] & 0x7FFFFFFFu)];
                cons[k] = s_rec[RECORD * (g.ts[k] & 0x7FFFFFFFu) + 1];
            }
#pragma unroll
            for (int k = 0; k < K; ++k) {
                if ((uint32_t)k >= count || alive_bits == 0) break; // uniform
                const float4 uv = uvs[k], con = cons[k];
                float dx = gaussian_offset(uv.x, uv.z, roll, rx);
                float dy = gaussian_offset(uv.y, uv.w, roll, ry);
                if (g.ts[k] >> 31) { // uniform, rare: half a turn away from the tile
                    dx = angle_difference(fmaf(roll, uv.z, uv.x), rx);
                    dy = angle_difference(fmaf(roll, uv.w, uv.y), ry);
                }
                const float power = gaussian_power(con, dx, dy);
                const float alpha = fminf(0.999f, __builtin_amdgcn_exp2f(con.w - power));
                const float weight = alpha * T;
                const float next_T = transmittance_behind(T, alpha);
                const uint64_t valid_bits = alive_bits & wave_ballot(!(power < 0.f)) &
                                            wave_ballot(!(alpha < 1.f / 255.f));
                const uint64_t stop_bits = valid_bits & wave_ballot(next_T <= 1e-4f);
                const uint64_t take_bits = valid_bits & ~stop_bits;
                alive_bits &= ~stop_bits;
                if (take_bits != 0) {
                    const bool take = wave_lanes(take_bits);
                    const float vis = take ? weight : 0.f;
                    const int word = __float_as_int(g.pay[k]);
                    const float4 ext = make_float4(__int_as_float(__builtin_amdgcn_readlane(word, 33)),
                                                   __int_as_float(__builtin_amdgcn_readlane(word, 34)),
                                                   __int_as_float(__builtin_amdgcn_readlane(word, 35)),
                                                   __int_as_float(__builtin_amdgcn_readlane(word, 36)));
                    if constexpr (MATRIX) {
                        if constexpr (CH == 33) out[0] += __int_as_float(__builtin_amdgcn_readlane(word, 32)) * vis;
                        if (pair_open) add_pair(pair_weight, vis, pair_feature, g.pay[k]);
                        else { pair_weight = vis; pair_feature = g.pay[k]; }
                        pair_open = !pair_open;
                    } else { // accumulators beyond n_ch repeat the last channel and are never stored
#pragma unroll
                        for (int c = 0; c < CH; ++c) out[c] += __int_as_float(__builtin_amdgcn_readlane(word, c)) * vis;
                    }
                    const float extra = ext.y * dx + ext.z * dy + ext.x * roll;
                    depth_extra += extra * vis;
                    if (take && T > 0.5f && next_T <= 0.5f) median = ext.w + extra;
                    if (take && a.compute_alpha_sum && ext.w < pz - a.threshold) asum += alpha;
                    cur_idx = take ? batch_start + (g.ts[k] & 0x7FFFFFFFu) : cur_idx;
                    T -= vis;
                }
            }
        };
        if (n_surv != 0) {
            Group even, odd;
            request(even, 0);
            // (a request beyond the list repeats the last survivor: issued all the same, so that
            // the number of loads in flight at every wait is known when the kernel is compiled)
            for (uint32_t first = 0; first < n_surv && alive_bits != 0; first += 2 * K) { // uniform
                request(odd, first + K);
                composite(even, min((uint32_t)K, n_surv - first));
                if (first + K >= n_surv || alive_bits == 0) break;
                request(even, first + 2 * K);
                composite(odd, min((uint32_t)K, n_surv - first - K));
            }
        }
    }

    if (a.tile_batches != nullptr && a.write_aux && tr == 0)
        a.tile_batches[blockIdx.x] = (int32_t)min(batches_done * block_size, (uint32_t)(range_end - range_start));
    if (a.tile_cycles != nullptr && a.write_aux && tr == 0) a.tile_cycles[blockIdx.x] = clock64() - t_begin;
    if constexpr (MATRIX) {
        if (pair_open) add_pair(pair_weight, 0.f, pair_feature, 0.f);
        // what the D layout needs to know of a point: where it is stored, its transmittance
        // (negative: nothing composited, store zero; NaN: outside the image, store nothing)
        // and the depth term, through the LDS the batches no longer use
        __syncthreads();
        float4 *s_point = lds4;
        s_point[tr] = make_float4(__uint_as_float((uint32_t)(pix & 0xFFFFFFFFu)), __uint_as_float((uint32_t)(pix >> 32)),
                                  in_image ? (inside ? T : -1.f) : NAN, depth_extra);
        __syncthreads();
        const uint32_t n = lane & 31u, half = lane >> 5, wave_first = tr & ~(SPLATAD_WAVE - 1);
        const float bg_n = a.backgrounds ? a.backgrounds[(size_t)cam * a.color_stride + a.ch_offset + n] : 0.f;
        const bool depth_here = has_depth && n == a.depth_idx - a.ch_offset;
#pragma unroll
        for (int m = 0; m < 2; ++m) {
#pragma unroll
            for (int j = 0; j < 16; ++j) {
                const uint32_t i = 8u * (j / 4) + 4u * half + (j % 4);
                const float4 pt = s_point[wave_first + 32u * m + i];
                if (pt.z == pt.z) { // inside the image
                    const size_t at = ((size_t)__float_as_uint(pt.y) << 32) | __float_as_uint(pt.x);
                    float v = m == 0 ? acc_lo[j] : acc_hi[j];
                    if (depth_here) v += pt.w;
                    v += pt.z * bg_n; // no background: bg_n = 0
                    a.render_colors[at * a.color_stride + a.ch_offset + n] = pt.z >= 0.f ? v : 0.f;
                }
            }
        }
    }
    if (in_image) {
        float *dst = a.render_colors + pix * a.color_stride + a.ch_offset + (MATRIX ? 32 : 0);
        const float *bg = a.backgrounds ? a.backgrounds + (size_t)cam * a.color_stride + a.ch_offset + (MATRIX ? 32 : 0) : nullptr;
#pragma unroll
        for (int k = 0; k < NOUT; ++k) {
            if (MATRIX || (uint32_t)k < a.n_ch) {
                float v = out[k];
                if (has_depth && (uint32_t)k + (MATRIX ? 32u : 0u) == a.depth_idx - a.ch_offset) v += depth_extra;
                if (bg && inside) v += T * bg[k];
                dst[k] = inside ? v : 0.f;
            }
        }
        if (a.write_aux) {
            a.render_alphas[pix] = inside ? 1.0f - T : 0.f;
            a.last_ids[pix] = inside ? (int32_t)cur_idx : 0;
            a.median_depths[pix] = median;
            if (a.alpha_sum) a.alpha_sum[pix] = asum;
        }
    }
}

// Compiled accumulator widths; a pass of n channels uses the smallest width >= n.
constexpr int kWidths[] = {1, 2, 3, 4, 5, 8, 9, 16, 17, 32, 33};
constexpr int kMaxPass = 33;

static inline int pick_width(uint32_t n) {
    for (int w : kWidths)
        if ((uint32_t)w >= n) return w;
    return -1;
}

// Two pixels per lane where the tile makes whole wavefronts of 8 x 16 pixels.
static inline int pixels_per_lane(uint32_t tile_size) {
    return tile_size % 8 == 0 && (tile_size * tile_size / 2) % SPLATAD_WAVE == 0 ? 2 : 1;
}

template <int CH>
static size_t pixel_lds_bytes(uint32_t threads) {
    const size_t waves = (threads + SPLATAD_WAVE - 1) / SPLATAD_WAVE;
    return 16 * ((size_t)threads * (2 + (CH + 3) / 4) + waves * SPLATAD_WAVE * (CH <= 4 ? 3 : 2));
}

template <int CH, int PPL, bool STATS, bool SHC = false, bool LAST = true>
static int launch_pixels_as(const PixelArgs &a, dim3 grid, uint32_t threads, hipStream_t stream) {
    const size_t lds = pixel_lds_bytes<CH>(threads);
    if (lds > 64 * 1024)
        SPLATAD_CHECK_HIP(hipFuncSetAttribute((const void *)rasterize_to_pixels_fwd_kernel<CH, PPL, STATS, SHC, LAST>,
                                              hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
    hipLaunchKernelGGL((rasterize_to_pixels_fwd_kernel<CH, PPL, STATS, SHC, LAST>), grid, dim3(threads), lds, stream, a);
    SPLATAD_LAUNCH_CHECK();
    return 0;
}

// Colours from spherical harmonics: three or four channels in one pass.
template <int CH>
static int launch_pixels_sh(const PixelArgs &a, dim3 grid, dim3 block, hipStream_t stream) {
    const uint32_t pixels = block.x * block.y;
    const bool two = pixels_per_lane(a.tile_size) == 2;
    if (a.last_ids == nullptr) // a call that takes no gradient wants no last ids
        return two ? launch_pixels_as<CH, 2, false, true, false>(a, grid, pixels / 2, stream)
                   : launch_pixels_as<CH, 1, false, true, false>(a, grid, pixels, stream);
    return two ? launch_pixels_as<CH, 2, false, true>(a, grid, pixels / 2, stream)
               : launch_pixels_as<CH, 1, false, true>(a, grid, pixels, stream);
}

template <int CH>
static int launch_pixels(const PixelArgs &a, dim3 grid, dim3 block, hipStream_t stream) {
    const uint32_t pixels = block.x * block.y;
    if (pixels_per_lane(a.tile_size) == 2) return launch_pixels_as<CH, 2, false>(a, grid, pixels / 2, stream);
    return launch_pixels_as<CH, 1, false>(a, grid, pixels, stream);
}

template <int CH>
static int launch_points(const PointArgs &a, dim3 grid, dim3 block, hipStream_t stream) {
    // two float4 and the id per staged Gaussian, and a survivor list of that length per wavefront
    const size_t threads = (size_t)block.x * block.y;
    const size_t lds = threads * (2 * 16 + 4) + (threads / SPLATAD_WAVE) * threads * 8;
    if constexpr (CH == 32 || CH == 33) {
        // the matrix-core path: every channel of the kernel in use
        if (a.n_ch == (uint32_t)CH) {
            hipLaunchKernelGGL((rasterize_to_points_fwd_kernel<CH, true>), grid, block, lds, stream, a);
            SPLATAD_LAUNCH_CHECK();
            return 0;
        }
    }
    hipLaunchKernelGGL((rasterize_to_points_fwd_kernel<CH, false>), grid, block, lds, stream, a);
    SPLATAD_LAUNCH_CHECK();
    return 0;
}

#define DISPATCH_WIDTH(w, CALL)                                                              \
    switch (w) {                                                                             \
    case 1: return CALL(1);                                                                  \
    case 2: return CALL(2);                                                                  \
    case 3: return CALL(3);                                                                  \
    case 4: return CALL(4);                                                                  \
    case 5: return CALL(5);                                                                  \
    case 8: return CALL(8);                                                                  \
    case 9: return CALL(9);                                                                  \
    case 16: return CALL(16);                                                                \
    case 17: return CALL(17);                                                                \
    case 32: return CALL(32);                                                                \
    case 33: return CALL(33);                                                                \
    default: break;                                                                          \
    }

static int dispatch_pixels(int w, const PixelArgs &a, dim3 grid, dim3 block, hipStream_t s) {
#define CALL_PIX(W) launch_pixels<W>(a, grid, block, s)
    DISPATCH_WIDTH(w, CALL_PIX)
#undef CALL_PIX
    splatad_set_error("rasterize_to_pixels: no kernel for %d channels per pass", w);
    return -1;
}

static int dispatch_points(int w, const PointArgs &a, dim3 grid, dim3 block, hipStream_t s) {
#define CALL_PTS(W) launch_points<W>(a, grid, block, s)
    DISPATCH_WIDTH(w, CALL_PTS)
#undef CALL_PTS
    splatad_set_error("rasterize_to_points: no kernel for %d channels per pass", w);
    return -1;
}

} // namespace

extern "C" int splatad_rasterize_to_pixels_fwd(
    uint32_t C, int64_t n_isects, uint32_t channels, const float *means2d, const float *conics,
    const float *colors, const float *opacities, const float *pix_vels, const float *rs_time,
    const float *backgrounds, uint32_t W, uint32_t H, uint32_t tile_size, uint32_t tile_w,
    uint32_t tile_h, const int32_t *tile_offsets, const int32_t *flatten_ids,
    float *render_colors, float *render_alphas, int32_t *last_ids, int32_t *tile_batches,
    int64_t *tile_cycles, splatad_stream_t stream) {
    SPLATAD_REQUIRE(channels >= 1, "rasterize_to_pixels: zero channels");
    SPLATAD_REQUIRE(tile_size >= 1 && tile_size * tile_size <= 1024,
                    "rasterize_to_pixels: tile_size %u is outside 1..32", tile_size);
    if (C == 0 || W == 0 || H == 0) return 0;
    SPLATAD_REQUIRE((uint64_t)tile_w * tile_size >= W && (uint64_t)tile_h * tile_size >= H,
                    "rasterize_to_pixels: tile grid %ux%u of size %u does not cover %ux%u", tile_w,
                    tile_h, tile_size, W, H);
    SPLATAD_REQUIRE(n_isects >= 0 && n_isects < (1ll << 31), "rasterize_to_pixels: bad n_isects");
    SPLATAD_REQUIRE(rs_time && tile_offsets && render_colors && render_alphas && last_ids,
                    "rasterize_to_pixels: null pointer argument");
    SPLATAD_REQUIRE(n_isects == 0 || (means2d && conics && colors && opacities && pix_vels && flatten_ids),
                    "rasterize_to_pixels: null pointer argument");
    PixelArgs a;
    a.C = C; a.n_isects = n_isects; a.color_stride = channels;
    a.means2d = means2d; a.conics = conics; a.colors = colors; a.opacities = opacities;
    a.pix_vels = pix_vels; a.rs_time = rs_time; a.backgrounds = backgrounds;
    a.W = W; a.H = H; a.tile_size = tile_size; a.tile_w = tile_w; a.tile_h = tile_h;
    a.tile_offsets = tile_offsets; a.flatten_ids = flatten_ids;
    a.render_colors = render_colors; a.render_alphas = render_alphas; a.last_ids = last_ids;
    a.tile_batches = tile_batches;
    a.tile_cycles = tile_cycles;
    a.lane_stats = nullptr;
    const dim3 grid(C * tile_w * tile_h), block(tile_size, tile_size);
    const uint32_t pass = channels <= (uint32_t)kMaxPass ? channels : 32u;
    for (uint32_t off = 0; off < channels; off += pass) {
        a.ch_offset = off;
        a.n_ch = min(pass, channels - off);
        a.write_aux = off == 0;
        int rc = dispatch_pixels(pick_width(a.n_ch), a, grid, block, (hipStream_t)stream);
        if (rc) return rc;
    }
    return 0;
}

extern "C" int splatad_rasterize_to_pixels_fwd_sh(
    uint32_t C, uint32_t N, int64_t n_isects, uint32_t K, uint32_t degree, const float *means,
    const float *viewmats, const float *coeffs, int coeffs_per_sensor,
    const int64_t *gaussian_ids, const float *depths, float *color_cache,
    const float *means2d, const float *conics, const float *opacities, const float *pix_vels,
    const float *rs_time, const float *backgrounds, uint32_t W, uint32_t H, uint32_t tile_size,
    uint32_t tile_w, uint32_t tile_h, const int32_t *tile_offsets, const int32_t *flatten_ids,
    float *render_colors, float *render_alphas, int32_t *last_ids, splatad_stream_t stream) {
    SPLATAD_REQUIRE(degree <= 4 && K >= (degree + 1) * (degree + 1),
                    "rasterize_to_pixels: %u coefficients do not hold degree %u", K, degree);
    SPLATAD_REQUIRE(tile_size >= 1 && tile_size * tile_size <= 1024,
                    "rasterize_to_pixels: tile_size %u is outside 1..32", tile_size);
    if (C == 0 || W == 0 || H == 0) return 0;
    SPLATAD_REQUIRE((uint64_t)tile_w * tile_size >= W && (uint64_t)tile_h * tile_size >= H,
                    "rasterize_to_pixels: tile grid %ux%u of size %u does not cover %ux%u", tile_w,
                    tile_h, tile_size, W, H);
    SPLATAD_REQUIRE(n_isects >= 0 && n_isects < (1ll << 31), "rasterize_to_pixels: bad n_isects");
    SPLATAD_REQUIRE((uint64_t)C * N < (1ull << 31), "rasterize_to_pixels: %u x %u rows exceed the id range", C, N);
    SPLATAD_REQUIRE(rs_time && viewmats && tile_offsets && render_colors && render_alphas,
                    "rasterize_to_pixels: null pointer argument");
    SPLATAD_REQUIRE(n_isects == 0 || (means && coeffs && color_cache && means2d && conics && opacities &&
                                      pix_vels && flatten_ids),
                    "rasterize_to_pixels: null pointer argument");
    PixelArgs a = {};
    a.C = C; a.n_isects = n_isects;
    a.color_stride = depths != nullptr ? 4u : 3u;
    a.ch_offset = 0; a.n_ch = a.color_stride; a.write_aux = 1;
    a.means2d = means2d; a.conics = conics; a.opacities = opacities;
    a.pix_vels = pix_vels; a.rs_time = rs_time; a.backgrounds = backgrounds;
    a.W = W; a.H = H; a.tile_size = tile_size; a.tile_w = tile_w; a.tile_h = tile_h;
    a.tile_offsets = tile_offsets; a.flatten_ids = flatten_ids;
    a.render_colors = render_colors; a.render_alphas = render_alphas; a.last_ids = last_ids;
    a.sh_means = means; a.sh_viewmats = viewmats; a.sh_coeffs = coeffs; a.sh_depths = depths;
    a.sh_gaussian_ids = gaussian_ids; a.sh_cache = color_cache;
    a.sh_N = N; a.sh_K = K; a.sh_degree = degree; a.sh_per_sensor = coeffs_per_sensor;
    const dim3 grid(C * tile_w * tile_h), block(tile_size, tile_size);
    if (depths != nullptr) return launch_pixels_sh<4>(a, grid, block, (hipStream_t)stream);
    return launch_pixels_sh<3>(a, grid, block, (hipStream_t)stream);
}

extern "C" int splatad_rasterize_to_pixels_lane_stats(
    uint32_t C, int64_t n_isects, const float *means2d, const float *conics, const float *opacities,
    const float *pix_vels, const float *rs_time, uint32_t W, uint32_t H, uint32_t tile_size,
    uint32_t tile_w, uint32_t tile_h, const int32_t *tile_offsets, const int32_t *flatten_ids,
    unsigned long long *stats, splatad_stream_t stream) {
    SPLATAD_REQUIRE(tile_size >= 1 && tile_size * tile_size <= 1024,
                    "rasterize_to_pixels: tile_size %u is outside 1..32", tile_size);
    if (C == 0 || W == 0 || H == 0 || n_isects == 0) return 0;
    SPLATAD_REQUIRE((uint64_t)tile_w * tile_size >= W && (uint64_t)tile_h * tile_size >= H,
                    "rasterize_to_pixels: tile grid does not cover the image");
    SPLATAD_REQUIRE(n_isects > 0 && n_isects < (1ll << 31), "rasterize_to_pixels: bad n_isects");
    SPLATAD_REQUIRE(rs_time && tile_offsets && means2d && conics && opacities && pix_vels && flatten_ids && stats,
                    "rasterize_to_pixels: null pointer argument");
    PixelArgs a = {};
    a.C = C; a.n_isects = n_isects; a.color_stride = 0; a.ch_offset = 0; a.n_ch = 0;
    a.means2d = means2d; a.conics = conics; a.opacities = opacities;
    a.pix_vels = pix_vels; a.rs_time = rs_time;
    a.W = W; a.H = H; a.tile_size = tile_size; a.tile_w = tile_w; a.tile_h = tile_h;
    a.tile_offsets = tile_offsets; a.flatten_ids = flatten_ids;
    a.lane_stats = stats;
    const dim3 grid(C * tile_w * tile_h);
    const uint32_t pixels = tile_size * tile_size;
    if (pixels_per_lane(tile_size) == 2) return launch_pixels_as<1, 2, true>(a, grid, pixels / 2, (hipStream_t)stream);
    return launch_pixels_as<1, 1, true>(a, grid, pixels, (hipStream_t)stream);
}

extern "C" int splatad_rasterize_to_points_fwd(
    uint32_t C, int64_t n_isects, uint32_t channels, const float *means2d, const float *conics,
    const float *colors, const float *range_channel, const float *opacities, const float *pix_vels,
    const float *depth_comps, const float *backgrounds, const float *raster_pts, uint32_t W,
    uint32_t H, uint32_t tile_width, uint32_t tile_height, uint32_t grid_w, uint32_t grid_h,
    int compute_alpha_sum, float threshold, const int32_t *tile_offsets,
    const int32_t *flatten_ids, uint32_t depth_idx, float *render_colors, float *render_alphas,
    float *alpha_sum, int32_t *last_ids, float *median_depths, int32_t *tile_batches,
    int64_t *tile_cycles, splatad_stream_t stream) {
    SPLATAD_REQUIRE(channels >= 1, "rasterize_to_points: zero channels");
    SPLATAD_REQUIRE(depth_idx < channels, "rasterize_to_points: depth channel %u of %u", depth_idx, channels);
    SPLATAD_REQUIRE(range_channel == nullptr || (depth_idx + 1 == channels && channels >= 2),
                    "rasterize_to_points: a separate range channel must be the last of at least two");
    SPLATAD_REQUIRE(tile_width >= 1 && tile_height >= 1 && tile_width * tile_height <= 256,
                    "rasterize_to_points: tile %ux%u exceeds 256 points", tile_width, tile_height);
    if (C == 0 || W == 0 || H == 0) return 0;
    SPLATAD_REQUIRE((uint64_t)grid_w * tile_width >= W && (uint64_t)grid_h * tile_height >= H,
                    "rasterize_to_points: tile grid does not cover the point image");
    SPLATAD_REQUIRE(n_isects >= 0 && n_isects < (1ll << 31), "rasterize_to_points: bad n_isects");
    SPLATAD_REQUIRE(raster_pts && tile_offsets && render_colors && render_alphas && last_ids && median_depths,
                    "rasterize_to_points: null pointer argument");
    SPLATAD_REQUIRE(!compute_alpha_sum || alpha_sum, "rasterize_to_points: alpha_sum output is null");
    SPLATAD_REQUIRE(n_isects == 0 || (means2d && conics && colors && opacities && pix_vels && depth_comps && flatten_ids),
                    "rasterize_to_points: null pointer argument");
    PointArgs a;
    a.C = C; a.n_isects = n_isects; a.color_stride = channels;
    a.feat_stride = range_channel ? channels - 1 : channels;
    a.range_channel = range_channel;
    a.means2d = means2d; a.conics = conics; a.colors = colors; a.opacities = opacities;
    a.pix_vels = pix_vels; a.depth_comps = depth_comps; a.backgrounds = backgrounds;
    a.raster_pts = raster_pts; a.W = W; a.H = H; a.tile_width = tile_width;
    a.tile_height = tile_height; a.grid_w = grid_w; a.grid_h = grid_h;
    a.compute_alpha_sum = compute_alpha_sum; a.threshold = threshold;
    a.tile_offsets = tile_offsets; a.flatten_ids = flatten_ids; a.depth_idx = depth_idx;
    a.render_colors = render_colors; a.render_alphas = render_alphas;
    a.alpha_sum = compute_alpha_sum ? alpha_sum : nullptr;
    a.last_ids = last_ids; a.median_depths = median_depths; a.tile_batches = tile_batches;
    a.tile_cycles = tile_cycles;
    const dim3 grid(C * grid_w * grid_h), block((tile_width * tile_height + SPLATAD_WAVE - 1) / SPLATAD_WAVE * SPLATAD_WAVE);
    const uint32_t pass = channels <= (uint32_t)kMaxPass ? channels : 32u;
    for (uint32_t off = 0; off < channels; off += pass) {
        a.ch_offset = off;
        a.n_ch = min(pass, channels - off);
        a.write_aux = off == 0;
        int rc = dispatch_points(pick_width(a.n_ch), a, grid, block, (hipStream_t)stream);
        if (rc) return rc;
    }
    return 0;
}
