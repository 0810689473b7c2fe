// Backward of the alpha compositing for camera pixels and lidar points on gfx950.
//
// One workgroup per (sensor, tile), one lane per pixel / point, lanes laid out as in the
// forward kernels.  Each pixel replays its tile's list back to front, starting at the last
// Gaussian it took in the forward pass, and recovers the transmittance by dividing
// (T_before = T_after / (1 - alpha)).  Batches of the list are staged in LDS in the same form
// as in the forward pass, so that both passes take the same alpha >= 1/255 decisions.  Every
// wavefront first tests the batch against its footprint, 64 Gaussians at a time, and then
// walks only those Gaussians some lane of it can see.  Per Gaussian, the pixel gradients
// (colours and geometry, up to 46 values) are summed over the wavefront with one
// reduce-scatter, accumulated across the wavefronts of the workgroup in LDS, and flushed
// with one global atomic per value and (tile, Gaussian) when the batch is finished.  Batches
// behind the deepest entry any pixel of the tile consumed are never loaded.
//
// Gradient rules follow gsplat/cuda/csrc/rasterization.cu:2833-3089 (pixels) and :3728-4054
// (points) of the reference.  Channels beyond 33 are handled in passes; the geometry
// gradients are linear in the per-channel terms, so the passes add up exactly (the absolute
// gradient v_means2d_abs then adds the per-pass magnitudes).
#include "raster_common.h"

namespace {

struct BwdArgs {
    uint32_t C;
    int64_t n_isects;
    uint32_t color_stride, ch_offset, n_ch;
    // Lidar only: with range_channel given, `colors` and `v_colors` have rows of feat_stride =
    // color_stride - 1 values and channel depth_idx (the last one) lives in range_channel /
    // v_range, one value per Gaussian; otherwise feat_stride == color_stride.
    uint32_t feat_stride;
    const float *range_channel;
    float *v_range;
    const float *means2d, *conics, *colors, *opacities, *pix_vels, *depth_comps, *rs_time,
        *backgrounds, *raster_pts;
    uint32_t W, H, tile_w_px, tile_h_px, grid_w, grid_h;
    int compute_alpha_sum;
    float threshold;
    const int32_t *tile_offsets, *flatten_ids;
    uint32_t depth_idx;
    const float *render_alphas;
    const int32_t *last_ids;
    const float *v_render_colors, *v_render_alphas, *v_alpha_sum;
    float *v_means2d_abs, *v_means2d, *v_conics, *v_colors, *v_opacities, *v_pix_vels, *v_depth_comps;
    int first_pass; // adds the alpha / alpha-sum terms exactly once over the channel passes
    // Packed accumulation: when given, the gradients of Gaussian g go to packed[g * packed_stride
    // + slot] (slot = channel of the pass, then the geometry slots below) instead of the v_*
    // arrays; unpack_gradients_kernel distributes them afterwards.
    float *packed;
    uint32_t packed_stride;
    uint32_t batch; // Gaussians staged per batch, at most the workgroup size
    // `colors` is the colour cache a forward pass that evaluated the colours itself left behind:
    // rows no tile staged hold NaN; no pixel composited them, and they are taken as zero
    int colors_from_cache;
};

// Geometry slots per Gaussian in the LDS accumulator, after the CH colour slots; those from
// G_VELZ on exist for lidars only.  While a batch is worked on the slots hold moments of the
// pixels' gradients of the exponent, s = dL/dsigma per pixel, not yet the gradients themselves:
// G_CONIC: sum s dx^2, s dx dy, s dy^2; G_XY: sum s dx, s dy; G_VEL: sum s dx roll, s dy roll;
// G_OPAC: sum s; and for the lidar's depth term d = dL/d(depth value) per point, G_DC: sum d dx,
// d dy; G_VELZ: sum d roll; G_D0: sum d.  Every geometry gradient is a combination of these
// with coefficients that belong to the Gaussian, not the pixel (its conic, its opacity, its
// depth compensation), so the pixels accumulate the moments -- a dozen multiply-adds instead of
// the two conic rows and a product per gradient -- and the flush forms the gradients once per
// (tile, Gaussian), see gradients_from_moments().  G_ABS (the absolute image-plane gradients, which
// are sums of absolute values and do not factor) is accumulated as such, and only where wanted.
// The two G_ABS slots come last (behind G_OPAC for cameras, behind G_D0 for lidars), so that a
// kernel compiled without them sums two values less per Gaussian over the wavefront; records
// and unpacking always have room for them.
enum { G_CONIC = 0, G_XY = 3, G_VEL = 5, G_OPAC = 7, G_VELZ = 8, G_DC = 9, G_D0 = 11 };
constexpr int geo_abs(bool lidar) { return lidar ? 12 : 8; }
constexpr int geo_count(bool lidar, bool with_abs = true) { return geo_abs(lidar) + (with_abs ? 2 : 0); }

// Turns the moments `m` (the geometry slots of one Gaussian) into the gradients, in place, from
// its staged exponent e = {A, B, C, L}, 1 / opacity and, for lidars, ext = {range velocity,
// depth compensation x, y, depth}: with a = 2 ln2 A, b = ln2 B, c = 2 ln2 C the conic,
//   v_conic = (m_xx / 2, m_xy, m_yy / 2),        v_mean = (a m_x + b m_y, b m_x + c m_y) [+ dc m_d0],
//   v_vel   = the same of (m_xr, m_yr) [+ dc m_dr], v_opacity = -m_0 / opacity;
// the absolute gradients, G_VELZ and G_DC are gradients as accumulated, G_D0 is none and is cleared.
template <bool LIDAR>
__device__ __forceinline__ void gradients_from_moments(float *m, float4 e, float rop, float4 ext) {
    const float a = 2.f * kLn2 * e.x, b = kLn2 * e.y, c = 2.f * kLn2 * e.z;
    const float mx = m[G_XY], my = m[G_XY + 1], mxr = m[G_VEL], myr = m[G_VEL + 1];
    float gx = a * mx + b * my, gy = b * mx + c * my;
    float vx = a * mxr + b * myr, vy = b * mxr + c * myr;
    if constexpr (LIDAR) {
        const float d0 = m[G_D0], dr = m[G_VELZ];
        gx += ext.y * d0; gy += ext.z * d0;
        vx += ext.y * dr; vy += ext.z * dr;
        m[G_D0] = 0.f;
    }
    m[G_CONIC] *= 0.5f;
    m[G_CONIC + 2] *= 0.5f;
    m[G_XY] = gx; m[G_XY + 1] = gy;
    m[G_VEL] = vx; m[G_VEL + 1] = vy;
    m[G_OPAC] *= -rop;
}

// The per-Gaussian values are summed over the wavefront in one or two power-of-two groups (a
// reduce-scatter of n values costs about 2 n operations): first(n) values, then second(n).
constexpr int reduce_first(int n) { return n <= 12 ? 8 : (n <= 24 ? 16 : (n <= 48 ? 32 : 64)); }
constexpr int reduce_second(int n) {
    return n <= 8 ? 0 : (n <= 12 ? 4 : (n <= 16 ? 0 : (n <= 24 ? 8 : (n <= 32 ? 0 : (n <= 48 ? 16 : 0)))));
}

// PPL: pixels per lane.  Two for camera tiles that make whole wavefronts of 8 x 16 pixels (rows y
// and y + 8 of a column, as in the forward kernel) and few channels: the wavefront reduction of
// the per-Gaussian gradients, about 40 of the 110 vector instructions of a (wavefront, Gaussian)
// step, is then paid once per 128 pixels, and a Gaussian is fetched from the LDS half as often.
// ABS: the kernel also sums the absolute image-plane gradients (v_means2d_abs not null).
template <int CH, bool LIDAR, int PPL, bool ABS = true>
__global__ void __launch_bounds__(256)
rasterize_bwd_kernel(BwdArgs a) {
    static_assert(PPL == 1 || (PPL == 2 && !LIDAR), "two pixels per lane are a camera layout");
    constexpr int G_ABS = geo_abs(LIDAR);
    extern __shared__ float4 lds4[];
    __shared__ int32_t s_block_final;
    __shared__ uint32_t s_ref_thread;
    __shared__ float s_ref[2];
    // the workgroup is one-dimensional and padded to whole wavefronts: the wavefront
    // reductions below need all 64 lanes; lanes beyond the tile own no pixel
    const uint32_t block_size = blockDim.x;
    // {x, y, vx, vy}, staged exponent, then the lidar extras or, for cameras, the polynomial of
    // the exponent as the forward kernel stages it (same functions, same bits)
    constexpr int RECORD = LIDAR ? 3 : 4;
    constexpr int GEO = geo_count(LIDAR, ABS);
    constexpr int ACC = CH + GEO;
    constexpr int NA = reduce_first(ACC), NB = reduce_second(ACC), NV = NA + NB;
    static_assert(ACC <= SPLATAD_WAVE, "the flush gives every accumulator slot a lane");
    float4 *s_rec = lds4;
    // Gaussians per batch: the first `batch` lanes stage one each.  Fewer than the workgroup has
    // lanes where the LDS of a full batch would leave a compute unit with a single workgroup.
    const uint32_t batch = a.batch;
    float2 *s_aux = reinterpret_cast<float2 *>(lds4 + (size_t)RECORD * batch); // {id, 1/opacity}
    float *s_col = reinterpret_cast<float *>(s_aux + batch);                   // [batch][CH]
    float *s_acc = s_col + (size_t)batch * CH;                                 // [batch][ACC]

    const uint32_t tiles_per_cam = a.grid_w * a.grid_h;
    const uint32_t cam = blockIdx.x / tiles_per_cam;
    const uint32_t tile_id = blockIdx.x % tiles_per_cam;
    const uint32_t tr = threadIdx.x;
    const int lane = tr & (SPLATAD_WAVE - 1);
    uint32_t lx, ly;
    if (LIDAR) {
        point_of_lane(a.tile_w_px, a.tile_h_px, tr, lx, ly);
    } else if (PPL == 2) {
        const uint32_t waves_per_row = a.tile_w_px / 8, wave = tr / SPLATAD_WAVE;
        lx = (wave % waves_per_row) * 8 + ((uint32_t)lane & 7u);
        ly = (wave / waves_per_row) * 16 + ((uint32_t)lane >> 3);
    } else {
        pixel_of_lane(a.tile_w_px, tr, lx, ly);
    }
    const uint32_t j = (tile_id % a.grid_w) * a.tile_w_px + lx;
    // per pixel of the lane (index p below): row, position, rolling-shutter factor
    uint32_t i[PPL];
    bool in_image[PPL], inside[PPL];
    size_t pix[PPL];
    uint64_t inside_bits[PPL];
    float px, py[PPL], pz = 1.f, roll[PPL];
    px = (float)j + 0.5f;
#pragma unroll
    for (int p = 0; p < PPL; ++p) {
        i[p] = (tile_id / a.grid_w) * a.tile_h_px + ly + 8u * p;
        in_image[p] = (tr * PPL < a.tile_w_px * a.tile_h_px && i[p] < a.H && j < a.W);
        pix[p] = in_image[p] ? ((size_t)cam * a.H + i[p]) * a.W + j : 0;
        if (LIDAR) {
            px = py[p] = roll[p] = 0.f;
            pz = 0.f;
            if (in_image[p]) {
                const float4 pt = reinterpret_cast<const float4 *>(a.raster_pts)[pix[p]];
                px = pt.x; py[p] = pt.y; pz = pt.z; roll[p] = pt.w;
            }
        } else {
            py[p] = (float)i[p] + 0.5f;
            roll[p] = a.rs_time[cam] * ((py[p] - 0.5f) / (float)(a.H - 1) - 0.5f);
        }
        inside[p] = in_image[p] && pz > 0.f;
        inside_bits[p] = wave_ballot(inside[p]);
    }
    // Cameras: alpha comes from the forward kernel's polynomial in tile-centred pixel
    // coordinates, evaluated by the same function on the same staged coefficients, so that this
    // pass takes the forward pass's alpha >= 1/255 and sigma < 0 decisions bit for bit; the
    // offsets to the Gaussian's centre are still needed, for the gradients.
    TileFrame frame = {};
    PixelConstants pc[PPL] = {};
    if (!LIDAR) {
        frame = tile_frame(tile_id % a.grid_w, tile_id / a.grid_w, a.tile_w_px, a.rs_time[cam], a.H);
#pragma unroll
        for (int p = 0; p < PPL; ++p) pc[p].init(px, py[p], frame);
    }

    // lidar: angles relative to the tile's first valid point, as in the forward kernel
    float ref_x = 0.f, ref_y = 0.f;
    if (tr == 0) { s_block_final = -1; s_ref_thread = 0xFFFFFFFFu; }
    __syncthreads();
    if (LIDAR) {
        if (inside[0]) atomicMin(&s_ref_thread, tr);
        __syncthreads();
        if (tr == s_ref_thread) { s_ref[0] = px; s_ref[1] = py[0]; }
        __syncthreads();
        if (s_ref_thread != 0xFFFFFFFFu) { ref_x = s_ref[0]; ref_y = s_ref[1]; }
        px = angle_difference(px, ref_x); // from here on px, py are relative
        py[0] = angle_difference(py[0], ref_y);
    }

    const int32_t *offs = a.tile_offsets + (size_t)cam * tiles_per_cam;
    const int32_t range_start = offs[tile_id];
    const int32_t range_end = (cam == a.C - 1 && tile_id == tiles_per_cam - 1)
                                  ? (int32_t)a.n_isects
                                  : offs[tile_id + 1];

    // The reference keeps, per channel, the colour accumulated behind the current Gaussian
    // (`buffer`) and forms v_alpha = sum_k (c_k T - buffer_k / (1 - alpha)) v_out_k.  Only the
    // product of the buffer with v_out is ever used, so one running number per pixel replaces
    // the CH buffers: with cv = sum_k c_k v_out_k, v_alpha = cv T - behind / (1 - alpha) and
    // behind += cv alpha T.
    float T_final[PPL], T[PPL], behind[PPL], v_out[PPL][CH], v_render_a[PPL], bg_dot[PPL];
    int32_t bin_final[PPL];
#pragma unroll
    for (int p = 0; p < PPL; ++p) {
        T_final[p] = inside[p] ? 1.0f - a.render_alphas[pix[p]] : 1.0f;
        T[p] = T_final[p];
        bin_final[p] = inside[p] ? a.last_ids[pix[p]] : -1;
        behind[p] = 0.f;
#pragma unroll
        for (int k = 0; k < CH; ++k)
            v_out[p][k] = (inside[p] && (uint32_t)k < a.n_ch)
                              ? a.v_render_colors[pix[p] * a.color_stride + a.ch_offset + k] : 0.f;
        v_render_a[p] = (inside[p] && a.first_pass) ? a.v_render_alphas[pix[p]] : 0.f;
        bg_dot[p] = 0.f; // sum_k background_k v_out_k
        if (a.backgrounds != nullptr) {
            const float *bg = a.backgrounds + (size_t)cam * a.color_stride + a.ch_offset;
#pragma unroll
            for (int k = 0; k < CH; ++k)
                if ((uint32_t)k < a.n_ch) bg_dot[p] += bg[k] * v_out[p][k];
        }
    }
    const float v_asum = (LIDAR && inside[0] && a.first_pass && a.compute_alpha_sum && a.v_alpha_sum) ? a.v_alpha_sum[pix[0]] : 0.f;
    const bool has_depth = LIDAR && a.depth_idx >= a.ch_offset && a.depth_idx < a.ch_offset + a.n_ch;
    const int depth_local = has_depth ? (int)(a.depth_idx - a.ch_offset) : -1;
    float v_out_depth = 0.f; // v_out of the depth channel, valid in the pass that owns it
#pragma unroll
    for (int k = 0; k < CH; ++k)
        if (k == depth_local) v_out_depth = v_out[0][k];

    // deepest entry any pixel of the tile consumed
    int32_t lane_final = bin_final[0];
#pragma unroll
    for (int p = 1; p < PPL; ++p) lane_final = max(lane_final, bin_final[p]);
    const int32_t wave_final = wave_max_i32(lane_final);
    if (lane == 0 && wave_final >= 0) atomicMax(&s_block_final, wave_final);
    __syncthreads();
    const int32_t list_end = min(range_end, s_block_final + 1); // exclusive
    if (list_end <= range_start) return;
    const uint32_t num_batches = (uint32_t)(list_end - range_start + batch - 1) / batch;

    // footprint of this wavefront over the lanes that consumed anything
    WaveCull cull;
    WavePointCull pcull;
    if (LIDAR) pcull.init(inside[0] && bin_final[0] >= range_start, px, py[0], roll[0], true);
    else cull.init(px, py[0], py[PPL - 1], roll[0], roll[PPL - 1], true);

    // what a lane reads for the Gaussian it stages
    struct Fetched {
        float2 xy, dc;
        float cn[3], v[3], opac, depth_col, col[CH];
    };
    auto id_of = [&](uint32_t b) -> int32_t { // Gaussian this lane stages in batch b, or -1
        const int32_t idx = list_end - 1 - (int32_t)(batch * b) - (int32_t)tr;
        return (b < num_batches && tr < batch && idx >= range_start) ? a.flatten_ids[idx] : -1;
    };
    auto fetch = [&](int32_t g) -> Fetched {
        Fetched f = {};
        if (g >= 0) {
            f.xy = reinterpret_cast<const float2 *>(a.means2d)[g];
            const float *cn = a.conics + (size_t)g * 3;
            f.cn[0] = cn[0]; f.cn[1] = cn[1]; f.cn[2] = cn[2];
            f.opac = a.opacities[g];
            const float *crow = a.colors + (size_t)g * a.feat_stride;
            const bool split = LIDAR && a.range_channel != nullptr;
            if (LIDAR) {
                const float *v = a.pix_vels + (size_t)g * 3;
                f.v[0] = v[0]; f.v[1] = v[1]; f.v[2] = v[2];
                f.dc = reinterpret_cast<const float2 *>(a.depth_comps)[g];
                f.depth_col = split ? a.range_channel[g] : crow[a.depth_idx];
            } else {
                const float2 v = reinterpret_cast<const float2 *>(a.pix_vels)[g];
                f.v[0] = v.x; f.v[1] = v.y;
            }
#pragma unroll
            for (int k = 0; k < CH; ++k) {
                const uint32_t c = a.ch_offset + k;
                float v = 0.f;
                if ((uint32_t)k < a.n_ch) v = split && c == a.depth_idx ? f.depth_col : crow[min(c, a.feat_stride - 1u)];
                if (!LIDAR && a.colors_from_cache && !(v == v)) v = 0.f;
                f.col[k] = v;
            }
        }
        return f;
    };
    // where slot `lane` of a Gaussian's accumulator goes: slot_base + id * slot_stride
    float *slot_base = nullptr;
    uint32_t slot_stride = 0;
    if (lane < CH) {
        if ((uint32_t)lane < a.n_ch) {
            const uint32_t c = a.ch_offset + lane;
            if (a.v_range != nullptr && c == a.depth_idx) { slot_base = a.v_range; slot_stride = 1; }
            else { slot_base = a.v_colors + c; slot_stride = a.feat_stride; }
        }
    } else if (lane < ACC) {
        const int geo = lane - CH;
        const uint32_t nv = LIDAR ? 3 : 2;
        if (geo < G_XY) { slot_base = a.v_conics + geo; slot_stride = 3; }
        else if (geo < G_VEL) { slot_base = a.v_means2d + (geo - G_XY); slot_stride = 2; }
        else if (geo < G_OPAC) { slot_base = a.v_pix_vels + (geo - G_VEL); slot_stride = nv; }
        else if (geo == G_OPAC) { slot_base = a.v_opacities; slot_stride = 1; }
        else if (geo >= G_ABS) { if (a.v_means2d_abs != nullptr) { slot_base = a.v_means2d_abs + (geo - G_ABS); slot_stride = 2; } }
        else if (geo == G_VELZ) { slot_base = a.v_pix_vels + 2; slot_stride = 3; }
        else if (geo < G_D0) { slot_base = a.v_depth_comps + (geo - G_DC); slot_stride = 2; }
    }

    for (uint32_t b = 0; b < num_batches; ++b) {
        __syncthreads(); // previous batch fully flushed
        const int32_t batch_end = list_end - 1 - (int32_t)(batch * b);
        const int32_t batch_size = min((int32_t)batch, batch_end + 1 - range_start);
        const int32_t g_now = id_of(b);
        const Fetched now = fetch(g_now);
        if (g_now >= 0) {
            float4 *rec = s_rec + (size_t)RECORD * tr;
            if (LIDAR) {
                rec[0] = make_float4(angle_difference(now.xy.x, ref_x), angle_difference(now.xy.y, ref_y), now.v[0], now.v[1]);
                rec[RECORD - 1] = make_float4(now.v[2], now.dc.x, now.dc.y, now.depth_col);
            } else {
                rec[0] = make_float4(now.xy.x, now.xy.y, now.v[0], now.v[1]);
                float4 pa, pb;
                pixel_polynomial(frame, now.xy, make_float2(now.v[0], now.v[1]), now.cn[0], now.cn[1], now.cn[2],
                                 now.opac, pa, pb);
                rec[2] = pa;
                // {cXY, cYY, the exponent above which sigma < 0 (+inf where that cannot be), -}
                rec[3] = make_float4(pb.x, pb.y, pb.z == pb.z ? INFINITY : pb.w, 0.f);
            }
            rec[1] = staged_exponent(now.cn[0], now.cn[1], now.cn[2], now.opac);
            s_aux[tr] = make_float2(__int_as_float(g_now), now.opac > 0.f ? 1.0f / now.opac : 0.f); // finite
#pragma unroll
            for (int k = 0; k < CH; ++k) s_col[tr * CH + k] = now.col[k];
        }
        for (uint32_t k = tr; k < (uint32_t)batch_size * ACC; k += block_size) s_acc[k] = 0.f;
        __syncthreads();

        // entry t of the batch sits at list position batch_end - t; this wavefront starts at
        // the deepest entry any of its lanes consumed
        const int32_t t0 = max(0, batch_end - wave_final);
        for (int32_t base = t0 & ~(SPLATAD_WAVE - 1); base < batch_size; base += SPLATAD_WAVE) {
            const int32_t tt = base + lane;
            bool keep = tt >= t0 && tt < batch_size, unfolded_ok = true;
            if (keep) {
                const float4 *rec = s_rec + (size_t)RECORD * tt;
                keep = LIDAR ? pcull.may_touch(rec[0], rec[1], unfolded_ok) : cull.may_touch(rec[0], rec[1]);
            }
            uint64_t todo = wave_ballot(keep);
            const uint64_t folded = wave_ballot(keep && !unfolded_ok);
            while (todo) {
                const int32_t bit = __ffsll((unsigned long long)todo) - 1;
                const int32_t t = base + bit;
                todo &= todo - 1;
                const float4 *rec = s_rec + (size_t)RECORD * t;
                const float4 xyv = rec[0];
                const float4 e = rec[1];
                // per pixel: offsets, alpha before the clamp, and the lanes that took this Gaussian
                // in the forward pass (scalar logic on lane masks)
                float dx[PPL], dy[PPL], au[PPL];
                uint64_t valid_bits[PPL], any_valid = 0;
#pragma unroll
                for (int p = 0; p < PPL; ++p) {
                    dx[p] = gaussian_offset(xyv.x, xyv.z, roll[p], px);
                    dy[p] = gaussian_offset(xyv.y, xyv.w, roll[p], py[p]);
                    if (LIDAR && ((folded >> bit) & 1ull)) { // uniform, rare
                        dx[p] = angle_difference(fmaf(roll[p], xyv.z, xyv.x), px);
                        dy[p] = angle_difference(fmaf(roll[p], xyv.w, xyv.y), py[p]);
                    }
                    bool sigma_ok;
                    if constexpr (LIDAR) {
                        const float power = gaussian_power(e, dx[p], dy[p]);
                        au[p] = __builtin_amdgcn_exp2f(e.w - power); // opacity * exp(-sigma)
                        sigma_ok = !(power < 0.f);
                    } else {
                        const float4 pb = rec[3];
                        const float ex = pixel_exponent(rec[2], pb.x, pb.y, pc[p]);
                        au[p] = __builtin_amdgcn_exp2f(ex);
                        sigma_ok = !(ex > pb.z);
                    }
                    valid_bits[p] = inside_bits[p] & wave_ballot(batch_end - t <= bin_final[p]) &
                                    wave_ballot(sigma_ok) & wave_ballot(!(fminf(0.999f, au[p]) < 1.f / 255.f));
                    any_valid |= valid_bits[p];
                }
                if (any_valid == 0) continue;

                // Branch-free from here on: a pixel that does not take this Gaussian runs the same
                // arithmetic with alpha = 0 and alpha-before-clamping = 0, which makes every
                // gradient term an exact zero (all other factors are finite) and leaves its
                // transmittance and colour buffer as they are.  The pixels of a lane add up in
                // the lane before the wavefront reduction.
                float v[NV];
#pragma unroll
                for (int k = 0; k < NV; ++k) v[k] = 0.f;
                float4 ext = make_float4(0.f, 0.f, 0.f, 0.f);
                if constexpr (LIDAR) ext = rec[RECORD - 1];
#pragma unroll
                for (int p = 0; p < PPL; ++p) {
                    const bool valid = wave_lanes(valid_bits[p]);
                    const float alpha_s = valid ? fminf(0.999f, au[p]) : 0.f;
                    const float ra = __builtin_amdgcn_rcpf(1.0f - alpha_s); // 1 ulp; exactly 1 for alpha = 0
                    T[p] *= ra; // transmittance in front of this Gaussian
                    const float fac = alpha_s * T[p];
                    // a clamped alpha passes no gradient on to the exponent or the opacity
                    const float au_g = (valid && au[p] <= 0.999f) ? au[p] : 0.f;
                    float cv = 0.f;
#pragma unroll
                    for (int k = 0; k < CH; ++k) {
                        v[k] += fac * v_out[p][k];
                        cv += s_col[t * CH + k] * v_out[p][k];
                    }
                    float extra = 0.f;
                    if constexpr (LIDAR) {
                        extra = ext.y * dx[p] + ext.z * dy[p] + ext.x * roll[p];
                        cv += extra * v_out_depth; // depth channel = colour + extra
                    }
                    float v_alpha = cv * T[p] - behind[p] * ra;
                    behind[p] += cv * fac;
                    v_alpha += T_final[p] * ra * v_render_a[p];
                    v_alpha += -T_final[p] * ra * bg_dot[p];
                    const float v_sigma = -au_g * v_alpha;
                    float s_all = v_sigma, v_sig2 = 0.f; // every term that multiplies the conic rows
                    float g_depth = 0.f;
                    if constexpr (LIDAR) {
                        // gradient of the depth channel value, under the same clamp rule
                        g_depth = au_g != 0.f ? fac * v_out_depth : 0.f;
                        v[CH + G_DC] += g_depth * dx[p];
                        v[CH + G_DC + 1] += g_depth * dy[p];
                        v[CH + G_VELZ] += g_depth * roll[p];
                        v[CH + G_D0] += g_depth;
                        if (a.compute_alpha_sum) { // uniform
                            const float au_s = (valid && ext.w < pz - a.threshold) ? au[p] : 0.f;
                            v_sig2 = -v_asum * au_s;
                            s_all += v_sig2;
                        }
                    }
                    const float sx = s_all * dx[p], sy = s_all * dy[p];
                    v[CH + G_CONIC] = fmaf(sx, dx[p], v[CH + G_CONIC]);
                    v[CH + G_CONIC + 1] = fmaf(sx, dy[p], v[CH + G_CONIC + 1]);
                    v[CH + G_CONIC + 2] = fmaf(sy, dy[p], v[CH + G_CONIC + 2]);
                    v[CH + G_XY] += sx;
                    v[CH + G_XY + 1] += sy;
                    v[CH + G_VEL] = fmaf(sx, roll[p], v[CH + G_VEL]);
                    v[CH + G_VEL + 1] = fmaf(sy, roll[p], v[CH + G_VEL + 1]);
                    v[CH + G_OPAC] += s_all;
                    if (ABS && a.v_means2d_abs != nullptr) { // (uniform) sums of absolute values, pixel by pixel
                        // conic row products a dx + b dy and b dx + c dy from the staged form
                        const float row_x = kLn2 * (2.f * e.x * dx[p] + e.y * dy[p]);
                        const float row_y = kLn2 * (e.y * dx[p] + 2.f * e.z * dy[p]);
                        float g_x = v_sigma * row_x, g_y = v_sigma * row_y;
                        if constexpr (LIDAR) { g_x += g_depth * ext.y; g_y += g_depth * ext.z; }
                        v[CH + G_ABS] += fabsf(g_x) + fabsf(v_sig2 * row_x);
                        v[CH + G_ABS + 1] += fabsf(g_y) + fabsf(v_sig2 * row_y);
                    }
                }
                // sum over the wavefront; the lane that ends up with slot s adds it in LDS
                wave_reduce_scatter<NA>(*reinterpret_cast<float(*)[NA]>(&v[0]), lane);
                const int slot = wave_reduce_slot<NA>(lane);
                if (slot < ACC && (lane & (64 / NA - 1)) == 0 && v[0] != 0.f)
                    atomicAdd(s_acc + (size_t)t * ACC + slot, v[0]);
                if constexpr (NB > 0) {
                    wave_reduce_scatter<NB>(*reinterpret_cast<float(*)[NB]>(&v[NA]), lane);
                    const int slot_b = NA + wave_reduce_slot<NB>(lane);
                    if (slot_b < ACC && (lane & (64 / NB - 1)) == 0 && v[NA] != 0.f)
                        atomicAdd(s_acc + (size_t)t * ACC + slot_b, v[NA]);
                }
            }
        }
        __syncthreads();

        // Flush the batch.  Global atomics are served per memory request, about one per clock and
        // L2 channel, so what counts is how many requests an instruction spreads over: with the
        // packed layout the slots of one Gaussian are neighbours in memory and in the wavefront
        // (lane = (Gaussian, slot)), and a Gaussian costs one or two requests instead of one per
        // value.
        // the geometry slots hold moments: the gradients are formed here, once per Gaussian of the
        // batch (a lane per Gaussian, the same straight-line code for all)
        for (uint32_t t = tr; t < (uint32_t)batch_size; t += block_size) {
            const float4 *rec = s_rec + (size_t)RECORD * t;
            gradients_from_moments<LIDAR>(s_acc + (size_t)t * ACC + CH, rec[1], s_aux[t].y,
                                          LIDAR ? rec[RECORD - 1] : make_float4(0.f, 0.f, 0.f, 0.f));
        }
        __syncthreads();
        if (a.packed != nullptr) {
            for (uint32_t idx = tr; idx < (uint32_t)batch_size * ACC; idx += block_size) {
                const uint32_t t = idx / ACC, slot = idx - t * ACC;
                const float val = s_acc[idx];
                if (val != 0.f)
                    atomicAdd(a.packed + (size_t)__float_as_int(s_aux[t].x) * a.packed_stride + slot, val);
            }
        } else {
            // lane = slot: a wavefront adds one Gaussian's values per instruction, so the channels
            // of a Gaussian (neighbours in v_colors) and the members of each geometry gradient
            // share memory requests
            for (uint32_t t = tr / SPLATAD_WAVE; t < (uint32_t)batch_size; t += block_size / SPLATAD_WAVE) {
                const float val = lane < ACC ? s_acc[t * ACC + lane] : 0.f;
                if (slot_base != nullptr && val != 0.f)
                    atomicAdd(slot_base + (size_t)__float_as_int(s_aux[t].x) * slot_stride, val);
            }
        }
    }
}

// Adds the packed gradients of one channel pass into the arrays of the interface: one thread
// per (Gaussian, slot), `width` colour slots (the first n_ch of them in use) followed by the
// geometry slots.  Every output element has exactly one writer.
template <bool LIDAR>
__global__ void __launch_bounds__(SPLATAD_THREADS)
unpack_gradients_kernel(uint64_t total, uint32_t stride, uint32_t width, BwdArgs a) {
    const uint64_t idx = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= total * stride) return;
    const uint64_t g = idx / stride;
    const uint32_t slot = (uint32_t)(idx - g * stride);
    constexpr uint32_t GEO = geo_count(LIDAR), G_ABS = geo_abs(LIDAR);
    if (slot >= width + GEO) return;
    const float val = a.packed[idx];
    if (val == 0.f) return;
    if (slot < width) {
        if (slot < a.n_ch) {
            const uint32_t c = a.ch_offset + slot;
            if (a.v_range != nullptr && c == a.depth_idx) a.v_range[g] += val;
            else a.v_colors[g * a.feat_stride + c] += val;
        }
        return;
    }
    const uint32_t geo = slot - width;
    constexpr uint32_t nv = LIDAR ? 3 : 2;
    if (geo < G_XY) a.v_conics[g * 3 + geo] += val;
    else if (geo < G_VEL) a.v_means2d[g * 2 + (geo - G_XY)] += val;
    else if (geo < G_OPAC) a.v_pix_vels[g * nv + (geo - G_VEL)] += val;
    else if (geo == G_OPAC) a.v_opacities[g] += val;
    else if (geo >= G_ABS) { if (a.v_means2d_abs != nullptr) a.v_means2d_abs[g * 2 + (geo - G_ABS)] += val; }
    else if (geo == G_VELZ) a.v_pix_vels[g * 3 + 2] += val;
    else if (geo < G_D0) a.v_depth_comps[g * 2 + (geo - G_DC)] += val;
}

__global__ void __launch_bounds__(SPLATAD_THREADS) fill_zero_f32x4_kernel(float4 *p, uint64_t n4) {
    const uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n4) p[i] = make_float4(0.f, 0.f, 0.f, 0.f);
}

constexpr int kWidths[] = {1, 2, 3, 4, 5, 8, 9, 16, 17, 32, 33};
constexpr int kMaxPass = 33;

static inline int pick_width(uint32_t n) {
    for (int w : kWidths)
        if ((uint32_t)w >= n) return w;
    return -1;
}

template <int CH, bool LIDAR, int PPL, bool ABS = true>
static int launch_bwd_as(BwdArgs a, dim3 grid, dim3 block, hipStream_t stream) {
    const size_t per_gaussian = ((LIDAR ? 48 : 64) + 8) + 4 * CH + 4 * (CH + geo_count(LIDAR, ABS));
    // Batches of the whole workgroup, unless that leaves fewer than four workgroups to a compute
    // unit (160 KB of LDS): a lidar sweep's 1024 tiles then run all at once instead of in two
    // rounds (with 33 channels: 104 Gaussians per batch, 0.39 ms instead of 0.51 ms with 128).
    // The two-pixel kernels' registers allow five wavefronts per SIMD, twenty per compute unit:
    // their batches leave room for the workgroups that makes (ten of 128 lanes: 104 Gaussians per
    // batch with four channels, 0.54 instead of 0.57 ms for the 1080p frame's backward pass).
    a.batch = block.x;
    const size_t wgs = PPL == 2 ? std::max<size_t>(4, 20 / ((block.x + SPLATAD_WAVE - 1) / SPLATAD_WAVE)) : 4;
    const size_t room = 160 * 1024 / wgs - 1024; // LDS is granted in blocks, and 16 bytes are static
    if (a.batch * per_gaussian > room) a.batch = (uint32_t)(room / per_gaussian) / 8 * 8;
    const size_t lds = a.batch * per_gaussian;
    if (lds > 64 * 1024)
        SPLATAD_CHECK_HIP(hipFuncSetAttribute((const void *)rasterize_bwd_kernel<CH, LIDAR, PPL, ABS>,
                                              hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
    hipLaunchKernelGGL((rasterize_bwd_kernel<CH, LIDAR, PPL, ABS>), grid, block, lds, stream, a);
    SPLATAD_LAUNCH_CHECK();
    return 0;
}

// Cameras with few channels and tiles of whole 8 x 16 wavefronts: two pixels per lane.
template <int CH, bool LIDAR>
static int launch_bwd(const BwdArgs &a, dim3 grid, dim3 block, hipStream_t stream) {
    if constexpr (!LIDAR && CH <= 5) {
        const uint32_t pixels = a.tile_w_px * a.tile_h_px;
        // (without the absolute gradients the two-pixel kernels sum 8 + 4 instead of 16 values per
        // Gaussian over the wavefront)
        if (a.tile_w_px % 8 == 0 && (pixels / 2) % SPLATAD_WAVE == 0 && block.x == pixels)
            return a.v_means2d_abs != nullptr ? launch_bwd_as<CH, LIDAR, 2, true>(a, grid, dim3(pixels / 2), stream)
                                              : launch_bwd_as<CH, LIDAR, 2, false>(a, grid, dim3(pixels / 2), stream);
    }
    return launch_bwd_as<CH, LIDAR, 1>(a, grid, block, stream);
}

template <bool LIDAR>
static int dispatch_bwd(int w, const BwdArgs &a, dim3 grid, dim3 block, hipStream_t s) {
    switch (w) {
    case 1: return launch_bwd<1, LIDAR>(a, grid, block, s);
    case 2: return launch_bwd<2, LIDAR>(a, grid, block, s);
    case 3: return launch_bwd<3, LIDAR>(a, grid, block, s);
    case 4: return launch_bwd<4, LIDAR>(a, grid, block, s);
    case 5: return launch_bwd<5, LIDAR>(a, grid, block, s);
    case 8: return launch_bwd<8, LIDAR>(a, grid, block, s);
    case 9: return launch_bwd<9, LIDAR>(a, grid, block, s);
    case 16: return launch_bwd<16, LIDAR>(a, grid, block, s);
    case 17: return launch_bwd<17, LIDAR>(a, grid, block, s);
    case 32: return launch_bwd<32, LIDAR>(a, grid, block, s);
    case 33: return launch_bwd<33, LIDAR>(a, grid, block, s);
    default: break;
    }
    splatad_set_error("rasterize backward: no kernel for %d channels per pass", w);
    return -1;
}

// Floats per Gaussian of the packed accumulation buffer: the widest pass plus the geometry
// slots, in whole 64-byte lines.
static uint32_t packed_stride(uint32_t channels, bool lidar) {
    const uint32_t pass = channels <= (uint32_t)kMaxPass ? channels : 32u;
    const uint32_t acc = (uint32_t)pick_width(pass) + (uint32_t)geo_count(lidar);
    return (acc + 15u) / 16u * 16u;
}

template <bool LIDAR>
static int run_passes(BwdArgs &a, uint32_t channels, dim3 grid, dim3 block, uint64_t total,
                      void *workspace, size_t workspace_bytes, hipStream_t stream) {
    const uint32_t pass = channels <= (uint32_t)kMaxPass ? channels : 32u;
    const uint32_t stride = packed_stride(channels, LIDAR);
    a.packed = nullptr;
    if (workspace != nullptr) {
        SPLATAD_REQUIRE(total > 0 && total < (1ull << 31), "rasterize backward: bad number of Gaussians");
        SPLATAD_REQUIRE(workspace_bytes >= total * stride * sizeof(float),
                        "rasterize backward: workspace of %zu bytes, %zu needed", workspace_bytes,
                        (size_t)(total * stride * sizeof(float)));
        SPLATAD_REQUIRE(((uintptr_t)workspace & 15) == 0, "rasterize backward: workspace is not 16-byte aligned");
        a.packed = reinterpret_cast<float *>(workspace);
        a.packed_stride = stride;
    }
    for (uint32_t off = 0; off < channels; off += pass) {
        a.ch_offset = off;
        a.n_ch = min(pass, channels - off);
        a.first_pass = off == 0;
        const int width = pick_width(a.n_ch);
        if (a.packed != nullptr) {
            const uint64_t n4 = total * stride / 4;
            hipLaunchKernelGGL(fill_zero_f32x4_kernel, dim3((uint32_t)((n4 + SPLATAD_THREADS - 1) / SPLATAD_THREADS)),
                               dim3(SPLATAD_THREADS), 0, stream, reinterpret_cast<float4 *>(a.packed), n4);
            SPLATAD_LAUNCH_CHECK();
        }
        int rc = dispatch_bwd<LIDAR>(width, a, grid, block, stream);
        if (rc) return rc;
        if (a.packed != nullptr) {
            const uint64_t n = total * stride;
            hipLaunchKernelGGL(unpack_gradients_kernel<LIDAR>, dim3((uint32_t)((n + SPLATAD_THREADS - 1) / SPLATAD_THREADS)),
                               dim3(SPLATAD_THREADS), 0, stream, total, stride, (uint32_t)width, a);
            SPLATAD_LAUNCH_CHECK();
        }
    }
    return 0;
}

} // namespace

extern "C" size_t splatad_rasterize_bwd_workspace_bytes(uint64_t total, uint32_t channels, int lidar) {
    return (size_t)(total * packed_stride(channels ? channels : 1, lidar != 0) * sizeof(float));
}

static int pixels_bwd(int colors_from_cache,
    uint32_t C, int64_t n_isects, uint32_t channels, const float *means2d, const float *conics,
    const float *colors, const float *opacities, const float *pix_vels, const float *rs_time,
    const float *backgrounds, uint32_t W, uint32_t H, uint32_t tile_size, uint32_t tile_w,
    uint32_t tile_h, const int32_t *tile_offsets, const int32_t *flatten_ids,
    const float *render_alphas, const int32_t *last_ids, const float *v_render_colors,
    const float *v_render_alphas, float *v_means2d_abs, float *v_means2d, float *v_conics,
    float *v_colors, float *v_depths, float *v_opacities, float *v_pix_vels, uint64_t total, void *workspace,
    size_t workspace_bytes, splatad_stream_t stream) {
    SPLATAD_REQUIRE(channels >= 1, "rasterize_to_pixels bwd: zero channels");
    SPLATAD_REQUIRE(tile_size >= 1 && tile_size * tile_size <= 256,
                    "rasterize_to_pixels bwd: tile_size %u is outside 1..16", tile_size);
    if (C == 0 || W == 0 || H == 0 || n_isects == 0) return 0;
    SPLATAD_REQUIRE((uint64_t)tile_w * tile_size >= W && (uint64_t)tile_h * tile_size >= H,
                    "rasterize_to_pixels bwd: tile grid does not cover the image");
    SPLATAD_REQUIRE(n_isects > 0 && n_isects < (1ll << 31), "rasterize_to_pixels bwd: bad n_isects");
    SPLATAD_REQUIRE(means2d && conics && colors && opacities && pix_vels && rs_time && tile_offsets &&
                        flatten_ids && render_alphas && last_ids && v_render_colors && v_render_alphas &&
                        v_means2d && v_conics && v_colors && v_opacities && v_pix_vels,
                    "rasterize_to_pixels bwd: null pointer argument");
    BwdArgs a = {};
    a.colors_from_cache = colors_from_cache;
    a.C = C; a.n_isects = n_isects; a.color_stride = channels; a.feat_stride = channels;
    a.means2d = means2d; a.conics = conics; a.colors = colors; a.opacities = opacities;
    a.pix_vels = pix_vels; a.rs_time = rs_time; a.backgrounds = backgrounds;
    a.W = W; a.H = H; a.tile_w_px = tile_size; a.tile_h_px = tile_size; a.grid_w = tile_w; a.grid_h = tile_h;
    a.tile_offsets = tile_offsets; a.flatten_ids = flatten_ids;
    a.render_alphas = render_alphas; a.last_ids = last_ids;
    a.v_render_colors = v_render_colors; a.v_render_alphas = v_render_alphas;
    a.v_means2d_abs = v_means2d_abs; a.v_means2d = v_means2d; a.v_conics = v_conics;
    a.v_colors = v_colors; a.v_opacities = v_opacities; a.v_pix_vels = v_pix_vels;
    // the last channel's gradient in an array of its own (the depth channel of a colour cache row)
    a.v_range = v_depths; a.depth_idx = channels - 1;
    return run_passes<false>(a, channels, dim3(C * tile_w * tile_h),
                             dim3((tile_size * tile_size + 63) / 64 * 64), total, workspace,
                             workspace_bytes, (hipStream_t)stream);
}

extern "C" int splatad_rasterize_to_pixels_bwd(
    uint32_t C, int64_t n_isects, uint32_t channels, const float *means2d, const float *conics,
    const float *colors, const float *opacities, const float *pix_vels, const float *rs_time,
    const float *backgrounds, uint32_t W, uint32_t H, uint32_t tile_size, uint32_t tile_w,
    uint32_t tile_h, const int32_t *tile_offsets, const int32_t *flatten_ids,
    const float *render_alphas, const int32_t *last_ids, const float *v_render_colors,
    const float *v_render_alphas, float *v_means2d_abs, float *v_means2d, float *v_conics,
    float *v_colors, float *v_opacities, float *v_pix_vels, uint64_t total, void *workspace,
    size_t workspace_bytes, splatad_stream_t stream) {
    return pixels_bwd(0, C, n_isects, channels, means2d, conics, colors, opacities, pix_vels, rs_time,
                      backgrounds, W, H, tile_size, tile_w, tile_h, tile_offsets, flatten_ids,
                      render_alphas, last_ids, v_render_colors, v_render_alphas, v_means2d_abs, v_means2d,
                      v_conics, v_colors, nullptr, v_opacities, v_pix_vels, total, workspace, workspace_bytes,
                      stream);
}

extern "C" int splatad_rasterize_to_pixels_bwd_sh(
    uint32_t C, int64_t n_isects, uint32_t channels, const float *means2d, const float *conics,
    const float *colors, const float *opacities, const float *pix_vels, const float *rs_time,
    const float *backgrounds, uint32_t W, uint32_t H, uint32_t tile_size, uint32_t tile_w,
    uint32_t tile_h, const int32_t *tile_offsets, const int32_t *flatten_ids,
    const float *render_alphas, const int32_t *last_ids, const float *v_render_colors,
    const float *v_render_alphas, float *v_means2d_abs, float *v_means2d, float *v_conics,
    float *v_colors, float *v_depths, float *v_opacities, float *v_pix_vels, uint64_t total, void *workspace,
    size_t workspace_bytes, splatad_stream_t stream) {
    SPLATAD_REQUIRE(v_depths == nullptr || channels == 4,
                    "rasterize_to_pixels bwd: v_depths goes with the four channels of a colour cache row");
    return pixels_bwd(1, C, n_isects, channels, means2d, conics, colors, opacities, pix_vels, rs_time,
                      backgrounds, W, H, tile_size, tile_w, tile_h, tile_offsets, flatten_ids,
                      render_alphas, last_ids, v_render_colors, v_render_alphas, v_means2d_abs, v_means2d,
                      v_conics, v_colors, v_depths, v_opacities, v_pix_vels, total, workspace, workspace_bytes,
                      stream);
}

extern "C" int splatad_rasterize_to_points_bwd(
    uint32_t C, int64_t n_isects, uint32_t channels, const float *means2d, const float *conics,
    const float *colors, const float *range_channel, const float *opacities, const float *pix_vels,
    const float *depth_comps, const float *backgrounds, const float *raster_pts, uint32_t W,
    uint32_t H, uint32_t tile_width, uint32_t tile_height, uint32_t grid_w, uint32_t grid_h,
    int compute_alpha_sum, float threshold, const int32_t *tile_offsets,
    const int32_t *flatten_ids, uint32_t depth_idx, const float *render_alphas,
    const int32_t *last_ids, const float *v_render_colors, const float *v_render_alphas,
    const float *v_alpha_sum, float *v_means2d_abs, float *v_means2d, float *v_conics,
    float *v_colors, float *v_range, float *v_opacities, float *v_pix_vels, float *v_depth_comps,
    uint64_t total,
    void *workspace, size_t workspace_bytes, splatad_stream_t stream) {
    SPLATAD_REQUIRE(channels >= 1, "rasterize_to_points bwd: zero channels");
    SPLATAD_REQUIRE(depth_idx < channels, "rasterize_to_points bwd: depth channel %u of %u", depth_idx, channels);
    SPLATAD_REQUIRE((range_channel == nullptr) == (v_range == nullptr),
                    "rasterize_to_points bwd: range_channel and v_range go together");
    SPLATAD_REQUIRE(range_channel == nullptr || (depth_idx + 1 == channels && channels >= 2),
                    "rasterize_to_points bwd: a separate range channel must be the last of at least two");
    SPLATAD_REQUIRE(tile_width >= 1 && tile_height >= 1 && tile_width * tile_height <= 256,
                    "rasterize_to_points bwd: tile %ux%u exceeds 256 points", tile_width, tile_height);
    if (C == 0 || W == 0 || H == 0 || n_isects == 0) return 0;
    SPLATAD_REQUIRE((uint64_t)grid_w * tile_width >= W && (uint64_t)grid_h * tile_height >= H,
                    "rasterize_to_points bwd: tile grid does not cover the point image");
    SPLATAD_REQUIRE(n_isects > 0 && n_isects < (1ll << 31), "rasterize_to_points bwd: bad n_isects");
    SPLATAD_REQUIRE(means2d && conics && colors && opacities && pix_vels && depth_comps && raster_pts &&
                        tile_offsets && flatten_ids && render_alphas && last_ids && v_render_colors &&
                        v_render_alphas && v_means2d && v_conics && v_colors && v_opacities &&
                        v_pix_vels && v_depth_comps,
                    "rasterize_to_points bwd: null pointer argument");
    BwdArgs a = {};
    a.C = C; a.n_isects = n_isects; a.color_stride = channels;
    a.feat_stride = range_channel ? channels - 1 : channels;
    a.range_channel = range_channel; a.v_range = v_range;
    a.means2d = means2d; a.conics = conics; a.colors = colors; a.opacities = opacities;
    a.pix_vels = pix_vels; a.depth_comps = depth_comps; a.backgrounds = backgrounds;
    a.raster_pts = raster_pts; a.W = W; a.H = H; a.tile_w_px = tile_width; a.tile_h_px = tile_height;
    a.grid_w = grid_w; a.grid_h = grid_h; a.compute_alpha_sum = compute_alpha_sum;
    a.threshold = threshold; a.tile_offsets = tile_offsets; a.flatten_ids = flatten_ids;
    a.depth_idx = depth_idx; a.render_alphas = render_alphas; a.last_ids = last_ids;
    a.v_render_colors = v_render_colors; a.v_render_alphas = v_render_alphas; a.v_alpha_sum = v_alpha_sum;
    a.v_means2d_abs = v_means2d_abs; a.v_means2d = v_means2d; a.v_conics = v_conics;
    a.v_colors = v_colors; a.v_opacities = v_opacities; a.v_pix_vels = v_pix_vels;
    a.v_depth_comps = v_depth_comps;
    return run_passes<true>(a, channels, dim3(C * grid_w * grid_h),
                            dim3((tile_width * tile_height + 63) / 64 * 64), total, workspace,
                            workspace_bytes, (hipStream_t)stream);
}
