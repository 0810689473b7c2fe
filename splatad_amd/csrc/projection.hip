// Forward projection of 3D Gaussians to pinhole image space and to lidar spherical
// (azimuth, elevation, range) space, with rolling-shutter velocities, for gfx950.
//
// One lane per (sensor, Gaussian).  The covariance never leaves factored form when it
// comes from (quat, scale): with M = R_q diag(s) and W = R_cw M, the projected
// covariance is (J W)(J W)^T, which is symmetric positive semi-definite by
// construction and needs fewer multiplies than two full 3x3 sandwiches.
//
// Semantics follow gsplat/cuda/csrc/projection.cu:605-751 (camera) and :2268-2417
// (lidar) of the reference, except that rows of culled Gaussians are written as zeros
// instead of being left uninitialised.
#include "common.h"
#include "host_word.h"
#include "scan.h"
#include "tile_rect.h"

#define RAD_TO_DEG 57.2957795131f

namespace {

struct SensorPose {
    Mat3 R;     // world -> sensor rotation
    float t[3]; // world -> sensor translation
};

__device__ __forceinline__ SensorPose load_pose(const float *__restrict__ vm) {
    SensorPose p;
    p.R.m[0] = vm[0]; p.R.m[1] = vm[1]; p.R.m[2] = vm[2];  p.t[0] = vm[3];
    p.R.m[3] = vm[4]; p.R.m[4] = vm[5]; p.R.m[5] = vm[6];  p.t[1] = vm[7];
    p.R.m[6] = vm[8]; p.R.m[7] = vm[9]; p.R.m[8] = vm[10]; p.t[2] = vm[11];
    return p;
}

__device__ __forceinline__ void to_sensor(const SensorPose &p, const float *__restrict__ m,
                                          float pc[3]) {
    const float x = m[0], y = m[1], z = m[2];
#pragma unroll
    for (int i = 0; i < 3; ++i) pc[i] = p.R.m[i * 3] * x + p.R.m[i * 3 + 1] * y + p.R.m[i * 3 + 2] * z + p.t[i];
}

// Sensor-frame "square root" W of the covariance (Sigma_c = W W^T) from (quat, scale), or
// the full sensor-frame covariance from the 6-vector upper triangle.
struct SensorCov {
    Mat3 a;
    bool factored; // true: a = W with Sigma_c = W W^T; false: a = Sigma_c
};

__device__ __forceinline__ SensorCov load_sensor_cov(uint32_t gid, const SensorPose &p,
                                                     const float *__restrict__ covars,
                                                     const float *__restrict__ quats,
                                                     const float *__restrict__ scales) {
    SensorCov sc;
    if (covars != nullptr) {
        const float *c = covars + (size_t)gid * 6;
        Mat3 S;
        S.m[0] = c[0]; S.m[1] = c[1]; S.m[2] = c[2];
        S.m[3] = c[1]; S.m[4] = c[3]; S.m[5] = c[4];
        S.m[6] = c[2]; S.m[7] = c[4]; S.m[8] = c[5];
        sc.a = mat3_mul_bt(mat3_mul(p.R, S), p.R);
        sc.factored = false;
    } else {
        const float4 q = *reinterpret_cast<const float4 *>(quats + (size_t)gid * 4);
        const float *s = scales + (size_t)gid * 3;
        Mat3 Rq = quat_to_rotmat(q.x, q.y, q.z, q.w);
        const float s0 = s[0], s1 = s[1], s2 = s[2];
#pragma unroll
        for (int i = 0; i < 3; ++i) {
            Rq.m[i * 3] *= s0; Rq.m[i * 3 + 1] *= s1; Rq.m[i * 3 + 2] *= s2;
        }
        sc.a = mat3_mul(p.R, Rq);
        sc.factored = true;
    }
    return sc;
}

// rows(J)[r] . Sigma_c . rows(J)[s] for a Jacobian with NR rows of 3.
template <int NR>
__device__ __forceinline__ void project_cov(const SensorCov &sc, const float *J, float *out /*NR*NR*/) {
    float T[NR * 3];
    if (sc.factored) {
        // T = J W ; out = T T^T
#pragma unroll
        for (int r = 0; r < NR; ++r)
#pragma unroll
            for (int j = 0; j < 3; ++j)
                T[r * 3 + j] = J[r * 3] * sc.a.m[j] + J[r * 3 + 1] * sc.a.m[3 + j] + J[r * 3 + 2] * sc.a.m[6 + j];
#pragma unroll
        for (int r = 0; r < NR; ++r)
#pragma unroll
            for (int s = 0; s < NR; ++s)
                out[r * NR + s] = T[r * 3] * T[s * 3] + T[r * 3 + 1] * T[s * 3 + 1] + T[r * 3 + 2] * T[s * 3 + 2];
    } else {
        // T = J Sigma ; out = T J^T
#pragma unroll
        for (int r = 0; r < NR; ++r)
#pragma unroll
            for (int j = 0; j < 3; ++j)
                T[r * 3 + j] = J[r * 3] * sc.a.m[j] + J[r * 3 + 1] * sc.a.m[3 + j] + J[r * 3 + 2] * sc.a.m[6 + j];
#pragma unroll
        for (int r = 0; r < NR; ++r)
#pragma unroll
            for (int s = 0; s < NR; ++s)
                out[r * NR + s] = T[r * 3] * J[s * 3] + T[r * 3 + 1] * J[s * 3 + 1] + T[r * 3 + 2] * J[s * 3 + 2];
    }
}

// Relative velocity of the scene point seen from the moving sensor:
// v_lin + omega x p - R v_gaussian (helpers.cuh:114-115 of the reference).
__device__ __forceinline__ void relative_velocity(const SensorPose &p, const float pc[3],
                                                  const float *__restrict__ lin,
                                                  const float *__restrict__ ang,
                                                  const float *__restrict__ vel_w, float tv[3]) {
    const float ax = ang[0], ay = ang[1], az = ang[2];
    tv[0] = lin[0] + (ay * pc[2] - az * pc[1]);
    tv[1] = lin[1] + (az * pc[0] - ax * pc[2]);
    tv[2] = lin[2] + (ax * pc[1] - ay * pc[0]);
    if (vel_w != nullptr) {
        const float vx = vel_w[0], vy = vel_w[1], vz = vel_w[2];
#pragma unroll
        for (int i = 0; i < 3; ++i) tv[i] -= p.R.m[i * 3] * vx + p.R.m[i * 3 + 1] * vy + p.R.m[i * 3 + 2] * vz;
    }
}

// COUNT: every workgroup also writes how many of its rows are kept (radii.x > 0) and how many
// tiles of the camera's grid those meet: the counts of the packed layout and of its tile
// intersection, gathered while the rows are in registers; and every row the number of kept
// rows before it in its workgroup (kept_before), which with the exclusive prefix of the
// workgroups' counts is the row's place among the kept rows: no scan pass over the rows.
template <bool COUNT>
__global__ void __launch_bounds__(SPLATAD_THREADS)
projection_fwd_kernel(uint32_t C, uint32_t N, const float *__restrict__ means,
                      const float *__restrict__ covars, const float *__restrict__ quats,
                      const float *__restrict__ scales, const float *__restrict__ velocities,
                      const float *__restrict__ viewmats, const float *__restrict__ Ks,
                      uint32_t W, uint32_t H, const float *__restrict__ lin_vel,
                      const float *__restrict__ ang_vel, const float *__restrict__ rs_time,
                      float eps2d, float near_plane, float far_plane, float radius_clip,
                      int32_t *__restrict__ radii, float *__restrict__ means2d,
                      float *__restrict__ depths, float *__restrict__ conics,
                      float *__restrict__ compensations, float *__restrict__ pix_vels,
                      uint32_t tile_size, uint32_t tile_w, uint32_t tile_h,
                      int64_t *__restrict__ kept_sums, int64_t *__restrict__ tile_sums,
                      int32_t *__restrict__ kept_before) {
    const uint64_t idx = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const bool live = idx < (uint64_t)C * N;
    if (!COUNT && !live) return;
    // (a lane beyond the last row works on row 0 and stores nothing: it is needed for the sums)
    const uint32_t cid = live ? (uint32_t)(idx / N) : 0u, gid = live ? (uint32_t)(idx % N) : 0u;

    int2 o_radii = make_int2(0, 0);
    float2 o_mean = make_float2(0.f, 0.f), o_vel = make_float2(0.f, 0.f);
    float o_depth = 0.f, o_comp = 0.f, o_c0 = 0.f, o_c1 = 0.f, o_c2 = 0.f;

    const SensorPose pose = load_pose(viewmats + cid * 16);
    float pc[3];
    to_sensor(pose, means + (size_t)gid * 3, pc);
    if (!(pc[2] < near_plane || pc[2] > far_plane)) {
        const float *K = Ks + cid * 9;
        const float fx = K[0], fy = K[4], cx = K[2], cy = K[5];
        const float x = pc[0], y = pc[1], z = pc[2];
        const float tan_fovx = 0.5f * (float)W / fx, tan_fovy = 0.5f * (float)H / fy;
        const float lim_x_pos = ((float)W - cx) / fx + 0.3f * tan_fovx;
        const float lim_x_neg = cx / fx + 0.3f * tan_fovx;
        const float lim_y_pos = ((float)H - cy) / fy + 0.3f * tan_fovy;
        const float lim_y_neg = cy / fy + 0.3f * tan_fovy;
        const float rz = 1.f / z, rz2 = rz * rz;
        const float tx = z * fminf(lim_x_pos, fmaxf(-lim_x_neg, x * rz));
        const float ty = z * fminf(lim_y_pos, fmaxf(-lim_y_neg, y * rz));
        float J[6] = {fx * rz, 0.f, -fx * tx * rz2, 0.f, fy * rz, -fy * ty * rz2};

        const SensorCov sc = load_sensor_cov(gid, pose, covars, quats, scales);
        float c2[4];
        project_cov<2>(sc, J, c2);
        float sxx = c2[0], sxy = c2[1], syy = c2[3];
        const float mx = fx * x * rz + cx, my = fy * y * rz + cy;

        const float det_orig = sxx * syy - sxy * sxy;
        sxx += eps2d;
        syy += eps2d;
        const float det = sxx * syy - sxy * sxy;
        if (det > 0.f) {
            float ext_x = 3.f * sqrtf(sxx), ext_y = 3.f * sqrtf(syy);
            if (!(ext_x <= radius_clip && ext_y <= radius_clip)) {
                float pvx = 0.f, pvy = 0.f;
                const float rs = rs_time[cid];
                if (rs > 0.f) {
                    float tv[3];
                    relative_velocity(pose, pc, lin_vel + cid * 3, ang_vel + cid * 3,
                                      velocities ? velocities + (size_t)gid * 3 : nullptr, tv);
                    pvx = -(J[0] * tv[0] + J[2] * tv[2]);
                    pvy = -(J[4] * tv[1] + J[5] * tv[2]);
                    ext_x += fabsf(pvx) * 0.5f * rs;
                    ext_y += fabsf(pvy) * 0.5f * rs;
                }
                if (!(mx + ext_x <= 0.f || mx - ext_x >= (float)W || my + ext_y <= 0.f ||
                      my - ext_y >= (float)H)) {
                    const float inv_det = 1.f / det;
                    o_radii = make_int2((int32_t)ext_x, (int32_t)ext_y);
                    o_mean = make_float2(mx, my);
                    o_depth = z;
                    o_c0 = syy * inv_det; o_c1 = -sxy * inv_det; o_c2 = sxx * inv_det;
                    o_comp = sqrtf(fmaxf(0.f, det_orig / det));
                    o_vel = make_float2(pvx, pvy);
                }
            }
        }
    }
    if (live) {
        reinterpret_cast<int2 *>(radii)[idx] = o_radii;
        reinterpret_cast<float2 *>(means2d)[idx] = o_mean;
        depths[idx] = o_depth;
        conics[idx * 3] = o_c0; conics[idx * 3 + 1] = o_c1; conics[idx * 3 + 2] = o_c2;
        if (compensations != nullptr) compensations[idx] = o_comp;
        reinterpret_cast<float2 *>(pix_vels)[idx] = o_vel;
    }
    if (COUNT) {
        __shared__ int64_t s_sums[2 * (SPLATAD_THREADS / SPLATAD_WAVE)];
        int64_t kept = 0, tiles = 0;
        const bool keep = live && o_radii.x > 0;
        if (keep) {
            int32_t x0, y0, x1, y1;
            splatad_camera_tile_rect(tile_size, tile_w, tile_h, o_mean, o_radii, x0, y0, x1, y1);
            kept = 1;
            tiles = (int64_t)max(y1 - y0, 0) * max(x1 - x0, 0);
        }
        const uint64_t keepers = wave_ballot(keep);
        const uint32_t before_in_wave =
            __builtin_amdgcn_mbcnt_hi((uint32_t)(keepers >> 32), __builtin_amdgcn_mbcnt_lo((uint32_t)keepers, 0u));
#pragma unroll
        for (int off = SPLATAD_WAVE / 2; off > 0; off >>= 1) {
            kept += __shfl_xor(kept, off, SPLATAD_WAVE);
            tiles += __shfl_xor(tiles, off, SPLATAD_WAVE);
        }
        const uint32_t wave = threadIdx.x / SPLATAD_WAVE;
        if ((threadIdx.x & (SPLATAD_WAVE - 1)) == 0) { s_sums[2 * wave] = kept; s_sums[2 * wave + 1] = tiles; }
        __syncthreads();
        if (live) {
            uint32_t before = before_in_wave;
            for (uint32_t w = 0; w < wave; ++w) before += (uint32_t)s_sums[2 * w];
            kept_before[idx] = (int32_t)before;
        }
        if (threadIdx.x == 0) {
            kept = tiles = 0;
            for (uint32_t w = 0; w < SPLATAD_THREADS / SPLATAD_WAVE; ++w) { kept += s_sums[2 * w]; tiles += s_sums[2 * w + 1]; }
            kept_sums[blockIdx.x] = kept;
            tile_sums[blockIdx.x] = tiles;
        }
    }
}

__global__ void __launch_bounds__(SPLATAD_THREADS)
lidar_projection_fwd_kernel(uint32_t C, uint32_t N, const float *__restrict__ means,
                            const float *__restrict__ covars, const float *__restrict__ quats,
                            const float *__restrict__ scales, const float *__restrict__ velocities,
                            const float *__restrict__ viewmats, float min_elev, float max_elev,
                            float min_azim, float max_azim, const float *__restrict__ lin_vel,
                            const float *__restrict__ ang_vel, const float *__restrict__ rs_time,
                            float eps2d, float near_plane, float far_plane, float radius_clip,
                            float *__restrict__ radii, float *__restrict__ means2d,
                            float *__restrict__ depths, float *__restrict__ conics,
                            float *__restrict__ compensations, float *__restrict__ pix_vels,
                            float *__restrict__ depth_comps) {
    const uint64_t idx = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= (uint64_t)C * N) return;
    const uint32_t cid = (uint32_t)(idx / N), gid = (uint32_t)(idx % N);

    float2 o_radii = make_float2(0.f, 0.f), o_mean = make_float2(0.f, 0.f), o_dc = make_float2(0.f, 0.f);
    float o_depth = 0.f, o_comp = 0.f, o_c0 = 0.f, o_c1 = 0.f, o_c2 = 0.f;
    float o_v0 = 0.f, o_v1 = 0.f, o_v2 = 0.f;

    const SensorPose pose = load_pose(viewmats + cid * 16);
    float pc[3];
    to_sensor(pose, means + (size_t)gid * 3, pc);
    const float x = pc[0], y = pc[1], z = pc[2];
    const float rho2 = x * x + y * y;
    const float r2 = rho2 + z * z;
    const float dist = sqrtf(r2);
    if (!(dist < near_plane || dist > far_plane)) {
        // rows: d(azimuth deg), d(elevation deg), d(range) with respect to (x, y, z)
        const float rinv = 1.f / dist;
        const float rho = sqrtf(rho2);
        const float k_az = RAD_TO_DEG / rho2;
        const float k_el = RAD_TO_DEG / (r2 * rho);
        float J[9] = {-y * k_az, x * k_az, 0.f,
                      -x * z * k_el, -y * z * k_el, rho2 * k_el,
                      x * rinv, y * rinv, z * rinv};
        const SensorCov sc = load_sensor_cov(gid, pose, covars, quats, scales);
        float cs[9];
        project_cov<3>(sc, J, cs);
        float saa = cs[0], sae = cs[1], see = cs[4];
        const float mx = atan2f(y, x) * RAD_TO_DEG, my = asinf(z * rinv) * RAD_TO_DEG;
        // range/angle coupling: Lambda[2,:2] / Lambda[2,2] of the eps-augmented covariance
        const float a1 = saa + eps2d, a2 = sae, b1 = cs[3], b2 = see + eps2d, c1 = cs[6], c2 = cs[7];
        const float invD = 1.f / (a1 * b2 - a2 * b1);
        const float dc0 = (b1 * c2 - b2 * c1) * invD, dc1 = (a2 * c1 - a1 * c2) * invD;

        const float det_orig = saa * see - sae * sae;
        saa += eps2d;
        see += eps2d;
        const float det = saa * see - sae * sae;
        if (det > 0.f) {
            float ext_az = 3.f * sqrtf(fmaxf(0.f, saa)), ext_el = 3.f * sqrtf(fmaxf(0.f, see));
            if (!(ext_az <= radius_clip && ext_el <= radius_clip)) {
                float pv0 = 0.f, pv1 = 0.f, pv2 = 0.f;
                const float rs = rs_time[cid];
                if (rs > 0.f) {
                    float tv[3];
                    relative_velocity(pose, pc, lin_vel + cid * 3, ang_vel + cid * 3,
                                      velocities ? velocities + (size_t)gid * 3 : nullptr, tv);
                    pv0 = -(J[0] * tv[0] + J[1] * tv[1]);
                    pv1 = -(J[3] * tv[0] + J[4] * tv[1] + J[5] * tv[2]);
                    pv2 = -(J[6] * tv[0] + J[7] * tv[1] + J[8] * tv[2]);
                    ext_az += fabsf(pv0) * 0.5f * rs;
                    ext_el += fabsf(pv1) * 0.5f * rs;
                }
                if (!(my + ext_el <= min_elev || my - ext_el >= max_elev ||
                      mx + ext_az <= min_azim || mx - ext_az >= max_azim)) {
                    const float inv_det = 1.f / det;
                    o_radii = make_float2(ext_az, ext_el);
                    o_mean = make_float2(mx, my);
                    o_depth = dist;
                    o_c0 = see * inv_det; o_c1 = -sae * inv_det; o_c2 = saa * inv_det;
                    o_comp = sqrtf(fmaxf(0.f, det_orig / det));
                    o_v0 = pv0; o_v1 = pv1; o_v2 = pv2;
                    o_dc = make_float2(dc0, dc1);
                }
            }
        }
    }
    reinterpret_cast<float2 *>(radii)[idx] = o_radii;
    reinterpret_cast<float2 *>(means2d)[idx] = o_mean;
    depths[idx] = o_depth;
    conics[idx * 3] = o_c0; conics[idx * 3 + 1] = o_c1; conics[idx * 3 + 2] = o_c2;
    if (compensations != nullptr) compensations[idx] = o_comp;
    pix_vels[idx * 3] = o_v0; pix_vels[idx * 3 + 1] = o_v1; pix_vels[idx * 3 + 2] = o_v2;
    reinterpret_cast<float2 *>(depth_comps)[idx] = o_dc;
}

// ---- packed (COO) variant: compaction of the dense projection ----------------

struct PackedWorkspace {
    int32_t *radii;   // [T, 2]
    float *means2d;   // [T, 2]
    float *depths;    // [T]
    float *conics;    // [T, 3]
    float *comps;     // [T]
    float *pix_vels;  // [T, 2]
    int32_t *pos;     // [T] kept rows before the row: in all, or in its projection workgroup, with
    int32_t *offsets; // [T / SPLATAD_THREADS + 1] the kept rows before the workgroup (zeros in the first case)
    int64_t *total;   // [1]
    int64_t *block_sums;
    int64_t *tile_sums; // tiles met by the kept rows of a scan block or projection workgroup (optional count)
    int32_t *tiles;     // [T] tiles per dense row (intersection started by the counting call)
};

static PackedWorkspace carve_packed(void *ws, uint64_t T) {
    char *p = (char *)ws;
    PackedWorkspace w;
    w.total = (int64_t *)p;       p += 256;
    w.radii = (int32_t *)p;       p += splatad_align256(T * 8);
    w.means2d = (float *)p;       p += splatad_align256(T * 8);
    w.depths = (float *)p;        p += splatad_align256(T * 4);
    w.conics = (float *)p;        p += splatad_align256(T * 12);
    w.comps = (float *)p;         p += splatad_align256(T * 4);
    w.pix_vels = (float *)p;      p += splatad_align256(T * 8);
    w.pos = (int32_t *)p;         p += splatad_align256(T * 4);
    // (room for the counts of every projection workgroup, SCAN_ITEMS per scan block)
    w.block_sums = (int64_t *)p;  p += SCAN_ITEMS * scan_workspace_bytes((int64_t)T);
    w.tile_sums = (int64_t *)p;   p += SCAN_ITEMS * scan_workspace_bytes((int64_t)T);
    w.offsets = (int32_t *)p;     p += splatad_align256((T / SPLATAD_THREADS + 1) * 4);
    w.tiles = (int32_t *)p;
    return w;
}

// One workgroup: publishes the number of kept rows (low 32 bits) and of their tile
// intersections (high 32 bits, saturated at 2^31 - 1, which the caller refuses) in one word.
// The kept rows are *total when that is given, the sum of kept_sums otherwise.
// offsets (with kept_sums): receives the exclusive prefix of kept_sums, the kept rows before
// each workgroup of the projection.
__global__ void __launch_bounds__(SPLATAD_THREADS)
packed_publish_kernel(const int64_t *__restrict__ total, const int64_t *__restrict__ kept_sums,
                      const int64_t *__restrict__ tile_sums, int64_t n_blocks,
                      unsigned long long *__restrict__ word, int32_t *__restrict__ offsets) {
    // a lane takes a run of consecutive blocks, so that its prefix is that of its first block
    const int64_t per = (n_blocks + SPLATAD_THREADS - 1) / SPLATAD_THREADS;
    const int64_t b0 = min(n_blocks, (int64_t)threadIdx.x * per), b1 = min(n_blocks, b0 + per);
    int64_t part = 0, part_kept = 0;
    for (int64_t b = b0; b < b1; ++b) {
        part += tile_sums[b];
        if (total == nullptr) part_kept += kept_sums[b];
    }
    int64_t tiles, kept;
    block_exclusive_scan(part, &tiles);
    int64_t before = block_exclusive_scan(part_kept, &kept);
    if (offsets != nullptr)
        for (int64_t b = b0; b < b1; ++b) {
            offsets[b] = (int32_t)before;
            before += kept_sums[b];
        }
    if (threadIdx.x == 0) {
        if (total != nullptr) kept = *total;
        const unsigned long long hi = tiles > 0x7FFFFFFFll ? 0x7FFFFFFFull : (unsigned long long)tiles;
        __hip_atomic_store(word, (hi << 32) | (unsigned long long)(uint32_t)kept, __ATOMIC_RELAXED,
                           __HIP_MEMORY_SCOPE_SYSTEM);
    }
}

__global__ void __launch_bounds__(SPLATAD_THREADS)
packed_compact_kernel(uint32_t C, uint32_t N, int64_t nnz, const int32_t *__restrict__ w_radii,
                      const float *__restrict__ w_means2d, const float *__restrict__ w_depths,
                      const float *__restrict__ w_conics, const float *__restrict__ w_comps,
                      const float *__restrict__ w_pix_vels, const int32_t *__restrict__ pos,
                      const int32_t *__restrict__ offsets, int32_t *__restrict__ indptr, int64_t *__restrict__ camera_ids,
                      int64_t *__restrict__ gaussian_ids, int32_t *__restrict__ radii,
                      float *__restrict__ means2d, float *__restrict__ depths,
                      float *__restrict__ conics, float *__restrict__ comps,
                      float *__restrict__ pix_vels, const float *__restrict__ opacities,
                      float *__restrict__ row_opacities) {
    const uint32_t idx = blockIdx.x * blockDim.x + threadIdx.x; // C * N < 2^31
    const uint32_t T = C * N;
    if (idx >= T) return;
    const uint32_t cid = idx / N, gid = idx - cid * N;
    // everything a kept row needs is requested before the test on the radius (culled rows of
    // the workspace hold zeros): one memory round trip instead of two
    const int32_t o = pos[idx] + offsets[idx / SPLATAD_THREADS];
    const int2 r = reinterpret_cast<const int2 *>(w_radii)[idx];
    const float2 mean = reinterpret_cast<const float2 *>(w_means2d)[idx];
    const float depth = w_depths[idx];
    const float c0 = w_conics[(size_t)idx * 3], c1 = w_conics[(size_t)idx * 3 + 1], c2 = w_conics[(size_t)idx * 3 + 2];
    const float2 vel = reinterpret_cast<const float2 *>(w_pix_vels)[idx];
    const float comp = comps != nullptr ? w_comps[idx] : 1.f;
    const float opacity = row_opacities != nullptr ? opacities[gid] : 0.f;
    if (gid == 0) indptr[cid] = o; // first element of each row holds the row start
    if (idx == T - 1) indptr[C] = (int32_t)nnz;
    if (r.x <= 0) return;
    camera_ids[o] = cid;
    gaussian_ids[o] = gid;
    reinterpret_cast<int2 *>(radii)[o] = r;
    reinterpret_cast<float2 *>(means2d)[o] = mean;
    depths[o] = depth;
    conics[(size_t)o * 3] = c0;
    conics[(size_t)o * 3 + 1] = c1;
    conics[(size_t)o * 3 + 2] = c2;
    if (comps != nullptr) comps[o] = comp;
    reinterpret_cast<float2 *>(pix_vels)[o] = vel;
    // the opacity the compositing takes for the row: the Gaussian's, times the compensation
    // when there is one (rendering.py:311-314 of the reference)
    if (row_opacities != nullptr) row_opacities[o] = comps != nullptr ? opacity * comp : opacity;
}

__global__ void fill_i32_kernel(int32_t *p, int64_t n, int32_t v) {
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) p[i] = v;
}

} // namespace

// kept_sums / tile_sums (both or neither): per-workgroup counts for the packed layout, see
// projection_fwd_kernel<true>.
static int projection_fwd(uint32_t C, uint32_t N, const float *means,
                                      const float *covars, const float *quats,
                                      const float *scales, const float *velocities,
                                      const float *viewmats, const float *Ks, uint32_t W,
                                      uint32_t H, const float *lin_vel, const float *ang_vel,
                                      const float *rs_time, float eps2d, float near_plane,
                                      float far_plane, float radius_clip, int32_t *radii,
                                      float *means2d, float *depths, float *conics,
                                      float *compensations, float *pix_vels,
                                      uint32_t tile_size, uint32_t tile_w, uint32_t tile_h,
                                      int64_t *kept_sums, int64_t *tile_sums, int32_t *kept_before,
                                      splatad_stream_t stream) {
    SPLATAD_REQUIRE((covars != nullptr) != (quats != nullptr && scales != nullptr),
                    "projection: pass either covars or (quats, scales)");
    SPLATAD_REQUIRE((uint64_t)C * N < (1ull << 31), "projection: C*N must be below 2^31");
    if (C == 0 || N == 0) return 0;
    SPLATAD_REQUIRE(means && viewmats && Ks && lin_vel && ang_vel && rs_time && radii && means2d &&
                        depths && conics && pix_vels,
                    "projection: null pointer argument");
    const uint64_t T = (uint64_t)C * N;
    const bool count = kept_sums != nullptr;
    SPLATAD_REQUIRE(!count || (tile_sums != nullptr && kept_before != nullptr && tile_size > 0),
                    "projection: incomplete count arguments");
    hipLaunchKernelGGL((count ? projection_fwd_kernel<true> : projection_fwd_kernel<false>),
                       dim3((uint32_t)((T + SPLATAD_THREADS - 1) / SPLATAD_THREADS)),
                       dim3(SPLATAD_THREADS), 0, (hipStream_t)stream, C, N, means, covars, quats,
                       scales, velocities, viewmats, Ks, W, H, lin_vel, ang_vel, rs_time, eps2d,
                       near_plane, far_plane, radius_clip, radii, means2d, depths, conics,
                       compensations, pix_vels, tile_size, tile_w, tile_h, kept_sums, tile_sums, kept_before);
    SPLATAD_LAUNCH_CHECK();
    return 0;
}

extern "C" int splatad_projection_fwd(uint32_t C, uint32_t N, const float *means,
                                      const float *covars, const float *quats,
                                      const float *scales, const float *velocities,
                                      const float *viewmats, const float *Ks, uint32_t W,
                                      uint32_t H, const float *lin_vel, const float *ang_vel,
                                      const float *rs_time, float eps2d, float near_plane,
                                      float far_plane, float radius_clip, int32_t *radii,
                                      float *means2d, float *depths, float *conics,
                                      float *compensations, float *pix_vels,
                                      splatad_stream_t stream) {
    return projection_fwd(C, N, means, covars, quats, scales, velocities, viewmats, Ks, W, H, lin_vel,
                          ang_vel, rs_time, eps2d, near_plane, far_plane, radius_clip, radii, means2d,
                          depths, conics, compensations, pix_vels, 0, 0, 0, nullptr, nullptr, nullptr, stream);
}

extern "C" int splatad_lidar_projection_fwd(uint32_t C, uint32_t N, const float *means,
                                            const float *covars, const float *quats,
                                            const float *scales, const float *velocities,
                                            const float *viewmats, float min_elev, float max_elev,
                                            float min_azim, float max_azim, const float *lin_vel,
                                            const float *ang_vel, const float *rs_time,
                                            float eps2d, float near_plane, float far_plane,
                                            float radius_clip, float *radii, float *means2d,
                                            float *depths, float *conics, float *compensations,
                                            float *pix_vels, float *depth_comps,
                                            splatad_stream_t stream) {
    SPLATAD_REQUIRE((covars != nullptr) != (quats != nullptr && scales != nullptr),
                    "lidar projection: pass either covars or (quats, scales)");
    SPLATAD_REQUIRE((uint64_t)C * N < (1ull << 31), "lidar projection: C*N must be below 2^31");
    if (C == 0 || N == 0) return 0;
    SPLATAD_REQUIRE(means && viewmats && lin_vel && ang_vel && rs_time && radii && means2d &&
                        depths && conics && pix_vels && depth_comps,
                    "lidar projection: null pointer argument");
    const uint64_t T = (uint64_t)C * N;
    hipLaunchKernelGGL(lidar_projection_fwd_kernel,
                       dim3((uint32_t)((T + SPLATAD_THREADS - 1) / SPLATAD_THREADS)),
                       dim3(SPLATAD_THREADS), 0, (hipStream_t)stream, C, N, means, covars, quats,
                       scales, velocities, viewmats, min_elev, max_elev, min_azim, max_azim,
                       lin_vel, ang_vel, rs_time, eps2d, near_plane, far_plane, radius_clip, radii,
                       means2d, depths, conics, compensations, pix_vels, depth_comps);
    SPLATAD_LAUNCH_CHECK();
    return 0;
}

extern "C" size_t splatad_projection_packed_workspace_bytes(uint32_t C, uint32_t N) {
    const uint64_t T = (uint64_t)C * N;
    return 256 + splatad_align256(T * 8) * 3 + splatad_align256(T * 4) * 3 +
           splatad_align256(T * 12) + 2 * SCAN_ITEMS * scan_workspace_bytes((int64_t)T) +
           splatad_align256((T / SPLATAD_THREADS + 1) * 4) + splatad_align256(T * 4);
}

// tile_size == 0: only the kept rows are counted.
static int packed_count(uint32_t C, uint32_t N, const float *means, const float *covars, const float *quats,
                        const float *scales, const float *velocities, const float *viewmats, const float *Ks,
                        uint32_t W, uint32_t H, const float *lin_vel, const float *ang_vel, const float *rs_time,
                        float eps2d, float near_plane, float far_plane, float radius_clip, int calc_compensations,
                        uint32_t tile_size, uint32_t tile_width, uint32_t tile_height, void *workspace,
                        void *isect_workspace, int64_t *nnz_host, int64_t *n_isects_host,
                        splatad_stream_t stream) {
    SPLATAD_REQUIRE(nnz_host != nullptr, "packed projection: nnz_host is null");
    *nnz_host = 0;
    if (n_isects_host) *n_isects_host = 0;
    if (C == 0 || N == 0) return 0;
    SPLATAD_REQUIRE(workspace != nullptr, "packed projection: workspace is null");
    const uint64_t T = (uint64_t)C * N;
    PackedWorkspace w = carve_packed(workspace, T);
    if (int rc = host_word_refuse_capture((hipStream_t)stream, "packed projection")) return rc;
    // the counts reach the host through a leased pinned word
    HostWordLease lease((hipStream_t)stream);
    if (int rc = host_word_acquire(&lease.word)) return rc;
    // With a tile grid the projection itself counts, per workgroup, the kept rows and their
    // tiles, and leaves every row's place among the kept rows of its workgroup: the host word is
    // published right behind it by the kernel that also adds up the workgroups' places.
    const int64_t n_groups = ((int64_t)T + SPLATAD_THREADS - 1) / SPLATAD_THREADS;
    const bool fused = tile_size != 0;
    int rc = projection_fwd(C, N, means, covars, quats, scales, velocities, viewmats, Ks, W, H, lin_vel,
                            ang_vel, rs_time, eps2d, near_plane, far_plane, radius_clip, w.radii, w.means2d,
                            w.depths, w.conics, calc_compensations ? w.comps : nullptr, w.pix_vels,
                            fused ? tile_size : 0, tile_width, tile_height, fused ? w.block_sums : nullptr,
                            fused ? w.tile_sums : nullptr, fused ? w.pos : nullptr, stream);
    if (rc) return rc;
    if (fused) {
        hipLaunchKernelGGL(packed_publish_kernel, dim3(1), dim3(SPLATAD_THREADS), 0, (hipStream_t)stream,
                           (const int64_t *)nullptr, (const int64_t *)w.block_sums, (const int64_t *)w.tile_sums,
                           n_groups, lease.word.device, w.offsets);
        SPLATAD_LAUNCH_CHECK();
        // (no scan over the rows: the projection left every row's place inside its workgroup
        // in w.pos, and the publishing kernel the workgroups' places in w.offsets)
        if (isect_workspace != nullptr) {
            rc = splatad_isect_tiles_prepare(T, N, nullptr, w.means2d, w.radii, w.depths, C, tile_size,
                                             tile_width, tile_height, 1, nullptr, isect_workspace, stream);
            if (rc) return rc;
        }
    } else if (tile_size == 0) {
        hipLaunchKernelGGL(fill_i32_kernel, dim3((uint32_t)((n_groups + 1 + 255) / 256)), dim3(256), 0,
                           (hipStream_t)stream, w.offsets, n_groups + 1, 0);
        rc = launch_exclusive_scan<int32_t>(w.radii, (int64_t)T, 2, 1, w.pos, w.total, w.block_sums,
                                            (hipStream_t)stream);
        if (rc) return rc;
        hipLaunchKernelGGL(host_word_publish_kernel, dim3(1), dim3(1), 0, (hipStream_t)stream, w.total,
                           lease.word.device);
    }
    SPLATAD_LAUNCH_CHECK();
    unsigned long long word = 0;
    rc = host_word_wait(&lease, "packed projection", &word);
    if (rc) return rc;
    if (tile_size == 0) {
        *nnz_host = (int64_t)word;
    } else {
        *nnz_host = (int64_t)(word & 0xFFFFFFFFull);
        SPLATAD_REQUIRE((word >> 32) < 0x7FFFFFFFull,
                        "packed projection: the kept rows meet 2^31 - 1 tiles or more, beyond the int32 offset range");
        if (n_isects_host) *n_isects_host = (int64_t)(word >> 32);
    }
    return 0;
}

extern "C" int splatad_projection_packed_count(
    uint32_t C, uint32_t N, const float *means, const float *covars, const float *quats,
    const float *scales, const float *velocities, const float *viewmats, const float *Ks,
    uint32_t W, uint32_t H, const float *lin_vel, const float *ang_vel, const float *rs_time,
    float eps2d, float near_plane, float far_plane, float radius_clip, int calc_compensations,
    void *workspace, int64_t *nnz_host, splatad_stream_t stream) {
    return packed_count(C, N, means, covars, quats, scales, velocities, viewmats, Ks, W, H, lin_vel, ang_vel,
                        rs_time, eps2d, near_plane, far_plane, radius_clip, calc_compensations, 0, 0, 0,
                        workspace, nullptr, nnz_host, nullptr, stream);
}

extern "C" int splatad_projection_packed_count_tiles(
    uint32_t C, uint32_t N, const float *means, const float *covars, const float *quats,
    const float *scales, const float *velocities, const float *viewmats, const float *Ks,
    uint32_t W, uint32_t H, const float *lin_vel, const float *ang_vel, const float *rs_time,
    float eps2d, float near_plane, float far_plane, float radius_clip, int calc_compensations,
    uint32_t tile_size, uint32_t tile_width, uint32_t tile_height, void *workspace, void *isect_workspace,
    int64_t *nnz_host, int64_t *n_isects_host, splatad_stream_t stream) {
    SPLATAD_REQUIRE(tile_size > 0 && n_isects_host != nullptr,
                    "packed projection: tile_size is zero or n_isects_host is null");
    return packed_count(C, N, means, covars, quats, scales, velocities, viewmats, Ks, W, H, lin_vel, ang_vel,
                        rs_time, eps2d, near_plane, far_plane, radius_clip, calc_compensations, tile_size,
                        tile_width, tile_height, workspace, isect_workspace, nnz_host, n_isects_host, stream);
}

extern "C" int splatad_isect_tiles_fill_packed(uint32_t C, uint32_t N, uint32_t tile_size, uint32_t tile_width,
                                               uint32_t tile_height, int64_t n_isects,
                                               const void *packed_workspace, void *isect_workspace,
                                               void *lists, int32_t *tiles_per_gauss, int64_t *isect_ids,
                                               int32_t *flatten_ids, int32_t *tile_offsets,
                                               splatad_stream_t beside_stream, splatad_beside_fn beside_work,
                                               void *beside_context, splatad_stream_t stream) {
    SPLATAD_REQUIRE(packed_workspace && isect_workspace, "isect_tiles: null workspace");
    const uint64_t T = (uint64_t)C * N;
    PackedWorkspace w = carve_packed((void *)packed_workspace, T);
    return splatad_isect_tiles_fill_remapped(T, N, w.means2d, w.radii, w.depths, C, tile_size, tile_width,
                                             tile_height, n_isects, w.tiles, w.pos, w.offsets, isect_workspace, lists,
                                             tiles_per_gauss, isect_ids, flatten_ids, tile_offsets,
                                             beside_stream, beside_work, beside_context, stream);
}

extern "C" int splatad_view_colors_fwd_packed(uint32_t C, uint32_t N, uint32_t K, uint32_t degree,
                                              const float *means, const float *viewmats,
                                              const void *packed_workspace, const float *coeffs,
                                              int coeffs_per_sensor, int with_depth, float *colors,
                                              splatad_stream_t stream) {
    SPLATAD_REQUIRE(packed_workspace != nullptr, "view colours: null workspace");
    PackedWorkspace w = carve_packed((void *)packed_workspace, (uint64_t)C * N);
    return splatad_view_colors_fwd_remapped(C, N, K, degree, means, viewmats, w.radii, w.pos, w.offsets, coeffs,
                                            coeffs_per_sensor, with_depth ? w.depths : nullptr, colors, stream);
}

extern "C" int splatad_projection_packed_fill(uint32_t C, uint32_t N, int64_t nnz,
                                              const void *workspace, int32_t *indptr,
                                              int64_t *camera_ids, int64_t *gaussian_ids,
                                              int32_t *radii, float *means2d, float *depths,
                                              float *conics, float *compensations,
                                              float *pix_vels, const float *opacities,
                                              float *row_opacities, splatad_stream_t stream) {
    SPLATAD_REQUIRE(indptr != nullptr, "packed projection: indptr is null");
    const uint64_t T = (uint64_t)C * N;
    if (T == 0 || nnz == 0) {
        hipLaunchKernelGGL(fill_i32_kernel, dim3((C + 1 + 255) / 256), dim3(256), 0,
                           (hipStream_t)stream, indptr, (int64_t)C + 1, 0);
        SPLATAD_LAUNCH_CHECK();
        return 0;
    }
    SPLATAD_REQUIRE(workspace && camera_ids && gaussian_ids && radii && means2d && depths &&
                        conics && pix_vels,
                    "packed projection: null pointer argument");
    SPLATAD_REQUIRE((opacities != nullptr) == (row_opacities != nullptr),
                    "packed projection: opacities and row_opacities go together");
    PackedWorkspace w = carve_packed((void *)workspace, T);
    hipLaunchKernelGGL(packed_compact_kernel,
                       dim3((uint32_t)((T + SPLATAD_THREADS - 1) / SPLATAD_THREADS)),
                       dim3(SPLATAD_THREADS), 0, (hipStream_t)stream, C, N, nnz, w.radii,
                       w.means2d, w.depths, w.conics, w.comps, w.pix_vels, w.pos, w.offsets, indptr,
                       camera_ids, gaussian_ids, radii, means2d, depths, conics, compensations,
                       pix_vels, opacities, row_opacities);
    SPLATAD_LAUNCH_CHECK();
    return 0;
}
