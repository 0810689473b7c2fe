/*
 * CPU ORACLE -- TEST INFRASTRUCTURE ONLY.
 *
 * A plain-C restatement of the rendering hot path of carlinds/splatad
 * (projection -> tile intersection + sort + offsets -> alpha compositing, for
 * pinhole cameras and spinning lidars with rolling-shutter compensation).
 * Nothing in the shipped package may link, load or call this file: it exists
 * to check the HIP kernels (tests/), to smoke-test them
 * (__graft_entry__.smoke) and to be timed as the CPU baseline (bench.py).
 *
 * The file is compiled twice: -DORACLE_F64=0 gives single-precision
 * arithmetic (same rounding class as the GPU kernels; needed for the
 * bit-exact integer outputs), -DORACLE_F64=1 gives double precision (the
 * "truth" for floating-point tolerances).  Inputs are always float32 arrays,
 * outputs are `real` arrays.
 *
 * Every function cites the reference file:line it follows (paths relative to
 * the reference checkout).  How each function is pinned (closed forms, brute
 * force, known-answer cases of the reference's own tests) is written next to
 * its test in tests/test_oracle_*.py.  Parity status: every function below has
 * at least one such pin; none is "parity unpinned".
 *
 * On a culled Gaussian the reference writes only radii[2*idx]=0 and leaves
 * the other outputs uninitialised (projection.cu:658-661); this oracle (and
 * the HIP kernels) zero-fill them instead.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#ifndef ORACLE_F64
#define ORACLE_F64 0
#endif

#if ORACLE_F64
typedef double real;
#define NAME(x) oracle_f64_##x
#define R_SQRT sqrt
#define R_FABS fabs
#define R_EXP exp
#define R_FMOD fmod
#define R_FLOOR floor
#define R_CEIL ceil
#define R_ATAN2 atan2
#define R_ASIN asin
#define R_HYPOT hypot
#define R_FMIN fmin
#define R_FMAX fmax
#else
typedef float real;
#define NAME(x) oracle_f32_##x
#define R_SQRT sqrtf
#define R_FABS fabsf
#define R_EXP expf
#define R_FMOD fmodf
#define R_FLOOR floorf
#define R_CEIL ceilf
#define R_ATAN2 atan2f
#define R_ASIN asinf
#define R_HYPOT hypotf
#define R_FMIN fminf
#define R_FMAX fmaxf
#endif

#define RC(x) ((real)(x))
/* utils.cuh:10 */
#define RAD_TO_DEG RC(57.2957795131)

/* ------------------------------------------------------------------ */
/* small dense algebra, row-major 3x3                                   */
/* ------------------------------------------------------------------ */

static void mat3_mul(const real *A, const real *B, real *C) {
    for (int i = 0; i < 3; ++i)
        for (int j = 0; j < 3; ++j) {
            real s = 0;
            for (int k = 0; k < 3; ++k) s += A[i * 3 + k] * B[k * 3 + j];
            C[i * 3 + j] = s;
        }
}

static void mat3_mul_t(const real *A, const real *B, real *C) { /* A * B^T */
    for (int i = 0; i < 3; ++i)
        for (int j = 0; j < 3; ++j) {
            real s = 0;
            for (int k = 0; k < 3; ++k) s += A[i * 3 + k] * B[j * 3 + k];
            C[i * 3 + j] = s;
        }
}

/* utils.cuh:57-75 (quat_to_rotmat): quaternion (w,x,y,z), normalised inside. */
static void quat_to_rotmat(const real q[4], real R[9]) {
    real w = q[0], x = q[1], y = q[2], z = q[3];
    real inv = RC(1) / R_SQRT(w * w + x * x + y * y + z * z);
    w *= inv; x *= inv; y *= inv; z *= inv;
    real x2 = x * x, y2 = y * y, z2 = z * z;
    real xy = x * y, xz = x * z, yz = y * z;
    real wx = w * x, wy = w * y, wz = w * z;
    R[0] = RC(1) - RC(2) * (y2 + z2); R[1] = RC(2) * (xy - wz); R[2] = RC(2) * (xz + wy);
    R[3] = RC(2) * (xy + wz); R[4] = RC(1) - RC(2) * (x2 + z2); R[5] = RC(2) * (yz - wx);
    R[6] = RC(2) * (xz - wy); R[7] = RC(2) * (yz + wx); R[8] = RC(1) - RC(2) * (x2 + y2);
}

/* utils.cuh:100-111 (quat_scale_to_covar_preci, covariance branch):
 * covar = (R S)(R S)^T. */
static void quat_scale_to_covar(const real q[4], const real s[3], real cov[9]) {
    real R[9], M[9];
    quat_to_rotmat(q, R);
    for (int i = 0; i < 3; ++i)
        for (int j = 0; j < 3; ++j) M[i * 3 + j] = R[i * 3 + j] * s[j];
    mat3_mul_t(M, M, cov);
}

/* projection.cu:665-677: covariance either from the 6-vector upper triangle
 * or from (quat, scale). */
static void load_covar(int g, const float *covars, const float *quats, const float *scales,
                       real cov[9]) {
    if (covars) {
        const float *c = covars + (size_t)g * 6;
        cov[0] = c[0]; cov[1] = c[1]; cov[2] = c[2];
        cov[3] = c[1]; cov[4] = c[3]; cov[5] = c[4];
        cov[6] = c[2]; cov[7] = c[4]; cov[8] = c[5];
    } else {
        real q[4] = {quats[g * 4], quats[g * 4 + 1], quats[g * 4 + 2], quats[g * 4 + 3]};
        real s[3] = {scales[g * 3], scales[g * 3 + 1], scales[g * 3 + 2]};
        quat_scale_to_covar(q, s, cov);
    }
}

/* utils.cuh:447-451, 467-471: p_c = R p + t, covar_c = R covar R^T.
 * viewmats are row-major [4,4] (projection.cu:647-652). */
static void world_to_cam(const float *vm, const float *p, const real cov[9], real R[9],
                         real pc[3], real covc[9]) {
    R[0] = vm[0]; R[1] = vm[1]; R[2] = vm[2];
    R[3] = vm[4]; R[4] = vm[5]; R[5] = vm[6];
    R[6] = vm[8]; R[7] = vm[9]; R[8] = vm[10];
    real t[3] = {vm[3], vm[7], vm[11]};
    for (int i = 0; i < 3; ++i)
        pc[i] = R[i * 3] * RC(p[0]) + R[i * 3 + 1] * RC(p[1]) + R[i * 3 + 2] * RC(p[2]) + t[i];
    if (cov) {
        real tmp[9];
        mat3_mul(R, cov, tmp);
        mat3_mul_t(tmp, R, covc);
    }
}

/* utils.cuh:190-217 (persp_proj) Jacobian rows; shared with
 * helpers.cuh:80-118 (compute_pix_velocity). J is 2x3 row-major. */
static void persp_jacobian(const real pc[3], real fx, real fy, real cx, real cy, int W, int H,
                           real J[6]) {
    real x = pc[0], y = pc[1], z = pc[2];
    real tan_fovx = RC(0.5) * (real)W / fx;
    real tan_fovy = RC(0.5) * (real)H / fy;
    real lim_x_pos = ((real)W - cx) / fx + RC(0.3) * tan_fovx;
    real lim_x_neg = cx / fx + RC(0.3) * tan_fovx;
    real lim_y_pos = ((real)H - cy) / fy + RC(0.3) * tan_fovy;
    real lim_y_neg = cy / fy + RC(0.3) * tan_fovy;
    real rz = RC(1) / z;
    real rz2 = rz * rz;
    real tx = z * R_FMIN(lim_x_pos, R_FMAX(-lim_x_neg, x * rz));
    real ty = z * R_FMIN(lim_y_pos, R_FMAX(-lim_y_neg, y * rz));
    J[0] = fx * rz; J[1] = 0; J[2] = -fx * tx * rz2;
    J[3] = 0; J[4] = fy * rz; J[5] = -fy * ty * rz2;
}

/* utils.cuh:511-519 (add_blur). cov2 = {xx, xy, yy}. */
static real add_blur(real eps2d, real cov2[3], real *compensation) {
    real det_orig = cov2[0] * cov2[2] - cov2[1] * cov2[1];
    cov2[0] += eps2d;
    cov2[2] += eps2d;
    real det_blur = cov2[0] * cov2[2] - cov2[1] * cov2[1];
    *compensation = R_SQRT(R_FMAX(RC(0), det_orig / det_blur));
    return det_blur;
}

static void cross3(const real a[3], const real b[3], real c[3]) {
    c[0] = a[1] * b[2] - a[2] * b[1];
    c[1] = a[2] * b[0] - a[0] * b[2];
    c[2] = a[0] * b[1] - a[1] * b[0];
}

/* ------------------------------------------------------------------ */
/* P1: fused camera projection (projection.cu:605-751)                  */
/* ------------------------------------------------------------------ */
void NAME(projection_fwd)(int C, int N, const float *means, const float *covars,
                          const float *quats, const float *scales, const float *velocities,
                          const float *viewmats, const float *Ks, int W, int H,
                          const float *lin_vel, const float *ang_vel, const float *rs_time,
                          float eps2d_f, float near_f, float far_f, float radius_clip_f,
                          int32_t *radii, real *means2d, real *depths, real *conics,
                          real *compensations, real *pix_vels) {
    const real eps2d = eps2d_f, near_plane = near_f, far_plane = far_f, radius_clip = radius_clip_f;
#pragma omp parallel for schedule(static)
    for (long idx = 0; idx < (long)C * N; ++idx) {
        int cid = (int)(idx / N), gid = (int)(idx % N);
        radii[idx * 2] = 0; radii[idx * 2 + 1] = 0;
        means2d[idx * 2] = 0; means2d[idx * 2 + 1] = 0;
        depths[idx] = 0;
        conics[idx * 3] = 0; conics[idx * 3 + 1] = 0; conics[idx * 3 + 2] = 0;
        if (compensations) compensations[idx] = 0;
        pix_vels[idx * 2] = 0; pix_vels[idx * 2 + 1] = 0;

        const float *vm = viewmats + cid * 16;
        const float *K = Ks + cid * 9;
        real R[9], pc[3];
        world_to_cam(vm, means + (size_t)gid * 3, NULL, R, pc, NULL);
        /* projection.cu:658 */
        if (pc[2] < near_plane || pc[2] > far_plane) continue;

        real cov[9], covc[9];
        load_covar(gid, covars, quats, scales, cov);
        {
            real tmp[9];
            mat3_mul(R, cov, tmp);
            mat3_mul_t(tmp, R, covc);
        }
        real fx = K[0], fy = K[4], cx = K[2], cy = K[5];
        real J[6];
        persp_jacobian(pc, fx, fy, cx, cy, W, H, J);
        /* cov2d = J covc J^T (utils.cuh:215) */
        real JC[6];
        for (int i = 0; i < 2; ++i)
            for (int j = 0; j < 3; ++j)
                JC[i * 3 + j] = J[i * 3] * covc[j] + J[i * 3 + 1] * covc[3 + j] + J[i * 3 + 2] * covc[6 + j];
        real cov2[3];
        cov2[0] = JC[0] * J[0] + JC[1] * J[1] + JC[2] * J[2];
        cov2[1] = JC[0] * J[3] + JC[1] * J[4] + JC[2] * J[5];
        cov2[2] = JC[3] * J[3] + JC[4] * J[4] + JC[5] * J[5];
        real rz = RC(1) / pc[2];
        real m2x = fx * pc[0] * rz + cx, m2y = fy * pc[1] * rz + cy; /* utils.cuh:216 */

        real comp;
        real det = add_blur(eps2d, cov2, &comp);
        if (det <= 0) continue; /* projection.cu:689 */

        real ext_x = RC(3) * R_SQRT(cov2[0]); /* projection.cu:702-703 */
        real ext_y = RC(3) * R_SQRT(cov2[2]);
        if (ext_x <= radius_clip && ext_y <= radius_clip) continue; /* :705 */

        real pvx = 0, pvy = 0;
        real rs = rs_time[cid];
        if (rs > 0) { /* projection.cu:712-723, helpers.cuh:80-118 */
            real velc[3] = {0, 0, 0};
            if (velocities) {
                const float *v = velocities + (size_t)gid * 3;
                for (int i = 0; i < 3; ++i)
                    velc[i] = R[i * 3] * RC(v[0]) + R[i * 3 + 1] * RC(v[1]) + R[i * 3 + 2] * RC(v[2]);
            }
            real lv[3] = {lin_vel[cid * 3], lin_vel[cid * 3 + 1], lin_vel[cid * 3 + 2]};
            real av[3] = {ang_vel[cid * 3], ang_vel[cid * 3 + 1], ang_vel[cid * 3 + 2]};
            real rot[3], tv[3];
            cross3(av, pc, rot);
            for (int i = 0; i < 3; ++i) tv[i] = lv[i] + rot[i] - velc[i];
            pvx = -(J[0] * tv[0] + J[1] * tv[1] + J[2] * tv[2]);
            pvy = -(J[3] * tv[0] + J[4] * tv[1] + J[5] * tv[2]);
            ext_x += R_FABS(pvx) * RC(0.5) * rs;
            ext_y += R_FABS(pvy) * RC(0.5) * rs;
        }
        /* projection.cu:727-728 */
        if (m2x + ext_x <= 0 || m2x - ext_x >= (real)W || m2y + ext_y <= 0 || m2y - ext_y >= (real)H)
            continue;
        /* utils.cuh:491-502 (inverse); det > 0 here */
        real inv_det = RC(1) / det;
        radii[idx * 2] = (int32_t)ext_x; /* truncation, projection.cu:738 */
        radii[idx * 2 + 1] = (int32_t)ext_y;
        means2d[idx * 2] = m2x; means2d[idx * 2 + 1] = m2y;
        depths[idx] = pc[2];
        conics[idx * 3] = cov2[2] * inv_det;
        conics[idx * 3 + 1] = -cov2[1] * inv_det;
        conics[idx * 3 + 2] = cov2[0] * inv_det;
        if (compensations) compensations[idx] = comp;
        pix_vels[idx * 2] = pvx; pix_vels[idx * 2 + 1] = pvy;
    }
}

/* ------------------------------------------------------------------ */
/* L1: fused lidar projection (projection.cu:2268-2417,                 */
/*     utils.cuh:12-31, 281-318, helpers.cuh:120-153)                   */
/* ------------------------------------------------------------------ */
void NAME(lidar_projection_fwd)(int C, int N, const float *means, const float *covars,
                                const float *quats, const float *scales, const float *velocities,
                                const float *viewmats, float min_elev_f, float max_elev_f,
                                float min_azim_f, float max_azim_f, const float *lin_vel,
                                const float *ang_vel, const float *rs_time, float eps2d_f,
                                float near_f, float far_f, float radius_clip_f, real *radii,
                                real *means2d, real *depths, real *conics, real *compensations,
                                real *pix_vels, real *depth_comps) {
    const real eps2d = eps2d_f, near_plane = near_f, far_plane = far_f, radius_clip = radius_clip_f;
    const real min_elev = min_elev_f, max_elev = max_elev_f, min_azim = min_azim_f, max_azim = max_azim_f;
#pragma omp parallel for schedule(static)
    for (long idx = 0; idx < (long)C * N; ++idx) {
        int cid = (int)(idx / N), gid = (int)(idx % N);
        radii[idx * 2] = 0; radii[idx * 2 + 1] = 0;
        means2d[idx * 2] = 0; means2d[idx * 2 + 1] = 0;
        depths[idx] = 0;
        conics[idx * 3] = 0; conics[idx * 3 + 1] = 0; conics[idx * 3 + 2] = 0;
        if (compensations) compensations[idx] = 0;
        pix_vels[idx * 3] = 0; pix_vels[idx * 3 + 1] = 0; pix_vels[idx * 3 + 2] = 0;
        depth_comps[idx * 2] = 0; depth_comps[idx * 2 + 1] = 0;

        const float *vm = viewmats + cid * 16;
        real R[9], pc[3];
        world_to_cam(vm, means + (size_t)gid * 3, NULL, R, pc, NULL);
        real x = pc[0], y = pc[1], z = pc[2];
        real r2 = x * x + y * y + z * z;
        real dist = R_SQRT(r2);
        if (dist < near_plane || dist > far_plane) continue; /* projection.cu:2322 */

        real cov[9], covc[9];
        load_covar(gid, covars, quats, scales, cov);
        {
            real tmp[9];
            mat3_mul(R, cov, tmp);
            mat3_mul_t(tmp, R, covc);
        }
        /* utils.cuh:290-306: rows d(az), d(el), d(range) w.r.t. (x,y,z) */
        real rinv = RC(1) / dist;
        real rho2 = x * x + y * y;
        real rho = R_HYPOT(x, y);
        real rho_inv = RC(1) / rho;
        real r2rho_inv = RC(1) / r2 * rho_inv;
        real J[9];
        J[0] = -y / rho2 * RAD_TO_DEG; J[1] = x / rho2 * RAD_TO_DEG; J[2] = 0;
        J[3] = -x * z * r2rho_inv * RAD_TO_DEG; J[4] = -y * z * r2rho_inv * RAD_TO_DEG;
        J[5] = rho / r2 * RAD_TO_DEG;
        J[6] = x * rinv; J[7] = y * rinv; J[8] = z * rinv;
        real tmp[9], cs[9];
        mat3_mul(J, covc, tmp);
        mat3_mul_t(tmp, J, cs);
        real cov2[3] = {cs[0], cs[1], cs[4]};
        real m2x = R_ATAN2(y, x) * RAD_TO_DEG, m2y = R_ASIN(z * rinv) * RAD_TO_DEG;
        /* utils.cuh:12-31 */
        real a1 = cs[0] + eps2d, a2 = cs[1], b1 = cs[3], b2 = cs[4] + eps2d, c1 = cs[6], c2 = cs[7];
        real invD = RC(1) / (a1 * b2 - a2 * b1);
        real dc0 = (b1 * c2 - b2 * c1) * invD, dc1 = (a2 * c1 - a1 * c2) * invD;

        real comp;
        real det = add_blur(eps2d, cov2, &comp);
        if (det <= 0) continue;
        real ext_az = RC(3) * R_SQRT(R_FMAX(RC(0), cov2[0])); /* projection.cu:2366-2367 */
        real ext_el = RC(3) * R_SQRT(R_FMAX(RC(0), cov2[2]));
        if (ext_az <= radius_clip && ext_el <= radius_clip) continue;

        real pv[3] = {0, 0, 0};
        real rs = rs_time[cid];
        if (rs > 0) { /* projection.cu:2376-2386 */
            real velc[3] = {0, 0, 0};
            if (velocities) {
                const float *v = velocities + (size_t)gid * 3;
                for (int i = 0; i < 3; ++i)
                    velc[i] = R[i * 3] * RC(v[0]) + R[i * 3 + 1] * RC(v[1]) + R[i * 3 + 2] * RC(v[2]);
            }
            real lv[3] = {lin_vel[cid * 3], lin_vel[cid * 3 + 1], lin_vel[cid * 3 + 2]};
            real av[3] = {ang_vel[cid * 3], ang_vel[cid * 3 + 1], ang_vel[cid * 3 + 2]};
            real rot[3], tv[3];
            cross3(av, pc, rot);
            for (int i = 0; i < 3; ++i) tv[i] = lv[i] + rot[i] - velc[i];
            for (int i = 0; i < 3; ++i)
                pv[i] = -(J[i * 3] * tv[0] + J[i * 3 + 1] * tv[1] + J[i * 3 + 2] * tv[2]);
            ext_az += R_FABS(pv[0]) * RC(0.5) * rs;
            ext_el += R_FABS(pv[1]) * RC(0.5) * rs;
        }
        /* projection.cu:2388-2394 */
        if (m2y + ext_el <= min_elev || m2y - ext_el >= max_elev || m2x + ext_az <= min_azim ||
            m2x - ext_az >= max_azim)
            continue;
        real inv_det = RC(1) / det;
        radii[idx * 2] = ext_az; radii[idx * 2 + 1] = ext_el;
        means2d[idx * 2] = m2x; means2d[idx * 2 + 1] = m2y;
        depths[idx] = dist;
        conics[idx * 3] = cov2[2] * inv_det;
        conics[idx * 3 + 1] = -cov2[1] * inv_det;
        conics[idx * 3 + 2] = cov2[0] * inv_det;
        if (compensations) compensations[idx] = comp;
        pix_vels[idx * 3] = pv[0]; pix_vels[idx * 3 + 1] = pv[1]; pix_vels[idx * 3 + 2] = pv[2];
        depth_comps[idx * 2] = dc0; depth_comps[idx * 2 + 1] = dc1;
    }
}

/* ------------------------------------------------------------------ */
/* S1: spherical harmonics (sh.cu:13-93, 355-374)                        */
/* ------------------------------------------------------------------ */
void NAME(sh_fwd)(long n, int K, int degree, const float *dirs, const float *coeffs,
                  const uint8_t *masks, real *colors) {
#pragma omp parallel for schedule(static)
    for (long e = 0; e < n; ++e) {
        for (int c = 0; c < 3; ++c) colors[e * 3 + c] = 0;
        if (masks && !masks[e]) continue;
        const float *cf = coeffs + (size_t)e * K * 3;
        real b[25];
        int nb = 1;
        b[0] = RC(0.2820947917738781);
        if (degree >= 1) {
            real dx = dirs[e * 3], dy = dirs[e * 3 + 1], dz = dirs[e * 3 + 2];
            real inorm = RC(1) / R_SQRT(dx * dx + dy * dy + dz * dz);
            real x = dx * inorm, y = dy * inorm, z = dz * inorm;
            b[1] = RC(-0.48860251190292) * y;
            b[2] = RC(0.48860251190292) * z;
            b[3] = RC(-0.48860251190292) * x;
            nb = 4;
            if (degree >= 2) {
                real z2 = z * z;
                real fTmp0B = RC(-1.092548430592079) * z;
                real fC1 = x * x - y * y, fS1 = RC(2) * x * y;
                b[4] = RC(0.5462742152960395) * fS1;
                b[5] = fTmp0B * y;
                b[6] = RC(0.9461746957575601) * z2 - RC(0.3153915652525201);
                b[7] = fTmp0B * x;
                b[8] = RC(0.5462742152960395) * fC1;
                nb = 9;
                if (degree >= 3) {
                    real fTmp0C = RC(-2.285228997322329) * z2 + RC(0.4570457994644658);
                    real fTmp1B = RC(1.445305721320277) * z;
                    real fC2 = x * fC1 - y * fS1, fS2 = x * fS1 + y * fC1;
                    b[9] = RC(-0.5900435899266435) * fS2;
                    b[10] = fTmp1B * fS1;
                    b[11] = fTmp0C * y;
                    b[12] = z * (RC(1.865881662950577) * z2 - RC(1.119528997770346));
                    b[13] = fTmp0C * x;
                    b[14] = fTmp1B * fC1;
                    b[15] = RC(-0.5900435899266435) * fC2;
                    nb = 16;
                    if (degree >= 4) {
                        real fTmp0D = z * (RC(-4.683325804901025) * z2 + RC(2.007139630671868));
                        real fTmp1C = RC(3.31161143515146) * z2 - RC(0.47308734787878);
                        real fTmp2B = RC(-1.770130769779931) * z;
                        real fC3 = x * fC2 - y * fS2, fS3 = x * fS2 + y * fC2;
                        b[16] = RC(0.6258357354491763) * fS3;
                        b[17] = fTmp2B * fS2;
                        b[18] = fTmp1C * fS1;
                        b[19] = fTmp0D * y;
                        b[20] = RC(1.984313483298443) * z * b[12] - RC(1.006230589874905) * b[6];
                        b[21] = fTmp0D * x;
                        b[22] = fTmp1C * fC1;
                        b[23] = fTmp2B * fC2;
                        b[24] = RC(0.6258357354491763) * fC3;
                        nb = 25;
                    }
                }
            }
        }
        for (int c = 0; c < 3; ++c) {
            real s = 0;
            for (int k = 0; k < nb; ++k) s += b[k] * RC(cf[k * 3 + c]);
            colors[e * 3 + c] = s;
        }
    }
}

/* ------------------------------------------------------------------ */
/* I1/I2: tile intersection.  Always single precision: the inputs are    */
/* float32 and the tile bounds are float32 arithmetic in the reference.  */
/* Only built into the f32 library.                                      */
/* ------------------------------------------------------------------ */
#if !ORACLE_F64

/* CUDA float->uint32 conversion saturates (negatives and NaN -> 0); plain C
 * leaves it undefined, so spell it out (rasterization.cu:53-56). */
static uint32_t f2u_sat(float v) {
    if (!(v > 0.0f)) return 0u;
    if (v >= 4294967296.0f) return 0xFFFFFFFFu;
    return (uint32_t)v;
}
static uint32_t umin(uint32_t a, uint32_t b) { return a < b ? a : b; }

/* rasterization.cu:46-56: inclusive tile_min, exclusive tile_max. */
static void cam_tile_rect(const float *means2d, const int32_t *radii, long idx, uint32_t tile_size,
                          uint32_t tile_w, uint32_t tile_h, uint32_t rect[4]) {
    float tile_extent_x = (float)radii[idx * 2] / (float)tile_size;
    float tile_extent_y = (float)radii[idx * 2 + 1] / (float)tile_size;
    float tile_x = means2d[idx * 2] / (float)tile_size;
    float tile_y = means2d[idx * 2 + 1] / (float)tile_size;
    rect[0] = umin(f2u_sat(floorf(tile_x - tile_extent_x)), tile_w);
    rect[1] = umin(f2u_sat(floorf(tile_y - tile_extent_y)), tile_h);
    rect[2] = umin(f2u_sat(ceilf(tile_x + tile_extent_x)), tile_w);
    rect[3] = umin(f2u_sat(ceilf(tile_y + tile_extent_y)), tile_h);
}

/* rasterization.cu:321-357: azimuth range may be negative or exceed
 * n_tiles_azim (wrapped at emission); elevation by linear scan with strict <. */
static void lidar_tile_rect(const float *means2d, const float *radii, long idx,
                            const float *elev_boundaries, float tile_azim_res, float min_azim,
                            uint32_t n_tiles_azim, uint32_t n_tiles_elev, int32_t rect[4]) {
    float tile_elev = means2d[idx * 2 + 1];
    float tile_elev_low = tile_elev - radii[idx * 2 + 1];
    float tile_elev_high = tile_elev + radii[idx * 2 + 1];
    float azim = means2d[idx * 2] - min_azim;
    float azim_low = azim - radii[idx * 2];
    float azim_high = azim + radii[idx * 2];
    float azim_max = (float)n_tiles_azim * tile_azim_res;
    float tile_azim_low, tile_azim_high;
    if (azim_low >= 0)
        tile_azim_low = azim_low / tile_azim_res;
    else
        tile_azim_low = (fmodf(azim_low + 360.f, 360.f) - azim_max) / tile_azim_res;
    if (azim_high <= 360.f)
        tile_azim_high = azim_high / tile_azim_res;
    else
        tile_azim_high = (float)n_tiles_azim + fmodf(azim_high + 360.f, 360.f) / tile_azim_res;
    rect[0] = (int32_t)floorf(tile_azim_low);
    rect[2] = (int32_t)ceilf(tile_azim_high);
    int32_t i = 0, n = (int32_t)n_tiles_elev;
    while (i <= n && elev_boundaries[i] < tile_elev_low) ++i;
    rect[1] = i - 1 > 0 ? i - 1 : 0;
    while (i <= n && elev_boundaries[i] < tile_elev_high) ++i;
    rect[3] = i < n ? i : n;
}

/* rasterization.cu:134-135 */
static uint32_t bit_width_u32(uint32_t v) {
    uint32_t b = 0;
    while (v) { ++b; v >>= 1; }
    return b; /* == floor(log2(v)) + 1 for v >= 1 */
}

/* Pass 1 of isect_tiles / isect_lidar_tiles: tiles_per_gauss.  Returns
 * n_isects.  `lidar` selects rasterization.cu:287-364 over :15-63. */
long oracle_isect_count(int lidar, long total, const float *means2d, const void *radii,
                        uint32_t tile_size, uint32_t tile_w, uint32_t tile_h,
                        const float *elev_boundaries, float tile_azim_res, float min_azim,
                        int32_t *tiles_per_gauss) {
    long n = 0;
    for (long idx = 0; idx < total; ++idx) {
        int32_t cnt = 0;
        if (!lidar) {
            const int32_t *r = (const int32_t *)radii;
            if (r[idx * 2] > 0) {
                uint32_t rect[4];
                cam_tile_rect(means2d, r, idx, tile_size, tile_w, tile_h, rect);
                cnt = (int32_t)((rect[3] - rect[1]) * (rect[2] - rect[0]));
            }
        } else {
            const float *r = (const float *)radii;
            if (r[idx * 2] > 0) {
                int32_t rect[4];
                lidar_tile_rect(means2d, r, idx, elev_boundaries, tile_azim_res, min_azim, tile_w,
                                tile_h, rect);
                /* An empty rectangle counts as zero tiles.  With tile columns that span
                 * less than a full turn, a Gaussian that straddles min_azim gets
                 * rect[2] < rect[0]; the reference's product goes negative there
                 * (rasterization.cu:359-361), its cumulative sum and every list entry
                 * behind that Gaussian are then corrupt.  The emission loop below emits
                 * nothing for such a rectangle, so zero is the consistent count. */
                int32_t h = rect[3] - rect[1], w = rect[2] - rect[0];
                cnt = (h > 0 ? h : 0) * (w > 0 ? w : 0);
            }
        }
        tiles_per_gauss[idx] = cnt;
        n += cnt;
    }
    return n;
}

/* Pass 2 (rasterization.cu:65-89, 366-394): emit keys in emission order.
 * key = cid << (32 + tile_n_bits) | tile_id << 32 | bits(depth). */
void oracle_isect_emit(int lidar, long total, long N, const int64_t *camera_ids,
                       const float *means2d, const void *radii, const float *depths,
                       uint32_t tile_size, uint32_t tile_w, uint32_t tile_h,
                       const float *elev_boundaries, float tile_azim_res, float min_azim,
                       int64_t *isect_ids, int32_t *flatten_ids) {
    uint32_t tile_n_bits = bit_width_u32(tile_w * tile_h);
    long cur = 0;
    for (long idx = 0; idx < total; ++idx) {
        int64_t cid = camera_ids ? camera_ids[idx] : idx / N;
        int64_t cid_enc = cid << (32 + tile_n_bits);
        int32_t dbits;
        memcpy(&dbits, depths + idx, 4);
        int64_t depth_enc = (int64_t)dbits; /* sign-extended as in :77 */
        if (!lidar) {
            const int32_t *r = (const int32_t *)radii;
            if (r[idx * 2] <= 0) continue;
            uint32_t rect[4];
            cam_tile_rect(means2d, r, idx, tile_size, tile_w, tile_h, rect);
            for (int32_t i = (int32_t)rect[1]; i < (int32_t)rect[3]; ++i)
                for (int32_t j = (int32_t)rect[0]; j < (int32_t)rect[2]; ++j) {
                    int64_t tile_id = (int64_t)i * tile_w + j;
                    isect_ids[cur] = cid_enc | (tile_id << 32) | depth_enc;
                    flatten_ids[cur] = (int32_t)idx;
                    ++cur;
                }
        } else {
            const float *r = (const float *)radii;
            if (r[idx * 2] <= 0) continue;
            int32_t rect[4];
            lidar_tile_rect(means2d, r, idx, elev_boundaries, tile_azim_res, min_azim, tile_w,
                            tile_h, rect);
            for (int32_t i = rect[1]; i < rect[3]; ++i)
                for (int32_t j = rect[0]; j < rect[2]; ++j) {
                    /* mathematical modulo: identical to (j + n) % n of the reference
                     * (rasterization.cu:384) for j >= -n.  The reference's sum is
                     * unsigned, so for azimuth extents below -360 degrees (j < -n) it
                     * wraps modulo 2^32 first: the same column as here when n is a power
                     * of two, a column shifted by 2^32 mod n otherwise. */
                    int32_t wj = ((j % (int32_t)tile_w) + (int32_t)tile_w) % (int32_t)tile_w;
                    int64_t tile_id = (int64_t)i * tile_w + wj;
                    isect_ids[cur] = cid_enc | (tile_id << 32) | depth_enc;
                    flatten_ids[cur] = (int32_t)idx;
                    ++cur;
                }
        }
    }
}

/* I3: stable ascending sort on key bits [0, end_bit)
 * (rasterization.cu:181-211: cub::DeviceRadixSort::SortPairs).  Implemented
 * as a bottom-up merge sort, which is stable by construction. */
void oracle_sort_pairs(long n, int end_bit, int64_t *keys, int32_t *vals) {
    if (n <= 1) return;
    uint64_t mask = end_bit >= 64 ? ~0ull : ((1ull << end_bit) - 1ull);
    int64_t *kb = (int64_t *)malloc(sizeof(int64_t) * (size_t)n);
    int32_t *vb = (int32_t *)malloc(sizeof(int32_t) * (size_t)n);
    int64_t *ks = keys, *kd = kb;
    int32_t *vs = vals, *vd = vb;
    for (long w = 1; w < n; w *= 2) {
        for (long lo = 0; lo < n; lo += 2 * w) {
            long mid = lo + w < n ? lo + w : n, hi = lo + 2 * w < n ? lo + 2 * w : n;
            long a = lo, b = mid, o = lo;
            while (a < mid && b < hi) {
                if (((uint64_t)ks[b] & mask) < ((uint64_t)ks[a] & mask)) {
                    kd[o] = ks[b]; vd[o] = vs[b]; ++b;
                } else {
                    kd[o] = ks[a]; vd[o] = vs[a]; ++a;
                }
                ++o;
            }
            while (a < mid) { kd[o] = ks[a]; vd[o] = vs[a]; ++a; ++o; }
            while (b < hi) { kd[o] = ks[b]; vd[o] = vs[b]; ++b; ++o; }
        }
        int64_t *tk = ks; ks = kd; kd = tk;
        int32_t *tv = vs; vs = vd; vd = tv;
    }
    if (ks != keys) {
        memcpy(keys, ks, sizeof(int64_t) * (size_t)n);
        memcpy(vals, vs, sizeof(int32_t) * (size_t)n);
    }
    free(kb);
    free(vb);
}

/* I4: isect_offset_encode (rasterization.cu:218-285).  offsets[id] = index of
 * the first sorted intersection whose (cam, tile) >= id; all zero when empty. */
void oracle_isect_offset_encode(long n_isects, const int64_t *isect_ids, uint32_t C,
                                uint32_t n_tiles, int32_t *offsets) {
    uint32_t tile_n_bits = bit_width_u32(n_tiles);
    long total = (long)C * n_tiles;
    if (n_isects == 0) {
        for (long i = 0; i < total; ++i) offsets[i] = 0;
        return;
    }
    long next = 0; /* first offset slot not yet written */
    for (long idx = 0; idx < n_isects; ++idx) {
        int64_t hi = isect_ids[idx] >> 32;
        int64_t cid = hi >> tile_n_bits;
        int64_t tid = hi & ((1 << tile_n_bits) - 1);
        long id = (long)(cid * n_tiles + tid);
        while (next <= id && next < total) offsets[next++] = (int32_t)idx;
    }
    while (next < total) offsets[next++] = (int32_t)n_isects;
}

/* ------------------------------------------------------------------ */
/* Lidar point binning (rasterization.cu:531-833)                       */
/* ------------------------------------------------------------------ */

/* map_points_to_lidar_tiles, rasterization.cu:596-656: one key (camera << 32 | tile) per
 * point, no radius.  The azimuth column is the truncated quotient (wrapped with fmodf only
 * outside [0, 360)), the elevation row the last boundary below the point, found by a linear
 * scan over the first n_tiles_elev boundaries with strict <. */
void oracle_map_points_to_lidar_tiles(long total, long N, const int64_t *camera_ids,
                                      const float *points2d, const float *elev_boundaries,
                                      float tile_azim_res, float min_azim, uint32_t n_tiles_azim,
                                      uint32_t n_tiles_elev, int64_t *tile_ids,
                                      int32_t *flatten_ids) {
    for (long idx = 0; idx < total; ++idx) {
        float tile_elev = points2d[idx * 2 + 1];
        float azim = points2d[idx * 2] - min_azim;
        float tile_azim;
        if (azim >= 0.f && azim < 360.f)
            tile_azim = azim / tile_azim_res;
        else
            tile_azim = fmodf(azim + 360.f, 360.f) / tile_azim_res;
        int32_t x = (int32_t)tile_azim;
        int32_t i = 0;
        while (i < (int32_t)n_tiles_elev && elev_boundaries[i] < tile_elev) ++i;
        int32_t y = i - 1 > 0 ? i - 1 : 0;
        int64_t cid = camera_ids ? camera_ids[idx] : idx / N;
        int64_t tile_id = (int64_t)y * n_tiles_azim + x;
        tile_ids[idx] = (cid << 32) | tile_id;
        flatten_ids[idx] = (int32_t)idx;
    }
}

/* points_mapping_offset_encode, rasterization.cu:531-574: offsets[camera * n_tiles + tile] =
 * index of the first sorted point whose (camera, tile) >= that entry; all zero when empty. */
void oracle_points_mapping_offset_encode(long n_points, const int64_t *point_ids, uint32_t C,
                                         uint32_t n_tiles, int32_t *offsets) {
    long total = (long)C * n_tiles;
    if (n_points == 0) {
        for (long i = 0; i < total; ++i) offsets[i] = 0;
        return;
    }
    long next = 0;
    for (long idx = 0; idx < n_points; ++idx) {
        int64_t cid = point_ids[idx] >> 32;
        int64_t tid = point_ids[idx] & 0xFFFFFFFFll;
        long id = (long)(cid * n_tiles + tid);
        while (next <= id && next < total) offsets[next++] = (int32_t)idx;
    }
    while (next < total) offsets[next++] = (int32_t)n_points;
}

/* populate_image_from_points, rasterization.cu:772-833: the k-th point of a tile's list
 * (k < tile_width * tile_height) lands on the tile's k-th pixel in row-major order, if that
 * pixel is inside the image; everything else stays zero. */
void oracle_populate_image_from_points(uint32_t C, long n_points, const float *points,
                                       uint32_t image_width, uint32_t image_height,
                                       uint32_t tile_width, uint32_t tile_height,
                                       uint32_t grid_w, uint32_t grid_h,
                                       const int32_t *tile_offsets, const int32_t *flatten_ids,
                                       float *image) {
    long n_tiles = (long)grid_w * grid_h;
    for (uint32_t c = 0; c < C; ++c)
        for (long t = 0; t < n_tiles; ++t) {
            long start = tile_offsets[c * n_tiles + t];
            long end = (c == C - 1 && t == n_tiles - 1) ? n_points : tile_offsets[c * n_tiles + t + 1];
            long cap = start + (long)tile_width * tile_height;
            if (end > cap) end = cap;
            for (long k = start; k < end; ++k) {
                long tr = k - start;
                uint32_t i = (uint32_t)(t / grid_w) * tile_height + (uint32_t)(tr / tile_width);
                uint32_t j = (uint32_t)(t % grid_w) * tile_width + (uint32_t)(tr % tile_width);
                if (i >= image_height || j >= image_width) continue;
                const float *src = points + (long)flatten_ids[k] * 5;
                float *dst = image + (((long)c * image_height + i) * image_width + j) * 5;
                for (int q = 0; q < 5; ++q) dst[q] = src[q];
            }
        }
}

/* compute_relocation, gsplat/cuda/csrc/relocation.cu:4-30: powers and square root in double
 * (pow / sqrt on mixed arguments promote), sum in float. */
void oracle_compute_relocation(long N, const float *opacities, const float *scales,
                               const int32_t *ratios, const float *binoms, int n_max,
                               float *new_opacities, float *new_scales) {
    for (long idx = 0; idx < N; ++idx) {
        int n_idx = ratios[idx];
        float denom_sum = 0.0f;
        new_opacities[idx] = 1.0f - powf(1.0f - opacities[idx], 1.0f / n_idx);
        for (int i = 1; i <= n_idx; ++i)
            for (int k = 0; k <= i - 1; ++k) {
                float bin_coeff = binoms[(long)(i - 1) * n_max + k];
                float term = (float)((pow(-1.0, k) / sqrt((double)(float)(k + 1))) *
                                     pow((double)new_opacities[idx], k + 1));
                denom_sum += bin_coeff * term;
            }
        float coeff = opacities[idx] / denom_sum;
        for (int q = 0; q < 3; ++q) new_scales[idx * 3 + q] = coeff * scales[idx * 3 + q];
    }
}

#endif /* !ORACLE_F64 */

/* The discontinuous decisions of the compositing rule.  The values are the reference's
 * (rasterization.cu:1476-1488, 2186-2197): a Gaussian is skipped below alpha = 1/255, a
 * pixel stops when its transmittance would fall to 1e-4 or below, the median depth is
 * taken where the transmittance crosses 0.5, alpha is summed while the Gaussian lies
 * in front of range - threshold.  A float32 implementation whose alpha or transmittance
 * differs from this file's in the last bits takes the other branch for inputs within
 * rounding distance of a threshold.  Parity tests find exactly those pixels by rendering
 * again with the thresholds moved by a few rounding errors (set_thresholds); with the
 * defaults below the functions restate the reference. */
static real g_alpha_min = RC(1) / RC(255);
static real g_T_min = RC(1e-4);
static real g_median_T = RC(0.5);
static real g_asum_shift = RC(0);

void NAME(set_thresholds)(double alpha_scale, double t_scale, double median_scale,
                          double asum_shift) {
    g_alpha_min = (real)(alpha_scale * (1.0 / 255.0));
    if (alpha_scale == 1.0) g_alpha_min = RC(1) / RC(255);
    g_T_min = t_scale == 1.0 ? RC(1e-4) : (real)(t_scale * 1e-4);
    g_median_T = median_scale == 1.0 ? RC(0.5) : (real)(median_scale * 0.5);
    g_asum_shift = (real)asum_shift;
}

/* ------------------------------------------------------------------ */
/* R1: rasterize_to_pixels forward (rasterization.cu:1360-1518)          */
/* One scalar loop per pixel over its tile's sorted list.                */
/* ------------------------------------------------------------------ */
void NAME(rasterize_to_pixels_fwd)(int C, long n_isects, int D, const float *means2d,
                                   const float *conics, const float *colors,
                                   const float *opacities, const float *pix_vels,
                                   const float *rs_time, const float *backgrounds, int W, int H,
                                   int tile_size, int tile_w, int tile_h,
                                   const int32_t *tile_offsets, const int32_t *flatten_ids,
                                   real *render_colors, real *render_alphas, int32_t *last_ids) {
    long n_tiles = (long)tile_w * tile_h;
#pragma omp parallel for schedule(dynamic, 64)
    for (long pix = 0; pix < (long)C * H * W; ++pix) {
        int cid = (int)(pix / ((long)H * W));
        long rem = pix % ((long)H * W);
        int i = (int)(rem / W), j = (int)(rem % W);
        long tile_id = (long)(i / tile_size) * tile_w + (j / tile_size);
        long t_glob = cid * n_tiles + tile_id;
        long start = tile_offsets[t_glob];
        long end = (cid == C - 1 && tile_id == n_tiles - 1) ? n_isects : tile_offsets[t_glob + 1];
        real px = (real)j + RC(0.5), py = (real)i + RC(0.5);
        /* rasterization.cu:1401 */
        real roll = RC(rs_time[cid]) * ((py - RC(0.5)) / (real)(H - 1) - RC(0.5));
        real T = 1;
        long cur_idx = 0;
        real *out = render_colors + pix * D;
        for (int k = 0; k < D; ++k) out[k] = 0;
        for (long s = start; s < end; ++s) {
            long g = flatten_ids[s];
            real dx = RC(means2d[g * 2]) + roll * RC(pix_vels[g * 2]) - px;
            real dy = RC(means2d[g * 2 + 1]) + roll * RC(pix_vels[g * 2 + 1]) - py;
            real ca = conics[g * 3], cb = conics[g * 3 + 1], cc = conics[g * 3 + 2];
            real sigma = RC(0.5) * (ca * dx * dx + cc * dy * dy) + cb * dx * dy;
            real alpha = R_FMIN(RC(0.999), RC(opacities[g]) * R_EXP(-sigma));
            if (sigma < 0 || alpha < g_alpha_min) continue;
            real next_T = T * (RC(1) - alpha);
            if (next_T <= g_T_min) break; /* exclusive: :1485-1488 */
            real vis = alpha * T;
            const float *c = colors + g * D;
            for (int k = 0; k < D; ++k) out[k] += RC(c[k]) * vis;
            cur_idx = s;
            T = next_T;
        }
        render_alphas[pix] = RC(1) - T;
        if (backgrounds)
            for (int k = 0; k < D; ++k) out[k] += T * RC(backgrounds[cid * D + k]);
        last_ids[pix] = (int32_t)cur_idx;
    }
}

/* utils.cuh:552-555 */
static real angle_difference(real a, real b) {
    real d = R_FMOD(a - b + RC(180), RC(360)) - RC(180);
    return d < RC(-180) ? d + RC(360) : d;
}

/* ------------------------------------------------------------------ */
/* R3: rasterize_to_points forward (rasterization.cu:2021-2219)          */
/* ------------------------------------------------------------------ */
void NAME(rasterize_to_points_fwd)(int C, long n_isects, int D, const float *means2d,
                                   const float *conics, const float *colors,
                                   const float *opacities, const float *pix_vels,
                                   const float *depth_comps, const float *backgrounds,
                                   const float *raster_pts, int W, int H, int tile_width,
                                   int tile_height, int grid_w, int grid_h, int compute_alpha_sum,
                                   float alpha_sum_threshold, const int32_t *tile_offsets,
                                   const int32_t *flatten_ids, int depth_idx, real *render_colors,
                                   real *render_alphas, real *alpha_sum, int32_t *last_ids,
                                   real *median_depths) {
    long n_tiles = (long)grid_w * grid_h;
#pragma omp parallel for schedule(dynamic, 64)
    for (long pix = 0; pix < (long)C * H * W; ++pix) {
        int cid = (int)(pix / ((long)H * W));
        long rem = pix % ((long)H * W);
        int i = (int)(rem / W), j = (int)(rem % W);
        real *out = render_colors + pix * D;
        for (int k = 0; k < D; ++k) out[k] = 0;
        render_alphas[pix] = 0;
        median_depths[pix] = 0;
        if (alpha_sum) alpha_sum[pix] = 0;
        last_ids[pix] = 0;
        const float *rp = raster_pts + pix * 4;
        real px = rp[0], py = rp[1], pz = rp[2], roll = rp[3];
        if (pz <= 0) continue; /* :2087-2089: outputs stay zero */
        long tile_id = (long)(i / tile_height) * grid_w + (j / tile_width);
        long t_glob = cid * n_tiles + tile_id;
        long start = tile_offsets[t_glob];
        long end = (cid == C - 1 && tile_id == n_tiles - 1) ? n_isects : tile_offsets[t_glob + 1];
        real T = 1, asum = 0;
        long cur_idx = 0;
        for (long s = start; s < end; ++s) {
            long g = flatten_ids[s];
            real vx = pix_vels[g * 3], vy = pix_vels[g * 3 + 1], vz = pix_vels[g * 3 + 2];
            real dx = angle_difference(RC(means2d[g * 2]) + roll * vx, px);
            real dy = angle_difference(RC(means2d[g * 2 + 1]) + roll * vy, py);
            real ca = conics[g * 3], cb = conics[g * 3 + 1], cc = conics[g * 3 + 2];
            real sigma = RC(0.5) * (ca * dx * dx + cc * dy * dy) + cb * dx * dy;
            real alpha = R_FMIN(RC(0.999), RC(opacities[g]) * R_EXP(-sigma));
            if (sigma < 0 || alpha < g_alpha_min) continue;
            real next_T = T * (RC(1) - alpha);
            if (next_T <= g_T_min) break;
            real vis = alpha * T;
            const float *c = colors + g * D;
            for (int k = 0; k < D; ++k) out[k] += RC(c[k]) * vis;
            real extra = RC(depth_comps[g * 2]) * dx + RC(depth_comps[g * 2 + 1]) * dy + vz * roll;
            out[depth_idx] += extra * vis; /* :2184-2185 */
            if (T > g_median_T && next_T <= g_median_T) median_depths[pix] = RC(c[depth_idx]) + extra;
            if (compute_alpha_sum && RC(c[depth_idx]) < pz - RC(alpha_sum_threshold) + g_asum_shift) asum += alpha;
            cur_idx = s;
            T = next_T;
        }
        render_alphas[pix] = RC(1) - T;
        if (backgrounds)
            for (int k = 0; k < D; ++k) out[k] += T * RC(backgrounds[cid * D + k]);
        if (alpha_sum) alpha_sum[pix] = asum;
        last_ids[pix] = (int32_t)cur_idx;
    }
}

/* ------------------------------------------------------------------ */
/* (Gaussian, pixel) index lists: rasterize_to_indices_in_range_kernel   */
/* (rasterization.cu:839-1001) and its lidar twin (:1100-1268).          */
/* One scalar loop per pixel over batches [range_start, range_end) of    */
/* its tile's list, a batch being tile_width * tile_height entries; the  */
/* pixel starts from transmittances[pix].  With chunk_starts == NULL the */
/* pairs of every pixel are counted into counts[pix]; otherwise they are */
/* written from chunk_starts[pix] on (the reference's two passes,        */
/* :1054-1090).  lidar: sensor = raster_pts [C,H,W,4], points with       */
/* range <= 0 take nothing (:1218-1222); camera: sensor = rolling        */
/* shutter time [C].                                                     */
/* ------------------------------------------------------------------ */
void NAME(rasterize_to_indices_in_range)(int lidar, long range_start, long range_end, int C,
                                         long N, long n_isects, const float *transmittances,
                                         const float *means2d, const float *conics,
                                         const float *opacities, const float *pix_vels,
                                         const float *sensor, int W, int H, int tile_width,
                                         int tile_height, int grid_w, int grid_h,
                                         const int32_t *tile_offsets, const int32_t *flatten_ids,
                                         int32_t *counts, const int64_t *chunk_starts,
                                         int64_t *gaussian_ids, int64_t *indices) {
    long n_tiles = (long)grid_w * grid_h;
    long block = (long)tile_width * tile_height;
    int vs = lidar ? 3 : 2;
#pragma omp parallel for schedule(dynamic, 64)
    for (long pix = 0; pix < (long)C * H * W; ++pix) {
        int cid = (int)(pix / ((long)H * W));
        long rem = pix % ((long)H * W);
        int i = (int)(rem / W), j = (int)(rem % W);
        long tile_id = (long)(i / tile_height) * grid_w + (j / tile_width);
        long t_glob = cid * n_tiles + tile_id;
        long start = tile_offsets[t_glob];
        long end = (cid == C - 1 && tile_id == n_tiles - 1) ? n_isects : tile_offsets[t_glob + 1];
        long num_batches = (end - start + block - 1) / block;
        long b_end = range_end < num_batches ? range_end : num_batches;
        long cnt = 0;
        real px, py, roll;
        int active = 1;
        if (lidar) {
            const float *rp = sensor + pix * 4;
            px = rp[0]; py = rp[1]; roll = rp[3];
            active = rp[2] > 0;
        } else {
            px = (real)j + RC(0.5); py = (real)i + RC(0.5);
            roll = RC(sensor[cid]) * ((py - RC(0.5)) / (real)(H - 1) - RC(0.5)); /* :876 */
        }
        real T = transmittances[pix];
        if (active && range_start < num_batches) {
            long s_end = start + b_end * block < end ? start + b_end * block : end;
            for (long s = start + range_start * block; s < s_end; ++s) {
                long g = flatten_ids[s];
                real dx = RC(means2d[g * 2]) + roll * RC(pix_vels[g * vs]);
                real dy = RC(means2d[g * 2 + 1]) + roll * RC(pix_vels[g * vs + 1]);
                if (lidar) { dx = angle_difference(dx, px); dy = angle_difference(dy, py); }
                else { dx -= px; dy -= py; }
                real ca = conics[g * 3], cb = conics[g * 3 + 1], cc = conics[g * 3 + 2];
                real sigma = RC(0.5) * (ca * dx * dx + cc * dy * dy) + cb * dx * dy;
                real alpha = R_FMIN(RC(0.999), RC(opacities[g]) * R_EXP(-sigma));
                if (sigma < 0 || alpha < RC(1) / RC(255)) continue;
                real next_T = T * (RC(1) - alpha);
                if (next_T <= RC(1e-4)) break;
                if (chunk_starts) {
                    gaussian_ids[chunk_starts[pix] + cnt] = g % N;
                    indices[chunk_starts[pix] + cnt] = pix;
                }
                ++cnt;
                T = next_T;
            }
        }
        if (!chunk_starts) counts[pix] = (int32_t)cnt;
    }
}

int NAME(sizeof_real)(void) { return (int)sizeof(real); }
