// Vector-Jacobian products of the fused camera and lidar projections for gfx950.
//
// The forward quantities of every (sensor, Gaussian) pair that survived the forward culls (or
// of every packed row) are recomputed from the inputs; the chain rule is written with
// explicit symmetric Hessians of the sensor mappings:
//   camera:  J = d(pixel)/d(p) with the field-of-view clamp of the forward pass,
//   lidar:   J = d(azimuth deg, elevation deg, range)/d(p); every dependence of J on p
//            (projected covariance, depth compensation, spherical velocity) is collected
//            into one cotangent v_J and contracted once with the three Hessians.
// Semantics follow gsplat/cuda/csrc/projection.cu:753-964, :1466-1716 and :2419-2629 of the
// reference (no gradient to the intrinsics or to the sensor velocities).  Additionally the
// gradient of the per-Gaussian world velocities is returned when asked for.
//
// Accumulation.  Unpacked input: one lane per Gaussian walks over the sensors, sums the
// gradients that reach the Gaussian in registers and stores them once (no atomics, no
// cleared outputs, the same bits on every run).  Packed input: one lane per row, one atomic
// add per row and component (or a plain store when sparse gradients are asked for).  The
// pose gradient is summed over the wavefront first when all its lanes share the sensor.
#include "common.h"

#define RAD_TO_DEG 57.2957795131f

namespace {

struct Sym2 { float xx, xy, yy; };

// Gradient w.r.t. the blurred 2x2 covariance from the gradients of conic (its inverse,
// upper triangle, off-diagonal counted once) and of the compensation factor.
__device__ __forceinline__ Sym2 conic_and_compensation_vjp(float ca, float cb, float cc,
                                                           float va, float vb, float vc,
                                                           bool has_comp, float comp, float v_comp,
                                                           float eps2d) {
    // v_S = -P v_P P with P = [[ca, cb], [cb, cc]], v_P = [[va, vb/2], [vb/2, vc]]
    const float h = 0.5f * vb;
    const float m00 = va * ca + h * cb, m01 = va * cb + h * cc; // v_P P
    const float m10 = h * ca + vc * cb, m11 = h * cb + vc * cc;
    Sym2 g;
    g.xx = -(ca * m00 + cb * m10);
    const float g01 = -(ca * m01 + cb * m11);
    const float g10 = -(cb * m00 + cc * m10);
    g.yy = -(cb * m01 + cc * m11);
    g.xy = 0.5f * (g01 + g10); // kept as the symmetric part; used as v_S[0][1] = v_S[1][0]
    if (has_comp) {
        // comp = sqrt(det(S - eps I) / det(S)):  d(comp^2)/dS = (1 - comp^2) P - eps det(P) I
        const float det_p = ca * cc - cb * cb;
        const float v_sqr = v_comp * 0.5f / (comp + 1e-6f);
        const float om = 1.f - comp * comp;
        g.xx += v_sqr * (om * ca - eps2d * det_p);
        g.xy += v_sqr * (om * cb);
        g.yy += v_sqr * (om * cc - eps2d * det_p);
    }
    return g;
}

struct GaussianCov {
    Mat3 Rq;        // rotation of the quaternion (quat/scale input only)
    float s[3];     // scales
    float q[4];     // raw quaternion (w, x, y, z)
    Mat3 cov;       // world covariance
    bool from_quat;
};

__device__ __forceinline__ GaussianCov load_cov(uint32_t gid, const float *__restrict__ covars,
                                                const float *__restrict__ quats,
                                                const float *__restrict__ scales) {
    GaussianCov gc;
    if (covars != nullptr) {
        const float *c = covars + (size_t)gid * 6;
        gc.cov.m[0] = c[0]; gc.cov.m[1] = c[1]; gc.cov.m[2] = c[2];
        gc.cov.m[3] = c[1]; gc.cov.m[4] = c[3]; gc.cov.m[5] = c[4];
        gc.cov.m[6] = c[2]; gc.cov.m[7] = c[4]; gc.cov.m[8] = c[5];
        gc.from_quat = false;
    } else {
        const float4 q = *reinterpret_cast<const float4 *>(quats + (size_t)gid * 4);
        gc.q[0] = q.x; gc.q[1] = q.y; gc.q[2] = q.z; gc.q[3] = q.w;
        gc.s[0] = scales[(size_t)gid * 3]; gc.s[1] = scales[(size_t)gid * 3 + 1]; gc.s[2] = scales[(size_t)gid * 3 + 2];
        gc.Rq = quat_to_rotmat(q.x, q.y, q.z, q.w);
        Mat3 M;
#pragma unroll
        for (int i = 0; i < 3; ++i)
#pragma unroll
            for (int j = 0; j < 3; ++j) M.m[i * 3 + j] = gc.Rq.m[i * 3 + j] * gc.s[j];
        gc.cov = mat3_mul_bt(M, M);
        gc.from_quat = true;
    }
    return gc;
}

// Gradients of (quat, scale) from the gradient G of the world covariance Sigma = M M^T,
// M = R(q) diag(s).
__device__ __forceinline__ void quat_scale_vjp(const GaussianCov &gc, const Mat3 &G, float vq[4],
                                               float vs[3]) {
    Mat3 Gs; // G + G^T
#pragma unroll
    for (int i = 0; i < 3; ++i)
#pragma unroll
        for (int j = 0; j < 3; ++j) Gs.m[i * 3 + j] = G.m[i * 3 + j] + G.m[j * 3 + i];
    Mat3 M;
#pragma unroll
    for (int i = 0; i < 3; ++i)
#pragma unroll
        for (int j = 0; j < 3; ++j) M.m[i * 3 + j] = gc.Rq.m[i * 3 + j] * gc.s[j];
    const Mat3 vM = mat3_mul(Gs, M);
    Mat3 vR;
#pragma unroll
    for (int j = 0; j < 3; ++j) {
        float acc = 0.f;
#pragma unroll
        for (int i = 0; i < 3; ++i) {
            acc += gc.Rq.m[i * 3 + j] * vM.m[i * 3 + j];
            vR.m[i * 3 + j] = vM.m[i * 3 + j] * gc.s[j];
        }
        vs[j] = acc;
    }
    // d R(q_n) / d q_n
    const float inv = rsqrtf(gc.q[0] * gc.q[0] + gc.q[1] * gc.q[1] + gc.q[2] * gc.q[2] + gc.q[3] * gc.q[3]);
    const float w = gc.q[0] * inv, x = gc.q[1] * inv, y = gc.q[2] * inv, z = gc.q[3] * inv;
    const float *g = vR.m;
    float vn[4];
    vn[0] = 2.f * (x * (g[7] - g[5]) + y * (g[2] - g[6]) + z * (g[3] - g[1]));
    vn[1] = 2.f * (-2.f * x * (g[4] + g[8]) + y * (g[1] + g[3]) + z * (g[2] + g[6]) + w * (g[7] - g[5]));
    vn[2] = 2.f * (x * (g[1] + g[3]) - 2.f * y * (g[0] + g[8]) + z * (g[5] + g[7]) + w * (g[2] - g[6]));
    vn[3] = 2.f * (x * (g[2] + g[6]) + y * (g[5] + g[7]) - 2.f * z * (g[0] + g[4]) + w * (g[3] - g[1]));
    const float qn[4] = {w, x, y, z};
    const float dot = vn[0] * w + vn[1] * x + vn[2] * y + vn[3] * z;
#pragma unroll
    for (int i = 0; i < 4; ++i) vq[i] = (vn[i] - dot * qn[i]) * inv;
}

struct PoseGrad {
    Mat3 vR;
    float vt[3];
};

struct BwdOutputs {
    float *v_means, *v_covars, *v_quats, *v_scales, *v_viewmats, *v_velocities;
};

// What one (sensor, Gaussian) pair sends back: to the Gaussian's mean, world covariance and
// velocity, and to the sensor pose.
struct PairGrad {
    float v_mean[3];
    Mat3 v_cov;
    float v_vel[3];
    PoseGrad pg;
};

__device__ __forceinline__ PairGrad pair_grad_zero() {
    PairGrad g;
#pragma unroll
    for (int i = 0; i < 3; ++i) g.v_mean[i] = g.v_vel[i] = g.pg.vt[i] = 0.f;
    g.v_cov = mat3_zero();
    g.pg.vR = mat3_zero();
    return g;
}

// Writes the gradients of a Gaussian to row `row` of the outputs (the Gaussian id, or the
// packed row for sparse gradients).  ADD: atomic adds into cleared outputs; otherwise stores.
// The velocity gradient always belongs to the Gaussian `gid`.
template <bool ADD>
__device__ __forceinline__ void emit_gaussian(const BwdOutputs &o, bool store_velocity, uint32_t row,
                                              uint32_t gid, const GaussianCov &gc, const PairGrad &g) {
    auto put = [](float *p, float v) { if (ADD) atomicAdd(p, v); else *p = v; };
    float *vm = o.v_means + (size_t)row * 3;
#pragma unroll
    for (int i = 0; i < 3; ++i) put(vm + i, g.v_mean[i]);
    if (o.v_covars != nullptr) {
        const float c6[6] = {g.v_cov.m[0], g.v_cov.m[1] + g.v_cov.m[3], g.v_cov.m[2] + g.v_cov.m[6],
                             g.v_cov.m[4], g.v_cov.m[5] + g.v_cov.m[7], g.v_cov.m[8]};
        float *vc = o.v_covars + (size_t)row * 6;
#pragma unroll
        for (int i = 0; i < 6; ++i) put(vc + i, c6[i]);
    } else {
        float vq[4], vs[3];
        quat_scale_vjp(gc, g.v_cov, vq, vs);
        float *pq = o.v_quats + (size_t)row * 4, *ps = o.v_scales + (size_t)row * 3;
#pragma unroll
        for (int i = 0; i < 4; ++i) put(pq + i, vq[i]);
#pragma unroll
        for (int i = 0; i < 3; ++i) put(ps + i, vs[i]);
    }
    if (o.v_velocities != nullptr && store_velocity) {
        float *vv = o.v_velocities + (size_t)gid * 3;
#pragma unroll
        for (int i = 0; i < 3; ++i) put(vv + i, g.v_vel[i]);
    }
}

// Adds a pair's pose gradient to v_viewmats (cleared by the caller).  All lanes of the
// wavefront arrive here; inactive ones carry nothing.
__device__ __forceinline__ void emit_pose(const BwdOutputs &o, bool active, uint32_t cid,
                                          const PoseGrad &pg) {
    if (o.v_viewmats == nullptr) return;
    const uint32_t first_cid = __shfl(cid, 0, SPLATAD_WAVE);
    const bool uniform = __all(cid == first_cid);
    float vals[12];
#pragma unroll
    for (int i = 0; i < 3; ++i) {
#pragma unroll
        for (int j = 0; j < 3; ++j) vals[i * 4 + j] = active ? pg.vR.m[i * 3 + j] : 0.f;
        vals[i * 4 + 3] = active ? pg.vt[i] : 0.f;
    }
    if (uniform) {
#pragma unroll
        for (int i = 0; i < 12; ++i) vals[i] = wave_sum(vals[i]);
        if ((threadIdx.x & (SPLATAD_WAVE - 1)) == 0) {
#pragma unroll
            for (int i = 0; i < 12; ++i)
                if (vals[i] != 0.f) atomicAdd(o.v_viewmats + (size_t)first_cid * 16 + i, vals[i]);
        }
    } else if (active) {
#pragma unroll
        for (int i = 0; i < 12; ++i) atomicAdd(o.v_viewmats + (size_t)cid * 16 + i, vals[i]);
    }
}

// Shared tail of both kernels: pose and covariance chain rule from the sensor-frame
// gradients (v_pc, v_cov_c) back to world-frame inputs.
__device__ __forceinline__ void sensor_to_world_vjp(const Mat3 &R, const float *__restrict__ p_world,
                                                    const Mat3 &cov, const float v_pc[3],
                                                    const Mat3 &v_cov_c, float v_mean[3],
                                                    Mat3 &v_cov, PoseGrad &pg) {
    // p_c = R p + t
#pragma unroll
    for (int i = 0; i < 3; ++i) {
        pg.vt[i] = v_pc[i];
        v_mean[i] = R.m[i] * v_pc[0] + R.m[3 + i] * v_pc[1] + R.m[6 + i] * v_pc[2];
#pragma unroll
        for (int j = 0; j < 3; ++j) pg.vR.m[i * 3 + j] += v_pc[i] * p_world[j];
    }
    // cov_c = R cov R^T:  v_cov = R^T G R,  v_R += G R cov^T + G^T R cov
    v_cov = mat3_mul(mat3_mul_at(R, v_cov_c), R);
    const Mat3 Rc = mat3_mul(R, cov); // cov symmetric: R cov^T = R cov
    const Mat3 a = mat3_mul(v_cov_c, Rc);
    const Mat3 b = mat3_mul_at(v_cov_c, Rc);
#pragma unroll
    for (int i = 0; i < 9; ++i) pg.vR.m[i] += a.m[i] + b.m[i];
}

struct CamArgs {
    uint32_t C, N;
    const float *means, *covars, *quats, *scales, *velocities, *viewmats, *Ks;
    uint32_t W, H;
    const float *lin_vel, *ang_vel, *rs_time;
    float eps2d;
    const int64_t *camera_ids, *gaussian_ids;
    int64_t nnz;
    const int32_t *radii;
    const float *conics, *compensations, *v_means2d, *v_depths, *v_conics, *v_compensations, *v_pix_vels;
    int sparse_grad;
    BwdOutputs out;
};

// The gradients of the pair (sensor cid, Gaussian gid); idx is the pair's row in the
// per-pair tensors, pw the Gaussian's mean, gc its covariance.
__device__ __forceinline__ PairGrad camera_pair_vjp(const CamArgs &a, uint64_t idx, uint32_t cid,
                                                    uint32_t gid, const float pw[3],
                                                    const GaussianCov &gc) {
    PairGrad g = pair_grad_zero();
    const float *vm = a.viewmats + cid * 16;
    Mat3 R;
    R.m[0] = vm[0]; R.m[1] = vm[1]; R.m[2] = vm[2];
    R.m[3] = vm[4]; R.m[4] = vm[5]; R.m[5] = vm[6];
    R.m[6] = vm[8]; R.m[7] = vm[9]; R.m[8] = vm[10];
    float pc[3];
#pragma unroll
    for (int i = 0; i < 3; ++i) pc[i] = R.m[i * 3] * pw[0] + R.m[i * 3 + 1] * pw[1] + R.m[i * 3 + 2] * pw[2] + vm[i * 4 + 3];
    const Mat3 cov_c = mat3_mul_bt(mat3_mul(R, gc.cov), R);

    const float *K = a.Ks + cid * 9;
    const float fx = K[0], fy = K[4], cx = K[2], cy = K[5];
    const float x = pc[0], y = pc[1], z = pc[2];
    const float tan_fovx = 0.5f * (float)a.W / fx, tan_fovy = 0.5f * (float)a.H / fy;
    const float lim_x_pos = ((float)a.W - cx) / fx + 0.3f * tan_fovx;
    const float lim_x_neg = cx / fx + 0.3f * tan_fovx;
    const float lim_y_pos = ((float)a.H - cy) / fy + 0.3f * tan_fovy;
    const float lim_y_neg = cy / fy + 0.3f * tan_fovy;
    const float rz = 1.f / z, rz2 = rz * rz, rz3 = rz2 * rz;
    const bool x_in = (x * rz <= lim_x_pos && x * rz >= -lim_x_neg);
    const bool y_in = (y * rz <= lim_y_pos && y * rz >= -lim_y_neg);
    const float tx = z * fminf(lim_x_pos, fmaxf(-lim_x_neg, x * rz));
    const float ty = z * fminf(lim_y_pos, fmaxf(-lim_y_neg, y * rz));
    const float J00 = fx * rz, J02 = -fx * tx * rz2, J11 = fy * rz, J12 = -fy * ty * rz2;

    const float *cn = a.conics + idx * 3;
    const float *vcn = a.v_conics + idx * 3;
    const bool has_comp = a.v_compensations != nullptr;
    const Sym2 g2 = conic_and_compensation_vjp(cn[0], cn[1], cn[2], vcn[0], vcn[1], vcn[2], has_comp,
                                               has_comp ? a.compensations[idx] : 0.f,
                                               has_comp ? a.v_compensations[idx] : 0.f, a.eps2d);
    float v_pc[3] = {0.f, 0.f, 0.f};
    // cotangent of J (2x3); entries (0,1) and (1,0) of J are constant zeros
    float vJ00 = 0.f, vJ02 = 0.f, vJ11 = 0.f, vJ12 = 0.f;

    // rolling shutter: pix_vel = -J tv, tv = v_lin + omega x p - R v_gaussian
    const float rs = a.rs_time[cid];
    if (rs > 0.f) {
        const float *lv = a.lin_vel + cid * 3, *av = a.ang_vel + cid * 3;
        float tv[3] = {lv[0] + (av[1] * pc[2] - av[2] * pc[1]), lv[1] + (av[2] * pc[0] - av[0] * pc[2]),
                       lv[2] + (av[0] * pc[1] - av[1] * pc[0])};
        float vw[3] = {0.f, 0.f, 0.f};
        if (a.velocities != nullptr) {
                        vw[0] = a.velocities[(size_t)gid * 3]; vw[1] = a.velocities[(size_t)gid * 3 + 1]; vw[2] = a.velocities[(size_t)gid * 3 + 2];
#pragma unroll
            for (int i = 0; i < 3; ++i) tv[i] -= R.m[i * 3] * vw[0] + R.m[i * 3 + 1] * vw[1] + R.m[i * 3 + 2] * vw[2];
        }
        const float vpx = a.v_pix_vels[idx * 2], vpy = a.v_pix_vels[idx * 2 + 1];
        // through J
        vJ00 += -vpx * tv[0]; vJ02 += -vpx * tv[2];
        vJ11 += -vpy * tv[1]; vJ12 += -vpy * tv[2];
        // through tv: v_tv = -J^T v_pv
        const float vtv[3] = {-J00 * vpx, -J11 * vpy, -(J02 * vpx + J12 * vpy)};
        // tv = ... + omega x p  ->  v_p += -(omega x v_tv)
        v_pc[0] += -(av[1] * vtv[2] - av[2] * vtv[1]);
        v_pc[1] += -(av[2] * vtv[0] - av[0] * vtv[2]);
        v_pc[2] += -(av[0] * vtv[1] - av[1] * vtv[0]);
        if (a.velocities != nullptr) {
            // tv = ... - R v_w:  v_R -= v_tv v_w^T,  v_vw = -R^T v_tv
#pragma unroll
            for (int i = 0; i < 3; ++i) {
#pragma unroll
                for (int j = 0; j < 3; ++j) g.pg.vR.m[i * 3 + j] += -vtv[i] * vw[j];
                g.v_vel[i] = -(R.m[i] * vtv[0] + R.m[3 + i] * vtv[1] + R.m[6 + i] * vtv[2]);
            }
        }
    }

    // cov2d = J cov_c J^T with cotangent g2 (symmetric)
    const float *S = cov_c.m;
    // v_cov_c = J^T g2 J
    Mat3 v_cov_c;
    {
        const float Jr0[3] = {J00, 0.f, J02}, Jr1[3] = {0.f, J11, J12};
#pragma unroll
        for (int i = 0; i < 3; ++i)
#pragma unroll
            for (int j = 0; j < 3; ++j)
                v_cov_c.m[i * 3 + j] = Jr0[i] * (g2.xx * Jr0[j] + g2.xy * Jr1[j]) + Jr1[i] * (g2.xy * Jr0[j] + g2.yy * Jr1[j]);
        // v_J = 2 g2 J cov_c (g2 and cov_c symmetric)
        float JS0[3], JS1[3];
#pragma unroll
        for (int j = 0; j < 3; ++j) {
            JS0[j] = Jr0[0] * S[j] + Jr0[2] * S[6 + j];
            JS1[j] = Jr1[1] * S[3 + j] + Jr1[2] * S[6 + j];
        }
        vJ00 += 2.f * (g2.xx * JS0[0] + g2.xy * JS1[0]);
        vJ02 += 2.f * (g2.xx * JS0[2] + g2.xy * JS1[2]);
        vJ11 += 2.f * (g2.xy * JS0[1] + g2.yy * JS1[1]);
        vJ12 += 2.f * (g2.xy * JS0[2] + g2.yy * JS1[2]);
    }
    // J(p): J00 = fx/z, J11 = fy/z, J02 = -fx tx/z^2, J12 = -fy ty/z^2
    if (x_in) v_pc[0] += -fx * rz2 * vJ02; else v_pc[2] += -fx * rz3 * vJ02 * tx;
    if (y_in) v_pc[1] += -fy * rz2 * vJ12; else v_pc[2] += -fy * rz3 * vJ12 * ty;
    v_pc[2] += -fx * rz2 * vJ00 - fy * rz2 * vJ11 + 2.f * fx * tx * rz3 * vJ02 + 2.f * fy * ty * rz3 * vJ12;
    // mean2d = (fx x/z + cx, fy y/z + cy), depth = z
    const float vm0 = a.v_means2d[idx * 2], vm1 = a.v_means2d[idx * 2 + 1];
    v_pc[0] += fx * rz * vm0;
    v_pc[1] += fy * rz * vm1;
    v_pc[2] += -(fx * x * vm0 + fy * y * vm1) * rz2 + a.v_depths[idx];

    sensor_to_world_vjp(R, pw, gc.cov, v_pc, v_cov_c, g.v_mean, g.v_cov, g.pg);
    return g;
}

// Adds b's per-Gaussian parts to a.
__device__ __forceinline__ void pair_grad_add(PairGrad &a, const PairGrad &b) {
#pragma unroll
    for (int i = 0; i < 3; ++i) { a.v_mean[i] += b.v_mean[i]; a.v_vel[i] += b.v_vel[i]; }
#pragma unroll
    for (int i = 0; i < 9; ++i) a.v_cov.m[i] += b.v_cov.m[i];
}

// The driver of both kernels.  GATHER: unpacked input, lane = Gaussian, loop over the sensors.
// Otherwise lane = packed row.  pair(idx, cid, gid, pw, gc) gives a pair's gradients,
// visible(idx) tells whether an unpacked pair survived the forward culls.
template <bool GATHER, typename Args, typename Visible, typename Pair>
__device__ __forceinline__ void projection_bwd_driver(const Args &a, const int64_t *camera_ids,
                                                      const int64_t *gaussian_ids, uint64_t rows,
                                                      bool sparse_grad, Visible &&visible,
                                                      Pair &&pair) {
    const uint64_t t = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const bool mine = t < (GATHER ? (uint64_t)a.N : rows);
    // lanes past the end stay for the wavefront sums of the pose gradient; they read row 0
    const uint32_t gid = !mine ? 0u : GATHER ? (uint32_t)t : (uint32_t)gaussian_ids[t];
    const float pw[3] = {a.means[(size_t)gid * 3], a.means[(size_t)gid * 3 + 1], a.means[(size_t)gid * 3 + 2]};
    const GaussianCov gc = load_cov(gid, a.covars, a.quats, a.scales);
    if (GATHER) {
        PairGrad sum = pair_grad_zero();
        for (uint32_t cid = 0; cid < a.C; ++cid) { // uniform
            const uint64_t idx = (uint64_t)cid * a.N + gid;
            const bool active = mine && visible(idx);
            PairGrad g = pair_grad_zero();
            if (active) g = pair(idx, cid, gid, pw, gc);
            pair_grad_add(sum, g);
            emit_pose(a.out, active, cid, g.pg);
        }
        if (mine) emit_gaussian<false>(a.out, true, gid, gid, gc, sum);
    } else {
        const uint32_t cid = mine ? (uint32_t)camera_ids[t] : 0u;
        PairGrad g = pair_grad_zero();
        if (mine) g = pair(t, cid, gid, pw, gc);
        if (mine) {
            // a row's velocity gradient exists only under a rolling shutter
            const bool vel = a.velocities != nullptr && a.rs_time[cid] > 0.f;
            if (sparse_grad) {
                emit_gaussian<false>(a.out, false, (uint32_t)t, gid, gc, g);
                if (vel && a.out.v_velocities != nullptr)
                    for (int i = 0; i < 3; ++i) atomicAdd(a.out.v_velocities + (size_t)gid * 3 + i, g.v_vel[i]);
            } else {
                emit_gaussian<true>(a.out, vel, gid, gid, gc, g);
            }
        }
        emit_pose(a.out, mine, cid, g.pg);
    }
}

template <bool GATHER>
__global__ void __launch_bounds__(SPLATAD_THREADS)
projection_bwd_kernel(CamArgs a) {
    projection_bwd_driver<GATHER>(
        a, a.camera_ids, a.gaussian_ids, (uint64_t)a.nnz, a.sparse_grad != 0,
        [&](uint64_t idx) { return a.radii[idx * 2] > 0; },
        [&](uint64_t idx, uint32_t cid, uint32_t gid, const float pw[3], const GaussianCov &gc) {
            return camera_pair_vjp(a, idx, cid, gid, pw, gc);
        });
}

struct LidarArgs {
    uint32_t C, N;
    const float *means, *covars, *quats, *scales, *velocities, *viewmats;
    const float *lin_vel, *ang_vel, *rs_time;
    float eps2d;
    const float *radii, *conics, *compensations, *v_means2d, *v_depths, *v_conics, *v_compensations,
        *v_pix_vels, *v_depth_comps;
    BwdOutputs out;
};

__device__ __forceinline__ PairGrad lidar_pair_vjp(const LidarArgs &a, uint64_t idx, uint32_t cid,
                                                   uint32_t gid, const float pw[3],
                                                   const GaussianCov &gc) {
    PairGrad g = pair_grad_zero();
    const float *vm = a.viewmats + cid * 16;
    Mat3 R;
    R.m[0] = vm[0]; R.m[1] = vm[1]; R.m[2] = vm[2];
    R.m[3] = vm[4]; R.m[4] = vm[5]; R.m[5] = vm[6];
    R.m[6] = vm[8]; R.m[7] = vm[9]; R.m[8] = vm[10];
    float pc[3];
#pragma unroll
    for (int i = 0; i < 3; ++i) pc[i] = R.m[i * 3] * pw[0] + R.m[i * 3 + 1] * pw[1] + R.m[i * 3 + 2] * pw[2] + vm[i * 4 + 3];
    const Mat3 cov_c = mat3_mul_bt(mat3_mul(R, gc.cov), R);

    const float x = pc[0], y = pc[1], z = pc[2];
    const float x2 = x * x, y2 = y * y, z2 = z * z;
    const float rho2 = x2 + y2, r2 = rho2 + z2;
    const float rho = sqrtf(rho2), r = sqrtf(r2);
    const float rinv = 1.f / r;
    const float k_az = RAD_TO_DEG / rho2, k_el = RAD_TO_DEG / (r2 * rho);
    Mat3 J;
    J.m[0] = -y * k_az; J.m[1] = x * k_az; J.m[2] = 0.f;
    J.m[3] = -x * z * k_el; J.m[4] = -y * z * k_el; J.m[5] = rho2 * k_el;
    J.m[6] = x * rinv; J.m[7] = y * rinv; J.m[8] = z * rinv;
    const Mat3 JS = mat3_mul(J, cov_c);
    const Mat3 cs = mat3_mul_bt(JS, J);

    const float *cn = a.conics + idx * 3;
    const float *vcn = a.v_conics + idx * 3;
    const bool has_comp = a.v_compensations != nullptr;
    const Sym2 g2 = conic_and_compensation_vjp(cn[0], cn[1], cn[2], vcn[0], vcn[1], vcn[2], has_comp,
                                               has_comp ? a.compensations[idx] : 0.f,
                                               has_comp ? a.v_compensations[idx] : 0.f, a.eps2d);
    // cotangent of the 3x3 spherical covariance cs
    Mat3 v_cs = mat3_zero();
    v_cs.m[0] = g2.xx; v_cs.m[1] = g2.xy; v_cs.m[3] = g2.xy; v_cs.m[4] = g2.yy;
    {
        // depth compensation dc = [(b1 c2 - b2 c1), (a2 c1 - a1 c2)] / (a1 b2 - a2 b1)
        const float a1 = cs.m[0] + a.eps2d, a2 = cs.m[1], b1 = cs.m[3], b2 = cs.m[4] + a.eps2d;
        const float c1 = cs.m[6], c2 = cs.m[7];
        const float invD = 1.f / (a1 * b2 - a2 * b1);
        const float dc0 = (b1 * c2 - b2 * c1) * invD, dc1 = (a2 * c1 - a1 * c2) * invD;
        const float v0 = a.v_depth_comps[idx * 2], v1 = a.v_depth_comps[idx * 2 + 1];
        v_cs.m[0] += (v0 * (-dc0 * b2) + v1 * (-c2 - dc1 * b2)) * invD;
        v_cs.m[1] += (v0 * (dc0 * b1) + v1 * (c1 + dc1 * b1)) * invD;
        v_cs.m[3] += (v0 * (c2 + dc0 * a2) + v1 * (dc1 * a2)) * invD;
        v_cs.m[4] += (v0 * (-c1 - dc0 * a1) + v1 * (-dc1 * a1)) * invD;
        v_cs.m[6] += (v0 * (-b2) + v1 * (a2)) * invD;
        v_cs.m[7] += (v0 * (b1) + v1 * (-a1)) * invD;
    }
    // cs = J cov_c J^T:  v_cov_c = J^T v_cs J,  v_J = v_cs J cov_c^T + v_cs^T J cov_c
    const Mat3 v_cov_c = mat3_mul(mat3_mul_at(J, v_cs), J);
    Mat3 vJ;
    {
        const Mat3 t1 = mat3_mul(v_cs, JS);    // cov_c symmetric
        const Mat3 t2 = mat3_mul_at(v_cs, JS);
#pragma unroll
        for (int i = 0; i < 9; ++i) vJ.m[i] = t1.m[i] + t2.m[i];
    }
    float v_pc[3] = {0.f, 0.f, 0.f};

    const float rs = a.rs_time[cid];
    if (rs > 0.f) {
        const float *lv = a.lin_vel + cid * 3, *av = a.ang_vel + cid * 3;
        float tv[3] = {lv[0] + (av[1] * pc[2] - av[2] * pc[1]), lv[1] + (av[2] * pc[0] - av[0] * pc[2]),
                       lv[2] + (av[0] * pc[1] - av[1] * pc[0])};
        float vw[3] = {0.f, 0.f, 0.f};
        if (a.velocities != nullptr) {
                        vw[0] = a.velocities[(size_t)gid * 3]; vw[1] = a.velocities[(size_t)gid * 3 + 1]; vw[2] = a.velocities[(size_t)gid * 3 + 2];
#pragma unroll
            for (int i = 0; i < 3; ++i) tv[i] -= R.m[i * 3] * vw[0] + R.m[i * 3 + 1] * vw[1] + R.m[i * 3 + 2] * vw[2];
        }
        const float vpv[3] = {a.v_pix_vels[idx * 3], a.v_pix_vels[idx * 3 + 1], a.v_pix_vels[idx * 3 + 2]};
        float vtv[3];
#pragma unroll
        for (int j = 0; j < 3; ++j) {
            vtv[j] = -(J.m[j] * vpv[0] + J.m[3 + j] * vpv[1] + J.m[6 + j] * vpv[2]);
#pragma unroll
            for (int i = 0; i < 3; ++i) vJ.m[i * 3 + j] += -vpv[i] * tv[j];
        }
        v_pc[0] += -(av[1] * vtv[2] - av[2] * vtv[1]);
        v_pc[1] += -(av[2] * vtv[0] - av[0] * vtv[2]);
        v_pc[2] += -(av[0] * vtv[1] - av[1] * vtv[0]);
        if (a.velocities != nullptr) {
#pragma unroll
            for (int i = 0; i < 3; ++i) {
#pragma unroll
                for (int j = 0; j < 3; ++j) g.pg.vR.m[i * 3 + j] += -vtv[i] * vw[j];
                g.v_vel[i] = -(R.m[i] * vtv[0] + R.m[3 + i] * vtv[1] + R.m[6 + i] * vtv[2]);
            }
        }
    }

    // Hessians of azimuth (rad), elevation (rad) and range w.r.t. (x, y, z); symmetric.
    const float rho4_inv = 1.f / (rho2 * rho2);
    const float Haz[6] = {2.f * x * y * rho4_inv, (y2 - x2) * rho4_inv, 0.f,   // xx xy xz
                          -2.f * x * y * rho4_inv, 0.f, 0.f};                  // yy yz zz
    const float r4 = r2 * r2;
    const float d1 = 1.f / (rho * rho2 * r4), d2 = 1.f / (r4 * rho);
    const float Hel[6] = {z * (2.f * x2 * x2 + x2 * y2 - y2 * (y2 + z2)) * d1,
                          x * y * z * (3.f * x2 + 3.f * y2 + z2) * d1,
                          -x * (rho2 - z2) * d2,
                          z * (2.f * y2 * y2 + x2 * y2 - x2 * (x2 + z2)) * d1,
                          -y * (rho2 - z2) * d2,
                          -2.f * z * rho / r4};
    const float r3_inv = rinv / r2;
    const float Hr[6] = {(y2 + z2) * r3_inv, -x * y * r3_inv, -x * z * r3_inv,
                         (x2 + z2) * r3_inv, -y * z * r3_inv, rho2 * r3_inv};
    // v_p[k] += sum_c vJ[row][c] * H_row[c][k]
    auto hess_apply = [&](const float *H, const float *vrow, float scale) {
        v_pc[0] += scale * (vrow[0] * H[0] + vrow[1] * H[1] + vrow[2] * H[2]);
        v_pc[1] += scale * (vrow[0] * H[1] + vrow[1] * H[3] + vrow[2] * H[4]);
        v_pc[2] += scale * (vrow[0] * H[2] + vrow[1] * H[4] + vrow[2] * H[5]);
    };
    hess_apply(Haz, vJ.m, RAD_TO_DEG);
    hess_apply(Hel, vJ.m + 3, RAD_TO_DEG);
    hess_apply(Hr, vJ.m + 6, 1.f);

    // means2d = (azimuth, elevation) in degrees: rows 0 and 1 of J; depth = range: row 2
    const float vm0 = a.v_means2d[idx * 2], vm1 = a.v_means2d[idx * 2 + 1], vd = a.v_depths[idx];
#pragma unroll
    for (int k = 0; k < 3; ++k) v_pc[k] += vm0 * J.m[k] + vm1 * J.m[3 + k] + vd * J.m[6 + k];

    sensor_to_world_vjp(R, pw, gc.cov, v_pc, v_cov_c, g.v_mean, g.v_cov, g.pg);
    return g;
}

__global__ void __launch_bounds__(SPLATAD_THREADS)
lidar_projection_bwd_kernel(LidarArgs a) {
    projection_bwd_driver<true>(
        a, nullptr, nullptr, 0, false, [&](uint64_t idx) { return a.radii[idx * 2] > 0.f; },
        [&](uint64_t idx, uint32_t cid, uint32_t gid, const float pw[3], const GaussianCov &gc) {
            return lidar_pair_vjp(a, idx, cid, gid, pw, gc);
        });
}

} // namespace

extern "C" int splatad_projection_bwd(
    uint32_t C, uint32_t N, const float *means, const float *covars, const float *quats,
    const float *scales, const float *velocities, const float *viewmats, const float *Ks,
    uint32_t W, uint32_t H, const float *lin_vel, const float *ang_vel, const float *rs_time,
    float eps2d, const int64_t *camera_ids, const int64_t *gaussian_ids, int64_t nnz,
    const int32_t *radii, const float *conics, const float *compensations,
    const float *v_means2d, const float *v_depths, const float *v_conics,
    const float *v_compensations, const float *v_pix_vels, int sparse_grad, float *v_means,
    float *v_covars, float *v_quats, float *v_scales, float *v_viewmats, float *v_velocities,
    splatad_stream_t stream) {
    SPLATAD_REQUIRE((covars != nullptr) != (quats != nullptr && scales != nullptr),
                    "projection bwd: pass either covars or (quats, scales)");
    SPLATAD_REQUIRE((covars != nullptr) == (v_covars != nullptr) &&
                        (covars == nullptr) == (v_quats != nullptr && v_scales != nullptr),
                    "projection bwd: gradient outputs do not match the covariance inputs");
    const bool packed = camera_ids != nullptr;
    SPLATAD_REQUIRE(packed == (gaussian_ids != nullptr), "projection bwd: camera_ids and gaussian_ids go together");
    SPLATAD_REQUIRE(packed || radii != nullptr, "projection bwd: radii is null");
    SPLATAD_REQUIRE(!sparse_grad || packed, "projection bwd: sparse gradients need packed inputs");
    SPLATAD_REQUIRE(v_compensations == nullptr || compensations != nullptr,
                    "projection bwd: v_compensations without compensations");
    const uint64_t total = packed ? (uint64_t)nnz : (uint64_t)C * N;
    if (total == 0) return 0;
    SPLATAD_REQUIRE(total < (1ull << 31), "projection bwd: too many elements");
    SPLATAD_REQUIRE(means && viewmats && Ks && lin_vel && ang_vel && rs_time && conics && v_means2d &&
                        v_depths && v_conics && v_pix_vels && v_means,
                    "projection bwd: null pointer argument");
    CamArgs a;
    a.C = C; a.N = N; a.means = means; a.covars = covars; a.quats = quats; a.scales = scales;
    a.velocities = velocities; a.viewmats = viewmats; a.Ks = Ks; a.W = W; a.H = H;
    a.lin_vel = lin_vel; a.ang_vel = ang_vel; a.rs_time = rs_time; a.eps2d = eps2d;
    a.camera_ids = camera_ids; a.gaussian_ids = gaussian_ids; a.nnz = nnz; a.radii = radii;
    a.conics = conics; a.compensations = compensations; a.v_means2d = v_means2d;
    a.v_depths = v_depths; a.v_conics = v_conics; a.v_compensations = v_compensations;
    a.v_pix_vels = v_pix_vels; a.sparse_grad = sparse_grad;
    a.out = BwdOutputs{v_means, v_covars, v_quats, v_scales, v_viewmats, v_velocities};
    const uint64_t lanes = packed ? total : (uint64_t)N;
    const dim3 grid((uint32_t)((lanes + SPLATAD_THREADS - 1) / SPLATAD_THREADS));
    if (packed)
        hipLaunchKernelGGL(projection_bwd_kernel<false>, grid, dim3(SPLATAD_THREADS), 0, (hipStream_t)stream, a);
    else
        hipLaunchKernelGGL(projection_bwd_kernel<true>, grid, dim3(SPLATAD_THREADS), 0, (hipStream_t)stream, a);
    SPLATAD_LAUNCH_CHECK();
    return 0;
}

extern "C" int splatad_lidar_projection_bwd(
    uint32_t C, uint32_t N, const float *means, const float *covars, const float *quats,
    const float *scales, const float *velocities, const float *viewmats, const float *lin_vel,
    const float *ang_vel, const float *rs_time, float eps2d, const float *radii,
    const float *conics, const float *compensations, const float *v_means2d,
    const float *v_depths, const float *v_conics, const float *v_compensations,
    const float *v_pix_vels, const float *v_depth_comps, float *v_means, float *v_covars,
    float *v_quats, float *v_scales, float *v_viewmats, float *v_velocities,
    splatad_stream_t stream) {
    SPLATAD_REQUIRE((covars != nullptr) != (quats != nullptr && scales != nullptr),
                    "lidar projection bwd: pass either covars or (quats, scales)");
    SPLATAD_REQUIRE((covars != nullptr) == (v_covars != nullptr) &&
                        (covars == nullptr) == (v_quats != nullptr && v_scales != nullptr),
                    "lidar projection bwd: gradient outputs do not match the covariance inputs");
    SPLATAD_REQUIRE(v_compensations == nullptr || compensations != nullptr,
                    "lidar projection bwd: v_compensations without compensations");
    const uint64_t total = (uint64_t)C * N;
    if (total == 0) return 0;
    SPLATAD_REQUIRE(total < (1ull << 31), "lidar projection bwd: too many elements");
    SPLATAD_REQUIRE(means && viewmats && lin_vel && ang_vel && rs_time && radii && conics && v_means2d &&
                        v_depths && v_conics && v_pix_vels && v_depth_comps && v_means,
                    "lidar projection bwd: null pointer argument");
    LidarArgs a;
    a.C = C; a.N = N; a.means = means; a.covars = covars; a.quats = quats; a.scales = scales;
    a.velocities = velocities; a.viewmats = viewmats; a.lin_vel = lin_vel; a.ang_vel = ang_vel;
    a.rs_time = rs_time; a.eps2d = eps2d; a.radii = radii; a.conics = conics;
    a.compensations = compensations; a.v_means2d = v_means2d; a.v_depths = v_depths;
    a.v_conics = v_conics; a.v_compensations = v_compensations; a.v_pix_vels = v_pix_vels;
    a.v_depth_comps = v_depth_comps;
    a.out = BwdOutputs{v_means, v_covars, v_quats, v_scales, v_viewmats, v_velocities};
    hipLaunchKernelGGL(lidar_projection_bwd_kernel, dim3((uint32_t)((N + SPLATAD_THREADS - 1) / SPLATAD_THREADS)),
                       dim3(SPLATAD_THREADS), 0, (hipStream_t)stream, a);
    SPLATAD_LAUNCH_CHECK();
    return 0;
}
