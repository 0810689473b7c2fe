// The unfused projection operators for gfx950: quaternion/scale -> covariance and precision,
// world -> sensor frame, pinhole and spherical projection of a mean and covariance, and the
// image-space / spherical velocity of a point under sensor motion, each with its
// vector-Jacobian product.  One lane per element; every kernel streams its rows once.
//
// Semantics follow gsplat/cuda/csrc/projection.cu:18-599 and :1841-2266 of the reference
// (device rules in utils.cuh:57-480, helpers.cuh:80-160).  The fused kernels in
// projection.hip / projection_bwd.hip compute the same quantities without materialising the
// intermediate tensors; these operators exist for code that composes the steps itself.
#include "common.h"

#define RAD_TO_DEG 57.2957795131f

namespace {

__device__ __forceinline__ Mat3 load_mat3(const float *p) {
    Mat3 m;
#pragma unroll
    for (int i = 0; i < 9; ++i) m.m[i] = p[i];
    return m;
}

__device__ __forceinline__ void store_mat3(float *p, const Mat3 &m) {
#pragma unroll
    for (int i = 0; i < 9; ++i) p[i] = m.m[i];
}

__device__ __forceinline__ void store_triu(float *p, const Mat3 &m) {
    p[0] = m.m[0]; p[1] = m.m[1]; p[2] = m.m[2]; p[3] = m.m[4]; p[4] = m.m[5]; p[5] = m.m[8];
}

// cotangent matrix of a [3,3] or upper-triangular [6] gradient (off-diagonals halved,
// projection.cu:118-126)
__device__ __forceinline__ Mat3 load_cotangent(const float *p, bool triu) {
    if (!triu) return load_mat3(p);
    Mat3 g;
    g.m[0] = p[0]; g.m[1] = 0.5f * p[1]; g.m[2] = 0.5f * p[2];
    g.m[3] = 0.5f * p[1]; g.m[4] = p[3]; g.m[5] = 0.5f * p[4];
    g.m[6] = 0.5f * p[2]; g.m[7] = 0.5f * p[4]; g.m[8] = p[5];
    return g;
}

// ---------------------------------------------------------------- quat, scale -> matrices

__global__ void __launch_bounds__(SPLATAD_THREADS)
quat_scale_fwd_kernel(uint32_t N, const float *__restrict__ quats, const float *__restrict__ scales,
                      int triu, float *__restrict__ covars, float *__restrict__ precis) {
    const uint32_t idx = blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= N) return;
    const float4 q = reinterpret_cast<const float4 *>(quats)[idx];
    const Mat3 R = quat_to_rotmat(q.x, q.y, q.z, q.w);
    const float s[3] = {scales[idx * 3], scales[idx * 3 + 1], scales[idx * 3 + 2]};
    if (covars != nullptr) {
        Mat3 M;
#pragma unroll
        for (int i = 0; i < 3; ++i)
#pragma unroll
            for (int j = 0; j < 3; ++j) M.m[i * 3 + j] = R.m[i * 3 + j] * s[j];
        const Mat3 cov = mat3_mul_bt(M, M);
        if (triu) store_triu(covars + (size_t)idx * 6, cov); else store_mat3(covars + (size_t)idx * 9, cov);
    }
    if (precis != nullptr) {
        Mat3 M;
#pragma unroll
        for (int i = 0; i < 3; ++i)
#pragma unroll
            for (int j = 0; j < 3; ++j) M.m[i * 3 + j] = R.m[i * 3 + j] * (1.f / s[j]);
        const Mat3 pre = mat3_mul_bt(M, M);
        if (triu) store_triu(precis + (size_t)idx * 6, pre); else store_mat3(precis + (size_t)idx * 9, pre);
    }
}

// Sigma = M M^T, M = R diag(d): adds the gradient w.r.t. R to vR and returns that w.r.t. d
__device__ __forceinline__ void rot_diag_vjp(const Mat3 &R, const float d[3], const Mat3 &G, Mat3 &vR,
                                             float vd[3]) {
    Mat3 Gs, M;
#pragma unroll
    for (int i = 0; i < 3; ++i)
#pragma unroll
        for (int j = 0; j < 3; ++j) {
            Gs.m[i * 3 + j] = G.m[i * 3 + j] + G.m[j * 3 + i];
            M.m[i * 3 + j] = R.m[i * 3 + j] * d[j];
        }
    const Mat3 vM = mat3_mul(Gs, M);
#pragma unroll
    for (int j = 0; j < 3; ++j) {
        float acc = 0.f;
#pragma unroll
        for (int i = 0; i < 3; ++i) {
            acc += R.m[i * 3 + j] * vM.m[i * 3 + j];
            vR.m[i * 3 + j] += vM.m[i * 3 + j] * d[j];
        }
        vd[j] = acc;
    }
}

// gradient of the raw quaternion (w, x, y, z) from that of R(q / |q|), utils.cuh:77-98
__device__ __forceinline__ void quat_vjp(const float4 q, const Mat3 &vR, float vq[4]) {
    const float inv = rsqrtf(q.x * q.x + q.y * q.y + q.z * q.z + q.w * q.w);
    const float w = q.x * inv, x = q.y * inv, y = q.z * inv, z = q.w * inv;
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

__global__ void __launch_bounds__(SPLATAD_THREADS)
quat_scale_bwd_kernel(uint32_t N, const float *__restrict__ quats, const float *__restrict__ scales,
                      const float *__restrict__ v_covars, const float *__restrict__ v_precis, int triu,
                      float *__restrict__ v_quats, float *__restrict__ v_scales) {
    const uint32_t idx = blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= N) return;
    const float4 q = reinterpret_cast<const float4 *>(quats)[idx];
    const Mat3 R = quat_to_rotmat(q.x, q.y, q.z, q.w);
    const float s[3] = {scales[idx * 3], scales[idx * 3 + 1], scales[idx * 3 + 2]};
    Mat3 vR = mat3_zero();
    float vs[3] = {0.f, 0.f, 0.f};
    const size_t stride = triu ? 6 : 9;
    if (v_covars != nullptr) {
        float vd[3];
        rot_diag_vjp(R, s, load_cotangent(v_covars + idx * stride, triu), vR, vd);
#pragma unroll
        for (int j = 0; j < 3; ++j) vs[j] += vd[j];
    }
    if (v_precis != nullptr) {
        const float d[3] = {1.f / s[0], 1.f / s[1], 1.f / s[2]};
        float vd[3];
        rot_diag_vjp(R, d, load_cotangent(v_precis + idx * stride, triu), vR, vd);
#pragma unroll
        for (int j = 0; j < 3; ++j) vs[j] += -vd[j] * d[j] * d[j];
    }
    float vq[4];
    quat_vjp(q, vR, vq);
#pragma unroll
    for (int i = 0; i < 4; ++i) v_quats[(size_t)idx * 4 + i] = vq[i];
#pragma unroll
    for (int i = 0; i < 3; ++i) v_scales[(size_t)idx * 3 + i] = vs[i];
}

// ---------------------------------------------------------------- world -> sensor frame

__global__ void __launch_bounds__(SPLATAD_THREADS)
world_to_cam_fwd_kernel(uint32_t C, uint32_t N, const float *__restrict__ means,
                        const float *__restrict__ covars, const float *__restrict__ viewmats,
                        float *__restrict__ means_c, float *__restrict__ covars_c) {
    const uint64_t idx = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= (uint64_t)C * N) return;
    const uint32_t cid = (uint32_t)(idx / N), gid = (uint32_t)(idx % N);
    const float *vm = viewmats + cid * 16;
    Mat3 R;
#pragma unroll
    for (int i = 0; i < 3; ++i)
#pragma unroll
        for (int j = 0; j < 3; ++j) R.m[i * 3 + j] = vm[i * 4 + j];
    const float *p = means + (size_t)gid * 3;
#pragma unroll
    for (int i = 0; i < 3; ++i)
        means_c[idx * 3 + i] = R.m[i * 3] * p[0] + R.m[i * 3 + 1] * p[1] + R.m[i * 3 + 2] * p[2] + vm[i * 4 + 3];
    store_mat3(covars_c + idx * 9, mat3_mul_bt(mat3_mul(R, load_mat3(covars + (size_t)gid * 9)), R));
}

// outputs are accumulated with atomics (zero-filled by the caller); the pose gradient is summed
// over the wavefront first when all its lanes share the sensor
__global__ void __launch_bounds__(SPLATAD_THREADS)
world_to_cam_bwd_kernel(uint32_t C, uint32_t N, const float *__restrict__ means,
                        const float *__restrict__ covars, const float *__restrict__ viewmats,
                        const float *__restrict__ v_means_c, const float *__restrict__ v_covars_c,
                        float *__restrict__ v_means, float *__restrict__ v_covars,
                        float *__restrict__ v_viewmats) {
    const uint64_t idx = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const bool active = idx < (uint64_t)C * N;
    const uint32_t cid = active ? (uint32_t)(idx / N) : C - 1, gid = active ? (uint32_t)(idx % N) : 0;
    float pose[12];
#pragma unroll
    for (int i = 0; i < 12; ++i) pose[i] = 0.f;
    if (active) {
        const float *vm = viewmats + cid * 16;
        Mat3 R;
#pragma unroll
        for (int i = 0; i < 3; ++i)
#pragma unroll
            for (int j = 0; j < 3; ++j) R.m[i * 3 + j] = vm[i * 4 + j];
        const float *p = means + (size_t)gid * 3;
        const float vp[3] = {v_means_c[idx * 3], v_means_c[idx * 3 + 1], v_means_c[idx * 3 + 2]};
        const Mat3 G = load_mat3(v_covars_c + idx * 9);
        const Mat3 cov = load_mat3(covars + (size_t)gid * 9);
        if (v_means != nullptr) {
#pragma unroll
            for (int i = 0; i < 3; ++i)
                atomicAdd(v_means + (size_t)gid * 3 + i, R.m[i] * vp[0] + R.m[3 + i] * vp[1] + R.m[6 + i] * vp[2]);
        }
        if (v_covars != nullptr) {
            const Mat3 vc = mat3_mul(mat3_mul_at(R, G), R); // R^T G R
#pragma unroll
            for (int i = 0; i < 9; ++i) atomicAdd(v_covars + (size_t)gid * 9 + i, vc.m[i]);
        }
        if (v_viewmats != nullptr) {
            // v_R = v_p p^T + G R cov^T + G^T R cov, v_t = v_p
            const Mat3 a = mat3_mul(G, mat3_mul_bt(R, cov));
            const Mat3 b = mat3_mul_at(G, mat3_mul(R, cov));
#pragma unroll
            for (int i = 0; i < 3; ++i) {
#pragma unroll
                for (int j = 0; j < 3; ++j) pose[i * 4 + j] = vp[i] * p[j] + a.m[i * 3 + j] + b.m[i * 3 + j];
                pose[i * 4 + 3] = vp[i];
            }
        }
    }
    if (v_viewmats != nullptr) {
        const uint32_t first = (uint32_t)__shfl((int)cid, 0, SPLATAD_WAVE);
        if (__all(cid == first)) {
#pragma unroll
            for (int i = 0; i < 12; ++i) pose[i] = wave_sum(pose[i]);
            if ((threadIdx.x & (SPLATAD_WAVE - 1)) == 0) {
#pragma unroll
                for (int i = 0; i < 12; ++i) atomicAdd(v_viewmats + (size_t)first * 16 + i, pose[i]);
            }
        } else if (active) {
#pragma unroll
            for (int i = 0; i < 12; ++i) atomicAdd(v_viewmats + (size_t)cid * 16 + i, pose[i]);
        }
    }
}

// ---------------------------------------------------------------- pinhole projection

// J = d(pixel)/d(p) with the field-of-view clamp of utils.cuh:190-217
struct PerspJ {
    float fx, fy, cx, cy, rz, rz2, rz3, tx, ty;
    float J00, J02, J11, J12;
    bool x_in, y_in;
};

__device__ __forceinline__ PerspJ persp_jacobian(const float *K, uint32_t W, uint32_t H, float x, float y,
                                                 float z) {
    PerspJ j;
    j.fx = K[0]; j.fy = K[4]; j.cx = K[2]; j.cy = K[5];
    const float tan_fovx = 0.5f * (float)W / j.fx, tan_fovy = 0.5f * (float)H / j.fy;
    const float lim_x_pos = ((float)W - j.cx) / j.fx + 0.3f * tan_fovx;
    const float lim_x_neg = j.cx / j.fx + 0.3f * tan_fovx;
    const float lim_y_pos = ((float)H - j.cy) / j.fy + 0.3f * tan_fovy;
    const float lim_y_neg = j.cy / j.fy + 0.3f * tan_fovy;
    j.rz = 1.f / z; j.rz2 = j.rz * j.rz; j.rz3 = j.rz2 * j.rz;
    j.x_in = (x * j.rz <= lim_x_pos && x * j.rz >= -lim_x_neg);
    j.y_in = (y * j.rz <= lim_y_pos && y * j.rz >= -lim_y_neg);
    j.tx = z * fminf(lim_x_pos, fmaxf(-lim_x_neg, x * j.rz));
    j.ty = z * fminf(lim_y_pos, fmaxf(-lim_y_neg, y * j.rz));
    j.J00 = j.fx * j.rz; j.J02 = -j.fx * j.tx * j.rz2;
    j.J11 = j.fy * j.rz; j.J12 = -j.fy * j.ty * j.rz2;
    return j;
}

// adds to v_p the gradient that reaches p through J, given the cotangent of J's four entries
__device__ __forceinline__ void persp_jacobian_vjp(const PerspJ &j, float vJ00, float vJ02, float vJ11,
                                                   float vJ12, float v_p[3]) {
    if (j.x_in) v_p[0] += -j.fx * j.rz2 * vJ02; else v_p[2] += -j.fx * j.rz3 * vJ02 * j.tx;
    if (j.y_in) v_p[1] += -j.fy * j.rz2 * vJ12; else v_p[2] += -j.fy * j.rz3 * vJ12 * j.ty;
    v_p[2] += -j.fx * j.rz2 * vJ00 - j.fy * j.rz2 * vJ11 + 2.f * j.fx * j.tx * j.rz3 * vJ02 +
              2.f * j.fy * j.ty * j.rz3 * vJ12;
}

__global__ void __launch_bounds__(SPLATAD_THREADS)
persp_proj_fwd_kernel(uint32_t C, uint32_t N, const float *__restrict__ means,
                      const float *__restrict__ covars, const float *__restrict__ Ks, uint32_t W,
                      uint32_t H, float *__restrict__ means2d, float *__restrict__ covars2d) {
    const uint64_t idx = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= (uint64_t)C * N) return;
    const uint32_t cid = (uint32_t)(idx / N);
    const float x = means[idx * 3], y = means[idx * 3 + 1], z = means[idx * 3 + 2];
    const PerspJ j = persp_jacobian(Ks + cid * 9, W, H, x, y, z);
    const float *S = covars + idx * 9;
    const float r0[3] = {j.J00, 0.f, j.J02}, r1[3] = {0.f, j.J11, j.J12};
    float JS0[3], JS1[3];
#pragma unroll
    for (int k = 0; k < 3; ++k) {
        JS0[k] = r0[0] * S[k] + r0[2] * S[6 + k];
        JS1[k] = r1[1] * S[3 + k] + r1[2] * S[6 + k];
    }
    float *o = covars2d + idx * 4;
    o[0] = JS0[0] * r0[0] + JS0[2] * r0[2];
    o[1] = JS0[1] * r1[1] + JS0[2] * r1[2];
    o[2] = JS1[0] * r0[0] + JS1[2] * r0[2];
    o[3] = JS1[1] * r1[1] + JS1[2] * r1[2];
    means2d[idx * 2] = j.fx * x * j.rz + j.cx;
    means2d[idx * 2 + 1] = j.fy * y * j.rz + j.cy;
}

__global__ void __launch_bounds__(SPLATAD_THREADS)
persp_proj_bwd_kernel(uint32_t C, uint32_t N, const float *__restrict__ means,
                      const float *__restrict__ covars, const float *__restrict__ Ks, uint32_t W,
                      uint32_t H, const float *__restrict__ v_means2d,
                      const float *__restrict__ v_covars2d, float *__restrict__ v_means,
                      float *__restrict__ v_covars) {
    const uint64_t idx = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= (uint64_t)C * N) return;
    const uint32_t cid = (uint32_t)(idx / N);
    const float x = means[idx * 3], y = means[idx * 3 + 1], z = means[idx * 3 + 2];
    const PerspJ j = persp_jacobian(Ks + cid * 9, W, H, x, y, z);
    const float *S = covars + idx * 9;
    const float *G = v_covars2d + idx * 4; // [[g00, g01], [g10, g11]]
    const float r0[3] = {j.J00, 0.f, j.J02}, r1[3] = {0.f, j.J11, j.J12};
    // v_cov = J^T G J
    float *vc = v_covars + idx * 9;
#pragma unroll
    for (int a = 0; a < 3; ++a)
#pragma unroll
        for (int b = 0; b < 3; ++b)
            vc[a * 3 + b] = r0[a] * (G[0] * r0[b] + G[1] * r1[b]) + r1[a] * (G[2] * r0[b] + G[3] * r1[b]);
    // v_J = G J S^T + G^T J S
    float JSt0[3], JSt1[3], JS0[3], JS1[3];
#pragma unroll
    for (int k = 0; k < 3; ++k) {
        JSt0[k] = r0[0] * S[k * 3] + r0[2] * S[k * 3 + 2];     // (J S^T)[0][k]
        JSt1[k] = r1[1] * S[k * 3 + 1] + r1[2] * S[k * 3 + 2];
        JS0[k] = r0[0] * S[k] + r0[2] * S[6 + k];              // (J S)[0][k]
        JS1[k] = r1[1] * S[3 + k] + r1[2] * S[6 + k];
    }
    const float vJ00 = G[0] * JSt0[0] + G[1] * JSt1[0] + G[0] * JS0[0] + G[2] * JS1[0];
    const float vJ02 = G[0] * JSt0[2] + G[1] * JSt1[2] + G[0] * JS0[2] + G[2] * JS1[2];
    const float vJ11 = G[2] * JSt0[1] + G[3] * JSt1[1] + G[1] * JS0[1] + G[3] * JS1[1];
    const float vJ12 = G[2] * JSt0[2] + G[3] * JSt1[2] + G[1] * JS0[2] + G[3] * JS1[2];
    const float vm0 = v_means2d[idx * 2], vm1 = v_means2d[idx * 2 + 1];
    float v_p[3] = {j.fx * j.rz * vm0, j.fy * j.rz * vm1, -(j.fx * x * vm0 + j.fy * y * vm1) * j.rz2};
    persp_jacobian_vjp(j, vJ00, vJ02, vJ11, vJ12, v_p);
#pragma unroll
    for (int k = 0; k < 3; ++k) v_means[idx * 3 + k] = v_p[k];
}

// total velocity of a point in the moving sensor frame: v_lin + omega x p - v_point
__device__ __forceinline__ void relative_velocity(const float *lv, const float *av, const float p[3],
                                                  const float *vp, float tv[3]) {
    tv[0] = lv[0] + (av[1] * p[2] - av[2] * p[1]) - vp[0];
    tv[1] = lv[1] + (av[2] * p[0] - av[0] * p[2]) - vp[1];
    tv[2] = lv[2] + (av[0] * p[1] - av[1] * p[0]) - vp[2];
}

__global__ void __launch_bounds__(SPLATAD_THREADS)
pix_velocity_fwd_kernel(uint32_t C, uint32_t N, const float *__restrict__ p_view,
                        const float *__restrict__ lin_vel, const float *__restrict__ ang_vel,
                        const float *__restrict__ vel_view, const float *__restrict__ Ks, uint32_t W,
                        uint32_t H, float *__restrict__ out) {
    const uint64_t idx = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= (uint64_t)C * N) return;
    const uint32_t cid = (uint32_t)(idx / N);
    const float p[3] = {p_view[idx * 3], p_view[idx * 3 + 1], p_view[idx * 3 + 2]};
    const PerspJ j = persp_jacobian(Ks + cid * 9, W, H, p[0], p[1], p[2]);
    float tv[3];
    relative_velocity(lin_vel + cid * 3, ang_vel + cid * 3, p, vel_view + idx * 3, tv);
    out[idx * 2] = -(j.J00 * tv[0] + j.J02 * tv[2]);
    out[idx * 2 + 1] = -(j.J11 * tv[1] + j.J12 * tv[2]);
}

__global__ void __launch_bounds__(SPLATAD_THREADS)
pix_velocity_bwd_kernel(uint32_t C, uint32_t N, const float *__restrict__ p_view,
                        const float *__restrict__ lin_vel, const float *__restrict__ ang_vel,
                        const float *__restrict__ vel_view, const float *__restrict__ Ks, uint32_t W,
                        uint32_t H, const float *__restrict__ v_out, float *__restrict__ v_p_view,
                        float *__restrict__ v_vel_view) {
    const uint64_t idx = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= (uint64_t)C * N) return;
    const uint32_t cid = (uint32_t)(idx / N);
    const float p[3] = {p_view[idx * 3], p_view[idx * 3 + 1], p_view[idx * 3 + 2]};
    const PerspJ j = persp_jacobian(Ks + cid * 9, W, H, p[0], p[1], p[2]);
    const float *av = ang_vel + cid * 3;
    float tv[3];
    relative_velocity(lin_vel + cid * 3, av, p, vel_view + idx * 3, tv);
    const float vx = v_out[idx * 2], vy = v_out[idx * 2 + 1];
    // out = -J tv:  v_tv = -J^T v,  v_J = -v tv^T
    const float vtv[3] = {-j.J00 * vx, -j.J11 * vy, -(j.J02 * vx + j.J12 * vy)};
    float v_p[3] = {-(av[1] * vtv[2] - av[2] * vtv[1]), -(av[2] * vtv[0] - av[0] * vtv[2]),
                    -(av[0] * vtv[1] - av[1] * vtv[0])};
    persp_jacobian_vjp(j, -vx * tv[0], -vx * tv[2], -vy * tv[1], -vy * tv[2], v_p);
#pragma unroll
    for (int k = 0; k < 3; ++k) {
        v_p_view[idx * 3 + k] = v_p[k];
        v_vel_view[idx * 3 + k] = -vtv[k];
    }
}

// ---------------------------------------------------------------- spherical projection

// J = d(azimuth deg, elevation deg, range)/d(p), utils.cuh:281-318
struct SphereJ {
    Mat3 J;
    float x, y, z, x2, y2, z2, rho2, r2, rho, r, rinv;
};

__device__ __forceinline__ SphereJ sphere_jacobian(float x, float y, float z) {
    SphereJ s;
    s.x = x; s.y = y; s.z = z;
    s.x2 = x * x; s.y2 = y * y; s.z2 = z * z;
    s.rho2 = s.x2 + s.y2; s.r2 = s.rho2 + s.z2;
    s.rho = sqrtf(s.rho2); s.r = sqrtf(s.r2); s.rinv = 1.f / s.r;
    const float k_az = RAD_TO_DEG / s.rho2, k_el = RAD_TO_DEG / (s.r2 * s.rho);
    s.J.m[0] = -y * k_az; s.J.m[1] = x * k_az; s.J.m[2] = 0.f;
    s.J.m[3] = -x * z * k_el; s.J.m[4] = -y * z * k_el; s.J.m[5] = s.rho2 * k_el;
    s.J.m[6] = x * s.rinv; s.J.m[7] = y * s.rinv; s.J.m[8] = z * s.rinv;
    return s;
}

// adds to v_p the gradient that reaches p through J (cotangent vJ), by contracting with the
// symmetric Hessians of azimuth, elevation (radians) and range
__device__ __forceinline__ void sphere_jacobian_vjp(const SphereJ &s, const Mat3 &vJ, float v_p[3]) {
    const float x = s.x, y = s.y, z = s.z, x2 = s.x2, y2 = s.y2, z2 = s.z2, rho2 = s.rho2, r2 = s.r2;
    const float rho4_inv = 1.f / (rho2 * rho2);
    const float Haz[6] = {2.f * x * y * rho4_inv, (y2 - x2) * rho4_inv, 0.f, -2.f * x * y * rho4_inv, 0.f, 0.f};
    const float r4 = r2 * r2;
    const float d1 = 1.f / (s.rho * rho2 * r4), d2 = 1.f / (r4 * s.rho);
    const float Hel[6] = {z * (2.f * x2 * x2 + x2 * y2 - y2 * (y2 + z2)) * d1,
                          x * y * z * (3.f * x2 + 3.f * y2 + z2) * d1,
                          -x * (rho2 - z2) * d2,
                          z * (2.f * y2 * y2 + x2 * y2 - x2 * (x2 + z2)) * d1,
                          -y * (rho2 - z2) * d2,
                          -2.f * z * s.rho / r4};
    const float r3_inv = s.rinv / r2;
    const float Hr[6] = {(y2 + z2) * r3_inv, -x * y * r3_inv, -x * z * r3_inv,
                         (x2 + z2) * r3_inv, -y * z * r3_inv, rho2 * r3_inv};
    auto apply = [&](const float *H, const float *row, float scale) {
        v_p[0] += scale * (row[0] * H[0] + row[1] * H[1] + row[2] * H[2]);
        v_p[1] += scale * (row[0] * H[1] + row[1] * H[3] + row[2] * H[4]);
        v_p[2] += scale * (row[0] * H[2] + row[1] * H[4] + row[2] * H[5]);
    };
    apply(Haz, vJ.m, RAD_TO_DEG);
    apply(Hel, vJ.m + 3, RAD_TO_DEG);
    apply(Hr, vJ.m + 6, 1.f);
}

__global__ void __launch_bounds__(SPLATAD_THREADS)
lidar_proj_fwd_kernel(uint32_t C, uint32_t N, const float *__restrict__ means,
                      const float *__restrict__ covars, float eps2d, float *__restrict__ means2d,
                      float *__restrict__ covars2d, float *__restrict__ depth_comps) {
    const uint64_t idx = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= (uint64_t)C * N) return;
    const SphereJ s = sphere_jacobian(means[idx * 3], means[idx * 3 + 1], means[idx * 3 + 2]);
    const Mat3 cs = mat3_mul_bt(mat3_mul(s.J, load_mat3(covars + idx * 9)), s.J);
    float *o = covars2d + idx * 4;
    o[0] = cs.m[0]; o[1] = cs.m[1]; o[2] = cs.m[3]; o[3] = cs.m[4];
    means2d[idx * 2] = atan2f(s.y, s.x) * RAD_TO_DEG;
    means2d[idx * 2 + 1] = asinf(s.z * s.rinv) * RAD_TO_DEG;
    // utils.cuh:12-31; glm's cov3d[col][row] is cs.m[row * 3 + col] here
    const float a1 = cs.m[0] + eps2d, a2 = cs.m[1], b1 = cs.m[3], b2 = cs.m[4] + eps2d;
    const float c1 = cs.m[6], c2 = cs.m[7];
    const float invD = 1.f / (a1 * b2 - a2 * b1);
    depth_comps[idx * 2] = (b1 * c2 - b2 * c1) * invD;
    depth_comps[idx * 2 + 1] = (a2 * c1 - a1 * c2) * invD;
}

__global__ void __launch_bounds__(SPLATAD_THREADS)
lidar_proj_bwd_kernel(uint32_t C, uint32_t N, const float *__restrict__ means,
                      const float *__restrict__ covars, float eps2d,
                      const float *__restrict__ v_means2d, const float *__restrict__ v_covars2d,
                      const float *__restrict__ v_depth_comps, float *__restrict__ v_means,
                      float *__restrict__ v_covars) {
    const uint64_t idx = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= (uint64_t)C * N) return;
    const SphereJ s = sphere_jacobian(means[idx * 3], means[idx * 3 + 1], means[idx * 3 + 2]);
    const Mat3 S = load_mat3(covars + idx * 9);
    const Mat3 cs = mat3_mul_bt(mat3_mul(s.J, S), s.J);
    // cotangent of the 3x3 spherical covariance (row-major, v_cs[i][j] pairs with cs[i][j])
    Mat3 v_cs = mat3_zero();
    const float *G = v_covars2d + idx * 4;
    v_cs.m[0] = G[0]; v_cs.m[1] = G[1]; v_cs.m[3] = G[2]; v_cs.m[4] = G[3];
    {
        const float a1 = cs.m[0] + eps2d, a2 = cs.m[1], b1 = cs.m[3], b2 = cs.m[4] + eps2d;
        const float c1 = cs.m[6], c2 = cs.m[7];
        const float invD = 1.f / (a1 * b2 - a2 * b1);
        const float dc0 = (b1 * c2 - b2 * c1) * invD, dc1 = (a2 * c1 - a1 * c2) * invD;
        const float v0 = v_depth_comps[idx * 2], v1 = v_depth_comps[idx * 2 + 1];
        // utils.cuh:33-55
        v_cs.m[0] += (v0 * (-dc0 * b2) + v1 * (-c2 - dc1 * b2)) * invD; // a1
        v_cs.m[1] += (v0 * (dc0 * b1) + v1 * (c1 + dc1 * b1)) * invD;   // a2
        v_cs.m[3] += (v0 * (c2 + dc0 * a2) + v1 * (dc1 * a2)) * invD;   // b1
        v_cs.m[4] += (v0 * (-c1 - dc0 * a1) + v1 * (-dc1 * a1)) * invD; // b2
        v_cs.m[6] += (v0 * (-b2) + v1 * (a2)) * invD;                   // c1
        v_cs.m[7] += (v0 * (b1) + v1 * (-a1)) * invD;                   // c2
    }
    // cs = J S J^T:  v_S = J^T v_cs J,  v_J = v_cs J S^T + v_cs^T J S
    store_mat3(v_covars + idx * 9, mat3_mul(mat3_mul_at(s.J, v_cs), s.J));
    const Mat3 t1 = mat3_mul(v_cs, mat3_mul_bt(s.J, S));
    const Mat3 t2 = mat3_mul_at(v_cs, mat3_mul(s.J, S));
    Mat3 vJ;
#pragma unroll
    for (int i = 0; i < 9; ++i) vJ.m[i] = t1.m[i] + t2.m[i];
    const float vm0 = v_means2d[idx * 2], vm1 = v_means2d[idx * 2 + 1];
    float v_p[3];
#pragma unroll
    for (int k = 0; k < 3; ++k) v_p[k] = vm0 * s.J.m[k] + vm1 * s.J.m[3 + k];
    sphere_jacobian_vjp(s, vJ, v_p);
#pragma unroll
    for (int k = 0; k < 3; ++k) v_means[idx * 3 + k] = v_p[k];
}

__global__ void __launch_bounds__(SPLATAD_THREADS)
lidar_velocity_fwd_kernel(uint32_t C, uint32_t N, const float *__restrict__ p_view,
                          const float *__restrict__ lin_vel, const float *__restrict__ ang_vel,
                          const float *__restrict__ vel_view, float *__restrict__ out) {
    const uint64_t idx = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= (uint64_t)C * N) return;
    const uint32_t cid = (uint32_t)(idx / N);
    const float p[3] = {p_view[idx * 3], p_view[idx * 3 + 1], p_view[idx * 3 + 2]};
    const SphereJ s = sphere_jacobian(p[0], p[1], p[2]);
    float tv[3];
    relative_velocity(lin_vel + cid * 3, ang_vel + cid * 3, p, vel_view + idx * 3, tv);
#pragma unroll
    for (int i = 0; i < 3; ++i)
        out[idx * 3 + i] = -(s.J.m[i * 3] * tv[0] + s.J.m[i * 3 + 1] * tv[1] + s.J.m[i * 3 + 2] * tv[2]);
}

__global__ void __launch_bounds__(SPLATAD_THREADS)
lidar_velocity_bwd_kernel(uint32_t C, uint32_t N, const float *__restrict__ p_view,
                          const float *__restrict__ lin_vel, const float *__restrict__ ang_vel,
                          const float *__restrict__ vel_view, const float *__restrict__ v_out,
                          float *__restrict__ v_p_view, float *__restrict__ v_vel_view) {
    const uint64_t idx = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= (uint64_t)C * N) return;
    const uint32_t cid = (uint32_t)(idx / N);
    const float p[3] = {p_view[idx * 3], p_view[idx * 3 + 1], p_view[idx * 3 + 2]};
    const SphereJ s = sphere_jacobian(p[0], p[1], p[2]);
    const float *av = ang_vel + cid * 3;
    float tv[3];
    relative_velocity(lin_vel + cid * 3, av, p, vel_view + idx * 3, tv);
    const float v[3] = {v_out[idx * 3], v_out[idx * 3 + 1], v_out[idx * 3 + 2]};
    float vtv[3];
    Mat3 vJ;
#pragma unroll
    for (int j = 0; j < 3; ++j) {
        vtv[j] = -(s.J.m[j] * v[0] + s.J.m[3 + j] * v[1] + s.J.m[6 + j] * v[2]);
#pragma unroll
        for (int i = 0; i < 3; ++i) vJ.m[i * 3 + j] = -v[i] * tv[j];
    }
    float v_p[3] = {-(av[1] * vtv[2] - av[2] * vtv[1]), -(av[2] * vtv[0] - av[0] * vtv[2]),
                    -(av[0] * vtv[1] - av[1] * vtv[0])};
    sphere_jacobian_vjp(s, vJ, v_p);
#pragma unroll
    for (int k = 0; k < 3; ++k) {
        v_p_view[idx * 3 + k] = v_p[k];
        v_vel_view[idx * 3 + k] = -vtv[k];
    }
}

static inline dim3 grid_of(uint64_t n) { return dim3((uint32_t)((n + SPLATAD_THREADS - 1) / SPLATAD_THREADS)); }

} // namespace

#define UNFUSED_LAUNCH(kernel, n, stream, ...)                                                \
    hipLaunchKernelGGL(kernel, grid_of(n), dim3(SPLATAD_THREADS), 0, (hipStream_t)(stream),   \
                       __VA_ARGS__);                                                          \
    SPLATAD_LAUNCH_CHECK();                                                                   \
    return 0

extern "C" int splatad_quat_scale_to_covar_preci_fwd(uint32_t N, const float *quats, const float *scales,
                                                     int triu, float *covars, float *precis,
                                                     splatad_stream_t stream) {
    if (N == 0 || (!covars && !precis)) return 0;
    SPLATAD_REQUIRE(quats && scales, "quat_scale_to_covar_preci: null pointer argument");
    UNFUSED_LAUNCH(quat_scale_fwd_kernel, N, stream, N, quats, scales, triu, covars, precis);
}

extern "C" int splatad_quat_scale_to_covar_preci_bwd(uint32_t N, const float *quats, const float *scales,
                                                     const float *v_covars, const float *v_precis,
                                                     int triu, float *v_quats, float *v_scales,
                                                     splatad_stream_t stream) {
    if (N == 0) return 0;
    SPLATAD_REQUIRE(quats && scales && v_quats && v_scales, "quat_scale_to_covar_preci bwd: null pointer argument");
    UNFUSED_LAUNCH(quat_scale_bwd_kernel, N, stream, N, quats, scales, v_covars, v_precis, triu, v_quats,
                   v_scales);
}

extern "C" int splatad_world_to_cam_fwd(uint32_t C, uint32_t N, const float *means, const float *covars,
                                        const float *viewmats, float *means_c, float *covars_c,
                                        splatad_stream_t stream) {
    if ((uint64_t)C * N == 0) return 0;
    SPLATAD_REQUIRE(means && covars && viewmats && means_c && covars_c, "world_to_cam: null pointer argument");
    UNFUSED_LAUNCH(world_to_cam_fwd_kernel, (uint64_t)C * N, stream, C, N, means, covars, viewmats, means_c,
                   covars_c);
}

extern "C" int splatad_world_to_cam_bwd(uint32_t C, uint32_t N, const float *means, const float *covars,
                                        const float *viewmats, const float *v_means_c,
                                        const float *v_covars_c, float *v_means, float *v_covars,
                                        float *v_viewmats, splatad_stream_t stream) {
    if ((uint64_t)C * N == 0 || (!v_means && !v_covars && !v_viewmats)) return 0;
    SPLATAD_REQUIRE(means && covars && viewmats && v_means_c && v_covars_c,
                    "world_to_cam bwd: null pointer argument");
    UNFUSED_LAUNCH(world_to_cam_bwd_kernel, (uint64_t)C * N, stream, C, N, means, covars, viewmats, v_means_c,
                   v_covars_c, v_means, v_covars, v_viewmats);
}

extern "C" int splatad_persp_proj_fwd(uint32_t C, uint32_t N, const float *means, const float *covars,
                                      const float *Ks, uint32_t width, uint32_t height, float *means2d,
                                      float *covars2d, splatad_stream_t stream) {
    if ((uint64_t)C * N == 0) return 0;
    SPLATAD_REQUIRE(means && covars && Ks && means2d && covars2d, "persp_proj: null pointer argument");
    UNFUSED_LAUNCH(persp_proj_fwd_kernel, (uint64_t)C * N, stream, C, N, means, covars, Ks, width, height,
                   means2d, covars2d);
}

extern "C" int splatad_persp_proj_bwd(uint32_t C, uint32_t N, const float *means, const float *covars,
                                      const float *Ks, uint32_t width, uint32_t height,
                                      const float *v_means2d, const float *v_covars2d, float *v_means,
                                      float *v_covars, splatad_stream_t stream) {
    if ((uint64_t)C * N == 0) return 0;
    SPLATAD_REQUIRE(means && covars && Ks && v_means2d && v_covars2d && v_means && v_covars,
                    "persp_proj bwd: null pointer argument");
    UNFUSED_LAUNCH(persp_proj_bwd_kernel, (uint64_t)C * N, stream, C, N, means, covars, Ks, width, height,
                   v_means2d, v_covars2d, v_means, v_covars);
}

extern "C" int splatad_compute_pix_velocity_fwd(uint32_t C, uint32_t N, const float *p_view,
                                                const float *lin_vel, const float *ang_vel,
                                                const float *velocities, const float *Ks, uint32_t width,
                                                uint32_t height, float *vel, splatad_stream_t stream) {
    if ((uint64_t)C * N == 0) return 0;
    SPLATAD_REQUIRE(p_view && lin_vel && ang_vel && velocities && Ks && vel,
                    "compute_pix_velocity: null pointer argument");
    UNFUSED_LAUNCH(pix_velocity_fwd_kernel, (uint64_t)C * N, stream, C, N, p_view, lin_vel, ang_vel,
                   velocities, Ks, width, height, vel);
}

extern "C" int splatad_compute_pix_velocity_bwd(uint32_t C, uint32_t N, const float *p_view,
                                                const float *lin_vel, const float *ang_vel,
                                                const float *velocities, const float *Ks, uint32_t width,
                                                uint32_t height, const float *v_vel, float *v_p_view,
                                                float *v_velocities, splatad_stream_t stream) {
    if ((uint64_t)C * N == 0) return 0;
    SPLATAD_REQUIRE(p_view && lin_vel && ang_vel && velocities && Ks && v_vel && v_p_view && v_velocities,
                    "compute_pix_velocity bwd: null pointer argument");
    UNFUSED_LAUNCH(pix_velocity_bwd_kernel, (uint64_t)C * N, stream, C, N, p_view, lin_vel, ang_vel,
                   velocities, Ks, width, height, v_vel, v_p_view, v_velocities);
}

extern "C" int splatad_lidar_proj_fwd(uint32_t C, uint32_t N, const float *means, const float *covars,
                                      float eps2d, float *means2d, float *covars2d,
                                      float *depth_compensations, splatad_stream_t stream) {
    if ((uint64_t)C * N == 0) return 0;
    SPLATAD_REQUIRE(means && covars && means2d && covars2d && depth_compensations,
                    "lidar_proj: null pointer argument");
    UNFUSED_LAUNCH(lidar_proj_fwd_kernel, (uint64_t)C * N, stream, C, N, means, covars, eps2d, means2d,
                   covars2d, depth_compensations);
}

extern "C" int splatad_lidar_proj_bwd(uint32_t C, uint32_t N, const float *means, const float *covars,
                                      float eps2d, const float *v_means2d, const float *v_covars2d,
                                      const float *v_depth_compensations, float *v_means,
                                      float *v_covars, splatad_stream_t stream) {
    if ((uint64_t)C * N == 0) return 0;
    SPLATAD_REQUIRE(means && covars && v_means2d && v_covars2d && v_depth_compensations && v_means && v_covars,
                    "lidar_proj bwd: null pointer argument");
    UNFUSED_LAUNCH(lidar_proj_bwd_kernel, (uint64_t)C * N, stream, C, N, means, covars, eps2d, v_means2d,
                   v_covars2d, v_depth_compensations, v_means, v_covars);
}

extern "C" int splatad_compute_lidar_velocity_fwd(uint32_t C, uint32_t N, const float *p_view,
                                                  const float *lin_vel, const float *ang_vel,
                                                  const float *velocities, float *vel,
                                                  splatad_stream_t stream) {
    if ((uint64_t)C * N == 0) return 0;
    SPLATAD_REQUIRE(p_view && lin_vel && ang_vel && velocities && vel,
                    "compute_lidar_velocity: null pointer argument");
    UNFUSED_LAUNCH(lidar_velocity_fwd_kernel, (uint64_t)C * N, stream, C, N, p_view, lin_vel, ang_vel,
                   velocities, vel);
}

extern "C" int splatad_compute_lidar_velocity_bwd(uint32_t C, uint32_t N, const float *p_view,
                                                  const float *lin_vel, const float *ang_vel,
                                                  const float *velocities, const float *v_vel,
                                                  float *v_p_view, float *v_velocities,
                                                  splatad_stream_t stream) {
    if ((uint64_t)C * N == 0) return 0;
    SPLATAD_REQUIRE(p_view && lin_vel && ang_vel && velocities && v_vel && v_p_view && v_velocities,
                    "compute_lidar_velocity bwd: null pointer argument");
    UNFUSED_LAUNCH(lidar_velocity_bwd_kernel, (uint64_t)C * N, stream, C, N, p_view, lin_vel, ang_vel,
                   velocities, v_vel, v_p_view, v_velocities);
}
