// libmlpsp_hip: reverse compositing over saved forward records (scannet/cuda/primitive_records.cuh:3-46).
//
// One thread per pixel walks the pixel's records last to first, carrying `next` = the gradient-weighted colour
// of everything behind the current record.  Per record it writes d4, the adjoint of the four pre-activation
// MLP outputs (sigmoid and softplus derivatives included), and adds the geometry gradients that flow through
// the Gaussian falloff to the record's primitive: positions (through the rotated local offset), log-scales
// and quaternions (chain rule through the rotation matrix, np_tile_kernels.cu:439-479).  No MLP is evaluated.
// Neighbouring pixels are on different records of different primitives at any moment, so the per-primitive
// sums are plain f32 atomics; their order, and with it the last bits of the sums, is not fixed (the
// reference's warp-aggregated atomics are not either).
#include "mlpsp_device.hpp"
#include "mlpsp_host.hpp"

namespace mlpsp {

// ATOMIC = false: no geometry sums; instead falloff_adjoint[r] = dL/d(decay) * decay is written per record and
// geometry_gradients_kernel below forms the per-primitive sums from a primitive-major ordering of the records.
template <bool ATOMIC>
__global__ __launch_bounds__(128) void records_reverse_kernel(
    const int32_t* __restrict__ ids, const long long* __restrict__ offsets, const float* __restrict__ x6,
    const float* __restrict__ raw, const float* __restrict__ logs, const float* __restrict__ quats,
    const float* __restrict__ grgb, const float* __restrict__ gt, long long pixels, float* __restrict__ d4,
    float* __restrict__ gp, float* __restrict__ gs, float* __restrict__ gq, float* __restrict__ falloff_adjoint) {
  const long long pix = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (pix >= pixels) return;
  float next = gt[pix];
  const float g0 = grgb[pix * 3], g1 = grgb[pix * 3 + 1], g2 = grgb[pix * 3 + 2];
  const long long first = offsets[pix];
  for (long long r = offsets[pix + 1] - 1; r >= first; --r) {
    const int p = ids[r];
    const float4 va = *reinterpret_cast<const float4*>(raw + r * 8);
    const float4 vb = *reinterpret_cast<const float4*>(raw + r * 8 + 4);
    const float R = va.x, G = va.y, B = va.z, sigma_raw = va.w, trans = vb.x, alpha = vb.y, decay = vb.z;
    const float dotg = (g0 * R + g1 * G) + g2 * B;
    const float grad_alpha = trans * (dotg - next);
    next = next * (1.f - alpha) + dotg * alpha;
    const float grad_sigma = grad_alpha * det_exp(-sigma_raw * decay);
    const float grad_decay = grad_sigma * sigma_raw;
    float4 d;
    d.x = g0 * (trans * alpha) * R * (1.f - R);
    d.y = g1 * (trans * alpha) * G * (1.f - G);
    d.z = g2 * (trans * alpha) * B * (1.f - B);
    d.w = grad_sigma * decay * sigmoid(vb.w);
    *reinterpret_cast<float4*>(d4 + r * 4) = d;
    if constexpr (!ATOMIC) {
      falloff_adjoint[r] = grad_decay * decay;
      continue;
    }
    const float dx = x6[r * 6 + 3], dy = x6[r * 6 + 4], dz = x6[r * 6 + 5];
    const float4 qv = *reinterpret_cast<const float4*>(quats + (size_t)p * 4);
    const float qw = qv.x, qx = qv.y, qy = qv.z, qz = qv.w;
    const Vec3 q = quat_rotate_conj(qw, qx, qy, qz, Vec3{dx, dy, dz});
    const float mx = det_exp(-2.f * logs[p * 3]), my = det_exp(-2.f * logs[p * 3 + 1]),
                mz = det_exp(-2.f * logs[p * 3 + 2]);
    const float gx = -grad_decay * decay * mx * q.x;
    const float gy = -grad_decay * decay * my * q.y;
    const float gz = -grad_decay * decay * mz * q.z;
    const Vec3 gd = quat_rotate(qw, qx, qy, qz, Vec3{gx, gy, gz});
    atomicAdd(gp + p * 3, gd.x);
    atomicAdd(gp + p * 3 + 1, gd.y);
    atomicAdd(gp + p * 3 + 2, gd.z);
    atomicAdd(gs + p * 3, grad_decay * decay * mx * q.x * q.x);
    atomicAdd(gs + p * 3 + 1, grad_decay * decay * my * q.y * q.y);
    atomicAdd(gs + p * 3 + 2, grad_decay * decay * mz * q.z * q.z);
    const float r00 = dx * gx, r01 = dx * gy, r02 = dx * gz, r10 = dy * gx, r11 = dy * gy, r12 = dy * gz,
                r20 = dz * gx, r21 = dz * gy, r22 = dz * gz;
    atomicAdd(gq + p * 4, r01 * (-2.f * qz) + r02 * (2.f * qy) + r10 * (2.f * qz) + r12 * (-2.f * qx) +
                              r20 * (-2.f * qy) + r21 * (2.f * qx));
    atomicAdd(gq + p * 4 + 1, r01 * (2.f * qy) + r02 * (2.f * qz) + r10 * (2.f * qy) + r11 * (-4.f * qx) +
                                  r12 * (-2.f * qw) + r20 * (2.f * qz) + r21 * (2.f * qw) + r22 * (-4.f * qx));
    atomicAdd(gq + p * 4 + 2, r00 * (-4.f * qy) + r01 * (2.f * qx) + r02 * (2.f * qw) + r10 * (2.f * qx) +
                                  r12 * (2.f * qz) + r20 * (-2.f * qw) + r21 * (2.f * qz) + r22 * (-4.f * qy));
    atomicAdd(gq + p * 4 + 3, r00 * (-4.f * qz) + r01 * (-2.f * qw) + r02 * (2.f * qx) + r10 * (2.f * qw) +
                                  r11 * (-4.f * qz) + r12 * (2.f * qy) + r20 * (2.f * qx) + r21 * (2.f * qy));
  }
}

// Geometry gradients from records in primitive-major order, in two steps.  Step 1, one wavefront per segment
// (at most `segment` consecutive records of one primitive, the segments of the grouped weight gradients): over
// the segment's rows i (hit offset d_i = x6_sorted[i][3:6], falloff adjoint a_i = falloff_adjoint[record_indices[i]])
// the local-frame sums
//     sum g,   sum a m q^2,   sum d (x) g        with  q_i = R(q)^T d_i,  g_i = -a_i m .* q_i
// go to partial[segment][15].  Step 2, one thread per primitive, adds its segments and applies the per-primitive
// linear maps once: grad_position = R sum g, grad_log_scale = sum a m q^2, grad_quat = rotation-matrix chain rule
// of sum d (x) g (np_tile_kernels.cu:439-479).  Same terms as the atomic variant adds record by record; no
// atomics, fixed summation order, and a primitive with very many records is spread over many wavefronts.
__global__ __launch_bounds__(256) void geometry_partials_kernel(
    const long long* __restrict__ csr_offsets, const long long* __restrict__ record_indices,
    const float* __restrict__ x6_sorted, const float* __restrict__ falloff_adjoint, const float* __restrict__ logs,
    const float* __restrict__ quats, const long long* __restrict__ group_prim,
    const long long* __restrict__ group_start, long long num_groups, int segment, float* __restrict__ partial) {
  const long long group = (long long)blockIdx.x * 4 + (threadIdx.x >> 6);
  const int lane = threadIdx.x & 63;
  if (group >= num_groups) return;
  const long long p = group_prim[group];
  const long long begin = group_start[group];
  const long long seg_end = begin + segment, list_end = csr_offsets[p + 1];
  const long long end = seg_end < list_end ? seg_end : list_end;
  const float qw = quats[p * 4], qx = quats[p * 4 + 1], qy = quats[p * 4 + 2], qz = quats[p * 4 + 3];
  const float mx = det_exp(-2.f * logs[p * 3]), my = det_exp(-2.f * logs[p * 3 + 1]), mz = det_exp(-2.f * logs[p * 3 + 2]);
  float v[15];
#pragma unroll
  for (int k = 0; k < 15; ++k) v[k] = 0.f;
  for (long long i = begin + lane; i < end; i += 64) {
    const float a = falloff_adjoint[record_indices[i]];
    const float dx = x6_sorted[i * 6 + 3], dy = x6_sorted[i * 6 + 4], dz = x6_sorted[i * 6 + 5];
    const Vec3 q = quat_rotate_conj(qw, qx, qy, qz, Vec3{dx, dy, dz});
    const float gx = -a * mx * q.x, gy = -a * my * q.y, gz = -a * mz * q.z;
    v[0] += gx;
    v[1] += gy;
    v[2] += gz;
    v[3] += a * mx * q.x * q.x;
    v[4] += a * my * q.y * q.y;
    v[5] += a * mz * q.z * q.z;
    v[6] += dx * gx; v[7] += dx * gy; v[8] += dx * gz;
    v[9] += dy * gx; v[10] += dy * gy; v[11] += dy * gz;
    v[12] += dz * gx; v[13] += dz * gy; v[14] += dz * gz;
  }
#pragma unroll
  for (int d = 1; d < 64; d <<= 1) {
#pragma unroll
    for (int k = 0; k < 15; ++k) v[k] += __shfl_xor(v[k], d);
  }
  if (lane < 15) {
    float mine = v[0];
#pragma unroll
    for (int k = 1; k < 15; ++k) mine = (lane == k) ? v[k] : mine;
    partial[group * 16 + lane] = mine;
  }
}

__global__ __launch_bounds__(256) void geometry_finish_kernel(const float* __restrict__ partial,
                                                              const long long* __restrict__ group_offsets,
                                                              const float* __restrict__ quats, int N,
                                                              float* __restrict__ gp, float* __restrict__ gs,
                                                              float* __restrict__ gq) {
  const int p = blockIdx.x * blockDim.x + threadIdx.x;
  if (p >= N) return;
  float v[15];
#pragma unroll
  for (int k = 0; k < 15; ++k) v[k] = 0.f;
  for (long long g = group_offsets[p]; g < group_offsets[p + 1]; ++g) {
#pragma unroll
    for (int k = 0; k < 15; ++k) v[k] += partial[g * 16 + k];
  }
  const float qw = quats[p * 4], qx = quats[p * 4 + 1], qy = quats[p * 4 + 2], qz = quats[p * 4 + 3];
  const Vec3 gd = quat_rotate(qw, qx, qy, qz, Vec3{v[0], v[1], v[2]});
  gp[p * 3] = gd.x;
  gp[p * 3 + 1] = gd.y;
  gp[p * 3 + 2] = gd.z;
  gs[p * 3] = v[3];
  gs[p * 3 + 1] = v[4];
  gs[p * 3 + 2] = v[5];
  const float r00 = v[6], r01 = v[7], r02 = v[8], r10 = v[9], r11 = v[10], r12 = v[11], r20 = v[12], r21 = v[13],
              r22 = v[14];
  gq[p * 4] = r01 * (-2.f * qz) + r02 * (2.f * qy) + r10 * (2.f * qz) + r12 * (-2.f * qx) + r20 * (-2.f * qy) +
              r21 * (2.f * qx);
  gq[p * 4 + 1] = r01 * (2.f * qy) + r02 * (2.f * qz) + r10 * (2.f * qy) + r11 * (-4.f * qx) + r12 * (-2.f * qw) +
                  r20 * (2.f * qz) + r21 * (2.f * qw) + r22 * (-4.f * qx);
  gq[p * 4 + 2] = r00 * (-4.f * qy) + r01 * (2.f * qx) + r02 * (2.f * qw) + r10 * (2.f * qx) + r12 * (2.f * qz) +
                  r20 * (-2.f * qw) + r21 * (2.f * qz) + r22 * (-4.f * qy);
  gq[p * 4 + 3] = r00 * (-4.f * qz) + r01 * (-2.f * qw) + r02 * (2.f * qx) + r10 * (2.f * qw) + r11 * (-4.f * qz) +
                  r12 * (2.f * qy) + r20 * (2.f * qx) + r21 * (2.f * qy);
}

}  // namespace mlpsp

using namespace mlpsp;

MLPSP_API int mlpsp_records_reverse(const int32_t* ids_dev, const int64_t* pixel_offsets_dev, const float* x6_dev,
                                    const float* raw_dev, const float* log_scales_dev, const float* quats_dev,
                                    const float* grad_rgb_dev, const float* grad_t_dev, int64_t num_pixels,
                                    int num_primitives, float* d4_dev, float* grad_positions_dev,
                                    float* grad_log_scales_dev, float* grad_quats_dev, mlpsp_stream_t stream) {
  if (num_pixels < 0 || num_primitives < 0 || num_pixels > 2147483647LL * 128) return MLPSP_E_ARGUMENT;
  hipStream_t s = (hipStream_t)stream;
  if (num_primitives > 0) {
    if (!grad_positions_dev || !grad_log_scales_dev || !grad_quats_dev) return MLPSP_E_ARGUMENT;
    MLPSP_HIP_TRY(hipMemsetAsync(grad_positions_dev, 0, sizeof(float) * 3 * (size_t)num_primitives, s));
    MLPSP_HIP_TRY(hipMemsetAsync(grad_log_scales_dev, 0, sizeof(float) * 3 * (size_t)num_primitives, s));
    MLPSP_HIP_TRY(hipMemsetAsync(grad_quats_dev, 0, sizeof(float) * 4 * (size_t)num_primitives, s));
  }
  if (num_pixels == 0) return MLPSP_OK;
  if (!pixel_offsets_dev || !grad_rgb_dev || !grad_t_dev) return MLPSP_E_ARGUMENT;
  // record arrays may be null only if there are no records (the offsets then end at zero)
  if (((uintptr_t)raw_dev | (uintptr_t)d4_dev | (uintptr_t)quats_dev) & 15u) return MLPSP_E_ARGUMENT;
  const dim3 grid((unsigned)((num_pixels + 127) / 128)), block(128);
  hipLaunchKernelGGL(records_reverse_kernel<true>, grid, block, 0, s, ids_dev, (const long long*)pixel_offsets_dev,
                     x6_dev, raw_dev, log_scales_dev, quats_dev, grad_rgb_dev, grad_t_dev, (long long)num_pixels, d4_dev,
                     grad_positions_dev, grad_log_scales_dev, grad_quats_dev, (float*)nullptr);
  MLPSP_LAUNCH_CHECK();
  return MLPSP_OK;
}

MLPSP_API int mlpsp_records_reverse_adjoints(const int32_t* ids_dev, const int64_t* pixel_offsets_dev,
                                             const float* raw_dev, const float* grad_rgb_dev, const float* grad_t_dev,
                                             int64_t num_pixels, float* d4_dev, float* falloff_adjoint_dev,
                                             mlpsp_stream_t stream) {
  if (num_pixels < 0 || num_pixels > 2147483647LL * 128) return MLPSP_E_ARGUMENT;
  if (num_pixels == 0) return MLPSP_OK;
  if (!pixel_offsets_dev || !grad_rgb_dev || !grad_t_dev) return MLPSP_E_ARGUMENT;
  if (((uintptr_t)raw_dev | (uintptr_t)d4_dev) & 15u) return MLPSP_E_ARGUMENT;
  const dim3 grid((unsigned)((num_pixels + 127) / 128)), block(128);
  hipLaunchKernelGGL(records_reverse_kernel<false>, grid, block, 0, (hipStream_t)stream, ids_dev,
                     (const long long*)pixel_offsets_dev, (const float*)nullptr, raw_dev, (const float*)nullptr,
                     (const float*)nullptr, grad_rgb_dev, grad_t_dev, (long long)num_pixels, d4_dev, (float*)nullptr,
                     (float*)nullptr, (float*)nullptr, falloff_adjoint_dev);
  MLPSP_LAUNCH_CHECK();
  return MLPSP_OK;
}

MLPSP_API int mlpsp_geometry_gradients(const int64_t* csr_offsets_dev, const int64_t* record_indices_dev,
                                       const float* x6_sorted_dev, const float* falloff_adjoint_dev,
                                       const float* log_scales_dev, const float* quats_dev,
                                       const int64_t* group_primitives_dev, const int64_t* group_starts_dev,
                                       const int64_t* group_offsets_dev, int64_t num_groups, int segment,
                                       int num_primitives, float* partial_dev, float* grad_positions_dev,
                                       float* grad_log_scales_dev, float* grad_quats_dev, mlpsp_stream_t stream) {
  if (num_primitives < 0 || num_groups < 0 || num_groups > 2147483647LL * 4 || segment <= 0) return MLPSP_E_ARGUMENT;
  if (num_primitives == 0) return MLPSP_OK;
  if (!csr_offsets_dev || !log_scales_dev || !quats_dev || !group_offsets_dev || !grad_positions_dev ||
      !grad_log_scales_dev || !grad_quats_dev)
    return MLPSP_E_ARGUMENT;
  hipStream_t s = (hipStream_t)stream;
  if (num_groups > 0) {
    if (!record_indices_dev || !x6_sorted_dev || !falloff_adjoint_dev || !group_primitives_dev || !group_starts_dev ||
        !partial_dev)
      return MLPSP_E_ARGUMENT;
    hipLaunchKernelGGL(geometry_partials_kernel, dim3((unsigned)((num_groups + 3) / 4)), dim3(256), 0, s,
                       (const long long*)csr_offsets_dev, (const long long*)record_indices_dev, x6_sorted_dev,
                       falloff_adjoint_dev, log_scales_dev, quats_dev, (const long long*)group_primitives_dev,
                       (const long long*)group_starts_dev, (long long)num_groups, segment, partial_dev);
    MLPSP_LAUNCH_CHECK();
  }
  hipLaunchKernelGGL(geometry_finish_kernel, dim3((unsigned)((num_primitives + 255) / 256)), dim3(256), 0, s,
                     partial_dev, (const long long*)group_offsets_dev, quats_dev, num_primitives, grad_positions_dev,
                     grad_log_scales_dev, grad_quats_dev);
  MLPSP_LAUNCH_CHECK();
  return MLPSP_OK;
}
