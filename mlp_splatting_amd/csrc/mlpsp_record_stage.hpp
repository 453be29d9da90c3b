// Staging of training records on their way to global memory, for the emit passes of the record forwards.
//
// A record is 84 bytes in five arrays (ids 4, x6 24, masks 8, raw 32, gates 16), and the records of one pixel
// are consecutive; a wavefront produces one record per hitting pixel and step.  Written as they are produced,
// every store instruction touches 64 different cache lines with 4..16 bytes each: at the 200k-primitive frame
// the hardware counters show 7.0 GB written for 3.2 GB of records (lines leave L2 partly filled and come back)
// and 2.9 GB of weights fetched again that those lines pushed out -- the emit pass of the matrix-core record
// forward takes 3.4 ms where the same pass without its stores takes 1.1 ms.
//
// Here a pixel's records wait in LDS until one pixel of the wavefront has K of them; then the wavefront writes
// every pixel's pending records out together, lanes walking the staged records in memory order, so that the K
// records of a pixel leave as one contiguous piece per array (K x 32 bytes of raw, ...).  One wavefront per
// workgroup: no barrier, LDS operations of a wavefront execute in order.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace mlpsp {

struct RecordArrays {
  int32_t* ids;     // [R]
  float* x6;        // [R,6]
  int32_t* masks;   // [R,2]
  float* raw;       // [R,8]
  float* gates;     // [R,4]
};

// Row strides (dwords per pixel) are padded so that the 64 lanes of a put land in different banks.
template <int K>
struct RecordStage {
  static_assert(K == 2 || K == 4, "K is a power of two");
  static constexpr int LR = K * 8 + 4, LG = K * 4 + 4, LX = K * 3 + 1, LM = K * 2 + 2, LI = K + 1;
  __attribute__((aligned(16))) float raw[64 * LR];
  __attribute__((aligned(16))) float gates[64 * LG];
  float x3[64 * LX];
  __attribute__((aligned(8))) int32_t masks[64 * LM];
  int32_t ids[64 * LI];
  float rd[64 * 3];
  long long dst[64];
  int cnt[64];
};

template <int K>
__device__ __forceinline__ void stage_begin(RecordStage<K>& s, int lane, float rdx, float rdy, float rdz) {
  s.rd[lane * 3 + 0] = rdx;
  s.rd[lane * 3 + 1] = rdy;
  s.rd[lane * 3 + 2] = rdz;
}

// lane = pixel; slot = how many records of this pixel are already waiting (< K)
template <int K>
__device__ __forceinline__ void stage_put(RecordStage<K>& s, int lane, int slot, int id, float dx, float dy, float dz,
                                          unsigned mask1, unsigned mask2, const float raw[8], const float gates[4]) {
  using S = RecordStage<K>;
  float4* r = reinterpret_cast<float4*>(&s.raw[lane * S::LR + slot * 8]);
  r[0] = make_float4(raw[0], raw[1], raw[2], raw[3]);
  r[1] = make_float4(raw[4], raw[5], raw[6], raw[7]);
  *reinterpret_cast<float4*>(&s.gates[lane * S::LG + slot * 4]) = make_float4(gates[0], gates[1], gates[2], gates[3]);
  float* x = &s.x3[lane * S::LX + slot * 3];
  x[0] = dx;
  x[1] = dy;
  x[2] = dz;
  *reinterpret_cast<int2*>(&s.masks[lane * S::LM + slot * 2]) = make_int2((int)mask1, (int)mask2);
  s.ids[lane * S::LI + slot] = id;
}

// Every pixel's `count` waiting records go to records first .. first + count - 1 (first, count: this lane's pixel).
template <int K>
__device__ __forceinline__ void stage_flush(RecordStage<K>& s, int lane, long long first, int count, const RecordArrays& out) {
  using S = RecordStage<K>;
  s.dst[lane] = first;
  s.cnt[lane] = count;
  // raw: 2 K pieces of 16 bytes per pixel
#pragma unroll
  for (int it = 0; it < 2 * K; ++it) {
    const int item = it * 64 + lane, px = item / (2 * K), sub = item % (2 * K), j = sub >> 1, half = sub & 1;
    if (j < s.cnt[px])
      *reinterpret_cast<float4*>(out.raw + (s.dst[px] + j) * 8 + half * 4) =
          *reinterpret_cast<const float4*>(&s.raw[px * S::LR + j * 8 + half * 4]);
  }
  // gates: K pieces of 16 bytes per pixel
#pragma unroll
  for (int it = 0; it < K; ++it) {
    const int item = it * 64 + lane, px = item / K, j = item % K;
    if (j < s.cnt[px])
      *reinterpret_cast<float4*>(out.gates + (s.dst[px] + j) * 4) = *reinterpret_cast<const float4*>(&s.gates[px * S::LG + j * 4]);
  }
  // x6: per record the pixel's ray direction and the record's hit offset, 12 bytes each
#pragma unroll
  for (int it = 0; it < 2 * K; ++it) {
    const int item = it * 64 + lane, px = item / (2 * K), sub = item % (2 * K), j = sub >> 1, half = sub & 1;
    if (j < s.cnt[px]) {
      const float* src = half ? &s.x3[px * S::LX + j * 3] : &s.rd[px * 3];
      float* dstp = out.x6 + (s.dst[px] + j) * 6 + half * 3;
      const float a = src[0], b = src[1], c = src[2];
      dstp[0] = a;
      dstp[1] = b;
      dstp[2] = c;
    }
  }
  // masks (8 bytes) and ids (4 bytes)
#pragma unroll
  for (int it = 0; it < K; ++it) {
    const int item = it * 64 + lane, px = item / K, j = item % K;
    if (j < s.cnt[px]) {
      *reinterpret_cast<int2*>(out.masks + (s.dst[px] + j) * 2) = *reinterpret_cast<const int2*>(&s.masks[px * S::LM + j * 2]);
      out.ids[s.dst[px] + j] = s.ids[px * S::LI + j];
    }
  }
}

}  // namespace mlpsp
