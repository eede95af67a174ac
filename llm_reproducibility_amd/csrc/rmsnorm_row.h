// RMSNorm of ONE row by ONE wavefront, shared by the stand-alone kernel (reductions.hip) and by the matmul that
// normalises its activations while it stages them (gemm_single_acc_stream.hip): one body, so both give the same bits.
//
// Lane l owns the 16-byte chunks l, l+64, l+128, ... of the row (8 elements each, CPL of them at most); the sum of
// squares runs sequentially inside a lane (chunk by chunk, element by element, fused multiply-adds) and then through
// the fixed butterfly across the lanes.  Arithmetic as vLLM's RMSNorm.forward_native, which the reference routes to
// (src/patch/patch_batch_invariant.py:9-16): fp32 math, an optional residual added in fp32 with the sum rounded to the
// element type as the new residual, the normalised value rounded to the element type, then a multiply by the weight in
// the element type.
#pragma once
#include "common.h"

namespace tbik {

// The row of one lane in flight: `load` issues every load of the row (activations, residual, weights) and returns at
// once; `finish` consumes them.  A caller with other loads to issue (the weight stream of a matmul) puts them between
// the two: a wave's loads return in the order they were issued, so the row must be asked for first or it would wait
// behind the stream.
//
// x, res (may be null), w (may be null), res_out (may be null: the sum is not stored): rows of `hidden` elements, 16-byte
// aligned.  `store(c, chunk)` receives output chunk c (elements 8c .. 8c+7) of this lane.
// UNCOND: every load is issued whatever the arguments (chunks past the end of the row re-read its last chunk, a missing
// residual or weight vector re-reads the row) and the spare values are never used.  A caller that issues further loads
// behind the row needs this: the compiler counts outstanding loads per path, and loads under branches make it wait for
// ALL of them, the caller's included, before the first use.
template <int CPL, bool F16, bool UNCOND = false>
struct RmsnormRow {
  using Num = Num16<F16>;
  uint4 xq[CPL], rq[CPL], wq[CPL];
  bool has_res, has_w;

  __device__ __forceinline__ void load(const uint16_t* x, const uint16_t* res, const uint16_t* w, int hidden, int lane) {
    const int nchunks = hidden >> 3;
    const uint4* xr = reinterpret_cast<const uint4*>(x);
    const uint4* rr = reinterpret_cast<const uint4*>(res);
    // the weights do not depend on the row: fetched together with it, not after the reduction (with a single row
    // the kernel is nothing but memory round trips in a chain)
    const uint4* wr = reinterpret_cast<const uint4*>(w);
    has_res = res != nullptr;
    has_w = w != nullptr;
    if constexpr (UNCOND) {
      rr = rr ? rr : xr;
      wr = wr ? wr : xr;
#pragma unroll
      for (int i = 0; i < CPL; i++) {
        const int c = min(lane + 64 * i, nchunks - 1);
        xq[i] = xr[c];
        rq[i] = rr[c];
        wq[i] = wr[c];
      }
      return;
    }
    if (wr) {
#pragma unroll
      for (int i = 0; i < CPL; i++) {
        const int c = lane + 64 * i;
        if (c < nchunks) wq[i] = wr[c];
      }
    }
    // all loads of the row go out before the first store: the residual output may alias the inputs as far as the
    // compiler knows, and loads issued behind a store would wait for one memory round trip per chunk
#pragma unroll
    for (int i = 0; i < CPL; i++) {
      const int c = lane + 64 * i;
      if (c < nchunks) {
        xq[i] = xr[c];
        if (rr) rq[i] = rr[c];
      }
    }
  }

  template <typename Store>
  __device__ __forceinline__ void finish(uint16_t* res_out, int hidden, float eps, int lane, Store&& store) {
    const int nchunks = hidden >> 3;
    float v[CPL][8];
    float ss = 0.f;
#pragma unroll
    for (int i = 0; i < CPL; i++) {
      const int c = lane + 64 * i;
      if (c < nchunks) {
        const uint32_t u[4] = {xq[i].x, xq[i].y, xq[i].z, xq[i].w};
#pragma unroll
        for (int e = 0; e < 4; e++) {
          v[i][2 * e] = Num::lo(u[e]);
          v[i][2 * e + 1] = Num::hi(u[e]);
        }
        if (has_res) {
          const uint32_t ru[4] = {rq[i].x, rq[i].y, rq[i].z, rq[i].w};
          uint32_t so[4];
#pragma unroll
          for (int e = 0; e < 4; e++) {
            v[i][2 * e] += Num::lo(ru[e]);
            v[i][2 * e + 1] += Num::hi(ru[e]);
            so[e] = Num::pack(v[i][2 * e], v[i][2 * e + 1]);
          }
          if (res_out) reinterpret_cast<uint4*>(res_out)[c] = make_uint4(so[0], so[1], so[2], so[3]);
        }
#pragma unroll
        for (int e = 0; e < 8; e++) ss = fmaf(v[i][e], v[i][e], ss);
      }
    }
    ss = wave_sum(ss);
    const float var = ss / (float)hidden;
    const float rs = 1.0f / sqrtf(var + eps);
#pragma unroll
    for (int i = 0; i < CPL; i++) {
      const int c = lane + 64 * i;
      if (c < nchunks) {
        uint32_t o[4];
#pragma unroll
        for (int e = 0; e < 4; e++) o[e] = Num::pack(v[i][2 * e] * rs, v[i][2 * e + 1] * rs);
        if (has_w) {
          const uint32_t wu[4] = {wq[i].x, wq[i].y, wq[i].z, wq[i].w};
#pragma unroll
          for (int e = 0; e < 4; e++)
            o[e] = Num::pack(Num::lo(o[e]) * Num::lo(wu[e]), Num::hi(o[e]) * Num::hi(wu[e]));
        }
        store(c, make_uint4(o[0], o[1], o[2], o[3]));
      }
    }
  }
};

template <int CPL, bool F16, typename Store>
__device__ __forceinline__ void rmsnorm_row(const uint16_t* x, const uint16_t* res, const uint16_t* w, uint16_t* res_out,
                                            int hidden, float eps, int lane, Store&& store) {
  RmsnormRow<CPL, F16> row;
  row.load(x, res, w, hidden, lane);
  row.finish(res_out, hidden, eps, lane, store);
}

}  // namespace tbik
