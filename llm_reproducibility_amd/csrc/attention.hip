// Fixed-order causal attention for gfx950 (bf16, head_dim 128, grouped-query heads).  A query row is always the four
// lanes {j, j+16, j+32, j+48} of one wavefront; three kernels differ in what else the wavefront and its work-group hold:
//   attention_kernel        one wavefront per (16 consecutive queries of a sequence, query head), operands from global
//                           memory (any cache length);
//   attention_group_kernel  the G query heads of a KV head as the G wavefronts of a work-group, K/V tiles staged in LDS
//                           once for all of them (prefill and chunked prefill);
//   attention_decode_kernel the few new queries of a sequence times the G heads as the 16 rows of ONE tile, the output
//                           channels split over four wavefronts, four more wavefronts bringing the tiles in (decode).
//
// Counterpart of the reference's fixed-tile attention for train/inference alignment
// (_kernel_unified_attention_2d, src/patch/patch_training_inference_align.py:171-487: one pass over the
// keys in tiles of 32, online softmax, no split over the key axis, the same kernel for prefill and decode).
//
// Invariance argument: a query row is owned by the four lanes {j, j+16, j+32, j+48}; its scores, its
// running maximum / denominator and its output accumulators never mix with another row's.  Keys are
// visited in ascending tiles of 32 whatever the batch or the block looks like; a tile that lies entirely
// behind a row's causal horizon contributes exp(-inf) = 0 and a rescale by exactly 1.0, so the number of
// tiles the BLOCK walks does not change the row.  Prefill (16 rows per block) and decode (1 valid row)
// therefore produce the same bits for the same token, and heads can be sharded freely.
//
// Layouts: q/out [tokens, q_heads, 128]; K cache [batch, kv_heads, max_len, 128]; V cache TRANSPOSED
// [batch, kv_heads, 128, max_len] so that the P*V MFMA operand (8 consecutive keys of one channel) is a
// contiguous load.  Cache entries behind ctx_len must be finite (they are multiplied by an exact 0).
#include "common.h"
#include "lds_direct.h"
#include "qk_norm_rope.h"

namespace tbik {

struct AttnArgs {
  const uint16_t* q;
  const uint16_t* k_cache;
  const uint16_t* vt_cache;
  uint16_t* out;
  const int* q_start;  // [batch] first token row of the sequence in q/out
  const int* q_len;    // [batch] new tokens of the sequence
  const int* ctx_len;  // [batch] keys visible to the LAST new token (cache length including the new tokens)
  int q_heads, kv_heads, max_len;
  float scale_log2;    // log2(e) / sqrt(head_dim): scores are kept in the base-2 domain
};

constexpr int HD = 128;

// The decode kernel that forms its own queries and the new key/value (FUSED): sequence b's one new token is row b of the
// fused qkv projection output, at position ctx_len[b] - 1.
struct QkvArgs {
  const uint16_t* qkv;    // [batch, (q_heads + 2 kv_heads) * 128], row stride ld
  int64_t ld;
  const uint16_t* qw;     // per-head q norm weight [128]
  const uint16_t* kw;     // per-head k norm weight [128]
  const float* inv_freq;  // [64]
  uint16_t* k_cache;      // the caches of AttnArgs, writable: the new key and value are filed here as well
  uint16_t* vt_cache;
  float eps;
};

// One online-softmax update of a query row for a tile of 32 keys, shared by all kernels of this file (one body: the same
// bits).  Lane (j, g) holds the scores of query j for keys k0 + 16u + 4g + i in s[u][i]; on return p holds the four packed
// probability pairs of the lane (the B operand of the P*V MFMA) and alpha the factor for the output accumulators of the
// row (exactly 1.0 when the reference point of the exponentials did not move).  MASK: apply the causal mask (needed only for tiles that
// reach beyond some row's horizon; the values are the same either way for the others).
// 2^x is the hardware exponential: the arguments are <= 0, and a result below 2^-126 is dropped, which neither the
// denominator (>= 1: the row's maximum contributes 2^0) nor a bf16 probability can show.
template <bool MASK>
__device__ __forceinline__ void softmax_tile(const f32x4 (&s)[2], int k0, int g, int qpos, float scale_log2, float& m, float& l,
                                             float& alpha, bf16x8& p) {
  // every product and sum below is rounded on its own, except where a fused multiply-add is written out: left to the
  // compiler, a multiplication could be fused with the next addition in one instantiation and not in another, and the
  // kernels would no longer agree bit for bit
#pragma clang fp contract(off)
  float sv[8];
#pragma unroll
  for (int u = 0; u < 2; u++)
#pragma unroll
    for (int i = 0; i < 4; i++) {
      float v = s[u][i];
      if (MASK) v = (k0 + 16 * u + 4 * g + i <= qpos) ? v : -INFINITY;
      sv[4 * u + i] = v;
    }
  // the maximum is taken over the raw scores and scaled once (the scale is positive and rounding is monotonic, so this
  // is the maximum of the scaled scores); 2^(score * scale - maximum) is then one fused multiply-add and one exponential
  // (NaN-propagating maxima: a NaN score makes the row NaN, as it would through the sum)
  float tmax = LaneMaxNaN::f(LaneMaxNaN::f(LaneMaxNaN::f(sv[0], sv[1]), LaneMaxNaN::f(sv[2], sv[3])),
                             LaneMaxNaN::f(LaneMaxNaN::f(sv[4], sv[5]), LaneMaxNaN::f(sv[6], sv[7])));
  tmax = xor_step<16, LaneMaxNaN>(tmax);
  tmax = xor_step<32, LaneMaxNaN>(tmax);
  // The reference point of the exponentials moves lazily: only when a score of this tile exceeds it by more than 2^kLazy
  // (probabilities then stay below 2^kLazy instead of 1: no loss in fp32 sums or in the relative precision of a bf16
  // probability, and out = o / l is the same quotient).  After the first tiles of a row it practically never moves, so
  // the rescale of the output accumulators is skipped for whole rows of tiles.  The rule looks at a row's own scores
  // in its fixed tile order only, so it is the same for prefill, chunked prefill and decode.
  // Key 0 is visible to every query: the reference point is finite from tile 0 on.
  constexpr float kLazy = 8.0f;
  const float cand = tmax * scale_log2;
  const float m_new = cand > m + kLazy ? cand : m;
  alpha = __builtin_amdgcn_exp2f(m - m_new);        // exactly 1.0 when the reference point did not move
  float pv[8];
#pragma unroll
  for (int e = 0; e < 8; e++) pv[e] = __builtin_amdgcn_exp2f(__builtin_fmaf(sv[e], scale_log2, -m_new));
  float psum = pv[0];
#pragma unroll
  for (int e = 1; e < 8; e++) psum += pv[e];
  psum = xor_step<16, LaneSum>(psum);
  psum = xor_step<32, LaneSum>(psum);
  l = __builtin_fmaf(l, alpha, psum);
  m = m_new;
  // P as the MFMA "B" operand: k slots 0..3 = keys k0+4g.., slots 4..7 = keys k0+16+4g..
  p = __builtin_bit_cast(bf16x8, u32x4{pack_bf16x2(pv[0], pv[1]), pack_bf16x2(pv[2], pv[3]), pack_bf16x2(pv[4], pv[5]),
                                       pack_bf16x2(pv[6], pv[7])});
}

__global__ __launch_bounds__(64) void attention_kernel(const AttnArgs a) {
  const int b = blockIdx.z;
  const int h = blockIdx.y;
  const int qb = blockIdx.x;
  const int qlen = a.q_len[b];
  if (qb * 16 >= qlen) return;
  const int lane = threadIdx.x;
  const int j = lane & 15;   // query row inside the block (also: key row of a K fragment, channel row of a V fragment)
  const int g = lane >> 4;   // lane group: which 8-wide k slice of an MFMA operand, which 4 rows of an MFMA result
  const int ctx = a.ctx_len[b];
  const int kvh = h / (a.q_heads / a.kv_heads);
  const int qrow = qb * 16 + j;                     // row inside the sequence's new tokens
  const bool qvalid = qrow < qlen;
  const int qpos = ctx - qlen + min(qrow, qlen - 1);  // absolute position of this lane's query
  const int last_pos = ctx - qlen + min(qb * 16 + 15, qlen - 1);

  // Q as the MFMA "B" operand: lane (j, g) holds q[j][32c + 8g .. +7] for the four 32-wide channel chunks c
  const uint16_t* qp = a.q + ((int64_t)(a.q_start[b] + min(qrow, qlen - 1)) * a.q_heads + h) * HD;
  bf16x8 qf[4];
#pragma unroll
  for (int c = 0; c < 4; c++) qf[c] = *reinterpret_cast<const bf16x8*>(qp + c * 32 + g * 8);

  const uint16_t* kbase = a.k_cache + ((int64_t)b * a.kv_heads + kvh) * a.max_len * HD;
  const uint16_t* vbase = a.vt_cache + ((int64_t)b * a.kv_heads + kvh) * (int64_t)HD * a.max_len;

  f32x4 o[8];  // output accumulators, transposed: lane (j, g) holds out[j][16t + 4g .. +3] for the channel tiles t
#pragma unroll
  for (int t = 0; t < 8; t++) o[t] = f32x4{0.f, 0.f, 0.f, 0.f};
  float m = -INFINITY;  // reference point of the exponentials (base-2 domain; a lazily updated running maximum), identical in the four lanes of a row
  float l = 0.f;        // running denominator

  const int ntiles = last_pos / 32 + 1;
  for (int tile = 0; tile < ntiles; tile++) {
    const int k0 = tile * 32;
    // ---- scores: two 16-key sub-tiles; lane (j, g) receives keys k0 + 16u + 4g + i of query j
    f32x4 s[2];
#pragma unroll
    for (int u = 0; u < 2; u++) {
      const int krow = min(k0 + 16 * u + j, a.max_len - 1);
      const uint16_t* kp = kbase + (int64_t)krow * HD + g * 8;
      f32x4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int c = 0; c < 4; c++) {
        const bf16x8 kf = *reinterpret_cast<const bf16x8*>(kp + c * 32);
        acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf, qf[c], acc, 0, 0, 0);
      }
      s[u] = acc;
    }
    float alpha;
    bf16x8 pf;
    softmax_tile<true>(s, k0, g, qpos, a.scale_log2, m, l, alpha, pf);
    // ---- out^T += V^T * P: "A" operand lane (j, g) holds channel 16t + j, the same 8 key slots
    const int kv0 = min(k0 + 4 * g, a.max_len - 4);
    const int kv1 = min(k0 + 16 + 4 * g, a.max_len - 4);
#pragma unroll
    for (int t = 0; t < 8; t++) {
      const uint16_t* vp = vbase + (int64_t)(16 * t + j) * a.max_len;
      const uint2 va = *reinterpret_cast<const uint2*>(vp + kv0);
      const uint2 vb = *reinterpret_cast<const uint2*>(vp + kv1);
      const bf16x8 vf = __builtin_bit_cast(bf16x8, u32x4{va.x, va.y, vb.x, vb.y});
      f32x4 scaled = {o[t][0] * alpha, o[t][1] * alpha, o[t][2] * alpha, o[t][3] * alpha};
      o[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf, pf, scaled, 0, 0, 0);
    }
  }
  if (!qvalid) return;
  const float inv = 1.0f / l;
  uint16_t* op = a.out + ((int64_t)(a.q_start[b] + qrow) * a.q_heads + h) * HD;
#pragma unroll
  for (int t = 0; t < 8; t++) {
    const uint32_t lo = pack_bf16x2(o[t][0] * inv, o[t][1] * inv);
    const uint32_t hi = pack_bf16x2(o[t][2] * inv, o[t][3] * inv);
    *reinterpret_cast<uint2*>(op + 16 * t + 4 * g) = make_uint2(lo, hi);
  }
}

// ------------------------------------------------------------------------------------------------
// Grouped variant: one work-group per (16 consecutive queries, KV head, sequence); its G wavefronts are the G query
// heads that share the KV head.  Each 32-key tile of K and of V^T is fetched from global memory ONCE per group with
// coalesced 16-byte loads, staged in LDS (double buffered; K rows XOR-swizzled against bank conflicts, V^T rows stored in
// fragment order) and read from there
// by every wave.  A row's arithmetic -- the lanes that own it, the MFMA chain, the order of the softmax updates --
// is exactly that of attention_kernel above, so both kernels produce the same bits; this one just moves 1/G of
// the bytes and hides the load latency behind the previous tile.
// NLD > 0: that many more wavefronts in the work-group do all the staging (loads, LDS writes) at the same barriers and
// the G computing waves none of it: for launches that leave the chip short of work-groups, where a work-group's time is
// its own chain of tiles rather than its share of a CU.
// ------------------------------------------------------------------------------------------------
template <int G, bool DEEP, int NLD = 0>
__global__ __launch_bounds__(64 * (G + NLD)) void attention_group_kernel(const AttnArgs a) {
  __shared__ __attribute__((aligned(16))) uint8_t lds[2][16384];  // per buffer: K tile [32][128] (8 KiB), V^T tile [128][32] (8 KiB)
  const int b = blockIdx.y;
  // Work-groups are dealt to the eight XCDs round robin, each with an L2 of its own: with the KV head as the fastest
  // index every XCD serves the query blocks of the same few KV heads, and the key tiles those blocks share (every block
  // of a head walks the same keys) stay in ITS L2 instead of being fetched by all eight.
  // Causal attention: the last query blocks have the most keys, so they are dispatched first (longest work first
  // keeps the tail of the launch short); which work-group computes a block has no numeric effect.
  const int kvh = blockIdx.x % a.kv_heads;
  const int qb = gridDim.x / a.kv_heads - 1 - blockIdx.x / a.kv_heads;
  const int qlen = a.q_len[b];
  if (qb * 16 >= qlen) return;  // uniform over the work-group
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int h = kvh * G + (tid >> 6);
  const int j = lane & 15;
  const int g = lane >> 4;
  const int ctx = a.ctx_len[b];
  const int qrow = qb * 16 + j;
  const bool qvalid = qrow < qlen;
  const int qpos = ctx - qlen + min(qrow, qlen - 1);
  const int last_pos = ctx - qlen + min(qb * 16 + 15, qlen - 1);

  const uint8_t* kbase = reinterpret_cast<const uint8_t*>(a.k_cache + ((int64_t)b * a.kv_heads + kvh) * a.max_len * HD);
  const uint8_t* vbase = reinterpret_cast<const uint8_t*>(a.vt_cache + ((int64_t)b * a.kv_heads + kvh) * (int64_t)HD * a.max_len);

  // cooperative staging: 512 16-byte chunks per tile and operand, NCH per thread
  // (NLD loader waves, where the kernel has them, do all of it; the computing waves then neither load nor store tiles)
  constexpr int NT = NLD ? 64 * NLD : 64 * G;
  const int stid = NLD ? tid - 64 * G : tid;   // staging thread
  constexpr int NCH = (512 + NT - 1) / NT;
  // Key tiles are fetched DEPTH tiles ahead into DEPTH register sets (set = tile % DEPTH).  DEEP is for decode: a
  // single block of queries per sequence makes the kernel a chain of memory round trips, and one tile of arithmetic
  // hides none of them.  Prefill has arithmetic to overlap and prefers the registers (more waves per SIMD).
  constexpr int DEPTH = !DEEP ? 1 : (NCH <= 2 ? 4 : (NCH <= 4 ? 2 : 1));
  u32x4 kregs[DEPTH][NCH], vregs[DEPTH][NCH];
  // A K tile is 8 KiB of consecutive bytes (32 rows of 256), chunk ch at byte 16 ch; a V^T tile is 128 rows of 64 bytes,
  // max_len elements apart.  Per-thread byte offsets inside a tile (global and LDS side) are formed once; per tile only
  // a wave-uniform base moves, so the loads take a scalar base and the loop spends no vector instruction on addresses.
  uint32_t vsrc[NCH], kdst[NCH], vdst0[NCH], vdst1[NCH];
#pragma unroll
  for (int i = 0; i < NCH; i++) {
    const int ch = min(max(stid, 0) + i * NT, 511);
    const int kr = ch >> 4, kc = ch & 15;   // key row, 16-byte chunk of its 256 bytes
    kdst[i] = kr * 256 + ((kc ^ (2 * (kr & 7))) << 4);
    // V^T: channel row vr (64 bytes = 32 keys), 16-byte chunk vc = keys 8vc .. 8vc+7.  The keys of a row are stored
    // in the order a P*V fragment wants them -- lane group g takes keys 4g..4g+3 and 16+4g..16+4g+3 -- so that a
    // fragment is ONE 16-byte read at byte 16g of the row: keys 4a..4a+3 live in the 8-byte slot 2 (a & 3) + (a >> 2).
    // A 16-byte read is served for lanes {0-7, 16-23} together (then {8-15, 24-31}, ...): rows j and j + 4 of a 64-byte
    // pitch meet in the same banks, so rows with bit 2 set keep their chunks in the other half of the row (chunk ^ 2,
    // i.e. 8-byte slot ^ 4) and the sixteen lanes of a phase cover all 64 banks.
    const int vr = ch >> 2, vc = ch & 3;
    const int vx = 4 * ((vr >> 2) & 1);
    vsrc[i] = (uint32_t)vr * (uint32_t)a.max_len * 2u + vc * 16;
    vdst0[i] = 8192 + vr * 64 + ((2 * ((2 * vc) & 3) + (vc >> 1)) ^ vx) * 8;
    vdst1[i] = 8192 + vr * 64 + ((2 * ((2 * vc + 1) & 3) + (vc >> 1)) ^ vx) * 8;
  }
  // this (sequence, KV head)'s slice of each cache as a raw buffer (no stride, extent in bytes; the dispatcher keeps
  // max_len small enough for 32-bit offsets)
  const __amdgpu_buffer_rsrc_t krsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint8_t*>(kbase), 0, a.max_len * (HD * 2), 0x00020000);
  const __amdgpu_buffer_rsrc_t vrsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint8_t*>(vbase), 0, a.max_len * (HD * 2), 0x00020000);
  auto load_tile = [&](int tile, int set) __attribute__((always_inline)) {
    u32x4* kreg = kregs[set];
    u32x4* vreg = vregs[set];
    const int k0 = min(tile * 32, a.max_len - 32);  // max_len is a multiple of 32: never past the cache
    // buffer loads: the descriptors (one per cache, in scalar registers) and the tile's byte offset are wave-uniform,
    // the per-thread offsets are the constants formed above -- no vector instruction per load
    const int ks = k0 * (HD * 2), vs = k0 * 2;
#pragma unroll
    for (int i = 0; i < NCH; i++) {
      if (512 % NT == 0 || stid + i * NT < 512) {
        kreg[i] = __builtin_amdgcn_raw_buffer_load_b128(krsrc, (stid + i * NT) * 16, ks, 0);
        vreg[i] = __builtin_amdgcn_raw_buffer_load_b128(vrsrc, (int)vsrc[i], vs, 0);
      }
    }
  };
  auto store_tile = [&](int buf, int set) __attribute__((always_inline)) {
    const u32x4* kreg = kregs[set];
    const u32x4* vreg = vregs[set];
#pragma unroll
    for (int i = 0; i < NCH; i++) {
      if (512 % NT == 0 || stid + i * NT < 512) {
        *reinterpret_cast<u32x4*>(&lds[buf][kdst[i]]) = kreg[i];
        *reinterpret_cast<uint2*>(&lds[buf][vdst0[i]]) = make_uint2(vreg[i][0], vreg[i][1]);
        *reinterpret_cast<uint2*>(&lds[buf][vdst1[i]]) = make_uint2(vreg[i][2], vreg[i][3]);
      }
    }
  };

  const int ntiles = last_pos / 32 + 1;
  constexpr int UNROLL = DEPTH < 2 ? 2 : DEPTH;
  if (NLD && stid >= 0) {
    // ---- loader waves: the staging half of the loop below, at the same barriers
#pragma unroll
    for (int d = 0; d < DEPTH; d++) load_tile(d, d);
    store_tile(0, 0);
    __syncthreads();
    for (int t0 = 0; t0 < ntiles; t0 += UNROLL) {
#pragma unroll
      for (int d = 0; d < UNROLL; d++) {
        const int tile = t0 + d;
        if (tile >= ntiles) break;
        load_tile(tile + DEPTH, d % DEPTH);
        if (tile + 1 < ntiles) store_tile((d & 1) ^ 1, (d + 1) % DEPTH);
        __syncthreads();
      }
    }
    return;
  }
  const uint16_t* qp = a.q + ((int64_t)(a.q_start[b] + min(qrow, qlen - 1)) * a.q_heads + h) * HD;
  bf16x8 qf[4];
#pragma unroll
  for (int c = 0; c < 4; c++) qf[c] = *reinterpret_cast<const bf16x8*>(qp + c * 32 + g * 8);

  f32x4 o[8];
#pragma unroll
  for (int t = 0; t < 8; t++) o[t] = f32x4{0.f, 0.f, 0.f, 0.f};
  float m = -INFINITY;
  float l = 0.f;

  // LDS offsets of this lane's fragments inside a tile buffer, formed once: key row 16u + j of the K tile (256 bytes a
  // row, 16-byte chunk c*4 + g swizzled by the row; u adds 4096), channel row 16t + j of the V^T tile (64 bytes a row,
  // the lane group's eight keys are the 16-byte chunk g, or g ^ 2 in rows with bit 2 set; t adds 1024)
  uint32_t kofs[4];
#pragma unroll
  for (int c = 0; c < 4; c++) kofs[c] = j * 256 + (((c * 4 + g) ^ (2 * (j & 7))) << 4);
  const uint32_t vofs = 8192 + j * 64 + (g ^ (2 * ((j >> 2) & 1))) * 16;

  // loads past the last tile are clamped to a valid address and never used: issuing them unconditionally keeps the
  // number of loads in flight static, so the waits below can leave the newer tiles in flight
  if (!NLD) {
#pragma unroll
    for (int d = 0; d < DEPTH; d++) load_tile(d, d);
    store_tile(0, 0);
  }
  __syncthreads();
  // the loop body covers UNROLL (an even number of) tiles, so that the LDS buffer of each is a compile-time constant and
  // every LDS address is a per-thread offset plus an immediate
  for (int t0 = 0; t0 < ntiles; t0 += UNROLL) {
#pragma unroll
   for (int d = 0; d < UNROLL; d++) {
    const int tile = t0 + d;
    if (tile >= ntiles) break;
    const int cur = d & 1;
    if (!NLD) load_tile(tile + DEPTH, d % DEPTH);  // that set held this tile and went to LDS a tile ago
    const int k0 = tile * 32;
    const uint8_t* tb = &lds[cur][0];
    f32x4 s[2];
#pragma unroll
    for (int u = 0; u < 2; u++) {
      const f32x4 zero = {0.f, 0.f, 0.f, 0.f};
      f32x4 acc;
#pragma unroll
      for (int c = 0; c < 4; c++) {
        const bf16x8 kf = *reinterpret_cast<const bf16x8*>(tb + kofs[c] + u * 4096);
        acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf, qf[c], c == 0 ? zero : acc, 0, 0, 0);
      }
      s[u] = acc;
    }
    // only the tiles on the causal diagonal need the mask: when every key of the tile is visible to every query of
    // this wave (a uniform condition) the selects are skipped; the values are the same either way.  Prefill only:
    // in decode the tile loop is one dependent chain and a branch on a freshly computed value lengthens it.
    float alpha;
    bf16x8 pf;
    if (!DEEP && __builtin_amdgcn_ballot_w64(k0 + 31 > qpos) == 0) softmax_tile<false>(s, k0, g, qpos, a.scale_log2, m, l, alpha, pf);
    else softmax_tile<true>(s, k0, g, qpos, a.scale_log2, m, l, alpha, pf);
    // rescale the output accumulators only when some row's reference point moved (uniform over the wave): x * 1.0f is x bit
    // for bit, and after the first tiles of a long row the maximum rarely moves (prefill only, as above)
    if (DEEP || __builtin_amdgcn_ballot_w64(alpha != 1.0f) != 0) {
#pragma unroll
      for (int t = 0; t < 8; t++) o[t] = f32x4{o[t][0] * alpha, o[t][1] * alpha, o[t][2] * alpha, o[t][3] * alpha};
    }
#pragma unroll
    for (int t = 0; t < 8; t++) {
      const bf16x8 vf = *reinterpret_cast<const bf16x8*>(tb + vofs + t * 1024);
      o[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf, pf, o[t], 0, 0, 0);
    }
    if (!NLD && tile + 1 < ntiles) store_tile(cur ^ 1, (d + 1) % DEPTH);
    __syncthreads();
   }
  }
  if (!qvalid) return;
  const float inv = 1.0f / l;
  uint16_t* op = a.out + ((int64_t)(a.q_start[b] + qrow) * a.q_heads + h) * HD;
#pragma unroll
  for (int t = 0; t < 8; t++) {
    const uint32_t lo = pack_bf16x2(o[t][0] * inv, o[t][1] * inv);
    const uint32_t hi = pack_bf16x2(o[t][2] * inv, o[t][3] * inv);
    *reinterpret_cast<uint2*>(op + 16 * t + 4 * g) = make_uint2(lo, hi);
  }
}

// ------------------------------------------------------------------------------------------------
// Decode variant: every sequence brings so few new queries that all of them, for all G query heads of a KV head, fit
// the 16 rows of one MFMA tile (row = query * G + head of the group).  One work-group of eight wavefronts per
// (KV head, sequence):
//   * waves 0-3 compute.  All four form the scores and the softmax of the whole tile (the same instructions on the same
//     values, so the same bits in each) and each keeps the output accumulators of two of the eight 16-channel tiles: per
//     key tile a wave issues 8 + 2 MFMAs where a wave of the grouped kernel issues 16.  The scores of tile t + 1 are formed
//     before the softmax of tile t, so the MFMA chain of one tile runs beside the exponentials of the other.
//   * waves 4-7 do nothing but bring tiles in, with direct global->LDS loads (no staging registers, no LDS writes by a
//     wave): a decode step is one dependent chain of key tiles per sequence, and every load a computing wave issues is a
//     piece of that chain.  Loader i issues two of the eight 1 KiB load instructions of every K tile and V^T tile.
// A direct load puts lane l's 16 bytes at (wave-uniform address) + 16 l, so the LDS layout is made on the global side:
// each lane fetches the chunk that belongs at its fixed place.
//   K tile [32 keys][256 bytes]: chunk position pc of key row kr holds chunk pc ^ 2 (kr & 7) (the swizzle of the grouped
//     kernel, read the same way);
//   V^T tile [128 channels][64 bytes = 32 keys]: chunk position pc of channel row r holds chunk pc ^ ((r >> 2) & 3); a
//     P*V fragment (keys 4g .. 4g+3 and 16+4g .. 16+4g+3 of channel row 16t + j) is two 8-byte reads, and the sixteen
//     rows x two lane groups of a read pass cover all 64 banks.
// K tiles and V^T tiles have rings of NS slots each.  Iteration t reads K tile t + 1 and V^T tile t; the loaders request
// K tile t + NS (slot t % NS, read during iteration t - 1) and V^T tile t + NS - 1 (slot (t - 1) % NS, likewise), wait
// until what they requested NS - 2 iterations ago has landed (K tile t + 2, V^T tile t + 1: what iteration t + 1 reads),
// and all eight waves meet at the barrier.  Tiles behind the last one are clamped to the last tile of the cache and
// never used, so the number of loads in flight is static; nothing is in flight when a wave ends.
// A row's arithmetic -- the lanes that own it, the MFMA chains over channels and key slots, the order of the softmax
// updates -- is that of the kernels above: the same bits.
// ------------------------------------------------------------------------------------------------
template <int G, bool FUSED>
__global__ __launch_bounds__(512) void attention_decode_kernel(const AttnArgs a, const QkvArgs f) {
  constexpr int NS = 4;               // ring slots per operand (2 x 4 x 8 KiB of LDS)
  extern __shared__ __attribute__((aligned(1024))) uint8_t lds_dyn[];
  uint8_t (*lds_k)[8192] = reinterpret_cast<uint8_t (*)[8192]>(lds_dyn);
  uint8_t (*lds_v)[8192] = reinterpret_cast<uint8_t (*)[8192]>(lds_dyn + NS * 8192);
  constexpr int QMAX = 16 / G;
  constexpr int CT = 2;
  constexpr int NL = 4;               // loader waves
  constexpr int PI = 8 / NL;          // load instructions per tile, operand and loader wave
  const int b = blockIdx.y;
  const int kvh = blockIdx.x;
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wv = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int j = lane & 15;
  const int g = lane >> 4;
  const uint8_t* kbase = reinterpret_cast<const uint8_t*>(a.k_cache + ((int64_t)b * a.kv_heads + kvh) * a.max_len * HD);
  const uint8_t* vbase = reinterpret_cast<const uint8_t*>(a.vt_cache + ((int64_t)b * a.kv_heads + kvh) * (int64_t)HD * a.max_len);
  if (wv >= 4) {
    // ---------------- loader waves: loader li issues instructions li*PI .. li*PI+PI-1 of every K tile and V^T tile
    const int li = wv - 4;
    // K: instruction q covers key rows 4q .. 4q+3 (1 KiB): lane -> row 4q + (lane >> 4), chunk position lane & 15
    // V^T: instruction q covers channel rows 16q .. 16q+15: lane -> row 16q + (lane >> 2), chunk position lane & 3
    uint32_t kvoff[PI], vvoff[PI];
#pragma unroll
    for (int i = 0; i < PI; i++) {
      const int q = li * PI + i;
      const int kr = 4 * q + (lane >> 4), pc = lane & 15;
      const int r = 16 * q + (lane >> 2), vc = (lane & 3) ^ ((lane >> 4) & 3);
      kvoff[i] = (uint32_t)(kr * 256 + ((pc ^ (2 * (kr & 7))) << 4));
      vvoff[i] = (uint32_t)r * (uint32_t)a.max_len * 2u + vc * 16;
    }
    const uint32_t lk = (uint32_t)(uintptr_t)&lds_k[0][0] + li * PI * 1024;
    const uint32_t lv = (uint32_t)(uintptr_t)&lds_v[0][0] + li * PI * 1024;
    auto load_k = [&](int tile, int slot) __attribute__((always_inline)) {
      const uint8_t* src = kbase + (int64_t)min(tile * 32, a.max_len - 32) * (HD * 2);
#pragma unroll
      for (int i = 0; i < PI; i++) dma16(lk + slot * 8192 + i * 1024, kvoff[i], src);
    };
    auto load_v = [&](int tile, int slot) __attribute__((always_inline)) {
      const uint8_t* src = vbase + (int64_t)min(tile * 32, a.max_len - 32) * 2;
#pragma unroll
      for (int i = 0; i < PI; i++) dma16(lv + slot * 8192 + i * 1024, vvoff[i], src);
    };
    load_k(0, 0);
#pragma unroll
    for (int i = 0; i < NS - 1; i++) {
      load_k(i + 1, i + 1);
      load_v(i, i);
    }
    const int ctx = a.ctx_len[b];
    const int qlen = FUSED ? (ctx > 0 ? 1 : 0) : a.q_len[b];
    if (qlen <= 0) {
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
      return;
    }
    const int last_pos = ctx - qlen + min(QMAX - 1, qlen - 1);
    const int ntiles = last_pos / 32 + 1;
    if (FUSED) {
      // loaders 0 and 1 form the new key and file the new value while the first tiles are on their way (the computing
      // waves form the query heads meanwhile); everything they have in flight is drained before the barrier, so the waits
      // below still count the tile loads alone
      if (li < 2) {
        uint16_t* hs = reinterpret_cast<uint16_t*>(lds_dyn + 2 * NS * 8192);
        const int pos = ctx - 1;
        const uint16_t* src = f.qkv + (int64_t)b * f.ld + (int64_t)(a.q_heads + (li == 0 ? 0 : a.kv_heads) + kvh) * HD;
        const uint16_t r1 = src[lane], r2 = src[lane + 64];
        uint32_t o = (uint32_t)r1 | ((uint32_t)r2 << 16);
        if (li == 0) o = qk_norm_rope_head(r1, r2, f.kw, pos, f.inv_freq, f.eps, lane);
        hs[(G + li) * HD + lane] = (uint16_t)(o & 0xffffu);
        hs[(G + li) * HD + lane + 64] = (uint16_t)(o >> 16);
        if (pos < a.max_len) {
          if (li == 0) {
            uint16_t* dst = f.k_cache + (((int64_t)b * a.kv_heads + kvh) * a.max_len + pos) * HD;
            dst[lane] = (uint16_t)(o & 0xffffu);
            dst[lane + 64] = (uint16_t)(o >> 16);
          } else {
            uint16_t* dst = f.vt_cache + ((int64_t)b * a.kv_heads + kvh) * (int64_t)HD * a.max_len + pos;
            dst[(int64_t)lane * a.max_len] = r1;
            dst[(int64_t)(lane + 64) * a.max_len] = r2;
          }
        }
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
      }
      __syncthreads();  // the heads are in LDS
    }
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(2 * PI * (NS - 1)) : "memory");  // K tile 0
    __syncthreads();
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(2 * PI * (NS - 2)) : "memory");  // K tile 1, V^T tile 0
    __syncthreads();
    for (int t0 = 0; t0 < ntiles; t0 += NS) {
#pragma unroll
      for (int d = 0; d < NS; d++) {
        const int tile = t0 + d;
        if (tile >= ntiles) break;
        load_k(tile + NS, d);                          // slot t % NS, read during iteration t - 1
        load_v(tile + NS - 1, (d + NS - 1) % NS);      // slot (t - 1) % NS, likewise
        asm volatile("s_waitcnt vmcnt(%0)" ::"n"(2 * PI * (NS - 2)) : "memory");  // K tile t + 2, V^T tile t + 1
        __syncthreads();
      }
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    return;
  }
  // ---------------- computing waves
  const int ctx = a.ctx_len[b];
  const int qlen = FUSED ? (ctx > 0 ? 1 : 0) : a.q_len[b];
  if (qlen <= 0) return;
  const int qi = j / G;
  const int h = kvh * G + j % G;
  const bool qvalid = qi < qlen;
  const int qrow = min(qi, qlen - 1);
  const int qpos = ctx - qlen + qrow;
  const int last_pos = ctx - qlen + min(QMAX - 1, qlen - 1);
  const int ntiles = last_pos / 32 + 1;
  const int nfull = (ctx - qlen + 1) / 32;
  bf16x8 qf[4];
  // FUSED: the G query heads of this (sequence, KV head) are formed here, one head per wave at a time, the key and the
  // value by two of the loader waves (per-head RMSNorm and rotary embedding as the stand-alone kernel does them); all are
  // left in LDS for the four computing waves and, the key and the value, filed in the caches for the steps to come.  This step takes them from LDS: the tile
  // that a loader brings in for their position holds whatever the cache held there, and is patched below.
  uint16_t* hs = reinterpret_cast<uint16_t*>(lds_dyn + 2 * NS * 8192);  // [G + 2][128]: q heads, k, v
  const int pos = ctx - 1;
  if (FUSED) {
    const uint16_t* row = f.qkv + (int64_t)b * f.ld;
    for (int u = wv; u < G; u += 4) {  // wave-uniform: the query heads (loaders 0 and 1 take the key and the value)
      const uint16_t* src = row + (int64_t)(kvh * G + u) * HD;
      const uint32_t o = qk_norm_rope_head(src[lane], src[lane + 64], f.qw, pos, f.inv_freq, f.eps, lane);
      hs[u * HD + lane] = (uint16_t)(o & 0xffffu);
      hs[u * HD + lane + 64] = (uint16_t)(o >> 16);
    }
    __syncthreads();
#pragma unroll
    for (int c = 0; c < 4; c++) qf[c] = *reinterpret_cast<const bf16x8*>(hs + (j % G) * HD + c * 32 + g * 8);
  } else {
    const uint16_t* qp = a.q + ((int64_t)(a.q_start[b] + qrow) * a.q_heads + h) * HD;
#pragma unroll
    for (int c = 0; c < 4; c++) qf[c] = *reinterpret_cast<const bf16x8*>(qp + c * 32 + g * 8);
  }
  // the new key's row of the K tile in `slot` and the new value's column of this wave's rows of the V^T tile, from LDS
  // (each wave patches what it reads itself, right before it reads it: a wave's LDS operations keep their order)
  const int lt = pos >> 5, pr = pos & 31;
  auto patch_k = [&](int slot) __attribute__((always_inline)) {
    if (lane < 16)
      *reinterpret_cast<u32x4*>(&lds_k[slot][pr * 256 + ((lane ^ (2 * (pr & 7))) << 4)]) = *reinterpret_cast<const u32x4*>(hs + G * HD + lane * 8);
  };
  auto patch_v = [&](int slot) __attribute__((always_inline)) {
    if (lane < 16 * CT) {
      const int ch = 16 * CT * wv + lane;
      *reinterpret_cast<uint16_t*>(&lds_v[slot][ch * 64 + (((pr >> 3) ^ ((ch >> 2) & 3)) << 4) + (pr & 7) * 2]) = hs[(G + 1) * HD + ch];
    }
  };
  uint32_t kofs[4];
#pragma unroll
  for (int c = 0; c < 4; c++) kofs[c] = j * 256 + (((c * 4 + g) ^ (2 * (j & 7))) << 4);
  const int vsw = (j >> 2) & 3;
  const uint32_t vofs0 = (CT * wv) * 1024 + j * 64 + (((g >> 1) ^ vsw) << 4) + (g & 1) * 8;
  const uint32_t vofs1 = (CT * wv) * 1024 + j * 64 + (((2 + (g >> 1)) ^ vsw) << 4) + (g & 1) * 8;
  auto scores = [&](int slot, f32x4 (&s)[2]) __attribute__((always_inline)) {
    const uint8_t* tb = &lds_k[slot][0];
#pragma unroll
    for (int u = 0; u < 2; u++) {
      const f32x4 zero = {0.f, 0.f, 0.f, 0.f};
      f32x4 acc;
#pragma unroll
      for (int c = 0; c < 4; c++) {
        const bf16x8 kf = *reinterpret_cast<const bf16x8*>(tb + kofs[c] + u * 4096);
        acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf, qf[c], c == 0 ? zero : acc, 0, 0, 0);
      }
      s[u] = acc;
    }
  };
  f32x4 o[CT];
#pragma unroll
  for (int i = 0; i < CT; i++) o[i] = f32x4{0.f, 0.f, 0.f, 0.f};
  float m = -INFINITY;
  float l = 0.f;
  __syncthreads();
  if (FUSED && lt == 0) patch_k(0);
  f32x4 s_cur[2];
  scores(0, s_cur);
  __syncthreads();
  for (int t0 = 0; t0 < ntiles; t0 += NS) {
#pragma unroll
    for (int d = 0; d < NS; d++) {
      const int tile = t0 + d;
      if (tile >= ntiles) break;
      if (FUSED && tile == lt) patch_v(d);
      if (FUSED && tile + 1 == lt) patch_k((d + 1) % NS);
      bf16x8 vf[CT];
#pragma unroll
      for (int i = 0; i < CT; i++) {
        const uint2 va = *reinterpret_cast<const uint2*>(&lds_v[d][vofs0 + i * 1024]);
        const uint2 vb = *reinterpret_cast<const uint2*>(&lds_v[d][vofs1 + i * 1024]);
        vf[i] = __builtin_bit_cast(bf16x8, u32x4{va.x, va.y, vb.x, vb.y});
      }
      f32x4 s_next[2];
      scores((d + 1) % NS, s_next);
      float alpha;
      bf16x8 pf;
      if (tile < nfull) softmax_tile<false>(s_cur, tile * 32, g, qpos, a.scale_log2, m, l, alpha, pf);
      else softmax_tile<true>(s_cur, tile * 32, g, qpos, a.scale_log2, m, l, alpha, pf);
#pragma unroll
      for (int i = 0; i < CT; i++) o[i] = f32x4{o[i][0] * alpha, o[i][1] * alpha, o[i][2] * alpha, o[i][3] * alpha};
#pragma unroll
      for (int i = 0; i < CT; i++) o[i] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf[i], pf, o[i], 0, 0, 0);
      __syncthreads();
      s_cur[0] = s_next[0];
      s_cur[1] = s_next[1];
    }
  }
  if (!qvalid) return;
  const float inv = 1.0f / l;
  uint16_t* op = a.out + ((int64_t)(FUSED ? b : a.q_start[b] + qi) * a.q_heads + h) * HD + 16 * CT * wv;
#pragma unroll
  for (int i = 0; i < CT; i++) {
    const uint32_t lo = pack_bf16x2(o[i][0] * inv, o[i][1] * inv);
    const uint32_t hi = pack_bf16x2(o[i][2] * inv, o[i][3] * inv);
    *reinterpret_cast<uint2*>(op + 16 * i + 4 * g) = make_uint2(lo, hi);
  }
}

int attention_dispatch(const void* q, const void* k_cache, const void* vt_cache, void* out, const int* q_start,
                       const int* q_len, const int* ctx_len, int batch, int max_q_len, int q_heads, int kv_heads,
                       int head_dim, int max_len, float scale, hipStream_t stream) {
  if (!q || !k_cache || !vt_cache || !out || !q_start || !q_len || !ctx_len) return TBIK_ERR_INVALID;
  if (batch <= 0 || max_q_len <= 0 || q_heads <= 0 || kv_heads <= 0 || q_heads % kv_heads != 0) return TBIK_ERR_INVALID;
  if (head_dim != HD) return TBIK_ERR_UNSUPPORTED;
  if (max_len < 32 || (max_len & 3)) return TBIK_ERR_ALIGNMENT;
  auto mis = [](const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) != 0; };
  if (mis(q) || mis(k_cache) || mis(vt_cache) || mis(out)) return TBIK_ERR_ALIGNMENT;
  if (batch > 65535 || q_heads > 65535) return TBIK_ERR_INVALID;
  AttnArgs a{static_cast<const uint16_t*>(q), static_cast<const uint16_t*>(k_cache), static_cast<const uint16_t*>(vt_cache),
             static_cast<uint16_t*>(out), q_start, q_len, ctx_len, q_heads, kv_heads, max_len, scale * 1.4426950408889634f};
  // the grouped kernel needs whole 32-key tiles in the caches, at most 8 query heads per KV head and a (sequence, head)
  // slice of a cache below 2 GiB (32-bit byte offsets)
  const int G = q_heads / kv_heads;
  const bool grouped = (max_len & 31) == 0 && (G == 1 || G == 2 || G == 4 || G == 8) && kv_heads <= 65535 && max_len <= (1 << 22);
  if (grouped) {
    const bool deep = max_q_len <= 16;  // decode: one block of queries per sequence
    if ((int64_t)max_q_len * G <= 16) {  // all queries of a sequence and all heads of a group in one MFMA tile
      const dim3 grid((unsigned)kv_heads, (unsigned)batch, 1u);
      constexpr size_t lds = 2 * 4 * 8192;
      const QkvArgs none{};
      if (G == 1) hipLaunchKernelGGL((attention_decode_kernel<1, false>), grid, dim3(512), lds, stream, a, none);
      else if (G == 2) hipLaunchKernelGGL((attention_decode_kernel<2, false>), grid, dim3(512), lds, stream, a, none);
      else if (G == 4) hipLaunchKernelGGL((attention_decode_kernel<4, false>), grid, dim3(512), lds, stream, a, none);
      else hipLaunchKernelGGL((attention_decode_kernel<8, false>), grid, dim3(512), lds, stream, a, none);
      return hip_code(hipGetLastError());
    }
    const int64_t gx = (int64_t)((max_q_len + 15) / 16) * kv_heads;
    if (gx > 0x7fffffff) return TBIK_ERR_INVALID;
    const dim3 grid((unsigned)gx, (unsigned)batch, 1u);
    // Two more waves per work-group that only stage the tiles (NLD = 2) take the loads and LDS writes out of the computing
    // waves' instruction streams.  That pays while the launch leaves CUs short of work-groups (a chunk of a prompt, a few
    // sequences: up to two work-groups per CU: 3 - 18 % faster) and costs once the chip is full, where the extra waves
    // take the place of a whole work-group (from three per CU on: 35 % slower).  Same bits either way.
    const bool few = gx * batch <= 512;
#define TBIK_ATTN_GROUP(GG)                                                                                              \
  do {                                                                                                                   \
    if (few && deep) hipLaunchKernelGGL((attention_group_kernel<GG, true, 2>), grid, dim3(64 * (GG + 2)), 0, stream, a);   \
    else if (few) hipLaunchKernelGGL((attention_group_kernel<GG, false, 2>), grid, dim3(64 * (GG + 2)), 0, stream, a);    \
    else if (deep) hipLaunchKernelGGL((attention_group_kernel<GG, true, 0>), grid, dim3(64 * GG), 0, stream, a);          \
    else hipLaunchKernelGGL((attention_group_kernel<GG, false, 0>), grid, dim3(64 * GG), 0, stream, a);                   \
  } while (0)
    if (G == 1) TBIK_ATTN_GROUP(1);
    else if (G == 2) TBIK_ATTN_GROUP(2);
    else if (G == 4) TBIK_ATTN_GROUP(4);
    else TBIK_ATTN_GROUP(8);
#undef TBIK_ATTN_GROUP
  } else {
    const dim3 grid((unsigned)((max_q_len + 15) / 16), (unsigned)q_heads, (unsigned)batch);
    hipLaunchKernelGGL(attention_kernel, grid, dim3(64), 0, stream, a);
  }
  return hip_code(hipGetLastError());
}

// One decode step of an attention block from the fused qkv projection output: per-head q/k RMSNorm, rotary embedding, the
// cache write and the attention of every sequence's one new token (row b of qkv, position ctx_len[b] - 1) in one launch.
// The bits of qk_norm_rope_cache_dispatch followed by attention_dispatch.  TBIK_ERR_UNSUPPORTED where the decode kernel
// does not apply (cache length not a whole number of tiles, more than 8 or an odd number of query heads per KV head):
// the caller makes the two calls.
int attention_decode_qkv_dispatch(const void* qkv, int64_t ld, const void* q_weight, const void* k_weight, const float* inv_freq,
                                  void* k_cache, void* vt_cache, void* out, const int* ctx_len, int batch, int q_heads,
                                  int kv_heads, int head_dim, int max_len, float scale, float eps, hipStream_t stream) {
  if (!qkv || !q_weight || !k_weight || !inv_freq || !k_cache || !vt_cache || !out || !ctx_len) return TBIK_ERR_INVALID;
  if (batch <= 0 || q_heads <= 0 || kv_heads <= 0 || q_heads % kv_heads != 0) return TBIK_ERR_INVALID;
  if (head_dim != HD) return TBIK_ERR_UNSUPPORTED;
  if (ld < (int64_t)(q_heads + 2 * kv_heads) * HD) return TBIK_ERR_INVALID;
  if (max_len < 32 || (max_len & 3)) return TBIK_ERR_ALIGNMENT;
  auto mis = [](const void* p, uintptr_t m) { return (reinterpret_cast<uintptr_t>(p) & m) != 0; };
  if (mis(k_cache, 15) || mis(vt_cache, 15) || mis(out, 15) || mis(qkv, 1) || mis(q_weight, 1) || mis(k_weight, 1) || mis(inv_freq, 3))
    return TBIK_ERR_ALIGNMENT;
  if (batch > 65535 || kv_heads > 65535) return TBIK_ERR_INVALID;
  const int G = q_heads / kv_heads;
  if ((max_len & 31) != 0 || !(G == 1 || G == 2 || G == 4 || G == 8) || max_len > (1 << 22)) return TBIK_ERR_UNSUPPORTED;
  AttnArgs a{nullptr, static_cast<const uint16_t*>(k_cache), static_cast<const uint16_t*>(vt_cache), static_cast<uint16_t*>(out),
             nullptr, nullptr, ctx_len, q_heads, kv_heads, max_len, scale * 1.4426950408889634f};
  const QkvArgs f{static_cast<const uint16_t*>(qkv), ld, static_cast<const uint16_t*>(q_weight), static_cast<const uint16_t*>(k_weight),
                  inv_freq, static_cast<uint16_t*>(k_cache), static_cast<uint16_t*>(vt_cache), eps};
  const dim3 grid((unsigned)kv_heads, (unsigned)batch, 1u);
  const size_t lds = 2 * 4 * 8192 + (size_t)(G + 2) * HD * 2;
  if (G == 1) hipLaunchKernelGGL((attention_decode_kernel<1, true>), grid, dim3(512), lds, stream, a, f);
  else if (G == 2) hipLaunchKernelGGL((attention_decode_kernel<2, true>), grid, dim3(512), lds, stream, a, f);
  else if (G == 4) hipLaunchKernelGGL((attention_decode_kernel<4, true>), grid, dim3(512), lds, stream, a, f);
  else hipLaunchKernelGGL((attention_decode_kernel<8, true>), grid, dim3(512), lds, stream, a, f);
  return hip_code(hipGetLastError());
}

}  // namespace tbik
