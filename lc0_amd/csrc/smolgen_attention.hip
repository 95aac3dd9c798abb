// Smolgen generator and attention in one kernel for gfx950, head depth 32, at most 32 heads:
//   logits[b][h][q][k] = scale * Q.K^T + sum_j W[q*64+k][j] * gen[b][h][j],  out = softmax_k(logits) . V
// (the shared smolgen_w layer, src/neural/backends/blas/network_blas.cc:332-347, followed by the per-head attention,
// :352-439). Run as a GEMM of its own, the generator writes 8 KiB of logits per (sample, head) that the attention
// kernel reads back at once: at 256 positions and 32 heads that is 2 x 67 MB of memory traffic per encoder layer and a
// launch that competes with the QKV projection for the CUs. Here the logits never leave the CU.
//
// One workgroup of eight waves owns two samples (64 columns = 2 x 32 heads) and 16 queries.
//   Phase 1 (matrix cores): [1024 (query, key) rows] x [64 columns] x gen_sz. The weight rows are the MFMA "A" operand,
//     stored at load in fragment order (each wave streams 1 KiB per load, fully coalesced, a ring of loads ahead of the
//     MFMAs) and used for both column tiles; the generator vectors of the 64 (sample, head) columns are the "B"
//     operand and stay in registers. A lane ends up with the logits of one (sample, head) column: they go to LDS as
//     halves in the layout phase 2 reads (128 KiB for the workgroup: 32 contiguous bytes per reading lane, the
//     positions XOR-ed with the column so that the writers of one instruction spread over eight bank groups).
//   Phase 2 (memory and vector ALU): every wave takes 8 of the 64 (sample, head) columns. With 16-wide MFMA tiles the 16
//     queries are one tile: S^T = K.Q^T, plus the logits from LDS, softmax in registers with one lane exchange (the
//     maximum; the row sums come from the matrix cores as 1.P^T), O^T = V^T.P^T with V^T read from the staged V tile
//     by transposing LDS loads, and 8-byte output stores straight from the accumulators. K and V come in by full
//     128-byte rows of two neighbouring heads; the next pair's are in flight while this one is computed.
// Per workgroup 0.5 MiB of weights, 0.5 MiB of K and V and 64 KiB of Q come from L2; nothing but the output is written.
#include <hip/hip_runtime.h>

#include <stdexcept>
#include <type_traits>

#include "kernel_common.h"

namespace lc0mi {

namespace {

constexpr int kQueriesPerGroup = 16;               // queries of one workgroup
constexpr int kLogitBytes = 64 * 16 * 4 * 32;   // [column][query][key group of the lane][16-key tile] x 8 B
constexpr int kVBytesPerWave = 64 * 32 * 2;   // staging area of one wave: a tile of 32 rows x 128 bytes

// Byte offset of the four logits of query qq (0..15) and column c (0..63) for keys 16*t + 4*g4 + (0..3). The 32 bytes
// of one (c, qq, g4) are what a lane of phase 2 reads; the position of that block inside the column's 2 KiB is
// XOR-ed with the low bits of c, which leaves the readers of one column (all qq, g4) on a contiguous 2 KiB and spreads
// the 32 columns that phase 1 writes with one instruction over eight bank groups.
__device__ __forceinline__ int LogitSlot(int c, int qq, int g4, int t) {
  return (((c * 16 + (qq ^ ((c >> 2) & 1))) * 4 + (g4 ^ (c & 3))) * 32) + t * 8;
}

// x0 and x1 (two independent values: the two heads of a pair), each combined with its values in the lanes 16, 32 and
// 48 away, with the lane-swap instructions of gfx950 (two vector ALU operations per step instead of a round trip
// through the LDS crossbar). v_permlane16_swap exchanges the odd 16-lane rows of its first register with the even
// rows of its second, v_permlane32_swap the upper half of the first with the lower half of the second: fed the same
// value twice, the two registers afterwards hold the value of this lane's row (half) and of its neighbour's. Written
// as assembly: the compiler's builtin for these instructions loses track of the second result register. The no-ops
// cover the wait states between a vector ALU write and a lane swap that reads it, and between the swap and its
// readers; the swaps of the two values share them.
template <typename F>
__device__ __forceinline__ void Reduce4Rows2(float& x0, float& x1, F&& op) {
  float a0 = x0, b0 = x0, a1 = x1, b1 = x1;
  asm volatile("s_nop 1\n\tv_permlane16_swap_b32 %0, %1\n\tv_permlane16_swap_b32 %2, %3\n\ts_nop 1"
               : "+v"(a0), "+v"(b0), "+v"(a1), "+v"(b1));
  float y0 = op(a0, b0), y1 = op(a1, b1);
  float c0 = y0, c1 = y1;
  asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1\n\tv_permlane32_swap_b32 %2, %3\n\ts_nop 1"
               : "+v"(y0), "+v"(c0), "+v"(y1), "+v"(c1));
  x0 = op(y0, c0);
  x1 = op(y1, c1);
}

// FULL: 32 heads, so that every (sample, head) column of every workgroup exists (or repeats an existing one), the
// loop over head pairs carries no branches and its interleaved order fits the registers.
// ET: half_t or bf16_t, the type of qkv, gen, wfrag, of the logits kept in LDS and of a 16-bit output (all typed
// half_t here: the same storage).
template <int NKS, typename OutT, bool FULL, typename ET>
__global__ __launch_bounds__(512, 1) void smolgen_attention_kernel(const half_t* __restrict__ qkv,
                                                                    const half_t* __restrict__ gen,
                                                                    const half_t* __restrict__ wfrag,
                                                                    OutT* __restrict__ out, int batch, int heads,
                                                                    float scale, float out_mul) {
  using ev8 = typename Vec16<ET>::v8;
  using ev4 = typename Vec16<ET>::v4;
  constexpr int DEPTH = 32;
  // Two arrays, not one with offsets: the compiler can then tell that staging a K or V tile never touches the logits
  // and moves the staging of the next pair of heads in among the softmax arithmetic of this one.
  __shared__ __attribute__((aligned(1024))) unsigned char smem[kLogitBytes];
  __shared__ __attribute__((aligned(1024))) unsigned char stage_lds[8 * kVBytesPerWave];
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int r = lane & 31, g = lane >> 5;
  // Workgroups are handed to the 8 XCDs in turn: the four query groups of a sample pair get ids 8 apart, so that they
  // run on one XCD at about the same time and share its L2 for K and V.
  const int id = blockIdx.x;
  const int pair = (id >> 5) * 8 + (id & 7);
  const int qt = (id >> 3) & 3;
  if (pair * 2 >= batch) return;
  const int b0 = pair * 2;
  const bool valid1 = b0 + 1 < batch;
  const int b1 = valid1 ? b0 + 1 : b0;
  const int d_model = heads * DEPTH, ld = 3 * d_model;
  constexpr int G = NKS * 16;

  // ---- phase 1: logits of the 16 queries for the 64 columns ----
  {
    // This wave's four row tiles (two queries x two key halves) are 4 * NKS consecutive fragments of 1 KiB.
    constexpr int NF = 4 * NKS;
    constexpr int PF = NF < 12 ? NF : 12;   // loads in flight per wave
    const ev8* wp = reinterpret_cast<const ev8*>(wfrag) + ((long long)(32 * qt + wave * 4) * NKS) * 64 + lane;
    ev8 ring[PF];
#pragma unroll
    for (int f = 0; f < PF; f++) ring[f] = wp[f * 64];
    // The generator vectors of the 64 columns: once per workgroup through LDS (the region phase 2 stages K and V in), 16-byte
    // slot s of column c at slot s ^ (c & 31) of its row, then into the registers of every wave as MFMA "B" operands.
    unsigned char* gl = stage_lds;
    constexpr int kSlotsPerCol = G / 8;
    for (int i = threadIdx.x; i < 64 * kSlotsPerCol; i += 512) {
      const int c = i / kSlotsPerCol, sl = i - c * kSlotsPerCol;
      const int hh = c & 31;
      uint4 v = make_uint4(0, 0, 0, 0);
      if (hh < heads) {
        v = *reinterpret_cast<const uint4*>(gen + ((long long)(c >= 32 ? b1 : b0) * heads + hh) * G + sl * 8);
      }
      *reinterpret_cast<uint4*>(gl + (c * kSlotsPerCol + (sl ^ (c & (kSlotsPerCol - 1)))) * 16) = v;
    }
    __syncthreads();
    ev8 bf[2][NKS];
#pragma unroll
    for (int ct = 0; ct < 2; ct++)
#pragma unroll
      for (int ks = 0; ks < NKS; ks++) {
        const int c = ct * 32 + r;
        bf[ct][ks] = *reinterpret_cast<const ev8*>(gl + (c * kSlotsPerCol + ((ks * 2 + g) ^ (c & (kSlotsPerCol - 1)))) * 16);
      }
    floatx16 acc[2];
#pragma unroll
    for (int f = 0; f < NF; f++) {
      const int ks = f % NKS;
      if (ks == 0) {
#pragma unroll
        for (int e = 0; e < 16; e++) { acc[0][e] = 0.0f; acc[1][e] = 0.0f; }
      }
      const ev8 a = ring[f % PF];
      if (f + PF < NF) ring[f % PF] = wp[(f + PF) * 64];
      acc[0] = Mfma32(a, bf[0][ks], acc[0]);
      acc[1] = Mfma32(a, bf[1][ks], acc[1]);
      if (ks == NKS - 1) {
        const int rt = wave * 4 + f / NKS;   // row tile within the query group
        const int qq = rt >> 1, mt = rt & 1;
        // register 4 q4 + e of lane (column r, g): key 32 mt + 8 q4 + 4 g + e = 4 u + e with u = 8 mt + 2 q4 + g
#pragma unroll
        for (int ct = 0; ct < 2; ct++)
#pragma unroll
          for (int q4 = 0; q4 < 4; q4++) {
            ev4 hv;
#pragma unroll
            for (int e = 0; e < 4; e++) hv[e] = (ET)acc[ct][q4 * 4 + e];
            const int u = 8 * mt + 2 * q4 + g;
            *reinterpret_cast<ev4*>(smem + LogitSlot(ct * 32 + r, qq, u & 3, u >> 2)) = hv;
          }
      }
    }
  }
  __syncthreads();

  // ---- phase 2: attention of the 16 queries, eight (sample, head) columns per wave ----
  // 16-wide MFMA tiles (v_mfma_f32_16x16x32_f16): the 16 queries are the columns of one tile, and lane (j, g4) = (query,
  // group of four keys per 16-key tile) holds 16 of the 64 logits of its query, so that all 64 lanes carry distinct
  // softmax elements:
  //   S^T tiles (16 keys x 16 queries, the whole head depth in one MFMA), plus the logits of phase 1 from LDS;
  //   softmax over the 16 values of a lane and the lanes 16, 32 and 48 away;
  //   V^T read from the staged V tile with the transposing LDS load of gfx950 (ds_read_b64_tr_b16), which hands a
  //   lane per depth index four keys at a time, in the order of P;
  //   O^T = V^T . P^T, so that a lane ends up with depth values of its own query, and 1 . P^T in the same way (the
  //   row sums of the rounded P that the product itself uses) to scale them by before storing.
  // K and V are fetched for two neighbouring heads at once by 128-byte rows (both heads' 32 halves side by side), eight
  // lanes per row, so that every load instruction touches eight full cache lines instead of 32 partial ones; a tile
  // of 32 rows then passes through this wave's 4 KiB of LDS to reach the lanes in operand layout, 16-byte chunk c of
  // row w at chunk c ^ swizzle(w): (w >> 1) & 7 for a K tile, read back as 16 bytes per lane from 16 rows, and
  // ((w & 3) << 1) | ((w >> 2) & 1) for a V tile, read back as 8 bytes per lane from 4 rows x 32 bytes per 16 lanes
  // (either way the lanes that are served together spread evenly over the banks).
  const int j = lane & 15, g4 = lane >> 4;
  const int lr = lane >> 3, ch = lane & 7;
  unsigned char* stg = stage_lds + wave * kVBytesPerWave;
  struct PairData {
    ev8 k[2][4], v[2][4];   // [32-row tile][8-row group]
    ev8 q[2];               // [head]: query j, depth 8 g4 .. 8 g4 + 7
  };
  // The pieces of a pair's rows are loaded separately, each into the registers that the same piece of the pair
  // before has just left for LDS: one set of registers serves all four pairs.
  auto pair_base = [&](int pi, const half_t*& Kp, const half_t*& Q, bool& has_b) {
    const int ca = wave * 8 + 2 * pi;
    const int b = ca >= 32 ? b1 : b0;
    const int ha = ca & 31;
    const int ha_c = (FULL || ha < heads) ? ha : 0;
    has_b = FULL || ha_c + 1 < heads;
    const half_t* base = qkv + (long long)b * 64 * ld;
    // (without a head B the upper half of the row repeats head A instead of running past the row)
    Kp = base + d_model + ha_c * DEPTH + (has_b ? ch : (ch & 3)) * 8 + (unsigned)lr * (unsigned)ld;
    Q = base + ha_c * DEPTH + (unsigned)(kQueriesPerGroup * qt + j) * (unsigned)ld + 8u * g4;
  };
  auto load_k = [&](int pi, int t, PairData& d) {
    const half_t *Kp, *Q;
    bool has_b;
    pair_base(pi, Kp, Q, has_b);
#pragma unroll
    for (int i = 0; i < 4; i++) d.k[t][i] = *reinterpret_cast<const ev8*>(Kp + (unsigned)(32 * t + 8 * i) * (unsigned)ld);
  };
  auto load_v = [&](int pi, int t, PairData& d) {
    const half_t *Kp, *Q;
    bool has_b;
    pair_base(pi, Kp, Q, has_b);
#pragma unroll
    for (int i = 0; i < 4; i++)
      d.v[t][i] = *reinterpret_cast<const ev8*>(Kp + d_model + (unsigned)(32 * t + 8 * i) * (unsigned)ld);
  };
  auto load_q = [&](int pi, PairData& d) {
    const half_t *Kp, *Q;
    bool has_b;
    pair_base(pi, Kp, Q, has_b);
    d.q[0] = *reinterpret_cast<const ev8*>(Q);
    d.q[1] = *reinterpret_cast<const ev8*>(Q + (has_b ? DEPTH : 0));
  };
  // fr[head][16-row half]: rows of the staged tile in operand layout (lane j = row of the half, g4 = 8-half group)
  auto stage_tile = [&](const ev8 (&raw)[4], ev8 (&fr)[2][2]) {
#pragma unroll
    for (int i = 0; i < 4; i++) {
      const int row = 8 * i + lr;
      *reinterpret_cast<ev8*>(stg + row * 128 + ((ch ^ ((row >> 1) & 7)) * 16)) = raw[i];
    }
#pragma unroll
    for (int hb = 0; hb < 2; hb++)
#pragma unroll
      for (int th = 0; th < 2; th++) {
        const int row = 16 * th + j, c = hb * 4 + g4;
        fr[hb][th] = *reinterpret_cast<const ev8*>(stg + row * 128 + ((c ^ ((row >> 1) & 7)) * 16));
      }
  };
  // V^T fragments of a staged V tile: the transposing load treats the 16 lanes of a group as a 16 x 4 matrix of
  // 16-bit elements D[s][c] (lane s supplies the address of its four contiguous elements) and returns to lane i the
  // elements D[4 e + (i >> 2)][i & 3], e = 0..3. With lane s of group g4 pointing at key 16 h + 4 g4 + (s >> 2),
  // depth 16 dt + 4 (s & 3), lane i = depth index receives the keys 16 h + 4 g4 + e of depth 16 dt + i.
  typedef short short4v __attribute__((ext_vector_type(4)));
  typedef short short8v __attribute__((ext_vector_type(8)));
  auto stage_v_tile = [&](const ev8 (&raw)[4], ev8 (&vt)[2][2]) {   // vt[head][depth half]
#pragma unroll
    for (int i = 0; i < 4; i++) {
      const int row = 8 * i + lr;
      const int swz = ((row & 3) << 1) | ((row >> 2) & 1);
      *reinterpret_cast<ev8*>(stg + row * 128 + ((ch ^ swz) * 16)) = raw[i];
    }
#pragma unroll
    for (int hb = 0; hb < 2; hb++)
#pragma unroll
      for (int dt = 0; dt < 2; dt++) {
        short4v part[2];
#pragma unroll
        for (int h = 0; h < 2; h++) {
          const int row = 16 * h + 4 * g4 + (j >> 2), q = j & 3;
          const int swz = ((row & 3) << 1) | ((row >> 2) & 1);
          const int c = hb * 4 + 2 * dt + (q >> 1);
          part[h] = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
              (__attribute__((address_space(3))) short4v*)(stg + row * 128 + ((c ^ swz) * 16) + (q & 1) * 8));
        }
        const short8v both = __builtin_shufflevector(part[0], part[1], 0, 1, 2, 3, 4, 5, 6, 7);
        vt[hb][dt] = __builtin_bit_cast(ev8, both);
      }
  };
  ev8 ones;
#pragma unroll
  for (int e = 0; e < 8; e++) ones[e] = (ET)1.0f;
  const floatx4 zero4 = {0.0f, 0.0f, 0.0f, 0.0f};

  // Software pipeline over the wave's four pairs of heads: while the softmax and P.V of pair p run (vector ALU work
  // with long dependency chains: exponentials, lane swaps), the scores and V^T of pair p + 1 are prepared (LDS round
  // trips and matrix instructions), and the rows of pair p + 2 are on their way from memory. The two kinds of work
  // are written alternately below, step by step and for both heads of a pair at once, because the compiler keeps
  // the order of the source here and would otherwise run every chain to its end before starting the next.
  struct Prep {
    floatx4 st[2][4];   // S^T[key][query] of both heads: [head][16-key tile], register e = key 16 t + 4 g4 + e
    ev8 vt[2][2][2];    // V^T of both heads as operands: [head][depth half][32-key step], lane (depth index, g4),
  };                    //   elements = keys 32 s + 4 g4 + (0..3) and 32 s + 16 + 4 g4 + (0..3), the order of P below
  auto prep_k = [&](const PairData& d, int tt, Prep& o) {
    ev8 kf[2][2];
    stage_tile(d.k[tt], kf);
#pragma unroll
    for (int hb = 0; hb < 2; hb++)
#pragma unroll
      for (int th = 0; th < 2; th++) o.st[hb][2 * tt + th] = Mfma16(kf[hb][th], d.q[hb], zero4);
  };
  auto prep_v = [&](const PairData& d, int tt, Prep& o) {
    ev8 vt[2][2];
    stage_v_tile(d.v[tt], vt);
#pragma unroll
    for (int hb = 0; hb < 2; hb++)
#pragma unroll
      for (int dt = 0; dt < 2; dt++) o.vt[hb][dt][tt] = vt[hb][dt];
  };

  // Step 0..3 of preparing the pair whose rows are in `raw`; every step refills the registers it has emptied with the
  // same piece of pair `next` (if there is one).
  PairData raw;
  auto prep_step = [&](int step, int next, Prep& o) {
    if (step < 2) {
      prep_k(raw, step, o);
      if (next < 4) {
        load_k(next, step, raw);
        if (step == 1) load_q(next, raw);
      }
    } else {
      prep_v(raw, step - 2, o);
      if (next < 4) load_v(next, step - 2, raw);
    }
  };
  Prep prep[2];
  load_k(0, 0, raw);
  load_q(0, raw);
  load_k(0, 1, raw);
  load_v(0, 0, raw);
  load_v(0, 1, raw);
#pragma unroll
  for (int step = 0; step < 4; step++) prep_step(step, 1, prep[0]);
#pragma unroll
  for (int pi = 0; pi < 4; pi++) {
    const int ca = wave * 8 + 2 * pi;
    const int ha = ca & 31;
    const int b = ca >= 32 ? b1 : b0;
    // (columns that do not exist - heads past the last, the second sample of an odd batch - are computed on the rows
    // of a head that does and not stored)
    const bool live_a = FULL || (ha < heads && (ca < 32 || valid1));   // uniform over the wave
    const bool live_b = FULL || (live_a && ha + 1 < heads);
    const bool more = pi + 1 < 4;
    const Prep& cp = prep[pi & 1];
    Prep& np = prep[(pi + 1) & 1];

    if (more && FULL) prep_step(0, pi + 2, np);
    // scale, add the logits, maximum over the 64 keys of this lane's query: 16 here, 48 in the lanes 16, 32, 48 away
    float sv[2][16], mx[2];
#pragma unroll
    for (int hb = 0; hb < 2; hb++) {
      const int c = ca + hb;
      const ev8 lg0 = *reinterpret_cast<const ev8*>(smem + LogitSlot(c, j, g4, 0));
      const ev8 lg1 = *reinterpret_cast<const ev8*>(smem + LogitSlot(c, j, g4, 2));
      mx[hb] = -3.0e38f;
#pragma unroll
      for (int t = 0; t < 4; t++)
#pragma unroll
        for (int e = 0; e < 4; e++) {
          const float lgv = (float)(t < 2 ? lg0[4 * t + e] : lg1[4 * (t - 2) + e]);
          sv[hb][4 * t + e] = cp.st[hb][t][e] * scale + lgv;
          mx[hb] = fmaxf(mx[hb], sv[hb][4 * t + e]);
        }
    }
    if (more && FULL) prep_step(1, pi + 2, np);
    Reduce4Rows2(mx[0], mx[1], [](float a, float b) { return fmaxf(a, b); });
    const float kLog2e = 1.44269504f;
#pragma unroll
    for (int hb = 0; hb < 2; hb++) {
      const float neg_mx = -mx[hb] * kLog2e;
#pragma unroll
      for (int e = 0; e < 16; e++) {
        sv[hb][e] = __builtin_amdgcn_exp2f(__builtin_fmaf(sv[hb][e], kLog2e, neg_mx));   // e^(s - mx) <= 1
      }
    }
    if (more && FULL) prep_step(2, pi + 2, np);
    ev8 pf[2][2];
#pragma unroll
    for (int hb = 0; hb < 2; hb++)
#pragma unroll
      for (int s2 = 0; s2 < 2; s2++)
#pragma unroll
        for (int e = 0; e < 8; e++) pf[hb][s2][e] = (ET)sv[hb][8 * s2 + e];
    if (more && FULL) prep_step(3, pi + 2, np);
    // O^T = V^T . P^T: lane (query j, g4), register e = depth index 16 dt + 4 g4 + e
#pragma unroll
    for (int hb = 0; hb < 2; hb++) {
      // Sum over all 64 keys of this lane's query, the same in all four registers: one more row block of the product,
      // with ones for V^T (no additions and no lane exchanges on the vector ALU).
      floatx4 den = zero4;
#pragma unroll
      for (int s2 = 0; s2 < 2; s2++) den = Mfma16(ones, pf[hb][s2], den);
      const float inv = __builtin_amdgcn_rcpf(den[0]);   // 1 ulp
      OutT* O = out + (long long)(b * 64 + kQueriesPerGroup * qt + j) * d_model + (ha + hb) * DEPTH + 4 * g4;
      const bool live = hb == 0 ? live_a : live_b;
#pragma unroll
      for (int dt = 0; dt < 2; dt++) {
        floatx4 o = zero4;
#pragma unroll
        for (int s2 = 0; s2 < 2; s2++) o = Mfma16(cp.vt[hb][dt][s2], pf[hb][s2], o);
        if (!live) continue;
        if constexpr (sizeof(OutT) == 1) {
          const float m = inv * out_mul;
          *reinterpret_cast<unsigned*>(O + 16 * dt) = PackFp8x4(o[0] * m, o[1] * m, o[2] * m, o[3] * m);
        } else {
          ev4 h4;
#pragma unroll
          for (int e = 0; e < 4; e++) h4[e] = (ET)(o[e] * inv);
          *reinterpret_cast<ev4*>(O + 16 * dt) = h4;
        }
      }
    }
    // (with liveness branches in the way the interleaved order needs more registers than there are: one pair after
    // the other then)
    if constexpr (!FULL) {
      if (more) {
#pragma unroll
        for (int step = 0; step < 4; step++) prep_step(step, pi + 2, np);
      }
    }
  }
}

template <typename OutT>
void LaunchT(const half_t* qkv, const half_t* gen, const half_t* wfrag, OutT* out, float out_mul, int batch, int heads,
             int depth, int gen_sz, float scale, hipStream_t stream, bool bf16 = false) {
  if (!SmolgenAttentionSupported(heads, depth, gen_sz)) {
    throw std::runtime_error("LaunchSmolgenAttention: unsupported shape");
  }
  if (batch <= 0) return;
  const int pairs = (batch + 1) / 2;
  const dim3 grid(((pairs + 7) / 8) * 32), block(512);
  // (an odd batch runs the full instance too: the last workgroup then takes its one sample twice and both halves store
  // the same values to the same places)
  const bool full = heads == 32;
  auto launch = [&](auto nks_tag, auto full_tag) {
    if constexpr (sizeof(OutT) == 2) {
      if (bf16) {
        hipLaunchKernelGGL((smolgen_attention_kernel<decltype(nks_tag)::value, OutT, decltype(full_tag)::value, bf16_t>), grid,
                           block, 0, stream, qkv, gen, wfrag, out, batch, heads, scale, out_mul);
        return;
      }
    }
    hipLaunchKernelGGL((smolgen_attention_kernel<decltype(nks_tag)::value, OutT, decltype(full_tag)::value, half_t>), grid,
                       block, 0, stream, qkv, gen, wfrag, out, batch, heads, scale, out_mul);
  };
  auto by_width = [&](auto full_tag) {
    switch (gen_sz) {
      case 256: launch(std::integral_constant<int, 16>{}, full_tag); break;
      case 128: launch(std::integral_constant<int, 8>{}, full_tag); break;
      default: launch(std::integral_constant<int, 2>{}, full_tag); break;
    }
  };
  if (full) by_width(std::true_type{});
  else by_width(std::false_type{});
}

}  // namespace

bool SmolgenAttentionSupported(int heads, int depth, int gen_sz) {
  return depth == 32 && heads >= 1 && heads <= 32 && (gen_sz == 32 || gen_sz == 128 || gen_sz == 256);
}

long long SmolgenFragmentIndex(int row, int col, int gen_sz) {
  const int nks = gen_sz / 16;
  const int rt = row / 32, rr = row % 32, ks = col / 16, gg = (col % 16) / 8, e = col % 8;
  return (((long long)rt * nks + ks) * 64 + gg * 32 + rr) * 8 + e;
}

void LaunchSmolgenAttention(const half_t* qkv, const half_t* gen, const half_t* wfrag, half_t* out, int batch,
                            int heads, int depth, int gen_sz, float scale, hipStream_t stream, bool bf16) {
  LaunchT<half_t>(qkv, gen, wfrag, out, 1.0f, batch, heads, depth, gen_sz, scale, stream, bf16);
}

void LaunchSmolgenAttentionF8Out(const half_t* qkv, const half_t* gen, const half_t* wfrag, uint8_t* out,
                                 float out_mul, int batch, int heads, int depth, int gen_sz, float scale,
                                 hipStream_t stream) {
  LaunchT<uint8_t>(qkv, gen, wfrag, out, out_mul, batch, heads, depth, gen_sz, scale, stream);
}

}  // namespace lc0mi
