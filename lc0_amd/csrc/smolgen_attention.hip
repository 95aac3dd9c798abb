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
//     halves in the layout phase 2 reads (128 KiB for the workgroup, XOR-swizzled so that both sides are free of
//     bank conflicts).
//   Phase 2 (memory and vector ALU): every wave takes 8 of the 64 (sample, head) columns, two at a time: S^T = K.Q^T for
//     the 16 queries of both heads (the 32-wide MFMA tile carries head A's queries in its lower and head B's in its
//     upper half), adds the logits from LDS, softmax over keys in registers plus one exchange with lane^32, then
//     O^T = V^T.P^T with V transposed on the matrix cores (no LDS staging) and 8-byte output stores straight from the
//     accumulators. K, Q and V of the next two heads are fetched while these are computed.
// Per workgroup 0.5 MiB of weights, 0.5 MiB of K and V and 64 KiB of Q come from L2; nothing but the output is written.
#include <hip/hip_runtime.h>

#include <stdexcept>

#include "device_math.h"
#include "kernels.h"

namespace lc0mi {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef _Float16 half4 __attribute__((ext_vector_type(4)));
typedef float floatx16 __attribute__((ext_vector_type(16)));

namespace {

constexpr int kQueriesPerGroup = 16;               // queries of one workgroup
constexpr int kLogitBytes = 2 * 2 * 16 * 2 * 64 * 16;   // [key half][8-key half][query][lane half][column slot] x 16 B
constexpr int kVBytesPerWave = 64 * 32 * 2;

// Byte offset of the 16-byte slot that holds eight logits (keys 32*mt + 8*(e/4) + 4*g + e%4 for e = 8*hf .. 8*hf+7)
// of query qq (0..15) in column c (0..63). Columns of one (mt, hf, qq, g) row are contiguous and rotated by qq, so that
// the 32 lanes that write one row (neighbouring columns) and the 16 x 2 lanes that read one column (all queries) each
// touch every bank group once.
__device__ __forceinline__ int LogitSlot(int c, int qq, int g, int mt, int hf) {
  return (((((mt * 2 + hf) * 16 + qq) * 2 + g) * 64) + (c ^ qq)) * 16;
}

template <int NKS, typename OutT>
__global__ __launch_bounds__(512, 1) void smolgen_attention_kernel(const half_t* __restrict__ qkv,
                                                                    const half_t* __restrict__ gen,
                                                                    const half_t* __restrict__ wfrag,
                                                                    OutT* __restrict__ out, int batch, int heads,
                                                                    float scale, float out_mul) {
  constexpr int DEPTH = 32;
  __shared__ __attribute__((aligned(1024))) unsigned char smem[kLogitBytes + 8 * kVBytesPerWave];
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
    const half8* wp = reinterpret_cast<const half8*>(wfrag) + ((long long)(32 * qt + wave * 4) * NKS) * 64 + lane;
    half8 ring[PF];
#pragma unroll
    for (int f = 0; f < PF; f++) ring[f] = wp[f * 64];
    // The generator vectors of the 64 columns: once per workgroup through LDS (the region phase 2 uses for V), 16-byte
    // slot s of column c at slot s ^ (c & 31) of its row, then into the registers of every wave as MFMA "B" operands.
    unsigned char* gl = smem + kLogitBytes;
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
    half8 bf[2][NKS];
#pragma unroll
    for (int ct = 0; ct < 2; ct++)
#pragma unroll
      for (int ks = 0; ks < NKS; ks++) {
        const int c = ct * 32 + r;
        bf[ct][ks] = *reinterpret_cast<const half8*>(gl + (c * kSlotsPerCol + ((ks * 2 + g) ^ (c & (kSlotsPerCol - 1)))) * 16);
      }
    floatx16 acc[2];
#pragma unroll
    for (int f = 0; f < NF; f++) {
      const int ks = f % NKS;
      if (ks == 0) {
#pragma unroll
        for (int e = 0; e < 16; e++) { acc[0][e] = 0.0f; acc[1][e] = 0.0f; }
      }
      const half8 a = ring[f % PF];
      if (f + PF < NF) ring[f % PF] = wp[(f + PF) * 64];
      acc[0] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, bf[0][ks], acc[0], 0, 0, 0);
      acc[1] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, bf[1][ks], acc[1], 0, 0, 0);
      if (ks == NKS - 1) {
        const int rt = wave * 4 + f / NKS;   // row tile within the query group
        const int qq = rt >> 1, mt = rt & 1;
#pragma unroll
        for (int ct = 0; ct < 2; ct++)
#pragma unroll
          for (int hf = 0; hf < 2; hf++) {
            half8 hv;
#pragma unroll
            for (int e = 0; e < 8; e++) hv[e] = (half_t)acc[ct][hf * 8 + e];
            *reinterpret_cast<half8*>(smem + LogitSlot(ct * 32 + r, qq, g, mt, hf)) = hv;
          }
      }
    }
  }
  __syncthreads();

  // ---- phase 2: attention of the 16 queries, eight (sample, head) columns per wave, two at a time ----
  // Lanes r < 16 of each half work on head A (an even column), lanes r >= 16 on head B (the next column), both for
  // queries 0..15, so that the softmax arithmetic is spent on 32 distinct (head, query) pairs per half:
  //   S^T:  one MFMA chain over the concatenated depth of both heads, [K_A | K_B] against query columns that carry
  //         [q_A ; 0] in lanes r < 16 and [0 ; q_B] in lanes r >= 16;
  //   V:    loaded by rows like K and transposed on the matrix cores (V_tile . I leaves, in the accumulator layout, a
  //         lane per depth index holding keys, which is the operand layout of the product below);
  //   O^T = V^T . P^T per head, so that a lane ends up with 16 depth values of its own query and stores them directly;
  //         each lane keeps the product with its own head's V.
  const int qq = r & 15;
  const bool is_b = r >= 16;
  // K and V of a head pair are fetched by 128-byte rows (both heads' 32 halves side by side), eight lanes per row, so
  // that every load instruction touches eight full cache lines instead of 32 partial ones; a tile of 32 rows then
  // passes through this wave's 4 KiB of LDS (16-byte chunk c of row w at chunk c ^ ((w >> 1) & 7): both directions
  // free of bank conflicts) to reach the lanes in operand layout.
  const int lr = lane >> 3, ch = lane & 7;
  unsigned char* stg = smem + kLogitBytes + wave * kVBytesPerWave;
  struct PairData {
    half8 k[2][4], v[2][4];   // [32-row tile][8-row group]
    half8 qf[2];              // this lane's head
  };
  auto load_pair = [&](int pi, PairData& d) {
    const int ca = wave * 8 + 2 * pi;
    const int b = ca >= 32 ? b1 : b0;
    const int ha = ca & 31;
    const int ha_c = ha < heads ? ha : 0;
    const bool has_b = ha_c + 1 < heads;
    const half_t* base = qkv + (long long)b * 64 * ld;
    // (without a head B the upper half of the row repeats head A instead of running past the row)
    const half_t* Kp = base + d_model + ha_c * DEPTH + (has_b ? ch : (ch & 3)) * 8 + (unsigned)lr * (unsigned)ld;
    const half_t* Vp = Kp + d_model;
#pragma unroll
    for (int t = 0; t < 2; t++)
#pragma unroll
      for (int i = 0; i < 4; i++) {
        const unsigned off = (unsigned)(32 * t + 8 * i) * (unsigned)ld;
        d.k[t][i] = *reinterpret_cast<const half8*>(Kp + off);
        d.v[t][i] = *reinterpret_cast<const half8*>(Vp + off);
      }
    const half_t* Q = base + (is_b && has_b ? ha_c + 1 : ha_c) * DEPTH +
                      (unsigned)(kQueriesPerGroup * qt + qq) * (unsigned)ld + 8u * g;
#pragma unroll
    for (int ks = 0; ks < 2; ks++) d.qf[ks] = *reinterpret_cast<const half8*>(Q + 16 * ks);
  };
  // fr[head][k-step]: rows of the tile in MFMA operand layout (lane r = row, g = 8-half group of the k-step)
  auto stage_tile = [&](const half8 (&raw)[4], half8 (&fr)[2][2]) {
#pragma unroll
    for (int i = 0; i < 4; i++) {
      const int row = 8 * i + lr;
      *reinterpret_cast<half8*>(stg + row * 128 + ((ch ^ ((row >> 1) & 7)) * 16)) = raw[i];
    }
#pragma unroll
    for (int hb = 0; hb < 2; hb++)
#pragma unroll
      for (int ks = 0; ks < 2; ks++) {
        const int c = hb * 4 + ks * 2 + g;
        fr[hb][ks] = *reinterpret_cast<const half8*>(stg + r * 128 + ((c ^ ((r >> 1) & 7)) * 16));
      }
  };
  // Identity fragments: B operand of the transposing product, element (k, j) = [k == j].
  half8 ident[2];
#pragma unroll
  for (int ks = 0; ks < 2; ks++)
#pragma unroll
    for (int e = 0; e < 8; e++) ident[ks][e] = (16 * ks + 8 * g + e == r) ? (half_t)1.0f : (half_t)0.0f;
  const half8 zero8 = {0, 0, 0, 0, 0, 0, 0, 0};

  PairData cur, nxt;
  load_pair(0, cur);
#pragma unroll
  for (int pi = 0; pi < 4; pi++) {
    const int ca = wave * 8 + 2 * pi;
    const int ha = ca & 31;
    const bool live_a = ha < heads && (ca < 32 || valid1);   // uniform over the wave
    const bool live_b = live_a && ha + 1 < heads;
    if (pi + 1 < 4) load_pair(pi + 1, nxt);
    if (live_a) {
      const int b = ca >= 32 ? b1 : b0;
      // S^T[key][lane's (head, query)]
      half8 qcat[4];
#pragma unroll
      for (int ks = 0; ks < 2; ks++) {
        qcat[ks] = is_b ? zero8 : cur.qf[ks];
        qcat[2 + ks] = is_b ? cur.qf[ks] : zero8;
      }
      floatx16 st[2];
#pragma unroll
      for (int mt = 0; mt < 2; mt++) {
        half8 kf[2][2];
        stage_tile(cur.k[mt], kf);
#pragma unroll
        for (int e = 0; e < 16; e++) st[mt][e] = 0.0f;
#pragma unroll
        for (int ks = 0; ks < 4; ks++)
          st[mt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(kf[ks >> 1][ks & 1], qcat[ks], st[mt], 0, 0, 0);
      }
      // V^T of both heads as halves in operand layout: vt[head][s] covers keys 16 s .. 16 s + 15
      half8 vt[2][4];
#pragma unroll
      for (int mt = 0; mt < 2; mt++) {
        half8 vr[2][2];
        stage_tile(cur.v[mt], vr);
#pragma unroll
        for (int hb = 0; hb < 2; hb++) {
          floatx16 tr;
#pragma unroll
          for (int e = 0; e < 16; e++) tr[e] = 0.0f;
#pragma unroll
          for (int ks = 0; ks < 2; ks++)
            tr = __builtin_amdgcn_mfma_f32_32x32x16_f16(vr[hb][ks], ident[ks], tr, 0, 0, 0);
#pragma unroll
          for (int e = 0; e < 8; e++) {
            vt[hb][2 * mt][e] = (half_t)tr[e];
            vt[hb][2 * mt + 1][e] = (half_t)tr[8 + e];
          }
        }
      }
      // scale, add the logits, softmax over the 64 keys of this lane's (head, query): 32 here, 32 in lane^32
      const int myc = ca + (is_b && live_b ? 1 : 0);
      float mx = -3.0e38f;
#pragma unroll
      for (int mt = 0; mt < 2; mt++)
#pragma unroll
        for (int hf = 0; hf < 2; hf++) {
          const half8 bv = *reinterpret_cast<const half8*>(smem + LogitSlot(myc, qq, g, mt, hf));
#pragma unroll
          for (int e = 0; e < 8; e++) {
            const float sv = st[mt][hf * 8 + e] * scale + (float)bv[e];
            st[mt][hf * 8 + e] = sv;
            mx = fmaxf(mx, sv);
          }
        }
      mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
      float sum = 0.0f;
      const float kLog2e = 1.44269504f, neg_mx = -mx * kLog2e;
#pragma unroll
      for (int mt = 0; mt < 2; mt++)
#pragma unroll
        for (int e = 0; e < 16; e++) {
          const float ev = __builtin_amdgcn_exp2f(__builtin_fmaf(st[mt][e], kLog2e, neg_mx));   // e^(s - mx)
          st[mt][e] = ev;
          sum += ev;
        }
      sum += __shfl_xor(sum, 32, 64);
      const float inv = 1.0f / sum;
      half8 pf[4];
#pragma unroll
      for (int s4 = 0; s4 < 4; s4++)
#pragma unroll
        for (int e = 0; e < 8; e++) pf[s4][e] = (half_t)st[s4 / 2][8 * (s4 % 2) + e];   // e^(s - mx) <= 1
      // O^T = V^T . P^T: lane (its head and query, g), register e = depth index 8*(e/4) + 4*g + e%4
      floatx16 oa, ob;
#pragma unroll
      for (int e = 0; e < 16; e++) { oa[e] = 0.0f; ob[e] = 0.0f; }
#pragma unroll
      for (int s4 = 0; s4 < 4; s4++) {
        oa = __builtin_amdgcn_mfma_f32_32x32x16_f16(vt[0][s4], pf[s4], oa, 0, 0, 0);
        ob = __builtin_amdgcn_mfma_f32_32x32x16_f16(vt[1][s4], pf[s4], ob, 0, 0, 0);
      }
      if (!is_b || live_b) {
        OutT* O = out + (long long)(b * 64 + kQueriesPerGroup * qt + qq) * d_model + (ha + (is_b ? 1 : 0)) * DEPTH + 4 * g;
#pragma unroll
        for (int j4 = 0; j4 < 4; j4++) {
          float v4[4];
#pragma unroll
          for (int e = 0; e < 4; e++) v4[e] = (is_b ? ob[4 * j4 + e] : oa[4 * j4 + e]) * inv;   // this lane's own query
          if constexpr (sizeof(OutT) == 1) {
            *reinterpret_cast<unsigned*>(O + 8 * j4) =
                PackFp8x4(v4[0] * out_mul, v4[1] * out_mul, v4[2] * out_mul, v4[3] * out_mul);
          } else {
            half4 h4;
#pragma unroll
            for (int e = 0; e < 4; e++) h4[e] = (half_t)v4[e];
            *reinterpret_cast<half4*>(O + 8 * j4) = h4;
          }
        }
      }
    }
    if (pi + 1 < 4) cur = nxt;
  }
}

template <typename OutT>
void LaunchT(const half_t* qkv, const half_t* gen, const half_t* wfrag, OutT* out, float out_mul, int batch, int heads,
             int depth, int gen_sz, float scale, hipStream_t stream) {
  if (!SmolgenAttentionSupported(heads, depth, gen_sz)) {
    throw std::runtime_error("LaunchSmolgenAttention: unsupported shape");
  }
  if (batch <= 0) return;
  const int pairs = (batch + 1) / 2;
  const dim3 grid(((pairs + 7) / 8) * 32), block(512);
  switch (gen_sz) {
    case 256:
      hipLaunchKernelGGL((smolgen_attention_kernel<16, OutT>), grid, block, 0, stream, qkv, gen, wfrag, out, batch,
                         heads, scale, out_mul);
      break;
    case 128:
      hipLaunchKernelGGL((smolgen_attention_kernel<8, OutT>), grid, block, 0, stream, qkv, gen, wfrag, out, batch,
                         heads, scale, out_mul);
      break;
    default:
      hipLaunchKernelGGL((smolgen_attention_kernel<2, OutT>), grid, block, 0, stream, qkv, gen, wfrag, out, batch,
                         heads, scale, out_mul);
      break;
  }
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
                            int heads, int depth, int gen_sz, float scale, hipStream_t stream) {
  LaunchT<half_t>(qkv, gen, wfrag, out, 1.0f, batch, heads, depth, gen_sz, scale, stream);
}

void LaunchSmolgenAttentionF8Out(const half_t* qkv, const half_t* gen, const half_t* wfrag, uint8_t* out,
                                 float out_mul, int batch, int heads, int depth, int gen_sz, float scale,
                                 hipStream_t stream) {
  LaunchT<uint8_t>(qkv, gen, wfrag, out, out_mul, batch, heads, depth, gen_sz, scale, stream);
}

}  // namespace lc0mi
