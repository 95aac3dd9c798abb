// Persistent large-shape GEMM for gfx950:  C = act(A . W^T + bias), half in, half out, fp32 accumulation
// (FullyConnectedLayer::Forward1D, src/neural/backends/blas/fully_connected_layer.cc:49-106, for the shapes of
// the encoder's QKV / output / FFN projections and the smolgen generator, src/neural/backends/blas/network_blas.cc:
// 320-347, 446-464).
//
// One workgroup of four waves (one per SIMD, 512 registers each) per CU walks over 256 x 256 output tiles:
//   * each wave owns a 128 x 128 part of the tile as 4 x 4 MFMA tiles (v_mfma_f32_32x32x16_f16, 256 accumulator
//     registers); in program order every MFMA is followed by exactly one LDS fragment read or one operand transfer,
//     so the single instruction stream of a SIMD keeps the matrix pipe, the LDS and the memory pipe busy together;
//   * operand tiles go from global memory straight into LDS (global_load_lds_dwordx4, two 64 KiB stages with the
//     XOR-swizzled layout of gemm_dma_kernel) and run two k-tiles ahead of the MFMAs, across tile boundaries: a new
//     tile starts with its first two k-tiles already in LDS;
//   * the bias enters through one extra MFMA per accumulator tile (ones x (hi, lo) halves of the bias), the finished
//     tile is converted to halves strip by strip (32 rows per wave): two strips are transposed through an 8 KiB LDS
//     buffer per wave and stored at once, the third waits in that buffer and the fourth in registers, and both are
//     stored in pieces of four 16-byte stores during the next tile's main loop, so that the memory system sees a
//     steady stream of writes instead of one burst per tile from all CUs at once.
// Vector memory operations retire in issue order (loads and stores share vmcnt), which the waits rely on: "the
// transfers of the next k-tile have landed" is vmcnt(number of stores issued after them).
//
// Shapes: M, N multiples of 256, K a multiple of 128 and at least 256, row strides multiples of 8 elements,
// one matrix per launch, scale 1. Everything else goes to the kernels in kernels.hip.
#include <hip/hip_runtime.h>

#include <type_traits>

#include "device_math.h"
#include "kernels.h"

namespace lc0mi {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef _Float16 half4 __attribute__((ext_vector_type(4)));
typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef unsigned uintx2 __attribute__((ext_vector_type(2)));
typedef unsigned uintx4 __attribute__((ext_vector_type(4)));

namespace {

#define LC0MI_SB() __builtin_amdgcn_sched_barrier(0)

// 16 bytes per lane from global memory (uniform base + 32-bit lane offset) into LDS at lds_addr + lane * 16, for
// all lanes or none (mask = all ones or zero): the transfers past the last tile are switched off without a branch.
__device__ __forceinline__ void DmaToLds16Masked(const half_t* base, unsigned byte_off, unsigned lds_addr,
                                                 unsigned long long mask) {
  asm volatile("s_mov_b64 exec, %3\n\ts_mov_b32 m0, %0\n\tglobal_load_lds_dwordx4 %1, %2\n\ts_mov_b64 exec, -1"
               ::"s"(lds_addr), "v"(byte_off), "s"(base), "s"(mask) : "memory", "m0");
}
__device__ __forceinline__ void LdsWrite8(unsigned lds_addr, uintx2 v) {
  *reinterpret_cast<__attribute__((address_space(3))) uintx2*>(lds_addr) = v;
}

template <int ACT>
__device__ __forceinline__ float ActivateT(float v) {
  if constexpr (ACT == kActNone) return v;
  else if constexpr (ACT == kActMish) return ActMish(v);
  else if constexpr (ACT == kActRelu) return v > 0.0f ? v : 0.0f;
  else if constexpr (ACT == kActSwish) return v * ActSigmoid(v);
  else if constexpr (ACT == kActRelu2) return v > 0.0f ? v * v : 0.0f;
  else return Activate(v, ACT);
}

template <int ACT>
__global__ __launch_bounds__(256, 1) void gemm_persistent_kernel(GemmArgs p, int tiles_m, int tiles_n, int stream_stores) {
  constexpr int BM = 256, BN = 256, BK = 64;
  constexpr int WM = 128, WN = 128, TM = 4, TN = 4;
  constexpr int STAGE_B = (BM + BN) * BK * 2;   // bytes
  constexpr int STRIP_B = 32 * WN * 2;          // bytes: 32 rows of this wave's 128 columns
  __shared__ __attribute__((aligned(1024))) char smem[2 * STAGE_B + 4 * STRIP_B];

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave >> 1, wn = wave & 1;
  const int nk = p.K / BK;   // even, at least 4
  const int ntiles = tiles_m * tiles_n;
  const int r = lane & 31, g = lane >> 5;
  const int swz = (r >> 1) % 8;   // chunk swizzle of the row
  const unsigned lds0 = (unsigned)(size_t)((__attribute__((address_space(3))) void*)smem);
  const unsigned strip_lds = lds0 + 2 * STAGE_B + wave * STRIP_B;

  // ---- operand transfer state (runs two k-tiles ahead of the computation, across tiles) ----
  // Chunk q of this wave covers tile rows (wave*8 + q)*8 .. +7; a lane moves 16 bytes of row lane/8. The
  // swizzled chunk column depends on the lane and on the parity of q only; the k offset lives in the lane part.
  int dma_tile = blockIdx.x, dma_k = 0;
  if (dma_tile >= ntiles) return;
  unsigned long long dma_mask = ~0ull;
  unsigned a_lane[2], w_lane[2];
#pragma unroll
  for (int par = 0; par < 2; par++) {
    const int c = (lane % 8) ^ ((4 * par + lane / 16) % 8);
    a_lane[par] = (unsigned)((lane / 8) * p.lda + c * 8) * 2u;
    w_lane[par] = (unsigned)((lane / 8) * p.ldw + c * 8) * 2u;
  }
  const half_t* abase[8];
  const half_t* wbase[8];
  auto set_bases = [&](int tile) {
    const int m0 = (tile % tiles_m) * BM, n0 = (tile / tiles_m) * BN;
#pragma unroll
    for (int q = 0; q < 8; q++) {
      abase[q] = p.A + (long long)(m0 + (wave * 8 + q) * 8) * p.lda;
      wbase[q] = p.W + (long long)(n0 + (wave * 8 + q) * 8) * p.ldw;
    }
  };
  set_bases(dma_tile);
  auto dma = [&](int q, int st) {
    if (q < 8) DmaToLds16Masked(abase[q], a_lane[q & 1], lds0 + st * STAGE_B + (wave * 8 + q) * 1024, dma_mask);
    else DmaToLds16Masked(wbase[q - 8], w_lane[q & 1], lds0 + st * STAGE_B + BM * BK * 2 + (wave * 8 + (q - 8)) * 1024, dma_mask);
  };
  auto dma_advance = [&]() {
    dma_k++;
#pragma unroll
    for (int par = 0; par < 2; par++) { a_lane[par] += BK * 2; w_lane[par] += BK * 2; }
    if (dma_k == nk) {
      dma_k = 0;
      dma_tile += gridDim.x;
      if (dma_tile < ntiles) set_bases(dma_tile); else dma_mask = 0;
#pragma unroll
      for (int par = 0; par < 2; par++) { a_lane[par] -= nk * BK * 2; w_lane[par] -= nk * BK * 2; }
    }
  };

  floatx16 acc[TM][TN];
  // Fragment addresses: row (wm*128 + r) resp. (wn*128 + r) of the stage, 16-byte chunk (2*ks + g) ^ swz. Bits 5..6
  // of the address carry ks, so one register per operand serves all four sub-steps through an XOR; the two
  // registers are passed through an empty asm at the start of every k-tile so that the derived addresses are
  // formed where they are used instead of living in registers (or in spill slots) across the loop.
  unsigned frag_a = lds0 + (wm * WM + r) * BK * 2 + ((g ^ swz) * 16);
  unsigned frag_w = lds0 + BM * BK * 2 + (wn * WN + r) * BK * 2 + ((g ^ swz) * 16);
  auto read_frag = [&](int st, int ks, int f) -> half8 {
    const unsigned base = ((f < 4 ? frag_a : frag_w) ^ (ks * 32)) + st * STAGE_B;
    return *reinterpret_cast<const __attribute__((address_space(3))) half8*>(base + (f & 3) * 32 * BK * 2);
  };

  // ---- deferred output of the previous tile: strip 2 waits in LDS, strip 3 in registers ----
  unsigned outp[32];
#pragma unroll
  for (int e = 0; e < 32; e++) outp[e] = 0;
  int pend = 5;                  // next deferred step (5 = nothing pending)
  const char* out_base = reinterpret_cast<const char*>(p.C);   // &C[m0 + wm*128][n0 + wn*128] of the pending tile (uniform)
  unsigned out_lane = (unsigned)((lane >> 4) * p.ldc + (lane & 15) * 8) * 2u;   // row lane/16, 16-byte piece lane%16
  auto store_piece = [&](int row0, uintx4 v) {   // rows row0 .. row0+3 of the wave's 128 x 128 part
    char* b = const_cast<char*>(out_base) + (long long)row0 * p.ldc * 2;
    uintx4* dst = reinterpret_cast<uintx4*>(b + out_lane);
    if (stream_stores) __builtin_nontemporal_store(v, dst); else *dst = v;
  };
  // element c = j * 4 + blk: columns j*32 + blk*8 + g*4 .. +3 of row r
  unsigned put_base = (strip_lds + r * 256 + g * 8) | ((r & 15) << 4);   // bits 4..7 of the strip row are free
  auto put_addr = [&](int c) -> unsigned { return put_base ^ (c * 16); };
  // (put_base is passed through an empty asm before each group of uses so that the sixteen addresses are
  // formed where they are used instead of being kept in registers across the main loop)
#define LC0MI_FRESH_PUT_BASE() asm volatile("" : "+v"(put_base))
  // row = h*16 + pass*4 + lane/16, chunk (lane%16) ^ (row%16) = ((lane%16) ^ (lane/16)) ^ (pass*4): one lane-dependent
  // address, an XOR on bits 6..7 and an immediate offset per (h, pass)
  unsigned rd_base = strip_lds + (lane >> 4) * 256 + (((lane & 15) ^ (lane >> 4)) * 16);
  auto strip_read = [&](int h, int pass) -> uintx4 {
    return *reinterpret_cast<const __attribute__((address_space(3))) uintx4*>((rd_base ^ (pass * 64)) + h * 4096 + pass * 1024);
  };
#define LC0MI_FRESH_RD_BASE() asm volatile("" : "+v"(rd_base))

  half8 fr[2][8];
  // One k-tile in stage ST. sub 0: nothing extra; 1: copy strip 3 of the pending tile from registers to LDS;
  // 2: write half sh of the strip in LDS to rows srow .. srow+15 of the pending tile.
  bool after_burst = false;   // the 16 stores of strips 0 and 1 were issued since the last transfer wait
  auto ktile = [&](auto st_c, int sub, int sh, int srow) {
    constexpr int ST = decltype(st_c)::value;
    asm volatile("" : "+v"(frag_a), "+v"(frag_w));
    uintx4 tmp[4];
#pragma unroll
    for (int ks = 0; ks < 4; ks++) {
      const int cb = ks & 1, nb = cb ^ 1;
#pragma unroll
      for (int q = 0; q < 16; q++) {
        const int i = q >> 2, j = (q & 3) ^ ((i & 1) ? 3 : 0);
        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(fr[cb][4 + j], fr[cb][i], acc[i][j], 0, 0, 0);
        LC0MI_SB();
        if (ks < 3) {
          if (q < 8) fr[nb][q] = read_frag(ST, ks + 1, q);
          if (ks == 0 && q == 8 && sub == 1) {
            LC0MI_FRESH_PUT_BASE();
#pragma unroll
            for (int c = 0; c < 16; c++) LdsWrite8(put_addr(c), uintx2{outp[c * 2], outp[c * 2 + 1]});
          }
          if (ks == 1 && q == 8 && sub == 2) {
            LC0MI_FRESH_RD_BASE();
#pragma unroll
            for (int z = 0; z < 4; z++) tmp[z] = strip_read(sh, z);
          }
        } else {
          if (q == 1) {
            // This wave's transfers of the next k-tile have landed. They are older than the stores of the tile
            // end, and loads and stores retire in order: right after a tile end 16 stores may still be in flight.
            if (after_burst) __builtin_amdgcn_s_waitcnt(0x4F70); else __builtin_amdgcn_s_waitcnt(0x0F70);
            after_burst = false;
            __builtin_amdgcn_s_barrier();         // everybody's transfers; everybody is done with stage ST
            if (sub == 2) {
#pragma unroll
              for (int z = 0; z < 4; z++) store_piece(srow + z * 4, tmp[z]);
            }
          }
          if (q >= 2 && q < 10) fr[nb][q - 2] = read_frag(ST ^ 1, 0, q - 2);
          if (q >= 2) { dma(q - 2, ST); if (q == 15) { dma(14, ST); dma(15, ST); } }
        }
        LC0MI_SB();
      }
    }
    dma_advance();
  };
  // deferred steps: 0,1 = halves of strip 2 (LDS -> memory), 2 = strip 3 registers -> LDS, 3,4 = halves of strip 3
  auto run_ktile = [&](auto st_c) {
    int sub = 0, sh = 0, srow = 0;
    if (pend < 5) {
      const int s = pend++;
      if (s == 2) sub = 1;
      else { sub = 2; sh = s < 2 ? s : s - 3; srow = (s < 2 ? 2 : 3) * 32 + sh * 16; }
    }
    ktile(st_c, sub, sh, srow);
  };
  auto flush = [&]() {
    while (pend < 5) {
      const int s = pend++;
      if (s == 2) {
        LC0MI_FRESH_PUT_BASE();
#pragma unroll
        for (int c = 0; c < 16; c++) LdsWrite8(put_addr(c), uintx2{outp[c * 2], outp[c * 2 + 1]});
      } else {
        const int si = s < 2 ? 2 : 3, sh = s < 2 ? s : s - 3;
        LC0MI_FRESH_RD_BASE();
#pragma unroll
        for (int pass = 0; pass < 4; pass++) store_piece(si * 32 + sh * 16 + pass * 4, strip_read(sh, pass));
      }
    }
  };

  // ---- prologue: k-tiles 0 and 1 of the first tile ----
#pragma unroll
  for (int q = 0; q < 16; q++) dma(q, 0);
  dma_advance();
#pragma unroll
  for (int q = 0; q < 16; q++) dma(q, 1);
  dma_advance();
  __builtin_amdgcn_s_waitcnt(0x4F70);   // vmcnt(16): k-tile 0 has landed
  __builtin_amdgcn_s_barrier();
#pragma unroll
  for (int f = 0; f < 8; f++) fr[0][f] = read_frag(0, 0, f);

  float bias_next[TN];
#pragma unroll
  for (int j = 0; j < TN; j++) bias_next[j] = p.bias ? p.bias[(blockIdx.x / tiles_m) * BN + wn * WN + j * 32 + r] : 0.0f;
  for (int tile = blockIdx.x; tile < ntiles; tile += gridDim.x) {
    const int m0 = (tile % tiles_m) * BM, n0 = (tile / tiles_m) * BN;
    // bias enters through one extra MFMA: A fragment = 1 at k = 0 and 1, W fragment = (hi, lo) halves of the bias
    {
      typedef unsigned uintx4v __attribute__((ext_vector_type(4)));
      floatx16 zero;
#pragma unroll
      for (int e = 0; e < 16; e++) zero[e] = 0.0f;
#pragma unroll
      for (int j = 0; j < TN; j++) {
        const float b = bias_next[j];
        const half_t hi = (half_t)b;
        const half_t lo = (half_t)(b - (float)hi);
        half8 bf = {0, 0, 0, 0, 0, 0, 0, 0};
        if (g == 0) { bf[0] = hi; bf[1] = lo; }
#pragma unroll
        for (int i = 0; i < TM; i++) {
          unsigned ob = g == 0 ? 0x3C003C00u : 0u;   // halves (1.0, 1.0) at k = 0, 1
          asm volatile("" : "+v"(ob));               // keeps the sixteen products apart (no copies between accumulator tiles)
          const uintx4v ov = {ob, 0u, 0u, 0u};
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(bf, *reinterpret_cast<const half8*>(&ov), zero, 0, 0, 0);
        }
      }
    }
    for (int t = 0; t < nk; t += 2) {
      run_ktile(std::integral_constant<int, 0>{});
      run_ktile(std::integral_constant<int, 1>{});
    }
    if (tile + (int)gridDim.x < ntiles) {
#pragma unroll
      for (int j = 0; j < TN; j++) bias_next[j] = p.bias ? p.bias[((tile + gridDim.x) / tiles_m) * BN + wn * WN + j * 32 + r] : 0.0f;
    }
    // ---- the tile is complete ----
    flush();
    out_base = reinterpret_cast<const char*>(static_cast<const half_t*>(p.C) + (long long)(m0 + wm * WM) * p.ldc + n0 + wn * WN);
    asm volatile("" : "+v"(out_lane));
    // strips 0 and 1 go out now, strip 2 stays in LDS, strip 3 in registers
#pragma unroll
    for (int i = 0; i < TM; i++) {
      LC0MI_FRESH_PUT_BASE();
#pragma unroll
      for (int j = 0; j < TN; j++) {
#pragma unroll
        for (int blk = 0; blk < 4; blk++) {
          half4 h;
#pragma unroll
          for (int rr = 0; rr < 4; rr++) h[rr] = (half_t)ActivateT<ACT>(acc[i][j][blk * 4 + rr]);
          const uintx2 v = *reinterpret_cast<const uintx2*>(&h);
          const int c = j * 4 + blk;
          if (i < 3) LdsWrite8(put_addr(c), v);
          else { outp[c * 2] = v.x; outp[c * 2 + 1] = v.y; }
        }
        LC0MI_SB();   // one accumulator tile at a time: keeps the conversion from needing 256 registers at once
      }
      if (i < 2) {
        LC0MI_FRESH_RD_BASE();
#pragma unroll
        for (int h2 = 0; h2 < 2; h2++)
#pragma unroll
          for (int pass = 0; pass < 4; pass++) store_piece(i * 32 + h2 * 16 + pass * 4, strip_read(h2, pass));
      }
    }
    pend = 0;
    after_burst = true;
  }
  flush();
}


#undef LC0MI_FRESH_PUT_BASE
#undef LC0MI_FRESH_RD_BASE

int NumCus() {
  static int cus = 0;
  if (cus == 0) {
    int dev = 0;
    hipDeviceProp_t prop;
    if (hipGetDevice(&dev) == hipSuccess && hipGetDeviceProperties(&prop, dev) == hipSuccess) cus = prop.multiProcessorCount;
    if (cus <= 0) cus = 256;
  }
  return cus;
}

template <int ACT>
void Launch(const GemmArgs& a, int tiles_m, int tiles_n, int stream_stores, hipStream_t stream) {
  const int tiles = tiles_m * tiles_n;
  const int grid = tiles < NumCus() ? tiles : NumCus();
  hipLaunchKernelGGL(gemm_persistent_kernel<ACT>, dim3(grid), dim3(256), 0, stream, a, tiles_m, tiles_n, stream_stores);
}

}  // namespace

bool GemmPersistentSupports(const GemmArgs& a) {
  if (a.out_f32 || a.split_k != 1 || a.batch != 1 || a.scale != 1.0f) return false;
  if (a.M % 256 || a.N % 256 || a.K % 128 || a.K < 256) return false;
  if (a.lda % 8 || a.ldw % 8 || a.ldc % 8) return false;
  if ((reinterpret_cast<uintptr_t>(a.A) | reinterpret_cast<uintptr_t>(a.W) | reinterpret_cast<uintptr_t>(a.C)) & 15) return false;
  // 32-bit lane offsets: eight rows of A / W plus the k range, four rows of C
  if ((long long)8 * a.lda * 2 + (long long)a.K * 2 >= (1ll << 31) || (long long)8 * a.ldw * 2 + (long long)a.K * 2 >= (1ll << 31)) return false;
  switch (a.act) {
    case kActNone: case kActMish: case kActRelu: case kActSwish: case kActRelu2: return true;
    default: return false;
  }
}

void LaunchGemmPersistent(const GemmArgs& a, bool stream_stores, hipStream_t stream) {
  const int tiles_m = a.M / 256, tiles_n = a.N / 256;
  switch (a.act) {
    case kActMish: Launch<kActMish>(a, tiles_m, tiles_n, stream_stores, stream); break;
    case kActRelu: Launch<kActRelu>(a, tiles_m, tiles_n, stream_stores, stream); break;
    case kActSwish: Launch<kActSwish>(a, tiles_m, tiles_n, stream_stores, stream); break;
    case kActRelu2: Launch<kActRelu2>(a, tiles_m, tiles_n, stream_stores, stream); break;
    default: Launch<kActNone>(a, tiles_m, tiles_n, stream_stores, stream); break;
  }
}

}  // namespace lc0mi
