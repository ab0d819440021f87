// Triangle contraction on bf16 MFMA:  T[c][i][j] = sum_k A[c][i][k] * B[c][j][k]
// for a batch of channels c, bf16 in and out, fp32 accumulation.
//
// Both operands are k-contiguous (the natural fragment order of
// v_mfma_f32_32x32x16_bf16).  What bounds this product on a CU is not the matrix
// unit but the operand traffic per MFMA, out of LDS and out of L2: a wave that
// owns a 64x64 corner reads one 16-byte fragment per MFMA and with eight such
// waves on a CU the LDS pipe is as busy as the matrix unit.  So the tile is as
// large as the register file allows: one workgroup of four waves per CU, a
// 256x256 block with a 64-deep k slab, each wave a 128x128 quadrant = 4x4 MFMA
// tiles = 256 fp32 accumulators (the unified 512-entry register file of a lone
// wave per SIMD), half a fragment read per MFMA and twice the FLOPs per byte
// fetched from L2.  Slabs are double-buffered in LDS (144 KB) and prefetched
// through two register sets (two slabs ahead of the MFMAs), one barrier per
// slab; global loads, LDS fragment reads and LDS stores are interleaved with
// the MFMA stream explicitly, because the lone wave of a SIMD has nobody to
// cover for it while one of them blocks its instruction stream.
//
// The accumulators hold T^T tiles (B fragments as the MFMA's A operand), so a
// lane owns one output row i and four consecutive columns j per register quad:
// the epilogue packs those to 8 bytes, stages each wave's quadrant through LDS
// and writes full 256-byte rows.
#include <type_traits>

#include "common.h"
#include "kernels.h"

namespace {

constexpr int CM = 256, CN = 256, CK = 64;
constexpr int LDT = CK + 8;      // LDS row stride of a slab (bf16): 144 B keeps the 16-byte reads conflict-free
constexpr int LDE = 128 + 8;     // LDS row stride of a wave's staged output quadrant (bf16)
constexpr int STAGE = (CM + CN) * LDT;

__global__ __launch_bounds__(256, 1) void contract_kernel(GemmArgs g) {
  __shared__ __attribute__((aligned(16))) bf16_t smem[2 * STAGE];
  static_assert(4 * 128 * LDE <= 2 * STAGE, "output staging must fit");

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int hh = lane >> 5, l31 = lane & 31;
  const int wm = (wave >> 1) * 128, wn = (wave & 1) * 128;

  // XCD-aware mapping: workgroup ids are dealt round-robin to the 8 XCDs, so
  // id -> (xcd, slot) -> logical id makes each XCD walk a contiguous range of
  // (channel, j-tile, i-tile), i-tile fastest: the tiles that share a channel's
  // A and B panels run on one XCD and find them in its L2.
  const int tiles_m = (g.M + CM - 1) / CM, tiles_n = (g.N + CN - 1) / CN;
  const int total = tiles_m * tiles_n * g.batch;
  const int per_xcd = (total + 7) / 8;
  const int logical = (blockIdx.x & 7) * per_xcd + (blockIdx.x >> 3);
  if (logical >= total) return;
  const int tm = logical % tiles_m, tn = (logical / tiles_m) % tiles_n;
  const int bz = logical / (tiles_m * tiles_n);
  const int m0 = tm * CM, n0 = tn * CN;

  const char* A = reinterpret_cast<const char*>(g.A + (int64_t)bz * g.sA);
  const char* B = reinterpret_cast<const char*>(g.B + (int64_t)bz * g.sB);

  // Per slab each thread moves eight 16-byte chunks of A and eight of B:
  // rows ld_row + 32 i, chunk ld_c.  Loads are unconditional from clamped rows:
  // a row past the end repeats the last one, and what it produces lands in
  // output rows that are never stored or in columns N..ldc-1 of T, which no
  // consumer reads.  Only a k chunk past K must contribute nothing; it is
  // zeroed on its way to LDS, in the one slab that can contain it.
  const int ld_row = tid >> 3, ld_c = tid & 7;
  uint32_t offa[8], offb[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const int row = ld_row + 32 * i;
    offa[i] = ((uint32_t)min(m0 + row, g.M - 1) * (uint32_t)g.lda + ld_c * 8) * 2u;
    offb[i] = ((uint32_t)min(n0 + row, g.N - 1) * (uint32_t)g.ldb + ld_c * 8) * 2u;
  }
  // Two register sets: while slab kt is multiplied out of LDS, slab kt + 1
  // waits in one set for its turn in the idle LDS buffer and slab kt + 2 is in
  // flight to the other, so a load has a whole slab of MFMA work (about 1 us)
  // plus its own issue time to come back before anything waits for it.
  u32x4 ra[2][8], rb[2][8];
  bool k_ok[2] = {true, true};
  uint32_t kb[2] = {0, 0};
  auto gload_begin = [&](int set, int kt) {  // kt may run past the last slab: such a slab is all zeros
    const int k0 = kt * CK;
    k_ok[set] = k0 + ld_c * 8 < g.K;
    kb[set] = k_ok[set] ? (uint32_t)k0 * 2u : 0u;
  };
  // chunk q of a slab: q < 8 is row group q of A, q >= 8 row group q - 8 of B
  auto gload = [&](int set, int q0, int q1) {
#pragma unroll
    for (int q = q0; q < q1; ++q) {
      if (q < 8) ra[set][q] = *reinterpret_cast<const u32x4*>(A + (offa[q] + kb[set]));
      else rb[set][q - 8] = *reinterpret_cast<const u32x4*>(B + (offb[q - 8] + kb[set]));
    }
  };
  auto sstore = [&](int set, int buf) {
    bf16_t* sA = smem + buf * STAGE;
    bf16_t* sB = sA + CM * LDT;
    if (!k_ok[set]) {
      const u32x4 z = {0, 0, 0, 0};
#pragma unroll
      for (int i = 0; i < 8; ++i) ra[set][i] = rb[set][i] = z;
    }
#pragma unroll
    for (int i = 0; i < 8; ++i) *reinterpret_cast<u32x4*>(sA + (ld_row + 32 * i) * LDT + ld_c * 8) = ra[set][i];
#pragma unroll
    for (int i = 0; i < 8; ++i) *reinterpret_cast<u32x4*>(sB + (ld_row + 32 * i) * LDT + ld_c * 8) = rb[set][i];
  };

  // acc[jt][it] = (T^T) tile: rows j = wn + 32 jt + .., columns i = wm + 32 it + ..
  f32x16 acc[4][4];
#pragma unroll
  for (int jt = 0; jt < 4; ++jt)
#pragma unroll
    for (int it = 0; it < 4; ++it)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[jt][it][r] = 0.f;

  const int nk = (g.K + CK - 1) / CK;
  gload_begin(0, 0);
  gload(0, 0, 16);
  gload_begin(1, 1);
  gload(1, 0, 16);
  sstore(0, 0);
  lds_barrier();

  // One slab = four k-steps of 16 MFMAs.  A lone wave per SIMD has nobody to
  // cover for it, and a burst of 16 global loads or 16 LDS stores blocks the
  // wave's instruction stream for longer than a k-step of MFMAs takes (the
  // memory pipeline accepts a CU's 64 KB slab no faster than 64 B per cycle).
  // So everything is spread over the MFMA stream, and the scheduler is told the
  // interleave explicitly:
  //   k-steps 0-2: a third of slab kt + 2's loads + the next step's fragments
  //                between the MFMAs
  //   k-step 3: slab kt + 1 goes from its registers to the idle LDS buffer
  // No load or store is decided by a branch: slabs past the end are fetched
  // from offset 0 and stored as zeros.
  auto stage = [&](int kt, auto par_c) {
    constexpr int par = decltype(par_c)::value;  // kt & 1: LDS buffer read, register set refilled
    const bf16_t* sA = smem + par * STAGE;
    const bf16_t* sB = sA + CM * LDT;
    bf16x8 fa[2][4], fb[2][4];
    auto frags = [&](int set, int ks) {
#pragma unroll
      for (int it = 0; it < 4; ++it) fa[set][it] = lds_frag(sA, LDT, wm + 32 * it, ks * 16, lane);
#pragma unroll
      for (int jt = 0; jt < 4; ++jt) fb[set][jt] = lds_frag(sB, LDT, wn + 32 * jt, ks * 16, lane);
    };
    auto mfmas = [&](int set) {
#pragma unroll
      for (int jt = 0; jt < 4; ++jt)
#pragma unroll
        for (int it = 0; it < 4; ++it) acc[jt][it] = mfma32(fb[set][jt], fa[set][it], acc[jt][it]);
    };
    frags(0, 0);
    gload_begin(par, kt + 2);
    __builtin_amdgcn_sched_barrier(0);
    // k-step 0
    gload(par, 0, 6);
    frags(1, 1);
    mfmas(0);
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      __builtin_amdgcn_sched_group_barrier(0x008, 2, 0);             // two MFMAs
      if (i < 6) __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);  // one global load
      __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);             // one LDS read
    }
    __builtin_amdgcn_sched_barrier(0);
    // k-step 1
    gload(par, 6, 11);
    frags(0, 2);
    mfmas(1);
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      __builtin_amdgcn_sched_group_barrier(0x008, 2, 0);
      if (i < 5) __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
    }
    __builtin_amdgcn_sched_barrier(0);
    // k-step 2
    gload(par, 11, 16);
    frags(1, 3);
    mfmas(0);
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      __builtin_amdgcn_sched_group_barrier(0x008, 2, 0);
      if (i < 5) __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
    }
    __builtin_amdgcn_sched_barrier(0);
    // k-step 3
    mfmas(1);
    sstore(par ^ 1, par ^ 1);
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);  // one MFMA
      __builtin_amdgcn_sched_group_barrier(0x200, 1, 0);  // one LDS store
    }
    lds_barrier();
  };
  // Two stages per trip (the register sets and LDS buffers are addressed
  // statically); an odd slab count runs one extra stage on an all-zero slab.
  for (int kt = 0; kt < nk; kt += 2) {
    stage(kt, std::integral_constant<int, 0>{});
    stage(kt + 1, std::integral_constant<int, 1>{});
  }

  // ------------------------------------------------------------- epilogue
  // Every wave has passed the last barrier, so the slabs are dead.  A wave
  // stages its own 128x128 quadrant (rows i, columns j) and reads it back
  // itself (a wave's LDS operations execute in order): no further barrier.
  // Lane (l31, hh), register quad q of tile (jt, it): row i = 32 it + l31,
  // columns j = 32 jt + 8 q + 4 hh + 0..3.
  bf16_t* sE = smem + wave * (128 * LDE);
#pragma unroll
  for (int jt = 0; jt < 4; ++jt)
#pragma unroll
    for (int it = 0; it < 4; ++it)
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        u32x2 v;
        v.x = pack2bf(acc[jt][it][4 * q], acc[jt][it][4 * q + 1]);
        v.y = pack2bf(acc[jt][it][4 * q + 2], acc[jt][it][4 * q + 3]);
        *reinterpret_cast<u32x2*>(sE + (32 * it + l31) * LDE + 32 * jt + 8 * q + 4 * hh) = v;
      }
  bf16_t* C = reinterpret_cast<bf16_t*>(g.C) + (int64_t)bz * g.sC;
  const int c16 = lane & 15, rsub = lane >> 4;  // 16 chunks of 8 columns per row, 4 rows per instruction
  const int col = n0 + wn + c16 * 8;
#pragma unroll
  for (int s = 0; s < 32; ++s) {
    const int r = 4 * s + rsub;
    const int row = m0 + wm + r;
    const u32x4 v = *reinterpret_cast<const u32x4*>(sE + r * LDE + c16 * 8);
    if (row < g.M && col < g.ldc) *reinterpret_cast<u32x4*>(C + (int64_t)row * g.ldc + col) = v;
  }
}

bool al16(const void* p) { return ((uintptr_t)p & 15) == 0; }

}  // namespace

// Plain bf16 batched NT product with the large tile; false if the operands do
// not meet its layout assumptions (the caller then takes the general GEMM).
bool contract_supported(const GemmArgs& g) {
  return g.epi == EPI_PLAIN && !g.out_f32 && !g.bias && !g.act_sigmoid && g.alpha == 1.f && g.M > 0 && g.N > 0 &&
         g.K > 0 && g.batch > 0 && (g.lda & 7) == 0 && (g.ldb & 7) == 0 && (g.ldc & 7) == 0 && (g.K & 7) == 0 &&
         g.K <= g.lda && g.K <= g.ldb && g.ldc >= ((g.N + 7) & ~7) && (g.sA & 7) == 0 && (g.sB & 7) == 0 &&
         (g.sC & 7) == 0 && al16(g.A) && al16(g.B) && al16(g.C) &&
         (int64_t)g.M * g.lda < (1ll << 30) && (int64_t)g.N * g.ldb < (1ll << 30);
}

int launch_contract(const GemmArgs& g, hipStream_t stream) {
  if (!g.A || !g.B || !g.C || !contract_supported(g)) return AF3_ERR_BAD_ARG;
  const int64_t total = (int64_t)((g.M + CM - 1) / CM) * ((g.N + CN - 1) / CN) * g.batch;
  const int64_t blocks = (total + 7) / 8 * 8;
  if (blocks > 0x7fffffff) return AF3_ERR_BAD_ARG;
  hipLaunchKernelGGL(contract_kernel, dim3((unsigned)blocks), dim3(256), 0, stream, g);
  return hipGetLastError() == hipSuccess ? AF3_OK : AF3_ERR_LAUNCH;
}
