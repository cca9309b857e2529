// Tile loop shared by the int8 and the FP8 GEMM: 1-byte operands, both K-contiguous in HBM ("NT"
// form: A is [M,K] row-major, Bt is [N,K] row-major), 32x32 MFMA tiles, LDS double buffer.
//
// A workgroup owns a BM x BN tile of Y and walks K in slabs of BK bytes.  A slab of A and of Bt is
// staged in LDS as rows of BK bytes cut into 16-byte chunks; chunk c of row r is stored at chunk
// position c ^ ((r / rows_per_256B) % chunks_per_row), so that the 16 lanes served together by one
// ds_read_b128 (16 consecutive rows, same logical chunk) fall into 16 different 16-byte bank groups.
// The MFMA is issued with the Bt rows as its first operand and the A rows as its second, so that a
// lane ends up holding 4 consecutive output columns n of one output row m and can store them as one
// vector.  Which K bytes a lane feeds to the MFMA only has to be the same for both operands, because
// the dot product does not depend on the order of its terms (exactly for int8, to rounding for FP8).
#pragma once
#include "common.hpp"

namespace sofie_hip {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v8i __attribute__((ext_vector_type(8)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef float v16f __attribute__((ext_vector_type(16)));

// int8: v_mfma_i32_32x32x32_i8, 16 bytes of K per lane and step.
struct MfmaI8 {
   typedef v16i acc_t;
   typedef int elem_t;
   static constexpr int KSTEP = 32;  // K bytes per MFMA
   static constexpr int CHUNKS = 1;  // 16-byte chunks per lane and operand
   struct frag_t {
      v4i c[1];
   };
   static __device__ __forceinline__ acc_t mma(const frag_t &a, const frag_t &b, acc_t c)
   {
      return __builtin_amdgcn_mfma_i32_32x32x32_i8(a.c[0], b.c[0], c, 0, 0, 0);
   }
};

// FP8 e4m3fn: v_mfma_f32_32x32x64_f8f6f4 (format code 0 = e4m3 for both operands, no block scaling),
// 32 bytes of K per lane and step.
struct MfmaF8 {
   typedef v16f acc_t;
   typedef float elem_t;
   static constexpr int KSTEP = 64;
   static constexpr int CHUNKS = 2;
   struct frag_t {
      v4i c[2];
   };
   static __device__ __forceinline__ acc_t mma(const frag_t &a, const frag_t &b, acc_t c)
   {
      v8i va = {a.c[0][0], a.c[0][1], a.c[0][2], a.c[0][3], a.c[1][0], a.c[1][1], a.c[1][2], a.c[1][3]};
      v8i vb = {b.c[0][0], b.c[0][1], b.c[0][2], b.c[0][3], b.c[1][0], b.c[1][1], b.c[1][2], b.c[1][3]};
      return __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(va, vb, c, 0, 0, 0, 0, 0, 0);
   }
};

// Maps the hardware workgroup id to an output tile.  Workgroups are dealt round-robin to the 8 XCDs,
// each with its own L2: ids that land on one XCD are made consecutive, and consecutive ids walk the
// tile grid in bands of GROUP_M tile rows, so the tiles resident on one XCD at a time share A and Bt
// slabs through that XCD's L2.
__device__ __forceinline__ void tile_of_block(int bid, int nwg, int tiles_m, int tiles_n, int &tm, int &tn)
{
   constexpr int NXCD = 8;
   constexpr int GROUP_M = 4;
   const int per = nwg / NXCD, rem = nwg % NXCD;
   const int xcd = bid % NXCD, local = bid / NXCD;
   const int id = (xcd < rem ? xcd * (per + 1) : rem * (per + 1) + (xcd - rem) * per) + local;
   const int width = GROUP_M * tiles_n;
   const int group = id / width;
   const int first_m = group * GROUP_M;
   const int gsz = (tiles_m - first_m) < GROUP_M ? (tiles_m - first_m) : GROUP_M;
   tm = first_m + (id % width) % gsz;
   tn = (id % width) / gsz;
}

template <int BK>
__device__ __forceinline__ int lds_chunk_offset(int r, int c)
{
   constexpr int CPR = BK / 16;                          // 16-byte chunks per row
   constexpr int RPB = (256 / BK) > 0 ? (256 / BK) : 1;  // rows per 256 bytes of LDS
   return r * BK + (((c ^ ((r / RPB) % CPR))) << 4);
}

// Loads one 16-byte chunk (bytes k..k+15 of the row at `row_ptr`); bytes at k >= K read as 0.
template <bool ALIGNED>
__device__ __forceinline__ v4i load_chunk(const int8_t *row_ptr, int k, int K)
{
   const int8_t *p = row_ptr + k;
   if (ALIGNED) {
      if (k < K)
         return *(const v4i *)p;
      return v4i{0, 0, 0, 0};
   } else {
      union {
         v4i v;
         int8_t b[16];
      } u;
      u.v = v4i{0, 0, 0, 0};
#pragma unroll
      for (int i = 0; i < 16; ++i)
         if (k + i < K)
            u.b[i] = p[i];
      return u.v;
   }
}

// Plain row-major operand: row r starts at base + r*ld.
struct RowMajorRows {
   const int8_t *base;
   int ld;
   __device__ __forceinline__ const int8_t *row(int r) const { return base + (size_t)r * (size_t)ld; }
};

// EPI must provide: void store4(int m, int n, elem_t a0, elem_t a1, elem_t a2, elem_t a3) const
// for the 4 consecutive columns n..n+3 of row m (n < N guaranteed, n+3 may exceed N-1).
template <class MMA, int BM, int BN, int BK, int WAVES_M, int WAVES_N, bool ALIGNED, class EPI>
__device__ __forceinline__ void mfma8_gemm_tile(const RowMajorRows A, const RowMajorRows Bt, int M, int N, int K,
                                                const EPI &ep, int tm, int tn, int8_t *smem)
{
   constexpr int NTHREADS = WAVES_M * WAVES_N * 64;
   constexpr int CPR = BK / 16;
   constexpr int TM = BM / WAVES_M, TN = BN / WAVES_N; // wave tile
   constexpr int MT = TM / 32, NT = TN / 32;           // 32x32 MFMA tiles per wave
   constexpr int A_LD = BM * CPR / NTHREADS, B_LD = BN * CPR / NTHREADS;
   static_assert(BM * CPR % NTHREADS == 0 && BN * CPR % NTHREADS == 0, "tile must divide over the threads");
   static_assert(TM % 32 == 0 && TN % 32 == 0, "wave tile must be a multiple of 32x32");
   static_assert(BK % MMA::KSTEP == 0, "BK must be a multiple of the MFMA K");
   typedef typename MMA::acc_t acc_t;
   typedef typename MMA::frag_t frag_t;

   int8_t *sA = smem;               // [2][BM*BK]
   int8_t *sB = smem + 2 * BM * BK; // [2][BN*BK]

   const int m0 = tm * BM, n0 = tn * BN;
   const int t = threadIdx.x;
   const int lane = t & 63, wave = t >> 6;
   const int wm = wave / WAVES_N, wn = wave % WAVES_N;

   acc_t acc[MT][NT];
#pragma unroll
   for (int i = 0; i < MT; ++i)
#pragma unroll
      for (int j = 0; j < NT; ++j)
#pragma unroll
         for (int v = 0; v < 16; ++v)
            acc[i][j][v] = 0;

   // global -> register staging: chunk id = t + i*NTHREADS -> (row, chunk)
   v4i ra[A_LD], rb[B_LD];
   const int8_t *a_row[A_LD], *b_row[B_LD];
#pragma unroll
   for (int i = 0; i < A_LD; ++i) {
      int gr = m0 + (t + i * NTHREADS) / CPR;
      a_row[i] = A.row(gr < M ? gr : M - 1);
   }
#pragma unroll
   for (int i = 0; i < B_LD; ++i) {
      int gr = n0 + (t + i * NTHREADS) / CPR;
      b_row[i] = Bt.row(gr < N ? gr : N - 1);
   }
   auto load_global = [&](int k0) {
#pragma unroll
      for (int i = 0; i < A_LD; ++i)
         ra[i] = load_chunk<ALIGNED>(a_row[i], k0 + ((t + i * NTHREADS) % CPR) * 16, K);
#pragma unroll
      for (int i = 0; i < B_LD; ++i)
         rb[i] = load_chunk<ALIGNED>(b_row[i], k0 + ((t + i * NTHREADS) % CPR) * 16, K);
   };
   auto store_lds = [&](int stage) {
#pragma unroll
      for (int i = 0; i < A_LD; ++i) {
         int id = t + i * NTHREADS;
         *(v4i *)(sA + stage * BM * BK + lds_chunk_offset<BK>(id / CPR, id % CPR)) = ra[i];
      }
#pragma unroll
      for (int i = 0; i < B_LD; ++i) {
         int id = t + i * NTHREADS;
         *(v4i *)(sB + stage * BN * BK + lds_chunk_offset<BK>(id / CPR, id % CPR)) = rb[i];
      }
   };

   const int KT = (K + BK - 1) / BK;
   load_global(0);
   store_lds(0);
   __syncthreads();

   const int lr = lane & 31, lk = lane >> 5;
   for (int kt = 0; kt < KT; ++kt) {
      const int cur = kt & 1;
      if (kt + 1 < KT)
         load_global((kt + 1) * BK);
      const int8_t *cA = sA + cur * BM * BK;
      const int8_t *cB = sB + cur * BN * BK;
#pragma unroll
      for (int ks = 0; ks < BK / MMA::KSTEP; ++ks) {
         frag_t fa[MT], fb[NT];
#pragma unroll
         for (int j = 0; j < NT; ++j)
#pragma unroll
            for (int c = 0; c < MMA::CHUNKS; ++c)
               fb[j].c[c] = *(const v4i *)(cB + lds_chunk_offset<BK>(wn * TN + j * 32 + lr, (ks * 2 + lk) * MMA::CHUNKS + c));
#pragma unroll
         for (int i = 0; i < MT; ++i)
#pragma unroll
            for (int c = 0; c < MMA::CHUNKS; ++c)
               fa[i].c[c] = *(const v4i *)(cA + lds_chunk_offset<BK>(wm * TM + i * 32 + lr, (ks * 2 + lk) * MMA::CHUNKS + c));
#pragma unroll
         for (int i = 0; i < MT; ++i)
#pragma unroll
            for (int j = 0; j < NT; ++j)
               acc[i][j] = MMA::mma(fb[j], fa[i], acc[i][j]);
      }
      if (kt + 1 < KT)
         store_lds(cur ^ 1);
      __syncthreads();
   }

   // epilogue: lane holds row m = .. + lane%32 and, per group g of 4 registers, columns
   // n = .. + 8*g + 4*(lane/32) + {0,1,2,3}
#pragma unroll
   for (int i = 0; i < MT; ++i) {
      const int m = m0 + wm * TM + i * 32 + lr;
      if (m >= M)
         continue;
#pragma unroll
      for (int j = 0; j < NT; ++j) {
#pragma unroll
         for (int g = 0; g < 4; ++g) {
            const int n = n0 + wn * TN + j * 32 + g * 8 + lk * 4;
            if (n < N)
               ep.store4(m, n, acc[i][j][4 * g + 0], acc[i][j][4 * g + 1], acc[i][j][4 * g + 2], acc[i][j][4 * g + 3]);
         }
      }
   }
}

template <class MMA, int BM, int BN, int BK, int WAVES_M, int WAVES_N, bool ALIGNED, class EPI>
__global__ __launch_bounds__(WAVES_M *WAVES_N * 64) void mfma8_gemm_kernel(RowMajorRows A, RowMajorRows Bt, int M, int N,
                                                                            int K, EPI ep, int tiles_m, int tiles_n)
{
   extern __shared__ __attribute__((aligned(16))) int8_t smem[];
   int tm, tn;
   tile_of_block(blockIdx.x, gridDim.x, tiles_m, tiles_n, tm, tn);
   mfma8_gemm_tile<MMA, BM, BN, BK, WAVES_M, WAVES_N, ALIGNED, EPI>(A, Bt, M, N, K, ep, tm, tn, smem);
}

template <class MMA, int BM, int BN, int BK, int WAVES_M, int WAVES_N, class EPI>
static int launch_mfma8(hipStream_t stream, const int8_t *A, const int8_t *Bt, int M, int N, int K, int lda, int ldb,
                        const EPI &ep, bool aligned)
{
   const int tiles_m = (M + BM - 1) / BM, tiles_n = (N + BN - 1) / BN;
   const long long nwg = (long long)tiles_m * tiles_n;
   if (nwg > 0x7fffffffLL)
      return fail(SOFIE_HIP_ERR_INVALID, "gemm: too many tiles");
   constexpr size_t smem = 2 * (size_t)(BM + BN) * BK;
   constexpr int NTHREADS = WAVES_M * WAVES_N * 64;
   RowMajorRows a{A, lda}, b{Bt, ldb};
   if (aligned) {
      auto kern = mfma8_gemm_kernel<MMA, BM, BN, BK, WAVES_M, WAVES_N, true, EPI>;
      SOFIE_HIP_CHECK(hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem));
      hipLaunchKernelGGL(kern, dim3((unsigned)nwg), dim3(NTHREADS), smem, stream, a, b, M, N, K, ep, tiles_m, tiles_n);
   } else {
      auto kern = mfma8_gemm_kernel<MMA, BM, BN, BK, WAVES_M, WAVES_N, false, EPI>;
      SOFIE_HIP_CHECK(hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem));
      hipLaunchKernelGGL(kern, dim3((unsigned)nwg), dim3(NTHREADS), smem, stream, a, b, M, N, K, ep, tiles_m, tiles_n);
   }
   return launch_status("mfma8_gemm_kernel");
}

// Picks the tile: the largest one that still gives every one of the 256 CUs a workgroup.
template <class MMA, class EPI>
static int launch_mfma8_auto(hipStream_t stream, const int8_t *A, const int8_t *Bt, int M, int N, int K, int lda, int ldb,
                             const EPI &ep, int force_tile)
{
   const bool aligned = (K % 16 == 0) && (lda % 16 == 0) && (ldb % 16 == 0) && (((uintptr_t)A & 15) == 0) &&
                        (((uintptr_t)Bt & 15) == 0);
   auto tiles = [&](int bm, int bn) { return (long long)((M + bm - 1) / bm) * ((N + bn - 1) / bn); };
   int tile = force_tile;
   if (tile == 0) {
      if (tiles(256, 256) >= 256)
         tile = 256;
      else if (tiles(128, 128) >= 192)
         tile = 128;
      else
         tile = 64;
   }
   switch (tile) {
   case 256: return launch_mfma8<MMA, 256, 256, 64, 2, 2, EPI>(stream, A, Bt, M, N, K, lda, ldb, ep, aligned);
   case 128: return launch_mfma8<MMA, 128, 128, 64, 2, 2, EPI>(stream, A, Bt, M, N, K, lda, ldb, ep, aligned);
   case 64: return launch_mfma8<MMA, 64, 64, 64, 2, 2, EPI>(stream, A, Bt, M, N, K, lda, ldb, ep, aligned);
   default: return fail(SOFIE_HIP_ERR_INVALID, "gemm: unknown tile %d", tile);
   }
}

int transpose_i8(hipStream_t stream, int8_t *dst, const int8_t *src, int rows, int cols, int ld_src, int ld_dst);

} // namespace sofie_hip
