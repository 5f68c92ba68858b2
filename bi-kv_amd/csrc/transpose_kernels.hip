// Fused page move + layout change between Bi-KV's two KV layouts, which the reference never converts:
//
//   token-major (storage / transfer): one token = [head_dim D][kv_heads H][layers L][2] elements,
//     Bi-KV/Model/qwen2.py:519-522 (token_shape), pools (tokens,)+token_shape at
//     Bi-KV/DistributedStorage/kvcache.py:38-43 and Bi-KV/Worker/Worker.py:57-62;
//   per-layer paged NHD (compute): L tensors addressed (block, kv, token, head, d) with D contiguous,
//     [blocks*block, 2, H, D] at Bi-KV/Worker/Worker.py:74-78 and [blocks, 2, block, H, D] at
//     Bi-KV/Model/qwen2.py:532-536 (the layout flashinfer's paged prefill reads).
//
// Per token this is the transpose of a [D][C] matrix (C = H*L*2, column c = (h*L + l)*2 + k) into
// C rows of D contiguous elements, each row landing in its own layer tensor. A workgroup stages a
// [D][Cc] block of one token in LDS: the token-major side is read or written as whole 16-byte
// vectors along c, the compute side as 16-byte vectors along d assembled from (or split into)
// single elements in LDS. Four neighbouring lanes cover 64 contiguous bytes of one compute row; the
// LDS pitch is padded by 4 bytes so that those strided element accesses fall on distinct banks.
#include "pagecopy_kernels.h"

namespace bikv {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
#define BIKV_GLOBAL __attribute__((address_space(1)))
#define BIKV_CONST __attribute__((address_space(4)))

template <class T>
__device__ __forceinline__ T tload(const T* p) {
  return *(const BIKV_CONST T*)(uint64_t)p;
}

template <int ES> struct ElemOf;
template <> struct ElemOf<1> { using T = uint8_t; };
template <> struct ElemOf<2> { using T = uint16_t; };
template <> struct ElemOf<4> { using T = uint32_t; };

// DIR 0: compute -> token-major (a Worker sending its KV to the cache)
// DIR 1: token-major -> compute (received KV landing in the paged pool)
template <int DIR, int ES>
__global__ __launch_bounds__(kBlock) void transpose_pages_kernel(const TransposeArgs a) {
  using E = typename ElemOf<ES>::T;
  constexpr int VE = 16 / ES;            // elements per 16-byte vector
  extern __shared__ uint32_t lds_words[];
  E* lds = reinterpret_cast<E*>(lds_words);
  uint64_t* row_addr = reinterpret_cast<uint64_t*>(lds_words + a.tile_words);  // Cc entries

  const uint32_t chunk = blockIdx.x % a.n_chunks;              // column chunk
  const uint32_t rest = blockIdx.x / a.n_chunks;
  const uint32_t dchunk = rest % a.n_dchunks;                  // slice of head_dim
  const uint32_t t = rest / a.n_dchunks;                       // token within the page
  const uint64_t i = (uint64_t)blockIdx.y + (uint64_t)blockIdx.z * gridDim.y;
  if (i >= (uint64_t)a.n_pages) return;
  const int64_t blk = tload(a.block_ids + i);
  const int64_t tmp = tload(a.tm_pages + i);
  const bool bad_blk = (uint64_t)blk >= (uint64_t)a.n_blocks;
  const bool bad_tm = (uint64_t)tmp >= (uint64_t)a.n_tm_pages;
  if (bad_blk || bad_tm) {
    if (threadIdx.x == 0 && blockIdx.x == 0) {
      if (bad_blk) *reinterpret_cast<volatile uint32_t*>(a.status + ST_SLOT_PAGE) = 1u;
      if (bad_tm) *reinterpret_cast<volatile uint32_t*>(a.status + (DIR == 0 ? ST_SLOT_DST : ST_SLOT_SRC)) = 1u;
    }
    return;
  }
  // the tile is rows [d0, d0+D) x columns [c0, c0+Cc) of the token's [head_dim][C] matrix
  const int D = a.chunk_rows, C = a.n_cols, Cc = a.chunk_cols, PC = a.pitch;
  const int c0 = (int)chunk * Cc;
  const int d0 = (int)dchunk * D;
  // compute-side address of every row (column c of the token) handled by this workgroup
  for (int c = threadIdx.x; c < Cc; c += kBlock) {
    const int cg = c0 + c;
    const int k = cg & 1;
    const int hl = cg >> 1;
    const int h = hl / a.n_layers;
    const int l = hl - h * a.n_layers;
    const int64_t off = blk * a.block_stride + (int64_t)k * a.kv_stride + (int64_t)t * a.token_stride +
                        (int64_t)h * a.head_dim + d0;
    row_addr[c] = (uint64_t)a.layer_base[l] + (uint64_t)off * ES;
  }
  // token-major side: row d of the tile starts at tm_tok + d*C
  const uint64_t tm_tok = (uint64_t)a.tm_base +
                          (((uint64_t)(tmp * a.block_tokens + t) * a.head_dim + d0) * C + c0) * ES;
  const int vec_per_row = Cc / VE;       // 16-byte vectors along c per matrix row
  const int n_tm_vec = D * vec_per_row;
  const int dgs = D / VE;                // 16-byte vectors along d per compute row
  const int n_cp_vec = Cc * ((dgs + 3) & ~3);   // lanes walk (4 vectors of a row, row, group of 4)

  // Global loads are issued U at a time before any of them is consumed, so that a lane keeps U
  // 16-byte requests in flight instead of one.
  constexpr int U = 8;
  if (DIR == 1) {
    for (int base = 0; base < n_tm_vec; base += kBlock * U) {
      u32x4 x[U];
#pragma unroll
      for (int u = 0; u < U; ++u) {
        // out-of-range lanes re-read the last vector instead of branching around the load: a
        // branch here makes the compiler wait for each load before issuing the next
        int v = base + u * kBlock + threadIdx.x;
        v = v < n_tm_vec ? v : n_tm_vec - 1;
        const int d = v / vec_per_row, cv = v - d * vec_per_row;
        x[u] = __builtin_nontemporal_load(
            (const BIKV_GLOBAL u32x4*)(tm_tok + ((uint64_t)d * C + cv * VE) * ES));
      }
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int v = base + u * kBlock + threadIdx.x;
        if (v < n_tm_vec) {
          const int d = v / vec_per_row, cv = v - d * vec_per_row;
          uint32_t* w = lds_words + (d * PC + cv * VE) * ES / 4;   // 4-byte aligned by construction
          w[0] = x[u].x; w[1] = x[u].y; w[2] = x[u].z; w[3] = x[u].w;
        }
      }
    }
  }
  __syncthreads();   // row_addr (and, for DIR 1, the tile) are in LDS
  if (DIR == 0) {
    for (int base = 0; base < n_cp_vec; base += kBlock * U) {
      u32x4 x[U];
#pragma unroll
      for (int u = 0; u < U; ++u) {
        int o = base + u * kBlock + threadIdx.x;
        o = o < n_cp_vec ? o : n_cp_vec - 1;
        const int dgl = o & 3, c = (o >> 2) % Cc;
        int dg = ((o >> 2) / Cc) * 4 + dgl;
        dg = dg < dgs ? dg : dgs - 1;              // branch-free, as above
        x[u] = *(const BIKV_GLOBAL u32x4*)(row_addr[c] + (uint64_t)dg * 16);
      }
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int o = base + u * kBlock + threadIdx.x;
        const int dgl = o & 3, c = (o >> 2) % Cc, dg = ((o >> 2) / Cc) * 4 + dgl;
        if (o < n_cp_vec && dg < dgs) {
          E e[VE];
          __builtin_memcpy(e, &x[u], 16);
#pragma unroll
          for (int j = 0; j < VE; ++j) lds[(dg * VE + j) * PC + c] = e[j];
        }
      }
    }
    __syncthreads();
    for (int v = threadIdx.x; v < n_tm_vec; v += kBlock) {
      const int d = v / vec_per_row, cv = v - d * vec_per_row;
      const uint32_t* w = lds_words + (d * PC + cv * VE) * ES / 4;
      u32x4 x = {w[0], w[1], w[2], w[3]};
      __builtin_nontemporal_store(x, (BIKV_GLOBAL u32x4*)(tm_tok + ((uint64_t)d * C + cv * VE) * ES));
    }
  } else {
    for (int o = threadIdx.x; o < n_cp_vec; o += kBlock) {
      const int dgl = o & 3, c = (o >> 2) % Cc, dg = ((o >> 2) / Cc) * 4 + dgl;
      if (dg >= dgs) continue;
      E e[VE];
#pragma unroll
      for (int j = 0; j < VE; ++j) e[j] = lds[(dg * VE + j) * PC + c];
      u32x4 x;
      __builtin_memcpy(&x, e, 16);
      *(BIKV_GLOBAL u32x4*)(row_addr[c] + (uint64_t)dg * 16) = x;
    }
  }
}

template <int DIR>
static hipError_t launch_transpose_dir(const TransposeArgs& a, dim3 grid, size_t lds, hipStream_t s) {
  switch (a.elem_bytes) {
    case 1: hipLaunchKernelGGL((transpose_pages_kernel<DIR, 1>), grid, dim3(kBlock), lds, s, a); break;
    case 2: hipLaunchKernelGGL((transpose_pages_kernel<DIR, 2>), grid, dim3(kBlock), lds, s, a); break;
    case 4: hipLaunchKernelGGL((transpose_pages_kernel<DIR, 4>), grid, dim3(kBlock), lds, s, a); break;
    default: return hipErrorInvalidValue;
  }
  return hipGetLastError();
}

// Chooses the column chunk (a divisor of C that is a whole number of 16-byte vectors and keeps the
// LDS tile near 32 KiB) and launches. Returns hipErrorInvalidValue for shapes the kernel does not
// take (the caller has already validated them; this is a second line of defence).
hipError_t launch_transpose_pages(int dir, TransposeArgs& a, hipStream_t stream) {
  if (a.n_pages <= 0) return hipSuccess;
  const int ES = a.elem_bytes;
  if (ES != 1 && ES != 2 && ES != 4) return hipErrorInvalidValue;
  const int VE = 16 / ES;
  const int C = a.n_cols, D = a.head_dim;
  if (C <= 0 || D <= 0 || C % VE != 0 || D % VE != 0 || (C & 1)) return hipErrorInvalidValue;
  // Tile = [Dd rows of head_dim] x [Cc columns]. Measured on MI355X (Qwen2-1.5B/7B and Llama-3-8B
  // token shapes): throughput follows the width of the contiguous pieces on BOTH sides — whole
  // compute rows (Dd = head_dim) and the widest column chunk that fits LDS. Cutting head_dim to make
  // room for wider chunks lost 10-25 %, a 16 KiB tile lost 30-60 %, so the default is the full
  // head_dim with a ~60 KiB tile (two workgroups per CU).
  const int budget_elems = (tuning().transpose_lds_kib * 1024) / ES;
  int dsplit = tuning().transpose_dsplit;
  if (dsplit <= 0) dsplit = 1;
  if (D % (dsplit * VE) != 0) return hipErrorInvalidValue;
  const int Dd = D / dsplit;
  int best = VE;
  for (int cc = VE; cc <= C; cc += VE) {
    if (C % cc != 0) continue;
    const int pitch = cc + 4 / ES;
    if ((int64_t)Dd * pitch <= budget_elems) best = cc;
  }
  a.chunk_rows = Dd;
  a.n_dchunks = (uint32_t)dsplit;
  a.chunk_cols = best;
  a.pitch = best + 4 / ES;                      // +4 bytes: strided element accesses hit distinct banks
  a.n_chunks = (uint32_t)(C / best);
  a.tile_words = (uint32_t)(((int64_t)Dd * a.pitch * ES + 7) / 8 * 2);   // keeps row_addr 8-byte aligned
  const size_t lds = (size_t)a.tile_words * 4 + (size_t)best * 8;
  if (lds > 64 * 1024) return hipErrorInvalidValue;
  const int64_t gx = (int64_t)a.n_chunks * a.n_dchunks * a.block_tokens;
  const int64_t gy = a.n_pages < 32768 ? a.n_pages : 32768;
  const int64_t gz = (a.n_pages + gy - 1) / gy;
  if (gx >= (int64_t(1) << 24) || gz > 65535) return hipErrorInvalidValue;
  const dim3 grid((uint32_t)gx, (uint32_t)gy, (uint32_t)gz);
  return dir == 0 ? launch_transpose_dir<0>(a, grid, lds, stream)
                  : launch_transpose_dir<1>(a, grid, lds, stream);
}

}  // namespace bikv
