// Shared definitions of the MLA attention kernels (gfx950).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <math.h>

#include "../../include/mla_attn.h"

namespace mla {


typedef __attribute__((ext_vector_type(4))) unsigned int u32x4;
typedef __attribute__((ext_vector_type(2))) unsigned int u32x2;
typedef __attribute__((ext_vector_type(4))) short        s16x4;
typedef __attribute__((ext_vector_type(16))) float       f32x16;
typedef __attribute__((ext_vector_type(4))) float        f32x4;
typedef __attribute__((ext_vector_type(8))) __bf16       bf16x8;
typedef __attribute__((ext_vector_type(8))) _Float16     f16x8;

#define LDS_PTR(T) T __attribute__((address_space(3))) *

constexpr int DK          = 576;
constexpr int KSTEPS      = DK / 16;  // 36 MFMA k-steps over the 576-d contraction
constexpr int TILE_TOK    = 32;       // tokens per LDS tile (= MFMA M of S^T)
constexpr int ROW_BYTES   = DK * 2;   // one latent row in LDS (bf16 / f16)
constexpr int PITCH       = ROW_BYTES + 16;  // padded row pitch: 292 dwords, conflict-free for the b128 K reads
constexpr int TILE_BYTES  = TILE_TOK * PITCH;
constexpr int Q8_ROW      = 612;      // 18 blocks of (fp16 d, 32 x int8)
constexpr int Q8_TILE_RAW = TILE_TOK * Q8_ROW;  // 19584 = 1224 x 16
constexpr int NTHREADS    = 256;
constexpr float LOG2E     = 1.4426950408889634f;

enum { SRC_BF16 = 0, SRC_F16 = 1, SRC_Q8 = 2, SRC_BF16_CVT = 3,     // SRC_BF16_CVT: decode kernel only (bf16 tiles converted to f16 inside LDS)
       SRC_BF16_CS = 4, SRC_F16_CS = 5,                             // decode kernel only: the column-split programs (gen_decode_cs_asm.py)
       SRC_BF16_KS = 6, SRC_F16_KS = 7,                             // and its k-split programs for at most 32 rows (gen_decode_cs_asm.py --ks)
       SRC_BF16_CSQ = 8, SRC_F16_CSQ = 9,                           // column-split programs behind a prologue that rounds Q itself (no pre-pack pass)
       SRC_BF16_CSB = 10, SRC_F16_CSB = 11,                         // column-split programs with mask, ALiBi slope and soft cap (gen_decode_cs_asm.py --mask --bias)
       SRC_BF16_KSB = 12, SRC_F16_KSB = 13,                         // k-split programs with mask, ALiBi slope and soft cap (gen_decode_cs_asm.py --ks --mask --bias)
       SRC_BF16_CSH = 14, SRC_F16_CSH = 15 };                       // column-split programs for 33 .. 64 rows: two of the four waves have rows (gen_decode_cs_asm.py --half)

struct KParams {
    const char *    q;
    int64_t         q_nb1, q_nb2, q_nb3;
    const char *    kv;
    int64_t         kv_nb1, kv_nb3;
    int64_t         n_kv;
    const char *    mask;
    int64_t         mask_nb1, mask_ne0;
    int64_t         mask_nb3;      // bytes from one sequence's mask rows to the next one's (0: all sequences share the rows)
    const int32_t * block_table;
    int64_t         bt_stride;
    const int32_t * seq_lens;
    float *         dst;
    int64_t         dst_stride;  // floats
    _Float16 *      part_o;      // split-K partials O_c / l_c as f16: [n_seq][n_splits][dv_total/8][n_rows][8], or, when
                                 // part_f32 is set (small problems: no second rounding), as f32 rows [n_seq][n_splits][n_rows][dv_total]
    int             part_f32;
    float *         part_ml;     // [n_seq][n_splits][n_rows][2]  (max in log2 units, sum)
    int             n_head, n_tok, n_rows;
    int             n_splits, split_tokens;
    int             dv_total, d_off;
    float           scale, softcap, max_bias, m0, m1;
    int             n_head_log2;
    int             c_log2_bits;   // bit pattern of scale * log2(e)
    void *          q_pack;        // decode kernel: Q in MFMA operand layout (workspace)
    int             n_pool_pages;  // block-table mode: pages in the pool
    int *           mask_ext;      // pipelined kernel with a mask: per block of 128 rows, 16 pairs (first, one past the last key that is not masked for all its rows) (workspace)
    int             rel_splits;    // the KV splits divide that key range (every split writes its (m, l), -inf when it has no key)
    int             balanced;      // pipelined kernel: 1 = ragged paged decode, workgroups take equal runs of the page list of all
                                   // sequences; 2 = masked launch, equal runs of the tile list of the row blocks' key ranges; 3 = the same with
                                   // every query token as an item (the token form of a launch issued in two forms, see `dual`)
    int             n_wg;          //   workgroups (grid = (n_wg, 1, 1)); partial slot of workgroup v's piece of item i = v + i
    int             n_units;       //   items: sequences (1) / row blocks (2) / query tokens (3)
    int             slot_rows;     // rows per partial slot: n_rows, or 128 with balanced == 2
    int             n_seq_sched;   // sequences of the launch (grids of the pre-pack passes)
    int *           wg_first;      //   [n_wg][8] first piece of every workgroup (balanced == 1; workspace, written by the pre-pass).  Masked launches
                                   //   (balanced >= 2) keep there, written by the kernel's first workgroup for the combine pass: [1] = the schedule is
                                   //   the aligned one, [8 ..] = workgroups before every item in that schedule
    int *           sched;         //   [n_units + 1] units before each item / in total (workspace; written by the pre-pass (1) or by the
                                   //   first workgroup of the kernel itself (2); the combine pass reads it)
    int             v_col0;        // pipelined kernel: V = columns v_col0 .. v_col0 + 511 of the rows (0, or 64 in the second pass of a
                                   // 576-wide V), and the 512 results go to columns v_col0 .. of the dst rows
    int             q_as_q8;       // the KV rows are the f16 expansion of a Q8_0 cache: Q is quantized the Q8_0 way
    int             bf16_direct;   // bf16 KV: the hi + lo program instead of the one that converts the tiles to f16 (MLA_FLAG_BF16_DIRECT)
    int             rows_contig;  // kv rows are packed (kv_nb1 == row bytes): whole tiles are one contiguous run
    int             mask_ext_in_pack;  // Q pre-pack launch: its last 16 mask_ext_sub layers of blocks scan the mask extents
    int             mask_ext_sub;      // 1, or the tokens of a row block that get a block each in that scan (a launch issued in two forms)
    int             q_in_kernel;   // pipelined kernel: the wave program rounds Q itself (no pre-pack pass, no operand image)
    // A masked launch of few heads that is issued in two forms, of which the device runs one (see mla_decode_dual_kernel):
    int             dual;          //   0: no; 1: these are the parameters of the row-block form (balanced == 2); 2: of the token form
                                   //   (balanced == 3: every query token a sequence of one token, its mask row that sequence's mask)
                                   //   mask_ext then holds 16 pairs per query token in both
    int *           form;          //   the form that ran (2 / 3), left by the kernel for the combine pass (workspace)
    const int *     seq_order;     // a paged decode batch of more than 256 sequences, a workgroup each: the sequences by falling length (workspace,
                                   //   written by the pre-pass; workgroups are dispatched in that order); nullptr: the order of the batch
    void *          tok_q_pack;    //   row-block form's parameters, pack launch: the token form's operand image, [token][wave][k-step][lane][16 B]
                                   //   (nullptr: its program rounds Q itself), and the rounding it wants (1: f16, 2: bf16 written as f16)
    int             tok_mode;
};

template <typename T, typename U> __device__ __forceinline__ T bitcast(U u) { return __builtin_bit_cast(T, u); }

template <bool F16> __device__ __forceinline__ f32x16 mfma32(u32x4 a, u32x4 b, f32x16 c) {
    if constexpr (F16) return __builtin_amdgcn_mfma_f32_32x32x16_f16(bitcast<f16x8>(a), bitcast<f16x8>(b), c, 0, 0, 0);
    else               return __builtin_amdgcn_mfma_f32_32x32x16_bf16(bitcast<bf16x8>(a), bitcast<bf16x8>(b), c, 0, 0, 0);
}

// f32 -> bf16 bits, round to nearest even, NaN quieted (ggml/src/ggml-impl.h:553-568)
__device__ __forceinline__ unsigned int f32_to_bf16_bits(float f) {
    unsigned int i = __float_as_uint(f);
    if ((i & 0x7fffffffu) > 0x7f800000u) return (i >> 16) | 64u;
    return (i + (0x7fffu + ((i >> 16) & 1u))) >> 16;
}
__device__ __forceinline__ unsigned int f32_to_f16_bits(float f) { return (unsigned int) bitcast<unsigned short>((_Float16) f); }
__device__ __forceinline__ float        f16_bits_to_f32(unsigned int h) { return (float) bitcast<_Float16>((unsigned short) h); }

template <bool F16> __device__ __forceinline__ unsigned int pack2(float a, float b) {
    if constexpr (F16) return f32_to_f16_bits(a) | (f32_to_f16_bits(b) << 16);
    else               return f32_to_bf16_bits(a) | (f32_to_bf16_bits(b) << 16);
}
template <bool F16> __device__ __forceinline__ float round_trip(float a) {
    if constexpr (F16) return (float) (_Float16) a;
    else               return __uint_as_float(f32_to_bf16_bits(a) << 16);
}

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }  // v_exp_f32; exp2(-inf) = 0

__device__ __forceinline__ float xor32(float v) { return __shfl_xor(v, 32, 64); }


// The pipelined decode kernel (mla_decode_kernel.hip); returns hipErrorInvalidValue for shapes it does not take.
bool       decode_fast_applicable(const mla_attn_args * a);
// Raises a kernel's dynamic-LDS limit to the 160 KB of a CU, once per device: the attribute belongs to the function on the
// device that is current.  `done` is the caller's per-function table (zero-initialised static); a second thread that gets
// here before the first has finished only repeats the same call.
constexpr int MLA_MAX_DEVICES = 64;
inline hipError_t raise_lds_limit(const void * fn, bool (&done)[MLA_MAX_DEVICES]) {
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return e;
    if (dev < 0 || dev >= MLA_MAX_DEVICES) return hipErrorInvalidDevice;
    if (done[dev]) return hipSuccess;
    e = hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
    if (e == hipSuccess) done[dev] = true;
    return e;
}

int64_t    decode_fast_q8_copy_rows(const mla_attn_args * a);   // > 0: Q8_0 + mask on rows the wave program cannot tile runs on an f16 copy of that many rows (workspace)
hipError_t launch_mask_extent(const KParams & kp, hipStream_t st);   // fills kp.mask_ext: 16 key pairs per block of 128 rows
hipError_t launch_q8_to_f16(const char * src, int64_t src_nb1, int64_t src_nb3, int64_t rows_per_batch, void * dst, int64_t n_rows, hipStream_t st);
hipError_t launch_decode_fast(const KParams & kp, int kv_type, dim3 grid, hipStream_t st, bool with_prepass, const KParams * tok = nullptr, bool scan_mask = true);
size_t     decode_fast_lds_bytes(int kv_type);
size_t     decode_fast_qpack_bytes(int n_seq, int n_row_blocks);

}  // namespace mla
