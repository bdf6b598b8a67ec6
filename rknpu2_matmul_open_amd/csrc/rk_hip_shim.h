/*
 * rk_hip_shim.h -- the narrow C ABI between the C++ host layer (handles,
 * validation, error codes) and the HIP side (device memory, stream, kernels).
 *
 * Everything here takes raw device pointers, plain sizes and an opaque stream
 * (hipStream_t passed as void*); no HIP type appears in a signature.  This is
 * what stands where the reference has rk_npu_mem_* + its DRM submit ioctls
 * (reference src/rk_npu_internal.h:247-299).
 *
 * Device data layouts
 * -------------------
 * "Tiled int8" (activations and int8 weights): a matrix X[R, K] is stored as
 * 1 KiB tiles of 32 rows x 32 k.  Tile (rb, kb) starts at byte
 * (rb * KB + kb) * 1024 with KB = Kp / 32 and Kp = K rounded up to 256 (RKH_K_ALIGN).
 * Inside a tile, lane l = (row % 32) + 32 * ((k % 32) / 16) owns 16
 * consecutive bytes at l * 16, holding k % 16 = 0..15.  One wavefront reads a
 * tile with a single 16-byte-per-lane load and has the int8 MFMA operand of
 * v_mfma_i32_32x32x32_i8 in its registers; rows beyond R and k beyond K are
 * zero.
 *
 * "Tiled int4" (int4 weights): 1 KiB super-tiles of 32 rows x 64 k.  Super-
 * tile (rb, kb2) starts at (rb * KB2 + kb2) * 1024, KB2 = Kp / 64.  Lane
 * l = (row % 32) + 32 * ((k % 32) / 16) owns 16 bytes: bytes 0..7 belong to
 * the first 32 k of the super-tile, bytes 8..15 to the second.  Each 4-byte
 * word packs 8 consecutive k: byte j holds code[k0 + j] in its low nibble and
 * code[k0 + 4 + j] in its high nibble, so (w << 4) & 0xF0F0F0F0 and
 * w & 0xF0F0F0F0 are the two int8x4 MFMA operand words, each value scaled by
 * 16 (undone exactly by an arithmetic shift of the int32 sum).
 *
 * Column order of weights: when `interleave_F` is non-zero the matrix has
 * N = 2F columns [gate(F), up(F)] and physical 32-column block p holds
 * logical columns (p even ? (p/2)*32 : F + (p/2)*32) .. +31, so a gate block
 * and its up block sit side by side for the fused SwiGLU epilogue.
 */
#ifndef RK_HIP_SHIM_H
#define RK_HIP_SHIM_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Return: 0 ok, -4 allocation failure, -5 any other runtime failure. */
#define RKH_OK 0
#define RKH_ERR_NOMEM (-4)
#define RKH_ERR_RUNTIME (-5)

enum { RKH_ROW_ALIGN = 128, RKH_COL_ALIGN = 256, RKH_K_ALIGN = 256 };

#if defined(__HIPCC__)
#define RKH_HD __host__ __device__
#else
#define RKH_HD
#endif
static inline RKH_HD int64_t rkh_align_up(int64_t v, int64_t a) { return (v + a - 1) / a * a; }
/* Bytes of a tiled int8 matrix with R rows (padded to row_align) and K depth. */
static inline size_t rkh_tiled_i8_bytes(int64_t R, int64_t K, int64_t row_align) {
    return (size_t)(rkh_align_up(R, row_align) * rkh_align_up(K, RKH_K_ALIGN));
}
static inline size_t rkh_tiled_i4_bytes(int64_t R, int64_t K, int64_t row_align) {
    return (size_t)(rkh_align_up(R, row_align) * rkh_align_up(K, RKH_K_ALIGN) / 2);
}

/* ---- device, stream, memory ---- */
int rkh_device_count(void);
int rkh_open(int device, void** stream_out, char* name_out, int name_len, int* cu_count,
             int* clock_khz);
void rkh_close(int device, void* stream);
int rkh_malloc(int device, void** ptr, size_t bytes);
void rkh_free(int device, void* ptr);
int rkh_host_alloc(void** ptr, size_t bytes); /* pinned staging */
void rkh_host_free(void* ptr);
int rkh_h2d(void* stream, void* dst, const void* src, size_t bytes);   /* async */
int rkh_d2h(void* stream, void* dst, const void* src, size_t bytes);   /* async */
int rkh_d2d(void* stream, void* dst, const void* src, size_t bytes);   /* async */
int rkh_fill32(void* stream, void* dst, uint32_t value, size_t words); /* fill kernel */
int rkh_exchange32(void* stream, void* x, void* y, size_t words);      /* swaps two disjoint arrays, async */
int rkh_sync(void* stream);
/* Test hook: make the n-th next rkh_malloc fail (n = 1 fails the next one,
 * 0 disables).  Lets allocation-failure paths be exercised from the host. */
void rkh_fail_malloc_after(int n);

/* Stream timing for the timings structs and the benchmark. */
int rkh_event_create(void** event);
void rkh_event_destroy(void* event);
int rkh_event_record(void* event, void* stream);
int rkh_event_sync(void* event);                                /* blocks until the event has happened */
int rkh_event_elapsed_us(void* start, void* stop, double* us); /* waits for stop */

/* ---- weight re-tiling at upload ---- */
/* src: B[K, N] row-major int8 on the device (raw copy of the caller's array).
 * dst: tiled int8, rows = output channels, Np = N rounded up to RKH_COL_ALIGN.
 * dst must be zero-filled by the caller beforehand only if it was not
 * allocated through this call's full coverage: the kernel writes every byte
 * of dst. */
int rkh_pack_w8(void* stream, const int8_t* src, int K, int N, int interleave_F, uint8_t* dst);
/* Same for int4 codes in [-8, 7] (one int8 per code in src).  bad_flag (device
 * int, may be NULL) is OR-ed with 1 if a code is outside [-8, 7].  colsum (device
 * int32 [N], zero-filled by the caller, may be NULL) receives sum_k B[k, n] per
 * logical column: the constant the int4 GEMV kernels add (rkh_gemm_args.w_colsum). */
int rkh_pack_w4(void* stream, const int8_t* src, int K, int N, int interleave_F, uint8_t* dst,
                int* bad_flag, int32_t* colsum);

/* ---- per-row activation quantization ---- */
enum rkh_quant_mode {
    RKH_Q_W8_DYNAMIC = 0, /* s = max>0 ? max/127 : 1 ; ties away ; no finite check     */
    RKH_Q_W8_STATIC = 1,  /* s given in scale[] ; ties away                             */
    RKH_Q_W4A8 = 2,       /* s = max==0 ? 1 : max(max/127, FLT_MIN) ; ties away ; check */
    RKH_Q_COPY_I8 = 4,    /* input already int8: re-tile only (scale[] passes through)  */
    RKH_Q_REUSE_BITS = 5, /* s from row_max_bits[] (W4A8 rule) ; ties away              */
    RKH_Q_REUSE_BITS_MOE = 6 /* s from row_max_bits[] (MoE rule) ; ties even            */
};
enum rkh_dtype { RKH_F16 = 0, RKH_F32 = 1, RKH_I8 = 2, RKH_I32 = 3 };

typedef struct rkh_quant_args {
    const void* src;     /* [M, K] row-major, element type in_dtype               */
    int in_dtype;        /* RKH_F16 / RKH_F32 / RKH_I8                             */
    int mode;            /* rkh_quant_mode                                         */
    int M, K;
    float* scale;        /* [M] out (in for STATIC)                                */
    uint8_t* dst;        /* tiled int8, Kp = align256(K)                           */
    int* bad_flag;       /* OR 1: non-finite input (modes with a check), may be NULL */
    const uint32_t* row_max_bits; /* REUSE modes: [M][row_max_parts] partial maxima of |x| bits */
    int row_max_parts;
    /* If non-NULL, rows at or beyond active_blocks[0] * 32 are skipped. */
    const int* active_blocks;
    /* src is pinned host memory read over the bus: every row must be read once,
     * so the quantization is not folded into a GEMV whose workgroups would each
     * fetch the rows again. */
    int src_is_host;
} rkh_quant_args;
int rkh_quant_rows(void* stream, const rkh_quant_args* args);

/* ---- GEMM / GEMV ---- */
enum rkh_epilogue {
    RKH_EPI_I32 = 0,    /* C int32 = acc                                           */
    RKH_EPI_F16 = 1,    /* C fp16  = rne16((float(acc) * as[m]) * ws[n])           */
    RKH_EPI_F32 = 2,    /* C fp32  = (float(acc) * as[m]) * ws[n]                  */
    RKH_EPI_SWIGLU = 3  /* C fp32 [M, F] = silu(g) * u, partial row maxima written  */
};

typedef struct rkh_gemm_args {
    const uint8_t* A;     /* tiled int8 activations                                */
    const uint8_t* W;     /* tiled int8 or int4 weights                            */
    int w_int4;           /* 0 / 1                                                 */
    int M, N, K;          /* logical sizes; N counts weight columns (2F for SwiGLU)*/
    int interleave_F;     /* 0, or F when the weight columns are gate/up interleaved */
    const float* a_scale; /* [align(M)]                                            */
    const float* w_scale; /* [N] in logical column order                           */
    const int32_t* w_colsum; /* int4 weights, dense: [N] column sums of the codes (rkh_pack_w4); the
                              * M <= 8 kernels need them, without them such calls take the MFMA path */
    int epilogue;         /* rkh_epilogue                                          */
    void* C;              /* [M, ldc]                                              */
    int ldc;
    uint32_t* row_max_bits; /* SwiGLU: [rows][F/32] max |middle| bits per 32 columns */
    int32_t* splitk_acc;  /* scratch [align(M,128) * align(N,256)] int32 for split-K, or NULL */
    /* Grouped (MoE) mode when blk_expert != NULL: row-block b (32 rows of the
     * sorted activation buffer) uses expert blk_expert[b]; blocks at or beyond
     * *num_blocks are skipped; M = upper bound of sorted rows. */
    const int* blk_expert;
    const int* num_blocks;
    int max_blocks;
    size_t w_expert_stride;  /* bytes between experts in W                        */
    size_t ws_expert_stride; /* floats between experts in w_scale                 */
    /* Grouped mode, expert formats: experts below int4_experts are tiled int4 images in W4
     * (expert e at e * w4_expert_stride), the others tiled int8 images in W (expert e at
     * (e - int4_experts) * w_expert_stride; W may be NULL when there is none).  A bank that
     * holds both formats takes one launch per format; w_int4 is not used in grouped mode. */
    const uint8_t* W4;
    int int4_experts;
    size_t w4_expert_stride;
} rkh_gemm_args;
int rkh_gemm(void* stream, const rkh_gemm_args* args);
/* quantize + GEMM as one request: for decode-sized M the quantization is fused
 * into the GEMV kernel (one launch); otherwise the two kernels run back to back.
 * Either way qargs->dst / qargs->scale end up holding the quantized rows. */
int rkh_quant_gemm(void* stream, const rkh_quant_args* qargs, const rkh_gemm_args* gargs);
/* Bytes of split-K scratch rkh_gemm may use for a dense problem of this shape
 * (0 when it never splits K); the caller passes a zero-filled buffer of at
 * least this size in splitk_acc. */
size_t rkh_gemm_scratch_bytes(int M, int N, int K, int w_int4);

/* ---- MoE routing and combine ---- */
/* Routing + token scatter in one launch: assignments with a non-zero
 * coefficient are bucketed by expert, stably, each bucket padded to 32 sorted
 * rows (the shared expert, id == experts, takes every token); each token is
 * quantized per row (s = max ? max/127 : 1, ties even, rejected input -> bad_flag)
 * or, for int8 input, copied, into the sorted rows of its assignments. */
typedef struct rkh_moe_scatter_args {
    const int32_t* ids;    /* [rows, top_k] device                                 */
    const float* routes;   /* [rows, top_k] device                                 */
    int rows, top_k, experts, shared; /* experts = routed count                    */
    int* dest_rows;        /* [rows, top_k + shared] out: sorted row or -1         */
    int* blk_expert;       /* [max_blocks] out                                     */
    int* num_blocks;       /* [2] out: {row blocks, assignments}                   */
    int max_blocks;
    const void* src;       /* [rows, K] tokens: RKH_F32, or RKH_I8 codes           */
    int in_dtype;
    int K;
    float* token_scale;    /* [rows]: out for fp32 tokens, in for int8 codes       */
    uint8_t* dst;          /* tiled int8 sorted rows                               */
    float* scale_rows;     /* [sorted rows] out: scale of the token in that row    */
    int* bad_flag;         /* OR 1 on rejected input, may be NULL: a non-finite fp32 token or one
                            * whose scale underflows, a token scale that is not finite and
                            * positive, an expert id outside [0, experts), a coefficient that is
                            * negative or not finite                                            */
} rkh_moe_scatter_args;
int rkh_moe_scatter(void* stream, const rkh_moe_scatter_args* args);

typedef struct rkh_moe_combine_args {
    const float* Y;        /* [sorted rows, H] fp32 expert outputs                 */
    const int* dest_rows;  /* [rows, slots]                                        */
    const float* routes;   /* [rows, top_k]                                        */
    int rows, top_k, shared, H;
    float* out;            /* [rows, H]                                            */
} rkh_moe_combine_args;
int rkh_moe_combine(void* stream, const rkh_moe_combine_args* args);

/* A MoE layer for a handful of tokens in two launches instead of five, same results: (1) per
 * (assignment, 32 middle columns) the token is quantized, multiplied with the gate and up blocks
 * of its expert and passed through SwiGLU -> hidden + partial row maxima; (2) per (token, 32
 * output columns) each live slot's hidden row is re-quantized from the partial maxima, multiplied
 * with the expert's down block, scaled and accumulated in slot order.  Everything device-resident.
 * Returns RKH_ERR_RUNTIME for shapes it does not take (rkh_moe_decode_applies). */
typedef struct rkh_moe_decode_args {
    const float* x;          /* [rows, H] fp32 tokens                                */
    const int32_t* ids;      /* [rows, top_k]                                        */
    const float* routes;     /* [rows, top_k]                                        */
    int rows, top_k, experts, shared; /* experts = routed count; the shared one is expert `experts` */
    int H, I;
    const uint8_t* gate_W;   /* int8 experts: tiled [2I x H] images, gate / up blocks interleaved */
    const uint8_t* gate_W4;  /* int4 experts (the first int4_experts of the bank)    */
    const uint8_t* down_W;
    const uint8_t* down_W4;
    int int4_experts;
    size_t gate_stride, gate_stride4, down_stride, down_stride4; /* bytes between experts */
    const float* gate_scales; /* [experts + shared][2I]                              */
    const float* down_scales; /* [experts + shared][H]                               */
    float* hidden;           /* scratch [rows * (top_k + shared)][I]                 */
    uint32_t* row_max_bits;  /* scratch [rows * (top_k + shared)][I / 32]            */
    float* out;              /* [rows, H]                                            */
    int* bad_flag;           /* OR 1 on a rejected token or routing entry, may be NULL */
} rkh_moe_decode_args;
int rkh_moe_decode_applies(int rows, int H, int I);
int rkh_moe_decode(void* stream, const rkh_moe_decode_args* args);


/* ---- measurement probes (practical ceilings beside the datasheet peaks) ---- */
/* One read-only pass over [src, src + bytes): a workgroup of 512 lanes per `span` bytes
 * (a multiple of 1024), pieces of 1 KiB interleaved over its eight waves. */
int rkh_probe_stream_read(void* stream, const void* src, size_t bytes, size_t span, void* sink);
/* `workgroups` x 8 waves x `iterations` x 4 int8 MFMAs (32x32x32) on operands read once from
 * `operands` (32 KiB: 4 x 512 lanes x 16 bytes). */
int rkh_probe_mfma_i8(void* stream, const void* operands, int workgroups, int iterations, void* sink);

/* ---- stage marker ----
 * While a marker is set, it is called with the kernel's name right before every kernel this
 * shim launches (on the launching thread, with the stream of the launch).  Process-wide;
 * NULL switches it off.  For per-kernel timing of multi-kernel steps with stream events. */
typedef void (*rkh_marker_fn)(void* user, void* stream, const char* kernel);
void rkh_set_marker(rkh_marker_fn fn, void* user);

/* ---- stream capture ---- */
int rkh_capture_begin(void* stream);
int rkh_capture_end(void* stream, void** graph_exec);
int rkh_graph_launch(void* graph_exec, void* stream);
void rkh_graph_destroy(void* graph_exec);

/* ---- static scratch: address and size of the file-scope device array on `device` ---- */
int rkh_static_scratch(int device, void** ptr, size_t* bytes);

#ifdef __cplusplus
}
#endif
#endif /* RK_HIP_SHIM_H */
