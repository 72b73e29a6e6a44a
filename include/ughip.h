/*
 * ughip.h -- C ABI of the MI355X (gfx950) backend for ug.
 *
 * This is the boundary a Rust `ug-hip` crate binds with `extern "C"` to implement
 * ug-core's `trait Device` / `trait Slice` (ug-core/src/lib.rs:29-73) and ug-llama's
 * `trait Device` (ug-llama/src/main.rs:22-28).  Plain pointers and sizes only.
 *
 * Conventions
 *   - every function returns 0 on success and a non-zero UGHIP_ERR_* code on failure;
 *     ughip_last_error() then returns a thread-local, NUL-terminated message
 *     (the shim maps it to ug::Error::Msg, ug-core/src/error.rs:3-100);
 *   - lengths are in ELEMENTS unless the name says bytes;
 *   - one HIP stream per device; work is stream-ordered and asynchronous unless stated;
 *   - the caller is single-threaded per device, like ug's Arc<RefCell<..>> graph
 *     (ug-core/src/lazy_buffer.rs:101-106).
 */
#ifndef UGHIP_H_
#define UGHIP_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ---- error codes -------------------------------------------------------------------- */
enum {
  UGHIP_OK = 0,
  UGHIP_ERR_INVALID = 1,      /* bad argument, dtype/len mismatch (cpu_runtime.rs:380-391) */
  UGHIP_ERR_HIP = 2,          /* a HIP runtime call failed */
  UGHIP_ERR_COMPILE = 3,      /* hiprtc rejected generated code, or malformed SSA */
  UGHIP_ERR_STRIDING = 4,     /* Error::MatMulUnexpectedStriding (error.rs:110-116) */
  UGHIP_ERR_UNSUPPORTED = 5,  /* dtype / op combination not implemented */
  UGHIP_ERR_BOUNDS = 6        /* a kernel would index past the end of one of its slices */
};

/* ---- ug::DType (ug-core/src/dtype.rs:5-12), same order ------------------------------ */
enum {
  UGHIP_BF16 = 0,
  UGHIP_F16 = 1,
  UGHIP_F32 = 2,
  UGHIP_I32 = 3,
  UGHIP_I64 = 4
};

/* ---- ssa IR on the wire (ug-core/src/lang.rs:611-753) ------------------------------- *
 * `ssa::Kernel` is a flat instruction list; the line number of an instruction is the
 * VarId of its result.  The structs below are a field-for-field POD image of
 * `ssa::A`, `ssa::Instr`, `(Arg, usize)` and `LaunchConfig` built from the public
 * accessors `instrs()`, `args()`, `launch_config()` (lang.rs:719-729).               */

/* ssa::A (lang.rs:642-646): a variable reference or an inline constant. */
typedef struct ughip_a {
  uint8_t is_const; /* 0: Var(var), 1: Const */
  uint8_t dtype;    /* Const only: UGHIP_* dtype of the constant */
  uint16_t pad_;
  uint32_t var;     /* Var only: VarId */
  int64_t i;        /* Const I32 / I64 value */
  float f;          /* Const F32 / F16 / BF16 value (exact: both widen losslessly to f32) */
  uint32_t pad2_;
} ughip_a;

/* ssa::Instr discriminant (lang.rs:690-709), same order. */
enum {
  UGHIP_I_DEFINE_ACC = 0,    /* a = initial Const */
  UGHIP_I_DEFINE_GLOBAL = 1, /* n = index, dtype */
  UGHIP_I_DEFINE_LOCAL = 2,  /* n = size (elements), dtype */
  UGHIP_I_SPECIAL = 3,       /* sub = UGHIP_SPECIAL_* */
  UGHIP_I_CONST = 4,         /* a = Const */
  UGHIP_I_UNARY = 5,         /* sub = UGHIP_U_*, a = arg, dtype = result dtype */
  UGHIP_I_BINARY = 6,        /* sub = UGHIP_B_*, a = lhs, b = rhs, dtype */
  UGHIP_I_RANGE = 7,         /* a = lo, b = up, n = step, v = end_idx */
  UGHIP_I_LOAD = 8,          /* v = src pointer var, a = offset, dtype */
  UGHIP_I_ASSIGN = 9,        /* v = dst var, a = src */
  UGHIP_I_END_RANGE = 10,    /* v = start_idx */
  UGHIP_I_IF = 11,           /* a = cond, v = end_idx */
  UGHIP_I_END_IF = 12,
  UGHIP_I_STORE = 13,        /* v = dst pointer var, a = offset, b = value, dtype */
  UGHIP_I_BARRIER = 14,
  UGHIP_I_REDUCE_LOCAL = 15  /* sub = UGHIP_R_*, a = arg, dtype */
};

enum { UGHIP_SPECIAL_THREAD_IDX = 0, UGHIP_SPECIAL_BLOCK_IDX = 1 };           /* lang.rs:637-640 */
enum { UGHIP_R_SUM = 0, UGHIP_R_MAX = 1, UGHIP_R_MIN = 2 };                   /* lang.rs:6-10   */
enum { UGHIP_U_ID = 0, UGHIP_U_EXP, UGHIP_U_SIN, UGHIP_U_COS, UGHIP_U_NEG,
       UGHIP_U_SQRT, UGHIP_U_CAST };                                          /* lang.rs:13-21  */
enum { UGHIP_B_ADD = 0, UGHIP_B_SUB, UGHIP_B_MUL, UGHIP_B_DIV, UGHIP_B_MOD,
       UGHIP_B_MIN, UGHIP_B_MAX };                                            /* lang.rs:24-32  */

typedef struct ughip_instr {
  int32_t op;    /* UGHIP_I_* */
  int32_t dtype; /* UGHIP_* dtype where the instruction carries one */
  int32_t sub;   /* op-specific selector, see the enum comments */
  uint32_t v;    /* VarId operand (pointer var, assign target, range partner) */
  uint64_t n;    /* index / size / step */
  ughip_a a;
  ughip_a b;
} ughip_instr;

/* One entry of ssa::Kernel::args(): (Arg, line_no) (lang.rs:714,727). */
typedef struct ughip_kernel_arg {
  uint64_t arg_id; /* ArgId, informational */
  uint8_t is_ptr;  /* Type::Ptr vs Type::Value; only pointers are supported (lower_op.rs:413-416) */
  uint8_t dtype;
  uint16_t pad_;
  uint32_t var;    /* line number of the DefineGlobal that introduces it */
} ughip_kernel_arg;

typedef struct ughip_ssa {
  const ughip_instr* instrs;
  size_t n_instrs;
  const ughip_kernel_arg* args;
  size_t n_args;
  uint32_t grid_dim;   /* LaunchConfig (lang.rs:34-39); honoured only for kernels that use */
  uint32_t block_dim;  /* Special / Barrier / ReduceLocal / DefineLocal -- serial loop nests */
  uint32_t shared_mem; /* are re-parallelised by the backend and ignore it.               */
  uint32_t pad_;
} ughip_ssa;

/* ---- opaque handles ------------------------------------------------------------------ */
typedef struct ughip_device ughip_device; /* ug_cuda::runtime::Device  (ug-cuda/src/runtime.rs:80-85) */
typedef struct ughip_slice ughip_slice;   /* ug_cuda::runtime::Slice   (runtime.rs:88-101)            */
typedef struct ughip_func ughip_func;     /* ug_cuda::runtime::Func    (runtime.rs:49-54)             */
typedef struct ughip_event ughip_event;

const char* ughip_last_error(void);
/* Tuning and test aid with no counterpart in the reference (cuBLAS picks its kernels out of sight,
 * ug-cuda/src/gemm.rs:130-290): the hand-written kernel the calling thread's last ughip_matmul
 * launched, e.g. "gemm_tiled<f32,NN,256x128,512t>", "gemm_tiled<bf16,NT,128x64,256t,ragged,splitK=12>",
 * "gemv_nt<f32>", "gemm_any<f16>".  Thread-local; "" before the first product. */
const char* ughip_last_kernel(void);

/* ---- device: Device::new / Clone / synchronize (runtime.rs:158-177,243-246) ---------- */
int ughip_device_create(int ordinal, ughip_device** out);
int ughip_device_retain(ughip_device* dev);
int ughip_device_release(ughip_device* dev);
int ughip_synchronize(ughip_device* dev);
/* "gfx950" etc.; buf receives a NUL-terminated arch name. */
int ughip_device_arch(ughip_device* dev, char* buf, size_t buf_len);
/* Introspection: code objects built by hiprtc so far, bytes cached in the allocation pool, bytes
 * handed out to live slices.  Any out pointer may be NULL. */
int ughip_device_stats(ughip_device* dev, size_t* n_code_objects, size_t* pool_bytes, size_t* live_bytes);
/* `Device::use_grid()` (lib.rs:72): this backend returns 0 -- it wants the serial loop
 * nest and chooses grid/block itself. */
int ughip_use_grid(void);

/* ---- memory: Device::allocate_uninit, trait Slice (lib.rs:29-54) --------------------- */
/* Zero-filled like CpuDevice::allocate_uninit (cpu_runtime.rs:255-264).  len 0 is legal
 * (ug-llama/src/model.rs:192) and yields a slice with a null device pointer. */
int ughip_alloc(ughip_device* dev, int dtype, size_t len, ughip_slice** out);
/* Turn the zero-fill of ughip_alloc off (on = 0) or back on: ug-cuda's allocate_uninit leaves memory
 * uninitialised (ug-cuda/src/runtime.rs:217-241), and a caller whose kernels overwrite every
 * destination -- the llama graph does -- saves one fill launch per allocation. */
int ughip_device_set_zero_fill(ughip_device* dev, int on);
int ughip_free(ughip_slice* s);
size_t ughip_slice_len(const ughip_slice* s);
int ughip_slice_dtype(const ughip_slice* s);
void* ughip_slice_ptr(const ughip_slice* s); /* raw device pointer (for interop / tests) */
/* Slice::copy_host_to_device / copy_device_to_host (lib.rs:35-36): error unless
 * dtype == slice dtype and len == slice len (cpu_runtime.rs:376-412).  The result is
 * visible when the call returns. */
int ughip_h2d(ughip_slice* dst, const void* src, int dtype, size_t len);
int ughip_d2h(const ughip_slice* src, void* dst, int dtype, size_t len);

/* Tuning switches, with no counterpart in the reference: tile, split and kernel-family overrides used by the
 * tests and for measurements (GEMM_SHAPE, GEMM_SPLIT, GEMM_4WAVES, GEMV_KS, GEMV_ROWS, GEMV_BF16_ROWS, X3_DMA,
 * X3_SPLIT, ATT_SPLIT, NO_PARAMETRIC, NO_NT_LOADS, GRID_REDUCE_BLOCKS, GRID_REDUCE_THREADS, NO_NT_STORES, SOFTMAX_STREAM; a leading "UGHIP_" is accepted).  The
 * table is read once per process from the environment (UGHIP_<NAME>) and changes afterwards only through this
 * call: set != 0 stores `value`, set == 0 clears the switch.  Dispatch reads the table, never the environment,
 * so the call is safe next to a thread that is launching. */
int ughip_set_tuning(const char* name, int set, int64_t value);

/* ---- kernels: Device::compile / Device::run (lib.rs:56-60) --------------------------- */
/* name may be NULL; it is sanitised and uniquified (runtime.rs:249-253).  Constants are
 * baked into the SSA (lib.rs:57-59). */
int ughip_compile(ughip_device* dev, const ughip_ssa* ssa, const char* name, ughip_func** out);
int ughip_func_release(ughip_func* f);
/* args in ssa.args() order (schedule.rs:190-195); asynchronous; zero-sized launch is a
 * no-op (runtime.rs:269-277).  Fails with UGHIP_ERR_BOUNDS if a slice is shorter than the
 * largest offset the kernel can form (ughip_codegen_min_len says how that is counted under an If). */
int ughip_run(ughip_device* dev, ughip_func* f, ughip_slice* const* args, size_t n_args);
/* Timing aid with no counterpart in the reference: a func lowered to two kernels (a grid-wide reduction:
 * partial sums, then the fold) launches only its first (part 1) or second (part 2) kernel, with the checks of
 * ughip_run.  Part 2 alone reads whatever partials the last part 1 left; a single-kernel func has no part 2. */
int ughip_run_part(ughip_device* dev, ughip_func* f, ughip_slice* const* args, size_t n_args, int part);
/* HIP source the SSA was lowered to (counterpart of `Kernel.cuda_code()`,
 * ug-pyo3/src/lib.rs:396-401).  Returns the length excluding NUL; copies at most buf_len. */
size_t ughip_func_source(const ughip_func* f, char* buf, size_t buf_len);
/* Lowering strategy and launch shape picked by the backend (for tests and profiling). */
typedef struct ughip_func_info {
  int32_t strategy; /* UGHIP_STRAT_* */
  uint32_t grid_dim;
  uint32_t block_dim;
  uint32_t lds_bytes;
  uint64_t scratch_bytes;
} ughip_func_info;
enum {
  UGHIP_STRAT_LITERAL = 0,     /* 1:1 translation, SSA launch config */
  UGHIP_STRAT_ELEMENTWISE = 1, /* flat thread-per-element(s) */
  UGHIP_STRAT_ROW_BLOCK = 2,   /* workgroup (or wave) per row, cooperative reduce */
  UGHIP_STRAT_ROW_THREAD = 3,  /* thread per row, serial reduce (strided reduce dims) */
  UGHIP_STRAT_GRID_REDUCE = 4  /* many workgroups per row + deterministic second stage */
};
int ughip_func_get_info(const ughip_func* f, ughip_func_info* out);
/* Lowering only, no device needed: SSA -> HIP source (for CPU-side inspection/tests). */
int ughip_codegen(const ughip_ssa* ssa, const char* name, char* buf, size_t buf_len,
                  size_t* out_len, ughip_func_info* info);
/* Lowering only, no device needed: per kernel argument, the number of elements a slice must hold for
 * ughip_run to accept it (1 + the largest offset the kernel can form; -1 where an offset is computed
 * from loaded data and cannot be bounded).  An access under an If counts with what the guard lets
 * through where the guard pins the offset (`If(max(n - i, 0))` around `dst[i]`: n elements); a guard
 * that says nothing about the offset leaves the full requirement.  n_args must be the kernel's. */
int ughip_codegen_min_len(const ughip_ssa* ssa, int64_t* min_len, size_t n_args);

/* The same kernel translated statement by statement, for its own launch configuration: a serial
 * loop nest stays one thread's loop nest, as in the text ug-cuda/src/code_gen.rs:68-186 produces
 * and ug-pyo3 hands out as `Kernel.cuda_code(name)` (ug-pyo3/src/lib.rs:396-401).  The entry point
 * is `extern "C" __global__ void <name>(...)` with one pointer per kernel argument; `name` must be
 * a C identifier.  Slow by construction; ughip_compile is the fast path. */
int ughip_codegen_as_written(const ughip_ssa* ssa, const char* name, char* buf, size_t buf_len,
                             size_t* out_len);
/* Device::compile_cu (ug-cuda/src/runtime.rs:179-186) as ug-pyo3 exposes it
 * (ug-pyo3/src/lib.rs:438-456): build HIP source text with hiprtc and take kernel `entry` with a
 * fixed launch configuration.  The kernel takes n_args pointers, one per slice passed to ughip_run;
 * arg_dtypes are checked against the slices, lengths are not (the library does not know what the
 * source indexes), and no slice may appear twice in one call. */
int ughip_compile_source(ughip_device* dev, const char* source, const char* entry, size_t n_args,
                         const int* arg_dtypes, unsigned grid_dim, unsigned block_dim,
                         unsigned shared_mem_bytes, ughip_func** out);

/* hiprtc only, no device needed: does `source` build for `arch` ("gfx950")?  Lets the CPU-side
 * test-suite check that every generated kernel compiles. */
int ughip_rtc_check(const char* source, const char* arch, size_t* code_size);

/* ---- matmul: Device::matmul (lib.rs:62-70) ------------------------------------------- */
/* dst[b,m,n] = lhs[b,m,k] x rhs[b,k,n], beta = 0, f32 accumulate.  `rank` (2..4) strides
 * per operand, in elements, as in ug::Layout (layout.rs:577-583); batch strides follow
 * the rules of cpu_runtime.rs:527-549 and ug-cuda/src/gemm.rs:59-74.  dtype triple must
 * match: F32, F16 or BF16 (ug-cuda/src/gemm.rs:303-330); integers are UGHIP_ERR_UNSUPPORTED.
 * One addition to the reference's contract: dst and lhs F32 with rhs BF16 (weights kept as a
 * checkpoint stores them, where the reference widens them at load time,
 * ug-core/src/safetensors.rs:120-271).  The rhs is widened on its way into LDS, so the result is
 * bit for bit that of the F32 product on the widened values.  Built for an [n, k]-major rhs
 * (strides (1, k)) with k % 32 == 0; other layouts are UGHIP_ERR_UNSUPPORTED (convert the rhs
 * with ughip_convert first).
 * With the tuning switch MATMUL_X6 set to 1 (ughip_set_tuning, or UGHIP_MATMUL_X6=1 in the environment), an F32 product of
 * contiguous operands with k % 64 == 0, n % 8 == 0 and m >= 9 runs on the bf16 matrix pipe: both operands are split into
 * three bf16 terms each (x = hi + mid + lo exactly) in a scratch block of the device (6 bytes per operand element), and six
 * of the nine term products -- everything above 2^-24 of a product -- are accumulated in f32.  The f32 product's accuracy
 * (same k eps bound against float64), not its bits; off by default. */
int ughip_matmul(ughip_device* dev, ughip_slice* dst, const ughip_slice* lhs,
                 const ughip_slice* rhs, size_t b, size_t m, size_t n, size_t k, size_t rank,
                 const size_t* lhs_dims, const size_t* lhs_strides, size_t lhs_offset,
                 const size_t* rhs_dims, const size_t* rhs_strides, size_t rhs_offset);
/* No counterpart in the reference, no device needed: the kernel ughip_matmul would launch for contiguous operands of
 * these shapes (rhs_nk != 0: the rhs stored [n, k]), by the name ughip_last_kernel() reports after the launch -- tile,
 * K split and all.  The choice follows from shapes and from the library's cost models; tests pin it for the shapes
 * that matter, so that a change of a model constant shows as a changed plan. */
int ughip_matmul_plan(int dtype, int rhs_dtype, size_t b, size_t m, size_t n, size_t k, int rhs_nk, char* buf,
                      size_t buf_len);

/* ughip_matmul for callers that cannot allocate (code under HIP graph capture, tight serving loops,
 * harnesses that forbid hipMalloc).  No counterpart in the reference.  Same arguments, same kernels and
 * the same bits as ughip_matmul, but it calls no hipMalloc / hipFree: products that split K (skinny
 * shapes with a long k, e.g. the projections of a 128-token prefill) put their f32 partial tiles into a
 * static device array of UGHIP_MATMUL_NOALLOC_SCRATCH_BYTES that each GPU holds until the process ends,
 * instead of the grown-on-demand block ughip_matmul keeps per device.  A product whose partial tiles
 * need more is refused with UGHIP_ERR_UNSUPPORTED (the message gives both sizes).  All calls on one GPU
 * share that GPU's array: calls that overlap on one GPU (two threads, two streams) race; calls of one
 * thread are ordered by the device's stream.  Nothing in the array has to start at zero. */
#define UGHIP_MATMUL_NOALLOC_SCRATCH_BYTES (64u << 20)
int ughip_matmul_noalloc(ughip_device* dev, ughip_slice* dst, const ughip_slice* lhs,
                         const ughip_slice* rhs, size_t b, size_t m, size_t n, size_t k, size_t rank,
                         const size_t* lhs_dims, const size_t* lhs_strides, size_t lhs_offset,
                         const size_t* rhs_dims, const size_t* rhs_strides, size_t rhs_offset);

/* ---- ug-llama custom ops (ug-llama/src/main.rs:22-28; oracle cpu_ops.rs:6-167) ------- */
/* rope / rope_i (cuda_ops.rs:17-104): src, dst are [bh, t*d] f32, cos/sin [max_pos, d/2]
 * f32, pos i32 (only pos[0] is read, cpu_ops.rs:67,100).
 * pos lives on the device, so the host cannot check it against the table: a position whose table row
 * pos[0] + i_t lies outside cos/sin is never read (no out-of-bounds access) and the rotated values of that
 * row come out as NaN, here and in every fused entry point below that takes (cos, sin, pos) -- where the
 * reference's slice index would panic (cpu_ops.rs:76-77,112-113).  Callers that know the position on the
 * host check it there (the llama graph refuses a step past its cache / table when it is built). */
int ughip_rope(ughip_device* dev, const ughip_slice* src, const ughip_slice* cos,
               const ughip_slice* sin, const ughip_slice* pos, ughip_slice* dst, size_t bh,
               size_t t, size_t d, int interleaved);
/* cat (cuda_ops.rs:106-141): [d1, d2_l] ++ [d1, d2_r] -> [d1, d2_l + d2_r], f32. */
int ughip_cat(ughip_device* dev, const ughip_slice* lhs, const ughip_slice* rhs,
              ughip_slice* dst, size_t d1, size_t d2_l, size_t d2_r);
/* custom_softmax (cuda_ops.rs:143-174): row softmax over the last dim, f32. */
int ughip_softmax_rows(ughip_device* dev, const ughip_slice* src, ughip_slice* dst,
                       size_t n_rows, size_t n_cols);
/* causal_mask (cpu_ops.rs:33-56; the CUDA and Metal backends bail): per [s1, s2] chunk,
 * keep i2 <= i1, else -inf. */
int ughip_causal_mask(ughip_device* dev, const ughip_slice* src, ughip_slice* dst, size_t bh,
                      size_t s1, size_t s2);

/* ---- attention fusions (no counterpart in the reference's device trait) ----------------------
 * The step either side of the softmax kernel: what ug-llama builds from several ops
 * (ug-llama/src/model.rs:231-244) as one launch each.  A caller opts in; the unfused ops above
 * stay the reference behaviour. */
/* causal_mask followed by custom_softmax over [bh, s1, s2], f32: row i1 keeps columns
 * i2 <= i1 (cpu_ops.rs:33-56), masked columns come out as 0. */
int ughip_causal_softmax_rows(ughip_device* dev, const ughip_slice* src, ughip_slice* dst,
                              size_t bh, size_t s1, size_t s2);
/* Attention of one query position, f32: q [b, n_heads, d], k and v [b, n_kv_heads, s, d]
 * (query head h reads kv head h / (n_heads / n_kv_heads), i.e. model.rs:80-92's repeat),
 * dst [b, n_heads, d] = softmax(q k^T * scale) v.  d a power of two in 16..256.  From 800 keys up
 * the keys of a head are split over several workgroups and merged by a second launch; the partial
 * rows live in a scratch block the device keeps (grown on demand). */
int ughip_attention_decode(ughip_device* dev, const ughip_slice* q, const ughip_slice* k,
                           const ughip_slice* v, ughip_slice* dst, size_t b, size_t n_heads,
                           size_t n_kv_heads, size_t s, size_t d, float scale);
/* The same with rope (interleaved = 0, cpu_ops.rs:91-126) or rope_i (1, cpu_ops.rs:58-89) applied
 * to q first, at table row pos[0]; q and dst are the flat [b, n_heads * d] rows the projections
 * read and write, so the transposes of model.rs:210 and :245 disappear for one position.
 * cos = sin = pos = NULL: no rotation. */
int ughip_attention_decode_rope(ughip_device* dev, const ughip_slice* q, const ughip_slice* k,
                                const ughip_slice* v, ughip_slice* dst, size_t b, size_t n_heads,
                                size_t n_kv_heads, size_t s, size_t d, float scale,
                                const ughip_slice* cos, const ughip_slice* sin,
                                const ughip_slice* pos, int interleaved);
/* Cache growth for one new position (model.rs:211-230 at t = 1): dst [bh, s_old + 1, d] =
 * cat(cache [bh, s_old, d], x [bh, 1, d]) with x rotated first when cos/sin/pos are given
 * (keys) and copied as is when they are NULL (values).  s_old may be 0 (cache may then be an
 * empty slice or NULL).  d % 8 == 0. */
int ughip_rope_append(ughip_device* dev, const ughip_slice* cache, const ughip_slice* x,
                      ughip_slice* dst, size_t bh, size_t s_old, size_t d,
                      const ughip_slice* cos, const ughip_slice* sin, const ughip_slice* pos,
                      int interleaved);
/* The same growth in place, for t new positions at once (replaces the cat of model.rs:226-230,
 * which copies the whole cache every step): cache [b, n, cap, d] is preallocated for cap
 * positions; rows s_old .. s_old + t - 1 of every head receive x [b, t, n * d] (the layout the
 * k / v projections write), rotated at table rows pos[0] + i when cos/sin/pos are given.
 * s_old + t <= cap, d % 4 == 0.  Rows past s_old + t are left untouched.
 * x may be a column range of wider rows (the k or v part of a packed q|k|v projection): row i
 * then starts at element x_offset + i * x_row_stride of the slice (multiples of 4);
 * x_row_stride = 0 means dense rows of n * d. */
int ughip_kv_append(ughip_device* dev, ughip_slice* cache, const ughip_slice* x, size_t x_offset,
                    size_t x_row_stride, size_t b, size_t n, size_t cap, size_t s_old, size_t t,
                    size_t d,
                    const ughip_slice* cos, const ughip_slice* sin, const ughip_slice* pos,
                    int interleaved);
/* Both appends of a layer in one launch: the k part (rotated when cos/sin/pos are given) and the v part
 * (copied) of packed rows x [b, t, x_row_stride], at elements k_offset and v_offset of every row, go into
 * rows s_old .. s_old + t - 1 of kcache and vcache [b, n, cap, d]: ughip_kv_append called twice
 * (model.rs:226-230 for keys and values), bit for bit.  Offsets and stride are multiples of 4. */
int ughip_kv_append_pair(ughip_device* dev, ughip_slice* kcache, ughip_slice* vcache,
                         const ughip_slice* x, size_t k_offset, size_t v_offset, size_t x_row_stride,
                         size_t b, size_t n, size_t cap, size_t s_old, size_t t, size_t d,
                         const ughip_slice* cos, const ughip_slice* sin, const ughip_slice* pos,
                         int interleaved);
/* Causal attention of t query positions over such caches, f32, without materialising the
 * [heads, t, s] scores (the chain model.rs:231-245: repeat, q k^T, scale, causal_mask, softmax,
 * x v, transpose, in one launch): q and dst [b, t, n_heads * d] (projection layout), k and v
 * [b, n_kv_heads, cap, d] with rows 0 .. s - 1 valid; query i sits at position s - t + i and
 * attends to keys 0 .. s - t + i; rope / rope_i is applied to q at table rows pos[0] + i when
 * cos/sin/pos are given.  t == 1 is ughip_attention_decode_rope on a cache of capacity cap;
 * t > 1 needs d = 32, 64 or 128 (UGHIP_ERR_UNSUPPORTED otherwise).  s - t == 0 and cap == s give
 * the reference's prefill.  q_offset / q_row_stride: as x_offset / x_row_stride of
 * ughip_kv_append (dst is always dense).  With d = 64 and t >= 256 both products run as six bf16
 * terms per f32 product (operands split into three bf16 terms each, f32 accumulation: the accuracy
 * of the f32 products, not their bits) over planes of K and V that a first launch writes into a
 * scratch block of the device (24 KiB per kv head and 32 keys, grown on demand). */
int ughip_attention_cached(ughip_device* dev, const ughip_slice* q, size_t q_offset,
                           size_t q_row_stride, const ughip_slice* k, const ughip_slice* v,
                           ughip_slice* dst, size_t b, size_t n_heads, size_t n_kv_heads,
                           size_t t, size_t s, size_t cap, size_t d, float scale, const ughip_slice* cos, const ughip_slice* sin,
                           const ughip_slice* pos, int interleaved);
/* ughip_attention_cached for t >= 2 query positions followed by the output projection and its residual
 * (model.rs:231-247 and 366-372): dst[b t, n] = attention(...) w^T + residual[b t, n], w a row-major [n, n_heads * d]
 * matrix stored as F32 or BF16, `product` as for ughip_linear_add_rows, dst may be residual.  The [b t, n_heads * d]
 * rows between the two stay in the device's scratch; where the kernel that takes the attention is the one on six bf16
 * terms and the projection reads planes, the attention writes its result as those planes (no f32 rows, no pass that
 * splits them).  Same results as the two entry points run one after the other. */
int ughip_attention_cached_linear_add_rows(ughip_device* dev, const ughip_slice* q, size_t q_offset,
                                           size_t q_row_stride, const ughip_slice* k,
                                           const ughip_slice* v, size_t b, size_t n_heads,
                                           size_t n_kv_heads, size_t t, size_t s, size_t cap, size_t d,
                                           float scale, const ughip_slice* cos, const ughip_slice* sin,
                                           const ughip_slice* pos, int interleaved, const ughip_slice* w,
                                           const ughip_slice* residual, ughip_slice* dst, size_t n,
                                           int product);

/* One decode position in one launch: ughip_kv_append of the k and v parts of a packed q|k|v row
 * (qkv [b, row_stride], parts at q_offset / k_offset / v_offset) into row s_old of both caches,
 * and ughip_attention_cached of the q part over rows 0 .. s_old.  The caches are read and
 * written; dst [b, n_heads * d].  d a power of two in 16..256, s_old + 1 <= cap. */
int ughip_attention_step(ughip_device* dev, const ughip_slice* qkv, size_t row_stride,
                         size_t q_offset, size_t k_offset, size_t v_offset, ughip_slice* kcache,
                         ughip_slice* vcache, ughip_slice* dst, size_t b, size_t n_heads,
                         size_t n_kv_heads, size_t s_old, size_t cap, size_t d, float scale,
                         const ughip_slice* cos, const ughip_slice* sin, const ughip_slice* pos,
                         int interleaved);

/* ---- projections of one position with their neighbours folded in (f32, one input row) ----------
 * No counterpart in the reference's device trait: there each is a matmul (lib.rs:62-70) followed
 * by the small kernels of the lazy graph.  Every product is x (k elements) against the rows of a
 * row-major [n, k] matrix, k % 4 == 0, summed in a fixed order.  x, alpha, residual and dst are F32;
 * the matrices are F32 or BF16 (all of one call alike).  A BF16 matrix gives the result of the same
 * values stored as F32 (a bf16 widens exactly; the f32 sums may run in another order, both within
 * the k * eps bound of the exact product) from half the bytes: the form a decoder keeps a bf16
 * checkpoint in, where the reference widens it at load time (ug-core/src/safetensors.rs:120-271).
 * ughip_gemv_multi: dst[0 .. n0+n1+n2) = [x W_0^T | x W_1^T | x W_2^T] for n_mats <= 3 matrices
 * (the q, k, v projections of ug-llama/src/model.rs:206-208 in one launch). */
int ughip_gemv_multi(ughip_device* dev, const ughip_slice* x, size_t n_mats,
                     const ughip_slice* const* w, const size_t* n, size_t k, ughip_slice* dst);
/* dst[c] = silu(x . gate[c]) * (x . up[c]), silu(g) = g / (1 + exp(-g)) (model.rs:99-109,160-168). */
int ughip_gemv_gate_up(ughip_device* dev, const ughip_slice* x, const ughip_slice* w_gate,
                       const ughip_slice* w_up, ughip_slice* dst, size_t n, size_t k);
/* The two above on rms_norm(x) = x / sqrt(mean(x^2) + eps) * alpha (ug-llama/src/model.rs:32-50)
 * instead of x: the norms in front of attention, the MLP and the output head.  k <= 4096. */
int ughip_rms_gemv_multi(ughip_device* dev, const ughip_slice* x, const ughip_slice* alpha, float eps,
                         size_t n_mats, const ughip_slice* const* w, const size_t* n, size_t k,
                         ughip_slice* dst);
int ughip_rms_gemv_gate_up(ughip_device* dev, const ughip_slice* x, const ughip_slice* alpha,
                           float eps, const ughip_slice* w_gate, const ughip_slice* w_up,
                           ughip_slice* dst, size_t n, size_t k);
/* dst[c] = x . w[c] + residual[c] (a projection followed by the residual add, model.rs:366-372). */
int ughip_gemv_add(ughip_device* dev, const ughip_slice* x, const ughip_slice* w,
                   const ughip_slice* residual, ughip_slice* dst, size_t n, size_t k);

/* ---- the same for several positions (a prefill) -------------------------------------------------
 * x is [m, k] F32 with contiguous rows, w a row-major [n, k] matrix stored as F32 or BF16, k % 32 == 0, n % 8 == 0;
 * m >= 9 with an F32 matrix (2 .. 8 rows are ughip_matmul's row-vector kernels), m >= 2 with a BF16 one.
 * The product is the tiled MFMA kernel's; skinny products split K over workgroups, and the fold of their
 * partial tiles (which a plain ughip_matmul of these shapes runs anyway) applies the neighbour on its way out,
 * so the residual add / SwiGLU of model.rs:99-109,160-168,366-372 costs no launch and no round trip.
 * `product` says how F32 rows meet a BF16 matrix:
 *   UGHIP_PRODUCT_F32     the matrix is widened on its way in and the f32 matrix pipe multiplies: bit for bit the F32
 *                         product on the same values (also the only choice for an F32 matrix);
 *   UGHIP_PRODUCT_BF16X3  every x is split into three bf16 terms, x = hi + mid + lo exactly to 2^-25 |x| (each term the
 *                         nearest-even bf16 of what the terms before it left), and the bf16 matrix pipe multiplies the
 *                         three planes by the matrix as it is stored: every product term is exact in f32, the sums are f32
 *                         sums in another order than the f32 pipe's, and three bf16 MFMAs replace eight times their work in
 *                         f32 ones.  Same accuracy class as the F32 product (k eps bound), not bit-identical to it.
 *                         Needs k % 64 == 0 and a BF16 matrix.  33 .. 128 rows take a kernel that reads the f32 rows as
 *                         they are and splits them on their way into LDS (no planes in memory, no launch for the
 *                         split); workgroups take runs of (column tile, k tile) units and a fold adds every tile's
 *                         partial sums in a fixed order.  Products of many rows (a prompt of several hundred
 *                         positions and more) run the planes on the one-wave-per-SIMD 16-bit kernel, whichever of the two
 *                         is priced cheaper; the terms are the same, the order of the sums is that kernel's.
 * ughip_linear_rows: dst[m, n] = x w^T.
 * ughip_linear_add_rows: dst[m, n] = x w^T + residual[m, n]; dst may be residual itself (every element is read,
 * then written, by one thread).
 * ughip_linear_swiglu_rows: w is [2n, k], gate rows first then up rows: dst[m, n] = silu(x gate^T) * (x up^T).
 * Shapes the tiled kernel does not take are refused with UGHIP_ERR_UNSUPPORTED (run the pieces instead). */
enum { UGHIP_PRODUCT_F32 = 0, UGHIP_PRODUCT_BF16X3 = 1 };
int ughip_linear_rows(ughip_device* dev, const ughip_slice* x, const ughip_slice* w, ughip_slice* dst,
                      size_t m, size_t n, size_t k, int product);
int ughip_linear_add_rows(ughip_device* dev, const ughip_slice* x, const ughip_slice* w,
                          const ughip_slice* residual, ughip_slice* dst, size_t m, size_t n, size_t k,
                          int product);
int ughip_linear_swiglu_rows(ughip_device* dev, const ughip_slice* x, const ughip_slice* w,
                             ughip_slice* dst, size_t m, size_t n, size_t k, int product);
/* The same with more of the layer folded in (model.rs:65-78 in front of 206-208 and 366-372; 160-168 whole).
 * ughip_rms_linear_rows: dst[m, n] = y w^T with y = x / sqrt(mean(x^2) + eps) * alpha (alpha: k F32 values; the
 *   division as a multiplication by the reciprocal, like ughip_rms_gemv_multi).  Where the three-term product reads
 *   planes from memory, the pass that writes them normalises the rows on its way (one launch and one round trip
 *   less); everywhere else the normalised rows go through the device's own scratch.
 * ughip_rms_mlp_rows: dst[m, n] = (silu(y gate^T) * (y up^T)) w_down^T + residual[m, n], with y as above, or y = x when
 *   alpha is NULL; w_gate_up is [2 inter, k] (gate rows, then up rows), w_down [n, inter], both of one dtype; dst may be
 *   residual.  The [m, inter] rows between the two products stay in the device's scratch: where both products read
 *   planes, the fold of the first writes them as the second one's planes (no f32 rows, no pass that splits them).
 *   ughip_last_kernel() names both products ("... -> ...").
 * Same shapes, dtypes and `product` as the entry points above (inter % 8 == 0), same results as the pieces run one
 * after the other (the norm's sum of squares is added in this library's order, not a generated kernel's).  The scratch
 * grows to m (k + 1.5 inter) floats and is kept until the device is released. */
int ughip_rms_linear_rows(ughip_device* dev, const ughip_slice* x, const ughip_slice* alpha, float eps,
                          const ughip_slice* w, ughip_slice* dst, size_t m, size_t n, size_t k,
                          int product);
int ughip_rms_mlp_rows(ughip_device* dev, const ughip_slice* x, const ughip_slice* alpha, float eps,
                       const ughip_slice* w_gate_up, const ughip_slice* w_down,
                       const ughip_slice* residual, ughip_slice* dst, size_t m, size_t n, size_t inter,
                       size_t k, int product);
/* No counterpart in the reference, no device needed: the kernel the three entry points above would launch (form 0:
 * ughip_linear_rows, 1: ughip_linear_add_rows, 2: ughip_linear_swiglu_rows) for m rows against an [n, k] matrix of
 * w_dtype, by the name ughip_last_kernel() reports after the launch -- kernel family, tile, units or K split, fold.
 * Like ughip_matmul_plan: tests pin the plans of the shapes that matter. */
int ughip_linear_rows_plan(int w_dtype, int product, int form, size_t m, size_t n, size_t k, char* buf,
                           size_t buf_len);

/* ---- greedy step on the device ----------------------------------------------------------------
 * Row `row` of logits [rows, n] (F32): the index of its largest value (the lowest index among
 * equal values -- what a host loop with `>` finds) goes to token[0] (I32; NULL: skipped) and to
 * ids[slot]; the largest value and the largest of the rest go to vals[2 * slot], vals[2 * slot + 1].
 * Lets a greedy decoder (the loop of ug-llama/src/main.rs:125-153 with argmax in place of sampling)
 * queue step i + 1 behind step i without reading the logits back in between. */
int ughip_argmax_row(ughip_device* dev, const ughip_slice* logits, size_t n, size_t row,
                     ughip_slice* token, ughip_slice* ids, ughip_slice* vals, size_t slot);

/* ---- element type conversion ------------------------------------------------------------------
 * dst[i] = (dtype of dst) src[i], same length, any pair of the five dtypes.  Replaces the host
 * loops of ug-core/src/safetensors.rs:141-271 (load_with_cast converts on the CPU, then uploads):
 * a checkpoint is uploaded in its stored dtype and widened on the device.  Same numerics as that
 * code: half::{bf16,f16}::from_f32 rounding, Rust `as` for float -> integer (truncate, saturate,
 * NaN -> 0) and for i64 -> i32 (wrap); integers reach bf16/f16 through f32. */
int ughip_convert(ughip_device* dev, const ughip_slice* src, ughip_slice* dst);

/* ---- timing on the device stream ----------------------------------------------------- */
int ughip_event_create(ughip_device* dev, ughip_event** out);
int ughip_event_record(ughip_event* ev);
int ughip_event_elapsed_ms(ughip_event* start, ughip_event* stop, float* ms); /* waits for stop */
int ughip_event_destroy(ughip_event* ev);

#ifdef __cplusplus
}
#endif
#endif /* UGHIP_H_ */
