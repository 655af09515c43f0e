/*
 * pccl_oracle.h -- CPU restatement of the reduce-copy semantics.
 *
 * TEST INFRASTRUCTURE ONLY.  This library is the checker the HIP path is
 * compared with; it is never part of the shipped product path.  Only the test
 * suite, the smoke check and the benchmark's cpu_baseline leg may load it.
 *
 * What it restates.  The reference tree (napplesty/pccl) holds no arithmetic
 * for this path: include/plugins/cpu_executor/executor.h and
 * include/plugins/cuda_executor/executor.h are empty files and
 * csrc/engine.cc:102-104 (Engine::regOp) is an empty body.  What the reference
 * does fix is the shape of the data:
 *   - the operand descriptor ChunkMeta{dtype_, addr_, num_elems_}
 *     (include/base/chunk.h:10-14),
 *   - the dtype / pack matrix f32, i32, f16, bf16 with 16-byte packs
 *     (include/plugins/cuda_executor/utils/vector_datatype.h:55-80),
 *   - the reduction set: N-input "add" and broadcast store
 *     (include/plugins/cuda_executor/utils/multimem.h:12-127),
 *   - the IR op kinds COPY / REDUCE (pccl/lang/chunk.py:6-10) and the DAG
 *     ordering rule (pccl/lang/utils/graph.py:94-112).
 * The arithmetic rules implemented here are therefore this build's definition:
 *
 *   out[j][i] = cvt_T( fold_op( up(in[0][i]), ..., up(in[n_in-1][i]) ) )
 *
 *   - strict left fold in input-index order, no tree, no FMA contraction;
 *   - accumulator float for f32/bf16/f16/f8, double for f64, uint32 two's-complement for
 *     i32 and u32 (u32 differs from i32 only in min / max comparing unsigned);
 *   - bf16/f16 are widened exactly, rounded to nearest-even ONCE at the end,
 *     NaN becomes a quiet NaN, overflow becomes +-inf;
 *   - min is (b < a ? b : a), max is (a < b ? b : a);
 *   - n_in == 1 is COPY and moves bytes unchanged.
 *
 * Parity status of each function:
 *   pccl_oracle_f32_to_bf16 / bf16_to_f32 / f32_to_f16 / f16_to_f32
 *       pinned: exhaustive 2^16 widening and a committed fixture of
 *       round-to-nearest-even cases checked against numpy/torch conversions
 *       (tests/test_oracle_convert.py).
 *   pccl_oracle_f32_to_e4m3 / e4m3_to_f32 / f32_to_e5m2 / e5m2_to_f32
 *       pinned: all 256 encodings widened against torch.float8_e4m3fn / float8_e5m2;
 *       narrowing against torch for every float that does not overflow (torch does
 *       not saturate) and for infinities, and against the closed form for the
 *       saturating range (tests/test_oracle_convert.py).
 *   pccl_oracle_reduce_copy
 *       pinned against the mathematics: exact-rational brute force with one
 *       rounding per step (binary32 and binary64), fold-order-sensitive known
 *       answers, int32 / uint32 wraparound closed forms in Python integers
 *       (tests/test_oracle_reduce.py).
 *       Parity against the reference's own arithmetic is UNPINNED because the
 *       reference contains none (no kernels, no tests, no golden vectors).
 *   pccl_oracle_topo_sort
 *       pinned by hand-worked DAGs following pccl/lang/utils/graph.py:94-112
 *       and the invariant that every dependency precedes its dependent.
 */
#ifndef PCCL_ORACLE_H
#define PCCL_ORACLE_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* dtype / compute / primitive codes: same numbering as include/pccl_hip.h. */
enum { PCCL_ORACLE_F32 = 0, PCCL_ORACLE_I32 = 1, PCCL_ORACLE_BF16 = 2, PCCL_ORACLE_F16 = 3,
       PCCL_ORACLE_F8E4M3 = 4, PCCL_ORACLE_F8E5M2 = 5, PCCL_ORACLE_F64 = 6, PCCL_ORACLE_U32 = 7 };
enum { PCCL_ORACLE_SUM = 0, PCCL_ORACLE_PROD = 1, PCCL_ORACLE_MIN = 2, PCCL_ORACLE_MAX = 3 };

/* ---- conversions -------------------------------------------------------- */
uint16_t pccl_oracle_f32_to_bf16(float x);
float pccl_oracle_bf16_to_f32(uint16_t h);
uint16_t pccl_oracle_f32_to_f16(float x);
float pccl_oracle_f16_to_f32(uint16_t h);
/* 8-bit floats of include/plugins/cuda_executor/utils/vector_datatype.h:11-16,75-80:
 * e4m3 = OCP E4M3FN (bias 7, no infinity, NaN = S.1111.111, largest finite 448),
 * e5m2 = OCP E5M2 (bias 15, IEEE-like infinities and NaNs, largest finite 57344).
 * Narrowing rounds to nearest even; a FINITE value beyond the largest finite one SATURATES
 * to it (what the __nv_fp8_* types the reference names do when built from float); a true
 * infinity stays infinite in e5m2 and becomes NaN in e4m3, which has none (no fold of e4m3
 * operands can produce one); NaN becomes S.1111.111 / S.11111.11 here, and any NaN encoding
 * of the format counts as equal to it. */
uint8_t pccl_oracle_f32_to_e4m3(float x);
float pccl_oracle_e4m3_to_f32(uint8_t h);
uint8_t pccl_oracle_f32_to_e5m2(float x);
float pccl_oracle_e5m2_to_f32(uint8_t h);
/* bulk forms used by the tests: dtype is BF16 or F16 (uint16_t storage) */
void pccl_oracle_narrow_array(int dtype, const float *src, uint16_t *dst, long n);
void pccl_oracle_widen_array(int dtype, const uint16_t *src, float *dst, long n);
/* dtype is F8E4M3 or F8E5M2 (uint8_t storage) */
void pccl_oracle_narrow_array8(int dtype, const float *src, uint8_t *dst, long n);
void pccl_oracle_widen_array8(int dtype, const uint8_t *src, float *dst, long n);

/* ---- the reduce-copy itself --------------------------------------------- */
/* Returns 0 on success, -1 on a bad argument.  Operand element type follows
 * ChunkMeta::dtype_ (include/base/chunk.h:10-14); all operands share it. */
int pccl_oracle_reduce_copy(int dtype, int op, const void *const *ins, int n_in,
                            void *const *outs, int n_out, long count);
/* Same result, element range split into contiguous slices over nthreads
 * POSIX threads (used only to time a multi-core CPU baseline). */
int pccl_oracle_reduce_copy_mt(int dtype, int op, const void *const *ins, int n_in,
                               void *const *outs, int n_out, long count, int nthreads);

/* ---- op lists ------------------------------------------------------------ */
typedef struct pccl_oracle_op {
  int dtype;
  int op;
  int n_in;
  int n_out;
  const void *ins[8];
  void *outs[8];
  long count;
} pccl_oracle_op;

/* Executes ops[order[0]], ops[order[1]], ... sequentially (order == NULL
 * means 0..n_ops-1).  Returns 0 or -1. */
int pccl_oracle_run_ops(const pccl_oracle_op *ops, int n_ops, const int *order);

/* Restates DirectedGraph.topological_sort (pccl/lang/utils/graph.py:94-112):
 * depth-first search visiting nodes in id order and successors in edge
 * insertion order, result is the reverse post-order.  Returns 0, or -1 if the
 * graph has a cycle (graph.py:95-96 raises ValueError) or an edge names a node
 * outside [0, n_nodes). */
int pccl_oracle_topo_sort(int n_nodes, const int *edge_src, const int *edge_dst,
                          int n_edges, int *order_out);

/* ---- seeded inputs -------------------------------------------------------- */
/* Counter-based generator: value i of stream `stream` under `seed` depends on
 * nothing else, so buffers can be produced in any order or in parallel. */
uint64_t pccl_oracle_rng_u64(uint64_t seed, uint64_t stream, uint64_t index);
void pccl_oracle_fill_uniform_f32(float *dst, long n, uint64_t seed, uint64_t stream,
                                  float lo, float hi);
/* N(mean, sigma) by Box-Muller in double, kept (F64) or narrowed to dtype
 * (F32, BF16, F16, F8E4M3, F8E5M2) with round-to-nearest-even. */
void pccl_oracle_fill_normal(void *dst, int dtype, long n, uint64_t seed, uint64_t stream,
                             double mean, double sigma);
/* Values first .. first + n - 1 of the same stream into dst[0 .. n): slices of one buffer can be
 * filled by several threads. */
void pccl_oracle_fill_normal_at(void *dst, int dtype, long first, long n, uint64_t seed, uint64_t stream,
                                double mean, double sigma);
/* uniform integers in [lo, hi] */
void pccl_oracle_fill_int32(int32_t *dst, long n, uint64_t seed, uint64_t stream,
                            int32_t lo, int32_t hi);

#ifdef __cplusplus
}
#endif
#endif
