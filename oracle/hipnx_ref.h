/*
 * hipnx_ref.h -- CPU restatement of Nx.BinaryBackend for the eager tensor hot path.
 *
 * TEST INFRASTRUCTURE ONLY.  This library is the parity checker: tests, the smoke
 * check and the CPU-baseline leg of the benchmark may call it; no product code path
 * may link, load or fall back to it.
 *
 * Every function restates the algorithm of the cited reference lines
 * (paths relative to the reference tree, nx/lib/nx/...).  All pointers are host
 * memory, tensors are dense row-major native-endian (binary_backend.ex:14-15).
 *
 * Return value: 0 on success, a positive REF_E* code where Nx.BinaryBackend would
 * raise (the message is available through ref_last_error()).
 */
#ifndef HIPNX_REF_H
#define HIPNX_REF_H
#include <stdint.h>
#ifdef __cplusplus
extern "C" {
#endif

/* element types: {:u,8} .. {:f,64} (type.ex:27-48) */
enum {
  REF_U8 = 0, REF_U16 = 1, REF_U32 = 2, REF_U64 = 3,
  REF_S8 = 4, REF_S16 = 5, REF_S32 = 6, REF_S64 = 7,
  REF_F16 = 8, REF_BF16 = 9, REF_F32 = 10, REF_F64 = 11, REF_NTYPES = 12
};

/* element-wise binary callbacks (backend.ex:115-123, binary_backend.ex:649-823) */
enum {
  REF_ADD = 0, REF_SUBTRACT, REF_MULTIPLY, REF_DIVIDE, REF_POW, REF_REMAINDER, REF_ATAN2,
  REF_MIN, REF_MAX, REF_QUOTIENT, REF_BITWISE_AND, REF_BITWISE_OR, REF_BITWISE_XOR,
  REF_LEFT_SHIFT, REF_RIGHT_SHIFT, REF_EQUAL, REF_NOT_EQUAL, REF_GREATER, REF_LESS,
  REF_GREATER_EQUAL, REF_LESS_EQUAL, REF_LOGICAL_AND, REF_LOGICAL_OR, REF_LOGICAL_XOR,
  REF_NBINARY
};

/* element-wise unary callbacks (shared.ex:311-376, backend.ex:125-132) */
enum {
  REF_EXP = 0, REF_EXPM1, REF_LOG, REF_LOG1P, REF_SIGMOID, REF_COS, REF_SIN, REF_TAN,
  REF_COSH, REF_SINH, REF_TANH, REF_ACOS, REF_ASIN, REF_ATAN, REF_ACOSH, REF_ASINH,
  REF_ATANH, REF_SQRT, REF_RSQRT, REF_CBRT, REF_ERF, REF_ERFC, REF_ERF_INV,
  REF_ABS, REF_BITWISE_NOT, REF_CEIL, REF_FLOOR, REF_NEGATE, REF_ROUND, REF_SIGN,
  REF_CLZ, REF_POPCOUNT, REF_IS_NAN, REF_IS_INFINITY, REF_NUNARY
};

enum { REF_RED_SUM = 0, REF_RED_MAX = 1, REF_RED_MIN = 2, REF_RED_PRODUCT = 3 };
enum { REF_ARGMAX = 0, REF_ARGMIN = 1 };
enum { REF_TIE_LOW = 0, REF_TIE_HIGH = 1 };

enum {
  REF_OK = 0,
  REF_EARG = 1,      /* malformed call (bad dtype / op code) */
  REF_ERAISE = 2,    /* the reference raises here (ArgumentError / ArithmeticError) */
  REF_EOVERFLOW = 3  /* finite f64 does not fit the float output: the VM raises on encode */
};

const char *ref_last_error(void);
int ref_dtype_size(int dt);
void ref_set_threads(int n); /* 0 = all cores; parallel only over independent outputs */

/* binary_backend.ex:662-706: out[i] = f(l[bcast i], r[bcast i]); strides in elements,
 * 0 = broadcast axis. */
int ref_binary(int op, int l_dt, int r_dt, int out_dt, int rank, const int64_t *out_dims,
               const int64_t *l_strides, const int64_t *r_strides, const void *l, const void *r,
               void *out);

/* binary_backend.ex:827-1005 + 2432-2438 */
int ref_unary(int op, int in_dt, int out_dt, int64_t n, const void *in, void *out);

/* binary_backend.ex:2031-2076 */
int ref_as_type(int in_dt, int out_dt, int64_t n, const void *in, void *out);

/* binary_backend.ex:1315-1375 + 2342-2360; input viewed as [outer, red, inner], the fold
 * runs over `red` in increasing index order for each (outer, inner). */
int ref_reduce(int op, int in_dt, int out_dt, int64_t outer, int64_t red, int64_t inner,
               const void *in, void *out);

/* binary_backend.ex:1393-1431; same [outer, red, inner] view */
int ref_argreduce(int op, int tie, int in_dt, int out_dt, int64_t outer, int64_t red,
                  int64_t inner, const void *in, void *out);

/* binary_backend.ex:549-559 + 2362-2385 after bin_dot_transpose_contract_axes:
 * l is [batch, M, K], r is [batch, N, K], out is [batch, M, N]. */
int ref_dot(int l_dt, int r_dt, int out_dt, int64_t batch, int64_t M, int64_t N, int64_t K,
            const void *l, const void *r, void *out);

/* binary_backend.ex:280-319: out = permute(in, perm) */
int ref_transpose(int elem_bytes, int rank, const int64_t *in_dims, const int *perm,
                  const void *in, void *out);

/* binary_backend.ex:228-276: explicit broadcast via strides (0 = broadcast) */
int ref_broadcast(int elem_bytes, int rank, const int64_t *out_dims, const int64_t *in_strides,
                  const void *in, void *out);

/* binary_backend.ex:1918-1959: tensor already has the indexed axes leading.  `depth` leading
 * axes are addressed by each index tuple; slice_elems trailing elements are copied.
 * Out-of-bounds / negative index -> REF_ERAISE with the reference's message. */
int ref_gather(int elem_bytes, int rank, const int64_t *t_dims, int idx_dt, int64_t n_tuples,
               int depth, const void *t, const void *idx, void *out);

#ifdef __cplusplus
}
#endif
#endif
