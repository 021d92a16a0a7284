/*
 * acc_hip_device.h -- device-side support for the gfx950 skeleton templates.
 *
 * Takes the place of the reference's device headers:
 *   cubits/accelerate_cuda_type.h:22-30      fixed-width element typedefs
 *   cubits/accelerate_cuda_function.h:28-193 atomicCAS wrappers, reinterpret, shfl_up/xor
 * but is written for 64-lane wavefronts: cross-lane traffic uses DPP row
 * operations and readlane, not 32-wide shuffles, and nothing relies on
 * warp-synchronous shared memory.
 *
 * Every skeleton instance is one translation unit compiled at run time:
 *     <generated #defines: ACC_ELT, ACC_ENV_PARAMS, ACC_GET, ACC_COMBINE, ...>
 *     #include "acc_hip_device.h"
 *     #include "skel_<name>.h"
 * User fragments are pasted as macros inside the kernel body so that they can
 * name the kernel's array parameters (arrIn0_0, shIn0_0, ...) directly.
 */
#ifndef ACC_HIP_DEVICE_H
#define ACC_HIP_DEVICE_H

/* element types, named as the Accelerate code generator names them
 * (CodeGen/Type.hs:106-145: Bool is Word8, Char is Word32, Int is Int64) */
typedef signed char        Int8;
typedef short              Int16;
typedef int                Int32;
typedef long long          Int64;
typedef unsigned char      Word8;
typedef unsigned short     Word16;
typedef unsigned int       Word32;
typedef unsigned long long Word64;
typedef signed char        int8_t;
typedef short              int16_t;
typedef int                int32_t;
typedef long long          int64_t;
typedef unsigned char      uint8_t;
typedef unsigned short     uint16_t;
typedef unsigned int       uint32_t;
typedef unsigned long long uint64_t;

#define ACC_WAVE 64
#define ACC_DEV  __device__ __forceinline__
#define ACC_IGNORE (-1LL)          /* linear image of the index `ignore` */

/* Haskell-flavoured integer helpers the scalar code generator relies on
 * (CodeGen/Arithmetic.hs:103-134: div/mod round towards minus infinity) */
template <typename T> ACC_DEV T acc_idiv(T x, T y) { T q = x / y; return ((x % y != 0) && ((x < 0) != (y < 0))) ? q - 1 : q; }
template <typename T> ACC_DEV T acc_imod(T x, T y) { T r = x % y; return ((r != 0) && ((r < 0) != (y < 0))) ? r + y : r; }
template <typename T> ACC_DEV T acc_min(T x, T y) { return x < y ? x : y; }
template <typename T> ACC_DEV T acc_max(T x, T y) { return x > y ? x : y; }

ACC_DEV int acc_lane() { return (int)__builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, 0u)); }

/* ------------------------------------------------------------------------ */
/* word-wise movement of arbitrary trivially copyable values across lanes    */

template <typename T> struct acc_words { enum { n = (sizeof(T) + 3) / 4 }; };

/* DPP control words (GFX9 encoding) */
#define ACC_DPP_ROW_SHL(n)   (0x100 + (n))
#define ACC_DPP_ROW_SHR(n)   (0x110 + (n))
#define ACC_DPP_WAVE_SHR1    0x138
#define ACC_DPP_ROW_BCAST15  0x142
#define ACC_DPP_ROW_BCAST31  0x143

/* result lane i = src of the lane the control selects; lanes with no source
 * (or masked out) keep `old` */
template <int CTRL, int ROW_MASK, typename T>
ACC_DEV T acc_dpp(const T &old, const T &src)
{
  unsigned int o[acc_words<T>::n], s[acc_words<T>::n];
  o[acc_words<T>::n - 1] = 0; s[acc_words<T>::n - 1] = 0;
  __builtin_memcpy(o, &old, sizeof(T));
  __builtin_memcpy(s, &src, sizeof(T));
#pragma unroll
  for (int w = 0; w < acc_words<T>::n; ++w)
    o[w] = (unsigned int)__builtin_amdgcn_update_dpp((int)o[w], (int)s[w], CTRL, ROW_MASK, 0xf, false);
  T r;
  __builtin_memcpy(&r, o, sizeof(T));
  return r;
}

template <typename T>
ACC_DEV T acc_readlane(const T &v, int lane)
{
  unsigned int s[acc_words<T>::n];
  s[acc_words<T>::n - 1] = 0;
  __builtin_memcpy(s, &v, sizeof(T));
#pragma unroll
  for (int w = 0; w < acc_words<T>::n; ++w)
    s[w] = (unsigned int)__builtin_amdgcn_readlane((int)s[w], lane);
  T r;
  __builtin_memcpy(&r, s, sizeof(T));
  return r;
}

/* ------------------------------------------------------------------------ */
/* Values that may be absent.  Accelerate's combining functions come with no
 * identity element (fold1, scanl1, permute), so "nothing here yet" is carried
 * as a flag and the operator is lifted: absent (+) x = x.                    */
template <typename T> struct acc_opt { T v; int ok; };

template <typename T> ACC_DEV acc_opt<T> acc_some(const T &v) { acc_opt<T> r; r.v = v; r.ok = 1; return r; }
template <typename T> ACC_DEV acc_opt<T> acc_none() { acc_opt<T> r; r.v = T(); r.ok = 0; return r; }

template <typename T, typename F>
struct acc_lifted {
  F f;
  ACC_DEV acc_lifted(F f_) : f(f_) {}
  ACC_DEV acc_opt<T> operator()(const acc_opt<T> &a, const acc_opt<T> &b) const
  {
    acc_opt<T> r;
    r.ok = a.ok | b.ok;
    r.v  = (a.ok && b.ok) ? f(a.v, b.v) : (a.ok ? a.v : b.v);
    return r;
  }
};
template <typename T, typename F> ACC_DEV acc_lifted<T, F> acc_lift(F f) { return acc_lifted<T, F>(f); }

/* ------------------------------------------------------------------------ */
/* wave64 inclusive scan, order preserving: lane i ends with
 * x_0 (+) x_1 (+) ... (+) x_i, `op(earlier, later)`.  Kogge-Stone inside each
 * 16-lane DPP row, then the two row-broadcast steps stitch the four rows.    */
template <typename T, typename F>
ACC_DEV T acc_wave_scan(T x, F op, int lane)
{
  const int r = lane & 15;
  T t;
  t = acc_dpp<ACC_DPP_ROW_SHR(1), 0xf>(x, x); if (r >= 1) x = op(t, x);
  t = acc_dpp<ACC_DPP_ROW_SHR(2), 0xf>(x, x); if (r >= 2) x = op(t, x);
  t = acc_dpp<ACC_DPP_ROW_SHR(4), 0xf>(x, x); if (r >= 4) x = op(t, x);
  t = acc_dpp<ACC_DPP_ROW_SHR(8), 0xf>(x, x); if (r >= 8) x = op(t, x);
  t = acc_dpp<ACC_DPP_ROW_BCAST15, 0xa>(x, x); if (lane & 16) x = op(t, x);
  t = acc_dpp<ACC_DPP_ROW_BCAST31, 0xc>(x, x); if (lane & 32) x = op(t, x);
  return x;
}

/* value of the previous lane (lane 0 keeps its own value: caller masks it) */
template <typename T> ACC_DEV T acc_wave_shift_up1(const T &x) { return acc_dpp<ACC_DPP_WAVE_SHR1, 0xf>(x, x); }

/* wave64 reduction, order preserving; the result is uniform across the wave */
template <typename T, typename F>
ACC_DEV T acc_wave_reduce(T x, F op)
{
  T t;
  t = acc_dpp<ACC_DPP_ROW_SHL(1), 0xf>(x, x); x = op(x, t);
  t = acc_dpp<ACC_DPP_ROW_SHL(2), 0xf>(x, x); x = op(x, t);
  t = acc_dpp<ACC_DPP_ROW_SHL(4), 0xf>(x, x); x = op(x, t);
  t = acc_dpp<ACC_DPP_ROW_SHL(8), 0xf>(x, x); x = op(x, t);
  /* lane 0 of each row now holds its row; lanes whose partner fell off the
   * row combined with themselves and are ignored */
  T r0 = acc_readlane(x, 0), r1 = acc_readlane(x, 16), r2 = acc_readlane(x, 32), r3 = acc_readlane(x, 48);
  return op(op(r0, r1), op(r2, r3));
}

/* the same over each row of 16 lanes on its own, order preserving; the result is in the row's first lane */
template <typename T, typename F>
ACC_DEV T acc_row_reduce(T x, F op)
{
  T t;
  t = acc_dpp<ACC_DPP_ROW_SHL(1), 0xf>(x, x); x = op(x, t);
  t = acc_dpp<ACC_DPP_ROW_SHL(2), 0xf>(x, x); x = op(x, t);
  t = acc_dpp<ACC_DPP_ROW_SHL(4), 0xf>(x, x); x = op(x, t);
  t = acc_dpp<ACC_DPP_ROW_SHL(8), 0xf>(x, x); x = op(x, t);
  return x;
}

/* ------------------------------------------------------------------------ */
/* atomics on 4- and 8-byte elements of any type, by compare-and-swap on the
 * bit pattern (replaces cubits/accelerate_cuda_function.h:28-114)            */
template <int N> struct acc_bits;
template <> struct acc_bits<4> { typedef unsigned int type; };
template <> struct acc_bits<8> { typedef unsigned long long type; };

template <typename T, typename F>
ACC_DEV void acc_atomic_rmw(T *addr, const T &x, F combine_new_old)
{
  typedef typename acc_bits<sizeof(T)>::type B;
  B *p = (B *)addr;
  B old = *p, assumed;
  do {
    assumed = old;
    T cur, nxt;
    __builtin_memcpy(&cur, &assumed, sizeof(T));
    nxt = combine_new_old(x, cur);
    B nb;
    __builtin_memcpy(&nb, &nxt, sizeof(T));
    old = atomicCAS(p, assumed, nb);
  } while (old != assumed);
}

/* Workgroups are handed to the 8 compute dies (XCDs) round-robin, and each die
 * has its own L2.  This renumbering gives every die one contiguous run of the
 * logical work items instead of every eighth one, so that neighbours in the
 * logical order -- which share halo rows, or continue each other's memory
 * stream -- also share an L2.  It is a bijection on [0, gridDim.x) whatever
 * the hardware really does; only the locality depends on the assumption.    */
#define ACC_XCDS 8
ACC_DEV Int64 acc_xcd_contiguous_block()
{
  const Int64 n = gridDim.x, b = blockIdx.x;
  const Int64 q = n / ACC_XCDS, r = n % ACC_XCDS;
  const Int64 xcd = b % ACC_XCDS, i = b / ACC_XCDS;
  return xcd * q + acc_min<Int64>(xcd, r) + i;
}

/* Waits of one workgroup for another are bounded: after ACC_SPIN_LIMIT polls the waiting lane gives up, says so
 * in the context's status block -- words in host memory that the host looks at whenever it synchronises -- and
 * carries on with whatever value it has, so that every kernel ends.  Nothing of that launch's result is to be
 * trusted then.  A healthy run never writes here.  Word numbers as in the host's StatusWord. */
#ifndef ACC_SPIN_LIMIT
#define ACC_SPIN_LIMIT (1 << 22)
#endif
#define ACC_STATUS_SCAN_LOOKBACK 0
#define ACC_STATUS_FOLD_COLLECT  1
#define ACC_STATUS_PERMUTE_LOCK  2
ACC_DEV void acc_report(unsigned int *status, const int word)
{
  if (status) __hip_atomic_store(status + word, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
}

/* A value handed from one workgroup to another without fences: it is cut into
 * 4-byte pieces and every piece travels in a 64-bit word of its own together
 * with the tag of the launch, written and read with relaxed device-scope
 * atomics (write-through, no cache-wide write-back or invalidate as a
 * release/acquire pair costs).  The value has arrived when all its words
 * carry the tag.                                                            */
template <typename T>
struct acc_tagged {
  static constexpr int NW = (int)((sizeof(T) + 3) / 4);
  unsigned long long *d;
  ACC_DEV void put(unsigned int slot, unsigned int tag, const T &v) const
  {
    unsigned int b[NW] = {};
    __builtin_memcpy(b, &v, sizeof(T));
#pragma unroll
    for (int k = 0; k < NW; ++k)
      __hip_atomic_store(d + (Int64)slot * NW + k, ((unsigned long long)tag << 32) | b[k], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
  /* (bounded: a word that does not turn up within ACC_SPIN_LIMIT polls is taken as it is and reported) */
  ACC_DEV T wait(unsigned int slot, unsigned int tag, unsigned int *status) const
  {
    unsigned int b[NW];
    int polls = 0;
#pragma unroll
    for (int k = 0; k < NW; ++k) {
      unsigned long long w;
      while ((unsigned int)((w = __hip_atomic_load(d + (Int64)slot * NW + k, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)) >> 32) != tag &&
             polls < ACC_SPIN_LIMIT) {
        ++polls;
        __builtin_amdgcn_s_sleep(1);
      }
      b[k] = (unsigned int)w;
    }
    if (polls >= ACC_SPIN_LIMIT) acc_report(status, ACC_STATUS_FOLD_COLLECT);
    T v;
    __builtin_memcpy(&v, b, sizeof(T));
    return v;
  }
};

/* ACC_GUARDED: the kernels of an instance built for the body or the predicate of an array-level loop take one more
 * parameter, a word in device memory that says whether the loop is still running, and return at once when it is
 * zero (a NULL pointer means no loop).  The host can then enqueue several iterations ahead without knowing how
 * many will be wanted: the ones past the end do nothing.  The test is one scalar load per wave; instances built
 * without the flag carry neither the parameter nor the test.                                                  */
#ifndef ACC_GUARDED
#define ACC_GUARDED 0
#endif
#if ACC_GUARDED
#define ACC_GUARD_PARAM , const unsigned int *__restrict__ acc_guard
#define ACC_GUARD_CHECK if (acc_guard != (const unsigned int *)0 && *acc_guard == 0u) return;
#else
#define ACC_GUARD_PARAM
#define ACC_GUARD_CHECK
#endif

/* Keep a value where it was computed.  The compiler otherwise moves the tail of a long dependent chain -- load an
 * index, gather through it, multiply -- down to its first use, past whatever stands in between, so that its memory
 * round trips start only there and are waited for one after the other. */
template <typename T> ACC_DEV void acc_pin(T &v)
{
  unsigned int w[acc_words<T>::n];
  w[acc_words<T>::n - 1] = 0;
  __builtin_memcpy(w, &v, sizeof(T));
#pragma unroll
  for (int k = 0; k < acc_words<T>::n; ++k) asm volatile("" : "+v"(w[k]));
  __builtin_memcpy(&v, w, sizeof(T));
}

/* a compile-time flag passed as a value (to generic lambdas) */
template <bool B> struct acc_bool { static constexpr bool value = B; };

/* the bulk stores of a streaming skeleton (a result that this kernel never
 * reads back): non-temporal if the generator asks for it */
#ifndef ACC_NT_STORE
#define ACC_NT_STORE 0
#endif
template <typename T> ACC_DEV void acc_store(T *p, const T &v)
{
#if ACC_NT_STORE
  __builtin_nontemporal_store(v, p);
#else
  *p = v;
#endif
}

/* Loads and stores that meet at device scope: relaxed atomics, which go past the
 * caches that are not coherent across the compute dies instead of asking for a
 * cache-wide invalidate or write-back.  Any size: in pieces of 8, 4, 2 or 1 bytes
 * (an element is only ever accessed this way under a lock, so the pieces need
 * not be atomic together).                                                   */
template <int N> struct acc_piece;
template <> struct acc_piece<8> { typedef unsigned long long type; };
template <> struct acc_piece<4> { typedef unsigned int type; };
template <> struct acc_piece<2> { typedef unsigned short type; };
template <> struct acc_piece<1> { typedef unsigned char type; };
template <typename T> struct acc_piece_of {
  static constexpr int N = (sizeof(T) % 8 == 0 && alignof(T) >= 8) ? 8 : (sizeof(T) % 4 == 0 && alignof(T) >= 4) ? 4 :
                           (sizeof(T) % 2 == 0 && alignof(T) >= 2) ? 2 : 1;
  typedef typename acc_piece<N>::type type;
  static constexpr int COUNT = (int)(sizeof(T) / N);
};
template <typename T> ACC_DEV T acc_load_device(const T *p)
{
  typedef typename acc_piece_of<T>::type P;
  P b[acc_piece_of<T>::COUNT];
#pragma unroll
  for (int k = 0; k < acc_piece_of<T>::COUNT; ++k)
    b[k] = __hip_atomic_load((const P *)p + k, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  T v;
  __builtin_memcpy(&v, b, sizeof(T));
  return v;
}
template <typename T> ACC_DEV void acc_store_device(T *p, const T &v)
{
  typedef typename acc_piece_of<T>::type P;
  P b[acc_piece_of<T>::COUNT];
  __builtin_memcpy(b, &v, sizeof(T));
#pragma unroll
  for (int k = 0; k < acc_piece_of<T>::COUNT; ++k)
    __hip_atomic_store((P *)p + k, b[k], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

/* A read of an array element that will not be needed again (a manifest input
 * consumed once, in index order).  It is marked non-temporal so that it does
 * not evict data that IS reused -- a gathered vector, a small table -- from
 * the L2.  The code generator uses it for linear reads next to indirect ones. */
#ifndef ACC_STREAM_POLICY
#define ACC_STREAM_POLICY 1
#endif
template <typename T> ACC_DEV T acc_stream(const T *p, const Int64 ix)
{
#if ACC_STREAM_POLICY == 0
  return p[ix];
#elif ACC_STREAM_POLICY == 2 || ACC_STREAM_POLICY == 3
  typedef typename acc_piece_of<T>::type P;
  P b[acc_piece_of<T>::COUNT];
#pragma unroll
  for (int k = 0; k < acc_piece_of<T>::COUNT; ++k)
    b[k] = __hip_atomic_load((const P *)(p + ix) + k, __ATOMIC_RELAXED, ACC_STREAM_POLICY == 2 ? __HIP_MEMORY_SCOPE_AGENT : __HIP_MEMORY_SCOPE_SYSTEM);
  T v;
  __builtin_memcpy(&v, b, sizeof(T));
  return v;
#else
  return __builtin_nontemporal_load(p + ix);
#endif
}

/* row-major index helpers (CodeGen/Base.hs:193-218): shapes and indices are
 * listed innermost dimension LAST, e.g. acc_to_index2(h, w, y, x)            */
ACC_DEV Int64 acc_to_index2(Int64, Int64 w, Int64 y, Int64 x) { return y * w + x; }
ACC_DEV Int64 acc_to_index3(Int64, Int64 h, Int64 w, Int64 z, Int64 y, Int64 x) { return (z * h + y) * w + x; }

/* The multi-index of a linear index (cfromIndex, CodeGen/Base.hs:207-218): acc_from_index<R>({ext_0, ..., ext_<R-1>},
 * ix).i[d], outermost dimension first.  An index into fewer than 2^31 elements is taken apart in 32 bits -- a 64-bit
 * division by an extent that is not a literal is a hundred instructions, the 32-bit one a quarter of that; the test
 * is the same in every lane.  (A generator that knows the extents writes them as literals instead, and the divisions
 * become multiplications.) */
template <int R> struct acc_multi_index { Int64 i[R]; };
template <int R>
ACC_DEV acc_multi_index<R> acc_from_index(const Int64 (&sh)[R], const Int64 ix)
{
  acc_multi_index<R> m;
  Int64 count = 1;
#pragma unroll
  for (int d = 0; d < R; ++d) count *= sh[d];
  if (count > 0 && count < (Int64)0x7fffffff) {
    unsigned int rest = (unsigned int)ix;
#pragma unroll
    for (int d = R - 1; d > 0; --d) {
      const unsigned int ext = (unsigned int)sh[d];
      m.i[d] = (Int64)(rest % ext);
      rest /= ext;
    }
    m.i[0] = (Int64)rest;
  } else {
    Int64 rest = ix;
#pragma unroll
    for (int d = R - 1; d > 0; --d) {
      const Int64 ext = sh[d] > 0 ? sh[d] : 1;
      m.i[d] = rest % ext;
      rest /= ext;
    }
    m.i[0] = rest;
  }
  return m;
}

/* the scalar primitives of the expression language */
#include "acc_prim.h"

#endif /* ACC_HIP_DEVICE_H */
