/*
 * acc_prim.h -- the scalar primitives of the expression language, as device
 * functions a code generator can call by name.
 *
 * The reference's generator (CodeGen.hs:406-476 dispatching to
 * CodeGen/Arithmetic.hs) writes each primitive out as a C expression, binding
 * operands to fresh locals where they are used twice.  Here every primitive
 * that is more than one C operator is a function template over the operand
 * type, so a fragment stays an expression:
 *
 *   PrimAbs, PrimSig                Arithmetic.hs:54-84     acc_abs, acc_signum
 *   PrimQuot, PrimRem, PrimQuotRem  :90-104                 acc_quot, acc_rem, acc_quot_rem
 *   PrimIDiv, PrimMod, PrimDivMod   :106-158                acc_idiv, acc_imod, acc_div_mod
 *   PrimBShiftL/R, PrimBRotateL/R   :173-217                acc_shift_l, acc_shift_r, acc_shift_rl, acc_rotate_l, acc_rotate_r
 *   PrimRecip .. PrimLogBase        :223-279                acc_recip, acc_sin ... acc_log_base
 *   PrimTruncate/Round/Floor/Ceiling :285-295               acc_truncate<To>, acc_round<To>, acc_floor<To>, acc_ceiling<To>
 *   PrimAtan2, PrimIsNaN            :301-305                acc_atan2, acc_is_nan
 *   PrimMax, PrimMin                :330-336                acc_pmax, acc_pmin (fmax/fmin for floating types)
 *   PrimOrd, PrimChr, PrimBoolToInt, PrimFromIntegral :355-367   acc_ord, acc_chr, acc_bool_to_int, acc_from_integral<To>
 *
 * Results follow the reference's generated code, which is not always
 * Haskell's own definition: `round` is C's round (halves away from zero, not
 * to even), signum of a floating NaN is copysign(1, NaN), and the shifts are
 * unchecked (a count outside [0, bits) is undefined).
 *
 * Bool is Word8 (0 or 1), Char is Word32, Int and Word are 64 bits
 * (CodeGen/Type.hs:106-145).
 */
#ifndef ACC_PRIM_H
#define ACC_PRIM_H

/* ---- a little type machinery (no <type_traits> under hiprtc) -------------- */
template <typename T> struct acc_is_float { enum { value = 0 }; };
template <> struct acc_is_float<float> { enum { value = 1 }; };
template <> struct acc_is_float<double> { enum { value = 1 }; };
template <typename T> struct acc_is_unsigned { enum { value = (T(0) < T(-1)) }; };
template <typename T> struct acc_unsigned_of;
template <> struct acc_unsigned_of<Int8>   { typedef Word8 type; };
template <> struct acc_unsigned_of<Int16>  { typedef Word16 type; };
template <> struct acc_unsigned_of<Int32>  { typedef Word32 type; };
template <> struct acc_unsigned_of<Int64>  { typedef Word64 type; };
template <> struct acc_unsigned_of<Word8>  { typedef Word8 type; };
template <> struct acc_unsigned_of<Word16> { typedef Word16 type; };
template <> struct acc_unsigned_of<Word32> { typedef Word32 type; };
template <> struct acc_unsigned_of<Word64> { typedef Word64 type; };
template <> struct acc_unsigned_of<long>   { typedef unsigned long type; };
template <> struct acc_unsigned_of<unsigned long> { typedef unsigned long type; };
template <> struct acc_unsigned_of<char>   { typedef unsigned char type; };

template <typename A, typename B> struct acc_pair { A fst; B snd; };

/* ---- Num ------------------------------------------------------------------ */
template <typename T> ACC_DEV T acc_abs(T x)
{
  if (acc_is_float<T>::value) return (T)(sizeof(T) == 4 ? __builtin_fabsf((float)x) : __builtin_fabs((double)x));
  if (acc_is_unsigned<T>::value) return x;
  return x < T(0) ? (T)(-x) : x;
}

/* integers: (x > 0) - (x < 0), unsigned: x > 0; floating: x == 0 ? 0 : copysign(1, x) */
template <typename T> ACC_DEV T acc_signum(T x)
{
  if (acc_is_float<T>::value)
    return x == T(0) ? T(0) : (T)(sizeof(T) == 4 ? __builtin_copysignf(1.0f, (float)x) : __builtin_copysign(1.0, (double)x));
  if (acc_is_unsigned<T>::value) return (T)(x > T(0));
  return (T)((x > T(0)) - (x < T(0)));
}

/* ---- Integral -------------------------------------------------------------- */
template <typename T> ACC_DEV T acc_quot(T x, T y) { return (T)(x / y); }
template <typename T> ACC_DEV T acc_rem(T x, T y) { return (T)(x % y); }
template <typename T> ACC_DEV acc_pair<T, T> acc_quot_rem(T x, T y)
{
  acc_pair<T, T> r;
  r.fst = (T)(x / y);
  r.snd = (T)(x - y * r.fst);
  return r;
}
/* acc_idiv / acc_imod (rounding towards minus infinity) are defined with the
 * index helpers in acc_hip_device.h */
template <typename T> ACC_DEV acc_pair<T, T> acc_div_mod(T x, T y)
{
  acc_pair<T, T> r = acc_quot_rem(x, y);
  if (!acc_is_unsigned<T>::value && acc_signum(r.snd) == (T)(-acc_signum(y))) {
    r.fst = (T)(r.fst - T(1));
    r.snd = (T)(r.snd + y);
  }
  return r;
}

/* ---- Bits (counts are Int, unchecked) --------------------------------------- */
template <typename T> ACC_DEV T acc_shift_l(T x, Int64 i) { return (T)(x << i); }
template <typename T> ACC_DEV T acc_shift_r(T x, Int64 i) { return (T)(x >> i); }              /* arithmetic for signed types */
template <typename T> ACC_DEV T acc_shift_rl(T x, Int64 i)                                      /* logical */
{
  typedef typename acc_unsigned_of<T>::type U;
  return (T)((U)x >> i);
}
template <typename T> ACC_DEV T acc_rotate_l(T x, Int64 i)
{
  const Int64 bits = (Int64)(8 * sizeof(T));
  const Int64 k = i & (bits - 1);
  typedef typename acc_unsigned_of<T>::type U;
  /* the reference shifts by `bits - k` even for k == 0, which is undefined in C;
   * the rotation by zero is made explicit here */
  return k == 0 ? x : (T)(((U)x << k) | ((U)x >> (bits - k)));
}
template <typename T> ACC_DEV T acc_rotate_r(T x, Int64 i) { return acc_rotate_l(x, -i); }

/* ---- Fractional, Floating ---------------------------------------------------- */
template <typename T> ACC_DEV T acc_recip(T x) { return T(1) / x; }

#define ACC_MATH1(name, f32, f64)                                                                    \
  ACC_DEV float name(float x) { return f32(x); }                                                    \
  ACC_DEV double name(double x) { return f64(x); }
#define ACC_MATH2(name, f32, f64)                                                                    \
  ACC_DEV float name(float x, float y) { return f32(x, y); }                                        \
  ACC_DEV double name(double x, double y) { return f64(x, y); }
ACC_MATH1(acc_sin, sinf, sin)
ACC_MATH1(acc_cos, cosf, cos)
ACC_MATH1(acc_tan, tanf, tan)
ACC_MATH1(acc_asin, asinf, asin)
ACC_MATH1(acc_acos, acosf, acos)
ACC_MATH1(acc_atan, atanf, atan)
ACC_MATH1(acc_sinh, sinhf, sinh)
ACC_MATH1(acc_cosh, coshf, cosh)
ACC_MATH1(acc_tanh, tanhf, tanh)
ACC_MATH1(acc_asinh, asinhf, asinh)
ACC_MATH1(acc_acosh, acoshf, acosh)
ACC_MATH1(acc_atanh, atanhf, atanh)
ACC_MATH1(acc_exp, expf, exp)
ACC_MATH1(acc_sqrt, sqrtf, sqrt)
ACC_MATH1(acc_log, logf, log)
ACC_MATH2(acc_pow, powf, pow)
ACC_MATH2(acc_atan2, atan2f, atan2)
ACC_MATH2(acc_fmax, fmaxf, fmax)
ACC_MATH2(acc_fmin, fminf, fmin)
ACC_MATH1(acc_c_trunc, truncf, trunc)
ACC_MATH1(acc_c_round, roundf, round)
ACC_MATH1(acc_c_floor, floorf, floor)
ACC_MATH1(acc_c_ceil, ceilf, ceil)
#undef ACC_MATH1
#undef ACC_MATH2
/* logBase b y = log y / log b */
template <typename T> ACC_DEV T acc_log_base(T base, T y) { return acc_log(y) / acc_log(base); }

/* ---- RealFrac: to an integral type, through the C library function ------------ */
template <typename To, typename T> ACC_DEV To acc_truncate(T x) { return (To)acc_c_trunc(x); }
template <typename To, typename T> ACC_DEV To acc_round(T x)    { return (To)acc_c_round(x); }
template <typename To, typename T> ACC_DEV To acc_floor(T x)    { return (To)acc_c_floor(x); }
template <typename To, typename T> ACC_DEV To acc_ceiling(T x)  { return (To)acc_c_ceil(x); }

/* ---- RealFloat ----------------------------------------------------------------- */
template <typename T> ACC_DEV Word8 acc_is_nan(T x) { return (Word8)(x != x); }

/* ---- Ord: max/min (fmax/fmin on floating types: a NaN operand loses) -------------- */
ACC_DEV float  acc_pmax(float x, float y)   { return acc_fmax(x, y); }
ACC_DEV double acc_pmax(double x, double y) { return acc_fmax(x, y); }
ACC_DEV float  acc_pmin(float x, float y)   { return acc_fmin(x, y); }
ACC_DEV double acc_pmin(double x, double y) { return acc_fmin(x, y); }
template <typename T> ACC_DEV T acc_pmax(T x, T y) { return x > y ? x : y; }
template <typename T> ACC_DEV T acc_pmin(T x, T y) { return x < y ? x : y; }

/* ---- conversions ------------------------------------------------------------------ */
template <typename T> ACC_DEV Int64 acc_ord(T c) { return (Int64)c; }
template <typename T> ACC_DEV Word32 acc_chr(T i) { return (Word32)i; }
template <typename T> ACC_DEV Int64 acc_bool_to_int(T b) { return (Int64)b; }
template <typename To, typename T> ACC_DEV To acc_from_integral(T x) { return (To)x; }

#endif /* ACC_PRIM_H */
