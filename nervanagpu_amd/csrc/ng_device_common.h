// Device helpers shared by the compiled kernels and by the elementwise kernels
// generated at run time (this text is prepended to every hiprtc program, so it
// must not #include anything).
//
// Rounding and random-stream semantics follow nervanagpu/float_ew.py:113-321 of
// the reference: nearest-even stores by default; optional stochastic rounding
// that adds a uniform fraction of one unit-in-the-last-kept-place to the
// magnitude and truncates toward zero.  The reference's clock-seeded LFSR is
// replaced by a stateless hash of (seed, stream, element index) so results are
// reproducible.
#ifndef NG_DEVICE_COMMON_H
#define NG_DEVICE_COMMON_H

#define NG_DEV __device__ __forceinline__

NG_DEV unsigned ng_fmix32(unsigned h)
{
    h ^= h >> 16; h *= 0x85EBCA6Bu;
    h ^= h >> 13; h *= 0xC2B2AE35u;
    h ^= h >> 16;
    return h;
}

// 32 random bits for element idx of launch `stream` under `seed`.  The two keys
// depend only on (seed, stream) and are wavefront-uniform (scalar unit); per
// element the cost is two 32-bit multiplies and a few shifts/xors.  For fixed
// keys the map idx -> bits is a bijection.
NG_DEV unsigned ng_rand32(unsigned seed, unsigned stream, unsigned idx)
{
    const unsigned ka = ng_fmix32(seed ^ 0x9E3779B9u) + stream * 0x85EBCA77u;
    const unsigned kb = ng_fmix32(stream + 0xC2B2AE3Du) ^ seed;
    unsigned x = idx + ka;
    x ^= x >> 16; x *= 0x7FEB352Du;
    x ^= kb;
    x ^= x >> 15; x *= 0x846CA68Bu;
    x ^= x >> 16;
    return x;
}

// Random word for the fp16 stochastic rounding of element idx: fp16 needs at
// most 16 random bits, so elements 2i and 2i+1 share the draw of index i; the
// even element uses its high half, the odd one its low half.
NG_DEV unsigned ng_rand_sr16(unsigned seed, unsigned stream, unsigned idx)
{
    const unsigned h = ng_rand32(seed, stream, idx >> 1);
    return (idx & 1u) ? (h << 16) : h;
}

// uniform in [0,1]: nearest-even convert of 32 bits, times 2^-32
NG_DEV float ng_frand(unsigned seed, unsigned stream, unsigned idx)
{
    return __uint2float_rn(ng_rand32(seed, stream, idx)) * 2.3283064365386963e-10f;
}

// magnitude += uniform fraction of one unit at `bits` kept mantissa bits, then
// truncate to `bits` bits (round toward zero, never to infinity).
NG_DEV float ng_sr_f32(float v, unsigned bits, unsigned r)
{
    unsigned u    = __float_as_uint(v);
    unsigned d    = 23u - bits;
    unsigned mask = 0xFFFFFFFFu << d;
    unsigned sign = u & 0x80000000u;
    unsigned mag  = u & 0x7FFFFFFFu;
    unsigned m2   = (mag + (r >> (32u - d))) & mask;
    if (m2 >= 0x7F800000u) m2 = 0x7F7FFFFFu & mask;
    if (mag >= 0x7F800000u) m2 = mag;
    return __uint_as_float(sign | m2);
}

// fp32 -> fp16 bits, round toward zero (overflow saturates at 65504,
// subnormal results are truncated): the hardware pack-convert does exactly this.
NG_DEV unsigned short ng_f32_to_f16_rz(float v)
{
    typedef _Float16 ng_half2_t __attribute__((ext_vector_type(2)));
    const ng_half2_t h = __builtin_bit_cast(ng_half2_t, __builtin_amdgcn_cvt_pkrtz(v, 0.0f));
    const _Float16 lo = h[0];
    return __builtin_bit_cast(unsigned short, lo);
}

// fp32 -> fp16 bits with stochastic rounding at `bits` (1..10) mantissa bits.
// Finite magnitudes are first clamped to the largest fp16 value, so the random
// increment can never carry into the infinity pattern; the final truncating
// convert then drops whatever lies below the fp16 grid.
NG_DEV unsigned short ng_sr_f16(float v, unsigned bits, unsigned r)
{
    const unsigned u    = __float_as_uint(v);
    const unsigned d    = 23u - bits;
    const unsigned mag  = u & 0x7FFFFFFFu;
    unsigned m2 = (min(mag, 0x477FE000u) + (r >> (32u - d))) & (0xFFFFFFFFu << d);
    m2 = (mag >= 0x7F800000u) ? mag : m2;
    return ng_f32_to_f16_rz(__uint_as_float((u & 0x80000000u) | m2));
}

// The same rounding when all 10 mantissa bits of fp16 are kept, in three
// operations (add, compare, select).  The truncating convert drops exactly the
// bits the mask would clear, and the sign bit sits above every carry, so the
// increment is added to the signed pattern as it is.  Magnitudes within 2^13
// patterns of the largest finite fp32 could carry into the infinity pattern:
// they, infinities and NaNs are passed on unchanged (the convert saturates the
// former at 65504, as the clamp did, whatever was added).  Returns the fp32
// value whose truncating convert is the result.
NG_DEV float ng_sr10_bump(float v, unsigned r13)
{
    const float bumped = __uint_as_float(__float_as_uint(v) + r13);
    return (__builtin_fabsf(v) < __uint_as_float(0x7F7FE000u)) ? bumped : v;
}

// Two neighbouring elements sharing the draw h (even element: its high half,
// odd element: its low half, as in ng_rand_sr16) -> packed pair of fp16 bits.
NG_DEV unsigned ng_sr10_f16x2(float v_even, float v_odd, unsigned h)
{
    typedef _Float16 ng_half2_t __attribute__((ext_vector_type(2)));
    const ng_half2_t p = __builtin_bit_cast(
        ng_half2_t, __builtin_amdgcn_cvt_pkrtz(ng_sr10_bump(v_even, h >> 19), ng_sr10_bump(v_odd, (h >> 3) & 0x1FFFu)));
    return __builtin_bit_cast(unsigned, p);
}

// nearest-even fp32 -> fp16 bits
NG_DEV unsigned short ng_f32_to_f16_rn(float v)
{
    _Float16 h = (_Float16)v;
    return *reinterpret_cast<unsigned short*>(&h);
}

NG_DEV float ng_f16_to_f32(unsigned short b)
{
    _Float16 h = *reinterpret_cast<_Float16*>(&b);
    return (float)h;
}

// round-half-even + saturate to an integer range (NaN -> 0)
NG_DEV float ng_rint_sat(float v, float lo, float hi)
{
    float r = rintf(v);
    r = (r != r) ? 0.0f : r;
    return fminf(fmaxf(r, lo), hi);
}

#endif  // NG_DEVICE_COMMON_H
