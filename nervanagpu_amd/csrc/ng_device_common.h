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

// 32 random bits for element idx of launch `stream` under `seed`.
NG_DEV unsigned ng_rand32(unsigned seed, unsigned stream, unsigned idx)
{
    unsigned h = ng_fmix32(idx + seed * 0x9E3779B1u);
    unsigned k = stream * 0x85EBCA77u + 0xC2B2AE3Du;
    return ng_fmix32(h ^ k);
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
// subnormal results are truncated).
NG_DEV unsigned short ng_f32_to_f16_rz(float v)
{
    unsigned u    = __float_as_uint(v);
    unsigned sign = (u >> 16) & 0x8000u;
    unsigned mag  = u & 0x7FFFFFFFu;
    int      e    = (int)(mag >> 23);
    unsigned man  = mag & 0x7FFFFFu;
    unsigned h;
    if (mag > 0x7F800000u)       h = 0x7E00u;
    else if (mag == 0x7F800000u) h = 0x7C00u;
    else if (mag >= 0x47800000u) h = 0x7BFFu;
    else if (e >= 113)           h = ((unsigned)(e - 112) << 10) | (man >> 13);
    else if (e < 102)            h = 0u;
    else                         h = (man | 0x800000u) >> (unsigned)(126 - e);
    return (unsigned short)(h | sign);
}

NG_DEV unsigned short ng_sr_f16(float v, unsigned bits, unsigned r)
{
    return ng_f32_to_f16_rz(ng_sr_f32(v, bits, r));
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
