// Thin extern "C" window onto the reference's own scalar format structs, compiled from the
// reference tree where it lies (-I<reference>/cccc -I<reference>/include); nothing of the
// reference is copied here.  TEST INFRASTRUCTURE ONLY: used to validate cccc_oracle.c.
// Exposes cccc/types.h: bfloat16 (:39-59), fp8_e4m3 (:63-126), fp8_e5m2 (:130-202), fp4_e2m1 (:208-274).
#include "types.h"

extern "C" {

float ref_e5m2_to_float(unsigned char b)
{
    cccc::fp8_e5m2 v;
    v.bits = b;
    return (float)v;
}

float ref_e4m3_to_float(unsigned char b)
{
    cccc::fp8_e4m3 v;
    v.bits = b;
    return (float)v;
}

float ref_fp4_to_float(unsigned char nibble) { return cccc::fp4_e2m1::to_float(nibble); }

float ref_fp4_get(const unsigned char* bytes, int i) { return cccc::fp4_e2m1::get(bytes, i); }

unsigned char ref_float_to_e5m2(float f) { return cccc::fp8_e5m2(f).bits; }

unsigned char ref_float_to_e4m3(float f) { return cccc::fp8_e4m3(f).bits; }

unsigned char ref_float_to_fp4(float f) { return cccc::fp4_e2m1::from_float(f); }

void ref_fp4_set(unsigned char* bytes, int i, float v) { cccc::fp4_e2m1::set(bytes, i, v); }

unsigned short ref_float_to_bf16_host(float f) { return cccc::bfloat16(f).bits; }

}
