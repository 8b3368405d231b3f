/*
 * Exposes the reference's own E4M3FN conversions
 * (runtime/src/iree/base/internal/math.h:324-362 decode, :364-460 encode,
 * instantiated at :557-560 as iree_math_f8e4m3fn_to_f32 /
 * iree_math_f32_to_f8e4m3fn) from oracle/_ref/libiree_uk_ref.so, so that the
 * oracle's f8 decode and the tests' encoder can be compared with reference
 * code, all 256 codes. The header is included from where it lies under the
 * reference checkout; nothing of it is copied here. Test infrastructure, not
 * product code.
 */
#include <stdint.h>

#include "iree/base/internal/math.h"

float ref_f8e4m3fn_to_f32(uint8_t v) { return iree_math_f8e4m3fn_to_f32(v); }
uint8_t ref_f32_to_f8e4m3fn(float v) { return iree_math_f32_to_f8e4m3fn(v); }
