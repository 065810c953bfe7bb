// Host build (g++) of the LDS index arithmetic for the bank-model tests: exports the very
// functions the kernels use, one C entry point that fills the 64 per-lane byte addresses
// of a named access.
#include <cstring>

#include "lds_index_math.hpp"

extern "C" int bsa_lds_access(const char *name, int permuted, int arg0, int arg1, int arg2, int *addr64)
{
    using namespace bsa;
    for (int lane = 0; lane < 64; ++lane) {
        int a;
        if (!strcmp(name, "put_kc")) a = put_kc_addr(permuted, lane, arg0);
        else if (!strcmp(name, "get_kc")) a = get_kc_addr(lane, arg0);
        else if (!strcmp(name, "put_ks")) a = put_ks_addr(lane, arg0);
        else if (!strcmp(name, "get_ks")) a = get_ks_addr(permuted, lane, arg0, arg1);
        else if (!strcmp(name, "put_strip")) a = put_strip_addr(lane, arg0);
        else if (!strcmp(name, "put_strip_swapped")) a = put_strip_swapped_addr(lane, arg0);
        else if (!strcmp(name, "get_kc_tr_swapped")) a = get_kc_tr_swapped_addr(lane, arg0, arg1);
        else if (!strcmp(name, "get_strip")) a = get_strip_addr(permuted, lane, arg0 & 1, arg0 >> 1, arg1);
        else if (!strcmp(name, "put_strip16")) a = put_strip16_addr(lane, arg0);
        else if (!strcmp(name, "get_strip16")) a = get_strip16_addr(lane, arg0, arg1);
        else if (!strcmp(name, "put_result")) a = put_result_addr(lane, arg0);
        else if (!strcmp(name, "get_linear")) a = get_linear_addr(lane, arg0);
        else if (!strcmp(name, "put_f32")) a = put_f32_addr(lane, arg0);
        else if (!strcmp(name, "get_f32_kc")) a = get_f32_kc_addr(permuted, lane, arg0);
        else if (!strcmp(name, "get_f32_ks")) a = get_f32_ks_addr(permuted, lane, arg0);
        else return -1;
        addr64[lane] = a;
    }
    return 0;
}

extern "C" int bsa_col16(int t, int i) { return bsa::col16(t, i); }
extern "C" int bsa_strip16_half_swapped(int k) { return bsa::strip16_half_swapped(k); }
extern "C" int bsa_perm16(int i) { return bsa::perm16(i); }
extern "C" int bsa_invperm16(int i) { return bsa::invperm16(i); }
