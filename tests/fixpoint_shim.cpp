// Host build of the accumulator-word helpers for tests/test_host_fixpoint.py.
#include "../ponyexl3_amd/csrc/exl3_fixpoint.hpp"

extern "C" {
unsigned long long shim_fix_word(float v) { return exl3::fix_word(v); }
int shim_fix_count(unsigned long long w) { return exl3::fix_count(w); }
float shim_fix_value(unsigned long long w) { return exl3::fix_value(w); }
}
