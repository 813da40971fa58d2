// Host build of csrc/numerics.hpp for the CPU tests (g++ -ffp-contract=off): the same text the device compiles.
#include "../ferrite_amd/csrc/numerics.hpp"
extern "C" {
float shim_expf(float x) { return fe::fe_expf(x); }
float shim_sigmoid(float x) { return fe::sigmoid_ref(x); }
float shim_swiglu(float g, float u, float l) { return fe::swiglu_ref(g, u, l); }
unsigned shim_e4m3_encode(float x) { return fe::e4m3_encode(x); }
float shim_e4m3_decode(unsigned b) { return fe::e4m3_decode(b); }
float shim_e2m1_decode(unsigned c) { return fe::e2m1_decode(c); }
float shim_ue8m0_decode(unsigned b) { return fe::ue8m0_decode(b); }
unsigned shim_block_scale_e8m0(float amax) { return fe::block_scale_e8m0(amax); }
void shim_expf_many(const float* x, float* y, long n) { for (long i = 0; i < n; ++i) y[i] = fe::fe_expf(x[i]); }
}
