// ORACLE — TEST INFRASTRUCTURE ONLY.
// C-callable door to the reference's own CPU check `test::allreduce_rmsnorm_ref`
// (test/unit_test.cpp:175-217).  This file holds no reference code: the Makefile compiles the
// reference's unit_test.cpp where it lies (its main() renamed by -D) and links it with this
// wrapper into oracle/_ref/libunit_ref.so.
namespace test {
void allreduce_rmsnorm_ref(const float *allreduce_in, const float *residual_in, const float *rms_gamma, int size,
                           int hidden_dim, int nranks, float *residual_out, float *norm_out, float eps);
}

extern "C" int ref_allreduce_rmsnorm(const float *allreduce_in, const float *residual_in, const float *rms_gamma,
                                     int size, int hidden_dim, int nranks, float *residual_out, float *norm_out,
                                     float eps) {
    test::allreduce_rmsnorm_ref(allreduce_in, residual_in, rms_gamma, size, hidden_dim, nranks, residual_out, norm_out,
                                eps);
    return 0;
}
