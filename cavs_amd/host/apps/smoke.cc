// The reference's two printing smoke programs, written against this front end and
// returning the values they print: cavs/frontend/cxx/session_test.cc (C = A + B) and
// cavs/frontend/cxx/fusion_session_test.cc (two chains of Adds under OPT_FUSION).
#include <cstdio>
#include <cstring>
#include <exception>
#include <vector>

#include "cavs/frontend/c_api.h"
#include "cavs/frontend/cxx/session.h"
#include "cavs/proto/opt.pb.h"

using std::vector;

extern "C" {

// out[6] = A + B; returns 0, or -1 after printing the error
int cavs_smoke_session_add(float *out) {
  C_ResetGraph();
  int rc = 0;
  try {
    Sym A = Sym::Placeholder(DT_FLOAT, {2, 3});
    Sym B = Sym::Placeholder(DT_FLOAT, {2, 3});
    Sym C = A + B;
    Session sess;
    vector<float> A_data = {1, 2, 3, 4, 5, 6};
    vector<float> B_data = {6, 5, 4, 3, 2, 1};
    sess.Run(C, {{A, A_data.data()}, {B, B_data.data()}});
    std::memcpy(out, C.eval(), 6 * sizeof(float));
  } catch (const std::exception &e) {
    std::fprintf(stderr, "cavs_smoke_session_add: %s\n", e.what());
    rc = -1;
  }
  C_ResetGraph();
  return rc;
}

// e[6] = C + (A + B), yy[4] = (X + Y) + Z under `opt`; *generated = kernels the fusion pass made
int cavs_smoke_fusion(int opt, float *e, float *yy, int *generated) {
  C_ResetGraph();
  int rc = 0;
  try {
    Sym A = Sym::Placeholder(DT_FLOAT, {2, 3});
    Sym B = Sym::Placeholder(DT_FLOAT, {2, 3});
    Sym C = Sym::Placeholder(DT_FLOAT, {2, 3});
    Sym D = A + B;
    Sym E = C + D;
    Sym X = Sym::Placeholder(DT_FLOAT, {2, 2});
    Sym Y = Sym::Placeholder(DT_FLOAT, {2, 2});
    Sym Z = Sym::Placeholder(DT_FLOAT, {2, 2});
    Sym XX = X + Y;
    Sym YY = XX + Z;
    Session sess(opt);
    vector<float> A_data = {1, 2, 3, 4, 5, 6};
    vector<float> B_data = {6, 5, 4, 3, 2, 1};
    vector<float> C_data = {0.1f, 0.2f, 0.3f, 0.4f, 0.5f, 0.6f};
    vector<float> X_data = {1, 2, 3, 4};
    vector<float> Y_data = {6, 5, 4, 3};
    vector<float> Z_data = {0.1f, 0.2f, 0.3f, 0.4f};
    sess.Run({E, YY}, {{A, A_data.data()}, {B, B_data.data()}, {C, C_data.data()},
                       {X, X_data.data()}, {Y, Y_data.data()}, {Z, Z_data.data()}});
    std::memcpy(e, E.eval(), 6 * sizeof(float));
    std::memcpy(yy, YY.eval(), 4 * sizeof(float));
    *generated = sess.GeneratedKernels();
  } catch (const std::exception &e2) {
    std::fprintf(stderr, "cavs_smoke_fusion: %s\n", e2.what());
    rc = -1;
  }
  C_ResetGraph();
  return rc;
}

}  // extern "C"
