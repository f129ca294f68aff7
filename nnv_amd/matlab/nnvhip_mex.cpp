// MEX gateway between MATLAB and libnnvhip.so.  The only file that includes mex.h; it marshals
// mxArray <-> the C ABI of include/nnvhip.h and nothing else.  Build (where MATLAB exists):
//
//   mex -R2018a CXXFLAGS='$CXXFLAGS -std=c++17' -I<repo>/include nnvhip_mex.cpp -L<repo>/nnv_amd -lnnvhip
//
// Usage:  out = nnvhip_mex('command', args...).  Handles travel as uint64 scalars / row vectors.
// Index vectors are converted to MATLAB's 1-based doubles here.  A non-zero status becomes a MATLAB
// error carrying the library's message, which for NNV's own argument checks is NNV's error text.
#include <cstdint>
#include <cstring>
#include <string>
#include <vector>

#include "mex.h"
#include "nnvhip.h"

static nnvhip_ctx* g_ctx = nullptr;

static void check(int status) {
  if (status != NNVHIP_OK) mexErrMsgIdAndTxt("nnvhip:error", "%s", nnvhip_last_error());
}

static void at_exit() {
  if (g_ctx) {
    nnvhip_destroy(g_ctx);  // fails harmlessly if MATLAB still holds handles
    g_ctx = nullptr;
  }
}

static nnvhip_ctx* ctx() {
  if (!g_ctx) {
    check(nnvhip_create(0, &g_ctx));
    mexAtExit(at_exit);
  }
  return g_ctx;
}

static void need(int nrhs, int n, const char* cmd) {
  if (nrhs != n + 1) mexErrMsgIdAndTxt("nnvhip:args", "%s expects %d arguments", cmd, n);
}

static const double* dbl(const mxArray* a, const char* what) {
  if (mxIsEmpty(a)) return nullptr;
  if (!mxIsDouble(a) || mxIsComplex(a)) mexErrMsgIdAndTxt("nnvhip:type", "%s must be a real double array", what);
  return mxGetDoubles(a);
}

template <class T>
static T* handle_of(const mxArray* a) {
  if (!mxIsUint64(a) || mxGetNumberOfElements(a) != 1) mexErrMsgIdAndTxt("nnvhip:type", "expected a uint64 handle");
  return reinterpret_cast<T*>(static_cast<uintptr_t>(*static_cast<const uint64_t*>(mxGetData(a))));
}

static std::vector<nnvhip_star*> handles_of(const mxArray* a) {
  if (!mxIsUint64(a)) mexErrMsgIdAndTxt("nnvhip:type", "expected a uint64 handle array");
  const uint64_t* p = static_cast<const uint64_t*>(mxGetData(a));
  std::vector<nnvhip_star*> v(mxGetNumberOfElements(a));
  for (size_t i = 0; i < v.size(); ++i) v[i] = reinterpret_cast<nnvhip_star*>(static_cast<uintptr_t>(p[i]));
  return v;
}

static mxArray* to_mx(const std::vector<nnvhip_star*>& v) {
  mxArray* a = mxCreateNumericMatrix(1, v.size(), mxUINT64_CLASS, mxREAL);
  uint64_t* p = static_cast<uint64_t*>(mxGetData(a));
  for (size_t i = 0; i < v.size(); ++i) p[i] = static_cast<uint64_t>(reinterpret_cast<uintptr_t>(v[i]));
  return a;
}

static mxArray* to_mx(const void* h) {
  mxArray* a = mxCreateNumericMatrix(1, 1, mxUINT64_CLASS, mxREAL);
  *static_cast<uint64_t*>(mxGetData(a)) = static_cast<uint64_t>(reinterpret_cast<uintptr_t>(h));
  return a;
}

void mexFunction(int nlhs, mxArray* plhs[], int nrhs, const mxArray* prhs[]) {
  if (nrhs < 1 || !mxIsChar(prhs[0])) mexErrMsgIdAndTxt("nnvhip:args", "first argument must be a command string");
  char buf[64];
  mxGetString(prhs[0], buf, sizeof buf);
  const std::string cmd(buf);

  if (cmd == "star_create") {  // (V, C, d, pred_lb, pred_ub) -> handle      Star(V,C,d,lb,ub), set/Star.m:153-189
    need(nrhs, 5, "star_create");
    const mwSize N = mxGetM(prhs[1]), cols = mxGetN(prhs[1]);
    const mwSize p = mxGetM(prhs[2]);
    if (!mxIsEmpty(prhs[2]) && mxGetN(prhs[2]) + 1 != cols)
      mexErrMsgIdAndTxt("nnvhip:error", "Inconsistency between basic matrix and constraint matrix");
    nnvhip_star* s = nullptr;
    check(nnvhip_star_create(ctx(), (int64_t)N, (int64_t)cols - 1, dbl(prhs[1], "V"), dbl(prhs[4], "pred_lb"),
                             dbl(prhs[5], "pred_ub"), dbl(prhs[2], "C"), dbl(prhs[3], "d"), (int64_t)p, &s));
    plhs[0] = to_mx(s);
  } else if (cmd == "star_from_box") {  // (lb, ub), N x count -> handles    Star(lb,ub), set/Star.m:220-237
    need(nrhs, 2, "star_from_box");
    const mwSize N = mxGetM(prhs[1]), count = mxGetN(prhs[1]);
    if (mxGetM(prhs[2]) != N || mxGetN(prhs[2]) != count)
      mexErrMsgIdAndTxt("nnvhip:error", "Inconsistent dimensions between lb and ub");
    std::vector<nnvhip_star*> out(count);
    check(nnvhip_star_from_box(ctx(), (int64_t)N, (int64_t)count, dbl(prhs[1], "lb"), dbl(prhs[2], "ub"), out.data()));
    plhs[0] = to_mx(out);
  } else if (cmd == "star_release") {
    need(nrhs, 1, "star_release");
    const std::vector<nnvhip_star*> hs = handles_of(prhs[1]);
    check(nnvhip_star_release_array((int64_t)hs.size(), hs.data()));
  } else if (cmd == "star_dims") {  // handle -> [dim nVar nConstraintRows mayBeEmpty hasZono]
    need(nrhs, 1, "star_dims");
    int64_t N, n, p;
    int32_t user = 0;
    check(nnvhip_star_dims(handle_of<nnvhip_star>(prhs[1]), &N, &n, &p));
    check(nnvhip_star_has_user_constraints(handle_of<nnvhip_star>(prhs[1]), &user));
    int32_t zono = 0;
    check(nnvhip_star_has_zono(handle_of<nnvhip_star>(prhs[1]), &zono));
    plhs[0] = mxCreateDoubleMatrix(1, 5, mxREAL);
    double* o = mxGetDoubles(plhs[0]);
    o[0] = (double)N;
    o[1] = (double)n;
    o[2] = (double)p;
    o[3] = (double)user;  // 1: the set goes back to constraint rows the caller handed in (it may be empty)
    o[4] = (double)zono;  // 1: the reference's Star carries an outer zonotope here (= Zono(V(:,1), V(:,2:end)))
  } else if (cmd == "fetch_V") {  // handle -> V (dim x (nVar+1))
    need(nrhs, 1, "fetch_V");
    nnvhip_star* s = handle_of<nnvhip_star>(prhs[1]);
    int64_t N, n, p;
    check(nnvhip_star_dims(s, &N, &n, &p));
    plhs[0] = mxCreateDoubleMatrix((mwSize)N, (mwSize)(n + 1), mxREAL);
    check(nnvhip_star_fetch_V(s, mxGetDoubles(plhs[0])));
  } else if (cmd == "fetch_pred") {  // handle -> [pred_lb, pred_ub]
    need(nrhs, 1, "fetch_pred");
    nnvhip_star* s = handle_of<nnvhip_star>(prhs[1]);
    int64_t N, n, p;
    check(nnvhip_star_dims(s, &N, &n, &p));
    plhs[0] = mxCreateDoubleMatrix((mwSize)n, 1, mxREAL);
    mxArray* ub = mxCreateDoubleMatrix((mwSize)n, 1, mxREAL);
    check(nnvhip_star_fetch_pred_bounds(s, mxGetDoubles(plhs[0]), mxGetDoubles(ub)));
    if (nlhs > 1) plhs[1] = ub; else mxDestroyArray(ub);
  } else if (cmd == "fetch_constraints") {  // handle -> [C, d], NNV's dense [C0;C1;C2;C3] layout
    need(nrhs, 1, "fetch_constraints");
    nnvhip_star* s = handle_of<nnvhip_star>(prhs[1]);
    int64_t N, n, p;
    check(nnvhip_star_dims(s, &N, &n, &p));
    plhs[0] = mxCreateDoubleMatrix((mwSize)p, (mwSize)n, mxREAL);
    mxArray* d = mxCreateDoubleMatrix((mwSize)p, 1, mxREAL);
    check(nnvhip_star_fetch_constraints(s, mxGetDoubles(plhs[0]), mxGetDoubles(d)));
    if (nlhs > 1) plhs[1] = d; else mxDestroyArray(d);
  } else if (cmd == "fetch_crossing") {  // handle -> [index (1-based), lb, ub, n_inactive]
    need(nrhs, 1, "fetch_crossing");
    nnvhip_star* s = handle_of<nnvhip_star>(prhs[1]);
    int64_t ni, m;
    check(nnvhip_star_relu_counts(s, &ni, &m));
    std::vector<int32_t> idx((size_t)m);
    plhs[0] = mxCreateDoubleMatrix((mwSize)m, 1, mxREAL);
    mxArray* lb = mxCreateDoubleMatrix((mwSize)m, 1, mxREAL);
    mxArray* ub = mxCreateDoubleMatrix((mwSize)m, 1, mxREAL);
    check(nnvhip_star_fetch_crossing(s, idx.data(), mxGetDoubles(lb), mxGetDoubles(ub)));
    for (int64_t i = 0; i < m; ++i) mxGetDoubles(plhs[0])[i] = (double)idx[i] + 1.0;
    if (nlhs > 1) plhs[1] = lb; else mxDestroyArray(lb);
    if (nlhs > 2) plhs[2] = ub; else mxDestroyArray(ub);
    if (nlhs > 3) plhs[3] = mxCreateDoubleScalar((double)ni);
  } else if (cmd == "estimate_ranges") {  // handles -> [lb, ub] (dim x count)     Star.estimateRanges, set/Star.m:1078-1106
    need(nrhs, 1, "estimate_ranges");
    std::vector<nnvhip_star*> in = handles_of(prhs[1]);
    int64_t N, n, p;
    check(nnvhip_star_dims(in.at(0), &N, &n, &p));
    plhs[0] = mxCreateDoubleMatrix((mwSize)N, in.size(), mxREAL);
    mxArray* ub = mxCreateDoubleMatrix((mwSize)N, in.size(), mxREAL);
    check(nnvhip_estimate_ranges_batch(ctx(), (int64_t)in.size(), in.data(), mxGetDoubles(plhs[0]), mxGetDoubles(ub)));
    if (nlhs > 1) plhs[1] = ub; else mxDestroyArray(ub);
  } else if (cmd == "fc_create") {  // (W, b) -> layer handle      FullyConnectedLayer(W,b)
    need(nrhs, 2, "fc_create");
    nnvhip_fc* fc = nullptr;
    check(nnvhip_fc_create(ctx(), dbl(prhs[1], "W"), dbl(prhs[2], "b"), (int64_t)mxGetM(prhs[1]), (int64_t)mxGetN(prhs[1]), &fc));
    plhs[0] = to_mx(fc);
  } else if (cmd == "fc_destroy") {
    need(nrhs, 1, "fc_destroy");
    check(nnvhip_fc_destroy(handle_of<nnvhip_fc>(prhs[1])));
  } else if (cmd == "conv2d_create") {  // (W, bias, padding[t b l r], stride, dilation) -> layer handle
    need(nrhs, 5, "conv2d_create");
    const mwSize nd = mxGetNumberOfDimensions(prhs[1]);
    const mwSize* dm = mxGetDimensions(prhs[1]);
    int64_t dims[4] = {1, 1, 1, 1};
    for (mwSize i = 0; i < nd && i < 4; ++i) dims[i] = (int64_t)dm[i];
    int64_t pad[4], st[2], dl[2];
    const double *pp = dbl(prhs[3], "padding"), *sp = dbl(prhs[4], "stride"), *dp = dbl(prhs[5], "dilation");
    if (mxGetNumberOfElements(prhs[3]) != 4 || mxGetNumberOfElements(prhs[4]) != 2 || mxGetNumberOfElements(prhs[5]) != 2)
      mexErrMsgIdAndTxt("nnvhip:error", "Invalid padding, stride or dilation matrix");
    for (int i = 0; i < 4; ++i) pad[i] = (int64_t)pp[i];
    for (int i = 0; i < 2; ++i) { st[i] = (int64_t)sp[i]; dl[i] = (int64_t)dp[i]; }
    nnvhip_conv2d* cv = nullptr;
    check(nnvhip_conv2d_create(ctx(), dbl(prhs[1], "W"), dbl(prhs[2], "bias"), dims[0], dims[1], dims[2], dims[3], pad, st, dl, &cv));
    plhs[0] = to_mx(cv);
  } else if (cmd == "conv2d_destroy") {
    need(nrhs, 1, "conv2d_destroy");
    check(nnvhip_conv2d_destroy(handle_of<nnvhip_conv2d>(prhs[1])));
  } else if (cmd == "affine_fc") {  // (layer, handles) -> handles      FullyConnectedLayer.reach
    need(nrhs, 2, "affine_fc");
    std::vector<nnvhip_star*> in = handles_of(prhs[2]), out(in.size());
    check(nnvhip_affine_fc(ctx(), handle_of<nnvhip_fc>(prhs[1]), (int64_t)in.size(), in.data(), out.data()));
    plhs[0] = to_mx(out);
  } else if (cmd == "hint_next_fc") {  // (layer | [])      the FC layer that will follow the next ReLU step (an array of sets)
    need(nrhs, 1, "hint_next_fc");
    check(nnvhip_hint_next_fc(ctx(), mxIsEmpty(prhs[1]) ? nullptr : handle_of<nnvhip_fc>(prhs[1])));
  } else if (cmd == "affine_conv2d") {  // (layer, H, W, handles) -> handles      Conv2DLayer.reach
    need(nrhs, 4, "affine_conv2d");
    std::vector<nnvhip_star*> in = handles_of(prhs[4]), out(in.size());
    check(nnvhip_affine_conv2d(ctx(), handle_of<nnvhip_conv2d>(prhs[1]), (int64_t)mxGetScalar(prhs[2]),
                               (int64_t)mxGetScalar(prhs[3]), (int64_t)in.size(), in.data(), out.data()));
    plhs[0] = to_mx(out);
  } else if (cmd == "relu_relax") {  // (order 0|1|2, relaxFactor, handles) -> handles      ReluLayer.reach
    need(nrhs, 3, "relu_relax");
    std::vector<nnvhip_star*> in = handles_of(prhs[3]), out(in.size());
    check(nnvhip_relu_relax(ctx(), (int)mxGetScalar(prhs[1]), mxGetScalar(prhs[2]), (int64_t)in.size(), in.data(), out.data()));
    plhs[0] = to_mx(out);
  } else if (cmd == "relu_reduce_mem") {  // (handle, H, W, C) -> [handle, l, u]      ReluLayer.m:119-146
    need(nrhs, 4, "relu_reduce_mem");
    nnvhip_star* s = handle_of<nnvhip_star>(prhs[1]);
    const int64_t H = (int64_t)mxGetScalar(prhs[2]), W = (int64_t)mxGetScalar(prhs[3]), C = (int64_t)mxGetScalar(prhs[4]);
    mxArray* l = mxCreateDoubleMatrix((mwSize)(H * W * C), 1, mxREAL);
    mxArray* u = mxCreateDoubleMatrix((mwSize)(H * W * C), 1, mxREAL);
    nnvhip_star* out = nullptr;
    check(nnvhip_relu_reduce_mem(ctx(), s, H, W, C, &out, mxGetDoubles(l), mxGetDoubles(u)));
    plhs[0] = to_mx(out);
    if (nlhs > 1) plhs[1] = l;
    if (nlhs > 2) plhs[2] = u;
  } else if (cmd == "fetch_rows") {  // (handle, rows 1-based) -> V(rows, :)      objective rows of Star.getMin/getMax
    need(nrhs, 2, "fetch_rows");
    nnvhip_star* s = handle_of<nnvhip_star>(prhs[1]);
    int64_t N, n, p;
    check(nnvhip_star_dims(s, &N, &n, &p));
    const mwSize R = mxGetNumberOfElements(prhs[2]);
    const double* r1 = dbl(prhs[2], "rows");
    std::vector<int32_t> rows(R);
    for (mwSize t = 0; t < R; ++t) rows[t] = (int32_t)r1[t] - 1;
    plhs[0] = mxCreateDoubleMatrix(R, (mwSize)(n + 1), mxREAL);
    check(nnvhip_star_fetch_rows(s, (int64_t)R, rows.data(), mxGetDoubles(plhs[0])));
  } else if (cmd == "relu_apply_lists") {  // (handle, reset rows, index, lb, ub; 1-based) -> handle
    // PosLin.multipleStepReachStarApprox_at_one(I.resetRow(reset), index, lb, ub), nn/funcs/PosLin.m:685-742
    need(nrhs, 5, "relu_apply_lists");
    const mwSize nr = mxGetNumberOfElements(prhs[2]), m = mxGetNumberOfElements(prhs[3]);
    if (mxGetNumberOfElements(prhs[4]) != m || mxGetNumberOfElements(prhs[5]) != m)
      mexErrMsgIdAndTxt("nnvhip:error", "index, lb and ub must have the same length");
    const double* r1 = dbl(prhs[2], "reset");
    const double* i1 = dbl(prhs[3], "index");
    std::vector<int32_t> reset(nr), index(m);
    for (mwSize t = 0; t < nr; ++t) reset[t] = (int32_t)r1[t] - 1;
    for (mwSize t = 0; t < m; ++t) index[t] = (int32_t)i1[t] - 1;
    nnvhip_star* out = nullptr;
    check(nnvhip_relu_apply_lists(ctx(), handle_of<nnvhip_star>(prhs[1]), (int64_t)nr, reset.data(), (int64_t)m, index.data(),
                                  dbl(prhs[4], "lb"), dbl(prhs[5], "ub"), &out));
    plhs[0] = to_mx(out);
  } else if (cmd == "halfspace_check") {  // (handles, G (R x dim), g (R x 1), rows_per_halfspace) -> [verdict (count x n_hs), lo, hi]
    // LP-free part of utils/verify_specification.m:36-80; 1 = disjoint, 2 = undecided (LP), 3 = inside
    need(nrhs, 4, "halfspace_check");
    std::vector<nnvhip_star*> in = handles_of(prhs[1]);
    const mwSize R = mxGetM(prhs[2]), N = mxGetN(prhs[2]);
    if (mxGetNumberOfElements(prhs[3]) != R)
      mexErrMsgIdAndTxt("nnvhip:error", "Inconsistent dimension between Halfspace matrix and halfspace vector");
    const mwSize n_hs = mxGetNumberOfElements(prhs[4]);
    const double* rows = dbl(prhs[4], "rows_per_halfspace");
    std::vector<int64_t> row_ptr(n_hs + 1, 0);
    for (mwSize h = 0; h < n_hs; ++h) row_ptr[h + 1] = row_ptr[h] + (int64_t)rows[h];
    if (row_ptr[n_hs] != (int64_t)R)
      mexErrMsgIdAndTxt("nnvhip:error", "Inconsistent dimension between Halfspace matrix and halfspace vector");
    std::vector<int32_t> verdict(in.size() * n_hs);
    mxArray* lo = mxCreateDoubleMatrix(R, in.size(), mxREAL);
    mxArray* hi = mxCreateDoubleMatrix(R, in.size(), mxREAL);
    check(nnvhip_halfspace_check(ctx(), (int64_t)in.size(), in.data(), (int64_t)n_hs, row_ptr.data(), dbl(prhs[2], "G"),
                                 dbl(prhs[3], "g"), (int64_t)N, verdict.data(), mxGetDoubles(lo), mxGetDoubles(hi)));
    plhs[0] = mxCreateDoubleMatrix(in.size(), n_hs, mxREAL);
    for (size_t i = 0; i < verdict.size(); ++i) mxGetDoubles(plhs[0])[i] = (double)verdict[i];
    if (nlhs > 1) plhs[1] = lo; else mxDestroyArray(lo);
    if (nlhs > 2) plhs[2] = hi; else mxDestroyArray(hi);
  } else if (cmd == "halfspace_rows") {  // (handle, G, g) -> [C1, d1]      Star.intersectHalfSpace, set/Star.m:577-578
    need(nrhs, 3, "halfspace_rows");
    nnvhip_star* s = handle_of<nnvhip_star>(prhs[1]);
    int64_t N, n, p;
    check(nnvhip_star_dims(s, &N, &n, &p));
    const mwSize R = mxGetM(prhs[2]);
    if (mxGetNumberOfElements(prhs[3]) != R)
      mexErrMsgIdAndTxt("nnvhip:error", "Inconsistent dimension between Halfspace matrix and halfspace vector");
    plhs[0] = mxCreateDoubleMatrix(R, (mwSize)n, mxREAL);
    mxArray* d1 = mxCreateDoubleMatrix(R, 1, mxREAL);
    check(nnvhip_halfspace_rows(ctx(), s, (int64_t)R, dbl(prhs[2], "G"), dbl(prhs[3], "g"), (int64_t)mxGetN(prhs[2]),
                                mxGetDoubles(plhs[0]), mxGetDoubles(d1)));
    if (nlhs > 1) plhs[1] = d1; else mxDestroyArray(d1);
  } else if (cmd == "rowmap_create") {  // (ops (1 x S), scopes (1 x S), params (N x S)) -> layer handle
    // per-row affine programme: ops 0 add | 1 sub | 2 mul | 3 div; scopes 0 centre column | 1 all columns
    need(nrhs, 3, "rowmap_create");
    const mwSize S = mxGetN(prhs[3]), N = mxGetM(prhs[3]);
    if (mxGetNumberOfElements(prhs[1]) != S || mxGetNumberOfElements(prhs[2]) != S)
      mexErrMsgIdAndTxt("nnvhip:error", "one op and one scope per parameter column");
    std::vector<int32_t> op(S), sc(S);
    for (mwSize i = 0; i < S; ++i) {
      op[i] = (int32_t)dbl(prhs[1], "ops")[i];
      sc[i] = (int32_t)dbl(prhs[2], "scopes")[i];
    }
    nnvhip_rowmap* m = nullptr;
    check(nnvhip_rowmap_create(ctx(), (int64_t)N, (int32_t)S, op.data(), sc.data(), dbl(prhs[3], "params"), &m));
    plhs[0] = to_mx(m);
  } else if (cmd == "rowmap_destroy") {
    need(nrhs, 1, "rowmap_destroy");
    check(nnvhip_rowmap_destroy(handle_of<nnvhip_rowmap>(prhs[1])));
  } else if (cmd == "affine_rowmap") {  // (layer, handles) -> handles      BatchNormalizationLayer / ImageInputLayer reach
    need(nrhs, 2, "affine_rowmap");
    std::vector<nnvhip_star*> in = handles_of(prhs[2]), out(in.size());
    check(nnvhip_affine_rowmap(ctx(), handle_of<nnvhip_rowmap>(prhs[1]), (int64_t)in.size(), in.data(), out.data()));
    plhs[0] = to_mx(out);
  } else if (cmd == "avgpool2d_create") {  // (poolSize [h w], stride [sh sw], padding [t b l r]) -> layer handle
    need(nrhs, 3, "avgpool2d_create");
    if (mxGetNumberOfElements(prhs[1]) != 2) mexErrMsgIdAndTxt("nnvhip:error", "Invalid pool size");
    if (mxGetNumberOfElements(prhs[2]) != 2) mexErrMsgIdAndTxt("nnvhip:error", "Invalid stride");
    if (mxGetNumberOfElements(prhs[3]) != 4) mexErrMsgIdAndTxt("nnvhip:error", "Invalide padding size");
    int64_t pool[2], st[2], pad[4];
    for (int i = 0; i < 2; ++i) {
      pool[i] = (int64_t)dbl(prhs[1], "poolSize")[i];
      st[i] = (int64_t)dbl(prhs[2], "stride")[i];
    }
    for (int i = 0; i < 4; ++i) pad[i] = (int64_t)dbl(prhs[3], "padding")[i];
    nnvhip_avgpool2d* l = nullptr;
    check(nnvhip_avgpool2d_create(ctx(), pool, st, pad, &l));
    plhs[0] = to_mx(l);
  } else if (cmd == "avgpool2d_destroy") {
    need(nrhs, 1, "avgpool2d_destroy");
    check(nnvhip_avgpool2d_destroy(handle_of<nnvhip_avgpool2d>(prhs[1])));
  } else if (cmd == "affine_avgpool2d") {  // (layer, H, W, handles) -> [handles, Ho, Wo]      AveragePooling2DLayer.reach
    need(nrhs, 4, "affine_avgpool2d");
    std::vector<nnvhip_star*> in = handles_of(prhs[4]), out(in.size());
    nnvhip_avgpool2d* l = handle_of<nnvhip_avgpool2d>(prhs[1]);
    const int64_t H = (int64_t)mxGetScalar(prhs[2]), W = (int64_t)mxGetScalar(prhs[3]);
    int64_t Ho = 0, Wo = 0;
    check(nnvhip_avgpool2d_output_size(l, H, W, &Ho, &Wo));
    check(nnvhip_affine_avgpool2d(ctx(), l, H, W, (int64_t)in.size(), in.data(), out.data()));
    plhs[0] = to_mx(out);
    if (nlhs > 1) plhs[1] = mxCreateDoubleScalar((double)Ho);
    if (nlhs > 2) plhs[2] = mxCreateDoubleScalar((double)Wo);
  } else if (cmd == "permute_rows") {  // (src_row (1-based, N x 1), handles) -> handles      C-style FlattenLayer.reach
    need(nrhs, 2, "permute_rows");
    const mwSize N = mxGetNumberOfElements(prhs[1]);
    std::vector<int32_t> src(N);
    for (mwSize i = 0; i < N; ++i) src[i] = (int32_t)dbl(prhs[1], "src_row")[i] - 1;
    std::vector<nnvhip_star*> in = handles_of(prhs[2]), out(in.size());
    check(nnvhip_permute_rows(ctx(), (int64_t)N, src.data(), (int64_t)in.size(), in.data(), out.data()));
    plhs[0] = to_mx(out);
  } else if (cmd == "sync") {
    check(nnvhip_synchronize(ctx()));
  } else if (cmd == "set_timing") {
    need(nrhs, 1, "set_timing");
    check(nnvhip_set_timing(ctx(), mxGetScalar(prhs[1]) != 0));
  } else if (cmd == "set_eager_columns") {  // 1: FC layers write gathered columns in the call itself
    need(nrhs, 1, "set_eager_columns");
    check(nnvhip_set_eager_columns(ctx(), mxGetScalar(prhs[1]) != 0));
  } else if (cmd == "set_eager_relu") {  // 1: the ReLU step writes its whole output matrix in the call itself
    need(nrhs, 1, "set_eager_relu");
    check(nnvhip_set_eager_relu(ctx(), mxGetScalar(prhs[1]) != 0));
  } else if (cmd == "set_dense_affine") {  // 1: FC / conv layers as the full dense contraction (measurement switch)
    need(nrhs, 1, "set_dense_affine");
    check(nnvhip_set_dense_affine(ctx(), mxGetScalar(prhs[1]) != 0));
  } else if (cmd == "last_op_time_ms") {
    double ms = 0;
    check(nnvhip_last_op_time_ms(ctx(), &ms));
    plhs[0] = mxCreateDoubleScalar(ms);
  } else {
    mexErrMsgIdAndTxt("nnvhip:args", "unknown command '%s'", cmd.c_str());
  }
}
