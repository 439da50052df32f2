// C glue over the reference's OWN header-only descriptor logic
// (include/tensorview/gemm/core/{params.h,utils.h} of the reference), compiled
// from the reference tree where it lies by oracle/Makefile into oracle/_ref/.
//
// TEST INFRASTRUCTURE ONLY: used to check the Python mirror of GemmAlgoDesp /
// ConvAlgoDesp (names, validity, alignment, workspace sizes, m/n/k) and to mint
// the fixtures under tests/golden/.  Never linked into the shipped library.
#include <tensorview/gemm/core/params.h>

#include <cstring>
#include <string>

namespace {
// field order shared with tests/golden/make_desp_golden.py
enum Field {
  F_DTYPE_A, F_DTYPE_B, F_DTYPE_C, F_TRANS_A, F_TRANS_B, F_TRANS_C,
  F_TS0, F_TS1, F_TS2, F_WTS0, F_WTS1, F_WTS2, F_NUM_STAGE, F_DACC, F_DCOMP,
  F_TOP0, F_TOP1, F_TOP2, F_SPLITK_SERIAL, F_SPLITK_PARALLEL, F_SHUFFLE,
  F_EPA_A, F_EPA_B, F_EPA_C, F_APV,
  // conv only
  F_NDIM, F_OP_TYPE, F_MASK_SPARSE, F_INC_K_FIRST, F_DYN_MASK, F_INT8_INFER,
  F_COUNT
};

template <class D> void fill(D &d, const int *f, const char *algo) {
  d.dtype_a = f[F_DTYPE_A]; d.dtype_b = f[F_DTYPE_B]; d.dtype_c = f[F_DTYPE_C];
  d.trans_a_ = f[F_TRANS_A]; d.trans_b_ = f[F_TRANS_B]; d.trans_c_ = f[F_TRANS_C];
  d.tile_shape = {f[F_TS0], f[F_TS1], f[F_TS2]};
  d.warp_tile_shape = {f[F_WTS0], f[F_WTS1], f[F_WTS2]};
  d.num_stage = f[F_NUM_STAGE]; d.dacc = f[F_DACC]; d.dcomp = f[F_DCOMP];
  d.algo = algo;
  d.tensorop = {f[F_TOP0], f[F_TOP1], f[F_TOP2]};
  d.split_k_serial_ = f[F_SPLITK_SERIAL]; d.split_k_parallel_ = f[F_SPLITK_PARALLEL];
  d.shuffle_type = static_cast<tv::gemm::ShuffleStrideType>(f[F_SHUFFLE]);
  d.element_per_access_a = f[F_EPA_A]; d.element_per_access_b = f[F_EPA_B];
  d.element_per_access_c = f[F_EPA_C]; d.access_per_vector = f[F_APV];
}

tv::gemm::ConvAlgoDesp make_conv(const int *f, const char *algo) {
  tv::gemm::ConvAlgoDesp d(f[F_NDIM], static_cast<tv::gemm::ConvOpType>(f[F_OP_TYPE]));
  fill(d, f, algo);
  d.mask_sparse = f[F_MASK_SPARSE]; d.increment_k_first = f[F_INC_K_FIRST];
  d.dynamic_mask = f[F_DYN_MASK]; d.is_int8_inference = f[F_INT8_INFER];
  return d;
}

int put(const std::string &s, char *out, int cap) {
  if (cap > 0) { std::strncpy(out, s.c_str(), cap - 1); out[cap - 1] = 0; }
  return int(s.size());
}
} // namespace

extern "C" {
int ref_field_count() { return F_COUNT; }

// returns 0 and the name, or 1 and the exception text
int ref_gemm_repr(const int *f, const char *algo, char *out, int cap) {
  try { tv::gemm::GemmAlgoDesp d; fill(d, f, algo); put(d.__repr__(), out, cap); return 0; }
  catch (const std::exception &e) { put(e.what(), out, cap); return 1; }
}
int ref_conv_repr(const int *f, const char *algo, char *out, int cap) {
  try { auto d = make_conv(f, algo); put(d.__repr__(), out, cap); return 0; }
  catch (const std::exception &e) { put(e.what(), out, cap); return 1; }
}
int ref_gemm_workspace(const int *f, const char *algo, int m, int n, int k, int split) {
  try { tv::gemm::GemmAlgoDesp d; fill(d, f, algo); return d.query_workspace_size(m, n, k, split); }
  catch (const std::exception &) { return -1; }
}
int ref_conv_workspace(const int *f, const char *algo, int m, int n, int k, int split, int kv) {
  try { auto d = make_conv(f, algo); return d.query_conv_workspace_size(m, n, k, split, kv); }
  catch (const std::exception &) { return -1; }
}
int ref_gemm_supported(const int *f, const char *algo, int m, int n, int k) {
  tv::gemm::GemmAlgoDesp d; fill(d, f, algo); return d.supported(m, n, k);
}
int ref_gemm_supported_ldx(const int *f, const char *algo, int lda, int ldb, int ldc) {
  tv::gemm::GemmAlgoDesp d; fill(d, f, algo); return d.supported_ldx(lda, ldb, ldc);
}
int ref_conv_supported(const int *f, const char *algo, int m, int n, int k, int C, int K, int mw) {
  auto d = make_conv(f, algo); return d.supported(m, n, k, C, K, mw);
}
void ref_conv_dtypes_iwo(const int *f, const char *algo, int *out3) {
  auto d = make_conv(f, algo);
  out3[0] = d.dtype_input(); out3[1] = d.dtype_weight(); out3[2] = d.dtype_output();
}
void ref_implicit_gemm_mnk(int op_type, int N, int C, int K, int kv, int in_prod, int out_prod,
                           int mask_sparse, int *out3) {
  auto r = tv::gemm::implicit_gemm_mnk(static_cast<tv::gemm::ConvOpType>(op_type), N, C, K, kv,
                                       in_prod, out_prod, mask_sparse);
  out3[0] = r[0]; out3[1] = r[1]; out3[2] = r[2];
}
void ref_tile_count(int m, int n, int k, int tm, int tn, int split, int *out3) {
  auto r = tv::gemm::get_logical_tile_count(m, n, k, tm, tn, split);
  out3[0] = r[0]; out3[1] = r[1]; out3[2] = r[2];
}
void ref_spconv_tile_count(int m, int n, int k, int tm, int tn, int split, int kv, int op_type,
                           int *out3) {
  auto r = tv::gemm::get_spconv_logical_tile_count(m, n, k, tm, tn, split, kv,
                                                   static_cast<tv::gemm::ConvOpType>(op_type));
  out3[0] = r[0]; out3[1] = r[1]; out3[2] = r[2];
}
void ref_iwo_abc(int op_type, int *iwo2abc, int *abc2iwo) {
  auto a = tv::gemm::ConvAlgoDesp::conv_iwo_012_to_abc(static_cast<tv::gemm::ConvOpType>(op_type));
  auto b = tv::gemm::ConvAlgoDesp::gemm_abc_012_to_iwo(static_cast<tv::gemm::ConvOpType>(op_type));
  for (int i = 0; i < 3; ++i) { iwo2abc[i] = a[i]; abc2iwo[i] = b[i]; }
}
int ref_gemm_k_size_per_split(int k, int split_k, int tile_k) {
  return tv::gemm::get_gemm_k_size_per_split(k, split_k, tile_k);
}
}
