// C ABI entry points for the attention block kernels: argument validation and dispatch.
// The entry points of the elementwise kernels sit next to their kernels in lse_merge.hip.
#include "mhip_common.hpp"

namespace mhip {
int attn_fwd_bf16(const void* q, const void* k, const void* v, void* out, float* lse,
                  int B, int Sq, int Sc, int Hq, int Hkv, int D,
                  const int64_t* strides, float scale, int mask, hipStream_t stream);
int attn_fwd_fp8(const void* q, const void* k, const void* v, void* out, float* lse,
                 int B, int Sq, int Sc, int Hq, int Hkv, int D, const int64_t* strides, float scale, int mask,
                 const float* q_descale, const float* k_descale, const float* v_descale, hipStream_t stream);
}  // namespace mhip

using namespace mhip;

extern "C" int mhip_version(void) { return 1; }
extern "C" int mhip_abi_version(void) { return MHIP_ABI_VERSION; }

extern "C" const char* mhip_error_string(int code) {
  switch (code) {
    case MHIP_OK: return "ok";
    case MHIP_EINVAL: return "invalid argument (size, NULL pointer or softmax scale)";
    case MHIP_EDTYPE: return "element type not supported by this entry point";
    case MHIP_EHEADDIM: return "head dimension not supported (bf16: a multiple of 8 up to 128; e4m3: a multiple of 16 up to 128)";
    case MHIP_EALIGN: return "pointer or stride not aligned to 16 bytes";
    case MHIP_ELAUNCH: return "kernel launch failed";
    case MHIP_EUNSUPPORTED: return "feature not implemented";
    case MHIP_ETOOLARGE: return "problem exceeds the built-in scratch of the no-allocation entry point (B * Hq * Sq <= 1048576)";
    case MHIP_ERUNTIME: return "HIP runtime query failed (current device or symbol address)";
    default: return "unknown error code";
  }
}

namespace {
bool mult8(int64_t x) { return (x & 7) == 0; }
}  // namespace

extern "C" int mhip_attn_fwd_block(const void* q, const void* k, const void* v, void* out, float* lse,
                                   int B, int Sq, int Sc, int Hq, int Hkv, int D,
                                   int64_t q_sb, int64_t q_ss, int64_t q_sh,
                                   int64_t k_sb, int64_t k_ss, int64_t k_sh,
                                   int64_t v_sb, int64_t v_ss, int64_t v_sh,
                                   int64_t o_sb, int64_t o_ss, int64_t o_sh,
                                   float softmax_scale, int mask, int dtype,
                                   const float* q_descale, const float* k_descale, const float* v_descale,
                                   void* stream) {
  if (B < 0 || Sq < 0 || Sc < 0 || Hq <= 0 || Hkv <= 0 || Hq % Hkv != 0) return MHIP_EINVAL;
  if (!(softmax_scale > 0.f) || !(softmax_scale < INFINITY)) return MHIP_EINVAL;
  if (mask != MHIP_MASK_NONE && mask != MHIP_MASK_CAUSAL) return MHIP_EINVAL;
  if (dtype != MHIP_BF16 && dtype != MHIP_E4M3) return MHIP_EDTYPE;
  // any multiple of 8 (bf16) or of 16 (e4m3) up to 128: the kernels work on 128 columns, the missing ones zero on chip
  if (D <= 0 || D > 128 || (D & (dtype == MHIP_E4M3 ? 15 : 7)) != 0) return MHIP_EHEADDIM;
  if (B == 0 || Sq == 0) return MHIP_OK;
  if (!q || !out || !lse) return MHIP_EINVAL;
  if (Sc > 0 && (!k || !v)) return MHIP_EINVAL;
  hipStream_t st = static_cast<hipStream_t>(stream);
  // 16-byte vector accesses on every row of q, k, v and out
  if (!aligned16(q) || !aligned16(out) || (Sc > 0 && (!aligned16(k) || !aligned16(v)))) return MHIP_EALIGN;
  const bool fp8 = dtype == MHIP_E4M3;
  auto in_ok = [fp8](int64_t x) { return fp8 ? (x & 15) == 0 : mult8(x); };     // element strides
  if (!in_ok(q_sb) || !in_ok(q_ss) || !in_ok(q_sh) || !in_ok(k_sb) || !in_ok(k_ss) || !in_ok(k_sh) ||
      !in_ok(v_sb) || !in_ok(v_ss) || !in_ok(v_sh) || !mult8(o_sb) || !mult8(o_ss) || !mult8(o_sh))
    return MHIP_EALIGN;
  // K / V tiles are fetched through 32-bit buffer offsets relative to the (batch, head) base
  const int64_t kv_span = (int64_t)Sc * (k_ss > v_ss ? k_ss : v_ss) * (fp8 ? 1 : 2);
  if (k_ss < 0 || v_ss < 0 || kv_span >= (int64_t(1) << 31)) return MHIP_EUNSUPPORTED;
  // below 128 the lanes of the missing columns carry the offset 0x7fff0000, which has to stay out of range with
  // any tile offset added and must not wrap 32 bits
  if (D < 128 && kv_span >= (int64_t(1) << 30)) return MHIP_EUNSUPPORTED;
  const int64_t strides[12] = {q_sb, q_ss, q_sh, k_sb, k_ss, k_sh, v_sb, v_ss, v_sh, o_sb, o_ss, o_sh};
  if (fp8) {
    if ((reinterpret_cast<uintptr_t>(q_descale) | reinterpret_cast<uintptr_t>(k_descale) |
         reinterpret_cast<uintptr_t>(v_descale)) & 3u)
      return MHIP_EALIGN;
    return attn_fwd_fp8(q, k, v, out, lse, B, Sq, Sc, Hq, Hkv, D, strides, softmax_scale, mask,
                        q_descale, k_descale, v_descale, st);
  }
  return attn_fwd_bf16(q, k, v, out, lse, B, Sq, Sc, Hq, Hkv, D, strides, softmax_scale, mask, st);
}
