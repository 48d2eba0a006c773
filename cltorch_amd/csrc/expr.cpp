// User expressions for apply / map / map2: text rewrite and the HIP source
// handed to the runtime compiler.
//
// The reference rewrites with plain substring replacement, shielding only
// "exp" and "max" from the x -> (*out) substitution
// (src/lib/THClTensorMathPointwise.cpp:79-146).  Here the rewrite works on
// identifiers, so every function name containing x, y or z survives; both
// accepted spellings -- x/y/z and *out/*in1/*in2
// (src/test/unit_tensor.lua:583-635) -- give the same kernel.
#include <cctype>
#include <cstdio>
#include <cstring>
#include <string>

#include "internal.h"

namespace {
const char kSkeleton[] =
#include "apply_device_src.inc"
    ;

// OpenCL C built-ins an expression may use that HIP spells differently.
// Everything is fp32; nothing here is a fast-math variant.
const char kPrelude[] = R"PRELUDE(
#define pown(x, n) thcl_pown((x), (int)(n))
#define powr(x, y) powf((x), (y))
#define rootn(x, n) powf((x), 1.0f / (float)(n))
#define native_exp(x) expf(x)
#define native_log(x) logf(x)
#define native_sqrt(x) sqrtf(x)
#define native_sin(x) sinf(x)
#define native_cos(x) cosf(x)
#define native_tan(x) tanf(x)
#define native_recip(x) (1.0f / (x))
#define native_divide(x, y) ((x) / (y))
#define native_powr(x, y) powf((x), (y))
#define half_exp(x) expf(x)
#define half_log(x) logf(x)
#define half_sqrt(x) sqrtf(x)
#define mad(a, b, c) ((a) * (b) + (c))
__device__ __forceinline__ float clamp(float x, float lo, float hi) { return fminf(fmaxf(x, lo), hi); }
__device__ __forceinline__ float sign(float x) { return (float)((x > 0.0f) - (x < 0.0f)); }
__device__ __forceinline__ float mix(float a, float b, float t) { return a + (b - a) * t; }
__device__ __forceinline__ float step(float edge, float x) { return x < edge ? 0.0f : 1.0f; }
)PRELUDE";

bool ident_start(char c) { return std::isalpha((unsigned char)c) || c == '_'; }
bool ident_char(char c) { return std::isalnum((unsigned char)c) || c == '_'; }
}  // namespace

// x -> (*out), y -> (*in1), z -> (*in2) for as many tensors as the call has;
// floating literals without a suffix get `f` so arithmetic stays in fp32, the
// type an OpenCL C fp32 device gives them.
std::string thcl_rewrite_expr(const char *expr, int ntensors) {
  THCL_CHECK(expr != nullptr, "expression is NULL");
  const std::string s(expr);
  std::string out;
  out.reserve(s.size() * 2);
  size_t i = 0;
  while (i < s.size()) {
    const char c = s[i];
    if (ident_start(c)) {
      size_t j = i;
      while (j < s.size() && ident_char(s[j])) j++;
      const std::string id = s.substr(i, j - i);
      if (id == "x") out += "(*out)";
      else if (id == "y" && ntensors >= 2) out += "(*in1)";
      else if (id == "z" && ntensors >= 3) out += "(*in2)";
      else out += id;
      i = j;
    } else if (std::isdigit((unsigned char)c) || (c == '.' && i + 1 < s.size() && std::isdigit((unsigned char)s[i + 1]))) {
      size_t j = i;
      bool is_float = false, hex = false;
      if (c == '0' && j + 1 < s.size() && (s[j + 1] == 'x' || s[j + 1] == 'X')) {
        hex = true;
        j += 2;
        while (j < s.size() && std::isxdigit((unsigned char)s[j])) j++;
      } else {
        while (j < s.size() && std::isdigit((unsigned char)s[j])) j++;
        if (j < s.size() && s[j] == '.') {
          is_float = true;
          j++;
          while (j < s.size() && std::isdigit((unsigned char)s[j])) j++;
        }
        if (j < s.size() && (s[j] == 'e' || s[j] == 'E')) {
          size_t k = j + 1;
          if (k < s.size() && (s[k] == '+' || s[k] == '-')) k++;
          if (k < s.size() && std::isdigit((unsigned char)s[k])) {
            is_float = true;
            j = k;
            while (j < s.size() && std::isdigit((unsigned char)s[j])) j++;
          }
        }
      }
      out += s.substr(i, j - i);
      // keep an existing suffix (f, F, u, l ...)
      size_t k = j;
      while (k < s.size() && std::isalpha((unsigned char)s[k])) k++;
      if (k > j) out += s.substr(j, k - j);
      else if (is_float && !hex) out += 'f';
      i = k;
    } else {
      out += c;
      i++;
    }
  }
  return out;
}

// Kernel-name prefix of an expression: the names carry a hash of the text so
// that profiles tell one expression's kernels from another's.
std::string thcl_expr_tag(const std::string &rewritten, int ntensors) {
  unsigned h = 2166136261u;  // FNV-1a
  for (unsigned char c : rewritten) h = (h ^ c) * 16777619u;
  h = (h ^ (unsigned)ntensors) * 16777619u;
  char buf[32];
  snprintf(buf, sizeof(buf), "thcl_expr%d_%08x", ntensors, h);
  return buf;
}

std::string thcl_expr_source(const std::string &rewritten, int ntensors, int family) {
  THCL_CHECK(ntensors >= 1 && ntensors <= 3, "expression kernels take 1 to 3 tensors");
  std::string src;
  src.reserve(sizeof(kSkeleton) + sizeof(kPrelude) + rewritten.size() + 1024);
  src += thcl_apply_config_defines();
  src += kSkeleton;
  src += kPrelude;
  src += "struct ThclUserOp {\n";
  src += "  static constexpr int NT = " + std::to_string(ntensors) + ";\n";
  src += "  static __device__ __forceinline__ void run(float &o_, float a_, float b_, float val1, float val2,\n";
  src += "                                             float p1_, float p2_) {\n";
  src += "    float *out = &o_; float *in1 = &a_; float *in2 = &b_;\n";
  src += "    const float *pointTensor1 = &p1_; const float *pointTensor2 = &p2_;\n";
  src += "    (void)out; (void)in1; (void)in2; (void)val1; (void)val2; (void)pointTensor1; (void)pointTensor2;\n";
  src += "    " + rewritten + ";\n";
  src += "  }\n};\n";
  static const char *const kFamilyMacro[] = {"THCL_DEFINE_APPLY_CONTIG_V4", "THCL_DEFINE_APPLY_CONTIG_S", "THCL_DEFINE_APPLY_JOINT_V4",
                                             "THCL_DEFINE_APPLY_JOINT_S",   "THCL_DEFINE_APPLY_GENERIC",  "THCL_DEFINE_APPLY_TILED"};
  THCL_CHECK(family >= -1 && family < 6, "internal: no kernel family %d", family);
  src += std::string(family < 0 ? "THCL_DEFINE_APPLY_KERNELS" : kFamilyMacro[family]) + "(" + thcl_expr_tag(rewritten, ntensors) +
         ", ThclUserOp, " + std::to_string(ntensors) + ")\n";
  return src;
}
