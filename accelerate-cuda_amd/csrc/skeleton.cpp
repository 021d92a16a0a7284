// Skeleton instantiation: scalar fragments + a hand-written gfx950 template
// -> one translation unit -> (cache | hiprtc) -> loaded module -> kernel record.
//
// This is the job CUDA/CodeGen.hs:91-136 (dispatch on the array operation),
// CUDA/CodeGen/Base.hs:69-89,262-383 (naming and ordering of kernel parameters)
// and CUDA/Compile.hs:444-459,484-566 (build1 / compile / link) do in the
// reference.  The templates themselves live in device/*.h.
#include <algorithm>
#include <cctype>
#include <cstdlib>
#include <cstring>
#include <sstream>

#include "skeleton.hpp"

namespace acc {

// ---- element types --------------------------------------------------------

int type_size(const std::string &t)
{
  static const struct { const char *name; int size; } table[] = {
      {"float", 4},   {"double", 8},  {"Int8", 1},     {"Int16", 2},    {"Int32", 4},   {"Int64", 8},
      {"Word8", 1},   {"Word16", 2},  {"Word32", 4},   {"Word64", 8},   {"int8_t", 1},  {"int16_t", 2},
      {"int32_t", 4}, {"int64_t", 8}, {"uint8_t", 1},  {"uint16_t", 2}, {"uint32_t", 4}, {"uint64_t", 8},
      {"char", 1},    {"short", 2},   {"int", 4},      {"unsigned", 4}, {"unsigned int", 4},
      {"long long", 8}, {"unsigned long long", 8}};
  for (const auto &e : table)
    if (t == e.name) return e.size;
  return 0;
}

static bool is_integer_type(const std::string &t)
{
  return type_size(t) != 0 && t != "float" && t != "double";
}

// one-line form of a fragment so that it can sit in a #define
static std::string flat(const char *s)
{
  std::string r = s ? s : "";
  for (char &c : r)
    if (c == '\n' || c == '\r') c = ' ';
  return r;
}

// "a, f(b, c), {d, e}" -> ["a", "f(b, c)", "{d, e}"]: split at the commas that lie inside no bracket
static std::vector<std::string> split_top_level(const std::string &text)
{
  std::vector<std::string> parts;
  std::string cur;
  int depth = 0;
  for (char c : text) {
    if (c == '(' || c == '{' || c == '[' || c == '<') ++depth;
    if (c == ')' || c == '}' || c == ']' || c == '>') --depth;
    if (c == ',' && depth == 0) {
      parts.push_back(cur);
      cur.clear();
    } else {
      cur.push_back(c);
    }
  }
  parts.push_back(cur);
  for (std::string &p : parts) {
    while (!p.empty() && std::isspace((unsigned char)p.front())) p.erase(p.begin());
    while (!p.empty() && std::isspace((unsigned char)p.back())) p.pop_back();
  }
  return parts;
}

// ---- parameter groups (CodeGen/Base.hs:69-89,348-383) ----------------------

static std::string env_params(const std::vector<EnvSig> &env)
{
  std::ostringstream o;
  for (size_t k = 0; k < env.size(); ++k) {
    for (int d = env[k].rank - 1; d >= 0; --d) o << "const Int64 shIn" << k << "_" << d << ", ";
    for (int c = env[k].ncomp - 1; c >= 0; --c)
      o << "const " << env[k].type[c] << " *__restrict__ arrIn" << k << "_" << c << ", ";
  }
  return o.str();
}

static std::string env_assume(const std::vector<EnvSig> &env, bool aligned)
{
  std::ostringstream o;
  for (size_t k = 0; k < env.size(); ++k) {
    for (int d = env[k].rank - 1; d >= 0; --d) o << "(void)shIn" << k << "_" << d << "; ";
    for (int c = env[k].ncomp - 1; c >= 0; --c) {
      if (aligned)
        o << "arrIn" << k << "_" << c << " = (const " << env[k].type[c] << " *)__builtin_assume_aligned(arrIn" << k
          << "_" << c << ", 16); ";
      else
        o << "(void)arrIn" << k << "_" << c << "; ";
    }
  }
  return o.str();
}

static std::string out_params(int rank, const std::string &elt)
{
  std::ostringstream o;
  for (int d = rank - 1; d >= 0; --d) o << "const Int64 shOut_" << d << ", ";
  (void)elt;
  o << "ACC_OUT_ARRAY(arrOut)";
  return o.str();
}

static std::string out_size(int rank)
{
  if (rank == 0) return "1";
  std::ostringstream o;
  o << "(";
  for (int d = rank - 1; d >= 0; --d) o << "shOut_" << d << (d ? " * " : "");
  o << ")";
  return o.str();
}

static const char *kind_name(int kind)
{
  static const char *names[] = {"map", "generate", "transform", "fold", "fold1", "foldSeg", "fold1Seg", "scanl",
                                "scanl1", "scanl'", "scanr", "scanr1", "scanr'", "permute", "stencil", "stencil2"};
  return (kind >= 0 && kind < ACC_SKEL_KIND_COUNT) ? names[kind] : "?";
}

// ---- the generator -------------------------------------------------------------

int generate_source(const SkelSpec &sp, bool aligned, std::string *entry, std::string *source)
{
  const Tuning &knobs = *sp.tuning;
  auto tune = [&](const char *name, int dflt) { return knobs.get(name, dflt); };
  auto tuned = [&](const char *name) { return knobs.has(name); };
  std::ostringstream o;
  int vec = std::max(1, 16 / std::max(1, sp.vec_size));
  o << "// accelerate-hip " ACC_HIP_VERSION " skeleton instance: " << kind_name(sp.kind) << "\n";
  o << "#define ACC_ELT " << sp.elt_type << "\n";
  // The result array(s): one pointer per component, highest component first (CodeGen/Base.hs:344-357).
  //   ACC_OUT_ARRAY(name)   the pointer parameters  name_<c>
  //   ACC_OUT_ASSUME(name)  16-byte alignment of each
  //   ACC_PUT(name, ix, v)  element ix := v, as a streaming store
  //   ACC_SET(name, ix, v)  the same as an ordinary store (small results that are read again soon)
  {
    const int nc = sp.comp_types.empty() ? 1 : (int)sp.comp_types.size();
    std::ostringstream arr, assume, put, set, read, read_dev, set_dev;
    for (int i = 0; i < nc; ++i) {
      const int c = nc - 1 - i;
      const std::string t = sp.comp_types.empty() ? std::string("ACC_ELT") : sp.comp_types[i];
      arr << (i ? ", " : "") << t << " *__restrict__ name##_" << c;
      assume << "name##_" << c << " = (" << t << " *)__builtin_assume_aligned(name##_" << c << ", 16); ";
      read << (i ? ", " : "") << "name##_" << c << "[ix]";
      read_dev << (i ? ", " : "") << "acc_load_device(name##_" << c << " + (ix))";
      if (sp.comp_types.empty()) {
        put << "acc_store(name##_0 + (ix), (v))";
        set << "name##_0[ix] = (v)";
        set_dev << "acc_store_device(name##_0 + (ix), (ACC_ELT)(v))";
      } else {
        put << "acc_store(name##_" << c << " + (ix), acc_pv.a" << c << "); ";
        set << "name##_" << c << "[ix] = acc_pv.a" << c << "; ";
        set_dev << "acc_store_device(name##_" << c << " + (ix), acc_pv.a" << c << "); ";
      }
    }
    o << "#define ACC_NCOMP " << nc << "\n";
    //   ACC_FOR_COMPONENTS(M)  M(c, type) for every component;  ACC_COMPONENT(v, c)  component c of the value v
    {
      std::ostringstream each;
      for (int i = 0; i < nc; ++i) each << "M(" << (nc - 1 - i) << ", " << (sp.comp_types.empty() ? std::string("ACC_ELT") : sp.comp_types[i]) << ") ";
      o << "#define ACC_FOR_COMPONENTS(M) " << each.str() << "\n";
      o << "#define ACC_COMPONENT(v, c) " << (sp.comp_types.empty() ? "(v)" : "((v).a##c)") << "\n";
    }
    //   ACC_READ(name, ix)    element ix, assembled from its components
    //   ACC_READ_DEVICE / ACC_SET_DEVICE: the same at device scope, past the caches (elements shared under a lock)
    if (sp.comp_types.empty()) {
      o << "#define ACC_READ(name, ix) (" << read.str() << ")\n";
      o << "#define ACC_READ_DEVICE(name, ix) (" << read_dev.str() << ")\n";
      o << "#define ACC_SET_DEVICE(name, ix, v) " << set_dev.str() << "\n";
    } else {
      o << "#define ACC_READ(name, ix) (ACC_ELT{" << read.str() << "})\n";
      o << "#define ACC_READ_DEVICE(name, ix) (ACC_ELT{" << read_dev.str() << "})\n";
      o << "#define ACC_SET_DEVICE(name, ix, v) do { const ACC_ELT acc_pv = (v); " << set_dev.str() << "} while (0)\n";
    }
    o << "#define ACC_OUT_ARRAY(name) " << arr.str() << "\n";
    o << "#define ACC_OUT_ASSUME(name) " << (aligned ? assume.str() : std::string()) << "\n";
    if (sp.comp_types.empty()) {
      o << "#define ACC_PUT(name, ix, v) " << put.str() << "\n";
      o << "#define ACC_SET(name, ix, v) " << set.str() << "\n";
    } else {
      o << "#define ACC_PUT(name, ix, v) do { const ACC_ELT acc_pv = (v); " << put.str() << "} while (0)\n";
      o << "#define ACC_SET(name, ix, v) do { const ACC_ELT acc_pv = (v); " << set.str() << "} while (0)\n";
    }
  }
  o << "#define ACC_ALIGNED " << (aligned ? 1 : 0) << "\n";
  o << "#define ACC_ENV_PARAMS " << env_params(sp.env) << "\n";
  o << "#define ACC_ENV_ASSUME " << env_assume(sp.env, aligned) << "\n";
  if (!sp.get.empty()) o << "#define ACC_GET(ix) " << sp.get << "\n";
  if (!sp.combine.empty()) o << "#define ACC_COMBINE(x, y) " << sp.combine << "\n";
  o << "#define ACC_HAS_SEED " << (sp.has_seed ? 1 : 0) << "\n";
  if (sp.has_seed) o << "#define ACC_SEED " << sp.seed << "\n";

  const char *tmpl = nullptr;
  switch (sp.kind) {
    case ACC_SKEL_MAP:
    case ACC_SKEL_GENERATE:
    case ACC_SKEL_TRANSFORM:
      *entry = kind_name(sp.kind);
      o << "#define ACC_OUT_PARAMS " << out_params(sp.out_rank, sp.elt_type) << "\n";
      o << "#define ACC_OUT_SIZE " << out_size(sp.out_rank) << "\n";
      o << "#define ACC_BLOCK " << sp.block << "\n#define ACC_VEC " << vec << "\n#define ACC_UNROLL " << sp.unroll << "\n";
      o << "#define ACC_MAP_TILED " << (sp.map_tiled ? 1 : 0) << "\n#define ACC_TT " << sp.map_tile_block << "\n";
      if (sp.map_tiled) {
        // the tiles' second dimension: its extent, and the elements between neighbours along it
        o << "#define ACC_TILE_H shOut_" << sp.map_tile_dim << "\n#define ACC_TILE_STRIDE (";
        for (int dd = 0; dd < sp.map_tile_dim; ++dd) o << (dd ? " * " : "") << "shOut_" << dd;
        o << ")\n";
      }
      tmpl = "skel_map.h";
      break;
    case ACC_SKEL_FOLD:
    case ACC_SKEL_FOLD1:
      if (sp.out_rank > 0) {
        // along the innermost dimension: the segmented fold over rows of one length
        *entry = sp.has_seed ? "fold" : "fold1";
        o << "#define ACC_SEG_UNIFORM 1\n";
        o << "#define ACC_TROUNDS " << tune("foldseg.team_rounds", 3) << "\n";
        if (tuned("foldseg.pad")) o << "#define ACC_PAD_ON " << (tune("foldseg.pad", 1) ? 1 : 0) << "\n";
        if (tuned("foldseg.wide")) o << "#define ACC_WIDE " << std::max(1, tune("foldseg.wide", 256)) << "\n";
        o << "#define ACC_FOLD_RIGHT " << ((sp.flags & ACC_FLAG_FOLD_RIGHT) ? 1 : 0) << "\n";
        o << "#define ACC_BLOCK " << sp.block << "\n#define ACC_VEC " << vec << "\n#define ACC_CHUNK " << sp.chunk << "\n";
        tmpl = "skel_foldseg.h";
        break;
      }
      *entry = sp.has_seed ? "foldAll" : "fold1All";
      o << "#define ACC_FOLD_SINGLE " << (sp.fold_single ? 1 : 0) << "\n";
      o << "#define ACC_BLOCK " << sp.block << "\n#define ACC_VEC " << vec << "\n#define ACC_UNROLL " << sp.unroll << "\n";
      tmpl = "skel_fold.h";
      break;
    case ACC_SKEL_FOLDSEG:
    case ACC_SKEL_FOLD1SEG:
      *entry = sp.has_seed ? "foldSeg" : "fold1Seg";
      o << "#define ACC_SEG_TYPE " << sp.seg_type << "\n";
      if (sp.out_rank >= 2) o << "#define ACC_SEG_OUTER 1\n";      // the segments of every outer row: Reduction.hs:473-474
      o << "#define ACC_TROUNDS " << tune("foldseg.team_rounds", 3) << "\n";
      if (tuned("foldseg.pad")) o << "#define ACC_PAD_ON " << (tune("foldseg.pad", 1) ? 1 : 0) << "\n";
      if (tuned("foldseg.wide")) o << "#define ACC_WIDE " << std::max(1, tune("foldseg.wide", 256)) << "\n";
      o << "#define ACC_FOLD_RIGHT " << ((sp.flags & ACC_FLAG_FOLD_RIGHT) ? 1 : 0) << "\n";
      o << "#define ACC_BLOCK " << sp.block << "\n#define ACC_VEC " << vec << "\n#define ACC_CHUNK " << sp.chunk << "\n";
      tmpl = "skel_foldseg.h";
      break;
    case ACC_SKEL_SCANL: case ACC_SKEL_SCANL1: case ACC_SKEL_SCANLP:
    case ACC_SKEL_SCANR: case ACC_SKEL_SCANR1: case ACC_SKEL_SCANRP: {
      const bool right = sp.kind >= ACC_SKEL_SCANR;
      int mode = 1;
      if (sp.kind == ACC_SKEL_SCANL) mode = 0;
      if (sp.kind == ACC_SKEL_SCANLP || sp.kind == ACC_SKEL_SCANRP) mode = 2;
      if (sp.kind == ACC_SKEL_SCANR) mode = 3;
      // entry names as the reference builds them: "scan" ++ dir ++ ("1" if seedless), PrefixSum.hs:311
      *entry = std::string("scan") + (right ? "r" : "l") + (sp.has_seed ? "" : "1");
      o << "#define ACC_SCAN_RIGHT " << (right ? 1 : 0) << "\n#define ACC_SCAN_MODE " << mode << "\n";
      o << "#define ACC_BLOCK " << sp.block << "\n#define ACC_VEC " << vec << "\n#define ACC_ROWS " << sp.rows << "\n";
      o << "#define ACC_LOOKBACK " << tune("scan.lookback", 1) << "\n";
      o << "#define ACC_DESC_STRIDE " << sp.scan_desc_stride << "\n";
      o << "#define ACC_MIN_WAVES " << tune("scan.min_waves", 1) << "\n";
      if (sp.scan_ticket) o << "#define ACC_SCAN_TICKET 1\n";
      tmpl = "skel_scan.h";
      break;
    }
    case ACC_SKEL_PERMUTE:
      *entry = "permute";
      o << "#define ACC_OUT_PARAMS " << out_params(sp.out_rank, sp.elt_type) << "\n";
      o << "#define ACC_OUT_SIZE " << out_size(sp.out_rank) << "\n";
      o << "#define ACC_PERMUTATION(ix) " << sp.permutation << "\n";
      o << "#define ACC_COMBINE_HINT " << (sp.permute_replace && !sp.permute_locked ? 7 : sp.combine_hint) << "\n";
      o << "#define ACC_PERMUTE_LOCKED " << (sp.permute_locked ? 1 : 0) << "\n";
      o << "#define ACC_PERMUTE_WINDOWS " << (sp.permute_windows ? 1 : 0) << "\n";
      o << "#define ACC_PERMUTE_NARROW " << (sp.permute_narrow ? 1 : 0) << "\n";
      if (sp.permute_narrow) o << "#define ACC_NARROW_STOP " << tune("permute.narrow_stop", 0xA000) << "u\n";
      if (sp.permute_narrow && tuned("permute.dump_vec")) o << "#define ACC_NARROW_DUMP_VEC " << (tune("permute.dump_vec", 1) ? 1 : 0) << "\n";
      if (sp.permute_narrow && tuned("permute.dump_nt")) o << "#define ACC_NARROW_DUMP_NT " << (tune("permute.dump_nt", 0) ? 1 : 0) << "\n";
      if (sp.permute_narrow && tuned("permute.merge_batch")) o << "#define ACC_MERGE_BATCH " << tune("permute.merge_batch", 16) << "\n";
      if (sp.permute_narrow) o << "#define ACC_MERGE_WAVES " << sp.merge_waves << "\n";
      if (tuned("permute.runs")) o << "#define ACC_RUNS " << tune("permute.runs", 1) << "\n";
      if (tuned("permute.gather")) o << "#define ACC_GATHER " << (tune("permute.gather", 1) ? 1 : 0) << "\n";
      o << "#define ACC_ELT_IS_INTEGER " << (is_integer_type(sp.elt_type) ? 1 : 0) << "\n";
      o << "#define ACC_BLOCK " << sp.block << "\n#define ACC_VEC " << vec << "\n#define ACC_UNROLL " << sp.unroll << "\n";
      tmpl = "skel_permute.h";
      break;
    case ACC_SKEL_STENCIL:
    case ACC_SKEL_STENCIL2: {
      const bool two = sp.kind == ACC_SKEL_STENCIL2;
      *entry = two ? "stencil2" : "stencil";
      if (sp.stencil_nd) {
        // an element a thread, any rank and reach (skel_stencil_nd.h)
        const int rank = sp.out_rank;
        o << "#define ACC_OUT_PARAMS " << out_params(rank, sp.elt_type) << "\n";
        o << "#define ACC_STENCIL_RANK " << rank << "\n";
        if (tuned("stencil.nd_inner")) o << "#define ACC_ND_INNER " << (tune("stencil.nd_inner", 1) ? 1 : 0) << "\n";
        o << "#define ACC_STENCIL_SOURCES " << (two ? 2 : 1) << "\n";
        o << "#define ACC_OUT_EXTENTS";
        for (int dd = rank - 1; dd >= 0; --dd) o << " shOut_" << dd << (dd ? "," : "");
        o << "\n";
        auto source_nd = [&](const char *which, const char *tap_name, const std::string &elt_name, const std::vector<std::string> &comps,
                             const std::string &constant, const std::vector<int> &off, const char *array_name, bool with_extents) -> int {
          const int nc = (int)comps.size();
          std::vector<std::string> consts = split_top_level(constant);
          if (consts.empty() || (consts.size() == 1 && consts[0].empty())) consts.assign(nc, "0");
          if ((int)consts.size() != nc)
            return fail(ACC_ERR_INVALID, "stencil: the boundary constant has %d component(s), the source element has %d", (int)consts.size(), nc);
          o << "#define ACC_SRC" << which << "_COMPONENTS(X, arg)";
          for (int i = 0; i < nc; ++i) o << " X(" << (nc - 1 - i) << ", " << comps[i] << ", (" << consts[i] << "), arg)";
          o << "\n";
          o << "#define ACC_SRC" << which << "_PARAMS";
          if (with_extents)
            for (int dd = rank - 1; dd >= 0; --dd) o << " , const Int64 sh" << array_name << "_" << dd;
          for (int i = 0; i < nc; ++i) o << " , const " << comps[i] << " *__restrict__ arr" << array_name << "_" << (nc - 1 - i);
          o << "\n";
          // a stencil's one source has the result's extents; each source of a stencil2 its own
          o << "#define ACC_SRC" << which << "_EXTENTS";
          for (int dd = rank - 1; dd >= 0; --dd) o << " sh" << (with_extents ? array_name : "Out") << "_" << dd << (dd ? "," : "");
          o << "\n";
          o << "#define ACC_IN" << which << "_ELT " << (nc == 1 ? comps[0] : elt_name) << "\n";
          const size_t ntaps = off.size() / (size_t)rank;
          // how far the taps reach towards the beginning and the end of every dimension (outermost first)
          for (const char *side : {"LO", "HI"}) {
            o << "#define ACC_SRC" << which << "_REACH_" << side << " {";
            for (int dd = 0; dd < rank; ++dd) {
              int most = 0;
              for (size_t k = 0; k < ntaps; ++k) most = std::max(most, side[0] == 'L' ? -off[k * rank + dd] : off[k * rank + dd]);
              o << (dd ? ", " : "") << most;
            }
            o << "}\n";
          }
          o << "#define ACC_STENCIL_TAPS" << which << "_ND(READ) ";
          for (size_t k = 0; k < ntaps; ++k) {
            o << "const ACC_IN" << which << "_ELT " << tap_name << k << " = ";
            if (nc > 1) o << "{ ";
            for (int i = 0; i < nc; ++i) {
              o << (i ? ", " : "") << "READ(" << (nc - 1 - i);
              for (int dd = 0; dd < rank; ++dd) o << ", " << off[k * rank + dd];
              o << ")";
            }
            if (nc > 1) o << " }";
            o << "; ";
          }
          o << "\n";
          return ACC_OK;
        };
        ACC_TRY(source_nd("1", "t", "acc_in1_elt", sp.stencil_in_comps, sp.boundary_constant, sp.tap_off, two ? "Stencil1" : "Stencil", two));
        o << "#define ACC_BOUNDARY " << sp.boundary << "\n";
        if (two) {
          o << "#define ACC_BOUNDARY2 " << sp.boundary2 << "\n";
          ACC_TRY(source_nd("2", "u", "acc_in2_elt", sp.stencil_in2_comps, sp.boundary2_constant, sp.tap2_off, "Stencil2", true));
        }
        o << "#define ACC_STENCIL_FN " << sp.stencil_fn << "\n";
        o << "#define ACC_BLOCK " << sp.block << "\n";
        tmpl = "skel_stencil_nd.h";
        break;
      }
      int rz = 0, ry = 0, rx = 0;
      for (size_t k = 0; k < sp.tap_dy.size(); ++k) {
        rz = std::max(rz, std::abs(sp.tap_dz[k]));
        ry = std::max(ry, std::abs(sp.tap_dy[k]));
        rx = std::max(rx, std::abs(sp.tap_dx[k]));
      }
      for (size_t k = 0; k < sp.tap2_dy.size(); ++k) {
        rz = std::max(rz, std::abs(sp.tap2_dz[k]));
        ry = std::max(ry, std::abs(sp.tap2_dy[k]));
        rx = std::max(rx, std::abs(sp.tap2_dx[k]));
      }
      o << "#define ACC_OUT_PARAMS " << out_params(sp.out_rank, sp.elt_type) << "\n";
      o << "#define ACC_STENCIL_RANK " << sp.out_rank << "\n";
      o << "#define ACC_STENCIL_SOURCES " << (two ? 2 : 1) << "\n";
      o << "#define ACC_RADIUS_Z " << rz << "\n#define ACC_RADIUS_Y " << ry << "\n#define ACC_RADIUS_X " << rx << "\n";
      o << "#define ACC_BOUNDARY " << sp.boundary << "\n";
      // A source is one array per component of its element (Stencil/Extra.hs:53-128 reads every component of a tuple
      // array).  Per source the template gets: the list of its components -- number, type, value outside the array
      // under a constant boundary -- highest component first; its kernel parameters in that order; and one binding
      // per tap, read through whatever accessor the template passes, a struct of the components for a tuple.
      auto source = [&](const char *which, const char *tap_name, const std::string &elt_name, const std::vector<std::string> &comps,
                        const std::string &constant, const std::vector<int> &dz, const std::vector<int> &dy, const std::vector<int> &dx,
                        const char *array_name, bool with_extents) -> int {
        const int nc = (int)comps.size();
        std::vector<std::string> consts = split_top_level(constant);
        if (consts.empty() || (consts.size() == 1 && consts[0].empty())) consts.assign(nc, "0");
        if ((int)consts.size() != nc)
          return fail(ACC_ERR_INVALID, "stencil: the boundary constant has %d component(s), the source element has %d", (int)consts.size(), nc);
        o << "#define ACC_SRC" << which << "_COMPONENTS(X, arg)";
        for (int i = 0; i < nc; ++i) o << " X(" << (nc - 1 - i) << ", " << comps[i] << ", (" << consts[i] << "), arg)";
        o << "\n";
        o << "#define ACC_SRC" << which << "_PARAMS";
        if (with_extents)
          for (int dd = sp.out_rank - 1; dd >= 0; --dd) o << " , const Int64 sh" << array_name << "_" << dd;
        for (int i = 0; i < nc; ++i) o << " , const " << comps[i] << " *__restrict__ arr" << array_name << "_" << (nc - 1 - i);
        o << "\n";
        o << "#define ACC_IN" << which << "_ELT " << (nc == 1 ? comps[0] : elt_name) << "\n";
        o << "#define ACC_STENCIL_TAPS" << which << "(READ) ";
        for (size_t k = 0; k < dy.size(); ++k) {
          o << "const ACC_IN" << which << "_ELT " << tap_name << k << " = ";
          if (nc > 1) o << "{ ";
          for (int i = 0; i < nc; ++i)
            o << (i ? ", " : "") << "READ(" << (nc - 1 - i) << ", " << dz[k] << ", " << dy[k] << ", " << dx[k] << ")";
          if (nc > 1) o << " }";
          o << "; ";
        }
        o << "\n";
        return ACC_OK;
      };
      ACC_TRY(source("1", "t", "acc_in1_elt", sp.stencil_in_comps, sp.boundary_constant, sp.tap_dz, sp.tap_dy, sp.tap_dx,
                     two ? "Stencil1" : "Stencil", two));
      if (two) {
        o << "#define ACC_BOUNDARY2 " << sp.boundary2 << "\n";
        ACC_TRY(source("2", "u", "acc_in2_elt", sp.stencil_in2_comps, sp.boundary2_constant, sp.tap2_dz, sp.tap2_dy, sp.tap2_dx,
                       "Stencil2", true));
      }
      o << "#define ACC_STENCIL_FN " << sp.stencil_fn << "\n";
      o << "#define ACC_XCD_REMAP " << tune("stencil.xcd_remap", 0) << "\n";
      o << "#define ACC_STENCIL_NT " << tune("stencil.nt", 1) << "\n";
      o << "#define ACC_SCHED_BARRIER " << tune("stencil.sched_barrier", 3) << "\n";
      o << "#define ACC_SVEC " << sp.svec << "\n";
      o << "#define ACC_SHIFT_MIN " << tune("stencil.shift_min", sp.zmarch ? 1 : 24 * sp.svec) << "\n";
      o << "#define ACC_CUT_MIN " << tune("stencil.cut_min", sp.zmarch ? sp.svec : 16 * sp.svec) << "\n";
      o << "#define ACC_STACK_WAVES " << (sp.out_rank == 2 ? tune("stencil.stack", 0) : 0) << "\n";
      o << "#define ACC_TILE_H " << sp.tile_h << "\n#define ACC_PREFETCH " << sp.prefetch << "\n#define ACC_BLOCK " << sp.block << "\n";
      o << "#define ACC_TZ " << sp.tile_z << "\n";
      o << "#define ACC_ZMARCH " << sp.zmarch << "\n";
      tmpl = "skel_stencil.h";
      break;
    }
    default:
      return fail(ACC_ERR_INVALID, "unknown skeleton kind %d", sp.kind);
  }
  o << "#define ACC_ENTRY " << *entry << "\n";
  o << "#define ACC_NT_STORE " << tune("nt_store", 1) << "\n";
  if (sp.foldseg_giants) o << "#define ACC_GIANTS 1\n";
  if (tuned("foldseg.giant_chunks")) o << "#define ACC_GIANT_CHUNKS " << std::max(1, tune("foldseg.giant_chunks", 4)) << "\n";
  if (tuned("stream.policy")) o << "#define ACC_STREAM_POLICY " << tune("stream.policy", 1) << "\n";
  if (sp.guarded) o << "#define ACC_GUARDED 1\n";
  if (tuned("spin_limit")) o << "#define ACC_SPIN_LIMIT " << std::max(0, tune("spin_limit", 1 << 22)) << "\n";
  o << "#include \"acc_hip_device.h\"\n";
  if (!sp.comp_types.empty()) {
    // a tuple element: fields a<c>, component 0 last, so that brace initialisation reads like the tuple
    o << "struct acc_elt { ";
    const int nc = (int)sp.comp_types.size();
    for (int i = 0; i < nc; ++i) o << sp.comp_types[i] << " a" << (nc - 1 - i) << "; ";
    o << "};\n";
  }
  // a stencil source of tuple type: its taps are values of a struct of their own
  auto in_struct = [&](const char *name, const std::vector<std::string> &comps) {
    if (comps.size() < 2) return;
    o << "struct " << name << " { ";
    const int nc = (int)comps.size();
    for (int i = 0; i < nc; ++i) o << comps[i] << " a" << (nc - 1 - i) << "; ";
    o << "};\n";
  };
  if (sp.kind == ACC_SKEL_STENCIL || sp.kind == ACC_SKEL_STENCIL2) {
    in_struct("acc_in1_elt", sp.stencil_in_comps);
    in_struct("acc_in2_elt", sp.stencil_in2_comps);
  }
  if (!sp.preamble.empty()) o << sp.preamble << "\n";
  o << "#include \"" << tmpl << "\"\n";
  *source = o.str();
  return ACC_OK;
}

// ---- description -> spec ---------------------------------------------------------

// `text` is an integer literal 0..3, possibly parenthesised and cast: "1", "((Int32)(1))", "(Int64)1u"
static bool small_literal(std::string t)
{
  t.erase(std::remove_if(t.begin(), t.end(), [](unsigned char c) { return std::isspace(c); }), t.end());
  for (bool again = true; again && !t.empty();) {
    again = false;
    if (t.front() == '(' && t.back() == ')') {         // one pair around everything?
      int depth = 0;
      size_t k = 0;
      for (; k < t.size(); ++k) {
        depth += (t[k] == '(') - (t[k] == ')');
        if (depth == 0) break;
      }
      if (k == t.size() - 1) { t = t.substr(1, t.size() - 2); again = true; continue; }
    }
    if (t.front() == '(') {                            // a cast: "(Name)" followed by the rest
      size_t k = 1;
      while (k < t.size() && (std::isalnum((unsigned char)t[k]) || t[k] == '_')) ++k;
      if (k > 1 && k < t.size() - 1 && t[k] == ')') { t = t.substr(k + 1); again = true; }
    }
  }
  while (!t.empty() && (t.back() == 'u' || t.back() == 'U' || t.back() == 'l' || t.back() == 'L')) t.pop_back();
  return t.size() == 1 && t[0] >= '0' && t[0] <= '3';
}

// elements a workgroup of the segmented fold stages at a time: a whole number of its block-wide vector loads (a lane
// loads 16 bytes, so 16 elements of one byte: one load of 256 lanes is then 4096 of them)
static int segmented_chunk(const SkelSpec &sp, bool long_segments = false)
{
  auto tune = [&](const char *name, int dflt) { return sp.tuning->get(name, dflt); };
  const int per_load = sp.block * std::max(1, 16 / std::max(1, sp.vec_size));
  const int want = std::max(long_segments ? tune("foldseg.chunk_long", 3072) : tune("foldseg.chunk", 2048), per_load);
  return (want + per_load - 1) / per_load * per_load;
}

int make_spec(const acc_skel_desc *d, const TuningPtr &tuning, SkelSpec *sp)
{
  if (!d) return fail(ACC_ERR_INVALID, "NULL skeleton description");
  sp->tuning = tuning ? tuning : default_tuning();
  const Tuning &knobs = *sp->tuning;
  auto tune = [&](const char *name, int dflt) { return knobs.get(name, dflt); };
  auto tuned = [&](const char *name) { return knobs.has(name); };
  if (d->kind < 0 || d->kind >= ACC_SKEL_KIND_COUNT) return fail(ACC_ERR_INVALID, "unknown skeleton kind %d", d->kind);
  if (!d->elt_type || !*d->elt_type) return fail(ACC_ERR_INVALID, "skeleton description: elt_type missing");
  if (d->n_env < 0 || (d->n_env > 0 && !d->env)) return fail(ACC_ERR_INVALID, "skeleton description: bad env");
  sp->kind = d->kind;
  sp->flags = d->flags;
  sp->elt_type = d->elt_type;
  if (sp->elt_type.find(',') != std::string::npos) {
    // a tuple: "T<n-1>, ..., T0"; laid out as the struct the generator declares
    size_t pos = 0;
    int size = 0, align = 1;
    while (pos <= sp->elt_type.size()) {
      size_t end = sp->elt_type.find(',', pos);
      if (end == std::string::npos) end = sp->elt_type.size();
      std::string t = sp->elt_type.substr(pos, end - pos);
      t.erase(0, t.find_first_not_of(" \t"));
      t.erase(t.find_last_not_of(" \t") + 1);
      const int ts = type_size(t);
      if (ts <= 0) return fail(ACC_ERR_INVALID, "tuple element type: unknown component type '%s'", t.c_str());
      sp->comp_types.push_back(t);
      size = (size + ts - 1) / ts * ts + ts;
      align = std::max(align, ts);
      sp->vec_size = std::max(sp->vec_size, ts);
      pos = end + 1;
    }
    if ((int)sp->comp_types.size() > ACC_MAX_COMP) return fail(ACC_ERR_INVALID, "tuple element type: more than %d components", ACC_MAX_COMP);
    sp->elt_size = (size + align - 1) / align * align;
    sp->elt_type = "acc_elt";
    // a stencil may produce tuples; its sources are arrays of scalars, whose type must then be given
    if ((d->kind == ACC_SKEL_STENCIL || d->kind == ACC_SKEL_STENCIL2) && !(d->stencil_in_type && *d->stencil_in_type))
      return fail(ACC_ERR_INVALID, "%s: a tuple result needs `stencil_in_type` (the sources are arrays of scalars)", kind_name(d->kind));
    if (d->kind == ACC_SKEL_STENCIL2 && !(d->stencil_in2_type && *d->stencil_in2_type))
      return fail(ACC_ERR_INVALID, "stencil2: a tuple result needs `stencil_in2_type`");
  } else {
    sp->elt_size = d->elt_size > 0 ? d->elt_size : type_size(sp->elt_type);
    if (sp->elt_size <= 0) return fail(ACC_ERR_INVALID, "cannot size element type '%s': set elt_size", d->elt_type);
    sp->vec_size = sp->elt_size;
  }
  sp->guarded = (d->flags & ACC_FLAG_GUARDED) != 0;
  sp->map_tile_block = std::max(1, std::min(tune("map.tile_block", 4), 8));
  sp->map_tiled = (d->flags & ACC_FLAG_TILED) != 0 && d->out_rank >= 2 &&
                  (d->kind == ACC_SKEL_MAP || d->kind == ACC_SKEL_GENERATE || d->kind == ACC_SKEL_TRANSFORM) && tune("map.tiled", 1) != 0;
  sp->map_tile_dim = (int)((d->flags >> 8) & 15u);
  if (sp->map_tile_dim == 0) sp->map_tile_dim = 1;
  if (sp->map_tiled && sp->map_tile_dim >= d->out_rank)
    return fail(ACC_ERR_INVALID, "%s: ACC_FLAG_TILE_DIM(%d) on a result of rank %d", kind_name(d->kind), sp->map_tile_dim, d->out_rank);
  sp->fold_across = (d->flags & ACC_FLAG_TILED) != 0 && d->out_rank >= 1 && (d->kind == ACC_SKEL_FOLD || d->kind == ACC_SKEL_FOLD1);
  sp->out_rank = d->out_rank;
  if (sp->out_rank < 0 || sp->out_rank > ACC_MAX_RANK) return fail(ACC_ERR_INVALID, "bad out_rank %d", d->out_rank);
  for (int k = 0; k < d->n_env; ++k) {
    const acc_env_sig &e = d->env[k];
    if (e.rank < 0 || e.rank > ACC_MAX_RANK || e.ncomp < 1 || e.ncomp > ACC_MAX_COMP)
      return fail(ACC_ERR_INVALID, "env array %d: bad rank/ncomp", k);
    EnvSig s;
    s.rank = e.rank;
    s.ncomp = e.ncomp;
    for (int c = 0; c < e.ncomp; ++c) {
      if (!e.type[c] || !*e.type[c]) return fail(ACC_ERR_INVALID, "env array %d: component %d has no type", k, c);
      s.type.push_back(e.type[c]);
    }
    sp->env.push_back(s);
  }
  sp->preamble = d->preamble ? d->preamble : "";
  sp->get = flat(d->get);
  sp->get_small_constant = small_literal(sp->get);
  sp->combine = flat(d->combine);
  sp->has_seed = d->seed && *d->seed;
  sp->seed = flat(d->seed);
  sp->permutation = flat(d->permutation);
  sp->combine_hint = d->combine_hint;
  sp->seg_type = (d->seg_type && *d->seg_type) ? d->seg_type : "Int32";

  const bool needs_get = d->kind != ACC_SKEL_STENCIL && d->kind != ACC_SKEL_STENCIL2;
  if (needs_get && sp->get.empty()) return fail(ACC_ERR_INVALID, "%s: `get` fragment missing", kind_name(d->kind));
  const bool needs_combine = d->kind >= ACC_SKEL_FOLD && d->kind <= ACC_SKEL_PERMUTE;
  if (needs_combine && sp->combine.empty()) return fail(ACC_ERR_INVALID, "%s: `combine` fragment missing", kind_name(d->kind));

  switch (d->kind) {
    case ACC_SKEL_FOLD: case ACC_SKEL_FOLDSEG: case ACC_SKEL_SCANL: case ACC_SKEL_SCANLP:
    case ACC_SKEL_SCANR: case ACC_SKEL_SCANRP:
      if (!sp->has_seed) return fail(ACC_ERR_INVALID, "%s: `seed` fragment missing", kind_name(d->kind));
      break;
    case ACC_SKEL_FOLD1: case ACC_SKEL_FOLD1SEG: case ACC_SKEL_SCANL1: case ACC_SKEL_SCANR1:
      if (sp->has_seed) return fail(ACC_ERR_INVALID, "%s takes no seed", kind_name(d->kind));
      break;
    default:
      break;
  }

  sp->block = 256;
  sp->unroll = 4;
  sp->rows = 4;
  sp->chunk = 4096;
  switch (d->kind) {
    case ACC_SKEL_MAP: case ACC_SKEL_GENERATE: case ACC_SKEL_TRANSFORM:
      sp->block = tune("map.block", 256);
      sp->unroll = tune("map.unroll", 1);
      break;
    case ACC_SKEL_FOLD: case ACC_SKEL_FOLD1:
      sp->block = tune("fold.block", 256);
      sp->unroll = tune("fold.unroll", 4);
      sp->fold_single = tune("fold.single", 1) != 0;
      if (sp->out_rank > 0) {
        sp->block = tune("foldseg.block", 256);
        sp->chunk = segmented_chunk(*sp);
        sp->chunk_long = segmented_chunk(*sp, true);
      }
      break;
    case ACC_SKEL_FOLDSEG: case ACC_SKEL_FOLD1SEG:
      sp->block = tune("foldseg.block", 256);
      sp->chunk = segmented_chunk(*sp);
      sp->chunk_long = segmented_chunk(*sp, true);
      break;
    case ACC_SKEL_PERMUTE:
      if (sp->permutation.empty()) return fail(ACC_ERR_INVALID, "permute: `permutation` fragment missing");
      if (sp->out_rank < 1) return fail(ACC_ERR_UNSUPPORTED, "permute into a rank-0 array is not supported");   // IndexSpace.hs:230
      if (sp->combine_hint < ACC_COMBINE_GENERIC || sp->combine_hint > ACC_COMBINE_XOR)
        return fail(ACC_ERR_INVALID, "permute: bad combine_hint %d", sp->combine_hint);
      // no atomic read-modify-write covers a tuple or an element of another size than 4 or 8 bytes:
      // those go through a lock per target, as every permute does in the reference (IndexSpace.hs:285-303)
      sp->permute_locked = !sp->comp_types.empty() || (sp->elt_size != 4 && sp->elt_size != 8);
      {
        // `permute const`: the combination is the new value, whatever its spelling's blanks and brackets
        std::string c = d->combine ? d->combine : "";
        c.erase(std::remove_if(c.begin(), c.end(), [](unsigned char ch) { return std::isspace(ch) || ch == '(' || ch == ')'; }), c.end());
        // (a tuple's spelling: its components, first to last)
        std::string whole = "acc_elt{";
        for (size_t k = sp->comp_types.size(); k-- > 0;) whole += "x.a" + std::to_string(k) + (k ? "," : "}");
        sp->permute_replace = sp->combine_hint == ACC_COMBINE_GENERIC && (c == "x" || (!sp->comp_types.empty() && c == whole)) &&
                              tune("permute.replace", 1) != 0;
      }
      if (sp->permute_locked && sp->combine_hint != ACC_COMBINE_GENERIC)
        return fail(ACC_ERR_INVALID, "permute: combine_hint needs a 4- or 8-byte single-component element");
      if (sp->combine_hint >= ACC_COMBINE_AND && !is_integer_type(sp->elt_type))
        return fail(ACC_ERR_INVALID, "permute: bitwise combine_hint on non-integer element type '%s'", sp->elt_type.c_str());
      sp->block = tune("permute.block", 1024);
      sp->merge_waves = std::max(4, std::min(16, tune("permute.merge_waves", 4)));
      sp->unroll = tune("permute.unroll", 2);
      break;
    case ACC_SKEL_STENCIL:
    case ACC_SKEL_STENCIL2: {
      if (sp->out_rank < 1) return fail(ACC_ERR_INVALID, "stencil: rank %d", sp->out_rank);
      if (!d->stencil_fn || !*d->stencil_fn) return fail(ACC_ERR_INVALID, "stencil: `stencil_fn` fragment missing");
      // The taps of one source: as rows of out_rank offsets (`offs`, any rank), or as up to three lists (dz, dy, dx).
      // Either way they end up in both forms: (oz, oy, ox) for the strips of skel_stencil.h, `all` for the template
      // that takes any rank and reach, and `beyond` says that only the latter will do.
      const int rank = sp->out_rank;
      bool beyond = rank > 3 || tune("stencil.nd", 0) != 0;
      auto taps = [&](int n, const int32_t *offs, const int32_t *dzs, const int32_t *dys, const int32_t *dxs, int boundary,
                      std::vector<int> *oz, std::vector<int> *oy, std::vector<int> *ox, std::vector<int> *all) -> int {
        // (a 9 x 9 x 9 neighbourhood, the widest the array language's stencil patterns describe in three dimensions)
        if (n < 1 || n > 729 || (!offs && !dxs)) return fail(ACC_ERR_INVALID, "stencil: bad tap list");
        if (!offs && rank > 3) return fail(ACC_ERR_INVALID, "stencil: a stencil of rank %d gives its taps as `tap_offsets`", rank);
        if (boundary < ACC_BOUNDARY_CLAMP || boundary > ACC_BOUNDARY_CONSTANT) return fail(ACC_ERR_INVALID, "stencil: bad boundary %d", boundary);
        for (int k = 0; k < n; ++k) {
          int o[ACC_MAX_RANK] = {0};
          if (offs) {
            for (int dd = 0; dd < rank; ++dd) o[dd] = offs[k * rank + dd];
          } else {
            o[rank - 1] = dxs[k];
            if (rank >= 2) o[rank - 2] = dys ? dys[k] : 0;
            if (rank == 3) o[0] = dzs ? dzs[k] : 0;
          }
          for (int dd = 0; dd < rank; ++dd) {
            if (std::abs(o[dd]) > 64) return fail(ACC_ERR_INVALID, "stencil: a tap %d elements away", o[dd]);
            all->push_back(o[dd]);
          }
          const int dx = o[rank - 1], dy = rank >= 2 ? o[rank - 2] : 0, dz = rank == 3 ? o[0] : 0;
          if (std::abs(dy) > 4 || std::abs(dx) > 4 || std::abs(dz) > 2) beyond = true;      // more than a strip's register windows hold
          oz->push_back(dz);
          oy->push_back(dy);
          ox->push_back(dx);
        }
        return ACC_OK;
      };
      ACC_TRY(taps(d->n_taps, d->tap_offsets, d->tap_dz, d->tap_dy, d->tap_dx, d->boundary, &sp->tap_dz, &sp->tap_dy, &sp->tap_dx, &sp->tap_off));
      sp->boundary = d->boundary;
      sp->boundary_constant = flat(d->boundary_constant);
      sp->stencil_fn = flat(d->stencil_fn);
      sp->stencil_in_type = (d->stencil_in_type && *d->stencil_in_type) ? d->stencil_in_type : sp->elt_type;
      // "T<n-1>, ..., T0": a source of tuples, one array per component (as for elt_type)
      auto in_comps = [&](const std::string &type, std::vector<std::string> *comps, const char *what) -> int {
        *comps = split_top_level(type);
        if (comps->empty() || (int)comps->size() > ACC_MAX_COMP) return fail(ACC_ERR_INVALID, "stencil: %s has too many components", what);
        for (const std::string &c : *comps)
          if (c.empty() || type_size(c) <= 0) return fail(ACC_ERR_INVALID, "stencil: cannot size component '%s' of %s", c.c_str(), what);
        return ACC_OK;
      };
      ACC_TRY(in_comps(sp->stencil_in_type, &sp->stencil_in_comps, "stencil_in_type"));
      if (d->kind == ACC_SKEL_STENCIL2) {
        ACC_TRY(taps(d->n_taps2, d->tap2_offsets, d->tap2_dz, d->tap2_dy, d->tap2_dx, d->boundary2, &sp->tap2_dz, &sp->tap2_dy, &sp->tap2_dx, &sp->tap2_off));
        sp->boundary2 = d->boundary2;
        sp->boundary2_constant = flat(d->boundary2_constant);
        sp->stencil_in2_type = (d->stencil_in2_type && *d->stencil_in2_type) ? d->stencil_in2_type : sp->elt_type;
        ACC_TRY(in_comps(sp->stencil_in2_type, &sp->stencil_in2_comps, "stencil_in2_type"));
      }
      sp->block = tune("stencil.block", 256);
      sp->stencil_nd = beyond;
      if (sp->stencil_nd) {              // an element a thread: no strips to shape
        sp->svec = 1;
        sp->tile_w = sp->block;
        sp->tile_h = 1;
        break;
      }
      // Columns a lane holds of every row: four, or two of an element of 8 bytes -- one 128-bit access either way, and
      // half the registers for the row windows, so that strips stay as tall as for narrower elements (Float64, 3 x 3
      // on 8192^2: 202.7 -> 174.6 us; 7 points on 256 x 512 x 512: 249.5 -> 190.3) -- unless the stencil reaches
      // further to either side than that (the neighbouring lane supplies those columns).  Eight columns of 1- and
      // 2-byte elements are no gain (an element takes a register whatever its width: Word16 3 x 3 43.1 -> 57.9 us).
      {
        int widest = 1, reach_x = 0;
        for (const std::string &c : sp->stencil_in_comps) widest = std::max(widest, type_size(c));
        for (const std::string &c : sp->stencil_in2_comps) widest = std::max(widest, type_size(c));
        for (int t : sp->tap_dx) reach_x = std::max(reach_x, std::abs(t));
        for (int t : sp->tap2_dx) reach_x = std::max(reach_x, std::abs(t));
        const int svec = (widest >= 8 && reach_x <= 2) ? 2 : 4;
        sp->svec = tune("stencil.svec", svec);
        sp->reach_x = reach_x;
        if (sp->svec != 1 && sp->svec != 2 && sp->svec != 4 && sp->svec != 8) return fail(ACC_ERR_INVALID, "stencil: %d columns a lane", sp->svec);
        if (sp->svec < reach_x) return fail(ACC_ERR_INVALID, "stencil: a reach of %d columns with %d columns a lane", reach_x, sp->svec);
      }
      sp->tile_w = 64 * sp->svec;                        // one wave's strip
      sp->prefetch = sp->out_rank == 2 ? tune("stencil.prefetch", 3) : (sp->out_rank == 3 ? tune("stencil.prefetch3", 1) : 0);
      // 3-D: a strip that reaches across planes produces up to three planes of the result from one register window
      // (each source row it fetches then serves several planes instead of one), as many as keep the window of all
      // sources within 128 registers a lane
      int planes_per_strip = 1;
      int rz = 0, ry = 0, rx = 0;        // both sources' windows span the larger of the two radii
      if (sp->out_rank == 3) {
        auto reach = [&](const std::vector<int> &dz, const std::vector<int> &dy, const std::vector<int> &dx) {
          for (size_t k = 0; k < dx.size(); ++k) { rz = std::max(rz, std::abs(dz[k])); ry = std::max(ry, std::abs(dy[k])); rx = std::max(rx, std::abs(dx[k])); }
        };
        reach(sp->tap_dz, sp->tap_dy, sp->tap_dx);
        reach(sp->tap2_dz, sp->tap2_dy, sp->tap2_dx);
        int words = 0;
        for (const std::string &c : sp->stencil_in_comps) words += std::max(1, (type_size(c) + 3) / 4);
        for (const std::string &c : sp->stencil_in2_comps) words += std::max(1, (type_size(c) + 3) / 4);
        // Taps in other planes: the strip walks through the planes instead of down the rows, so that a row fetched once
        // serves all the planes that read it; it is as many rows tall as keep the windows within 144 registers
        // (2 ry + rows of them side by side, 2 rz + 1 + prefetch planes deep); within 192 for elements of two words or
        // more, which would otherwise get strips one row tall that read every row three times (Float64, 7 points,
        // 256 x 512 x 512: 249.5 us; two rows tall, 207 registers, 231.5).
        sp->zmarch = (rz > 0 && 2 * rx * (2 * ry + 1) <= 64) ? (tune("stencil.zmarch", 1) ? 1 : 0) : 0;
        if (sp->zmarch) {
          for (int ty = 4; ty > 1 && planes_per_strip == 1; --ty)
            if ((2 * ry + ty) * (2 * rz + 1 + sp->prefetch) * (sp->svec + 2 * rx) * words <= (words > 1 ? 192 : 144)) planes_per_strip = ty;
          while (2 * rx * (2 * ry + planes_per_strip) > 64) --planes_per_strip;     // one lane each for the elements outside the strip
        } else {
          for (int tz = 3; rz > 0 && tz > 1 && planes_per_strip == 1; --tz)
            if ((2 * rz + tz) * (2 * ry + 1 + sp->prefetch) * (sp->svec + 2 * rx) * words <= 128) planes_per_strip = tz;
        }
      }
      sp->tile_z = sp->out_rank == 3 ? tune("stencil.tile_z", planes_per_strip) : 1;
      // rows per strip: short in 2-D (a compact window of the image in flight), taller in 3-D where every row is
      // read from 2 rz + tile_z planes and the boundary rows of a strip cost that much more; planes per walk where
      // the strip goes through planes
      sp->tile_h = sp->out_rank == 2 ? tune("stencil.tile_h", 4)
                 : (sp->out_rank == 3 ? (sp->zmarch ? tune("stencil.walk", 64) : tune("stencil.tile_h3", sp->tile_z > 1 ? 8 : 16)) : 1);
      if (sp->zmarch && 2 * rx * (2 * ry + sp->tile_z) > 64) return fail(ACC_ERR_INVALID, "stencil: strip too tall for its reach");
      if (sp->tile_h < 1 || sp->prefetch < 0 || sp->prefetch > 8 || sp->tile_z < 1 || sp->tile_z > 8) return fail(ACC_ERR_INVALID, "stencil: bad tile shape");
      break;
    }
    default:   // scans
      // A tile of 128 KB either way (32 Ki Int32).  Four waves with up to 32 rows a lane leave room for two workgroups
      // on a compute unit, one loading while the other stores, as long as the instance keeps within 256 registers;
      // where it does not (operators that need temporaries) the first build falls back to sixteen waves with a
      // quarter of the rows (acc_skel_s::ensure_variant).  A shape given by hand is taken as it is.
      {
        const int vec = std::max(1, 16 / std::max(1, sp->vec_size));                                       // elements per lane and row
        const int per_row = std::max(1, vec * std::max(1, sp->elt_size));                                  // bytes of them
        // (an element takes a register whatever its width: no more than 128 of them a lane, 32 on sixteen waves)
        const int rows4 = std::max(2, std::min({32, 131072 / (256 * per_row), 128 / vec}));
        sp->scan_desc_stride = std::max(1, tune("scan.desc_stride", 16));
        sp->scan_shape_open = !tuned("scan.block") && !tuned("scan.rows");
        sp->scan_rows_fallback = std::max(2, std::min({8, 131072 / (1024 * per_row), 32 / vec}));
        sp->block = tune("scan.block", sp->scan_shape_open ? 256 : 1024);
        sp->rows = tune("scan.rows", sp->scan_shape_open ? rows4 : sp->scan_rows_fallback);
        sp->scan_small_rows = std::max(0, std::min(tune("scan.small_rows", 4), 32));
        sp->scan_ticket = tune("scan.ticket", 0) != 0;
      }
      break;
  }
  if (sp->block < 64 || sp->block > 1024 || (sp->block & 63)) return fail(ACC_ERR_INVALID, "block size %d is not a multiple of the 64-lane wavefront", sp->block);
  return ACC_OK;
}

std::vector<std::string> compile_options(const SkelSpec &sp)
{
  std::vector<std::string> o = {"-O3", "-std=c++17"};
  // scalar operations round one at a time, as the interpreter evaluates them,
  // unless the caller asks otherwise
  o.push_back((sp.flags & ACC_FLAG_FAST_MATH) ? "-ffp-contract=fast" : "-ffp-contract=off");
  // no packed two-lane Float32 instructions: scalar code stays scalar
  for (const char *f : {"-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"}) o.push_back(f);
  return o;
}

}  // namespace acc

using acc::fail;

// ---- acc_skel_s ----------------------------------------------------------------

namespace acc {
// what variant v of an instance is generated from (variants beyond 1 exist for permute only)
SkelSpec spec_of_variant(const SkelSpec &base, int v)
{
  SkelSpec spec = base;
  if (spec.kind == ACC_SKEL_PERMUTE) {
    if (v >= 2 && v < 4) spec.permute_locked = true;
    if (v >= 4 && v < 6) spec.permute_windows = true;
    if (v >= 6) spec.permute_narrow = true;
  }
  // a map in tiles: its variants 2 and 3 are the same map in runs, for results too thin for tiles
  if (spec.map_tiled && v >= 2) spec.map_tiled = false;
  // a segmented fold's variants 2 and 3 (6 and 7): a longer staged chunk, for segments of 8 elements or more on
  // average; 4 to 7: what is left of a very long segment is handed over to a second launch
  if (spec.kind != ACC_SKEL_PERMUTE && (v & 2) && spec.chunk_long > 0) spec.chunk = spec.chunk_long;
  if ((spec.kind == ACC_SKEL_FOLDSEG || spec.kind == ACC_SKEL_FOLD1SEG) && spec.out_rank <= 1 && v >= 4) spec.foldseg_giants = true;
  // a stencil's variants 2 and 3, 4 and 5: half and a quarter of the columns a lane, for arrays narrower than half or a
  // quarter of a strip, whose lanes would otherwise mostly lie outside the array
  // ... and 6 and 7: an element a thread (the form of stencils that strips cannot take), for arrays of a few columns,
  // where nearly every lane of a strip would lie outside the array
  if ((spec.kind == ACC_SKEL_STENCIL || spec.kind == ACC_SKEL_STENCIL2) && v >= 6 && !spec.stencil_nd) {
    spec.stencil_nd = true;
    spec.svec = 1;
    spec.tile_w = spec.block;
    spec.tile_h = 1;
  } else if ((spec.kind == ACC_SKEL_STENCIL || spec.kind == ACC_SKEL_STENCIL2) && v >= 2 && !spec.stencil_nd) {
    spec.svec = std::max(1, spec.svec >> (v / 2));
    spec.tile_w = 64 * spec.svec;
  }
  // a scan's variants 2 and 3: a small tile, for arrays of a few tiles at most (a lone workgroup runs through the
  // instructions of all its rows one after the other whether the array fills them or not)
  if (spec.scan_small_rows > 0 && v >= 2) {
    spec.block = std::min(spec.block, 256);
    spec.rows = std::min(spec.rows, spec.scan_small_rows);
  }
  return spec;
}
}  // namespace acc

// the job that compiles variant v (not yet started); fills in the variant's source and entry name
static int make_job(acc_skel_s *s, int v, std::shared_ptr<acc::CompileJob> *out)
{
  acc::Variant &var = s->variants[v];
  const acc::SkelSpec spec = acc::spec_of_variant(s->spec, v);
  ACC_TRY(acc::generate_source(spec, (v & 1) == 0, &var.entry, &var.source));
  if (s->entry.empty()) s->entry = var.entry;      // the same for every variant; set once, before the instance is shared
  auto job = std::make_shared<acc::CompileJob>();
  job->target = s->ctx->arch;
  job->source = var.source;
  job->options = acc::compile_options(spec);
  *out = job;
  return ACC_OK;
}

int acc_skel_s::start_variant(int v)
{
  std::lock_guard<std::mutex> lock(mu);
  acc::Variant &var = variants[v];
  if (var.ready || var.job) return ACC_OK;
  std::shared_ptr<acc::CompileJob> job;
  ACC_TRY(make_job(this, v, &job));
  if (acc::compile_submit(job)) var.job = job;      // else: compiled by the thread that first needs it
  return ACC_OK;
}

bool acc_skel_s::variant_compiled(int v)
{
  std::shared_ptr<acc::CompileJob> job;
  {
    std::lock_guard<std::mutex> lock(mu);
    if (variants[v].ready) return true;
    job = variants[v].job;
  }
  if (!job) return false;
  std::lock_guard<std::mutex> lock(job->mu);
  return job->done;
}

int acc_skel_s::ensure_variant(int v)
{
  // two threads may meet here on the first launch that needs the unaligned variant
  std::unique_lock<std::mutex> lock(mu);
  acc::Variant &var = variants[v];
  if (var.ready) return ACC_OK;
  // variants 2 and 3 of a permute: the locked template for an element the atomic template also covers
  acc::SkelSpec spec = acc::spec_of_variant(this->spec, v);
  if (!var.job) {                       // nobody has started it: this thread compiles
    std::shared_ptr<acc::CompileJob> job;
    ACC_TRY(make_job(this, v, &job));
    var.job = job;
    job->run();
  }
  // a kernel's first use: here the reference blocks on the compilation it started earlier (Compile.hs:451-457);
  // a failure is reported to every caller that comes by, with the compiler's log
  ACC_TRY(var.job->wait());
  const std::string entry_name = var.entry;
  const void *code = var.job->code;
  ACC_TRY(ctx->make_current());
  ACC_HIP_TRY(hipModuleLoadData(&var.module, code));
  hipError_t e = hipModuleGetFunction(&var.fn, var.module, entry_name.c_str());
  if (e != hipSuccess) {
    (void)hipModuleUnload(var.module);
    var.module = nullptr;
    return acc::fail_hip(e, ("hipModuleGetFunction(" + entry_name + ")").c_str());
  }
  const bool segmented = spec.kind == ACC_SKEL_FOLDSEG || spec.kind == ACC_SKEL_FOLD1SEG ||
                         ((spec.kind == ACC_SKEL_FOLD || spec.kind == ACC_SKEL_FOLD1) && spec.out_rank > 0);
  const bool two_kernels = ((spec.kind == ACC_SKEL_FOLD || spec.kind == ACC_SKEL_FOLD1) && spec.out_rank == 0) ||
                           spec.kind == ACC_SKEL_PERMUTE || segmented;
  const std::string second = entry_name + (spec.kind == ACC_SKEL_PERMUTE ? (spec.permute_locked ? "_join" : "_merge") : segmented ? "_team" : "_finish");
  if (two_kernels) {
    e = hipModuleGetFunction(&var.fn_finish, var.module, second.c_str());
    if (e != hipSuccess) {
      (void)hipModuleUnload(var.module);
      var.module = nullptr;
      return acc::fail_hip(e, ("hipModuleGetFunction(" + second + ")").c_str());
    }
  }
  if ((spec.kind == ACC_SKEL_PERMUTE && !spec.permute_locked) || segmented) {
    const std::string third = entry_name + (segmented ? "_join" : "_fill");
    e = hipModuleGetFunction(&var.fn_fill, var.module, third.c_str());
    if (e != hipSuccess) {
      (void)hipModuleUnload(var.module);
      var.module = nullptr;
      return acc::fail_hip(e, ("hipModuleGetFunction(" + third + ")").c_str());
    }
  }
  if (spec.kind == ACC_SKEL_PERMUTE && spec.permute_locked) {
    // `permute const` without locks: see skel_permute.h
    for (const char *name : {"permute_claim", "permute_place"}) {
      e = hipModuleGetFunction(name[8] == 'c' ? &var.fn_claim : &var.fn_place, var.module, name);
      if (e != hipSuccess) {
        (void)hipModuleUnload(var.module);
        var.module = nullptr;
        return acc::fail_hip(e, (std::string("hipModuleGetFunction(") + name + ")").c_str());
      }
    }
  }
  if ((spec.kind == ACC_SKEL_FOLDSEG || spec.kind == ACC_SKEL_FOLD1SEG) && spec.out_rank <= 1) {
    // variants 4 to 7: the launch that takes what was handed over; 0 to 3: the look at the segment lengths
    const std::string sweep = entry_name + (spec.foldseg_giants ? "_sweep" : "_probe");
    e = hipModuleGetFunction(&var.fn_sweep, var.module, sweep.c_str());
    if (e != hipSuccess) {
      (void)hipModuleUnload(var.module);
      var.module = nullptr;
      return acc::fail_hip(e, ("hipModuleGetFunction(" + sweep + ")").c_str());
    }
  }
  if ((spec.kind == ACC_SKEL_FOLD || spec.kind == ACC_SKEL_FOLD1) && spec.out_rank > 0) {
    const std::string rows = entry_name + "_rows";
    e = hipModuleGetFunction(&var.fn_rows, var.module, rows.c_str());
    if (e != hipSuccess) {
      (void)hipModuleUnload(var.module);
      var.module = nullptr;
      return acc::fail_hip(e, ("hipModuleGetFunction(" + rows + ")").c_str());
    }
    const std::string across = entry_name + "_across";
    e = hipModuleGetFunction(&var.fn_across, var.module, across.c_str());
    if (e != hipSuccess) {
      (void)hipModuleUnload(var.module);
      var.module = nullptr;
      return acc::fail_hip(e, ("hipModuleGetFunction(" + across + ")").c_str());
    }
  }
  (void)hipFuncGetAttribute(&var.num_regs, HIP_FUNC_ATTRIBUTE_NUM_REGS, var.fn);
  var.block = spec.block;
  var.rows = spec.rows;
  if (this->spec.scan_shape_open && v < 2) {
    // the first build of a scan decides its tile shape: see make_spec
    this->spec.scan_shape_open = false;
    if (var.num_regs > 256) {
      (void)hipModuleUnload(var.module);
      var = acc::Variant();                   // (its job goes with it: the next build starts from the new shape)
      this->spec.block = 1024;
      this->spec.rows = this->spec.scan_rows_fallback;
      lock.unlock();
      return ensure_variant(v);
    }
  }
  (void)hipFuncGetAttribute(&var.static_lds, HIP_FUNC_ATTRIBUTE_SHARED_SIZE_BYTES, var.fn);
  int bpc = 0;
  e = hipModuleOccupancyMaxActiveBlocksPerMultiprocessor(&bpc, var.fn, spec.block, 0);
  if (e != hipSuccess || bpc < 1) { (void)hipGetLastError(); bpc = 1; }
  var.blocks_per_cu = bpc;
  var.ready = true;
  return ACC_OK;
}

// how many variants an instance of this kind has (the numbering of acc_skel_preview)
static int variant_count(const acc::SkelSpec &sp)
{
  const bool stencil = sp.kind == ACC_SKEL_STENCIL || sp.kind == ACC_SKEL_STENCIL2;
  if ((sp.kind == ACC_SKEL_FOLDSEG || sp.kind == ACC_SKEL_FOLD1SEG) && sp.out_rank <= 1) return 8;
  if (sp.map_tiled) return 4;
  return sp.kind == ACC_SKEL_PERMUTE ? 8 : (stencil ? (sp.stencil_nd ? 2 : 8) : ((sp.scan_small_rows > 0 || sp.chunk_long > 0) ? 4 : 2));
}

extern "C" {

int acc_skel_create_async(acc_context ctx, const acc_skel_desc *desc, acc_skel *out)
{
  if (!ctx || !out) return fail(ACC_ERR_INVALID, "acc_skel_create: NULL argument");
  *out = nullptr;
  acc::SkelSpec sp;
  ACC_TRY(acc::make_spec(desc, ctx->tuning_now(), &sp));
  acc_skel_s *s = new acc_skel_s();
  s->ctx = ctx;
  s->spec = sp;
  s->knobs.resolve(*sp.tuning);
  if ((sp.kind == ACC_SKEL_FOLDSEG || sp.kind == ACC_SKEL_FOLD1SEG) && sp.out_rank <= 1 && ctx->status_host) {
    s->hint_slot = static_cast<int>(ctx->next_hint.fetch_add(1) % acc::HINT_WORDS);
    __atomic_store_n(const_cast<uint32_t *>(ctx->status_host) + acc::STATUS_WORDS + s->hint_slot, 0u, __ATOMIC_RELAXED);
  }
  const int rc = s->start_variant(0);     // the other variants are built when a call first needs them
  if (rc != ACC_OK) { delete s; return rc; }
  *out = s;
  return ACC_OK;
}

int acc_skel_create(acc_context ctx, const acc_skel_desc *desc, acc_skel *out)
{
  acc_skel s = nullptr;
  ACC_TRY(acc_skel_create_async(ctx, desc, &s));
  const int rc = s->ensure_variant(0);
  if (rc != ACC_OK) { acc_skel_destroy(s); return rc; }
  *out = s;
  return ACC_OK;
}

int acc_skel_prefetch(acc_skel s, int variant)
{
  if (!s) return fail(ACC_ERR_INVALID, "acc_skel_prefetch: NULL skeleton");
  if (variant < 0 || variant >= variant_count(s->spec))
    return fail(ACC_ERR_INVALID, "acc_skel_prefetch: this kind of skeleton has variants 0 to %d", variant_count(s->spec) - 1);
  // (the locked form of a permute is only generated for elements the atomic template does not take, and the other way round)
  if (s->spec.kind == ACC_SKEL_PERMUTE && s->spec.permute_locked && variant >= 2)
    return fail(ACC_ERR_INVALID, "acc_skel_prefetch: a permute under locks has variants 0 and 1");
  return s->start_variant(variant);
}

int acc_skel_wait(acc_skel s)
{
  if (!s) return fail(ACC_ERR_INVALID, "acc_skel_wait: NULL skeleton");
  return s->ensure_variant(0);
}

int acc_skel_poll(acc_skel s, int *ready)
{
  if (!s || !ready) return fail(ACC_ERR_INVALID, "acc_skel_poll: NULL argument");
  std::shared_ptr<acc::CompileJob> job;
  {
    std::lock_guard<std::mutex> lock(s->mu);
    if (s->variants[0].ready) { *ready = 1; return ACC_OK; }
    job = s->variants[0].job;
  }
  *ready = 0;
  if (job) {
    std::lock_guard<std::mutex> lock(job->mu);
    *ready = job->done ? 1 : 0;
  }
  return ACC_OK;
}

int acc_compile_threads(void) { return acc::compile_pool_threads(); }

int acc_compile_drain(void)
{
  acc::compile_drain();
  return ACC_OK;
}

int acc_skel_destroy(acc_skel s)
{
  if (!s) return ACC_OK;
  (void)s->ctx->make_current();
  for (acc::Variant &v : s->variants)
    if (v.module) (void)hipModuleUnload(v.module);
  delete s;
  return ACC_OK;
}

int acc_skel_source(acc_skel s, int variant, const char **source)
{
  if (!s || !source || variant < 0 || variant > 1) return fail(ACC_ERR_INVALID, "acc_skel_source: bad argument");
  std::lock_guard<std::mutex> lock(s->mu);
  if (s->variants[variant].source.empty()) {
    std::string e;
    ACC_TRY(acc::generate_source(s->spec, variant == 0, &e, &s->variants[variant].source));
  }
  *source = s->variants[variant].source.c_str();
  return ACC_OK;
}

int acc_skel_preview(const acc_skel_desc *desc, int variant, const char **source, const char **entry)
{
  static thread_local std::string text, name;
  if (!source || variant < 0 || variant > 7) return fail(ACC_ERR_INVALID, "acc_skel_preview: bad argument");
  acc::SkelSpec sp;
  ACC_TRY(acc::make_spec(desc, acc::default_tuning(), &sp));
  // beyond 1: a permute's forms (to 7), a stencil's fewer columns a lane (to 5), a scan's small tiles and a segmented
  // fold's longer chunk (2 and 3)
  const int most = variant_count(sp) - 1;
  if (variant > most) return fail(ACC_ERR_INVALID, "acc_skel_preview: this kind of skeleton has variants 0 to %d", most);
  ACC_TRY(acc::generate_source(acc::spec_of_variant(sp, variant), (variant & 1) == 0, &name, &text));
  *source = text.c_str();
  if (entry) *entry = name.c_str();
  return ACC_OK;
}

int acc_skel_compile_only(const char *target, const acc_skel_desc *desc, size_t *code_size)
{
  if (!target) return fail(ACC_ERR_INVALID, "acc_skel_compile_only: NULL target");
  acc::SkelSpec sp;
  ACC_TRY(acc::make_spec(desc, acc::default_tuning(), &sp));
  std::vector<std::string> opts = acc::compile_options(sp);
  // both variants at once, on the worker pool (a helper process each)
  size_t total = 0;
  std::shared_ptr<acc::CompileJob> jobs[2];
  for (int v = 0; v < 2; ++v) {
    std::string entry;
    jobs[v] = std::make_shared<acc::CompileJob>();
    ACC_TRY(acc::generate_source(sp, v == 0, &entry, &jobs[v]->source));
    jobs[v]->target = target;
    jobs[v]->options = opts;
    if (!acc::compile_submit(jobs[v])) jobs[v]->run();
  }
  for (int v = 0; v < 2; ++v) {
    ACC_TRY(jobs[v]->wait());
    total += jobs[v]->size;
  }
  if (code_size) *code_size = total;
  return ACC_OK;
}

int acc_skel_get_info(acc_skel s, acc_skel_info *out)
{
  if (!s || !out) return fail(ACC_ERR_INVALID, "acc_skel_get_info: NULL argument");
  ACC_TRY(s->ensure_variant(0));          // the record of a kernel that is still being compiled: wait for it
  std::memset(out, 0, sizeof(*out));
  std::snprintf(out->entry, sizeof(out->entry), "%s", s->entry.c_str());
  out->block = s->spec.block;
  out->blocks_per_cu = s->variants[0].blocks_per_cu;
  out->num_regs = s->variants[0].num_regs;
  out->static_lds = s->variants[0].static_lds;
  out->elements_per_block = s->elements_per_block();
  return ACC_OK;
}

}  // extern "C"
