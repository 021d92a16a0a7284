// Skeleton instances: what acc_skel_create builds and acc_exec_* run.
#pragma once
#include "acc_internal.hpp"

namespace acc {

struct EnvSig {
  int rank = 0;
  int ncomp = 1;
  std::vector<std::string> type;
};

// the validated, owned form of an acc_skel_desc plus the tuning of its template
struct SkelSpec {
  TuningPtr tuning;                     // the knobs the generator reads (never NULL once make_spec has run)
  int kind = 0;
  uint32_t flags = 0;
  std::vector<EnvSig> env;
  std::string elt_type;                 // C type of the element; "acc_elt" for a tuple
  int elt_size = 0;                     // sizeof(elt_type)
  std::vector<std::string> comp_types;  // tuple elements: the component types, left to right (component ncomp-1 first)
  int vec_size = 0;                     // bytes of the widest component: decides how many elements a lane takes per access
  int out_rank = 0;
  std::string preamble, get, combine, seed, permutation;
  bool has_seed = false;
  int combine_hint = 0;
  bool permute_windows = false;         // hinted permute over several LDS windows of targets (variants 4 and 5)
  bool get_small_constant = false;      // `get` is a literal 0..3 (under casts and parentheses): a permute that counts
  bool permute_narrow = false;          // integer addition with 16-bit counts in LDS (variants 6 and 7)
  bool permute_locked = false;          // permute of an element no atomic covers (tuples, 1/2/16-byte types): per-target locks
  std::string seg_type;
  // stencil
  int boundary = 0;
  std::string boundary_constant, stencil_fn, stencil_in_type;
  std::vector<std::string> stencil_in_comps, stencil_in2_comps;   // the sources' element types by component, highest first
  std::vector<int> tap_dz, tap_dy, tap_dx;
  // stencil2: the second source
  int boundary2 = 0;
  std::string boundary2_constant, stencil_in2_type;
  std::vector<int> tap2_dz, tap2_dy, tap2_dx;
  bool stencil_nd = false;              // an element a thread (skel_stencil_nd.h): rank > 3, or taps further away than the strips' windows hold
  std::vector<int> tap_off, tap2_off;   // ... its taps: n_taps rows of out_rank offsets, outermost dimension first
  int tile_w = 256, tile_h = 4, prefetch = 3;
  int svec = 4;                         // stencils: columns a lane holds of every row (tile_w = 64 of them)
  int reach_x = 0;                      // stencils: the furthest a tap reaches to either side
  int tile_z = 1;                       // rank-3 stencils: result planes per strip (rows per strip where the strip walks through planes)
  int zmarch = 0;                       // rank-3 stencils: strips tile_z rows tall walk through tile_h planes
  // tuning
  int block = 256, unroll = 4, rows = 4, chunk = 4096;
  int merge_waves = 4;                  // permute of 16-bit counts: waves of a workgroup of permute_merge
  int chunk_long = 0;                   // segmented folds: the staged chunk of variants 2 and 3 (segments of 8 elements or more on average); 0: none
  bool fold_across = false;             // ACC_FLAG_TILED on a fold along the innermost dimension: neighbouring rows are neighbours in memory
  bool permute_replace = false;         // permute whose combination is spelt `x` (the new value): plain stores
  int map_tile_dim = 1;                 // ACC_FLAG_TILE_DIM: which dimension of the result, counted from the innermost, the tiles pair with it
  bool map_tiled = false;               // ACC_FLAG_TILED on a map of rank 2 or more: tiles of 32 x 32 elements, a wave each
  int map_tile_block = 4;               // ... a lane's share of a tile: a block of that many elements either way
  bool guarded = false;                 // ACC_FLAG_GUARDED: every kernel takes the address of a loop's guard word last
  bool foldseg_giants = false;          // a segmented fold's variants 4-7: very long segments are handed over to a second launch (skel_foldseg.h)
  bool fold_single = true;              // foldAll in one launch (the last workgroup collects), as generated into the kernel
  int scan_rows_fallback = 8;
  int scan_small_rows = 0;              // rows a lane of a scan's small-tile variants (2 and 3); 0: none
  int scan_desc_stride = 16;            // 8-byte words between the tile descriptors of a scan, as generated into the kernel
  bool scan_ticket = false;             // measurement: tiles drawn from a counter instead of numbered by workgroup (knob scan.ticket)
  bool scan_shape_open = false;         // a scan whose tile shape the first build may still change (by its register count)
};

// one compiled form of an instance: AccKernel of the reference (AST.hs:51-59)
struct Variant {
  bool ready = false;
  std::string source;
  hipModule_t module = nullptr;
  hipFunction_t fn = nullptr;
  hipFunction_t fn_finish = nullptr;   // second kernel: foldAll's _finish, permute's _merge / _join, the segmented fold's _team
  hipFunction_t fn_fill = nullptr;     // third kernel: permute's _fill (identity into the table rows), the segmented fold's _join
  hipFunction_t fn_rows = nullptr;     // fold along the innermost dimension: _rows, a lane per short row
  hipFunction_t fn_claim = nullptr;    // a permute under locks: permute_claim and permute_place, for a combination that is the new value
  hipFunction_t fn_place = nullptr;
  hipFunction_t fn_across = nullptr;   // fold along the innermost dimension: _across, a lane per row of any length
  hipFunction_t fn_sweep = nullptr;    // a segmented fold's variants 4-7: _sweep, the segments that were handed over;
                                       // its variants 0-3: _probe, a look at the segment lengths
  int num_regs = 0;
  int static_lds = 0;
  int blocks_per_cu = 1;
  int block = 0;                       // workgroup size and rows a lane of this variant was built with (a scan's small
  int rows = 0;                        // variant differs from the instance's)
  std::shared_ptr<CompileJob> job;     // its compilation, once started: in the background, or by the thread that needs it
  std::string entry;                   // the main kernel's name in `job`'s code
};

int type_size(const std::string &t);
int make_spec(const acc_skel_desc *d, const TuningPtr &tuning, SkelSpec *sp);
int generate_source(const SkelSpec &sp, bool aligned, std::string *entry, std::string *source);
SkelSpec spec_of_variant(const SkelSpec &base, int variant);
std::vector<std::string> compile_options(const SkelSpec &sp);

}  // namespace acc

struct acc_skel_s {
  acc_context ctx = nullptr;
  acc::SkelSpec spec;
  acc::Knobs knobs;           // what the drivers read of the tuning table
  std::string entry;
  acc::Variant variants[8];   // [0] pointers 16-byte aligned, [1] no assumption; [2], [3]: the same for the
                              // table-in-LDS form of a permute whose combination has no atomic instruction;
                              // [4], [5]: for a hinted permute over several LDS windows of targets;
                              // [6], [7]: for integer addition on a table of 16-bit counts in LDS;
                              // of a segmented fold [2], [3]: a longer staged chunk, [4]-[7]: the same four with the table of
                              // jobs for very long segments; of a scan [2], [3]: small tiles;
                              // of a stencil [2], [3] and [4], [5]: half and a quarter of the columns a lane, [6], [7]: an
                              // element a thread
  int hint_slot = -1;         // a segmented fold: its word among the context's hints (its segments were looked at: a very long one)
  std::atomic<bool> met_giants{false};   // ... and that the word has been seen set
  std::atomic<unsigned> seg_calls{0};    // ... and how often it has been launched (the look happens on calls 1, 2, 4, 8 ...)
  std::mutex mu;

  // variant v compiled, loaded and measured; compiles on the calling thread unless a job for it is under way
  int ensure_variant(int v);
  // start variant v's compilation on the worker pool (nothing if it has been started or is ready)
  int start_variant(int v);
  bool variant_ready(int v) { std::lock_guard<std::mutex> lock(mu); return variants[v].ready; }
  // ... or its compilation has ended, so that ensure_variant would not wait for the compiler
  bool variant_compiled(int v);
  int ncomp() const { return spec.comp_types.empty() ? 1 : (int)spec.comp_types.size(); }
  int vec() const { int v = 16 / (spec.vec_size > 0 ? spec.vec_size : 1); return v < 1 ? 1 : v; }
  int elements_per_block() const
  {
    switch (spec.kind) {
      case ACC_SKEL_SCANL: case ACC_SKEL_SCANL1: case ACC_SKEL_SCANLP:
      case ACC_SKEL_SCANR: case ACC_SKEL_SCANR1: case ACC_SKEL_SCANRP:
        return spec.block * spec.rows * vec();
      case ACC_SKEL_STENCIL:
      case ACC_SKEL_STENCIL2:
        return spec.tile_w * spec.tile_h * (spec.block / 64);
      case ACC_SKEL_FOLDSEG: case ACC_SKEL_FOLD1SEG:
        return spec.block;   // segments per block
      default:
        return spec.block * spec.unroll * vec();
    }
  }
};
