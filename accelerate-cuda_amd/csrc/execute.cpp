// Skeleton drivers: allocate the temporaries a skeleton needs, marshal its
// arguments, pick the launch shape and enqueue the kernel(s).
//
// These are the roles of executeOp / foldCore / foldSegOp / scanCore /
// permuteOp / stencilOp in CUDA/Execute.hs:264-450, of the argument
// marshalling at :823-909,930-982 and of the launch arithmetic in
// CUDA/Analysis/Launch.hs:42-172 -- re-derived for 64-lane wavefronts, 256
// compute units and single-pass kernels (one launch where the reference needs
// two or three).
#include <algorithm>
#include <cstdlib>
#include <cstring>
#include <deque>

#include "skeleton.hpp"

using acc::fail;

namespace {

// Kernel arguments in launch order.  Every argument of these kernels is at
// most 8 bytes, so each gets one 8-byte slot whose address is handed to HIP.
// What the driver that is running on this thread launches for: the instance's entry name (for the launch trace) and,
// for an instance built with ACC_FLAG_GUARDED, the address of the guard word that every one of its kernels takes as
// its last parameter (0: no loop).
struct Running {
  const char *entry = "";
  bool dump_exec = false;     // the context was created under ACC_HIP_DEBUG=dump-exec
  bool guarded = false;
  uint64_t guard = 0;
};
thread_local Running t_run;

class Args {
 public:
  void i64(int64_t v) { push(&v, sizeof(v)); }
  void u32(uint32_t v) { push(&v, sizeof(v)); }
  void i32(int32_t v) { push(&v, sizeof(v)); }
  void ptr(uint64_t v) { push(&v, sizeof(v)); }
  size_t count() const { return slots_.size(); }
  // the arguments as HIP wants them, the guard's address appended for a guarded instance
  void **data()
  {
    if (t_run.guarded && !guard_pushed_) {
      ptr(t_run.guard);
      guard_pushed_ = true;
    }
    return data_without_guard();
  }
  // (for a launch whose last arguments are not 8-byte slots: the caller appends them, then the guard)
  void **data_without_guard()
  {
    ptrs_.clear();
    for (uint64_t &s : slots_) ptrs_.push_back(&s);
    return ptrs_.data();
  }

 private:
  void push(const void *p, size_t n)
  {
    uint64_t s = 0;
    std::memcpy(&s, p, n);
    slots_.push_back(s);
  }
  std::deque<uint64_t> slots_;
  std::vector<void *> ptrs_;
  bool guard_pushed_ = false;
};

// Every kernel launch of the drivers.  ACC_HIP_DEBUG=dump-exec prints one line per launch -- entry<<<grid, block,
// lds>>> and the time on the device -- as the reference's -ddump-exec does (Debug.hs:41-76, hooked at
// Execute.hs:975-982); timing a launch means waiting for it, so the trace serialises the stream.
// acc_trace_start .. acc_trace_stop on a thread: an event before and one behind every launch it makes
struct Trace {
  bool on = false;
  std::vector<std::pair<hipEvent_t, hipEvent_t>> spans;
};
thread_local Trace t_trace;

hipError_t launch_kernel(hipFunction_t f, unsigned gx, unsigned gy, unsigned gz, unsigned bx, unsigned by, unsigned bz, unsigned lds,
                         hipStream_t st, void **args, void **extra)
{
  if (t_trace.on) {
    hipEvent_t e0 = nullptr, e1 = nullptr;
    const bool timed = hipEventCreate(&e0) == hipSuccess && hipEventCreate(&e1) == hipSuccess && hipEventRecord(e0, st) == hipSuccess;
    const hipError_t rc = hipModuleLaunchKernel(f, gx, gy, gz, bx, by, bz, lds, st, args, extra);
    if (timed && rc == hipSuccess && hipEventRecord(e1, st) == hipSuccess) {
      t_trace.spans.emplace_back(e0, e1);
    } else {
      if (e0) (void)hipEventDestroy(e0);
      if (e1) (void)hipEventDestroy(e1);
    }
    return rc;
  }
  if (!t_run.dump_exec) return hipModuleLaunchKernel(f, gx, gy, gz, bx, by, bz, lds, st, args, extra);
  hipEvent_t e0 = nullptr, e1 = nullptr;
  const bool timed = hipEventCreate(&e0) == hipSuccess && hipEventCreate(&e1) == hipSuccess && hipEventRecord(e0, st) == hipSuccess;
  const hipError_t rc = hipModuleLaunchKernel(f, gx, gy, gz, bx, by, bz, lds, st, args, extra);
  float ms = -1.0f;
  if (timed && rc == hipSuccess && hipEventRecord(e1, st) == hipSuccess && hipEventSynchronize(e1) == hipSuccess)
    (void)hipEventElapsedTime(&ms, e0, e1);
  const char *name = hipKernelNameRef(f);
  std::fprintf(stderr, "[acc-hip exec] %s: %s<<<%u, %u, %u>>> gpu: %.3f ms%s\n", t_run.entry, name ? name : "?", gx, bx, lds, ms,
               rc == hipSuccess ? "" : " FAILED");
  if (e0) (void)hipEventDestroy(e0);
  if (e1) (void)hipEventDestroy(e1);
  (void)hipGetLastError();
  return rc;
}

int64_t array_size(const acc_array &a)
{
  int64_t n = 1;
  for (int d = 0; d < a.rank; ++d) n *= a.shape[d];
  return n;
}

bool aligned16(uint64_t p) { return (p & 15u) == 0; }

// free array variables first, in Gamma order; per array the extents outermost
// first, then the component pointers highest component first
// (CodeGen/Base.hs:344-357, Execute.hs:835-836,946-951)
int push_env(const acc_skel_s *s, const acc_array *env, Args *args, bool *aligned)
{
  const std::vector<acc::EnvSig> &sig = s->spec.env;
  if (!sig.empty() && !env) return fail(ACC_ERR_INVALID, "%s: env arrays missing", s->entry.c_str());
  for (size_t k = 0; k < sig.size(); ++k) {
    const acc_array &a = env[k];
    if (a.rank != sig[k].rank || a.ncomp != sig[k].ncomp)
      return fail(ACC_ERR_INVALID, "%s: env array %zu has rank %d / %d components, the kernel was built for %d / %d",
                  s->entry.c_str(), k, a.rank, a.ncomp, sig[k].rank, sig[k].ncomp);
    int64_t n = 1;
    for (int d = 0; d < a.rank; ++d) {
      if (a.shape[d] < 0) return fail(ACC_ERR_INVALID, "%s: env array %zu has a negative extent", s->entry.c_str(), k);
      n *= a.shape[d];
      args->i64(a.shape[d]);
    }
    for (int c = a.ncomp - 1; c >= 0; --c) {
      if (!a.ptr[c] && n > 0) return fail(ACC_ERR_INVALID, "%s: env array %zu component %d is NULL", s->entry.c_str(), k, c);
      if (!aligned16(a.ptr[c])) *aligned = false;
      args->ptr(a.ptr[c]);
    }
  }
  return ACC_OK;
}

int check_out(const acc_skel_s *s, const acc_array *out, int rank, const char *what, int ncomp)
{
  if (!out) return fail(ACC_ERR_INVALID, "%s: %s array missing", s->entry.c_str(), what);
  if (out->rank != rank) return fail(ACC_ERR_INVALID, "%s: %s array has rank %d, expected %d", s->entry.c_str(), what, out->rank, rank);
  if (out->ncomp != ncomp)
    return fail(ncomp == 1 ? ACC_ERR_UNSUPPORTED : ACC_ERR_INVALID, "%s: %s array has %d components, the kernel was built for %d",
                s->entry.c_str(), what, out->ncomp, ncomp);
  for (int d = 0; d < rank; ++d)
    if (out->shape[d] < 0) return fail(ACC_ERR_INVALID, "%s: %s array has a negative extent", s->entry.c_str(), what);
  for (int c = 0; c < ncomp; ++c)
    if (!out->ptr[c] && array_size(*out) > 0) return fail(ACC_ERR_INVALID, "%s: %s array is NULL", s->entry.c_str(), what);
  return ACC_OK;
}

// an array of the skeleton's element type: one component, or the tuple's
int check_out(const acc_skel_s *s, const acc_array *out, int rank, const char *what) { return check_out(s, out, rank, what, s->ncomp()); }

// the component pointers of a result array, highest component first; NULL array = that many null pointers
void push_ptrs(const acc_array *a, int ncomp, Args *args, bool *aligned)
{
  for (int c = ncomp - 1; c >= 0; --c) {
    const uint64_t p = a ? a->ptr[c] : 0;
    if (a && !aligned16(p)) *aligned = false;
    args->ptr(p);
  }
}

void push_out(const acc_array &out, Args *args, bool *aligned)
{
  for (int d = 0; d < out.rank; ++d) args->i64(out.shape[d]);
  push_ptrs(&out, out.ncomp, args, aligned);
}

int launch(acc_skel_s *s, int variant, int64_t grid, size_t dyn_lds, hipStream_t stream, Args *args)
{
  if (grid < 1 || grid > 0x7fffffffLL) return fail(ACC_ERR_INVALID, "%s: grid of %lld blocks", s->entry.c_str(), (long long)grid);
  ACC_TRY(s->ensure_variant(variant));
  ACC_TRY(s->ctx->make_current());
  ACC_HIP_TRY(launch_kernel(s->variants[variant].fn, static_cast<unsigned>(grid), 1, 1,
                                    static_cast<unsigned>(s->variants[variant].block), 1, 1, static_cast<unsigned>(dyn_lds), stream,
                                    args->data(), nullptr));
  return ACC_OK;
}

// For the length of one driver call: what Args::data() and launch_kernel read (see Running).  A stream under a guard
// only takes instances whose kernels look at it.
struct RunScope {
  Running saved;
  int rc = ACC_OK;
  RunScope(acc_skel_s *s, hipStream_t st) : saved(t_run)
  {
    t_run.entry = s->entry.c_str();
    t_run.dump_exec = s->ctx->dump_exec;
    t_run.guarded = s->spec.guarded;
    t_run.guard = 0;
    const uint64_t g = s->ctx->guard_of(st);
    if (g && !s->spec.guarded)
      rc = fail(ACC_ERR_INVALID, "%s: the stream is under a guard (acc_stream_set_guard) and this instance was created without ACC_FLAG_GUARDED",
                s->entry.c_str());
    else
      t_run.guard = g;
  }
  ~RunScope() { t_run = saved; }
  RunScope(const RunScope &) = delete;
  RunScope &operator=(const RunScope &) = delete;
};
#define ACC_RUN_SCOPE(s, st)                          \
  RunScope run_scope__((s), (st));                    \
  if (run_scope__.rc != ACC_OK) return run_scope__.rc

bool kind_is(const acc_skel_s *s, std::initializer_list<int> kinds)
{
  return std::find(kinds.begin(), kinds.end(), s->spec.kind) != kinds.end();
}

size_t round256(size_t n) { return (n + 255) & ~size_t(255); }

// resident-grid cap: compute units x workgroups per unit (Launch.hs:51-55)
int64_t resident(const acc_skel_s *s, int variant) { return (int64_t)s->ctx->props.multiProcessorCount * s->variants[variant].blocks_per_cu; }

}  // namespace

extern "C" {

int acc_trace_start(acc_context ctx)
{
  if (!ctx) return fail(ACC_ERR_INVALID, "acc_trace_start: NULL context");
  if (t_trace.on) return fail(ACC_ERR_INVALID, "acc_trace_start: this thread is tracing already");
  t_trace.on = true;
  return ACC_OK;
}

int acc_trace_stop(acc_context ctx, int32_t *launches, double *gpu_ms)
{
  if (!ctx) return fail(ACC_ERR_INVALID, "acc_trace_stop: NULL context");
  if (!t_trace.on) return fail(ACC_ERR_INVALID, "acc_trace_stop: this thread is not tracing");
  t_trace.on = false;
  int rc = ctx->make_current();
  double total = 0.0;
  int32_t count = 0;
  for (auto &span : t_trace.spans) {
    float ms = 0.0f;
    if (rc == ACC_OK) {
      hipError_t e = hipEventSynchronize(span.second);
      if (e == hipSuccess) e = hipEventElapsedTime(&ms, span.first, span.second);
      if (e != hipSuccess) rc = acc::fail_hip(e, "acc_trace_stop");
    }
    total += ms;
    ++count;
    (void)hipEventDestroy(span.first);
    (void)hipEventDestroy(span.second);
  }
  t_trace.spans.clear();
  if (launches) *launches = count;
  if (gpu_ms) *gpu_ms = total;
  return rc;
}

int acc_exec_map(acc_skel s, const acc_array *env, const acc_array *out, acc_stream stream)
{
  if (!s) return fail(ACC_ERR_INVALID, "acc_exec_map: NULL skeleton");
  ACC_RUN_SCOPE(s, static_cast<hipStream_t>(stream));
  if (!kind_is(s, {ACC_SKEL_MAP, ACC_SKEL_GENERATE, ACC_SKEL_TRANSFORM})) return fail(ACC_ERR_INVALID, "acc_exec_map: skeleton is '%s'", s->entry.c_str());
  ACC_TRY(check_out(s, out, s->spec.out_rank, "result"));
  Args args;
  bool aligned = true;
  ACC_TRY(push_env(s, env, &args, &aligned));
  push_out(*out, &args, &aligned);
  const int64_t n = array_size(*out);
  if (n == 0) return ACC_OK;
  int v = aligned ? 0 : 1;
  // A result of a few columns or rows leaves most of every tile outside it (a transpose of 2^23 x 2 either way:
  // 170 us in tiles, 23-34 in runs): such a call takes variants 2 and 3, the same map in runs.  (A result of 2^20 rows
  // of 8 / 16 / 24 / 32 columns: 45 / 56 / 100 / 44 us in tiles, 10 / 20 / 40 / 41 in runs, and 29 against 52 for 33
  // columns.  Of 6 / 8 / 12 / 16 rows of 2^20 columns: 41 / 41 / 43 / 43 in tiles, 17 / 31 / 82 / 151 in runs.)
  const bool in_tiles = s->spec.map_tiled && out->shape[s->spec.out_rank - 1] >= s->knobs.map_tiled_min_w &&
                        out->shape[s->spec.out_rank - 1 - s->spec.map_tile_dim] >= s->knobs.map_tiled_min_h;
  if (s->spec.map_tiled && !in_tiles) v += 2;
  ACC_TRY(s->ensure_variant(v));
  if (in_tiles) {
    // a wave per tile of 32 x 32 elements of the innermost dimension and the second innermost one, or the one that
    // ACC_FLAG_TILE_DIM names (skel_map.h)
    const int rank = s->spec.out_rank;
    const int64_t side = 8 * (int64_t)s->spec.map_tile_block;
    const int64_t w = out->shape[rank - 1], h = out->shape[rank - 1 - s->spec.map_tile_dim];
    const int64_t tiles = ((w + side - 1) / side) * ((h + side - 1) / side) * (n / (w * h));
    const int64_t waves = s->variants[v].block / 64;
    return launch(s, v, std::min<int64_t>((tiles + waves - 1) / waves, (int64_t)1 << 22), 0, static_cast<hipStream_t>(stream), &args);
  }
  // streaming with no reuse: one short-lived workgroup per tile keeps the most loads in flight
  const int64_t grid = acc_launch_grid(n, s->elements_per_block(), resident(s, v), s->knobs.map_oversub);
  return launch(s, v, grid, 0, static_cast<hipStream_t>(stream), &args);
}

namespace {

// The segmented fold over `nseg` segments holding `n` elements in all; `args` holds the kernel parameters up to and
// including the segment description (offsets, or rows and row length).
//   short segments: a lane per segment over chunks staged in LDS (skel_foldseg.h);
//   long ones (on average: the lengths themselves are on the device) would serialise on that lane, so a wave, or
//   from `foldseg.block_team_len` a workgroup, takes one segment at a time;
//   fewer long segments than the device has room for teams: every segment is cut into `split` pieces, a team
//   each, and a second launch joins the pieces in order.
// Very long segments among the others (skel_foldseg.h, ACC_GIANTS).  Variants 4 to 7 of a segmented fold hand such a
// segment over to a second launch, at a cost to sources that have none; so an instance takes them once a look at its
// segment lengths has found such a segment -- a small kernel behind calls number 1, 2, 4, 8 ... of the instance, which
// says so in a word of host memory -- and once they are compiled, which happens in the background meanwhile.
// `foldseg.giants`: 2 this, 1 always, 0 never.
struct GiantsPlan {
  bool hand_over = false;      // this call takes variant `lv + 4`
  bool look = false;           // this call is followed by the look at the segment lengths
};

int plan_giants(acc_skel_s *s, int lv, GiantsPlan *plan)
{
  plan->hand_over = s->knobs.foldseg_giants == 1;
  if (s->knobs.foldseg_giants != 2 || s->hint_slot < 0) return ACC_OK;
  // (the word is the device's to write, at any time: read as such)
  if (!s->met_giants.load(std::memory_order_relaxed) &&
      __atomic_load_n(const_cast<uint32_t *>(s->ctx->status_host) + acc::STATUS_WORDS + s->hint_slot, __ATOMIC_RELAXED) != 0)
    s->met_giants.store(true, std::memory_order_relaxed);
  if (s->met_giants.load(std::memory_order_relaxed)) {
    ACC_TRY(s->start_variant(lv + 4));
    plan->hand_over = s->variant_compiled(lv + 4);
  } else {
    const unsigned call = s->seg_calls.fetch_add(1, std::memory_order_relaxed) + 1;
    plan->look = (call & (call - 1)) == 0;
  }
  return ACC_OK;
}

// the look: the parameters of the fold's own kernel (`common`, a guard's address behind them) and the word's address
int launch_probe(acc_skel_s *s, int lv, Args *common, int64_t nseg, hipStream_t st)
{
  (void)common->data();
  common->ptr(s->ctx->status_dev + (uint64_t)(acc::STATUS_WORDS + s->hint_slot) * sizeof(uint32_t));
  const int64_t lookers = std::min<int64_t>((nseg + s->spec.block - 1) / s->spec.block, (int64_t)s->ctx->props.multiProcessorCount * 8);
  hipError_t e = launch_kernel(s->variants[lv].fn_sweep, static_cast<unsigned>(lookers), 1, 1, static_cast<unsigned>(s->spec.block), 1, 1, 0, st,
                               common->data_without_guard(), nullptr);
  return e == hipSuccess ? ACC_OK : acc::fail_hip(e, "hipModuleLaunchKernel(segmented fold, probe)");
}

// the table of jobs: head, 32 jobs of 8 words and 16 ticket counters 32 words apart, then values of tagged words -- two
// for every piece of 4 chunks the source has, and one a job
int acquire_jobs(acc_skel_s *s, int lv, int64_t n, hipStream_t st, acc::ScratchRef *jobs)
{
  const int64_t piece = (int64_t)std::max(1, s->knobs.foldseg_giant_chunks) * (int64_t)((lv & 2) ? s->spec.chunk_long : s->spec.chunk);
  const size_t words_a_value = ((size_t)s->spec.elt_size + 3) / 4;
  const size_t bytes = (8 + 32 * (8 + 16 * 32) + (2 * (size_t)(n / piece + 2) + 32) * words_a_value) * 8;
  return s->ctx->scratch_acquire(bytes, st, acc::SCRATCH_FLAGS, jobs);
}

// the second launch, which takes what the first has entered in the table: `common` with the table behind it
int launch_sweep(acc_skel_s *s, int lv, Args *common, const acc::ScratchRef &jobs, hipStream_t st)
{
  common->ptr(reinterpret_cast<uint64_t>(jobs.ptr));
  common->u32(jobs.epoch);
  common->ptr(s->ctx->status_dev);
  const int64_t sweepers = (int64_t)s->ctx->props.multiProcessorCount * std::max(1, std::min(s->knobs.foldseg_sweep_per_cu, 2048 / s->spec.block));
  hipError_t e = launch_kernel(s->variants[lv].fn_sweep, static_cast<unsigned>(sweepers), 1, 1, static_cast<unsigned>(s->spec.block), 1, 1, 0, st,
                               common->data(), nullptr);
  return e == hipSuccess ? ACC_OK : acc::fail_hip(e, "hipModuleLaunchKernel(segmented fold, sweep)");
}

// `args`: the parameters every kernel of the template begins with (free arrays, result, segments).  `giants`: the
// segments are a vector's (the kernels of rows and of arrays of rank > 1 know no table).
int launch_segmented(acc_skel_s *s, int v, Args *args, const acc_array *env, const acc_array *out, int64_t nseg, int64_t n,
                     hipStream_t st, bool giants = false)
{
  const int64_t avg = n / nseg;
  if (avg < s->knobs.foldseg_wave_team_len) {
    // Segments of 8 elements or more on average stage half as much again at a time (variants 2 and 3 of the
    // instance, built when first wanted): 2^25 elements in segments of 8 / 32 / 100 on average 36 / 31 / 51 us
    // -> 32 / 27 / 40; shorter segments lose by it (rows of 4: 46 -> 49 us), and so keep the shorter chunk.
    int lv = v;
    if (avg >= s->knobs.foldseg_long_from && s->spec.chunk_long > s->spec.chunk) {
      lv = v + 2;
      ACC_TRY(s->ensure_variant(lv));
    }
    GiantsPlan plan;
    if (giants) ACC_TRY(plan_giants(s, lv, &plan));
    if (!plan.hand_over) {
      const int64_t grid = acc_launch_grid(nseg, s->spec.block, resident(s, lv), s->knobs.foldseg_oversub);
      int rc = launch(s, lv, grid, 0, st, args);
      if (rc == ACC_OK && plan.look) rc = launch_probe(s, lv, args, nseg, st);
      return rc;
    }
    lv += 4;
    ACC_TRY(s->ensure_variant(lv));
    const int64_t grid = acc_launch_grid(nseg, s->spec.block, resident(s, lv), s->knobs.foldseg_oversub);
    acc::ScratchRef jobs;
    ACC_TRY(acquire_jobs(s, lv, n, st, &jobs));
    Args first = *args;
    first.ptr(reinterpret_cast<uint64_t>(jobs.ptr));
    first.u32(jobs.epoch);
    first.ptr(s->ctx->status_dev);
    int rc = launch(s, lv, grid, 0, st, &first);
    if (rc == ACC_OK) rc = launch_sweep(s, lv, args, jobs, st);
    s->ctx->scratch_release(jobs, st);
    return rc;
  }
  // teams: a workgroup (1) from `foldseg.block_team_len`, a row of 16 lanes (2) below `foldseg.row_team_below`, else a wave (0)
  const int block_team = avg >= s->knobs.foldseg_block_team_len ? 1 : (avg < s->knobs.foldseg_row_team_below ? 2 : 0);
  const int64_t cus = s->ctx->props.multiProcessorCount;
  const int64_t team_lanes = block_team == 1 ? s->spec.block : (block_team == 2 ? 16 : 64);
  const int64_t room = cus * (2048 / team_lanes);                    // teams the device holds at once
  const int64_t min_piece = team_lanes * 64;                          // a piece keeps its team busy for a while
  int64_t split = 1;
  if (nseg * 2 <= room) split = std::max<int64_t>(1, std::min<int64_t>({room / nseg, avg / min_piece, s->knobs.foldseg_max_split}));
  // (segments that are all cut into pieces are not looked at, and none is handed over)
  GiantsPlan plan;
  if (giants && split == 1) ACC_TRY(plan_giants(s, v, &plan));
  const int tv = plan.hand_over ? v + 4 : v;
  if (plan.hand_over) ACC_TRY(s->ensure_variant(tv));
  acc::ScratchRef blk, jobs;
  uint64_t part = 0, part_ok = 0;
  if (split > 1) {
    const size_t pieces = (size_t)(nseg * split);
    const size_t ok_off = round256(pieces * s->spec.elt_size);
    ACC_TRY(s->ctx->scratch_acquire(ok_off + pieces * 4, st, acc::SCRATCH_FOLD, &blk));
    part = reinterpret_cast<uint64_t>(blk.ptr);
    part_ok = part + ok_off;
  }
  if (plan.hand_over) {
    const int rj = acquire_jobs(s, tv, n, st, &jobs);
    if (rj != ACC_OK) { s->ctx->scratch_release(blk, st); return rj; }
  }
  Args team = *args;
  team.i32(block_team);
  team.i64(split);
  team.ptr(part);
  team.ptr(part_ok);
  if (plan.hand_over) {
    team.ptr(reinterpret_cast<uint64_t>(jobs.ptr));
    team.u32(jobs.epoch);
    team.ptr(s->ctx->status_dev);
  }
  const int64_t per_block = block_team == 1 ? 1 : s->spec.block / team_lanes;
  const int64_t tgrid = acc_launch_grid(nseg * split, per_block, cus, 2048 / s->spec.block);
  int rc = s->ctx->make_current();
  if (rc == ACC_OK) {
    hipError_t e = launch_kernel(s->variants[tv].fn_finish, static_cast<unsigned>(tgrid), 1, 1,
                                         static_cast<unsigned>(s->spec.block), 1, 1, 0, st, team.data(), nullptr);
    if (e != hipSuccess) rc = acc::fail_hip(e, "hipModuleLaunchKernel(segmented fold, team)");
  }
  if (rc == ACC_OK && split > 1) {
    Args join;
    bool al = true;
    rc = push_env(s, env, &join, &al);
    join.i64(nseg);
    push_ptrs(out, out->ncomp, &join, &al);
    join.i64(split);
    join.ptr(part);
    join.ptr(part_ok);
    if (rc == ACC_OK) {
      const int64_t waves = s->spec.block / 64;
      const int64_t jgrid = (nseg + waves - 1) / waves;          // a wave per segment
      hipError_t e = launch_kernel(s->variants[v].fn_fill, static_cast<unsigned>(jgrid), 1, 1,
                                           static_cast<unsigned>(s->spec.block), 1, 1, 0, st, join.data(), nullptr);
      if (e != hipSuccess) rc = acc::fail_hip(e, "hipModuleLaunchKernel(segmented fold, join)");
    }
  }
  if (rc == ACC_OK && plan.hand_over) rc = launch_sweep(s, tv, args, jobs, st);
  if (rc == ACC_OK && plan.look) rc = launch_probe(s, v, args, nseg, st);
  s->ctx->scratch_release(blk, st);
  if (plan.hand_over) s->ctx->scratch_release(jobs, st);
  return rc;
}

// A fold along the innermost dimension whose element function reads neighbouring addresses where the ROW moves by one
// (ACC_FLAG_TILED: the fold of a transposed matrix, a matrix product written as a fold): a lane per row, neighbouring
// rows in neighbouring lanes (<entry>_across) -- a team of lanes along such a row asks for 64 cache lines with every
// load (sums down the columns of 4096 x 4096 Int32: 0.9 ms).  With fewer rows than the device has lanes the rows are
// cut into pieces of at least `fold.across_min_piece` elements, joined in order by <entry>_join.
int launch_across(acc_skel_s *s, int v, Args *args, const acc_array *env, const acc_array *out, int64_t rows, int64_t inner, hipStream_t st)
{
  const int64_t cus = s->ctx->props.multiProcessorCount;
  const int64_t lanes = cus * 2048;
  int64_t split = 1;
  if (rows < lanes)
    split = std::max<int64_t>(1, std::min<int64_t>({lanes / rows, inner / std::max(1, s->knobs.fold_across_min_piece), s->knobs.foldseg_max_split}));
  acc::ScratchRef blk;
  uint64_t part = 0, part_ok = 0;
  if (split > 1) {
    const size_t pieces = (size_t)(rows * split);
    const size_t ok_off = round256(pieces * s->spec.elt_size);
    ACC_TRY(s->ctx->scratch_acquire(ok_off + pieces * 4, st, acc::SCRATCH_FOLD, &blk));
    part = reinterpret_cast<uint64_t>(blk.ptr);
    part_ok = part + ok_off;
  }
  Args first = *args;
  first.i64(split);
  first.ptr(part);
  first.ptr(part_ok);
  const int64_t grid = acc_launch_grid(rows * split, s->spec.block, cus, 4 * (2048 / s->spec.block));
  int rc = s->ctx->make_current();
  if (rc == ACC_OK) {
    hipError_t e = launch_kernel(s->variants[v].fn_across, static_cast<unsigned>(grid), 1, 1, static_cast<unsigned>(s->spec.block), 1, 1, 0, st,
                                 first.data(), nullptr);
    if (e != hipSuccess) rc = acc::fail_hip(e, "hipModuleLaunchKernel(fold, a lane a row)");
  }
  if (rc == ACC_OK && split > 1) {
    Args join;
    bool al = true;
    rc = push_env(s, env, &join, &al);
    join.i64(rows);
    push_ptrs(out, out->ncomp, &join, &al);
    join.i64(split);
    join.ptr(part);
    join.ptr(part_ok);
    if (rc == ACC_OK) {
      const int64_t waves = s->spec.block / 64;
      hipError_t e = launch_kernel(s->variants[v].fn_fill, static_cast<unsigned>((rows + waves - 1) / waves), 1, 1,
                                   static_cast<unsigned>(s->spec.block), 1, 1, 0, st, join.data(), nullptr);
      if (e != hipSuccess) rc = acc::fail_hip(e, "hipModuleLaunchKernel(fold, join)");
    }
  }
  s->ctx->scratch_release(blk, st);
  return rc;
}

}  // namespace

int acc_exec_fold(acc_skel s, const acc_array *env, int32_t in_rank, const int64_t *in_shape, const acc_array *out, acc_stream stream)
{
  if (!s) return fail(ACC_ERR_INVALID, "acc_exec_fold: NULL skeleton");
  ACC_RUN_SCOPE(s, static_cast<hipStream_t>(stream));
  if (!kind_is(s, {ACC_SKEL_FOLD, ACC_SKEL_FOLD1})) return fail(ACC_ERR_INVALID, "acc_exec_fold: skeleton is '%s'", s->entry.c_str());
  if (in_rank != s->spec.out_rank + 1 || !in_shape) return fail(ACC_ERR_INVALID, "%s: input rank %d, kernel was built for %d", s->entry.c_str(), in_rank, s->spec.out_rank + 1);
  ACC_TRY(check_out(s, out, s->spec.out_rank, "result"));
  for (int d = 0; d < in_rank; ++d)
    if (in_shape[d] < 0) return fail(ACC_ERR_INVALID, "%s: negative input extent", s->entry.c_str());
  int64_t inner = in_shape[in_rank - 1];
  // fold1 of an empty innermost dimension: Execute.hs:282-285
  if (inner == 0 && !s->spec.has_seed) return fail(ACC_ERR_INVALID, "%s: empty array", s->entry.c_str());
  // empty outer extents count as 1 in the result of a seeded fold: Execute.hs:287-289.  (The reference then runs its
  // kernel over rows that do not exist; here such a result is the seed in every position, as for rows without
  // elements, and a fold1 over no rows has nothing to do.)
  int64_t rows = 1;
  bool no_rows = false;
  for (int d = 0; d + 1 < in_rank; ++d) {
    rows *= std::max<int64_t>(1, in_shape[d]);
    no_rows = no_rows || in_shape[d] == 0;
  }
  if (no_rows) {
    if (!s->spec.has_seed) return ACC_OK;
    inner = 0;
  }
  if (array_size(*out) < rows && !(in_rank == 1)) return fail(ACC_ERR_INVALID, "%s: result holds %lld elements, %lld needed", s->entry.c_str(), (long long)array_size(*out), (long long)rows);

  hipStream_t st = static_cast<hipStream_t>(stream);
  Args args;
  bool aligned = true;
  ACC_TRY(push_env(s, env, &args, &aligned));
  const int v = aligned ? 0 : 1;
  ACC_TRY(s->ensure_variant(v));

  if (s->spec.out_rank > 0) {      // along the innermost dimension: a segmented fold over rows of one length
    args.i64(rows);
    push_ptrs(out, out->ncomp, &args, &aligned);
    args.i64(rows);
    args.i64(inner);
    if (inner == 0) {
      // rows without elements: every result is the seed; the one-lane-per-row entry does that
      const int64_t grid = acc_launch_grid(rows, s->spec.block, resident(s, v), 1 << 20);
      return launch(s, v, grid, 0, st, &args);
    }
    if (inner <= std::min(16, s->knobs.fold_rows_max)) {
      // short rows: a lane reads its row straight from memory (skel_foldseg.h, _rows)
      const int64_t r = inner == 1 ? 4 : (inner == 2 ? 2 : 1), u = r * inner >= 16 ? 1 : 16 / (r * inner);   // as the kernel's R and U
      const int64_t grid = acc_launch_grid(rows, s->spec.block * r * u, resident(s, v), s->knobs.foldseg_oversub);
      hipError_t e = launch_kernel(s->variants[v].fn_rows, static_cast<unsigned>(grid), 1, 1, static_cast<unsigned>(s->spec.block), 1, 1,
                                           0, st, args.data(), nullptr);
      return e == hipSuccess ? ACC_OK : acc::fail_hip(e, "hipModuleLaunchKernel(fold, short rows)");
    }
    if (s->knobs.fold_across == 1 || (s->knobs.fold_across == 2 && s->spec.fold_across))
      return launch_across(s, v, &args, env, out, rows, inner, st);
    return launch_segmented(s, v, &args, env, out, rows, rows * inner, st);
  }

  const int64_t n = inner;
  const int64_t tile = s->elements_per_block();
  int64_t grid = acc_launch_grid(n, tile, s->ctx->props.multiProcessorCount,
                                 std::min(s->variants[v].blocks_per_cu, s->knobs.fold_blocks_per_cu));
  const bool single = s->spec.fold_single;       // as generated into the kernel
  if (grid == 1) {                 // a lone block finishes the job itself
    push_ptrs(out, out->ncomp, &args, &aligned);
    args.i64(n);
    args.ptr(0);
    if (single) { args.u32(0); args.ptr(s->ctx->status_dev); }
    return launch(s, v, 1, 0, st, &args);
  }
  if (single) {
    // one launch: every block leaves its partial result in 64-bit words that carry the launch's epoch in their
    // upper half, and the last block collects them (skel_fold.h).  Every word of the scratch block is only ever
    // written in that form, so words of earlier launches, whatever their grid or element type, read as "not yet".
    const size_t words = (s->spec.elt_size + 3) / 4;
    acc::ScratchRef blk;
    ACC_TRY(s->ctx->scratch_acquire((size_t)grid * words * 8, st, acc::SCRATCH_FLAGS, &blk));
    push_ptrs(out, out->ncomp, &args, &aligned);
    args.i64(n);
    args.ptr(reinterpret_cast<uint64_t>(blk.ptr));
    args.u32(blk.epoch);
    args.ptr(s->ctx->status_dev);
    int rc = launch(s, v, grid, 0, st, &args);
    s->ctx->scratch_release(blk, st);
    return rc;
  }
  // one partial per block, then a single-block launch folds them: foldRec, Execute.hs:304-315,
  // always exactly one level deep because the first grid never exceeds what is resident
  acc::ScratchRef blk;
  ACC_TRY(s->ctx->scratch_acquire((size_t)grid * s->spec.elt_size, st, acc::SCRATCH_FOLD, &blk));
  const uint64_t partials = reinterpret_cast<uint64_t>(blk.ptr);
  push_ptrs(out, out->ncomp, &args, &aligned);
  args.i64(n);
  args.ptr(partials);
  int rc = launch(s, v, grid, 0, st, &args);
  if (rc == ACC_OK) {
    Args fin;
    bool al = true;
    rc = push_env(s, env, &fin, &al);
    push_ptrs(out, out->ncomp, &fin, &al);
    fin.ptr(partials);
    fin.i64(grid);
    if (rc == ACC_OK) {
      hipError_t e = launch_kernel(s->variants[v].fn_finish, 1, 1, 1, static_cast<unsigned>(s->spec.block), 1, 1, 0, st, fin.data(), nullptr);
      if (e != hipSuccess) rc = acc::fail_hip(e, "hipModuleLaunchKernel(fold finish)");
    }
  }
  s->ctx->scratch_release(blk, st);
  return rc;
}

int acc_exec_foldseg_nd(acc_skel s, const acc_array *env, int32_t in_rank, const int64_t *in_shape, const acc_array *offsets,
                        const acc_array *out, acc_stream stream)
{
  if (!s) return fail(ACC_ERR_INVALID, "acc_exec_foldseg: NULL skeleton");
  ACC_RUN_SCOPE(s, static_cast<hipStream_t>(stream));
  if (!kind_is(s, {ACC_SKEL_FOLDSEG, ACC_SKEL_FOLD1SEG})) return fail(ACC_ERR_INVALID, "acc_exec_foldseg: skeleton is '%s'", s->entry.c_str());
  const int rank = std::max(1, s->spec.out_rank);        // of the input and of the result alike
  if (in_rank != rank || !in_shape) return fail(ACC_ERR_INVALID, "%s: input rank %d, kernel was built for %d", s->entry.c_str(), in_rank, rank);
  ACC_TRY(check_out(s, offsets, 1, "segment offsets", 1));
  ACC_TRY(check_out(s, out, rank, "result"));
  int64_t rows = 1;
  for (int d = 0; d < rank; ++d) {
    if (in_shape[d] < 0) return fail(ACC_ERR_INVALID, "%s: negative input extent", s->entry.c_str());
    if (d + 1 < rank) rows *= in_shape[d];
  }
  const int64_t inner = in_shape[rank - 1];
  // the offsets vector is one longer than the number of segments of a row: Execute.hs:320-324;
  // the result is  sh :. number of segments  for an input  sh :. inner
  const int64_t per_row = offsets->shape[0] - 1;
  if (per_row <= 0 || rows == 0) return ACC_OK;
  for (int d = 0; d + 1 < rank; ++d)
    if (out->shape[d] != in_shape[d]) return fail(ACC_ERR_INVALID, "%s: the result's outer extents differ from the input's", s->entry.c_str());
  if (out->shape[rank - 1] < per_row)
    return fail(ACC_ERR_INVALID, "%s: result holds %lld segments a row, %lld needed", s->entry.c_str(), (long long)out->shape[rank - 1], (long long)per_row);
  if (rank > 1 && out->shape[rank - 1] != per_row)
    return fail(ACC_ERR_INVALID, "%s: the result's rows must be exactly the %lld segments long", s->entry.c_str(), (long long)per_row);
  const int64_t nseg = rows * per_row, n = rows * inner;
  Args args;
  bool aligned = true;
  ACC_TRY(push_env(s, env, &args, &aligned));
  args.i64(nseg);
  push_ptrs(out, out->ncomp, &args, &aligned);
  args.i64(n);
  args.ptr(offsets->ptr[0]);
  if (rank > 1) {        // segments restart in every outer row: CodeGen/Reduction.hs:473-474
    args.i64(inner);
    args.i64(per_row);
  }
  const int v = aligned ? 0 : 1;
  ACC_TRY(s->ensure_variant(v));
  return launch_segmented(s, v, &args, env, out, nseg, n, static_cast<hipStream_t>(stream), rank == 1);
}

int acc_exec_foldseg(acc_skel s, const acc_array *env, int64_t n, const acc_array *offsets, const acc_array *out, acc_stream stream)
{
  if (s && std::max(1, s->spec.out_rank) != 1)
    return fail(ACC_ERR_INVALID, "acc_exec_foldseg: the kernel was built for rank %d: use acc_exec_foldseg_nd", s->spec.out_rank);
  return acc_exec_foldseg_nd(s, env, 1, &n, offsets, out, stream);
}

namespace {

// scanOp / scan1Op / scan'Op / scanCore, Execute.hs:328-392, as ONE launch.  `noalloc`: the tile descriptors live in
// the library's file-scope device array instead of a block of the context's pool, and nothing may be allocated,
// compiled or loaded on the way.
int scan_core(acc_skel s, const acc_array *env, int64_t n, const acc_array *out, const acc_array *total, acc_stream stream,
              const bool noalloc, const char *who)
{
  if (!s) return fail(ACC_ERR_INVALID, "%s: NULL skeleton", who);
  ACC_RUN_SCOPE(s, static_cast<hipStream_t>(stream));
  if (!kind_is(s, {ACC_SKEL_SCANL, ACC_SKEL_SCANL1, ACC_SKEL_SCANLP, ACC_SKEL_SCANR, ACC_SKEL_SCANR1, ACC_SKEL_SCANRP}))
    return fail(ACC_ERR_INVALID, "%s: skeleton is '%s'", who, s->entry.c_str());
  if (n < 0) return fail(ACC_ERR_INVALID, "%s: negative input extent", s->entry.c_str());
  ACC_TRY(check_out(s, out, 1, "result"));
  const int kind = s->spec.kind;
  const bool plus_one = (kind == ACC_SKEL_SCANL || kind == ACC_SKEL_SCANR);     // Execute.hs:328-339
  const bool primed = (kind == ACC_SKEL_SCANLP || kind == ACC_SKEL_SCANRP);     // Execute.hs:352-362
  if (out->shape[0] < n + (plus_one ? 1 : 0))
    return fail(ACC_ERR_INVALID, "%s: result holds %lld elements, %lld needed", s->entry.c_str(), (long long)out->shape[0], (long long)(n + (plus_one ? 1 : 0)));
  if (primed) ACC_TRY(check_out(s, total, 0, "total"));
  if (n == 0 && !plus_one && !primed) return ACC_OK;       // scanl1 / scanr1 of nothing is nothing

  hipStream_t st = static_cast<hipStream_t>(stream);
  Args args;
  bool aligned = true;
  ACC_TRY(push_env(s, env, &args, &aligned));
  push_out(*out, &args, &aligned);
  {
    bool ignore = true;      // a scalar's alignment decides nothing
    push_ptrs(primed ? total : nullptr, s->ncomp(), &args, &ignore);
  }
  args.i64(n);

  // An array of up to 12 MB takes the small-tile variant (4 rows a lane instead of 32): a workgroup runs through the
  // instructions of all the rows of its tile whether the array fills them or not, and a small array spread over few
  // large tiles leaves most of the device idle (Int32: 1024 elements 10.6 us -> 4.4, 2^18 8.6 -> 4.1, 2^21 10.0 ->
  // 8.1, 3 M + 3 14.8 -> 9.3; at 2^22 the two are level, 11.7 and 11.2, and so are 2^21 Float64, 12.0 and 13.2).
  const bool small = s->spec.scan_small_rows > 0 &&
                     n * (int64_t)s->spec.elt_size <= (int64_t)s->knobs.scan_small_below_kb * 1024;
  int v = (aligned ? 0 : 1) + (small ? 2 : 0);
  if (noalloc) {
    // building a variant compiles and loads a module: not here
    if (!s->variant_ready(v))
      return fail(ACC_ERR_INVALID, "%s: the %s %s-tile variant of this instance is not loaded yet; run acc_exec_scan once on operands of the same alignment and of %s %d KB first",
                  who, aligned ? "aligned" : "unaligned", small ? "small" : "large", small ? "at most" : "more than", s->knobs.scan_small_below_kb);
  } else {
    ACC_TRY(s->ensure_variant(v));
  }
  const int block = s->variants[v].block;
  const int64_t tile = (int64_t)block * s->variants[v].rows * s->vec();
  const int64_t tiles = (n + tile - 1) / tile;
  const int64_t grid = std::max<int64_t>(1, tiles);     // one workgroup per tile, in dispatch order
  const int64_t ndesc = std::max<int64_t>(1, tiles);
  const size_t esz = s->spec.elt_size;
  // one descriptor per tile: 64-bit words {flag, 4 bytes of the value}, `desc_stride` words apart
  // (more when the element needs more words)
  const size_t words = std::max<size_t>((esz + 3) / 4, (size_t)s->spec.scan_desc_stride);
  const size_t off_d0 = 256, off_d1 = 256, off_d2 = 256;
  const size_t bytes = 256 + round256((size_t)ndesc * 8 * words);
  if (noalloc) {
    if (tiles > ACC_NOALLOC_MAX_TILES)
      return fail(ACC_ERR_INVALID, "%s: %lld elements are %lld tiles of %lld, more than the %d the scratch array has descriptors for",
                  who, (long long)n, (long long)tiles, (long long)tile, ACC_NOALLOC_MAX_TILES);
    ACC_TRY(s->ctx->make_current());
    void *nbase = nullptr;
    uint32_t nepoch = 0;
    ACC_TRY(acc::noalloc_scan_state(s->ctx->device, bytes, st, &nbase, &nepoch));
    char *b = static_cast<char *>(nbase);
    args.ptr(reinterpret_cast<uint64_t>(b + off_d0));
    args.ptr(reinterpret_cast<uint64_t>(b + off_d1));
    args.ptr(reinterpret_cast<uint64_t>(b + off_d2));
    args.u32(nepoch);
    args.i64(tiles);
    args.ptr(s->ctx->status_dev);
    if (grid < 1 || grid > 0x7fffffffLL) return fail(ACC_ERR_INVALID, "%s: grid of %lld blocks", who, (long long)grid);
    ACC_HIP_TRY(launch_kernel(s->variants[v].fn, static_cast<unsigned>(grid), 1, 1, static_cast<unsigned>(block), 1, 1,
                                      0, st, args.data(), nullptr));
    return ACC_OK;
  }
  // A scan with more tiles than the device holds at once does not share the device with another such scan: tiles of
  // one could fill a compute die waiting for a tile that another die, full of waiting tiles of the other, has no
  // room for.  (Not under `noalloc`: calls through that entry that overlap on one device are excluded as it is.)
  const bool big = grid > resident(s, v);
  if (big) ACC_TRY(acc::scan_order_before(s->ctx->device, st));
  acc::ScratchRef blk;
  {
    const int arc = s->ctx->scratch_acquire(bytes, st, acc::SCRATCH_SCAN, &blk);
    if (arc != ACC_OK) {
      if (big) acc::scan_order_after(s->ctx->device);
      return arc;
    }
  }
  const uint32_t epoch = blk.epoch;
  char *base = static_cast<char *>(blk.ptr);
  if (s->spec.scan_ticket) (void)hipMemsetAsync(base + 64, 0, 4, st);      // (measurement knob scan.ticket: the counter tiles are drawn from)
  args.ptr(reinterpret_cast<uint64_t>(base + off_d0));
  args.ptr(reinterpret_cast<uint64_t>(base + off_d1));
  args.ptr(reinterpret_cast<uint64_t>(base + off_d2));
  args.u32(epoch);
  args.i64(tiles);
  args.ptr(s->ctx->status_dev);
  const int rc = launch(s, v, grid, 0, st, &args);
  if (big) acc::scan_order_after(s->ctx->device);
  s->ctx->scratch_release(blk, st);
  return rc;
}

}  // namespace

int acc_exec_scan(acc_skel s, const acc_array *env, int64_t n, const acc_array *out, const acc_array *total, acc_stream stream)
{
  return scan_core(s, env, n, out, total, stream, false, "acc_exec_scan");
}

int acc_exec_scan_noalloc(acc_skel s, const acc_array *env, int64_t n, const acc_array *out, const acc_array *total, acc_stream stream)
{
  return scan_core(s, env, n, out, total, stream, true, "acc_exec_scan_noalloc");
}

int acc_exec_permute(acc_skel s, const acc_array *env, int64_t n_src, const acc_array *defaults, const acc_array *out, acc_stream stream)
{
  if (!s) return fail(ACC_ERR_INVALID, "acc_exec_permute: NULL skeleton");
  ACC_RUN_SCOPE(s, static_cast<hipStream_t>(stream));
  if (!kind_is(s, {ACC_SKEL_PERMUTE})) return fail(ACC_ERR_INVALID, "acc_exec_permute: skeleton is '%s'", s->entry.c_str());
  if (n_src < 0) return fail(ACC_ERR_INVALID, "permute: negative source extent");
  ACC_TRY(check_out(s, out, s->spec.out_rank, "result"));
  ACC_TRY(check_out(s, defaults, s->spec.out_rank, "defaults"));
  for (int d = 0; d < out->rank; ++d)
    if (defaults->shape[d] != out->shape[d]) return fail(ACC_ERR_INVALID, "permute: defaults and result differ in shape");
  const int64_t ntarget = array_size(*out);
  hipStream_t st = static_cast<hipStream_t>(stream);
  const size_t esz = s->spec.elt_size;
  ACC_TRY(s->ctx->make_current());
  // the result starts as a copy of the defaults: Execute.hs:401-406
  const bool copy_defaults = ntarget > 0 && defaults->ptr[0] != out->ptr[0];
  auto plain_copy = [&]() -> int {
    if (!copy_defaults) return ACC_OK;
    const int nc = s->ncomp();
    for (int c = 0; c < nc; ++c) {
      const size_t csz = nc == 1 ? esz : (size_t)acc::type_size(s->spec.comp_types[nc - 1 - c]);
      if (t_run.guard)      // under a loop's guard the copy, too, must not happen once the loop has ended
        ACC_TRY(acc::guarded_copy(out->ptr[c], defaults->ptr[c], (size_t)ntarget * csz, t_run.guard, st));
      else
        ACC_HIP_TRY(hipMemcpyAsync(reinterpret_cast<void *>(out->ptr[c]), reinterpret_cast<void *>(defaults->ptr[c]), (size_t)ntarget * csz, hipMemcpyDeviceToDevice, st));
    }
    return ACC_OK;
  };
  if (n_src == 0 || ntarget == 0) return plain_copy();

  // A combination without an atomic instruction of its own on few targets: compare-and-swap loops on the result
  // meet on those few addresses (16 M Float32 `max` updates on 1000 targets: 16.6 ms), the tables in LDS of the
  // locked template do not (74 us).  Such a skeleton carries that template as its variants 2 and 3.
  const int64_t lds_all = std::min<int64_t>((int64_t)s->ctx->props.sharedMemPerBlock, s->knobs.permute_lds_bytes);
  // targets per table in LDS (value + state word each), and how many such windows the targets need
  const int64_t lds_cap = std::max<int64_t>(1, (lds_all - 16) / ((int64_t)esz + 4));
  const int64_t lds_windows = (ntarget + lds_cap - 1) / lds_cap;
  const bool lds_table_fits = lds_windows <= s->knobs.permute_lock_max_windows &&
                              n_src >= s->knobs.permute_lock_lds_min_ratio * ntarget;
  // (Floating-point addition has an LDS atomic, but it runs at a fifth of the integer one's rate -- 16 M updates on
  // 1000 targets: 95 us against 63 us through the tables -- so between 48 and 6144 targets it goes the same way.
  // Below, the tables' locks are what lanes meet on (16 targets 149 us against 93, one target 2.1 ms against 0.12);
  // above, a table holds half the targets an array of plain values does and the passes over the source multiply
  // (16 384 targets 123 us against 102, 131 072: 407 against 107).)
  const bool fp_add = s->spec.combine_hint == ACC_COMBINE_ADD && (s->spec.elt_type == "float" || s->spec.elt_type == "double") &&
                      ntarget >= s->knobs.permute_fp_tables_from && ntarget <= s->knobs.permute_fp_tables_to;
  const bool generic_few = !s->spec.permute_locked && (s->spec.combine_hint == ACC_COMBINE_GENERIC || fp_add) && lds_table_fits &&
                           s->knobs.permute_generic_lds != 0;
  if (s->spec.permute_locked && s->spec.permute_replace && n_src <= (int64_t)0xffffffffLL) {
    // `permute const` of an element that no single store covers: nothing is read or locked.  A scalar of one or two
    // bytes is stored; of a tuple the source whose index stays in the target's word of a table wins, whole
    // (skel_permute.h, permute_claim / permute_place).
    ACC_TRY(plain_copy());
    Args pargs;
    bool al = true;
    ACC_TRY(push_env(s, env, &pargs, &al));
    push_out(*out, &pargs, &al);
    pargs.i64(n_src);
    const int pv = al ? 0 : 1;
    ACC_TRY(s->ensure_variant(pv));
    acc::ScratchRef wblk;
    const bool tuple = s->ncomp() > 1 || esz > 8;      // (what no single store of at most 8 bytes writes)
    if (tuple) ACC_TRY(s->ctx->scratch_acquire((size_t)ntarget * 4, st, acc::SCRATCH_FOLD, &wblk));
    pargs.ptr(reinterpret_cast<uint64_t>(wblk.ptr));
    const int64_t pgrid = acc_launch_grid(n_src, 256 * 4, s->ctx->props.multiProcessorCount, 32);
    int prc = ACC_OK;
    if (tuple) {
      hipError_t ce = launch_kernel(s->variants[pv].fn_claim, static_cast<unsigned>(pgrid), 1, 1, 256, 1, 1, 0, st, pargs.data(), nullptr);
      if (ce != hipSuccess) prc = acc::fail_hip(ce, "hipModuleLaunchKernel(permute_claim)");
    }
    if (prc == ACC_OK) {
      hipError_t pe = launch_kernel(s->variants[pv].fn_place, static_cast<unsigned>(pgrid), 1, 1, 256, 1, 1, 0, st, pargs.data(), nullptr);
      if (pe != hipSuccess) prc = acc::fail_hip(pe, "hipModuleLaunchKernel(permute_place)");
    }
    s->ctx->scratch_release(wblk, st);
    return prc;
  }
  if (s->spec.permute_locked || generic_few) {
    // elements no atomic covers: a lock per target (the reference's lock array, Execute.hs:402-405)
    ACC_TRY(plain_copy());
    Args largs;
    bool al = true;
    ACC_TRY(push_env(s, env, &largs, &al));
    push_out(*out, &largs, &al);
    largs.i64(n_src);
    const int lv = (al ? 0 : 1) + (s->spec.permute_locked ? 0 : 2);
    ACC_TRY(s->ensure_variant(lv));
    acc::ScratchRef lblk;
    ACC_TRY(s->ctx->scratch_acquire((size_t)ntarget * 4 + 256, st, acc::SCRATCH_LOCKS, &lblk));
    // the locks start 256 bytes in
    largs.ptr(reinterpret_cast<uint64_t>(lblk.ptr) + 256);
    // Lanes in flight are kept to a few per target: every failed attempt on a lock is an atomic that queues in front
    // of the holder's own accesses, and with hundreds of lanes waiting per lock the device's whole atomic rate goes
    // into failed attempts (1000 targets: 12 M updates/s with every compute unit full, 20 times that with 32 lanes
    // per target).
    const int64_t lanes = std::max<int64_t>(64, ntarget * s->knobs.permute_lock_lanes_per_target);
    int64_t lgrid = std::min(acc_launch_grid(n_src, s->spec.block, s->ctx->props.multiProcessorCount, 8),
                             (lanes + s->spec.block - 1) / s->spec.block);
    // With few targets every workgroup combines in a table of its own in LDS (value + state word per target),
    // leaves it as a row of a table in memory, and a second launch folds the rows into the result: no global lock.
    const int64_t lds_budget = lds_all;
    int32_t lds_bins = 0, lds_copies = 1, win_blocks = 1;
    int64_t lds_need = 0;
    acc::ScratchRef dblk;
    uint64_t dump_val = 0, dump_ok = 0;
    if (lds_table_fits) {
      // windows of equal size; a single window that is small is kept once per wave, within a quarter of the LDS so
      // that several workgroups still fit
      lds_bins = static_cast<int32_t>((ntarget + lds_windows - 1) / lds_windows);
      auto lds_for = [&](int64_t copies) { return (((int64_t)lds_bins * copies * (int64_t)esz + 15) & ~int64_t(15)) + (int64_t)lds_bins * copies * 4; };
      const int64_t waves = s->spec.block / 64;
      while (lds_windows == 1 && lds_copies * 2 <= waves &&
             lds_for(lds_copies * 2) <= std::min<int64_t>(lds_budget, s->knobs.permute_lock_copies_bytes)) lds_copies *= 2;
      lds_need = lds_for(lds_copies);
      int bpc = 0;
      hipError_t oe = hipModuleOccupancyMaxActiveBlocksPerMultiprocessor(&bpc, s->variants[lv].fn, s->spec.block, (size_t)lds_need);
      if (oe != hipSuccess || bpc < 1) { (void)hipGetLastError(); bpc = 1; }
      // the device full of workgroups, shared out between the windows, as long as their rows stay within
      // `permute.lock_table_mbytes`
      const int64_t row_bytes = (int64_t)lds_bins * ((int64_t)esz + 4);
      const int64_t row_cap = std::max<int64_t>(lds_windows, ((int64_t)s->knobs.permute_lock_table_mbytes << 20) / row_bytes);
      const int64_t blocks = std::max<int64_t>(lds_windows, std::min<int64_t>(
          lds_windows * acc_launch_grid(n_src, s->spec.block, s->ctx->props.multiProcessorCount, bpc), std::min<int64_t>((int64_t)s->ctx->props.multiProcessorCount * bpc, row_cap)));
      win_blocks = static_cast<int32_t>(std::max<int64_t>(1, blocks / lds_windows));
      lgrid = lds_windows * win_blocks;
      const size_t ok_off = round256((size_t)(lgrid * lds_bins) * esz);
      const int arc = s->ctx->scratch_acquire(ok_off + (size_t)(lgrid * lds_bins) * 4, st, acc::SCRATCH_FOLD, &dblk);
      if (arc != ACC_OK) { s->ctx->scratch_release(lblk, st); return arc; }
      dump_val = reinterpret_cast<uint64_t>(dblk.ptr);
      dump_ok = dump_val + ok_off;
    }
    largs.i32(lds_bins);
    largs.i32(lds_copies);
    largs.ptr(dump_val);
    largs.ptr(dump_ok);
    largs.i32(win_blocks);
    largs.ptr(s->ctx->status_dev);
    int lrc = launch(s, lv, lgrid, lds_bins ? (size_t)lds_need : 0, st, &largs);
    if (lrc == ACC_OK && lds_bins) {
      Args j;
      bool jal = true;
      lrc = push_env(s, env, &j, &jal);
      push_out(*out, &j, &jal);
      j.ptr(dump_val);
      j.ptr(dump_ok);
      j.i32(win_blocks);
      j.i32(lds_bins);
      j.i64(ntarget);
      if (lrc == ACC_OK) {
        hipError_t je = launch_kernel(s->variants[lv].fn_finish, static_cast<unsigned>((ntarget + 3) / 4), 1, 1, 256, 1, 1, 0, st,
                                              j.data(), nullptr);
        if (je != hipSuccess) lrc = acc::fail_hip(je, "hipModuleLaunchKernel(permute_join)");
      }
    }
    s->ctx->scratch_release(dblk, st);
    s->ctx->scratch_release(lblk, st);
    return lrc;
  }

  Args args;
  bool aligned = true;
  ACC_TRY(push_env(s, env, &args, &aligned));
  push_out(*out, &args, &aligned);
  args.i64(n_src);

  // Integer addition on more targets than one LDS table of whole elements holds, but no more than one of 16-bit
  // counts does (65536 Int32 or Int64 targets in 128 KB): one pass over the source instead of one per window.  Also
  // from `permute.narrow_from` targets that whole elements would still hold: a single copy of such a table is what
  // all sixteen waves add to, and the smaller one does better (2^24 keys into 16 384 / 40 960 targets: 25.2 / 31.4
  // -> 22.8 / 27.0 us).
  const bool int_add = s->spec.combine_hint == ACC_COMBINE_ADD &&
                       (s->spec.elt_type == "Int32" || s->spec.elt_type == "Word32" || s->spec.elt_type == "Int64" || s->spec.elt_type == "Word64");
  // Only where the source is spelt as a small constant -- the counting idiom, `permute (+) zeros bin ones` -- since any
  // other addend would go to the result one device-scope atomic at a time (`permute.narrow=2` takes every source).
  const int narrow = s->knobs.permute_narrow;
  if (int_add && ntarget > std::min<int64_t>(s->knobs.permute_narrow_from, lds_all / (int64_t)esz) && ((ntarget + 1) / 2) * 4 <= lds_all && n_src >= 4 * ntarget &&
      (narrow == 2 || (narrow == 1 && s->spec.get_small_constant))) {
    const int nv = (aligned ? 0 : 1) + 6;
    ACC_TRY(s->ensure_variant(nv));
    // A source spelt as a small constant never adds to the result directly: its corrections go to a table of carries
    // (all zero between launches: the merge clears what it reads) and the merge writes  defaults + carries + rows,
    // so nothing has to be in the result beforehand and the copy of the defaults is not a launch of its own.  Any
    // other source (`permute.narrow=2`) may hold addends the table does not take; those go to the result, which must
    // then hold the defaults before the main kernel starts.
    const bool direct_adds = !s->spec.get_small_constant;
    if (direct_adds && copy_defaults) {
      Args f;
      f.ptr(0);
      f.i64(0);
      f.ptr(out->ptr[0]);
      f.ptr(defaults->ptr[0]);
      f.i64(ntarget);
      const int64_t fill_grid = std::min<int64_t>((ntarget + 255) / 256, 8 * (int64_t)s->ctx->props.multiProcessorCount);
      hipError_t fe = launch_kernel(s->variants[nv].fn_fill, static_cast<unsigned>(fill_grid), 1, 1, 256, 1, 1, 0, st, f.data(), nullptr);
      if (fe != hipSuccess) return acc::fail_hip(fe, "hipModuleLaunchKernel(permute_fill, narrow counts)");
    }
    const int64_t nwords = (ntarget + 1) / 2;
    const size_t nlds = (size_t)nwords * 4;
    int bpc = 0;
    hipError_t oe = hipModuleOccupancyMaxActiveBlocksPerMultiprocessor(&bpc, s->variants[nv].fn, s->spec.block, nlds);
    if (oe != hipSuccess || bpc < 1) { (void)hipGetLastError(); bpc = 1; }
    const int64_t cus_n = s->ctx->props.multiProcessorCount;
    const int64_t ngrid = acc_launch_grid(n_src, s->elements_per_block(), cus_n, bpc);
    acc::ScratchRef nblk, cblk;
    ACC_TRY(s->ctx->scratch_acquire((size_t)ntarget * esz, st, acc::SCRATCH_CARRY, &cblk));
    const int64_t nd = (nwords + 1) / 2;             // words a workgroup's row of 8-bit counts takes
    int nrc = s->ctx->scratch_acquire((size_t)(ngrid * nd) * 4, st, acc::SCRATCH_FOLD, &nblk);
    if (nrc != ACC_OK) { s->ctx->scratch_release(cblk, st); return nrc; }
    const uint64_t ndump = reinterpret_cast<uint64_t>(nblk.ptr), ncarry = reinterpret_cast<uint64_t>(cblk.ptr);
    args.i32(static_cast<int32_t>(ntarget));
    args.i32(1);
    args.ptr(ndump);
    args.ptr(ncarry);
    args.ptr(s->ctx->status_dev);
    nrc = launch(s, nv, ngrid, nlds, st, &args);
    const bool main_launched = nrc == ACC_OK;
    if (nrc == ACC_OK) {
      Args m;
      bool mal = true;
      nrc = push_env(s, env, &m, &mal);
      push_out(*out, &m, &mal);
      m.ptr(ndump);
      m.i64(nwords);
      m.i32(static_cast<int32_t>(ngrid));
      m.i64(ntarget);
      m.ptr(ncarry);
      m.ptr(direct_adds ? out->ptr[0] : defaults->ptr[0]);
      if (nrc == ACC_OK) {
        // a workgroup per 64 words of a row, each of its waves its share of the rows
        const unsigned merge_threads = 64u * static_cast<unsigned>(s->spec.merge_waves);
        hipError_t me = launch_kernel(s->variants[nv].fn_finish, static_cast<unsigned>((nd + 63) / 64), 1, 1, merge_threads, 1, 1, 0, st,
                                      m.data(), nullptr);
        if (me != hipSuccess) nrc = acc::fail_hip(me, "hipModuleLaunchKernel(permute_merge, narrow counts)");
      }
    }
    // (the merge clears the carries it reads: if the main kernel went out and the merge did not, they stay behind)
    if (nrc != ACC_OK && main_launched) s->ctx->scratch_mark_dirty(cblk);
    s->ctx->scratch_release(cblk, st);
    s->ctx->scratch_release(nblk, st);
    return nrc;
  }

  // A hinted combination on more targets than two LDS tables hold: windows of targets, each with its share of the
  // workgroups, which walk the whole source (skel_permute.h).  Up to `permute.max_windows` passes are cheaper than
  // a device-scope atomic per element (27 G/s for the whole device).
  if (s->spec.combine_hint != ACC_COMBINE_GENERIC) {
    const int64_t wcap = std::max<int64_t>(1, lds_all / (int64_t)esz);
    int win_log = 0;                                       // a power of two of windows: targets are dealt out modulo it
    while (((ntarget + ((int64_t)1 << win_log) - 1) >> win_log) > wcap) ++win_log;
    const int64_t windows = (int64_t)1 << win_log;
    if (windows >= s->knobs.permute_windows_from && windows <= s->knobs.permute_max_windows && n_src >= 4 * ntarget) {
      const int wv = (aligned ? 0 : 1) + 4;
      ACC_TRY(s->ensure_variant(wv));
      ACC_TRY(plain_copy());
      const int64_t wbins = (ntarget + windows - 1) >> win_log;
      const size_t wlds = (size_t)wbins * esz;
      int bpc = 0;
      hipError_t oe = hipModuleOccupancyMaxActiveBlocksPerMultiprocessor(&bpc, s->variants[wv].fn, s->spec.block, wlds);
      if (oe != hipSuccess || bpc < 1) { (void)hipGetLastError(); bpc = 1; }
      const int64_t cus_w = s->ctx->props.multiProcessorCount;
      const int64_t win_blocks = std::max<int64_t>(1, std::min<int64_t>(cus_w * bpc / windows,
                                                                         acc_launch_grid(n_src, s->elements_per_block(), cus_w, bpc)));
      const int64_t wgrid = windows * win_blocks;
      acc::ScratchRef wblk;
      ACC_TRY(s->ctx->scratch_acquire((size_t)(wgrid * wbins) * esz, st, acc::SCRATCH_FOLD, &wblk));
      const uint64_t wdump = reinterpret_cast<uint64_t>(wblk.ptr);
      args.i32(static_cast<int32_t>(wbins));
      args.i32(1);
      args.ptr(wdump);
      args.ptr(0);
      args.i32(static_cast<int32_t>(win_blocks));
      args.i32(win_log);
      int wrc = launch(s, wv, wgrid, wlds, st, &args);
      if (wrc == ACC_OK) {
        struct MergeJob { uint64_t dump; int64_t stride, first, cols; int32_t nrows, slices, window_log; };
        const int64_t columns = (ntarget + 255) / 256;
        const int64_t slices = std::max<int64_t>(1, std::min<int64_t>(win_blocks, (2 * cus_w + columns - 1) / columns));
        MergeJob ja = {wdump, wbins, 0, ntarget, static_cast<int32_t>(win_blocks), static_cast<int32_t>(slices), win_log};
        MergeJob jb = {0, 0, 0, 0, 0, 1, -1};
        int32_t blocks_a32 = static_cast<int32_t>(columns * slices);
        Args m;
        bool mal = true;
        wrc = push_env(s, env, &m, &mal);
        push_out(*out, &m, &mal);
        void **mslots = m.data_without_guard();
        std::vector<void *> margs(mslots, mslots + m.count());
        margs.push_back(&ja);
        margs.push_back(&blocks_a32);
        margs.push_back(&jb);
        uint64_t mguard = t_run.guard;
        if (t_run.guarded) margs.push_back(&mguard);
        if (wrc == ACC_OK) {
          hipError_t me = launch_kernel(s->variants[wv].fn_finish, static_cast<unsigned>(blocks_a32), 1, 1, 256, 1, 1, 0, st,
                                                margs.data(), nullptr);
          if (me != hipSuccess) wrc = acc::fail_hip(me, "hipModuleLaunchKernel(permute_merge, windows)");
        }
      }
      s->ctx->scratch_release(wblk, st);
      return wrc;
    }
  }

  const int v = aligned ? 0 : 1;
  ACC_TRY(s->ensure_variant(v));

  // privatise target indices [0, bins) in LDS when the combine has a hardware
  // atomic and an identity; small targets get one copy per wave to spread
  // same-address traffic
  const int cus = s->ctx->props.multiProcessorCount;
  int64_t bins = 0, copies = 1;
  if (s->spec.combine_hint != ACC_COMBINE_GENERIC) {
    const int64_t budget = std::min<int64_t>((int64_t)s->ctx->props.sharedMemPerBlock, s->knobs.permute_lds_bytes) - s->variants[v].static_lds;
    const int64_t cap = std::max<int64_t>(0, budget / (int64_t)esz);
    bins = std::min(ntarget, cap);
    if (bins == ntarget && bins > 0) copies = std::max<int64_t>(1, std::min<int64_t>(s->spec.block / 64, cap / bins));
    copies = std::min<int64_t>(copies, s->knobs.permute_max_copies);
  }
  const size_t lds = (size_t)(bins * copies) * esz;
  int bpc = 0;
  hipError_t e = hipModuleOccupancyMaxActiveBlocksPerMultiprocessor(&bpc, s->variants[v].fn, s->spec.block, lds);
  if (e != hipSuccess || bpc < 1) { (void)hipGetLastError(); bpc = 1; }
  const int64_t grid = acc_launch_grid(n_src, s->elements_per_block(), cus, std::min(bpc, s->knobs.permute_max_blocks_per_cu));

  // How the privatised part leaves the blocks: atomics while they are few, otherwise a table of
  // per-block bins folded by a second kernel.
  // Targets beyond the LDS window would be hit with device-scope atomics, the slowest operation on
  // the machine.  While a row of the whole target stays well inside one XCD's L2, the workgroups of
  // each XCD share such a row instead, and the rows are folded into the result afterwards.
  constexpr int64_t XCD_ROWS = 16;                 // what the kernel's XCC_ID field can name
  const bool far_rows = bins > 0 && bins < ntarget &&
                        ntarget * (int64_t)esz <= (int64_t)s->knobs.permute_xcd_row_kbytes << 10;
  const bool table = bins > 0 && grid * bins > s->knobs.permute_atomic_flush_max;
  const size_t far_bytes = far_rows ? (size_t)(XCD_ROWS * ntarget) * esz : 0;
  const size_t dump_bytes = table ? (size_t)(grid * bins) * esz : 0;
  acc::ScratchRef blk;
  uint64_t far = 0, dump = 0;
  if (far_rows || table) {
    ACC_TRY(s->ctx->scratch_acquire(far_bytes + dump_bytes, st, acc::SCRATCH_FOLD, &blk));
    const uint64_t base = reinterpret_cast<uint64_t>(blk.ptr);
    if (far_rows) far = base;
    if (table) dump = base + far_bytes;
  }
  // Where every target has its bin in LDS and the bins leave by atomics, the result's first contents -- the defaults --
  // are copied by workgroup 0 of the main kernel while the others read the source, and a word in scratch memory
  // ({epoch, 1}, as the fold's partial results are tagged) tells them when their atomics may follow: one launch.
  const bool inline_fill = copy_defaults && !far_rows && !table && bins == ntarget && bins > 0 && n_src > 0 &&
                           s->knobs.permute_inline_fill != 0;
  acc::ScratchRef rblk;
  if (inline_fill) {
    const int arc = s->ctx->scratch_acquire(256, st, acc::SCRATCH_FLAGS, &rblk);
    if (arc != ACC_OK) { s->ctx->scratch_release(blk, st); return arc; }
  }
  int rc = ACC_OK;
  if (far_rows) {                       // one launch: identity into the XCD rows, defaults into the result
    Args f;
    f.ptr(far);
    f.i64(XCD_ROWS * ntarget);
    f.ptr(out->ptr[0]);
    f.ptr(defaults->ptr[0]);
    f.i64(copy_defaults ? ntarget : 0);
    const int64_t fill_grid = std::min<int64_t>((XCD_ROWS * ntarget + 255) / 256, 8 * (int64_t)cus);
    e = launch_kernel(s->variants[v].fn_fill, static_cast<unsigned>(fill_grid), 1, 1, 256, 1, 1, 0, st, f.data(), nullptr);
    if (e != hipSuccess) rc = acc::fail_hip(e, "hipModuleLaunchKernel(permute_fill)");
  } else if (copy_defaults && !inline_fill) {   // the defaults by the same kernel: a runtime copy of 1 KB takes 4 us, this launch 2
    Args f;
    f.ptr(0);
    f.i64(0);
    f.ptr(out->ptr[0]);
    f.ptr(defaults->ptr[0]);
    f.i64(ntarget);
    const int64_t fill_grid = std::min<int64_t>((ntarget + 255) / 256, 8 * (int64_t)cus);
    e = launch_kernel(s->variants[v].fn_fill, static_cast<unsigned>(fill_grid), 1, 1, 256, 1, 1, 0, st, f.data(), nullptr);
    if (e != hipSuccess) rc = acc::fail_hip(e, "hipModuleLaunchKernel(permute_fill, defaults)");
  }
  args.i32(static_cast<int32_t>(bins));
  args.i32(static_cast<int32_t>(copies));
  args.ptr(dump);
  args.ptr(far);
  args.ptr(inline_fill ? defaults->ptr[0] : 0);
  args.ptr(reinterpret_cast<uint64_t>(rblk.ptr));
  args.u32(rblk.epoch);
  args.ptr(s->ctx->status_dev);
  if (rc == ACC_OK) rc = launch(s, v, grid, lds, st, &args);
  if (inline_fill) s->ctx->scratch_release(rblk, st);
  if (rc == ACC_OK && (table || far_rows)) {
    // the tables are folded into the result by one launch: the per-block window rows, the per-XCD rows
    struct MergeJob { uint64_t dump; int64_t stride, first, cols; int32_t nrows, slices, window_log; };
    auto job = [&](uint64_t tbl, int64_t stride, int64_t first, int64_t cols, int64_t rows, int64_t *blocks) {
      // enough workgroups to fill the machine: columns x row slices
      const int64_t columns = (cols + 255) / 256;
      const int64_t slices = std::max<int64_t>(1, std::min<int64_t>(rows, (2 * cus + columns - 1) / columns));
      *blocks = columns * slices;
      return MergeJob{tbl, stride, first, cols, static_cast<int32_t>(rows), static_cast<int32_t>(slices), -1};
    };
    int64_t blocks_a = 0, blocks_b = 0;
    MergeJob ja = {0, 0, 0, 0, 0, 1, -1}, jb = {0, 0, 0, 0, 0, 1, -1};
    if (table) ja = job(dump, bins, 0, bins, grid, &blocks_a);
    if (far_rows) jb = job(far, ntarget, bins, ntarget - bins, XCD_ROWS, &blocks_b);
    Args m;
    bool al = true;
    rc = push_env(s, env, &m, &al);
    push_out(*out, &m, &al);
    int32_t blocks_a32 = static_cast<int32_t>(blocks_a);
    void **mslots = m.data_without_guard();
    std::vector<void *> margs(mslots, mslots + m.count());
    margs.push_back(&ja);
    margs.push_back(&blocks_a32);
    margs.push_back(&jb);
    uint64_t mguard = t_run.guard;
    if (t_run.guarded) margs.push_back(&mguard);
    if (rc == ACC_OK) {
      e = launch_kernel(s->variants[v].fn_finish, static_cast<unsigned>(blocks_a + blocks_b), 1, 1, 256, 1, 1, 0, st, margs.data(), nullptr);
      if (e != hipSuccess) rc = acc::fail_hip(e, "hipModuleLaunchKernel(permute_merge)");
    }
  }
  s->ctx->scratch_release(blk, st);
  return rc;
}

// `in2` is the second source of a stencil2, NULL for a stencil
static int stencil_once(acc_skel s, const acc_array *env, const acc_array *in, const acc_array *in2, const acc_array *out, hipStream_t st)
{
  ACC_RUN_SCOPE(s, st);
  const int rank = s->spec.out_rank;
  Args args;
  bool aligned = true;
  ACC_TRY(push_env(s, env, &args, &aligned));
  push_out(*out, &args, &aligned);
  const int64_t w = out->shape[rank - 1];
  const int64_t h = rank >= 2 ? out->shape[rank - 2] : 1;
  const int64_t planes = rank == 3 ? out->shape[0] : 1;
  // rows start on 16-byte boundaries only if the row pitch allows it: of every component of a source
  auto row_aligned = [&](const acc_array &a, const std::vector<std::string> &comps) {
    const int nc = (int)comps.size();
    for (int c = 0; c < nc; ++c) {
      const size_t esz = acc::type_size(comps[nc - 1 - c]);          // component c is the (nc - 1 - c)-th in writing order
      if (!aligned16(a.ptr[c]) || (a.shape[rank - 1] * (int64_t)esz) % 16 != 0) return false;
    }
    return true;
  };
  // (of a tuple result: the rows of every component's array)
  const int ncomp = s->ncomp();
  for (int c = 0; c < ncomp; ++c) {
    const int64_t csz = ncomp == 1 ? (int64_t)s->spec.elt_size : (int64_t)acc::type_size(s->spec.comp_types[ncomp - 1 - c]);
    if ((w * csz) % 16 != 0) aligned = false;
  }
  if (!row_aligned(*in, s->spec.stencil_in_comps)) aligned = false;
  if (in2) {      // each source with its extents (Stencil.hs:146-152)
    if (!row_aligned(*in2, s->spec.stencil_in2_comps)) aligned = false;
    bool ignore = true;
    push_out(*in, &args, &ignore);
    push_out(*in2, &args, &ignore);
  } else {
    bool ignore = true;
    push_ptrs(in, in->ncomp, &args, &ignore);
  }
  if (array_size(*out) == 0) return ACC_OK;
  // An array of a few columns leaves nearly every lane of a strip outside it (3 x 3 on 2^24 x 3: 1.9 ms, 7 points on
  // 2^22 x 2 x 2 and 2^24 x 1 x 1: 0.76 and 2.8 ms): variants 6 and 7 of the instance, an element a thread as for the
  // stencils that strips cannot take, run at 2.8 (2-D) and 2.1 TB/s (3-D) whatever the shape, which is more than the
  // strips reach up to 36 columns in 2-D (2^20 rows of 28 / 33: 117 / 119 us in strips, 84 / 98 so; 2^19 of 40: 60
  // either way) and 16 in 3-D (2^17 x 8 x 16: 74 against 65; 2^14 x 32 x 32: 51 against 65).
  const bool thin = !s->spec.stencil_nd && ((rank == 2 && w <= s->knobs.stencil_thin_2d) || (rank == 3 && w <= s->knobs.stencil_thin_3d));
  if (s->spec.stencil_nd || thin) {
    // an element of the result a thread (skel_stencil_nd.h); the kernel takes the strips' `walk` and ignores it
    args.i32(0);
    const int v = (aligned ? 0 : 1) + (thin ? 6 : 0);
    ACC_TRY(s->ensure_variant(v));
    const int64_t grid = acc_launch_grid(array_size(*out), s->spec.block, resident(s, v), s->knobs.map_oversub);
    return launch(s, v, grid, 0, st, &args);
  }
  // one wave per strip of 256 columns x tile_h rows
  // (for 2-D the waves of a workgroup are stacked vertically, so the row count is rounded up to whole groups)
  const int64_t waves = s->spec.block / 64;
  // An array narrower than half a strip (a quarter) takes the variant with half (a quarter) of the columns a lane,
  // where the stencil's reach allows: the lanes of a strip that lie outside the array do nothing.
  int narrow = 0;
  while (narrow < s->knobs.stencil_narrow_max && (s->spec.svec >> (narrow + 1)) >= std::max(1, s->spec.reach_x) &&
         w <= (int64_t)64 * (s->spec.svec >> (narrow + 1)))
    ++narrow;
  // Strips that walk through planes are bound by the instructions of a strip, whatever its share of columns inside the
  // array: one and a half strips' width is taken as three strips of half the width, not as two of the whole one
  // (200 x 200 x 300: 35.3 -> 27.4 us), and less than one strip's width as two of half the width, not as one that the
  // edge of the array cuts (150^3: 17.0 -> 13.3 us).  (In 2-D the columns a last strip produces a second time cost
  // next to nothing.)
  if (narrow == 0 && s->spec.zmarch && (s->spec.svec >> 1) >= std::max(1, s->spec.reach_x) && s->knobs.stencil_half_strips != 0) {
    const int64_t halves = (w + 32 * s->spec.svec - 1) / (32 * s->spec.svec);
    if (halves == 3 || (halves == 2 && w < 64 * s->spec.svec)) narrow = 1;
  }
  const int64_t tile_w = (int64_t)64 * (s->spec.svec >> narrow);
  const int64_t strips_x = (w + tile_w - 1) / tile_w;
  int64_t bands = (h + s->spec.tile_h - 1) / s->spec.tile_h;
  if (rank == 2 && s->knobs.stencil_stack) bands = (bands + waves - 1) / waves * waves;
  int64_t zbands = (planes + s->spec.tile_z - 1) / s->spec.tile_z;             // tile_z result planes per strip
  int64_t walk = s->spec.tile_h;
  if (s->spec.zmarch) {                  // strips tile_z rows tall that walk through tile_h planes
    bands = (h + s->spec.tile_z - 1) / s->spec.tile_z;
    // ... or through fewer, halving down to 4, until there are three strips for every compute unit: a volume of
    // 256^3 has 256 strips of 64 planes, a wave for every fourth SIMD (44.1 us; 23.4 with 1024 strips of 16 planes,
    // although each reads 2 rz planes beyond its own; 128 x 128 x 256: 40.5 us -> 6.6 at 4 planes a strip).
    const int64_t enough = (int64_t)s->knobs.stencil_strips_per_cu * s->ctx->props.multiProcessorCount;
    const int64_t shortest = std::max(1, std::min(s->knobs.stencil_walk_min, s->spec.tile_h));
    while (walk / 2 >= shortest && strips_x * bands * ((planes + walk - 1) / walk) < enough) walk /= 2;
    zbands = (planes + walk - 1) / walk;
  }
  args.i32(static_cast<int32_t>(walk));
  return launch(s, (aligned ? 0 : 1) + 2 * narrow, (strips_x * bands * zbands + waves - 1) / waves, 0, st, &args);
}

static int stencil_check(acc_skel s, const acc_array *in, const acc_array *out)
{
  if (!s) return fail(ACC_ERR_INVALID, "acc_exec_stencil: NULL skeleton");
  if (!kind_is(s, {ACC_SKEL_STENCIL})) return fail(ACC_ERR_INVALID, "acc_exec_stencil: skeleton is '%s'", s->entry.c_str());
  ACC_TRY(check_out(s, out, s->spec.out_rank, "result"));
  ACC_TRY(check_out(s, in, s->spec.out_rank, "source", (int)s->spec.stencil_in_comps.size()));
  for (int d = 0; d < out->rank; ++d)
    if (in->shape[d] != out->shape[d]) return fail(ACC_ERR_INVALID, "stencil: source and result differ in shape");
  for (int ci = 0; ci < in->ncomp && array_size(*out) > 0; ++ci)
    for (int co = 0; co < out->ncomp; ++co)
      if (in->ptr[ci] == out->ptr[co]) return fail(ACC_ERR_INVALID, "stencil: source and result must not alias");
  return ACC_OK;
}

int acc_exec_stencil(acc_skel s, const acc_array *env, const acc_array *in, const acc_array *out, acc_stream stream)
{
  ACC_TRY(stencil_check(s, in, out));
  return stencil_once(s, env, in, nullptr, out, static_cast<hipStream_t>(stream));
}

int acc_exec_stencil2(acc_skel s, const acc_array *env, const acc_array *in1, const acc_array *in2, const acc_array *out, acc_stream stream)
{
  if (!s) return fail(ACC_ERR_INVALID, "acc_exec_stencil2: NULL skeleton");
  if (!kind_is(s, {ACC_SKEL_STENCIL2})) return fail(ACC_ERR_INVALID, "acc_exec_stencil2: skeleton is '%s'", s->entry.c_str());
  ACC_TRY(check_out(s, out, s->spec.out_rank, "result"));
  ACC_TRY(check_out(s, in1, s->spec.out_rank, "first source", (int)s->spec.stencil_in_comps.size()));
  ACC_TRY(check_out(s, in2, s->spec.out_rank, "second source", (int)s->spec.stencil_in2_comps.size()));
  for (int d = 0; d < out->rank; ++d)
    if (out->shape[d] > std::min(in1->shape[d], in2->shape[d]))
      return fail(ACC_ERR_INVALID, "stencil2: the result is larger than the intersection of the sources' extents");
  for (const acc_array *in : {in1, in2})
    for (int ci = 0; ci < in->ncomp && array_size(*out) > 0; ++ci)
      for (int co = 0; co < out->ncomp; ++co)
        if (in->ptr[ci] == out->ptr[co]) return fail(ACC_ERR_INVALID, "stencil2: a source and the result must not alias");
  return stencil_once(s, env, in1, in2, out, static_cast<hipStream_t>(stream));
}

int acc_exec_stencil_iterate(acc_skel s, const acc_array *env, const acc_array *a, const acc_array *b, int32_t iters, acc_stream stream, int32_t *result_in_b)
{
  ACC_TRY(stencil_check(s, a, b));
  if (iters < 0) return fail(ACC_ERR_INVALID, "stencil: negative iteration count");
  const acc_array *src = a, *dst = b;
  for (int32_t i = 0; i < iters; ++i) {
    ACC_TRY(stencil_once(s, env, src, nullptr, dst, static_cast<hipStream_t>(stream)));
    std::swap(src, dst);
  }
  if (result_in_b) *result_in_b = (iters & 1);
  return ACC_OK;
}

}  // extern "C"
