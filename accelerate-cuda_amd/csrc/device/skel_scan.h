/*
 * skel_scan.h -- scanl, scanl1, scanl', scanr, scanr1, scanr' over a vector.
 *
 * Takes the place of the reference's three-kernel scan
 * (CodeGen/PrefixSum.hs:200-365 downsweep, :373-464 upsweep, :470-480 scan of
 * the interval totals, driven by Execute.hs:364-392).  Here it is ONE kernel:
 * a single-pass chained scan with decoupled look-back, so the input is read
 * once and the output written once.
 *
 *   - a tile is ACC_BLOCK threads x ACC_ROWS rows x ACC_VEC consecutive items;
 *     each lane touches ACC_VEC consecutive elements per row, so a wave reads
 *     64*ACC_VEC contiguous elements per row (128-bit accesses for 4-byte types);
 *   - inside a wave the row totals are scanned with DPP row shifts / row
 *     broadcasts (acc_wave_scan), waves are stitched through a few words of LDS;
 *   - tiles are chained through one descriptor per tile {state, value} in
 *     global memory.  A tile first publishes its own total (state AGGREGATE),
 *     then one wave walks back over its predecessors, 64 descriptors per step,
 *     until it meets an inclusive PREFIX, and finally publishes its own PREFIX.
 *     Every predecessor of a tile that is being worked on is itself held by a
 *     running workgroup (see the kernel), so the walk cannot deadlock.
 *   - descriptors are tagged with a launch epoch and the counter is used
 *     relative to a base, so nothing needs clearing between launches.
 *
 * The operator needs no identity and need not commute: `op(earlier, later)`
 * is applied in logical order only.  For the right-handed scans logical order
 * is the reverse of memory order and op(a, b) = f(b, a), i.e. the Data.List
 * convention out[i] = f x[i] out[i+1] (PrefixSum.hs:137-141).
 *
 * Output modes (physical index i, logical order as above):
 *   0  scanl : out[i] = exclusive(i),            out[n] = total     (n+1 results)
 *   1  scan?1: out[i] = inclusive(i)
 *   2  scan?': out[i] = exclusive(i),            sum[0] = total
 *   3  scanr : out[i] = inclusive(i) incl. seed, out[n] = seed      (n+1 results)
 * which is the pointer arithmetic of Execute.hs:328-362 folded into the kernel.
 *
 * Generated definitions expected: ACC_ENTRY, ACC_ELT, ACC_ENV_PARAMS,
 * ACC_ENV_ASSUME, ACC_GET(ix), ACC_COMBINE(x,y), ACC_HAS_SEED, ACC_SEED,
 * ACC_SCAN_RIGHT, ACC_SCAN_MODE, ACC_BLOCK, ACC_ROWS, ACC_VEC, ACC_ALIGNED.
 */

#define ACC_ITEMS (ACC_ROWS * ACC_VEC)
#define ACC_TILE  (ACC_BLOCK * ACC_ITEMS)
#define ACC_WAVES (ACC_BLOCK / ACC_WAVE)

#ifndef ACC_LOOKBACK
#define ACC_LOOKBACK 4
#endif

#ifndef ACC_DESC_STRIDE
#define ACC_DESC_STRIDE 1     /* 8-byte words between the descriptors of consecutive tiles */
#endif

#define ACC_ST_AGGREGATE 1u
#define ACC_ST_PREFIX    2u

/* ---- tile descriptors --------------------------------------------------- */
/* elements of at most 4 bytes: {flag, value} packed in one 64-bit word that is
 * read and written with relaxed device-scope atomics -- no fences at all     */
template <typename T, bool SMALL = (sizeof(T) <= 4)>
struct acc_scan_desc {
  unsigned long long *d;
  ACC_DEV acc_scan_desc(void *p0, void *, void *) : d((unsigned long long *)p0) {}
  ACC_DEV void put(Int64 tile, unsigned int flag, const T &v) const
  {
    unsigned int b = 0;
    __builtin_memcpy(&b, &v, sizeof(T));
    __hip_atomic_store(d + tile * ACC_DESC_STRIDE, ((unsigned long long)flag << 32) | b, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
  ACC_DEV unsigned int get(Int64 tile, T &v) const
  {
    unsigned long long w = __hip_atomic_load(d + tile * ACC_DESC_STRIDE, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    unsigned int b = (unsigned int)w;
    __builtin_memcpy(&v, &b, sizeof(T));
    return (unsigned int)(w >> 32);
  }
};

/* wider elements: cut into 4-byte pieces, each in a 64-bit word of its own next to
 * the same flag, all relaxed device-scope atomics as above.  (A plain value slot
 * plus a released flag costs a cache-wide write-back per tile and an invalidate
 * per poll on this part: scans of 8-byte elements ran at a third of the speed.)
 * A descriptor is complete when all its words carry the same flag; while a tile
 * replaces its AGGREGATE by its PREFIX a reader may meet both, and reads again. */
template <typename T>
struct acc_scan_desc<T, false> {
  static constexpr int NW = (int)((sizeof(T) + 3) / 4);
  static constexpr int SLOT = NW > ACC_DESC_STRIDE ? NW : ACC_DESC_STRIDE;     /* 8-byte words per tile */
  unsigned long long *d;
  ACC_DEV acc_scan_desc(void *p0, void *, void *) : d((unsigned long long *)p0) {}
  ACC_DEV void put(Int64 tile, unsigned int flag, const T &v) const
  {
    unsigned int b[NW] = {};
    __builtin_memcpy(b, &v, sizeof(T));
#pragma unroll
    for (int k = 0; k < NW; ++k)
      __hip_atomic_store(d + tile * SLOT + k, ((unsigned long long)flag << 32) | b[k], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
  ACC_DEV unsigned int get(Int64 tile, T &v) const
  {
    unsigned int b[NW];
    unsigned int f = 0;
    bool same = true;
#pragma unroll
    for (int k = 0; k < NW; ++k) {
      const unsigned long long w = __hip_atomic_load(d + tile * SLOT + k, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      b[k] = (unsigned int)w;
      if (k == 0) f = (unsigned int)(w >> 32);
      else same = same && (unsigned int)(w >> 32) == f;
    }
    __builtin_memcpy(&v, b, sizeof(T));
    return same ? f : 0u;                 /* 0 is no launch's flag: the caller reads again */
  }
};

/* ---- decoupled look-back, executed by wave 0 of a tile > 0 ---------------
 * Every step inspects ACC_LOOKBACK descriptors per lane, 64 * ACC_LOOKBACK
 * predecessors in one memory round trip.  The chain of tiles can advance by
 * at most one such window per round trip, so the window has to be wide
 * enough for the rate at which tiles retire.                                */
/* first window of the walk: only issues the loads, so that the caller can put
 * other memory traffic behind them before their results are needed          */
template <typename T>
struct acc_scan_window {
  T v[ACC_LOOKBACK];
  unsigned int fl[ACC_LOOKBACK];
};

template <typename T>
ACC_DEV void acc_scan_window_load(const acc_scan_desc<T> &desc, const Int64 look, const int lane, acc_scan_window<T> &w)
{
#pragma unroll
  for (int j = 0; j < ACC_LOOKBACK; ++j) {
    const Int64 idx = look - (lane * ACC_LOOKBACK + j);
    w.v[j] = T();
    w.fl[j] = 0;
    if (idx >= 0) w.fl[j] = desc.get(idx, w.v[j]);
  }
}

template <typename T, typename Op>
ACC_DEV T acc_scan_lookback(const acc_scan_desc<T> &desc, Int64 tile, const T &block_total, Op op,
                            unsigned int epoch, int lane, acc_scan_window<T> &w, unsigned int *status)
{
  /* slots are ordered nearest predecessor first, so a reduction in slot order
   * must combine (later, earlier) */
  auto back = acc_lift<T>([&](const T &later, const T &earlier) -> T { return op(earlier, later); });
  acc_opt<T> run = acc_none<T>();
  /* A descriptor that does not turn up within ACC_SPIN_LIMIT polls of this lane (all its waits together) is given
   * up: the walk ends there with whatever it has, the status block says so, and this tile still posts a PREFIX, so
   * that its successors do not wait for it in turn. */
  int polls = 0;

  for (Int64 look = tile - 1;; look -= ACC_WAVE * ACC_LOOKBACK) {
    if (look != tile - 1) acc_scan_window_load(desc, look, lane, w);
    int nearest = ACC_WAVE * ACC_LOOKBACK;              /* slot of the nearest PREFIX, if any */
#pragma unroll
    for (int j = 0; j < ACC_LOOKBACK; ++j) {
      const Int64 idx = look - (lane * ACC_LOOKBACK + j);
      if (idx >= 0) {
        while ((w.fl[j] >> 2) != epoch && polls < ACC_SPIN_LIMIT) {
          ++polls;
          __builtin_amdgcn_s_sleep(1);
          w.fl[j] = desc.get(idx, w.v[j]);
        }
      }
      const unsigned long long m = __ballot(idx >= 0 && (w.fl[j] & 3u) == ACC_ST_PREFIX);
      if (m) nearest = acc_min(nearest, (__ffsll((long long)m) - 1) * ACC_LOOKBACK + j);
    }
    acc_opt<T> c = acc_none<T>();
#pragma unroll
    for (int j = 0; j < ACC_LOOKBACK; ++j) {
      acc_opt<T> e;
      e.v = w.v[j];
      e.ok = (look - (lane * ACC_LOOKBACK + j) >= 0) && (lane * ACC_LOOKBACK + j <= nearest);
      c = back(c, e);
    }
    run = back(run, acc_wave_reduce(c, back));
    if (nearest < ACC_WAVE * ACC_LOOKBACK) break;       /* tile 0 always posts a PREFIX: the walk ends */
    if (__ballot(polls >= ACC_SPIN_LIMIT) != 0) {
      if (lane == 0) acc_report(status, ACC_STATUS_SCAN_LOOKBACK);
      break;
    }
  }
  const T prefix = run.v;
  if (lane == 0) desc.put(tile, (epoch << 2) | ACC_ST_PREFIX, op(prefix, block_total));
  return prefix;
}

/* the result arrays as the tile code sees them */
template <typename Put, typename Set, typename Total>
struct acc_scan_out {
  Put put_;  Set set_;  Total total_;
  ACC_DEV void put(const Int64 ix, const ACC_ELT &v) const { put_(ix, v); }
  ACC_DEV void set(const Int64 ix, const ACC_ELT &v) const { set_(ix, v); }
  ACC_DEV void total(const ACC_ELT &v) const { total_(v); }
};

/* ---- one tile ------------------------------------------------------------ */
/* physical index of item 0 of row r of this lane; item k is k further on in
 * logical order (for right-handed scans: k further back in memory)          */
ACC_DEV Int64 acc_scan_ix0(const Int64 base, const int wave, const int lane, const int r)
{
  const int q = ((wave * ACC_ROWS + r) * ACC_WAVE + lane) * ACC_VEC;     /* logical offset in the tile */
  return base + (ACC_SCAN_RIGHT ? (ACC_TILE - 1 - q) : q);
}

/* issue the loads of a tile; nothing here waits for them */
template <typename T, typename Get>
ACC_DEV void acc_scan_load(Get get, const Int64 base, const Int64 n, T (&x)[ACC_ROWS][ACC_VEC], const int wave, const int lane)
{
  if (base >= 0 && base + ACC_TILE <= n) {
#pragma unroll
    for (int r = 0; r < ACC_ROWS; ++r) {
      const Int64 i0 = acc_scan_ix0(base, wave, lane, r);
#pragma unroll
      for (int k = 0; k < ACC_VEC; ++k) x[r][k] = get(ACC_SCAN_RIGHT ? i0 - k : i0 + k);
    }
  } else if (n < ACC_VEC) {
    /* fewer elements than a vector: every position reads the nearest element of the array */
#pragma unroll
    for (int r = 0; r < ACC_ROWS; ++r) {
      const Int64 i0 = acc_scan_ix0(base, wave, lane, r);
#pragma unroll
      for (int k = 0; k < ACC_VEC; ++k) {
        const Int64 ix = ACC_SCAN_RIGHT ? i0 - k : i0 + k;
        x[r][k] = get(acc_max<Int64>(0, acc_min<Int64>(ix, n - 1)));
      }
    }
  } else {
    /* A tile that reaches outside the array, read WITHOUT a branch per row (a branch around a load makes the
     * compiler wait for that load on the spot, and 32 rows of such waits took 8 us): every row reads one whole
     * vector -- its own where that lies inside the array, else the last whole vector of the array, whose values
     * stand in positions that never reach a result -- and the one vector that lies across the end of the array
     * (there is one if the length is no multiple of the vector) is read once, element by element, by every
     * lane, and put in the place of the row that holds it. */
    const Int64 nv = n / ACC_VEC * ACC_VEC;                 /* where the vector across the end begins, if nv < n */
    T tail[ACC_VEC];
#pragma unroll
    for (int k = 0; k < ACC_VEC; ++k) tail[k] = get(acc_min<Int64>(nv + k, n - 1));
    const Int64 spare = nv - ACC_VEC;                      /* a whole vector inside the array (n >= ACC_VEC) */
#pragma unroll
    for (int r = 0; r < ACC_ROWS; ++r) {
      const Int64 i0 = acc_scan_ix0(base, wave, lane, r);
      const Int64 lo = ACC_SCAN_RIGHT ? i0 - (ACC_VEC - 1) : i0;
      const bool whole = lo >= 0 && lo + ACC_VEC <= n;
      const Int64 at = whole ? lo : spare;                 /* lowest physical index of the vector read */
      const Int64 a0 = ACC_SCAN_RIGHT ? at + (ACC_VEC - 1) : at;
#pragma unroll
      for (int k = 0; k < ACC_VEC; ++k) x[r][k] = get(ACC_SCAN_RIGHT ? a0 - k : a0 + k);
    }
    /* every load above is in flight before the first result is looked at */
    __builtin_amdgcn_sched_barrier(0);
    if (nv < n) {
#pragma unroll
      for (int r = 0; r < ACC_ROWS; ++r) {
        const Int64 i0 = acc_scan_ix0(base, wave, lane, r);
        const bool across = (ACC_SCAN_RIGHT ? i0 - (ACC_VEC - 1) : i0) == nv;
#pragma unroll
        for (int k = 0; k < ACC_VEC; ++k) x[r][k] = across ? tail[ACC_SCAN_RIGHT ? ACC_VEC - 1 - k : k] : x[r][k];
      }
    }
  }
}

/* scan one tile whose elements are already in registers.  `prefetch` is
 * called once the block total is known and before the look-back starts: the
 * caller uses it to put the next tile's loads in flight behind the wait.
 *
 * GUARD: the tile reaches outside the array.  Tiles are laid so that the
 * positions outside come LAST in scan order (left-handed scans count tiles
 * from element 0, right-handed ones from the end of the array rounded up to a
 * whole vector): whatever stands there only enters results that are never
 * stored and an aggregate no other tile reads, so the same code runs on it,
 * with the stores guarded.  The one exception is the rounding of a
 * right-handed scan: up to ACC_VEC - 1 positions past the end come FIRST, in
 * the first vector of the first tile, and the lane that holds them starts its
 * own scan at the first element inside (`lead` below).                       */
/* HOW: 0 the tile lies inside the array, 1 it reaches outside, 2 `outside` says which at run time.  (Two forms
 * side by side in one kernel cost registers: the compiler moves what they share above the branch between them.
 * For a right-handed scan of 32 rows that is 275 registers against 184 for the run-time form alone, and 256 is
 * where a second workgroup stops fitting on the compute unit.  Left-handed scans keep the two compiled forms: 185.) */
template <int HOW, typename T, typename Op, typename Prefetch, typename Out>
ACC_DEV void acc_scan_tile(const T (&x)[ACC_ROWS][ACC_VEC], Op op, const T seed, const Int64 tile, const Int64 base,
                           const Int64 n, const Out &out, const acc_scan_desc<T> &desc,
                           const unsigned int epoch, void *s_wave_raw, T *s_prefix, Prefetch prefetch, const bool outside,
                           unsigned int *status)
{
  const bool GUARD = HOW == 2 ? outside : (HOW == 1);
  typedef T V;
  struct S {
    static ACC_DEV V some(const T &v) { return v; }
    static ACC_DEV T val(const V &v) { return v; }
  };
  auto op_raw = op;

  const int lane = acc_lane();
  const int wave = (int)(threadIdx.x >> 6);
  V *s_wave = (V *)s_wave_raw;

  /* scan the ACC_VEC items each lane holds per row */
  V s[ACC_ROWS][ACC_VEC];
  /* positions past the end that come first in this lane's vector of row r.  (Neither this nor the row's first index
   * is kept from here to the stores: a tile of 32 rows would spend 100 registers on them.) */
  auto lead_of = [&](const Int64 i0) -> int {
    return (GUARD && ACC_SCAN_RIGHT) ? (int)acc_max<Int64>(0, acc_min<Int64>(i0 - (n - 1), ACC_VEC - 1)) : 0;
  };
#pragma unroll
  for (int r = 0; r < ACC_ROWS; ++r) {
    const int lead = (GUARD && ACC_SCAN_RIGHT) ? lead_of(acc_scan_ix0(base, wave, lane, r)) : 0;
    if (GUARD && ACC_SCAN_RIGHT) {
#pragma unroll
      for (int k = 0; k < ACC_VEC; ++k) {
        const V v = x[r][k];
        s[r][k] = (k == 0 || k == lead) ? v : op(s[r][k - 1], v);
      }
    } else {                                /* every other tile: no test per element */
#pragma unroll
      for (int k = 0; k < ACC_VEC; ++k) {
        const V v = x[r][k];
        s[r][k] = (k == 0) ? v : op(s[r][k - 1], v);
      }
    }
  }

  /* scan the per-lane totals of every row across the wave; the rows are
   * independent chains, which keeps the DPP pipeline busy */
  V ci[ACC_ROWS];
#pragma unroll
  for (int r = 0; r < ACC_ROWS; ++r) ci[r] = acc_wave_scan(s[r][ACC_VEC - 1], op, lane);

  /* (What the rows before row r of this wave come to is worked out again where it is used, by the same chain of
   * operations, instead of being kept from here: where the operator has no scalar instruction -- Float64 `+` --
   * that is two vector registers a row, and the instance then misses the 256 that let two workgroups share a
   * compute unit.) */
  /* (Elements of one register keep the values: the compiler holds them in scalar registers, and the headline
   * scan's code stays what it was measured as.) */
  constexpr bool KEEP_ROWS = sizeof(T) <= 4;
  V rowpre[KEEP_ROWS ? ACC_ROWS : 1];
  V wave_total = acc_readlane(ci[0], ACC_WAVE - 1);
  rowpre[0] = wave_total;                                   /* unused */
#pragma unroll
  for (int r = 1; r < ACC_ROWS; ++r) {
    if (KEEP_ROWS) rowpre[r] = wave_total;
    wave_total = op(wave_total, acc_readlane(ci[r], ACC_WAVE - 1));
  }

  /* stitch the waves of the block */
  if (lane == 0) s_wave[wave] = wave_total;
  __syncthreads();
  V wavepre = s_wave[0];
  V block_total = s_wave[0];
#pragma unroll
  for (int w = 1; w < ACC_WAVES; ++w) {
    if (w == wave) wavepre = block_total;
    block_total = op(block_total, s_wave[w]);
  }

  /* publish early, then start the next tile's loads, then look back */
  T prefix = seed;
  bool has_prefix = ACC_HAS_SEED;
  if (tile == 0) {
    if (threadIdx.x == 0)
      desc.put(0, (epoch << 2) | ACC_ST_PREFIX,
               ACC_HAS_SEED ? op_raw(seed, S::val(block_total)) : S::val(block_total));
    prefetch();
  } else {
    if (threadIdx.x == 0) desc.put(tile, (epoch << 2) | ACC_ST_AGGREGATE, S::val(block_total));
    acc_scan_window<T> win;
    if (wave == 0) acc_scan_window_load(desc, tile - 1, lane, win);   /* ahead of the prefetch: results return in issue order */
    prefetch();
    if (wave == 0) {
      const T p = acc_scan_lookback(desc, tile, S::val(block_total), op_raw, epoch, lane, win, status);
      if (lane == 0) *s_prefix = p;
    }
    __syncthreads();
    prefix = *s_prefix;
    has_prefix = true;
  }

  /* apply the prefixes and write.  The rows' indices are worked out again from a copy of `base` the compiler cannot
   * see through: otherwise it keeps the ones of the first loop alive across the whole tile, in the guarded form of
   * a right-handed scan three registers a row -- and that one tile's form sets the register count of the kernel. */
  Int64 late_base = base;
  asm volatile("" : "+s"(late_base));
  /* where the logically last element of the array sits, if in this tile: offset q in the tile's scan order is
   * item q % ACC_VEC of lane (q / ACC_VEC) % 64 in row (q / (64 ACC_VEC)) % ACC_ROWS of wave q / (64 ACC_VEC ACC_ROWS) */
  const Int64 last_q = ACC_SCAN_RIGHT ? base + (ACC_TILE - 1) : (n - 1) - base;
  const bool holds_last = (ACC_SCAN_MODE == 0 || ACC_SCAN_MODE == 2) && last_q >= 0 && last_q < ACC_TILE;
  const int last_k = (int)(last_q % ACC_VEC), last_lane = (int)((last_q / ACC_VEC) % ACC_WAVE);
  const int last_row = (int)((last_q / (ACC_VEC * ACC_WAVE)) % ACC_ROWS), last_wave = (int)(last_q / (ACC_VEC * ACC_WAVE * ACC_ROWS));
  V whole = V();
  V rows_before = V();                                      /* rows 0 .. r - 1 of this wave, for r > 0 */
#pragma unroll
  for (int r = 0; r < ACC_ROWS; ++r) {
    if (KEEP_ROWS)   rows_before = rowpre[r];
    else if (r == 1) rows_before = acc_readlane(ci[0], ACC_WAVE - 1);
    else if (r > 1)  rows_before = op(rows_before, acc_readlane(ci[r - 1], ACC_WAVE - 1));
    V b = S::some(prefix);
    bool has_b = has_prefix;
    if (wave > 0) { b = has_b ? op(b, wavepre) : wavepre; has_b = true; }
    if (r > 0)    { b = has_b ? op(b, rows_before) : rows_before; has_b = true; }

    const V e = acc_wave_shift_up1(ci[r]);                  /* total of the lanes before this one */
    V pre;
    bool has_pre;
    if (has_b) { pre = (lane == 0) ? b : op(b, e); has_pre = true; }
    else       { pre = e; has_pre = (lane > 0); }

    V inc[ACC_VEC];
#pragma unroll
    for (int k = 0; k < ACC_VEC; ++k) inc[k] = has_pre ? op(pre, s[r][k]) : s[r][k];

    /* the body: one straight run of stores per row so that they merge into
     * 128-bit accesses; in a tile that reaches outside the array only for the
     * vectors that lie inside it */
    const bool exclusive = (ACC_SCAN_MODE == 0 || ACC_SCAN_MODE == 2);
    const Int64 i0 = acc_scan_ix0(late_base, wave, lane, r);
    const Int64 lo = ACC_SCAN_RIGHT ? i0 - (ACC_VEC - 1) : i0;
    if (!GUARD || (lo >= 0 && lo + ACC_VEC <= n)) {
#pragma unroll
      for (int k = 0; k < ACC_VEC; ++k) {
        const Int64 ix = ACC_SCAN_RIGHT ? i0 - k : i0 + k;
        out.put(ix, exclusive ? S::val(k == 0 ? pre : inc[k - 1]) : S::val(inc[k]));
      }
    } else {
#pragma unroll
      for (int k = 0; k < ACC_VEC; ++k) {
        const Int64 ix = ACC_SCAN_RIGHT ? i0 - k : i0 + k;
        if (ix < 0 || ix >= n) continue;
        const bool first = (k == 0) || (ACC_SCAN_RIGHT && k == lead_of(i0));
        const V before = (k == 0) ? pre : (first ? pre : inc[k - 1]);     /* (k == 0 keeps inc[-1] out of the expression) */
        out.set(ix, exclusive ? S::val(before) : S::val(inc[k]));
      }
    }

    /* the reduction of the whole vector is the inclusive value of the logically last element: the row that holds
     * it keeps the value, and the one lane stores it after the loop (a store per row and position, each under its
     * own test, made the kernel half as long again, and the exclusive scans 2 % slower than the inclusive ones) */
    if (holds_last && r == last_row) {
      V c = inc[0];
#pragma unroll
      for (int k = 1; k < ACC_VEC; ++k) c = (k == last_k) ? inc[k] : c;
      whole = c;
    }
  }
  if (holds_last && wave == last_wave && lane == last_lane) {
    if (ACC_SCAN_MODE == 0) out.set(n, S::val(whole));
    else                    out.total(S::val(whole));
  }
}

/* One workgroup per tile, tile number = workgroup number.  Workgroups are dispatched in increasing order, so every
 * predecessor of a running tile has itself been dispatched and the look-back always makes progress.  (Resident
 * grids of workgroups that draw tiles from a counter, or take them in strides under a cooperative launch, and load
 * the next tile behind the look-back, were measured at 110-340 us against 96 and are gone.) */
/* second launch bound = waves per SIMD the register allocation must leave room for */
#ifndef ACC_MIN_WAVES
#define ACC_MIN_WAVES 1
#endif
#ifndef ACC_SCAN_TICKET
#define ACC_SCAN_TICKET 0
#endif
extern "C" __global__ void __launch_bounds__(ACC_BLOCK, ACC_MIN_WAVES)
ACC_ENTRY(ACC_ENV_PARAMS
          const Int64 shOut_0, ACC_OUT_ARRAY(arrOut),
          ACC_OUT_ARRAY(arrSum),
          const Int64 shIn_0,
          void *desc0, void *desc1, void *desc2,
          const unsigned int epoch_given, const Int64 num_tiles, unsigned int *acc_status ACC_GUARD_PARAM)
{
  ACC_GUARD_CHECK
  typedef ACC_ELT T;
  ACC_ENV_ASSUME
  /* The launch's tag: what the host chose for this launch, or -- 0 given -- what the first word of the 256-byte header
   * in front of the descriptors holds, put there by a kernel that ran just before on the same stream.  A launch
   * recorded into a graph keeps its arguments for every replay; its tag must not be among them, or the descriptors
   * the replay before left behind would read as published. */
  const unsigned int epoch = epoch_given ? epoch_given : *(const unsigned int *)((const char *)desc0 - 256);
#if ACC_ALIGNED
  ACC_OUT_ASSUME(arrOut)
#endif
  (void)shOut_0;

  __shared__ T s_prefix;
  __shared__ acc_opt<T> s_wave[ACC_WAVES];

  auto get = [&](const Int64 ix) -> T { return (ACC_GET(ix)); };
  auto f   = [&](const T &x, const T &y) -> T { return (ACC_COMBINE(x, y)); };
  auto op  = [&](const T &earlier, const T &later) -> T { return ACC_SCAN_RIGHT ? f(later, earlier) : f(earlier, later); };

  const Int64 n = shIn_0;
#if ACC_HAS_SEED
  const T seed = (ACC_SEED);
#else
  const T seed = T();
#endif
  const int lane = acc_lane();
  const int wave = (int)(threadIdx.x >> 6);
  const acc_scan_desc<T> desc(desc0, desc1, desc2);
  /* where results go: one array per component of the element */
  auto put_fn   = [&](const Int64 ix, const T &v) { ACC_PUT(arrOut, ix, v); };      /* the body, streaming */
  auto set_fn   = [&](const Int64 ix, const T &v) { ACC_SET(arrOut, ix, v); };
  auto total_fn = [&](const T &v) { ACC_SET(arrSum, 0, v); };
  const acc_scan_out<decltype(put_fn), decltype(set_fn), decltype(total_fn)> out = {put_fn, set_fn, total_fn};
  /* first physical index of scan tile t (right-handed: tiles count down from the end of the array, rounded up to a
   * whole vector so that the 128-bit accesses stay aligned; the last tile may start below 0) */
  const Int64 n_up = (n + ACC_VEC - 1) / ACC_VEC * ACC_VEC;
  auto tile_base = [&](const Int64 t) -> Int64 { return ACC_SCAN_RIGHT ? n_up - (t + 1) * (Int64)ACC_TILE : t * (Int64)ACC_TILE; };

#if ACC_SCAN_TICKET
  /* (measurement: tiles numbered by a counter in the header, zeroed by the host before the launch, instead of by
   * workgroup index -- no reliance on the order in which workgroups are dispatched, at the price of one device-scope
   * addition on one address per tile) */
  __shared__ unsigned int s_ticket;
  if (threadIdx.x == 0)
    s_ticket = __hip_atomic_fetch_add((unsigned int *)((char *)desc0 - 256 + 64), 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  __syncthreads();
  const Int64 tile = (Int64)s_ticket;
#else
  const Int64 tile = (Int64)blockIdx.x;
#endif

  if (n <= 0) {                                   /* PrefixSum.hs:249-251,330-334: scan of nothing is [seed] */
    if (threadIdx.x == 0 && tile == 0) {
      if (ACC_SCAN_MODE == 0 || ACC_SCAN_MODE == 3) ACC_SET(arrOut, 0, seed);
      if (ACC_SCAN_MODE == 2) ACC_SET(arrSum, 0, seed);
    }
    return;
  }
  if (ACC_SCAN_MODE == 3 && tile == 0 && threadIdx.x == 0) ACC_SET(arrOut, n, seed);

  T cur[ACC_ROWS][ACC_VEC];
  if (tile < num_tiles) acc_scan_load(get, tile_base(tile), n, cur, wave, lane);

  if (tile < num_tiles) {
    auto prefetch = [&]() {};
    const Int64 base = tile_base(tile);
    const bool inside = base >= 0 && base + ACC_TILE <= n;
    acc_scan_tile<2, T>(cur, op, seed, tile, base, n, out, desc, epoch, (void *)s_wave, &s_prefix, prefetch, !inside, acc_status);

  }
}
