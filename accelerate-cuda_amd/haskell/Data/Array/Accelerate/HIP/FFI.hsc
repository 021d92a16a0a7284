{-# LANGUAGE ForeignFunctionInterface, EmptyDataDecls, DeriveDataTypeable #-}
-- |
-- Module      : Data.Array.Accelerate.HIP.FFI
--
-- Bindings to libacchip (include/acc_hip.h), one foreign import per entry point of the
-- library, for a Data.Array.Accelerate.HIP backend that keeps the structure of
-- Data.Array.Accelerate.CUDA and replaces what that obtains from the `cuda` package,
-- from nvcc and from its own skeleton templates.
--
-- UNCOMPILED: the image this library is built and tested in holds no GHC.  The import
-- list is checked mechanically against the header (names and argument counts); the
-- Storable instances use hsc2hs against the same header, so offsets cannot drift.
--
-- Calls that can block (compilation, synchronisation, copies, anything that may
-- allocate) are `safe`; the two string getters and the pure launch arithmetic are `unsafe`.
-- Every entry point makes the context's device current itself and may be called from any
-- thread, so the bound-thread / push / pop discipline of State.hs:84-92 is not needed.
--
module Data.Array.Accelerate.HIP.FFI where

import Control.Exception
import Control.Monad
import Data.Typeable
import Foreign
import Foreign.C

#include "acc_hip.h"

data CContext
data CSkel
data CMemTable
data CGuard
type Context  = Ptr CContext
type Skel     = Ptr CSkel
type MemTable = Ptr CMemTable
type Guard    = Ptr CGuard
type Stream   = Ptr ()               -- hipStream_t; nullPtr is the default stream
type Event    = Ptr ()
type Module   = Ptr ()
type Function = Ptr ()
type DevPtr   = Word64               -- in place of Foreign.CUDA.Ptr.DevicePtr: advanceDevPtr / plusDevPtr are (+)
type Status   = CInt

-- ---------------------------------------------------------------------------------------------------------
-- status codes and the exception they become (the reference's CUDAException; State.hs:86-88)

accOK, accErrInvalid, accErrOOM, accErrCompile, accErrNotFound, accErrHIP, accErrUnsupported, accErrIO, accErrStuck :: Status
accOK             = #{const ACC_OK}
accErrInvalid     = #{const ACC_ERR_INVALID}
accErrOOM         = #{const ACC_ERR_OOM}
accErrCompile     = #{const ACC_ERR_COMPILE}
accErrNotFound    = #{const ACC_ERR_NOT_FOUND}
accErrHIP         = #{const ACC_ERR_HIP}
accErrUnsupported = #{const ACC_ERR_UNSUPPORTED}
accErrIO          = #{const ACC_ERR_IO}
accErrStuck       = #{const ACC_ERR_STUCK}

-- skeleton kinds, combination hints and flags of a skeleton description (acc_skel_desc)
accSkelMap, accSkelGenerate, accSkelTransform, accSkelFold, accSkelFold1, accSkelFoldSeg, accSkelFold1Seg,
  accSkelScanl, accSkelScanl1, accSkelScanlP, accSkelScanr, accSkelScanr1, accSkelScanrP, accSkelPermute,
  accSkelStencil, accSkelStencil2 :: Int32
accSkelMap       = #{const ACC_SKEL_MAP}
accSkelGenerate  = #{const ACC_SKEL_GENERATE}
accSkelTransform = #{const ACC_SKEL_TRANSFORM}
accSkelFold      = #{const ACC_SKEL_FOLD}
accSkelFold1     = #{const ACC_SKEL_FOLD1}
accSkelFoldSeg   = #{const ACC_SKEL_FOLDSEG}
accSkelFold1Seg  = #{const ACC_SKEL_FOLD1SEG}
accSkelScanl     = #{const ACC_SKEL_SCANL}
accSkelScanl1    = #{const ACC_SKEL_SCANL1}
accSkelScanlP    = #{const ACC_SKEL_SCANLP}
accSkelScanr     = #{const ACC_SKEL_SCANR}
accSkelScanr1    = #{const ACC_SKEL_SCANR1}
accSkelScanrP    = #{const ACC_SKEL_SCANRP}
accSkelPermute   = #{const ACC_SKEL_PERMUTE}
accSkelStencil   = #{const ACC_SKEL_STENCIL}
accSkelStencil2  = #{const ACC_SKEL_STENCIL2}

accCombineGeneric, accCombineAdd, accCombineMin, accCombineMax, accCombineAnd, accCombineOr, accCombineXor :: Int32
accCombineGeneric = #{const ACC_COMBINE_GENERIC}
accCombineAdd     = #{const ACC_COMBINE_ADD}
accCombineMin     = #{const ACC_COMBINE_MIN}
accCombineMax     = #{const ACC_COMBINE_MAX}
accCombineAnd     = #{const ACC_COMBINE_AND}
accCombineOr      = #{const ACC_COMBINE_OR}
accCombineXor     = #{const ACC_COMBINE_XOR}

accBoundaryClamp, accBoundaryMirror, accBoundaryWrap, accBoundaryConstant :: Int32
accBoundaryClamp    = #{const ACC_BOUNDARY_CLAMP}
accBoundaryMirror   = #{const ACC_BOUNDARY_MIRROR}
accBoundaryWrap     = #{const ACC_BOUNDARY_WRAP}
accBoundaryConstant = #{const ACC_BOUNDARY_CONSTANT}

accFlagFoldRight, accFlagFastMath, accFlagGuarded, accFlagTiled :: Word32
accFlagFoldRight = #{const ACC_FLAG_FOLD_RIGHT}
accFlagFastMath  = #{const ACC_FLAG_FAST_MATH}
accFlagGuarded   = #{const ACC_FLAG_GUARDED}
accFlagTiled     = #{const ACC_FLAG_TILED}

-- | ACC_FLAG_TILE_DIM(d): with 'accFlagTiled', which dimension of the result (counted from the innermost) the tiles
-- pair with the innermost one
accFlagTileDim :: Int -> Word32
accFlagTileDim d = fromIntegral d `shiftL` 8

data HIPException = HIPException Status String
  deriving (Typeable)

instance Show HIPException where
  show (HIPException s msg) = "libacchip (status " ++ show s ++ "): " ++ msg

instance Exception HIPException

-- | run an entry point; any status but ACC_OK is thrown with the library's message for it
check :: IO Status -> IO ()
check io = do
  s <- io
  when (s /= accOK) $ do
    msg <- peekCString =<< c_lastError
    throwIO (HIPException s msg)

-- | as `check`, for allocation: out of device memory is an ordinary result, so that the caller may evict and
-- try again (Array/Remote.hs:63-67)
checkAlloc :: IO Status -> IO Bool
checkAlloc io = do
  s <- io
  if s == accErrOOM then return False else check (return s) >> return True

-- ---------------------------------------------------------------------------------------------------------
-- structures

-- | a device-resident array as the kernels see it: extents outermost first, one pointer per tuple component
-- (what Execute.hs:823-873 `Marshalable` flattens into kernel arguments)
data AccArray = AccArray
  { arrayShape :: [Int64]            -- rank = length, at most ACC_MAX_RANK
  , arrayPtrs  :: [DevPtr]           -- component 0 first, at most ACC_MAX_COMP
  }

instance Storable AccArray where
  sizeOf    _ = #{size acc_array}
  alignment _ = #{alignment acc_array}
  peek p = do
    rank  <- #{peek acc_array, rank}  p :: IO Int32
    ncomp <- #{peek acc_array, ncomp} p :: IO Int32
    sh    <- peekArray (fromIntegral rank)  (#{ptr acc_array, shape} p)
    ps    <- peekArray (fromIntegral ncomp) (#{ptr acc_array, ptr}   p)
    return (AccArray sh ps)
  poke p (AccArray sh ps) = do
    #{poke acc_array, rank}  p (fromIntegral (length sh) :: Int32)
    #{poke acc_array, ncomp} p (fromIntegral (length ps) :: Int32)
    pokeArray (#{ptr acc_array, shape} p) sh
    pokeArray (#{ptr acc_array, ptr}   p) ps

-- | signature of one free array variable of the scalar fragments (Gamma, AST.hs:87-112)
data EnvSig = EnvSig
  { envRank  :: Int32
  , envTypes :: [CString]            -- C type of each component, component 0 first
  }

instance Storable EnvSig where
  sizeOf    _ = #{size acc_env_sig}
  alignment _ = #{alignment acc_env_sig}
  peek p = do
    rank  <- #{peek acc_env_sig, rank}  p
    ncomp <- #{peek acc_env_sig, ncomp} p :: IO Int32
    ts    <- peekArray (fromIntegral ncomp) (#{ptr acc_env_sig, type} p)
    return (EnvSig rank ts)
  poke p (EnvSig rank ts) = do
    #{poke acc_env_sig, rank}  p rank
    #{poke acc_env_sig, ncomp} p (fromIntegral (length ts) :: Int32)
    pokeArray (#{ptr acc_env_sig, type} p) ts

-- | acc_skel_desc is filled field by field into zeroed memory (every field left out is NULL / 0, which the
-- library reads as "not given"): see `withSkelDesc`
data SkelDesc
data SkelInfo
data DeviceProps
data CacheStats
data MemTableStats

-- | What the code generator hands over for one array operation (CodeGen.hs:91-136 builds a CUTranslSkel; this
-- is the same information as text fragments)
data Skeleton = Skeleton
  { skelKind        :: Int32                 -- ACC_SKEL_*
  , skelFlags       :: Word32
  , skelEnv         :: [(Int32, [String])]   -- per free array: rank, component types
  , skelEltType     :: String
  , skelOutRank     :: Int32
  , skelPreamble    :: Maybe String
  , skelGet         :: Maybe String
  , skelCombine     :: Maybe String
  , skelSeed        :: Maybe String
  , skelPermutation :: Maybe String
  , skelCombineHint :: Int32
  , skelSegType     :: Maybe String
  , skelStencilFn   :: Maybe String          -- stencils: the function over the taps t0.. (and u0..)
  , skelSources     :: [StencilSource]       -- one for a stencil, two for a stencil2
  }

-- | one source of a stencil: its element type ("T<n-1>, ..., T0" for tuples), its boundary condition, and its taps as
-- rows of out_rank offsets, outermost dimension first (acc_skel_desc.tap_offsets)
data StencilSource = StencilSource
  { sourceType     :: String
  , sourceBoundary :: Int32                  -- ACC_BOUNDARY_*
  , sourceConstant :: Maybe String
  , sourceTaps     :: [[Int32]]
  }

-- | a description with nothing given: the fields a kind does not use stay as they are here
emptySkeleton :: Skeleton
emptySkeleton = Skeleton
  { skelKind = accSkelMap, skelFlags = 0, skelEnv = [], skelEltType = "Int32", skelOutRank = 0, skelPreamble = Nothing
  , skelGet = Nothing, skelCombine = Nothing, skelSeed = Nothing, skelPermutation = Nothing
  , skelCombineHint = accCombineGeneric, skelSegType = Nothing, skelStencilFn = Nothing, skelSources = [] }

withMaybeCString :: Maybe String -> (CString -> IO a) -> IO a
withMaybeCString Nothing  k = k nullPtr
withMaybeCString (Just s) k = withCString s k

withCStrings :: [String] -> ([CString] -> IO a) -> IO a
withCStrings []     k = k []
withCStrings (s:ss) k = withCString s $ \c -> withCStrings ss (k . (c:))

-- | marshal a `Skeleton` for acc_skel_create[_async] / acc_skel_preview
withSkelDesc :: Skeleton -> (Ptr SkelDesc -> IO a) -> IO a
withSkelDesc sk k =
  allocaBytes #{size acc_skel_desc} $ \p ->
  withEnv (skelEnv sk) $ \envs ->
  withArrayLen envs $ \n penv ->
  withCString (skelEltType sk) $ \elt ->
  withMaybeCString (skelPreamble sk) $ \pre ->
  withMaybeCString (skelGet sk) $ \get ->
  withMaybeCString (skelCombine sk) $ \comb ->
  withMaybeCString (skelSeed sk) $ \seed ->
  withMaybeCString (skelPermutation sk) $ \perm ->
  withMaybeCString (skelSegType sk) $ \seg ->
  withMaybeCString (skelStencilFn sk) $ \sfn ->
  withSource (source 0) $ \(ty1, bc1, n1, taps1) ->
  withSource (source 1) $ \(ty2, bc2, n2, taps2) -> do
    _ <- fillBytes p 0 #{size acc_skel_desc}
    #{poke acc_skel_desc, kind}         p (skelKind sk)
    #{poke acc_skel_desc, flags}        p (skelFlags sk)
    #{poke acc_skel_desc, n_env}        p (fromIntegral n :: Int32)
    #{poke acc_skel_desc, env}          p penv
    #{poke acc_skel_desc, elt_type}     p elt
    #{poke acc_skel_desc, out_rank}     p (skelOutRank sk)
    #{poke acc_skel_desc, preamble}     p pre
    #{poke acc_skel_desc, get}          p get
    #{poke acc_skel_desc, combine}      p comb
    #{poke acc_skel_desc, seed}         p seed
    #{poke acc_skel_desc, permutation}  p perm
    #{poke acc_skel_desc, combine_hint} p (skelCombineHint sk)
    #{poke acc_skel_desc, seg_type}     p seg
    #{poke acc_skel_desc, stencil_fn}          p sfn
    #{poke acc_skel_desc, stencil_in_type}     p ty1
    #{poke acc_skel_desc, boundary}            p (maybe accBoundaryClamp sourceBoundary (source 0))
    #{poke acc_skel_desc, boundary_constant}   p bc1
    #{poke acc_skel_desc, n_taps}              p (n1 :: Int32)
    #{poke acc_skel_desc, tap_offsets}         p taps1
    #{poke acc_skel_desc, stencil_in2_type}    p ty2
    #{poke acc_skel_desc, boundary2}           p (maybe accBoundaryClamp sourceBoundary (source 1))
    #{poke acc_skel_desc, boundary2_constant}  p bc2
    #{poke acc_skel_desc, n_taps2}             p (n2 :: Int32)
    #{poke acc_skel_desc, tap2_offsets}        p taps2
    k p
  where
    source i = case drop i (skelSources sk) of { (x : _) -> Just x; [] -> Nothing }
    -- element type, constant, number of taps, and the taps' offsets row after row
    withSource :: Maybe StencilSource -> ((CString, CString, Int32, Ptr Int32) -> IO b) -> IO b
    withSource Nothing   kk = kk (nullPtr, nullPtr, 0, nullPtr)
    withSource (Just sc) kk =
      withCString (sourceType sc) $ \ty ->
      withMaybeCString (sourceConstant sc) $ \bc ->
      withArray (concat (sourceTaps sc)) $ \taps ->
        kk (ty, bc, fromIntegral (length (sourceTaps sc)), taps)
    withEnv []            kk = kk []
    withEnv ((r, ts):es)  kk = withCStrings ts $ \cs -> withEnv es (kk . (EnvSig r cs :))

-- | build (or fetch from the kernel cache) the kernels of one array operation: the role of build1 / compile /
-- link (Compile.hs:444-566).  The handle replaces the AccKernel record (AST.hs:51-59).
createSkeleton :: Context -> Skeleton -> IO Skel
createSkeleton ctx sk =
  withSkelDesc sk $ \pdesc ->
  alloca $ \pout -> do
    check (c_skelCreate ctx pdesc pout)
    peek pout

-- | the same with the compilation left to the library's pool of workers: the description is checked and the source
-- generated before this returns, and whatever first needs the kernel (acc_exec_*, acc_skel_wait) waits for it --
-- build1 forks its compilation and the executing thread blocks where the kernel is first used (Compile.hs:444-459,
-- 484-538), so a program's kernels compile side by side
createSkeletonAsync :: Context -> Skeleton -> IO Skel
createSkeletonAsync ctx sk =
  withSkelDesc sk $ \pdesc ->
  alloca $ \pout -> do
    check (c_skelCreateAsync ctx pdesc pout)
    peek pout

-- | device memory, or Nothing when the device is full (Array/Remote.hs:63-67 `mallocRemote`)
mallocDevice :: Context -> Int -> IO (Maybe DevPtr)
mallocDevice ctx bytes =
  alloca $ \pout -> do
    ok <- checkAlloc (c_malloc ctx (fromIntegral bytes) pout)
    if ok then Just `fmap` peek pout else return Nothing

-- | out[i] = f (in[i]) and the other members of the map family (Execute.hs:264-268 `executeOp`)
execMap :: Skel -> [AccArray] -> AccArray -> Stream -> IO ()
execMap sk env out stream =
  withArray env $ \penv ->
  with out $ \pout ->
    check (c_execMap sk penv pout stream)

-- | the six scans (Execute.hs:328-392): `total` is Nothing except for scanl' / scanr'
execScan :: Skel -> [AccArray] -> Int64 -> AccArray -> Maybe AccArray -> Stream -> IO ()
execScan sk env n out total stream =
  withArray env $ \penv ->
  with out $ \pout ->
  maybe ($ nullPtr) with total $ \ptot ->
    check (c_execScan sk penv n pout ptot stream)

-- | have the library's compilations wound up when the process exits (acc_compile_drain: exit() tears down the
-- compiler's static data, and a worker must not be inside the compiler then).  The C function itself is
-- registered with the C library's atexit: a Haskell callback could not run there, the run-time system being gone
-- by then.  Registered after the library (and with it the compiler) was loaded, it runs before their own
-- destructors.  (Its int result is ignored by the caller, which is harmless under the C ABIs in question.)
foreign import ccall unsafe "stdlib.h atexit" registerAtExit  :: FunPtr (IO Status) -> IO CInt
foreign import ccall        "&acc_compile_drain" compileDrainPtr :: FunPtr (IO Status)

drainCompilationsAtExit :: IO ()
drainCompilationsAtExit = void (registerAtExit compileDrainPtr)

-- ---------------------------------------------------------------------------------------------------------
-- the entry points, in the header's order

-- errors and version
foreign import ccall unsafe "acc_last_error" c_lastError :: IO CString
foreign import ccall unsafe "acc_version"    c_version   :: IO CString

-- State.hs:127-132, Analysis/Device.hs:31-41: initialise, count, props
foreign import ccall safe   "acc_init"             c_init           :: IO Status
foreign import ccall safe   "acc_device_count"     c_deviceCount    :: Ptr CInt -> IO Status
foreign import ccall safe   "acc_device_get_props" c_deviceGetProps :: CInt -> Ptr DeviceProps -> IO Status

-- Context.hs:55-111: create / destroy; CUDA.sync
foreign import ccall safe   "acc_context_create"  c_contextCreate  :: CInt -> Ptr Context -> IO Status
foreign import ccall safe   "acc_context_destroy" c_contextDestroy :: Context -> IO Status
foreign import ccall safe   "acc_context_device"  c_contextDevice  :: Context -> Ptr CInt -> IO Status
foreign import ccall safe   "acc_context_sync"    c_contextSync    :: Context -> IO Status
-- scratch memory of the skeleton drivers: give back what is not in use / how much is held
foreign import ccall safe   "acc_context_trim"          c_contextTrim         :: Context -> Ptr CSize -> IO Status
foreign import ccall unsafe "acc_context_scratch_bytes" c_contextScratchBytes :: Context -> Ptr CSize -> IO Status
-- tuning knobs: parsed once into a table, per process and per context (Debug.hs:100-140 reads its flags once, too)
foreign import ccall safe   "acc_tuning_set"         c_tuningSet        :: CString -> IO Status
foreign import ccall unsafe "acc_tuning_text"        c_tuningText       :: IO CString
foreign import ccall safe   "acc_context_set_tuning" c_contextSetTuning :: Context -> CString -> IO Status
-- tests of the failure path only
foreign import ccall safe   "acc_context_debug_poke_lock" c_contextDebugPokeLock :: Context -> CSize -> Word32 -> IO Status

-- Array/Remote.hs:63-79,191: mallocArray / free / getMemInfo.  ACC_ERR_OOM is the recoverable status
foreign import ccall safe   "acc_malloc"     c_malloc    :: Context -> CSize -> Ptr DevPtr -> IO Status
foreign import ccall safe   "acc_free"       c_free      :: Context -> DevPtr -> IO Status
foreign import ccall safe   "acc_mem_info"   c_memInfo   :: Context -> Ptr CSize -> Ptr CSize -> IO Status
foreign import ccall safe   "acc_host_alloc" c_hostAlloc :: Context -> CSize -> Ptr (Ptr ()) -> IO Status
foreign import ccall safe   "acc_host_free"  c_hostFree  :: Context -> Ptr () -> IO Status

-- Array/Prim.hs:189-391, Execute.hs:405: poke / peek / copy [Async], memsetAsync
foreign import ccall safe   "acc_memcpy_h2d"       c_memcpyH2d      :: Context -> DevPtr -> Ptr () -> CSize -> IO Status
foreign import ccall safe   "acc_memcpy_d2h"       c_memcpyD2h      :: Context -> Ptr () -> DevPtr -> CSize -> IO Status
foreign import ccall safe   "acc_memcpy_d2d"       c_memcpyD2d      :: Context -> DevPtr -> DevPtr -> CSize -> IO Status
foreign import ccall safe   "acc_memcpy_h2d_async" c_memcpyH2dAsync :: Context -> DevPtr -> Ptr () -> CSize -> Stream -> IO Status
foreign import ccall safe   "acc_memcpy_d2h_async" c_memcpyD2hAsync :: Context -> Ptr () -> DevPtr -> CSize -> Stream -> IO Status
foreign import ccall safe   "acc_memcpy_d2d_async" c_memcpyD2dAsync :: Context -> DevPtr -> DevPtr -> CSize -> Stream -> IO Status
foreign import ccall safe   "acc_memset32_async"   c_memset32Async  :: Context -> DevPtr -> Word32 -> CSize -> Stream -> IO Status

-- Execute/Stream.hs:102,134; Execute/Event.hs:70-127; Debug.hs:48-67
foreign import ccall safe   "acc_stream_create"     c_streamCreate    :: Context -> Ptr Stream -> IO Status
foreign import ccall safe   "acc_stream_destroy"    c_streamDestroy   :: Context -> Stream -> IO Status
foreign import ccall safe   "acc_stream_sync"       c_streamSync      :: Context -> Stream -> IO Status
foreign import ccall safe   "acc_stream_wait_event" c_streamWaitEvent :: Context -> Stream -> Event -> IO Status
foreign import ccall safe   "acc_event_create"      c_eventCreate     :: Context -> CInt -> Ptr Event -> IO Status
foreign import ccall safe   "acc_event_destroy"     c_eventDestroy    :: Context -> Event -> IO Status
foreign import ccall safe   "acc_event_record"      c_eventRecord     :: Context -> Event -> Stream -> IO Status
foreign import ccall safe   "acc_event_sync"        c_eventSync       :: Context -> Event -> IO Status
foreign import ccall safe   "acc_event_query"       c_eventQuery      :: Context -> Event -> Ptr CInt -> IO Status
foreign import ccall safe   "acc_event_elapsed_ms"  c_eventElapsedMs  :: Context -> Event -> Event -> Ptr CFloat -> IO Status

-- Compile.hs:543-594, Persistent.hs: run-time compilation through the kernel cache (blocks while the compiler runs)
foreign import ccall safe   "acc_compile"         c_compile       :: Context -> CString -> CString -> Ptr CString -> CInt -> Ptr (Ptr ()) -> Ptr CSize -> IO Status
foreign import ccall unsafe "acc_compile_log"     c_compileLog    :: IO CString
foreign import ccall safe   "acc_cache_set_dir"   c_cacheSetDir   :: CString -> IO Status
foreign import ccall unsafe "acc_cache_dir"       c_cacheDir      :: IO CString
foreign import ccall safe   "acc_cache_get_stats" c_cacheGetStats :: Ptr CacheStats -> IO Status
foreign import ccall safe   "acc_cache_clear"     c_cacheClear    :: CInt -> IO Status

-- Compile.hs:453-465,505,534; Analysis/Launch.hs:42-102; Execute.hs:975-978: raw modules, occupancy, launch
foreign import ccall safe   "acc_module_load"         c_moduleLoad        :: Context -> Ptr () -> CSize -> Ptr Module -> IO Status
foreign import ccall safe   "acc_module_unload"       c_moduleUnload      :: Context -> Module -> IO Status
foreign import ccall safe   "acc_module_get_function" c_moduleGetFunction :: Context -> Module -> CString -> Ptr Function -> IO Status
foreign import ccall safe   "acc_function_attr"       c_functionAttr      :: Context -> Function -> CInt -> Ptr CInt -> IO Status
foreign import ccall safe   "acc_occupancy"           c_occupancy         :: Context -> Function -> CInt -> CSize -> Ptr CInt -> IO Status
foreign import ccall safe   "acc_launch"              c_launch            :: Context -> Function -> Word32 -> Word32 -> Word32 -> Stream -> Ptr (Ptr ()) -> IO Status
foreign import ccall unsafe "acc_launch_grid"         c_launchGrid        :: Int64 -> Int64 -> Int64 -> Int64 -> Int64

-- Compile.hs:444-566 + CodeGen/*: one skeleton instance per array operation
foreign import ccall safe   "acc_skel_create"       c_skelCreate      :: Context -> Ptr SkelDesc -> Ptr Skel -> IO Status
foreign import ccall safe   "acc_skel_destroy"      c_skelDestroy     :: Skel -> IO Status
-- compilation on the library's worker pool; the first use of the kernel waits for it (Compile.hs:444-459,620-660)
foreign import ccall safe   "acc_skel_create_async" c_skelCreateAsync :: Context -> Ptr SkelDesc -> Ptr Skel -> IO Status
foreign import ccall safe   "acc_skel_wait"         c_skelWait        :: Skel -> IO Status
foreign import ccall safe   "acc_skel_prefetch"     c_skelPrefetch    :: Skel -> CInt -> IO Status
foreign import ccall unsafe "acc_skel_poll"         c_skelPoll        :: Skel -> Ptr CInt -> IO Status
foreign import ccall unsafe "acc_compile_threads"   c_compileThreads  :: IO CInt
foreign import ccall safe   "acc_compile_drain"     c_compileDrain    :: IO Status
foreign import ccall safe   "acc_skel_source"       c_skelSource      :: Skel -> CInt -> Ptr CString -> IO Status
foreign import ccall safe   "acc_skel_preview"      c_skelPreview     :: Ptr SkelDesc -> CInt -> Ptr CString -> Ptr CString -> IO Status
foreign import ccall safe   "acc_skel_compile_only" c_skelCompileOnly :: CString -> Ptr SkelDesc -> Ptr CSize -> IO Status
foreign import ccall safe   "acc_skel_get_info"     c_skelGetInfo     :: Skel -> Ptr SkelInfo -> IO Status

-- Execute.hs:264-450: the skeleton drivers; everything is enqueued on the stream
foreign import ccall safe   "acc_exec_map"             c_execMap            :: Skel -> Ptr AccArray -> Ptr AccArray -> Stream -> IO Status
foreign import ccall safe   "acc_exec_fold"            c_execFold           :: Skel -> Ptr AccArray -> Int32 -> Ptr Int64 -> Ptr AccArray -> Stream -> IO Status
foreign import ccall safe   "acc_exec_foldseg"         c_execFoldseg        :: Skel -> Ptr AccArray -> Int64 -> Ptr AccArray -> Ptr AccArray -> Stream -> IO Status
foreign import ccall safe   "acc_exec_foldseg_nd"      c_execFoldsegNd      :: Skel -> Ptr AccArray -> Int32 -> Ptr Int64 -> Ptr AccArray -> Ptr AccArray -> Stream -> IO Status
foreign import ccall safe   "acc_exec_scan"            c_execScan           :: Skel -> Ptr AccArray -> Int64 -> Ptr AccArray -> Ptr AccArray -> Stream -> IO Status
foreign import ccall safe   "acc_exec_scan_noalloc"    c_execScanNoalloc    :: Skel -> Ptr AccArray -> Int64 -> Ptr AccArray -> Ptr AccArray -> Stream -> IO Status
foreign import ccall safe   "acc_exec_permute"         c_execPermute        :: Skel -> Ptr AccArray -> Int64 -> Ptr AccArray -> Ptr AccArray -> Stream -> IO Status
foreign import ccall safe   "acc_exec_stencil"         c_execStencil        :: Skel -> Ptr AccArray -> Ptr AccArray -> Ptr AccArray -> Stream -> IO Status
foreign import ccall safe   "acc_exec_stencil2"        c_execStencil2       :: Skel -> Ptr AccArray -> Ptr AccArray -> Ptr AccArray -> Ptr AccArray -> Stream -> IO Status
foreign import ccall safe   "acc_exec_stencil_iterate" c_execStencilIterate :: Skel -> Ptr AccArray -> Ptr AccArray -> Ptr AccArray -> Int32 -> Stream -> Ptr Int32 -> IO Status

-- Execute.hs:236-244: awhile with its iterations enqueued ahead; the guard's words say how many were taken
foreign import ccall safe   "acc_guard_create"     c_guardCreate    :: Context -> Ptr Guard -> IO Status
foreign import ccall safe   "acc_guard_destroy"    c_guardDestroy   :: Guard -> IO Status
foreign import ccall safe   "acc_guard_reset"      c_guardReset     :: Guard -> Stream -> IO Status
foreign import ccall safe   "acc_guard_latch"      c_guardLatch     :: Guard -> Ptr AccArray -> Stream -> IO Status
foreign import ccall safe   "acc_guard_read"       c_guardRead      :: Guard -> Stream -> Ptr Int32 -> Ptr Int64 -> IO Status
foreign import ccall safe   "acc_stream_set_guard" c_streamSetGuard :: Context -> Stream -> Guard -> IO Status

-- Debug.hs:41-76: time on the device of the launches a thread makes
foreign import ccall safe   "acc_trace_start" c_traceStart :: Context -> IO Status
foreign import ccall safe   "acc_trace_stop"  c_traceStop  :: Context -> Ptr Int32 -> Ptr CDouble -> IO Status

-- Array/Remote.hs, Array/Table.hs, Array/Prim.hs:177-192: the memory table
foreign import ccall safe   "acc_memtable_create"           c_memtableCreate          :: Context -> Word64 -> Ptr MemTable -> IO Status
foreign import ccall safe   "acc_memtable_destroy"          c_memtableDestroy         :: MemTable -> IO Status
foreign import ccall safe   "acc_memtable_malloc"           c_memtableMalloc          :: MemTable -> Word64 -> Ptr () -> Word64 -> CInt -> Ptr CInt -> IO Status
foreign import ccall safe   "acc_memtable_acquire"          c_memtableAcquire         :: MemTable -> Word64 -> Stream -> Ptr DevPtr -> IO Status
foreign import ccall safe   "acc_memtable_release"          c_memtableRelease         :: MemTable -> Word64 -> Stream -> IO Status
foreign import ccall safe   "acc_memtable_free"             c_memtableFree            :: MemTable -> Word64 -> IO Status
foreign import ccall safe   "acc_memtable_insert_unmanaged" c_memtableInsertUnmanaged :: MemTable -> Word64 -> DevPtr -> Word64 -> IO Status
foreign import ccall safe   "acc_memtable_reclaim"          c_memtableReclaim         :: MemTable -> IO Status
foreign import ccall safe   "acc_memtable_get_stats"        c_memtableGetStats        :: MemTable -> Ptr MemTableStats -> IO Status
