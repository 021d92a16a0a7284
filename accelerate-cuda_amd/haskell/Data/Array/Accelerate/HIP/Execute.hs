{-# LANGUAGE GADTs, ScopedTypeVariables, BangPatterns #-}
-- |
-- Module      : Data.Array.Accelerate.HIP.Execute
--
-- Second traversal: the compiled program is walked bottom-up, every node with a kernel
-- allocates its result in the memory table and hands the node's free arrays to the matching
-- driver of libacchip, everything enqueued on the stream of the computation.  The role of
-- Execute.hs:164-450.  What that module does besides -- launch configuration, argument
-- marshalling (`Marshalable`, Execute.hs:823-909), temporaries of folds, scans and permute,
-- the two- and three-kernel protocols -- is inside `acc_exec_*`.
--
-- UNCOMPILED: no GHC in the image this library is built and tested in.
--
module Data.Array.Accelerate.HIP.Execute (

  executeAcc, executeAfun1,

) where

import Data.Array.Accelerate.AST
import Data.Array.Accelerate.Array.Sugar                       ( Array(..), Arrays, Shape, Elt, Scalar, Vector, Segments, Z(..), (:.)(..) )
import qualified Data.Array.Accelerate.Array.Sugar             as Sugar

import Data.Array.Accelerate.HIP.Compile
import Data.Array.Accelerate.HIP.FFI
import Data.Array.Accelerate.HIP.State
import Data.Array.Accelerate.HIP.Array                          -- allocateArray / useArray / peekScalar over acc_memtable_*

import Control.Monad
import Control.Monad.Trans                                      ( liftIO )
import Foreign
import Data.Int


-- the values of the free array variables
data Aval aenv where
  Aempty :: Aval ()
  Apush  :: Aval aenv -> arrs -> Aval (aenv, arrs)

aprj :: Idx aenv a -> Aval aenv -> a
aprj ZeroIdx      (Apush _ a)    = a
aprj (SuccIdx ix) (Apush aenv _) = aprj ix aenv


-- | CUDA.hs:209-216 `run` below `compileAcc`: evaluate on a stream of the reservoir, wait, hand the arrays over
executeAcc :: Arrays a => ExecAcc a -> HIP a
executeAcc acc = withStream $ \stream -> do
  r   <- executeOpenAcc acc Aempty stream
  ctx <- hipContext
  liftIO $ check (c_streamSync ctx stream)               -- ACC_ERR_STUCK surfaces here (include/acc_hip.h)
  return r

-- | CUDA.hs:318-333 `run1`: the kernels were built once, by compileAfun
executeAfun1 :: (Arrays a, Arrays b) => ExecAfun (a -> b) -> a -> HIP b
executeAfun1 (Alam (Abody f)) a = withStream $ \stream -> do
  useArrays a stream
  r   <- executeOpenAcc f (Aempty `Apush` a) stream
  ctx <- hipContext
  liftIO $ check (c_streamSync ctx stream)
  return r
executeAfun1 _ _ = error "executeAfun1: expected a unary function"


executeOpenAcc :: forall aenv a. ExecOpenAcc aenv a -> Aval aenv -> Stream -> HIP a
executeOpenAcc (ExecFused _) _ _ = error "a delayed array has no value of its own: it was fused into its consumer"
executeOpenAcc (ExecAcc kernel pacc) aenv stream =
  case pacc of
    -- array-level forms without a kernel (Execute.hs:187-219)
    Avar ix               -> return (aprj ix aenv)
    Alet bnd body         -> do { a <- travA bnd; executeOpenAcc body (aenv `Apush` a) stream }
    Apply (Alam (Abody f)) a -> do { a' <- travA a; executeOpenAcc f (Aempty `Apush` a') stream }
    Apply _ _             -> error "Apply: expected a unary function"
    Atuple tup            -> Sugar.toAtuple <$> travT tup
    Aprj ix tup           -> evalPrj ix . Sugar.fromAtuple <$> travA tup
    Acond p t e           -> do { c <- travE p; if c then travA t else travA e }
    Awhile p f a          -> awhile p f =<< travA a
    Use arrs              -> do { let a = Sugar.toArr arrs; useArrays a stream; return a }
    Unit e                -> unitArray stream =<< travE e
    Reshape sh a          -> reshapeArray <$> travE sh <*> travA a       -- same device storage, new extents

    -- one driver call each (Execute.hs:264-450)
    Generate sh _         -> mapFamily =<< travE sh
    Map _ a               -> mapFamily =<< extent a
    ZipWith _ a b         -> mapFamily =<< (Sugar.intersect <$> extent a <*> extent b)
    Backpermute sh _ _    -> mapFamily =<< travE sh
    Transform sh _ _ _    -> mapFamily =<< travE sh

    Fold  _ _ a           -> foldOp  =<< extent a
    Fold1 _   a           -> foldOp  =<< extent a
    FoldSeg  _ _ a s      -> join (foldSegOp <$> extent a <*> travA s)
    Fold1Seg _   a s      -> join (foldSegOp <$> extent a <*> travA s)

    Scanl  _ _ a          -> scanOp True  =<< extent a
    Scanr  _ _ a          -> scanOp True  =<< extent a
    Scanl1 _   a          -> scanOp False =<< extent a
    Scanr1 _   a          -> scanOp False =<< extent a
    Scanl' _ _ a          -> scan'Op =<< extent a
    Scanr' _ _ a          -> scan'Op =<< extent a

    Permute _ d _ a       -> join (permuteOp <$> extent a <*> travA d)
    Stencil _ _ a         -> stencilOp =<< travA a
    Stencil2 _ _ a _ b    -> join (stencil2Op <$> travA a <*> travA b)

    Replicate{}           -> error "Replicate survives fusion only as a Backpermute"
    Slice{}               -> error "Slice survives fusion only as a Backpermute"
    Aforeign{}            -> error "Aforeign is not supported by this backend"
  where
    Just (Kernel skel gamma) = kernel

    travA :: ExecOpenAcc aenv b -> HIP b
    travA acc = executeOpenAcc acc aenv stream

    travT :: Atuple (ExecOpenAcc aenv) t -> HIP t
    travT NilAtup        = return ()
    travT (SnocAtup t a) = (,) <$> travT t <*> travA a

    -- scalar expressions that run on the host (extents, conditions): Execute.hs:454-560, unchanged in structure
    travE :: PreExp ExecOpenAcc aenv t -> HIP t
    travE e = evalHostExp e aenv stream

    -- the extent of an operand: of a manifest one its array's, of a fused one its extent expression
    extent :: Shape sh => ExecOpenAcc aenv (Array sh e) -> HIP sh
    extent (ExecFused sh) = travE sh
    extent acc            = Sugar.shape <$> travA acc

    -- the node's free arrays as the kernel wants them, in the order the fragments numbered them
    environment :: ([AccArray] -> HIP r) -> HIP r
    environment = withArrays stream [ deviceArrayOf (aprjInt v aenv) | v <- gamma ]

    run :: IO Status -> HIP ()
    run = liftIO . check

    -- Execute.hs:264-268 `executeOp`
    mapFamily :: (Shape sh, Elt e) => sh -> HIP (Array sh e)
    mapFamily sh = do
      out <- allocateArray sh
      environment $ \env -> withDevice stream out $ \o ->
        liftIO $ withArrayLen env $ \_ penv -> with o $ \po -> check (c_execMap skel penv po stream)
      return out

    -- Execute.hs:282-318: fold1 of an empty innermost dimension comes back as ACC_ERR_INVALID "empty array"
    foldOp :: (Shape sh, Elt e) => (sh :. Int) -> HIP (Array sh e)
    foldOp (sh :. sz) = do
      out <- allocateArray sh
      let extents = map fromIntegral (reverse (Sugar.shapeToList (sh :. sz))) :: [Int64]
      environment $ \env -> withDevice stream out $ \o ->
        liftIO $ withArrayLen env $ \_ penv -> withArrayLen extents $ \r psh -> with o $ \po ->
          check (c_execFold skel penv (fromIntegral r) psh po stream)
      return out

    -- Execute.hs:320-324: the result is  sh :. number of segments ; `offs` is the scanned segment descriptor
    foldSegOp :: (Shape sh, Elt e) => (sh :. Int) -> Segments i -> HIP (Array (sh :. Int) e)
    foldSegOp (sh :. sz) offs = do
      let Z :. n = Sugar.shape offs
      out <- allocateArray (sh :. n - 1)
      let extents = map fromIntegral (reverse (Sugar.shapeToList (sh :. sz))) :: [Int64]
      environment $ \env -> withDevice stream offs $ \s -> withDevice stream out $ \o ->
        liftIO $ withArrayLen env $ \_ penv -> withArrayLen extents $ \r psh -> with s $ \ps -> with o $ \po ->
          check (c_execFoldsegNd skel penv (fromIntegral r) psh ps po stream)
      return out

    -- Execute.hs:328-349: n + 1 results with a seed, n without; no pointer arithmetic, one launch
    scanOp :: Elt e => Bool -> (Z :. Int) -> HIP (Vector e)
    scanOp seeded (Z :. n) = do
      out <- allocateArray (Z :. (if seeded then n + 1 else n))
      environment $ \env -> withDevice stream out $ \o ->
        liftIO $ withArrayLen env $ \_ penv -> with o $ \po ->
          check (c_execScan skel penv (fromIntegral n) po nullPtr stream)
      return out

    -- Execute.hs:352-362: the body and the reduction of the whole array
    scan'Op :: Elt e => (Z :. Int) -> HIP (Vector e, Scalar e)
    scan'Op (Z :. n) = do
      out <- allocateArray (Z :. n)
      tot <- allocateArray Z
      environment $ \env -> withDevice stream out $ \o -> withDevice stream tot $ \t ->
        liftIO $ withArrayLen env $ \_ penv -> with o $ \po -> with t $ \pt ->
          check (c_execScan skel penv (fromIntegral n) po pt stream)
      return (out, tot)

    -- Execute.hs:396-408: the copy of the defaults and whatever tables or locks the combination needs are the driver's
    permuteOp :: (Shape sh, Shape sh', Elt e) => sh -> Array sh' e -> HIP (Array sh' e)
    permuteOp shIn dfs = do
      out <- allocateArray (Sugar.shape dfs)
      environment $ \env -> withDevice stream dfs $ \d -> withDevice stream out $ \o ->
        liftIO $ withArrayLen env $ \_ penv -> with d $ \pd -> with o $ \po ->
          check (c_execPermute skel penv (fromIntegral (Sugar.size shIn)) pd po stream)
      return out

    -- Execute.hs:413-425: one launch (the reference launches twice, border and interior)
    stencilOp :: (Shape sh, Elt a, Elt b) => Array sh a -> HIP (Array sh b)
    stencilOp arr = do
      out <- allocateArray (Sugar.shape arr)
      environment $ \env -> withDevice stream arr $ \i -> withDevice stream out $ \o ->
        liftIO $ withArrayLen env $ \_ penv -> with i $ \pi' -> with o $ \po ->
          check (c_execStencil skel penv pi' po stream)
      return out

    -- Execute.hs:427-450: the result covers the intersection of the sources' extents
    stencil2Op :: (Shape sh, Elt a, Elt b, Elt c) => Array sh a -> Array sh b -> HIP (Array sh c)
    stencil2Op a b = do
      out <- allocateArray (Sugar.shape a `Sugar.intersect` Sugar.shape b)
      environment $ \env -> withDevice stream a $ \ia -> withDevice stream b $ \ib -> withDevice stream out $ \o ->
        liftIO $ withArrayLen env $ \_ penv -> with ia $ \pa -> with ib $ \pb -> with o $ \po ->
          check (c_execStencil2 skel penv pa pb po stream)
      return out

    -- Execute.hs:236-244.  The reference evaluates the predicate, reads its flag back and runs the body, every
    -- iteration.  Here `ahead` iterations are enqueued at a time under a guard: the predicate's flag is latched on
    -- the device, kernels of iterations past the loop's end do nothing, and the guard is read once per batch; the
    -- loop's value is what the count-th body produced.  (Predicate and body were compiled with ACC_FLAG_GUARDED.)
    awhile :: PreOpenAfun ExecOpenAcc aenv (arrs -> Scalar Bool) -> PreOpenAfun ExecOpenAcc aenv (arrs -> arrs) -> arrs -> HIP arrs
    awhile (Alam (Abody p)) (Alam (Abody f)) a0 = do
      ctx   <- hipContext
      guard <- liftIO $ alloca $ \pg -> check (c_guardCreate ctx pg) >> peek pg
      run (c_streamSetGuard ctx stream guard)
      run (c_guardReset guard stream)
      let ahead = 8 :: Int
          batch !taken a = do
            -- the states of this batch, oldest first: states !! k is the value after k more bodies
            states <- iterateM ahead a $ \cur -> do
              flag <- executeOpenAcc p (aenv `Apush` cur) stream
              withDevice stream flag $ \fl -> liftIO $ with fl $ \pf -> check (c_guardLatch guard pf stream)
              executeOpenAcc f (aenv `Apush` cur) stream
            (alive, count) <- liftIO $ alloca $ \pa -> alloca $ \pc -> do
              check (c_guardRead guard stream pa pc)
              (,) <$> peek pa <*> peek pc
            let done = fromIntegral count - taken
                a'   = states !! done
            if alive /= 0 then batch (taken + done) a' else return a'
      r <- batch 0 a0
      run (c_streamSetGuard ctx stream nullPtr)
      run (c_guardDestroy guard)
      return r
    awhile _ _ _ = error "awhile: expected unary functions"

    iterateM :: Int -> s -> (s -> HIP s) -> HIP [s]
    iterateM 0 s _    = return [s]
    iterateM k s step = do { s' <- step s; (s :) <$> iterateM (k - 1) s' step }


-- Supplied by Data.Array.Accelerate.HIP.Array (brackets around the memory table of the header, acc_memtable_*) and by the
-- host-side expression evaluator the reference already has (Execute.hs:454-560); named here so that the traversal
-- above reads as a whole.
aprjInt       :: Int -> Aval aenv -> SomeArrays
evalPrj       :: TupleIdx t a -> t -> a
evalHostExp   :: PreExp ExecOpenAcc aenv t -> Aval aenv -> Stream -> HIP t
useArrays     :: Arrays a => a -> Stream -> HIP ()
unitArray     :: Elt e => Stream -> e -> HIP (Scalar e)
reshapeArray  :: (Shape sh, Shape sh') => sh -> Array sh' e -> Array sh e
deviceArrayOf :: SomeArrays -> SomeDeviceArray
withArrays    :: Stream -> [SomeDeviceArray] -> ([AccArray] -> HIP r) -> HIP r
withDevice    :: Stream -> Array sh e -> (AccArray -> HIP r) -> HIP r
aprjInt       = undefined
evalPrj       = undefined
evalHostExp   = undefined
useArrays     = undefined
unitArray     = undefined
reshapeArray  = undefined
deviceArrayOf = undefined
withArrays    = undefined
withDevice    = undefined
data SomeArrays
data SomeDeviceArray
