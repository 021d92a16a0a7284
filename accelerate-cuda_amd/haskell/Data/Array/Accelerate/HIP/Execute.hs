{-# LANGUAGE GADTs, ScopedTypeVariables, BangPatterns, RankNTypes #-}
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
import Data.Array.Accelerate.Array.Sugar                       ( Array(..), Arrays, Shape, Elt, Scalar, Vector, Segments, Z(..), (:.)(..), Any(..) )
import Data.Array.Accelerate.Array.Representation              ( SliceIndex(..) )
import Data.Array.Accelerate.Interpreter                       ( evalPrim, evalPrimConst, evalPrj )
import qualified Data.Array.Accelerate.Array.Sugar             as Sugar

import Data.Array.Accelerate.HIP.CodeGen                       ( ArrayVar(..) )
import Data.Array.Accelerate.HIP.Compile
import Data.Array.Accelerate.HIP.FFI
import Data.Array.Accelerate.HIP.State
import Data.Array.Accelerate.HIP.Array                          -- arrays and their device copies, over acc_memtable_*

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
  useArrays a
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
    Use arrs              -> do { let a = Sugar.toArr arrs; useArrays a; return a }
    Unit e                -> unitArray =<< travE e
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
    travE e = evalHostExp e Empty aenv stream

    -- the extent of an operand: of a manifest one its array's, of a fused one its extent expression
    extent :: Shape sh => ExecOpenAcc aenv (Array sh e) -> HIP sh
    extent (ExecFused sh) = travE sh
    extent acc            = Sugar.shape <$> travA acc

    -- the node's free arrays as the kernel wants them, in the order the fragments numbered them
    environment :: ([AccArray] -> HIP r) -> HIP r
    environment = withArrays stream [ SomeArray (aprj ix aenv) | ArrayVar ix <- gamma ]

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


-- Scalar expressions on the host
-- -------------------------------

-- the values of the bound scalar variables
data Val env where
  Empty :: Val ()
  Push  :: Val env -> t -> Val (env, t)

prj :: Idx env t -> Val env -> t
prj ZeroIdx      (Push _   v) = v
prj (SuccIdx ix) (Push val _) = prj ix val

-- | extents, conditions, the seeds of units: scalar code that did not go into a kernel is interpreted, with the
-- primitives of the reference interpreter; an array it names is computed first and the one element it wants read
-- back from the device (Execute.hs:706-768 `executeOpenExp`)
evalHostExp :: forall env aenv t. PreOpenExp ExecOpenAcc env aenv t -> Val env -> Aval aenv -> Stream -> HIP t
evalHostExp root env aenv stream = go root
  where
    go :: forall s. PreOpenExp ExecOpenAcc env aenv s -> HIP s
    go e = case e of
      Var ix              -> return (prj ix env)
      Let a b             -> do { x <- go a; evalHostExp b (env `Push` x) aenv stream }
      Const c             -> return (Sugar.toElt c)
      PrimConst c         -> return (evalPrimConst c)
      PrimApp f x         -> evalPrim f <$> go x
      Tuple t             -> Sugar.toTuple <$> goT t
      Prj ix x            -> evalPrj ix . Sugar.fromTuple <$> go x
      Cond p t f          -> do { c <- go p; if c then go t else go f }
      While p f x         -> while p f =<< go x
      IndexAny            -> return Any
      IndexNil            -> return Z
      IndexCons sh i      -> (:.) <$> go sh <*> go i
      IndexHead sh        -> (\(_ :. i) -> i) <$> go sh
      IndexTail sh        -> (\(t :. _) -> t) <$> go sh
      IndexSlice ix s sh  -> restrictTo ix <$> go s <*> go sh
      IndexFull ix s sl   -> extendTo ix <$> go s <*> go sl
      ToIndex sh ix       -> Sugar.toIndex <$> go sh <*> go ix
      FromIndex sh i      -> Sugar.fromIndex <$> go sh <*> go i
      Intersect a b       -> Sugar.intersect <$> go a <*> go b
      Union a b           -> Sugar.union <$> go a <*> go b
      ShapeSize sh        -> Sugar.size <$> go sh
      Shape a             -> extentOf a
      Index a ix          -> do { arr <- goA a; i <- go ix; indexArray stream arr (Sugar.toIndex (Sugar.shape arr) i) }
      LinearIndex a i     -> do { arr <- goA a; indexArray stream arr =<< go i }
      Foreign{}           -> error "Data.Array.Accelerate.HIP: foreign scalar functions are not supported by this backend"

    goT :: forall s. Tuple (PreOpenExp ExecOpenAcc env aenv) s -> HIP s
    goT NilTup        = return ()
    goT (SnocTup t x) = (,) <$> goT t <*> go x

    goA :: forall a. ExecOpenAcc aenv a -> HIP a
    goA acc = executeOpenAcc acc aenv stream

    -- the extent of a fused array is an expression of its own; nothing is computed for it
    extentOf :: forall sh e. Shape sh => ExecOpenAcc aenv (Array sh e) -> HIP sh
    extentOf (ExecFused sh) = evalHostExp sh Empty aenv stream
    extentOf acc            = Sugar.shape <$> goA acc

    apply1 :: forall a b. PreOpenFun ExecOpenAcc env aenv (a -> b) -> a -> HIP b
    apply1 (Lam (Body b)) x = evalHostExp b (env `Push` x) aenv stream
    apply1 _              _ = error "expected a unary function"

    while :: forall a. PreOpenFun ExecOpenAcc env aenv (a -> Bool) -> PreOpenFun ExecOpenAcc env aenv (a -> a) -> a -> HIP a
    while p f x = do { ok <- apply1 p x; if ok then while p f =<< apply1 f x else return x }

    -- a slice index cuts dimensions out of a shape, or puts them back (Execute.hs:744-764)
    restrictTo :: (Elt slix, Elt sh, Elt sl) => SliceIndex (Sugar.EltRepr slix) (Sugar.EltRepr sl) co (Sugar.EltRepr sh) -> slix -> sh -> sl
    restrictTo ix slix sh = Sugar.toElt (cut ix (Sugar.fromElt slix) (Sugar.fromElt sh))
      where
        cut :: SliceIndex a b c d -> a -> d -> b
        cut SliceNil        ()       ()       = ()
        cut (SliceAll r)    (sx, ()) (sl, sz) = (cut r sx sl, sz)
        cut (SliceFixed r)  (sx, _)  (sl, _)  = cut r sx sl

    extendTo :: (Elt slix, Elt sh, Elt sl) => SliceIndex (Sugar.EltRepr slix) (Sugar.EltRepr sl) co (Sugar.EltRepr sh) -> slix -> sl -> sh
    extendTo ix slix sl = Sugar.toElt (grow ix (Sugar.fromElt slix) (Sugar.fromElt sl))
      where
        grow :: SliceIndex a b c d -> a -> b -> d
        grow SliceNil        ()       ()       = ()
        grow (SliceAll r)    (sx, ()) (sh, sz) = (grow r sx sh, sz)
        grow (SliceFixed r)  (sx, sz) sh       = (grow r sx sh, sz)
