{-# LANGUAGE GADTs, ScopedTypeVariables, RecordWildCards #-}
-- |
-- Module      : Data.Array.Accelerate.HIP.Compile
--
-- First traversal of a delayed array program: every node that needs a kernel gets its
-- skeleton instance -- fragments from CodeGen, `acc_skel_create` through the library's kernel
-- cache -- and the tree is rebuilt with the handles in place.  The role of Compile.hs:110-235
-- (`compileOpenAcc`); what that module does besides (temporary files, the nvcc subprocess,
-- the persistent cache, occupancy, Compile.hs:444-594 and Persistent.hs) lives inside
-- `acc_skel_create`.
--
-- UNCOMPILED: no GHC in the image this library is built and tested in.
--
module Data.Array.Accelerate.HIP.Compile (

  ExecOpenAcc(..), ExecAcc, ExecAfun, ExecOpenAfun, Kernel(..),
  compileAcc, compileAfun,

) where

import Data.Array.Accelerate.AST
import Data.Array.Accelerate.Trafo                              ( DelayedOpenAcc(..), DelayedOpenAfun, DelayedAcc, DelayedAfun )
import Data.Array.Accelerate.Array.Sugar                       ( Array, Shape, Elt, Arrays )
import qualified Data.Array.Accelerate.Array.Sugar             as Sugar

import Data.Array.Accelerate.HIP.CodeGen
import Data.Array.Accelerate.HIP.FFI
import Data.Array.Accelerate.HIP.State                          -- HIP monad: the context, the memory table, the stream reservoir

import Control.Monad.Trans                                      ( liftIO )
import Data.Bits                                              ( (.|.) )
import Data.Int
import Data.Word                                              ( Word32 )
import Data.List                                                ( intercalate )


-- | what the execution phase needs of a node's kernels: the instance, and which array variables to pass it, in
-- the order the fragments numbered them (the `AccKernel` record and `Gamma` of AST.hs:51-59,87-112)
data Kernel aenv = Kernel
  { kernelSkel :: !Skel
  , kernelEnv  :: [Int]                           -- de Bruijn indices into aenv, slot order
  }

-- | the program with a kernel where one is needed.  Array-level control flow, `use`, tuples and `reshape` have
-- none (Execute.hs:187-219 runs them on the host).
data ExecOpenAcc aenv a where
  ExecAcc  :: Maybe (Kernel aenv)
           -> PreOpenAcc ExecOpenAcc aenv a
           -> ExecOpenAcc aenv a
  -- a delayed operand: only its extent is evaluated at run time, its index function was fused into the consumer
  ExecFused :: (Shape sh, Elt e) => PreExp ExecOpenAcc aenv sh -> ExecOpenAcc aenv (Array sh e)

type ExecAcc a        = ExecOpenAcc () a
type ExecOpenAfun     = PreOpenAfun ExecOpenAcc
type ExecAfun a       = ExecOpenAfun () a


compileAcc :: Arrays a => DelayedAcc a -> HIP (ExecAcc a)
compileAcc = compileOpenAcc False

compileAfun :: DelayedAfun f -> HIP (ExecAfun f)
compileAfun = compileOpenAfun False

compileOpenAfun :: Bool -> DelayedOpenAfun aenv f -> HIP (ExecOpenAfun aenv f)
compileOpenAfun g (Alam l)  = Alam  <$> compileOpenAfun g l
compileOpenAfun g (Abody b) = Abody <$> compileOpenAcc g b

-- `guarded`: the node belongs to the predicate or the body of an `awhile` whose iterations are enqueued ahead, so
-- its kernels are built with ACC_FLAG_GUARDED (include/acc_hip.h, acc_guard_create)
compileOpenAcc :: forall aenv a. Bool -> DelayedOpenAcc aenv a -> HIP (ExecOpenAcc aenv a)
compileOpenAcc _       Delayed{..}    = ExecFused <$> travE extentD
compileOpenAcc guarded (Manifest pacc) =
  case pacc of
    -- no kernel
    Avar ix               -> plain (Avar ix)
    Alet a b              -> plain =<< Alet <$> travA a <*> travA b
    Apply f a             -> plain =<< Apply <$> compileOpenAfun guarded f <*> travA a
    Atuple tup            -> plain =<< Atuple <$> travAtup tup
    Aprj ix tup           -> plain =<< Aprj ix <$> travA tup
    Acond p t e           -> plain =<< Acond <$> travE p <*> travA t <*> travA e
    -- predicate and body under the loop's guard; a body that itself needs the host is found by Execute
    Awhile p f a          -> plain =<< Awhile <$> compileOpenAfun True p <*> compileOpenAfun True f <*> travA a
    Use arrs              -> plain (Use arrs)
    Unit e                -> plain =<< Unit <$> travE e
    Reshape sh a          -> plain =<< Reshape <$> travE sh <*> travA a
    Aforeign{}            -> unsupported "Aforeign"

    -- the map family: one kernel over the result's linear index space (Mapping.hs, IndexSpace.hs:47-141)
    Generate sh f         -> do
      let (get, g) = codegenFun1 emptyGamma (fromIndexFun f)
      kernel accSkelGenerate g get Nothing Nothing Nothing =<< (Generate <$> travE sh <*> travF f)
    Transform sh p f a    -> fusedOnly "Transform" sh p f a
    Map f a               -> do
      let (get, g) = mapOver f a
      kernel accSkelMap g get Nothing Nothing Nothing =<< (Map <$> travF f <*> travD a)
    ZipWith f a b         -> do
      let (get, g) = zipOver f a b
      kernel accSkelMap g get Nothing Nothing Nothing =<< (ZipWith <$> travF f <*> travD a <*> travD b)
    Backpermute sh p a    -> do
      let (get, g) = gatherThrough p a
          -- an index function that exchanges the two innermost components of the index (`transpose`) reads one
          -- element of every source row per run of the result: such a kernel produces its result in square tiles
          across   = if exchangesInnermost p then accFlagTiled else 0
      kernelWith across accSkelTransform g get Nothing Nothing Nothing =<< (Backpermute <$> travE sh <*> travF p <*> travD a)
    Replicate{}           -> fusedAway "Replicate"
    Slice{}               -> fusedAway "Slice"

    -- reductions (Reduction.hs): the operand is fused into `get`
    Fold f z a            -> reduction accSkelFold    f (Just z) a  (\f' z' a' -> Fold f' z' a')
    Fold1 f a             -> reduction accSkelFold1   f Nothing  a  (\f' _  a' -> Fold1 f' a')
    FoldSeg f z a s       -> segmented accSkelFoldSeg  f (Just z) a s
    Fold1Seg f a s        -> segmented accSkelFold1Seg f Nothing  a s

    -- scans (PrefixSum.hs): one single-pass kernel each
    Scanl  f z a          -> scan accSkelScanl   f (Just z) a (\f' z' a' -> Scanl  f' z' a')
    Scanl' f z a          -> scan accSkelScanlP  f (Just z) a (\f' z' a' -> Scanl' f' z' a')
    Scanl1 f a            -> scan accSkelScanl1  f Nothing  a (\f' _  a' -> Scanl1 f' a')
    Scanr  f z a          -> scan accSkelScanr   f (Just z) a (\f' z' a' -> Scanr  f' z' a')
    Scanr' f z a          -> scan accSkelScanrP  f (Just z) a (\f' z' a' -> Scanr' f' z' a')
    Scanr1 f a            -> scan accSkelScanr1  f Nothing  a (\f' _  a' -> Scanr1 f' a')

    -- forward permutation (IndexSpace.hs:160-303)
    Permute f d p a       -> do
      let (get, g0)  = codegenDelayed emptyGamma a
          (comb, g1) = codegenFun2 g0 f
          (perm, g2) = codegenPermutation g1 (extentNames a 0) outNames p
      kernel accSkelPermute g2 get (Just comb) Nothing (Just perm) =<< (Permute <$> travF f <*> travA d <*> travF p <*> travD a)

    -- stencils (Stencil.hs, Stencil/Extra.hs): the source is manifest, the function ranges over its taps
    Stencil f bnd a       -> stencilKernel accSkelStencil  =<< (Stencil  <$> travF f <*> pure bnd <*> travA a)
    Stencil2 f b1 a b2 b  -> stencilKernel accSkelStencil2 =<< (Stencil2 <$> travF f <*> pure b1 <*> travA a <*> pure b2 <*> travA b)
  where
    travA :: DelayedOpenAcc aenv b -> HIP (ExecOpenAcc aenv b)
    travA = compileOpenAcc guarded

    -- an operand that may be delayed: its kernel-side half has gone into the consumer's fragment
    travD :: DelayedOpenAcc aenv b -> HIP (ExecOpenAcc aenv b)
    travD = compileOpenAcc guarded

    travAtup :: Atuple (DelayedOpenAcc aenv) t -> HIP (Atuple (ExecOpenAcc aenv) t)
    travAtup NilAtup        = return NilAtup
    travAtup (SnocAtup t a) = SnocAtup <$> travAtup t <*> travA a

    -- scalar code that runs on the host at execution time (shapes, seeds read back, conditions): the arrays it
    -- names are compiled, the expression itself is interpreted (Execute.hs:454-560)
    travE :: PreOpenExp DelayedOpenAcc env aenv t -> HIP (PreOpenExp ExecOpenAcc env aenv t)
    travE = rebuildExp travA

    travF :: PreOpenFun DelayedOpenAcc env aenv t -> HIP (PreOpenFun ExecOpenAcc env aenv t)
    travF (Body b) = Body <$> travE b
    travF (Lam f)  = Lam  <$> travF f

    plain :: PreOpenAcc ExecOpenAcc aenv a -> HIP (ExecOpenAcc aenv a)
    plain = return . ExecAcc Nothing

    unsupported what = error ("Data.Array.Accelerate.HIP: " ++ what ++ " is not supported by this backend")
    fusedAway what   = error ("Data.Array.Accelerate.HIP: a manifest " ++ what ++ " survives fusion only as a Backpermute")
    fusedOnly what _ _ _ _ = fusedAway what

    outNames = [ "shOut_" ++ show d | d <- reverse [0 .. 8 :: Int] ]

    -- one skeleton instance: fragments -> description -> acc_skel_create (compiled, cached and loaded inside)
    kernel :: Int32 -> Gamma -> Fragment -> Maybe Fragment -> Maybe Fragment -> Maybe Fragment
           -> PreOpenAcc ExecOpenAcc aenv a -> HIP (ExecOpenAcc aenv a)
    kernel = kernelWith 0

    kernelWith :: Word32 -> Int32 -> Gamma -> Fragment -> Maybe Fragment -> Maybe Fragment -> Maybe Fragment
               -> PreOpenAcc ExecOpenAcc aenv a -> HIP (ExecOpenAcc aenv a)
    kernelWith flags kind gamma get combine seed permutation node = do
      ctx  <- hipContext
      skel <- liftIO $ createSkeleton ctx Skeleton
                { skelKind        = kind
                , skelFlags       = flags .|. (if guarded then accFlagGuarded else 0)
                , skelEnv         = environment gamma
                , skelEltType     = intercalate ", " (resultTypes node)
                , skelOutRank     = resultRank node
                , skelPreamble    = Nothing
                , skelGet         = Just (fragmentText get)
                , skelCombine     = fragmentText <$> combine
                , skelSeed        = fragmentText <$> seed
                , skelPermutation = fragmentText <$> permutation
                , skelCombineHint = maybe accCombineGeneric combineHint combine
                , skelSegType     = Nothing
                }
      return (ExecAcc (Just (Kernel skel (gammaArrays gamma))) node)

    reduction kind f z a rebuild = do
      let (get, g0)  = codegenDelayed emptyGamma a
          (comb, g1) = codegenFun2 g0 f
          (seed, g2) = maybe (Nothing, g1) (\e -> let (s, g') = codegenExp g1 e in (Just s, g')) z
      kernel kind g2 get (Just comb) seed Nothing =<< (rebuild <$> travF f <*> traverse travE z <*> travD a)

    segmented kind f z a s = do
      let (get, g0)  = codegenDelayed emptyGamma a
          (comb, g1) = codegenFun2 g0 f
          (seed, g2) = maybe (Nothing, g1) (\e -> let (sd, g') = codegenExp g1 e in (Just sd, g')) z
      -- the segment lengths become offsets by an ordinary scan node first (CUDA.hs:402 does the same in the front end)
      node <- case z of
                Just z' -> FoldSeg  <$> travF f <*> travE z' <*> travD a <*> travA s
                Nothing -> Fold1Seg <$> travF f <*> travD a <*> travA s
      kernel kind g2 get (Just comb) seed Nothing node

    scan kind f z a rebuild = do
      let (get, g0)  = codegenDelayed emptyGamma a
          (comb, g1) = codegenFun2 g0 f
          (seed, g2) = maybe (Nothing, g1) (\e -> let (s, g') = codegenExp g1 e in (Just s, g')) z
      kernel kind g2 get (Just comb) seed Nothing =<< (rebuild <$> travF f <*> traverse travE z <*> travD a)

    -- the stencil description carries tap offsets, boundary conditions and `stencil_fn` besides the fields above;
    -- withSkelDesc pokes them the same way (FFI.hsc)
    stencilKernel kind node = kernel kind emptyGamma (stencilFragment node) Nothing Nothing Nothing node


-- Supplied by the modules this backend shares with Data.Array.Accelerate.CUDA unchanged, or by small helpers that
-- are mechanical given the AST: naming them keeps this traversal readable.
fromIndexFun    :: PreOpenFun DelayedOpenAcc env aenv (sh -> e) -> PreOpenFun DelayedOpenAcc env aenv (Int -> e)
mapOver         :: PreOpenFun DelayedOpenAcc () aenv (a -> b) -> DelayedOpenAcc aenv (Array sh a) -> (Fragment, Gamma)
zipOver         :: PreOpenFun DelayedOpenAcc () aenv (a -> b -> c) -> DelayedOpenAcc aenv (Array sh a) -> DelayedOpenAcc aenv (Array sh b) -> (Fragment, Gamma)
gatherThrough   :: PreOpenFun DelayedOpenAcc () aenv (sh' -> sh) -> DelayedOpenAcc aenv (Array sh e) -> (Fragment, Gamma)
extentNames     :: DelayedOpenAcc aenv (Array sh e) -> Int -> [String]
environment     :: Gamma -> [(Int32, [String])]
resultTypes     :: PreOpenAcc ExecOpenAcc aenv a -> [String]
resultRank      :: PreOpenAcc ExecOpenAcc aenv a -> Int32
combineHint     :: Fragment -> Int32              -- ACC_COMBINE_ADD .. when the text is literally x + y, acc_pmin(x, y), ...
exchangesInnermost :: PreOpenFun DelayedOpenAcc () aenv (sh' -> sh) -> Bool   -- \(sh :. y :. x) -> (sh :. x :. y), structurally
stencilFragment :: PreOpenAcc ExecOpenAcc aenv a -> Fragment
rebuildExp      :: (forall b. DelayedOpenAcc aenv b -> HIP (ExecOpenAcc aenv b)) -> PreOpenExp DelayedOpenAcc env aenv t -> HIP (PreOpenExp ExecOpenAcc env aenv t)
fromIndexFun    = undefined
mapOver         = undefined
zipOver         = undefined
gatherThrough   = undefined
extentNames     = undefined
environment     = undefined
resultTypes     = undefined
resultRank      = undefined
combineHint     = undefined
exchangesInnermost = undefined
stencilFragment = undefined
rebuildExp      = undefined
