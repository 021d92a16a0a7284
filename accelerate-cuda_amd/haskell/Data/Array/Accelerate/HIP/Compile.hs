{-# LANGUAGE GADTs, ScopedTypeVariables, RecordWildCards, RankNTypes #-}
-- |
-- Module      : Data.Array.Accelerate.HIP.Compile
--
-- First traversal of a delayed array program: every node that needs a kernel gets its
-- skeleton instance -- fragments from CodeGen, `acc_skel_create_async` through the library's
-- kernel cache and its pool of compiler workers -- and the tree is rebuilt with the handles in
-- place; the kernels of a program compile side by side and a kernel's first launch waits for
-- its own.  The role of Compile.hs:110-235 (`compileOpenAcc`); what that module does besides
-- (temporary files, the nvcc subprocess, the persistent cache, occupancy, Compile.hs:444-594
-- and Persistent.hs) lives inside the library.
--
-- UNCOMPILED: no GHC in the image this library is built and tested in.
--
module Data.Array.Accelerate.HIP.Compile (

  ExecOpenAcc(..), ExecAcc, ExecAfun, ExecOpenAfun, Kernel(..),
  compileAcc, compileAfun,

) where

import Data.Array.Accelerate.AST
import Data.Array.Accelerate.Trafo                              ( DelayedOpenAcc(..), DelayedOpenAfun, DelayedAcc, DelayedAfun, DelayedOpenExp, DelayedOpenFun )
import Data.Array.Accelerate.Analysis.Stencil                  ( offsets, offsets2 )
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
  , kernelEnv  :: [ArrayVar aenv]                 -- the array variables to pass, slot order
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
      let (get, g) = codegenIndexFun emptyGamma f
      kernel accSkelGenerate g get Nothing Nothing Nothing =<< (Generate <$> travE sh <*> travF f)
    Transform sh p f a    -> fusedOnly "Transform" sh p f a
    Map f a               -> do
      let (get, g) = codegenMap emptyGamma f a
      kernel accSkelMap g get Nothing Nothing Nothing =<< (Map <$> travF f <*> travD a)
    ZipWith f a b         -> do
      let (get, g) = codegenZipWith emptyGamma f a b
      kernel accSkelMap g get Nothing Nothing Nothing =<< (ZipWith <$> travF f <*> travD a <*> travD b)
    Backpermute sh p a    -> do
      let (get, g) = codegenIndexedBy emptyGamma p a
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
          (perm, g2) = codegenPermutation g1 a p
      kernel accSkelPermute g2 get (Just comb) Nothing (Just perm) =<< (Permute <$> travF f <*> travA d <*> travF p <*> travD a)

    -- stencils (Stencil.hs, Stencil/Extra.hs): the source is manifest, the function ranges over its taps
    Stencil f bnd a       -> do
      let taps     = map shapeToOffsets (stencilOffsets f a)
          src      = stencilSource a bnd taps
          (fn, g)  = codegenStencilFun emptyGamma [("t", length taps, componentsOf a)] f
      stencilKernel accSkelStencil g fn [src] =<< (Stencil <$> travF f <*> pure bnd <*> travA a)
    Stencil2 f b1 a b2 b  -> do
      let (o1, o2) = stencilOffsets2 f a b
          taps1    = map shapeToOffsets o1
          taps2    = map shapeToOffsets o2
          (fn, g)  = codegenStencilFun emptyGamma [("t", length taps1, componentsOf a), ("u", length taps2, componentsOf b)] f
      stencilKernel accSkelStencil2 g fn [stencilSource a b1 taps1, stencilSource b b2 taps2]
        =<< (Stencil2 <$> travF f <*> pure b1 <*> travA a <*> pure b2 <*> travA b)
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
    travE = rebuildExp (compileOpenAcc guarded)

    travF :: PreOpenFun DelayedOpenAcc env aenv t -> HIP (PreOpenFun ExecOpenAcc env aenv t)
    travF (Body b) = Body <$> travE b
    travF (Lam f)  = Lam  <$> travF f

    plain :: PreOpenAcc ExecOpenAcc aenv a -> HIP (ExecOpenAcc aenv a)
    plain = return . ExecAcc Nothing

    unsupported what = error ("Data.Array.Accelerate.HIP: " ++ what ++ " is not supported by this backend")
    fusedAway what   = error ("Data.Array.Accelerate.HIP: a manifest " ++ what ++ " survives fusion only as a Backpermute")
    fusedOnly what _ _ _ _ = fusedAway what

    -- one skeleton instance: fragments -> description -> acc_skel_create_async (generated and checked now; compiled
    -- by the library's workers, cached and loaded inside; the node's first launch waits for it)
    kernel :: Int32 -> Gamma aenv -> Fragment -> Maybe Fragment -> Maybe Fragment -> Maybe Fragment
           -> PreOpenAcc ExecOpenAcc aenv a -> HIP (ExecOpenAcc aenv a)
    kernel = kernelWith 0

    kernelWith :: Word32 -> Int32 -> Gamma aenv -> Fragment -> Maybe Fragment -> Maybe Fragment -> Maybe Fragment
               -> PreOpenAcc ExecOpenAcc aenv a -> HIP (ExecOpenAcc aenv a)
    kernelWith flags kind gamma get combine seed permutation node =
      instantiate gamma node emptySkeleton
        { skelKind        = kind
        , skelFlags       = flags
        , skelGet         = Just (fragmentText get)
        , skelCombine     = fragmentText <$> combine
        , skelSeed        = fragmentText <$> seed
        , skelPermutation = fragmentText <$> permutation
        , skelCombineHint = maybe accCombineGeneric (combineHint (resultTypes node)) combine
        , skelSegType     = segmentType node
        }

    instantiate :: Gamma aenv -> PreOpenAcc ExecOpenAcc aenv a -> Skeleton -> HIP (ExecOpenAcc aenv a)
    instantiate gamma node sk = do
      ctx  <- hipContext
      skel <- liftIO $ createSkeletonAsync ctx sk
                { skelFlags   = skelFlags sk .|. (if guarded then accFlagGuarded else 0)
                , skelEnv     = gammaSignature gamma
                , skelEltType = intercalate ", " (resultTypes node)
                , skelOutRank = resultRank node
                }
      return (ExecAcc (Just (Kernel skel (gammaArrays gamma))) node)

    reduction kind f z a rebuild = do
      let (get, g0)  = codegenDelayed emptyGamma a
          (comb, g1) = codegenFun2 g0 f
          (seed, g2) = maybe (Nothing, g1) (\e -> let (s, g') = codegenExp g1 e in (Just s, g')) z
          -- an operand that reads its source across the rows (`fold f z (transpose m)`): the rows the fold sees lie
          -- across memory, and the kernel gives a row to a lane instead of a team of lanes (ACC_FLAG_TILED)
          across     = if readsAcross a then accFlagTiled else 0
      kernelWith across kind g2 get (Just comb) seed Nothing =<< (rebuild <$> travF f <*> traverse travE z <*> travD a)

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

    -- a stencil has no `get`: its function ranges over the taps of its manifest sources, which the driver is handed
    -- beside the environment (the free arrays of the function itself)
    stencilKernel :: Int32 -> Gamma aenv -> Fragment -> [StencilSource] -> PreOpenAcc ExecOpenAcc aenv a -> HIP (ExecOpenAcc aenv a)
    stencilKernel kind gamma fn sources node =
      instantiate gamma node emptySkeleton { skelKind = kind, skelStencilFn = Just (fragmentText fn), skelSources = sources }


-- The pieces of the traversal above
-- ---------------------------------

componentsOf :: forall acc aenv sh e. Elt e => acc aenv (Array sh e) -> Int
componentsOf _ = length (eltTypeNames (undefined :: e))

-- | the positions of a stencil pattern relative to its focus, in the order the pattern's (nested) tuple lists them,
-- left to right: Data.Array.Accelerate.Analysis.Stencil works them out from the types alone (Stencil.hs:97,203)
stencilOffsets :: forall acc aenv sh a b stencil. Stencil sh a stencil
               => PreOpenFun acc () aenv (stencil -> b) -> acc aenv (Array sh a) -> [sh]
stencilOffsets _ _ = offsets (undefined :: Fun aenv (stencil -> b)) (undefined :: OpenAcc aenv (Array sh a))

stencilOffsets2 :: forall acc aenv sh a b c stencil1 stencil2. (Stencil sh a stencil1, Stencil sh b stencil2)
                => PreOpenFun acc () aenv (stencil1 -> stencil2 -> c) -> acc aenv (Array sh a) -> acc aenv (Array sh b) -> ([sh], [sh])
stencilOffsets2 _ _ _ = offsets2 (undefined :: Fun aenv (stencil1 -> stencil2 -> c))
                                 (undefined :: OpenAcc aenv (Array sh a)) (undefined :: OpenAcc aenv (Array sh b))

-- | an offset of a stencil pattern as a row of acc_skel_desc.tap_offsets: outermost dimension first
shapeToOffsets :: Shape sh => sh -> [Int32]
shapeToOffsets = map fromIntegral . reverse . Sugar.shapeToList

stencilSource :: forall acc aenv sh e. Elt e => acc aenv (Array sh e) -> Boundary (Sugar.EltRepr e) -> [[Int32]] -> StencilSource
stencilSource _ bnd taps = StencilSource
  { sourceType     = intercalate ", " (eltTypeNames (undefined :: e))
  , sourceBoundary = case bnd of { Clamp -> accBoundaryClamp; Mirror -> accBoundaryMirror; Wrap -> accBoundaryWrap; Constant{} -> accBoundaryConstant }
  , sourceConstant = codegenBoundary (undefined :: e) bnd
  , sourceTaps     = taps
  }

-- | the C types of the components of a node's result element, highest first (acc_skel_desc.elt_type)
resultTypes :: forall aenv a. PreOpenAcc ExecOpenAcc aenv a -> [String]
resultTypes node = case node of
  Generate{}    -> elt node
  Map{}         -> elt node
  ZipWith{}     -> elt node
  Backpermute{} -> elt node
  Fold{}        -> elt node
  Fold1{}       -> elt node
  FoldSeg{}     -> elt node
  Fold1Seg{}    -> elt node
  Scanl{}       -> elt node
  Scanl1{}      -> elt node
  Scanr{}       -> elt node
  Scanr1{}      -> elt node
  Scanl' _ z _  -> expType z
  Scanr' _ z _  -> expType z
  Permute{}     -> elt node
  Stencil{}     -> elt node
  Stencil2{}    -> elt node
  _             -> error "resultTypes: a node without a kernel"
  where
    elt :: forall sh e. Elt e => PreOpenAcc ExecOpenAcc aenv (Array sh e) -> [String]
    elt _ = eltTypeNames (undefined :: e)
    expType :: forall env t. Elt t => PreOpenExp ExecOpenAcc env aenv t -> [String]
    expType _ = eltTypeNames (undefined :: t)

-- | the rank of a node's result (acc_skel_desc.out_rank: map family and stencils; the others take their extents
-- from the driver's arguments)
resultRank :: forall aenv a. PreOpenAcc ExecOpenAcc aenv a -> Int32
resultRank node = case node of
  Generate{}    -> rank node
  Map{}         -> rank node
  ZipWith{}     -> rank node
  Backpermute{} -> rank node
  Permute{}     -> rank node
  Stencil{}     -> rank node
  Stencil2{}    -> rank node
  _             -> 0
  where
    rank :: forall sh e. Shape sh => PreOpenAcc ExecOpenAcc aenv (Array sh e) -> Int32
    rank _ = fromIntegral (Sugar.rank (undefined :: sh))

-- | the C type of a segmented fold's offsets (acc_skel_desc.seg_type)
segmentType :: PreOpenAcc ExecOpenAcc aenv a -> Maybe String
segmentType node = case node of
  FoldSeg _ _ _ s -> Just (seg s)
  Fold1Seg _ _ s  -> Just (seg s)
  _               -> Nothing
  where
    seg :: forall acc aenv' i. Elt i => acc aenv' (Sugar.Segments i) -> String
    seg _ = head (eltTypeNames (undefined :: i))

-- | a combining function the hardware applies atomically, recognised by its generated text: x + y on 32- and
-- 64-bit integers and floats, min, max and the bitwise operators on the integers (ACC_COMBINE_ADD ..)
combineHint :: [String] -> Fragment -> Int32
combineHint [ty] frag
  | ty `elem` integers ++ floats, text `elem` operator "+"    = accCombineAdd
  | ty `elem` integers,           text `elem` call "acc_pmin" = accCombineMin
  | ty `elem` integers,           text `elem` call "acc_pmax" = accCombineMax
  | ty `elem` integers,           text `elem` operator "&"    = accCombineAnd
  | ty `elem` integers,           text `elem` operator "|"    = accCombineOr
  | ty `elem` integers,           text `elem` operator "^"    = accCombineXor
  where
    text        = fragmentText frag
    integers    = ["Int32", "Word32", "Int64", "Word64"]
    floats      = ["float", "double"]
    operator op = [ "((" ++ ty ++ ")(x " ++ op ++ " y))", "((" ++ ty ++ ")(y " ++ op ++ " x))" ]
    call fn     = [ fn ++ "(x, y)", fn ++ "(y, x)" ]
combineHint _ _ = accCombineGeneric

-- | \(sh :. y :. x) -> (sh :. x :. y), structurally: the index function of `transpose` and its like
exchangesInnermost :: DelayedOpenFun () aenv (sh' -> sh) -> Bool
exchangesInnermost (Lam (Body (IndexCons (IndexCons rest a) b)))
  | IndexHead (Var ZeroIdx)                         <- a
  , IndexHead (IndexTail (Var ZeroIdx))             <- b
  , outer rest                                      = True
  where
    -- what is left of the index is passed on as it is
    outer :: DelayedOpenExp env aenv t -> Bool
    outer (IndexTail (IndexTail (Var ZeroIdx))) = True
    outer IndexNil                              = True
    outer _                                     = False
exchangesInnermost _ = False

-- | a delayed array whose element at (sh :. y :. x) is a manifest array's element at (sh :. x :. y), whatever is done
-- to the element afterwards: what fusion makes of `map f (transpose m)`
readsAcross :: DelayedOpenAcc aenv (Array sh e) -> Bool
readsAcross Delayed{ indexD = f } = across f
  where
    across :: DelayedOpenFun () aenv (sh -> e) -> Bool
    across (Lam (Body b)) = reads b
    across _              = False
    reads :: DelayedOpenExp env aenv t -> Bool
    reads (Index Manifest{} (IndexCons (IndexCons _ a) b))
      | IndexHead (Var ZeroIdx)             <- a
      , IndexHead (IndexTail (Var ZeroIdx)) <- b = True
    reads (PrimApp _ x)                         = reads x
    reads _                                     = False
readsAcross _ = False

-- | scalar code that stays on the host: the arrays it names are compiled, the expression is rebuilt around them
-- (Compile.hs:237-300 `travE`)
rebuildExp :: forall aenv env t.
              (forall b. DelayedOpenAcc aenv b -> HIP (ExecOpenAcc aenv b))
           -> PreOpenExp DelayedOpenAcc env aenv t
           -> HIP (PreOpenExp ExecOpenAcc env aenv t)
rebuildExp travA = go
  where
    go :: forall env' s. PreOpenExp DelayedOpenAcc env' aenv s -> HIP (PreOpenExp ExecOpenAcc env' aenv s)
    go e = case e of
      Var ix              -> return (Var ix)
      Const c             -> return (Const c)
      PrimConst c         -> return (PrimConst c)
      IndexAny            -> return IndexAny
      IndexNil            -> return IndexNil
      Let a b             -> Let <$> go a <*> go b
      Tuple t             -> Tuple <$> goT t
      Prj ix x            -> Prj ix <$> go x
      IndexCons sh i      -> IndexCons <$> go sh <*> go i
      IndexHead sh        -> IndexHead <$> go sh
      IndexTail sh        -> IndexTail <$> go sh
      IndexSlice s ix sh  -> IndexSlice s <$> go ix <*> go sh
      IndexFull s ix sl   -> IndexFull s <$> go ix <*> go sl
      ToIndex sh ix       -> ToIndex <$> go sh <*> go ix
      FromIndex sh i      -> FromIndex <$> go sh <*> go i
      Cond p t f          -> Cond <$> go p <*> go t <*> go f
      While p f x         -> While <$> goF p <*> goF f <*> go x
      PrimApp f x         -> PrimApp f <$> go x
      Index a ix          -> Index <$> travA a <*> go ix
      LinearIndex a i     -> LinearIndex <$> travA a <*> go i
      Shape a             -> Shape <$> travA a
      ShapeSize sh        -> ShapeSize <$> go sh
      Intersect a b       -> Intersect <$> go a <*> go b
      Union a b           -> Union <$> go a <*> go b
      Foreign{}           -> error "Data.Array.Accelerate.HIP: foreign scalar functions are not supported by this backend"

    goT :: forall env' s. Tuple (PreOpenExp DelayedOpenAcc env' aenv) s -> HIP (Tuple (PreOpenExp ExecOpenAcc env' aenv) s)
    goT NilTup        = return NilTup
    goT (SnocTup t x) = SnocTup <$> goT t <*> go x

    goF :: forall env' s. PreOpenFun DelayedOpenAcc env' aenv s -> HIP (PreOpenFun ExecOpenAcc env' aenv s)
    goF (Body b) = Body <$> go b
    goF (Lam f)  = Lam  <$> goF f
