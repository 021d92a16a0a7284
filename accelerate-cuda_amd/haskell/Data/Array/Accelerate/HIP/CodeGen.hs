{-# LANGUAGE GADTs, RankNTypes, ScopedTypeVariables, PatternGuards, ExistentialQuantification #-}
-- |
-- Module      : Data.Array.Accelerate.HIP.CodeGen
--
-- Scalar functions and delayed arrays of the Accelerate AST as the TEXT FRAGMENTS that
-- libacchip's skeleton templates splice in (include/acc_hip.h, acc_skel_desc): `get` over the
-- linear index `ix`, `combine` over `x` and `y`, `seed`, `permutation`, a stencil's function
-- over its taps.  It takes the place of CodeGen.hs:338-821 and CodeGen/Arithmetic.hs, which
-- build language-c-quote ASTs for templates written in Haskell; here the templates are the
-- library's and only expressions cross the boundary.
--
-- UNCOMPILED: the image this library is built and tested in holds no GHC.  The module is
-- written against accelerate-1.0's Data.Array.Accelerate.AST / .Trafo; the names of the device
-- functions it emits are checked against csrc/device/acc_prim.h by tests/test_host.py.
--
-- A value of tuple type is a LIST of C expressions, one per component, highest component
-- first -- the order of the fields of the generated `struct acc_elt` and of the pointers of an
-- array of tuples (CodeGen/Base.hs:344-357).  A component nobody asks for is never emitted:
-- that is the reference's dead-code elimination for free (CodeGen.hs:283-314).
--
module Data.Array.Accelerate.HIP.CodeGen (

  Gamma, ArrayVar(..), emptyGamma, gammaArrays, gammaSignature,
  Fragment, fragmentText,
  codegenFun1, codegenFun2, codegenExp, codegenDelayed, codegenMap, codegenZipWith, codegenIndexFun, codegenIndexedBy,
  codegenPermutation,
  codegenStencilFun, codegenBoundary,
  eltTypeNames, cTypeOf, outExtents,

) where

import Data.Array.Accelerate.AST
import Data.Array.Accelerate.Trafo                              ( DelayedOpenAcc(..), DelayedOpenExp, DelayedOpenFun )
import Data.Array.Accelerate.Type
import Data.Array.Accelerate.Array.Sugar                       ( Elt, Shape, eltType, Array )
import qualified Data.Array.Accelerate.Array.Sugar             as Sugar

import Control.Monad.State.Strict
import Data.Int                                                 ( Int32 )
import Data.List                                                ( intercalate, sortBy )
import Data.Ord                                                 ( comparing )
import qualified Data.IntMap.Strict                             as IM


-- The free array variables of the fragments of one skeleton
-- ---------------------------------------------------------
--
-- Array variables are numbered in order of first use; variable k is spelt arrIn<k>_<c> /
-- shIn<k>_<d> in the text and becomes entry k of the `env` arrays handed to acc_exec_*
-- (AST.hs:87-112 `Gamma`, Execute.hs:835-836).

-- | an array variable together with what is known of its type where it was met: the execution phase looks its
-- value up in the array environment and needs the extent and the components (the `Idx_` of AST.hs:96-98)
data ArrayVar aenv = forall sh e. (Shape sh, Elt e) => ArrayVar (Idx aenv (Array sh e))

data Gamma aenv = Gamma
  { gammaNext :: !Int
  , gammaSlot :: !(IM.IntMap (Int, ArrayVar aenv))   -- de Bruijn index of the array variable -> its slot, and the variable
  }

emptyGamma :: Gamma aenv
emptyGamma = Gamma 0 IM.empty

-- | the arrays to pass, in slot order
gammaArrays :: Gamma aenv -> [ArrayVar aenv]
gammaArrays g = map snd (sortBy (comparing fst) (IM.elems (gammaSlot g)))

-- | what acc_skel_desc.env says of them: rank, and the C type of every component, component 0 first
gammaSignature :: Gamma aenv -> [(Int32, [String])]
gammaSignature g = [ sig v | v <- gammaArrays g ]
  where
    sig :: ArrayVar aenv -> (Int32, [String])
    sig (ArrayVar (_ :: Idx aenv (Array sh e))) =
      (fromIntegral (Sugar.rank (undefined :: sh)), reverse (eltTypeNames (undefined :: e)))

type Gen aenv = State (Gamma aenv, Int)          -- the environment so far, and a supply of names for local bindings

slotOf :: (Shape sh, Elt e) => Idx aenv (Array sh e) -> Gen aenv Int
slotOf ix = do
  (g, n) <- get
  let v = idxToInt ix
  case IM.lookup v (gammaSlot g) of
    Just (s, _) -> return s
    Nothing     -> do
      let s = gammaNext g
      put (g { gammaNext = s + 1, gammaSlot = IM.insert v (s, ArrayVar ix) (gammaSlot g) }, n)
      return s

fresh :: Gen aenv String
fresh = do
  (g, n) <- get
  put (g, n + 1)
  return ("v" ++ show n)

-- | an expression fragment: statements that bind locals, then one C expression per component
data Fragment = Fragment [String] [String]

-- | the closed text of a single-valued fragment, or of a tuple as a brace initialiser of acc_elt
fragmentText :: Fragment -> String
fragmentText (Fragment binds comps)
  | null binds = value
  | otherwise  = "({ " ++ unwords binds ++ " " ++ value ++ "; })"          -- a GNU statement expression
  where
    value = case comps of
              [c] -> c
              cs  -> "acc_elt{" ++ intercalate ", " cs ++ "}"


-- Types
-- -----

-- | C names of the components of an element type, highest component first ("float", "Int32", ...: the
-- typedefs of csrc/device/acc_hip_device.h)
eltTypeNames :: forall e. Elt e => e -> [String]
eltTypeNames _ = go (eltType (undefined :: e)) []
  where
    go :: TupleType t -> [String] -> [String]
    go UnitTuple         acc = acc
    go (SingleTuple t)   acc = cTypeOf t : acc
    go (PairTuple t1 t2) acc = go t1 (go t2 acc)

cTypeOf :: ScalarType t -> String
cTypeOf (NumScalarType (IntegralNumType t)) = integral t
  where
    integral :: IntegralType a -> String
    integral TypeInt{}     = "Int64"
    integral TypeInt8{}    = "Int8"
    integral TypeInt16{}   = "Int16"
    integral TypeInt32{}   = "Int32"
    integral TypeInt64{}   = "Int64"
    integral TypeWord{}    = "Word64"
    integral TypeWord8{}   = "Word8"
    integral TypeWord16{}  = "Word16"
    integral TypeWord32{}  = "Word32"
    integral TypeWord64{}  = "Word64"
    integral TypeCShort{}  = "Int16"
    integral TypeCUShort{} = "Word16"
    integral TypeCInt{}    = "Int32"
    integral TypeCUInt{}   = "Word32"
    integral TypeCLong{}   = "Int64"
    integral TypeCULong{}  = "Word64"
    integral TypeCLLong{}  = "Int64"
    integral TypeCULLong{} = "Word64"
cTypeOf (NumScalarType (FloatingNumType t)) = floating t
  where
    floating :: FloatingType a -> String
    floating TypeFloat{}   = "float"
    floating TypeDouble{}  = "double"
    floating TypeCFloat{}  = "float"
    floating TypeCDouble{} = "double"
cTypeOf (NonNumScalarType t) = other t
  where
    other :: NonNumType a -> String
    other TypeBool{}   = "Word8"                 -- Bool is one byte on the device, Char a code point
    other TypeChar{}   = "Word32"
    other TypeCChar{}  = "Int8"
    other TypeCSChar{} = "Int8"
    other TypeCUChar{} = "Word8"


-- Scalar environments
-- -------------------

-- what each bound scalar variable stands for: the texts of its components
data Val env where
  Empty :: Val ()
  Push  :: Val env -> [String] -> Val (env, t)

prj :: Idx env t -> Val env -> [String]
prj ZeroIdx      (Push _   v) = v
prj (SuccIdx ix) (Push val _) = prj ix val


-- Expressions
-- -----------

-- | a closed scalar expression (a seed, a shape): Execute.hs evaluates shapes on the host instead
codegenExp :: Gamma aenv -> DelayedOpenExp () aenv t -> (Fragment, Gamma aenv)
codegenExp g e = close g (expr e Empty)

-- | \x -> body, its argument spelt `x` (components x.a<n-1> .. x.a0 when it is a tuple)
codegenFun1 :: forall aenv a b. Elt a => Gamma aenv -> DelayedOpenFun () aenv (a -> b) -> (Fragment, Gamma aenv)
codegenFun1 g (Lam (Body b)) = close g (expr b (Empty `Push` argument "x" (eltTypeNames (undefined :: a))))
codegenFun1 _ _              = error "codegenFun1: expected a unary function"

-- | \x y -> body: the `combine` fragment of folds, scans and permute.  The new value is x (IndexSpace.hs:207).
codegenFun2 :: forall aenv a b c. (Elt a, Elt b) => Gamma aenv -> DelayedOpenFun () aenv (a -> b -> c) -> (Fragment, Gamma aenv)
codegenFun2 g (Lam (Lam (Body b))) =
  close g (expr b (Empty `Push` argument "x" (eltTypeNames (undefined :: a)) `Push` argument "y" (eltTypeNames (undefined :: b))))
codegenFun2 _ _ = error "codegenFun2: expected a binary function"

-- | a function of an index of the result, over the linear index `ix` the map family's kernels count in: the
-- argument is `ix` taken apart by the result's extents shOut_<d> (generate, backpermute: IndexSpace.hs:47-141)
codegenIndexFun :: forall aenv sh e. Shape sh => Gamma aenv -> DelayedOpenFun () aenv (sh -> e) -> (Fragment, Gamma aenv)
codegenIndexFun g (Lam (Body b)) = close g (expr b (Empty `Push` fromIndex (outExtents (Sugar.rank (undefined :: sh))) "ix"))
codegenIndexFun _ _              = error "codegenIndexFun: expected a unary function"

-- | a source array read through an index function of the result: backpermute's `get`
codegenIndexedBy :: forall aenv sh sh' e. (Shape sh, Shape sh', Elt e)
                 => Gamma aenv -> DelayedOpenFun () aenv (sh' -> sh) -> DelayedOpenAcc aenv (Array sh e) -> (Fragment, Gamma aenv)
codegenIndexedBy g (Lam (Body p)) a = close g $ do
  (b1, ix) <- expr p (Empty `Push` fromIndex (outExtents (Sugar.rank (undefined :: sh'))) "ix")
  (b2, vs) <- expr (Index a (Var ZeroIdx)) (Empty `Push` ix)
  return (b1 ++ b2, vs)
codegenIndexedBy _ _ _ = error "codegenIndexedBy: expected a unary function"

-- | the extents of the result as the kernels name them, outermost first
outExtents :: Int -> [String]
outExtents r = [ "shOut_" ++ show d | d <- reverse [0 .. r - 1] ]

-- | a stencil's function over its taps: t0, t1, ... in the order the stencil pattern lists them, flattened left to
-- right (u0, ... for the second source of a stencil2).  `sources` gives, per source, the name of its taps, how
-- many there are and how many components an element has: a tap of a source of tuples is a struct of its
-- components, t<k>.a<m-1> .. t<k>.a0 (include/acc_hip.h, stencil_in_type)
codegenStencilFun :: Gamma aenv -> [(String, Int, Int)] -> DelayedOpenFun () aenv f -> (Fragment, Gamma aenv)
codegenStencilFun g sources f = close g (go f sources Empty)
  where
    go :: DelayedOpenFun env aenv t -> [(String, Int, Int)] -> Val env -> Gen aenv ([String], [String])
    go (Body b) []                     env = expr b env
    go (Lam l)  ((name, n, m) : rest)  env = go l rest (env `Push` concat [ tap name k m | k <- [0 .. n - 1] ])
    go _        _                      _   = error "codegenStencilFun: one argument per source"
    tap name k 1 = [ name ++ show k ]
    tap name k m = [ name ++ show k ++ ".a" ++ show c | c <- reverse [0 .. m - 1] ]

-- | the value a constant boundary condition gives outside the source, as acc_skel_desc wants it: one literal per
-- component, "v<n-1>, ..., v0" (Stencil/Extra.hs:112-116)
codegenBoundary :: forall e. Elt e => e -> Boundary (Sugar.EltRepr e) -> Maybe String
codegenBoundary _ (Constant c) = Just (intercalate ", " (constants (eltType (undefined :: e)) c))
codegenBoundary _ _            = Nothing

argument :: String -> [String] -> [String]
argument name [_] = [name]
argument name ts  = [ name ++ ".a" ++ show k | k <- reverse [0 .. length ts - 1] ]

close :: Gamma aenv -> Gen aenv ([String], [String]) -> (Fragment, Gamma aenv)
close g m = let ((binds, comps), (g', _)) = runState m (g, 0) in (Fragment binds comps, g')

-- the statements an expression needs run before it, and its components
expr :: forall env aenv t. DelayedOpenExp env aenv t -> Val env -> Gen aenv ([String], [String])
expr e env = case e of
  Var ix                -> pure' (prj ix env)
  Const c               -> pure' (constants (eltType (undefined :: t)) c)
  PrimConst c           -> pure' [primConst c]
  Let bnd body          -> do
    (bs, vs) <- expr bnd env
    (decls, names) <- bindLocals vs
    (bs', vs') <- expr body (env `Push` names)
    return (bs ++ decls ++ bs', vs')
  Tuple tup             -> tuple tup
  Prj tix t             -> do
    (bs, vs) <- expr t env
    return (bs, projection tix (eltType (undefined :: t)) vs)
  Cond p t f            -> do
    (bp, [vp]) <- expr p env
    (bt, vt)   <- expr t env
    (bf, vf)   <- expr f env
    return (bp ++ bt ++ bf, [ "(" ++ vp ++ " ? " ++ a ++ " : " ++ b ++ ")" | (a, b) <- zip vt vf ])
  While p f x           -> while p f x
  PrimApp f x           -> do
    (bs, vs) <- expr x env
    return (bs, primApp f vs)
  IndexNil              -> pure' []
  IndexAny              -> pure' []
  IndexCons sh i        -> do
    (b1, v1) <- expr sh env
    (b2, v2) <- expr i env
    return (b1 ++ b2, v1 ++ v2)                                  -- outermost extent first, as shIn<k>_<d> are numbered
  IndexHead sh          -> do { (bs, vs) <- expr sh env; return (bs, [last vs]) }
  IndexTail sh          -> do { (bs, vs) <- expr sh env; return (bs, init vs) }
  ToIndex sh ix         -> do
    (b1, s) <- expr sh env
    (b2, i) <- expr ix env
    return (b1 ++ b2, [toIndex s i])
  FromIndex sh ix       -> do
    (b1, s)   <- expr sh env
    (b2, [i]) <- expr ix env
    return (b1 ++ b2, fromIndex s i)
  Shape acc             -> shapeOf acc
  ShapeSize sh          -> do { (bs, vs) <- expr sh env; return (bs, [product' vs]) }
  Intersect a b         -> do
    (b1, v1) <- expr a env
    (b2, v2) <- expr b env
    return (b1 ++ b2, [ "acc_min<Int64>(" ++ p ++ ", " ++ q ++ ")" | (p, q) <- zip v1 v2 ])
  Union a b             -> do
    (b1, v1) <- expr a env
    (b2, v2) <- expr b env
    return (b1 ++ b2, [ "acc_max<Int64>(" ++ p ++ ", " ++ q ++ ")" | (p, q) <- zip v1 v2 ])
  Index acc ix          -> do
    (bs, i) <- expr ix env
    (b2, s) <- shapeOf acc
    indexArray acc (bs ++ b2) (toIndex s i)
  LinearIndex acc ix    -> do
    (bs, [i]) <- expr ix env
    indexArray acc bs i
  IndexSlice{}          -> unsupported "IndexSlice"
  IndexFull{}           -> unsupported "IndexFull"
  Foreign{}             -> unsupported "Foreign"
  where
    pure' vs = return ([], vs)
    unsupported what = error ("Data.Array.Accelerate.HIP.CodeGen: " ++ what ++ " in a scalar expression is not generated")

    tuple :: Tuple (DelayedOpenExp env aenv) s -> Gen aenv ([String], [String])
    tuple NilTup          = pure' []
    tuple (SnocTup tup x) = do
      (b1, v1) <- tuple tup
      (b2, v2) <- expr x env
      return (b1 ++ b2, v1 ++ v2)

    -- do-while over local variables, bound ahead of the expression that uses the result
    while p f x = do
      (bx, vx)   <- expr x env
      names      <- mapM (const fresh) vx
      (bp, [vp]) <- funOver p names
      (bf, vf)   <- funOver f names
      let inits  = [ "auto " ++ n ++ " = " ++ v ++ ";" | (n, v) <- zip names vx ]
          steps  = [ "const auto " ++ n ++ "_next = " ++ v ++ ";" | (n, v) <- zip names vf ]
          copies = [ n ++ " = " ++ n ++ "_next;" | n <- names ]
          loop   = "for (;;) { " ++ unwords bp ++ " if (!(" ++ vp ++ ")) break; " ++ unwords (bf ++ steps ++ copies) ++ " }"
      return (bx ++ inits ++ [loop], names)

    funOver :: DelayedOpenFun env aenv (a -> b) -> [String] -> Gen aenv ([String], [String])
    funOver (Lam (Body b)) names = expr b (env `Push` names)
    funOver _              _     = error "while: expected a unary function"


-- Arrays inside fragments
-- ------------------------

-- the extents of an array variable are kernel parameters (CodeGen/Base.hs:69-89); those of a delayed array are an
-- expression, closed over the scalar environment: it is generated in the empty one
shapeOf :: forall aenv sh e. (Shape sh, Elt e) => DelayedOpenAcc aenv (Array sh e) -> Gen aenv ([String], [String])
shapeOf (Manifest (Avar ix)) = do
  k <- slotOf ix
  let r = Sugar.rank (undefined :: sh)
  return ([], [ "shIn" ++ show k ++ "_" ++ show d | d <- reverse [0 .. r - 1] ])
shapeOf Delayed{ extentD = sh } = expr sh Empty
shapeOf _                       = error "shape of an array that is neither a variable nor delayed"

-- reading an array inside a scalar function: a gather, left to the caches (no non-temporal hint)
indexArray :: forall aenv sh e. (Shape sh, Elt e) => DelayedOpenAcc aenv (Array sh e) -> [String] -> String -> Gen aenv ([String], [String])
indexArray (Manifest (Avar ix)) bs i = do
  k <- slotOf ix
  let n = length (eltTypeNames (undefined :: e))
  return (bs, [ "arrIn" ++ show k ++ "_" ++ show c ++ "[" ++ i ++ "]" | c <- reverse [0 .. n - 1] ])
indexArray Delayed{ linearIndexD = Lam (Body b) } bs i = do
  (bs', vs) <- expr b (Empty `Push` [i])
  return (bs ++ bs', vs)
indexArray _ _ _ = error "index into an array that is neither a variable nor delayed"

-- the operand of a skeleton at linear index `ix`.  A manifest array consumed in index order is read with a
-- non-temporal load, so that it does not evict what IS reused (gathered vectors, small tables) from the L2.
operandAt :: forall aenv sh e. (Shape sh, Elt e) => DelayedOpenAcc aenv (Array sh e) -> Gen aenv ([String], [String])
operandAt (Manifest (Avar ix)) = do
  k <- slotOf ix
  let n = length (eltTypeNames (undefined :: e))
  return ([], [ "acc_stream(arrIn" ++ show k ++ "_" ++ show c ++ ", ix)" | c <- reverse [0 .. n - 1] ])
operandAt Delayed{ linearIndexD = Lam (Body b) } = expr b (Empty `Push` ["ix"])
operandAt _ = error "the operand of a skeleton is an array variable or a delayed array"

-- the operand of a skeleton whose extents may differ from the result's (zipWith, whose result covers the
-- intersection): `ix` taken apart by the result's extents and put together again over the operand's own
operandThrough :: forall aenv sh e. (Shape sh, Elt e) => DelayedOpenAcc aenv (Array sh e) -> Gen aenv ([String], [String])
operandThrough a
  | Sugar.rank (undefined :: sh) <= 1 = operandAt a             -- the linear index of the result IS the operand's
  | otherwise                         = do
      (bs, sh) <- shapeOf a
      indexArray a bs (toIndex sh (fromIndex (outExtents (Sugar.rank (undefined :: sh))) "ix"))

-- every component bound to a local once, so that a value used twice is computed once (CodeGen/Monad.hs `bind`)
bindLocals :: [String] -> Gen aenv ([String], [String])
bindLocals vs = do
  names <- mapM (const fresh) vs
  return ([ "const auto " ++ n ++ " = " ++ v ++ ";" | (n, v) <- zip names vs ], names)


-- | a delayed (or manifest) array as the `get` fragment of a consumer: its element at linear index `ix`
codegenDelayed :: forall aenv sh e. (Shape sh, Elt e) => Gamma aenv -> DelayedOpenAcc aenv (Array sh e) -> (Fragment, Gamma aenv)
codegenDelayed g a = close g (operandAt a)

-- | map f a as one `get`: the operand's element at `ix` bound to the function's argument (Mapping.hs:39-78)
codegenMap :: forall aenv sh a b. (Shape sh, Elt a)
           => Gamma aenv -> DelayedOpenFun () aenv (a -> b) -> DelayedOpenAcc aenv (Array sh a) -> (Fragment, Gamma aenv)
codegenMap g (Lam (Body f)) a = close g $ do
  (b1, xs) <- operandAt a
  (b2, ns) <- bindLocals xs
  (b3, r)  <- expr f (Empty `Push` ns)
  return (b1 ++ b2 ++ b3, r)
codegenMap _ _ _ = error "codegenMap: expected a unary function"

-- | zipWith f a b as one `get` over the result's index space, the intersection of the operands' extents
codegenZipWith :: forall aenv sh a b c. (Shape sh, Elt a, Elt b)
               => Gamma aenv -> DelayedOpenFun () aenv (a -> b -> c)
               -> DelayedOpenAcc aenv (Array sh a) -> DelayedOpenAcc aenv (Array sh b) -> (Fragment, Gamma aenv)
codegenZipWith g (Lam (Lam (Body f))) a b = close g $ do
  (b1, xs) <- operandThrough a
  (b2, ys) <- operandThrough b
  (b3, nx) <- bindLocals xs
  (b4, ny) <- bindLocals ys
  (b5, r)  <- expr f (Empty `Push` nx `Push` ny)
  return (b1 ++ b2 ++ b3 ++ b4 ++ b5, r)
codegenZipWith _ _ _ _ = error "codegenZipWith: expected a binary function"

-- | permute's index function as the linear target index of source element `ix`, ACC_IGNORE for `ignore`
-- (IndexSpace.hs:160-303; `ignore` is the index whose every component is -1).  `ix` is taken apart by the
-- extents of the source, the target index put together over those of the result, shOut_<d>
codegenPermutation :: forall aenv sh sh' e. (Shape sh, Shape sh', Elt e)
                   => Gamma aenv -> DelayedOpenAcc aenv (Array sh e) -> DelayedOpenFun () aenv (sh -> sh') -> (Fragment, Gamma aenv)
codegenPermutation g a (Lam (Body b)) = close g $ do
  (b0, shIn)   <- shapeOf a
  (bs, target) <- expr b (Empty `Push` fromIndex shIn "ix")
  let shOut   = outExtents (Sugar.rank (undefined :: sh'))
      ignored = intercalate " && " [ "(" ++ t ++ ") == -1" | t <- target ]
  return (b0 ++ bs, [ if null target then "0" else "((" ++ ignored ++ ") ? ACC_IGNORE : " ++ toIndex shOut target ++ ")" ])
codegenPermutation _ _ _ = error "codegenPermutation: expected a unary function"


-- Index arithmetic (row-major, outermost extent first)
-- ----------------------------------------------------

toIndex :: [String] -> [String] -> String
toIndex sh ix = foldl (\acc (s, i) -> "(" ++ acc ++ " * " ++ s ++ " + " ++ i ++ ")") "((Int64)0)" (zip sh ix)

-- the device header's acc_from_index takes an index into fewer than 2^31 elements apart in 32 bits (the extents are
-- kernel parameters here, not literals: a 64-bit division by one of them is a hundred instructions); the compiler
-- makes one decomposition of the components' identical calls
fromIndex :: [String] -> String -> [String]
fromIndex []  _ = []
fromIndex [_] i = [i]
fromIndex sh  i = [ "acc_from_index<" ++ show n ++ ">({" ++ intercalate ", " [ "(Int64)(" ++ s ++ ")" | s <- sh ] ++ "}, " ++ i ++ ").i[" ++ show d ++ "]" | d <- [0 .. n - 1] ]
  where
    n = length sh

product' :: [String] -> String
product' [] = "((Int64)1)"
product' xs = "(" ++ intercalate " * " xs ++ ")"


-- Constants and primitives
-- ------------------------

constants :: TupleType t -> t -> [String]
constants UnitTuple         ()     = []
constants (SingleTuple t)   c      = [literal t c]
constants (PairTuple t1 t2) (a, b) = constants t1 a ++ constants t2 b

literal :: ScalarType t -> t -> String
literal t c = case t of
  NumScalarType (IntegralNumType it) | IntegralDict <- integralDict it -> "((" ++ cTypeOf t ++ ")" ++ show (toInteger c) ++ "LL)"
  NumScalarType (FloatingNumType ft) | FloatingDict <- floatingDict ft -> float (cTypeOf t) (realToFrac c :: Double)
  NonNumScalarType TypeBool{}                                          -> if c then "((Word8)1)" else "((Word8)0)"
  NonNumScalarType TypeChar{}                                          -> "((Word32)" ++ show (fromEnum c) ++ ")"
  NonNumScalarType _                                                   -> error "literal: C character types"
  where
    float ty v
      | isNaN v      = "((" ++ ty ++ ")__builtin_nan(\"\"))"
      | isInfinite v = (if v < 0 then "(-" else "(") ++ "__builtin_inf" ++ (if ty == "float" then "f" else "") ++ "())"
      | otherwise    = "((" ++ ty ++ ")" ++ show v ++ ")"

primConst :: PrimConst t -> String
primConst (PrimMinBound (IntegralBoundedType t)) | IntegralDict <- integralDict t = literal (NumScalarType (IntegralNumType t)) minBound
primConst (PrimMaxBound (IntegralBoundedType t)) | IntegralDict <- integralDict t = literal (NumScalarType (IntegralNumType t)) maxBound
primConst (PrimMinBound (NonNumBoundedType t))   | NonNumDict   <- nonNumDict t   = literal (NonNumScalarType t) minBound
primConst (PrimMaxBound (NonNumBoundedType t))   | NonNumDict   <- nonNumDict t   = literal (NonNumScalarType t) maxBound
primConst (PrimPi t)                             = "((" ++ cTypeOf (NumScalarType (FloatingNumType t)) ++ ")3.14159265358979323846)"

-- | every PrimFun of CodeGen.hs:406-476 as an operator or a call into csrc/device/acc_prim.h.  Operators are
-- parenthesised and cast to the result type, so that a narrow type wraps as Haskell's does.
primApp :: forall a r. (Elt a, Elt r) => PrimFun (a -> r) -> [String] -> [String]
primApp f args = [ case f of
  PrimAdd{}            -> binary "+"
  PrimSub{}            -> binary "-"
  PrimMul{}            -> binary "*"
  PrimNeg{}            -> cast ("-" ++ a)
  PrimAbs{}            -> call "acc_abs"
  PrimSig{}            -> call "acc_signum"
  PrimQuot{}           -> call "acc_quot"
  PrimRem{}            -> call "acc_rem"
  PrimIDiv{}           -> call "acc_idiv"
  PrimMod{}            -> call "acc_imod"
  PrimBAnd{}           -> binary "&"
  PrimBOr{}            -> binary "|"
  PrimBXor{}           -> binary "^"
  PrimBNot{}           -> cast ("~" ++ a)
  PrimBShiftL{}        -> call "acc_shift_l"
  PrimBShiftR{}        -> call "acc_shift_r"
  PrimBRotateL{}       -> call "acc_rotate_l"
  PrimBRotateR{}       -> call "acc_rotate_r"
  PrimFDiv{}           -> binary "/"
  PrimRecip{}          -> call "acc_recip"
  PrimSin{}            -> call "acc_sin"
  PrimCos{}            -> call "acc_cos"
  PrimTan{}            -> call "acc_tan"
  PrimAsin{}           -> call "acc_asin"
  PrimAcos{}           -> call "acc_acos"
  PrimAtan{}           -> call "acc_atan"
  PrimSinh{}           -> call "acc_sinh"
  PrimCosh{}           -> call "acc_cosh"
  PrimTanh{}           -> call "acc_tanh"
  PrimAsinh{}          -> call "acc_asinh"
  PrimAcosh{}          -> call "acc_acosh"
  PrimAtanh{}          -> call "acc_atanh"
  PrimExpFloating{}    -> call "acc_exp"
  PrimSqrt{}           -> call "acc_sqrt"
  PrimLog{}            -> call "acc_log"
  PrimFPow{}           -> call "acc_pow"
  PrimLogBase{}        -> call "acc_log_base"
  PrimAtan2{}          -> call "acc_atan2"
  PrimTruncate{}       -> convert "acc_truncate"
  PrimRound{}          -> convert "acc_round"
  PrimFloor{}          -> convert "acc_floor"
  PrimCeiling{}        -> convert "acc_ceiling"
  PrimIsNaN{}          -> call "acc_is_nan"
  PrimLt{}             -> compare' "<"
  PrimGt{}             -> compare' ">"
  PrimLtEq{}           -> compare' "<="
  PrimGtEq{}           -> compare' ">="
  PrimEq{}             -> compare' "=="
  PrimNEq{}            -> compare' "!="
  PrimMax{}            -> call "acc_pmax"
  PrimMin{}            -> call "acc_pmin"
  PrimLAnd             -> compare' "&&"
  PrimLOr              -> compare' "||"
  PrimLNot             -> "((Word8)(!" ++ a ++ "))"
  PrimOrd              -> call "acc_ord"
  PrimChr              -> call "acc_chr"
  PrimBoolToInt        -> call "acc_bool_to_int"
  PrimFromIntegral{}   -> convert "acc_from_integral"
  PrimQuotRem{}        -> error "quotRem yields a pair: see pairs below"
  PrimDivMod{}         -> error "divMod yields a pair: see pairs below"
  ] `orPairs` pairs
  where
    a : rest       = args
    b              = case rest of { (v : _) -> v; [] -> a }
    [result]       = eltTypeNames (undefined :: r)
    cast e         = "((" ++ result ++ ")(" ++ e ++ "))"
    binary op      = cast (a ++ " " ++ op ++ " " ++ b)
    compare' op    = "((Word8)(" ++ a ++ " " ++ op ++ " " ++ b ++ "))"
    call fn        = fn ++ "(" ++ intercalate ", " args ++ ")"
    convert fn     = fn ++ "<" ++ result ++ ">(" ++ a ++ ")"
    -- the two primitives that yield a pair: both halves from one call each (the compiler merges them)
    pairs          = case f of
                       PrimQuotRem{} -> Just [ "acc_quot(" ++ a ++ ", " ++ b ++ ")", "acc_rem(" ++ a ++ ", " ++ b ++ ")" ]
                       PrimDivMod{}  -> Just [ "acc_idiv(" ++ a ++ ", " ++ b ++ ")", "acc_imod(" ++ a ++ ", " ++ b ++ ")" ]
                       _             -> Nothing
    orPairs single = maybe single id

-- | the components a tuple projection keeps: `tix` counts elements of the tuple from the right, each of which
-- may itself span several components
projection :: TupleIdx t e -> TupleType t' -> [String] -> [String]
projection tix ty vs = take width (drop skip vs)
  where
    widths        = elementWidths ty                                    -- left to right
    n             = length widths
    k             = n - 1 - tupleIdxToInt tix                           -- position from the left
    skip          = sum (take k widths)
    width         = widths !! k

elementWidths :: TupleType t -> [Int]
elementWidths UnitTuple         = []
elementWidths (PairTuple t1 t2) = elementWidths t1 ++ [componentCount t2]
elementWidths (SingleTuple _)   = [1]

componentCount :: TupleType t -> Int
componentCount UnitTuple         = 0
componentCount (SingleTuple _)   = 1
componentCount (PairTuple t1 t2) = componentCount t1 + componentCount t2

tupleIdxToInt :: TupleIdx t e -> Int
tupleIdxToInt ZeroTupIdx     = 0
tupleIdxToInt (SuccTupIdx i) = 1 + tupleIdxToInt i
