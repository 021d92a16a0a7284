{-# LANGUAGE GADTs, ScopedTypeVariables, ExistentialQuantification, BangPatterns #-}
-- |
-- Module      : Data.Array.Accelerate.HIP.Array
--
-- Accelerate arrays and their device copies: every primitive component of an array's payload
-- is an entry of the library's memory table (include/acc_hip.h, acc_memtable_*), keyed by the
-- address of its host storage.  The roles of Array/Data.hs:130-330 (mallocArray, useArray,
-- indexArray, peekArray, withDevicePtrs over every component), Array/Sugar.hs:40-45
-- (allocateArray) and Array/Prim.hs:177-192; the table itself -- reuse of freed blocks,
-- eviction under memory pressure, upload on first use -- is the library's (Array/Remote.hs and
-- the LRU table of the accelerate package).
--
-- UNCOMPILED: no GHC in the image this library is built and tested in.  Written against
-- accelerate-1.0's Data.Array.Accelerate.Array.Data (the AD_* constructors over UniqueArray)
-- and Data.Array.Accelerate.Lifetime.
--
-- A host array and its device copy: an array made by `use` is FROZEN in the table (the host
-- copy is authoritative; it is uploaded when a kernel first wants it and dropped without a
-- write-back when the device is full); an array a kernel produces is not (the device copy is
-- authoritative until `collectArrays` brings it to the host, and eviction writes it back).
--
module Data.Array.Accelerate.HIP.Array (

  SomeArray(..),
  allocateArray, useArray, useArrays, unitArray, reshapeArray, indexArray,
  withDevice, withArrays,
  collectArrays, freeArrays,

) where

import Data.Array.Accelerate.Array.Data
import Data.Array.Accelerate.Array.Unique                      ( UniqueArray(..) )
import Data.Array.Accelerate.Lifetime                          ( Lifetime, addFinalizer, unsafeGetValue, touchLifetime )
import Data.Array.Accelerate.Array.Sugar                       ( Array(..), Arrays(..), ArraysR(..), Shape, Elt, Scalar, Z(..), EltRepr )
import qualified Data.Array.Accelerate.Array.Sugar             as Sugar

import Data.Array.Accelerate.HIP.FFI
import Data.Array.Accelerate.HIP.State

import Control.Exception                                        ( finally )
import Control.Monad
import Control.Monad.Reader                                     ( ask )
import Control.Monad.Trans                                      ( liftIO )
import Foreign
import Foreign.C.Types


-- | an array of any extent and element type: what an array environment slot holds
data SomeArray = forall sh e. (Shape sh, Elt e) => SomeArray (Array sh e)


-- Components
-- ----------

-- | one primitive component of an array's payload: where its host storage is, how wide an element is, and the
-- lifetime that storage hangs on (the table's entry goes when it ends)
data Component = forall a. Component !(Ptr ()) !Int (Lifetime (ForeignPtr a))

-- | the components of a payload, component 0 first: the rightmost field of the (nested) pair representation is
-- component 0, as the generated code numbers arrIn<k>_<c> (CodeGen/Base.hs:344-357)
components :: ArrayEltR e -> ArrayData e -> [Component]
components ArrayEltRunit         _  = []
components (ArrayEltRpair r1 r2) ad = components r2 (sndArrayData ad) ++ components r1 (fstArrayData ad)
components ArrayEltRint     (AD_Int     ua) = [prim ua]
components ArrayEltRint8    (AD_Int8    ua) = [prim ua]
components ArrayEltRint16   (AD_Int16   ua) = [prim ua]
components ArrayEltRint32   (AD_Int32   ua) = [prim ua]
components ArrayEltRint64   (AD_Int64   ua) = [prim ua]
components ArrayEltRword    (AD_Word    ua) = [prim ua]
components ArrayEltRword8   (AD_Word8   ua) = [prim ua]
components ArrayEltRword16  (AD_Word16  ua) = [prim ua]
components ArrayEltRword32  (AD_Word32  ua) = [prim ua]
components ArrayEltRword64  (AD_Word64  ua) = [prim ua]
components ArrayEltRcshort  (AD_CShort  ua) = [prim ua]
components ArrayEltRcushort (AD_CUShort ua) = [prim ua]
components ArrayEltRcint    (AD_CInt    ua) = [prim ua]
components ArrayEltRcuint   (AD_CUInt   ua) = [prim ua]
components ArrayEltRclong   (AD_CLong   ua) = [prim ua]
components ArrayEltRculong  (AD_CULong  ua) = [prim ua]
components ArrayEltRcllong  (AD_CLLong  ua) = [prim ua]
components ArrayEltRcullong (AD_CULLong ua) = [prim ua]
components ArrayEltRfloat   (AD_Float   ua) = [prim ua]
components ArrayEltRdouble  (AD_Double  ua) = [prim ua]
components ArrayEltRcfloat  (AD_CFloat  ua) = [prim ua]
components ArrayEltRcdouble (AD_CDouble ua) = [prim ua]
components ArrayEltRbool    (AD_Bool    ua) = [prim ua]          -- a byte an element, on the host as on the device
components ArrayEltRchar    (AD_Char    ua) = [prim ua]          -- a code point in 32 bits
components ArrayEltRcchar   (AD_CChar   ua) = [prim ua]
components ArrayEltRcschar  (AD_CSChar  ua) = [prim ua]
components ArrayEltRcuchar  (AD_CUChar  ua) = [prim ua]

prim :: forall a. Storable a => UniqueArray a -> Component
prim ua = Component (castPtr (unsafeForeignPtrToPtr (unsafeGetValue lt))) (sizeOf (undefined :: a)) lt
  where lt = uniqueArrayData ua

componentsOf :: forall sh e. (Shape sh, Elt e) => Array sh e -> [Component]
componentsOf (Array _ adata) = components arrayElt adata

elements :: (Shape sh, Elt e) => Array sh e -> Int
elements = Sugar.size . Sugar.shape

-- the key of a component in the memory table: the address of its host storage.  The entry is removed by a
-- finalizer of that storage's lifetime, which runs before the storage is released, so an address is never in the
-- table for two arrays at once
keyOf :: Component -> Word64
keyOf (Component p _ _) = fromIntegral (ptrToWordPtr p)

keepAlive :: Component -> IO ()
keepAlive (Component _ _ lt) = touchLifetime lt


-- Allocation
-- ----------

-- | enter every component of the array into the memory table.  Nothing happens to one that is there already: an
-- array `use`d twice is uploaded once (Array/Prim.hs:177-192).  An empty array has no entries.
mallocArray :: (Shape sh, Elt e) => Bool -> Array sh e -> HIP ()
mallocArray frozen arr = do
  mt <- hipMemTable
  let n = elements arr
  liftIO $ forM_ (componentsOf arr) $ \c@(Component p width lt) -> when (n > 0) $ do
    isNew <- alloca $ \pnew -> do
      check (c_memtableMalloc mt (keyOf c) p (fromIntegral (n * width)) (if frozen then 1 else 0) pnew)
      peek pnew
    when (isNew /= (0 :: CInt)) $
      addFinalizer lt (void (c_memtableFree mt (keyOf c)))       -- Array/Remote.hs:160-170: the host array is gone

-- | a new array on the host and, for the kernels to fill, on the device (Array/Sugar.hs:40-45)
allocateArray :: (Shape sh, Elt e) => sh -> HIP (Array sh e)
allocateArray sh = do
  arr <- liftIO (Sugar.allocateArray sh)
  mallocArray False arr
  return arr

-- | an array whose data is on the host: entered frozen, uploaded on the stream that first acquires it
-- (Array/Data.hs:175-195 `useArray`, which uploads at once)
useArray :: (Shape sh, Elt e) => Array sh e -> HIP ()
useArray = mallocArray True

-- | every array of a (nested) tuple of arrays (Execute.hs:146-154)
useArrays :: forall arrs. Arrays arrs => arrs -> HIP ()
useArrays arrs = go (arrays (undefined :: arrs)) (fromArr arrs)
  where
    go :: ArraysR a -> a -> HIP ()
    go ArraysRunit         ()       = return ()
    go ArraysRarray        arr      = useArray arr
    go (ArraysRpair r1 r2) (a1, a2) = go r1 a1 >> go r2 a2

-- | `unit e`: a one-element array holding a value the host computed (Execute.hs:209)
unitArray :: Elt e => e -> HIP (Scalar e)
unitArray e = do
  let arr = Sugar.fromList Z [e]
  useArray arr
  return arr

-- | the same storage under other extents of the same size: the table's entries hang on the storage, not on the
-- extents, so nothing moves (Execute.hs:211-214)
reshapeArray :: (Shape sh, Shape sh', Elt e) => sh -> Array sh' e -> Array sh e
reshapeArray sh (Array _ adata) = Array (Sugar.fromElt sh) adata


-- Device pointers
-- ---------------

-- | the array as the kernels see it, resident on the device for as long as the continuation runs: every component
-- is acquired (uploaded on `stream` first where the device holds no copy of it) and released on `stream`
-- afterwards, so that its block is not handed on before the work enqueued here has run (Array/Remote.hs:113-135
-- `withRemote`; Array/Data.hs:300-330 `withDevicePtrs`)
withDevice :: (Shape sh, Elt e) => Stream -> Array sh e -> (AccArray -> HIP r) -> HIP r
withDevice stream arr body = do
  env <- ask
  let mt     = envMemTable env
      comps  = if elements arr > 0 then componentsOf arr else []
      extent = map fromIntegral (reverse (Sugar.shapeToList (Sugar.shape arr))) :: [Int64]       -- outermost first
      acquire c = alloca $ \pp -> check (c_memtableAcquire mt (keyOf c) stream pp) >> peek pp
      release c = check (c_memtableRelease mt (keyOf c) stream) >> keepAlive c
      go []       ptrs = evalHIP env (body (AccArray extent (if null comps then nulls else reverse ptrs)))
      go (c : cs) ptrs = do { p <- acquire c; go cs (p : ptrs) `finally` release c }
      nulls  = map (const 0) (componentsOf arr)                    -- an empty array: no storage, no entries
  liftIO (go comps [])

-- | the same for the arrays of a kernel's environment, in slot order
withArrays :: Stream -> [SomeArray] -> ([AccArray] -> HIP r) -> HIP r
withArrays _      []                    body = body []
withArrays stream (SomeArray a : rest) body = withDevice stream a $ \d -> withArrays stream rest (body . (d :))


-- Host copies
-- -----------

-- | bring the device copy of every component to the host and wait for it (Array/Data.hs:230-250 `peekArray`;
-- CUDA.hs:383-389 `collect`).  The copy of a `use`d array, whose host storage already holds the data, moves the
-- same bytes again and changes nothing.
peekArray :: (Shape sh, Elt e) => Stream -> Array sh e -> HIP ()
peekArray stream arr = do
  ctx <- hipContext
  let n = elements arr
  withDevice stream arr $ \(AccArray _ ptrs) -> liftIO $
    forM_ (zip (componentsOf arr) ptrs) $ \(Component p width _, d) -> when (n > 0) $
      check (c_memcpyD2hAsync ctx p d (fromIntegral (n * width)) stream)
  liftIO $ check (c_streamSync ctx stream)

-- | the results of a computation, on the host
collectArrays :: forall arrs. Arrays arrs => arrs -> HIP arrs
collectArrays arrs = withStream $ \stream -> do
  go stream (arrays (undefined :: arrs)) (fromArr arrs)
  return arrs
  where
    go :: Stream -> ArraysR a -> a -> HIP ()
    go _ ArraysRunit         ()       = return ()
    go s ArraysRarray        arr      = peekArray s arr
    go s (ArraysRpair r1 r2) (a1, a2) = go s r1 a1 >> go s r2 a2

-- | one element of an array that lives on the device, for scalar code on the host (`arr ! ix` in a shape or a
-- condition: Array/Data.hs:215-228 `indexArray`).  The element's bytes are copied into their place in the host
-- storage, which they equal from then on, and read from there.
indexArray :: (Shape sh, Elt e) => Stream -> Array sh e -> Int -> HIP e
indexArray stream arr@(Array _ adata) i = do
  ctx <- hipContext
  withDevice stream arr $ \(AccArray _ ptrs) -> liftIO $ do
    forM_ (zip (componentsOf arr) ptrs) $ \(Component p width _, d) ->
      check (c_memcpyD2hAsync ctx (p `plusPtr` (i * width)) (d + fromIntegral (i * width)) (fromIntegral width) stream)
    check (c_streamSync ctx stream)
  return $! Sugar.toElt (unsafeIndexArrayData adata i)

-- | give the device copies back now instead of when the host arrays are collected (CUDA.hs:421-441 `unsafeFree`).
-- The arrays must not be used by a computation again.
freeArrays :: forall arrs. Arrays arrs => arrs -> HIP ()
freeArrays arrs = go (arrays (undefined :: arrs)) (fromArr arrs)
  where
    go :: ArraysR a -> a -> HIP ()
    go ArraysRunit         ()       = return ()
    go (ArraysRpair r1 r2) (a1, a2) = go r1 a1 >> go r2 a2
    go ArraysRarray        arr      = do
      mt <- hipMemTable
      liftIO $ forM_ (componentsOf arr) $ \c -> when (elements arr > 0) $
        check (c_memtableFree mt (keyOf c))                                -- a key that is not there: nothing to do
