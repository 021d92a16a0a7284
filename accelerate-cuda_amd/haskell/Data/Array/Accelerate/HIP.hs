{-# LANGUAGE BangPatterns #-}
-- |
-- Module      : Data.Array.Accelerate.HIP
--
-- The backend's front door, with the export list of Data.Array.Accelerate.CUDA
-- (CUDA.hs:184-200) under the same names, so that a program switches backends by
-- changing one import.  Everything below `run` is libacchip: `convertAcc` (sharing
-- recovery and fusion, from the accelerate package, unchanged), then
-- "Data.Array.Accelerate.HIP.Compile" (a skeleton instance per node) and
-- "Data.Array.Accelerate.HIP.Execute" (a driver call per node).
--
-- UNCOMPILED: no GHC in the image this library is built and tested in.  The Python
-- module accelerate_hip.py carries the same export list over the same C ABI and is what
-- the GPU tests drive.
--
module Data.Array.Accelerate.HIP (

  Arrays,

  -- * Synchronous execution
  run, run1, runN, stream, runWith, run1With, streamWith,
  streamOut, streamOutWith,

  -- * Asynchronous execution
  Async, wait, poll, cancel,
  runAsync, run1Async, runAsyncWith, run1AsyncWith,

  -- * Execution contexts
  Context, create, destroy,
  unsafeFree, unsafeFreeWith, performGC, performGCWith,

) where

import Data.Array.Accelerate.Trafo                              ( convertAccWith, convertAfunWith, Phase(..), phases )
import Data.Array.Accelerate.Smart                              ( Acc )
import Data.Array.Accelerate.Array.Sugar                       ( Arrays )
import Data.Array.Accelerate.Async                             ( Async, async, wait, poll, cancel )

import Data.Array.Accelerate.HIP.Compile
import Data.Array.Accelerate.HIP.Execute
import Data.Array.Accelerate.HIP.FFI                            ( check, c_memtableReclaim )
import Data.Array.Accelerate.HIP.State
import Data.Array.Accelerate.HIP.Array                          ( freeArrays, collectArrays )

import Control.Monad.Trans                                      ( liftIO )
import System.IO.Unsafe                                         ( unsafePerformIO )


-- | a device context with its memory table and streams (Context.hs:73-84)
type Context = Env

create :: Int -> IO Context
create = createEnv

destroy :: Context -> IO ()
destroy = destroyEnv

-- | CUDA.hs:209-216
run :: Arrays a => Acc a -> a
run = runWith defaultEnv

runWith :: Arrays a => Context -> Acc a -> a
runWith env a = unsafePerformIO (evaluate env a)

evaluate :: Arrays a => Context -> Acc a -> IO a
evaluate env a = evalHIP env $ do
  exec <- compileAcc (convertAccWith config a)
  r    <- executeAcc exec
  collectArrays r                                   -- Execute.hs:146-154: bring the results to the host

-- | CUDA.hs:318-333: partially applied, `run1 f` compiles once and every call only executes
run1 :: (Arrays a, Arrays b) => (Acc a -> Acc b) -> a -> b
run1 = run1With defaultEnv

run1With :: (Arrays a, Arrays b) => Context -> (Acc a -> Acc b) -> a -> b
run1With env f = \a -> unsafePerformIO (evalHIP env (executeAfun1 exec a >>= collectArrays))
  where
    !exec = unsafePerformIO (evalHIP env (compileAfun (convertAfunWith config f)))

-- | any number of array arguments; the kernels are built once, as for run1
runN :: (Arrays a, Arrays b) => (Acc a -> Acc b) -> a -> b
runN = run1

-- | CUDA.hs:345-349: one result per input, lazily; the kernels are those of the first
stream :: (Arrays a, Arrays b) => (Acc a -> Acc b) -> [a] -> [b]
stream = streamWith defaultEnv

streamWith :: (Arrays a, Arrays b) => Context -> (Acc a -> Acc b) -> [a] -> [b]
streamWith env f = map go
  where
    !go = run1With env f

-- | the results of a sequence of computations as a lazy list: an element is compiled, run and collected when it is
-- asked for, never the whole sequence at once.  The reference keeps its `streamOut` (CUDA.hs:349-372) commented out
-- together with the `Seq` language it ran (accelerate-1.0 has none); this is the part of it that does not need
-- one: the sequence is a list of array computations.
streamOut :: Arrays a => [Acc a] -> [a]
streamOut = streamOutWith defaultEnv

streamOutWith :: Arrays a => Context -> [Acc a] -> [a]
streamOutWith env = map (runWith env)

-- | CUDA.hs:256-333: the computation in a thread of its own; `wait`, `poll` and `cancel` from
-- Data.Array.Accelerate.Async.  The reference forks a BOUND thread, because a CUDA context belongs to an operating
-- system thread; every entry point of libacchip makes its context's device current itself, so any thread will do.
runAsync :: Arrays a => Acc a -> IO (Async a)
runAsync = runAsyncWith defaultEnv

runAsyncWith :: Arrays a => Context -> Acc a -> IO (Async a)
runAsyncWith env a = async (evaluate env a)

run1Async :: (Arrays a, Arrays b) => (Acc a -> Acc b) -> a -> IO (Async b)
run1Async = run1AsyncWith defaultEnv

run1AsyncWith :: (Arrays a, Arrays b) => Context -> (Acc a -> Acc b) -> a -> IO (Async b)
run1AsyncWith env f = \a -> async (return $! go a)
  where
    !go = run1With env f

-- | CUDA.hs:421-441: give the device copies of these arrays back now; return the table's pool of freed blocks
-- (and the scratch the skeleton drivers hold) to the device
unsafeFree :: Arrays a => a -> IO ()
unsafeFree = unsafeFreeWith defaultEnv

unsafeFreeWith :: Arrays a => Context -> a -> IO ()
unsafeFreeWith env = evalHIP env . freeArrays

performGC :: IO ()
performGC = performGCWith defaultEnv

performGCWith :: Context -> IO ()
performGCWith env = check (c_memtableReclaim (envMemTable env))

-- the front end's phases: sharing recovery and fusion on, as the reference has them (CUDA.hs:394-406)
config :: Phase
config = phases
