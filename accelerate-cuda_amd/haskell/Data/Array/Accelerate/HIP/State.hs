-- |
-- Module      : Data.Array.Accelerate.HIP.State
--
-- What an evaluation carries around: the library context of the device, the memory table every
-- array lives in, and the reservoir of streams.  The role of State.hs:60-132 and
-- Execute/Stream.hs:66-134; the kernel table and the persistent cache of State.hs:110-119 are
-- inside the library (`acc_skel_create` goes through its cache), and there is no context stack:
-- every entry point of libacchip makes the context's device current itself (State.hs:84-92).
--
-- UNCOMPILED: no GHC in the image this library is built and tested in.
--
module Data.Array.Accelerate.HIP.State (

  HIP, Env(..), evalHIP, hipContext, hipMemTable, withStream, createEnv, destroyEnv, defaultEnv,

) where

import Data.Array.Accelerate.HIP.FFI

import Control.Concurrent.MVar
import Control.Exception                                        ( bracket )
import Control.Monad.Reader
import Foreign
import System.IO.Unsafe                                         ( unsafePerformIO )


data Env = Env
  { envContext  :: !Context
  , envMemTable :: !MemTable
  , envStreams  :: !(MVar [Stream])               -- streams not in use: taken for an independent computation, put back after
  }

type HIP = ReaderT Env IO

evalHIP :: Env -> HIP a -> IO a
evalHIP = flip runReaderT

hipContext :: HIP Context
hipContext = asks envContext

hipMemTable :: HIP MemTable
hipMemTable = asks envMemTable

-- | a stream for one computation: one from the reservoir, or a new one (Execute/Stream.hs:66-74)
withStream :: (Stream -> HIP a) -> HIP a
withStream body = do
  env <- ask
  liftIO $ bracket (takeOne env) (\s -> modifyMVar_ (envStreams env) (return . (s :))) (\s -> evalHIP env (body s))
  where
    takeOne env = modifyMVar (envStreams env) $ \ss -> case ss of
      (s : rest) -> return (rest, s)
      []         -> do s <- alloca $ \p -> check (c_streamCreate (envContext env) p) >> peek p
                       return ([], s)

-- | Context.hs:73-84 `create`: a context on the given device with a memory table of its own (budget 0: the device decides)
createEnv :: Int -> IO Env
createEnv device = do
  check c_init
  drainCompilationsAtExit                           -- once per context is harmless: the second drain finds nothing to do
  ctx <- alloca $ \p -> check (c_contextCreate (fromIntegral device) p) >> peek p
  mt  <- alloca $ \p -> check (c_memtableCreate ctx 0 p) >> peek p
  Env ctx mt <$> newMVar []

-- | Context.hs:100-103 `destroy`
destroyEnv :: Env -> IO ()
destroyEnv env = do
  check (c_contextSync (envContext env))
  mapM_ (check . c_streamDestroy (envContext env)) =<< takeMVar (envStreams env)
  check (c_memtableDestroy (envMemTable env))
  check (c_contextDestroy (envContext env))

-- | CUDA.hs:205-206 `defaultContext`: device 0, made on first use
{-# NOINLINE defaultEnv #-}
defaultEnv :: Env
defaultEnv = unsafePerformIO (createEnv 0)
