{-# LANGUAGE ForeignFunctionInterface #-}
-- | Raw bindings to the host-layer C ABI (include/hordead_host.h,
-- libhordead_host.so).  One import per entry point; cheap metadata calls are
-- @unsafe@, everything that can enqueue or wait is @safe@.  Device values are
-- owned by 'ForeignPtr's whose finalizer is 'hh_free'.
--
-- Not compiled in the build environment of this repository (no GHC there);
-- it is the binding a maintainer adds next to
-- src/HordeAd/Core/CarriersConcrete.hs.
module HordeAd.Gpu.Foreign
  ( Ctx, Val, Ix, ValPtr, IxPtr
  , withGpu, theCtx, check
  , Graph, c_hh_capture_begin, c_hh_capture_end, c_hh_graph_launch, c_hh_graph_free, c_hh_force, c_hh_overwrite
  , c_hh_upload, c_hh_download, c_hh_constant, c_hh_val_rank, c_hh_val_shape
  , c_hh_ewise1, c_hh_ewise2, c_hh_compare, c_hh_compare_all, c_hh_select
  , c_hh_convert, c_hh_tssumN, c_hh_tssum0, c_hh_tsdot0, c_hh_tsdot1In
  , c_hh_tsmatvecmul, c_hh_tsmatmul2, c_hh_tsreplicateN, c_hh_tsappend
  , c_hh_tsslice, c_hh_tsreverse, c_hh_tstranspose, c_hh_tsreshape
  , c_hh_tsindex, c_hh_tsargminmax, c_hh_tsiota
  , c_hh_ix_var, c_hh_ix_const, c_hh_ix_lift, c_hh_ix_op1, c_hh_ix_op2
  , c_hh_ix_compare, c_hh_ix_select, c_hh_ix_convert, c_hh_ix_index0
  , c_hh_ix_argminmax, c_hh_tsgather, c_hh_tsscatter
  , c_hh_ix_from_val, c_hh_ix_to_val, c_hh_tconvert, c_hh_tprimalPart
  , p_hh_free, p_hh_ix_free
  ) where

import Control.Exception (ErrorCall (..), throwIO)
import Control.Monad (when)
import Data.Int (Int64)
import Data.IORef
import Foreign
import Foreign.C
import System.IO.Unsafe (unsafePerformIO)

data Ctx
data Val
data Ix
type ValPtr = ForeignPtr Val
type IxPtr = ForeignPtr Ix

foreign import ccall safe "hh_create_gpu" c_hh_create_gpu :: CInt -> Ptr (Ptr Ctx) -> IO CInt
foreign import ccall safe "hh_destroy" c_hh_destroy :: Ptr Ctx -> IO CInt
foreign import ccall unsafe "hh_last_error" c_hh_last_error :: Ptr Ctx -> IO CString
foreign import ccall safe "hh_upload" c_hh_upload
  :: Ptr Ctx -> CInt -> CInt -> Ptr Int64 -> Ptr () -> CInt -> Ptr (Ptr Val) -> IO CInt
foreign import ccall safe "hh_download" c_hh_download :: Ptr Ctx -> Ptr Val -> Ptr () -> IO CInt

-- One gradient program recorded as a device graph and launched per batch
-- (include/hordead_host.h, "evaluating one gradient program many times").
data Graph
foreign import ccall safe "hh_capture_begin" c_hh_capture_begin :: Ptr Ctx -> IO CInt
foreign import ccall safe "hh_capture_end" c_hh_capture_end :: Ptr Ctx -> Ptr (Ptr Graph) -> IO CInt
foreign import ccall safe "hh_graph_launch" c_hh_graph_launch :: Ptr Ctx -> Ptr Graph -> IO CInt
foreign import ccall safe "hh_graph_free" c_hh_graph_free :: Ptr Ctx -> Ptr Graph -> IO CInt
foreign import ccall safe "hh_force" c_hh_force :: Ptr Ctx -> Ptr Val -> IO CInt
foreign import ccall safe "hh_overwrite" c_hh_overwrite :: Ptr Ctx -> Ptr Val -> Ptr () -> IO CInt
foreign import ccall safe "hh_constant" c_hh_constant
  :: Ptr Ctx -> CInt -> CDouble -> CInt -> Ptr Int64 -> Ptr (Ptr Val) -> IO CInt
foreign import ccall unsafe "hh_val_rank" c_hh_val_rank :: Ptr Val -> IO CInt
foreign import ccall unsafe "hh_val_shape" c_hh_val_shape :: Ptr Val -> Ptr Int64 -> IO CInt
foreign import ccall unsafe "&hh_free" p_hh_free :: FunPtr (Ptr Val -> IO ())
foreign import ccall unsafe "&hh_ix_free" p_hh_ix_free :: FunPtr (Ptr Ix -> IO ())

foreign import ccall safe "hh_ewise1" c_hh_ewise1 :: Ptr Ctx -> CInt -> Ptr Val -> Ptr (Ptr Val) -> IO CInt
foreign import ccall safe "hh_ewise2" c_hh_ewise2 :: Ptr Ctx -> CInt -> Ptr Val -> Ptr Val -> Ptr (Ptr Val) -> IO CInt
foreign import ccall safe "hh_compare" c_hh_compare :: Ptr Ctx -> CInt -> Ptr Val -> Ptr Val -> Ptr (Ptr Val) -> IO CInt
foreign import ccall safe "hh_compare_all" c_hh_compare_all :: Ptr Ctx -> CInt -> Ptr Val -> Ptr Val -> Ptr CInt -> IO CInt
foreign import ccall safe "hh_select" c_hh_select :: Ptr Ctx -> Ptr Val -> Ptr Val -> Ptr Val -> Ptr (Ptr Val) -> IO CInt
foreign import ccall safe "hh_convert" c_hh_convert :: Ptr Ctx -> Ptr Val -> CInt -> CInt -> Ptr (Ptr Val) -> IO CInt
foreign import ccall safe "hh_tssumN" c_hh_tssumN :: Ptr Ctx -> Ptr Val -> CInt -> Ptr (Ptr Val) -> IO CInt
foreign import ccall safe "hh_tssum0" c_hh_tssum0 :: Ptr Ctx -> Ptr Val -> Ptr (Ptr Val) -> IO CInt
foreign import ccall safe "hh_tsdot0" c_hh_tsdot0 :: Ptr Ctx -> Ptr Val -> Ptr Val -> Ptr (Ptr Val) -> IO CInt
foreign import ccall safe "hh_tsdot1In" c_hh_tsdot1In :: Ptr Ctx -> Ptr Val -> Ptr Val -> Ptr (Ptr Val) -> IO CInt
foreign import ccall safe "hh_tsmatvecmul" c_hh_tsmatvecmul :: Ptr Ctx -> Ptr Val -> Ptr Val -> Ptr (Ptr Val) -> IO CInt
foreign import ccall safe "hh_tsmatmul2" c_hh_tsmatmul2 :: Ptr Ctx -> Ptr Val -> Ptr Val -> Ptr (Ptr Val) -> IO CInt
foreign import ccall safe "hh_tsreplicateN" c_hh_tsreplicateN :: Ptr Ctx -> Ptr Val -> CInt -> Ptr Int64 -> Ptr (Ptr Val) -> IO CInt
foreign import ccall safe "hh_tsappend" c_hh_tsappend :: Ptr Ctx -> Ptr Val -> Ptr Val -> Ptr (Ptr Val) -> IO CInt
foreign import ccall safe "hh_tsslice" c_hh_tsslice :: Ptr Ctx -> Ptr Val -> Int64 -> Int64 -> Ptr (Ptr Val) -> IO CInt
foreign import ccall safe "hh_tsreverse" c_hh_tsreverse :: Ptr Ctx -> Ptr Val -> Ptr (Ptr Val) -> IO CInt
foreign import ccall safe "hh_tstranspose" c_hh_tstranspose :: Ptr Ctx -> Ptr Val -> CInt -> Ptr CInt -> Ptr (Ptr Val) -> IO CInt
foreign import ccall safe "hh_tsreshape" c_hh_tsreshape :: Ptr Ctx -> Ptr Val -> CInt -> Ptr Int64 -> Ptr (Ptr Val) -> IO CInt
foreign import ccall safe "hh_tsindex" c_hh_tsindex :: Ptr Ctx -> Ptr Val -> CInt -> Ptr Int64 -> Ptr (Ptr Val) -> IO CInt
foreign import ccall safe "hh_tsargminmax" c_hh_tsargminmax :: Ptr Ctx -> Ptr Val -> CInt -> Ptr (Ptr Val) -> IO CInt
foreign import ccall safe "hh_tsiota" c_hh_tsiota :: Ptr Ctx -> Int64 -> CInt -> Ptr (Ptr Val) -> IO CInt

foreign import ccall safe "hh_ix_var" c_hh_ix_var :: Ptr Ctx -> CInt -> Ptr Int64 -> CInt -> Ptr (Ptr Ix) -> IO CInt
foreign import ccall safe "hh_ix_const" c_hh_ix_const :: Ptr Ctx -> CInt -> Ptr Int64 -> CInt -> CDouble -> Ptr (Ptr Ix) -> IO CInt
foreign import ccall safe "hh_ix_lift" c_hh_ix_lift :: Ptr Ctx -> CInt -> Ptr Int64 -> Ptr Val -> Ptr (Ptr Ix) -> IO CInt
foreign import ccall safe "hh_ix_op1" c_hh_ix_op1 :: Ptr Ctx -> CInt -> Ptr Ix -> Ptr (Ptr Ix) -> IO CInt
foreign import ccall safe "hh_ix_op2" c_hh_ix_op2 :: Ptr Ctx -> CInt -> Ptr Ix -> Ptr Ix -> Ptr (Ptr Ix) -> IO CInt
foreign import ccall safe "hh_ix_compare" c_hh_ix_compare :: Ptr Ctx -> CInt -> Ptr Ix -> Ptr Ix -> Ptr (Ptr Ix) -> IO CInt
foreign import ccall safe "hh_ix_select" c_hh_ix_select :: Ptr Ctx -> Ptr Ix -> Ptr Ix -> Ptr Ix -> Ptr (Ptr Ix) -> IO CInt
foreign import ccall safe "hh_ix_convert" c_hh_ix_convert :: Ptr Ctx -> Ptr Ix -> CInt -> CInt -> Ptr (Ptr Ix) -> IO CInt
foreign import ccall safe "hh_ix_index0" c_hh_ix_index0 :: Ptr Ctx -> Ptr Val -> CInt -> Ptr (Ptr Ix) -> Ptr (Ptr Ix) -> IO CInt
foreign import ccall safe "hh_ix_argminmax" c_hh_ix_argminmax :: Ptr Ctx -> Ptr Val -> CInt -> Ptr (Ptr Ix) -> CInt -> Ptr (Ptr Ix) -> IO CInt
-- tsmap0N / tszipWith0N / tkbuild: an array as a lane over its own index space, and a lane written out as an array
foreign import ccall safe "hh_ix_from_val" c_hh_ix_from_val :: Ptr Ctx -> Ptr Val -> Ptr (Ptr Ix) -> IO CInt
foreign import ccall safe "hh_ix_to_val" c_hh_ix_to_val :: Ptr Ctx -> Ptr Ix -> Ptr (Ptr Val) -> IO CInt
-- ConvertTensor: the checked identity (conversion code of enum hh_conversion, the shape the target type names)
foreign import ccall safe "hh_tconvert" c_hh_tconvert :: Ptr Ctx -> CInt -> Ptr Val -> CInt -> Ptr Int64 -> Ptr (Ptr Val) -> IO CInt
foreign import ccall safe "hh_tprimalPart" c_hh_tprimalPart :: Ptr Ctx -> Ptr Val -> Ptr (Ptr Val) -> IO CInt
foreign import ccall safe "hh_tsgather" c_hh_tsgather
  :: Ptr Ctx -> Ptr Val -> CInt -> Ptr Int64 -> CInt -> Ptr (Ptr Ix) -> Ptr (Ptr Val) -> IO CInt
foreign import ccall safe "hh_tsscatter" c_hh_tsscatter
  :: Ptr Ctx -> Ptr Val -> CInt -> CInt -> Ptr Int64 -> Ptr (Ptr Ix) -> Ptr (Ptr Val) -> IO CInt

-- Gradient descent on device arrays (External/OptimizerTools.hs:20-47, 137-225)
foreign import ccall safe "hh_update_with_gradient" c_hh_update_with_gradient
  :: Ptr Ctx -> CDouble -> Ptr Val -> Ptr Val -> Ptr (Ptr Val) -> IO CInt
foreign import ccall safe "hh_update_with_gradient_adam" c_hh_update_with_gradient_adam
  :: Ptr Ctx -> CDouble -> CDouble -> CDouble -> CDouble -> CInt -> Ptr Val -> Ptr Val -> Ptr Val -> Ptr Val
  -> Ptr (Ptr Val) -> Ptr (Ptr Val) -> Ptr (Ptr Val) -> IO CInt
foreign import ccall safe "hh_adam_step_size" c_hh_adam_step_size
  :: Ptr Ctx -> CInt -> CDouble -> CDouble -> CDouble -> CInt -> Ptr (Ptr Val) -> IO CInt
foreign import ccall safe "hh_adam_apply" c_hh_adam_apply
  :: Ptr Ctx -> Ptr Val -> CDouble -> CDouble -> CDouble -> Ptr Val -> Ptr Val -> Ptr Val -> Ptr Val
  -> Ptr (Ptr Val) -> Ptr (Ptr Val) -> Ptr (Ptr Val) -> IO CInt
foreign import ccall safe "hh_assign" c_hh_assign :: Ptr Ctx -> Ptr Val -> Ptr Val -> IO CInt

-- | The process-wide context (the tensor classes are pure, so there is no
-- place to thread a handle through; the reference has the same kind of global
-- in its AST variable counter, src/HordeAd/Core/AstFreshId.hs:35-48).
{-# NOINLINE ctxRef #-}
ctxRef :: IORef (Ptr Ctx)
ctxRef = unsafePerformIO (newIORef nullPtr)

theCtx :: IO (Ptr Ctx)
theCtx = do
  c <- readIORef ctxRef
  if c /= nullPtr then pure c else do
    c' <- alloca $ \out -> do
      rc <- c_hh_create_gpu 0 out
      when (rc /= 0) $ throwIO (ErrorCall "hordead-gpu: no usable MI355X device")
      peek out
    writeIORef ctxRef c'
    pure c'

withGpu :: IO a -> IO a
withGpu act = theCtx >> act

-- | Status codes become the @error@ calls the reference makes on shape
-- mismatches (src/HordeAd/ADEngine.hs:192-196).
check :: Ptr Ctx -> CInt -> IO ()
check _ 0 = pure ()
check ctx rc = do
  msg <- peekCString =<< c_hh_last_error ctx
  throwIO (ErrorCall ("hordead-gpu (status " ++ show rc ++ "): " ++ msg))
