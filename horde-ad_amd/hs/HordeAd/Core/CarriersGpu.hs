{-# LANGUAGE DataKinds, TypeFamilies, UndecidableInstances #-}
-- | The GPU carrier: the counterpart of @Concrete@
-- (src/HordeAd/Core/CarriersConcrete.hs:150-155, 293-308).  Every array kind is
-- a device value; scalars are rank-0 device values (no sync to make one);
-- products are Haskell pairs, as in @RepConcrete@.
--
-- Not compiled in this repository's build environment (no GHC there).
module HordeAd.Core.CarriersGpu
  ( Gpu (..), RepGpu, GpuFun (..), GpuIx (..), gpuShape
  ) where

import Data.Int (Int64)
import Data.Kind (Type)
import Foreign (withForeignPtr, allocaArray, peekArray)
import System.IO.Unsafe (unsafePerformIO)

import HordeAd.Core.TensorKind
import HordeAd.Core.Types
import HordeAd.Gpu.Foreign

type family RepGpu (y :: TK) :: Type where
  RepGpu (TKScalar r) = ValPtr
  RepGpu (TKR2 n x) = ValPtr
  RepGpu (TKS2 sh x) = ValPtr
  RepGpu (TKX2 sh x) = ValPtr
  RepGpu (TKProduct x z) = (RepGpu x, RepGpu z)

newtype Gpu y = Gpu { unGpu :: RepGpu y }

newtype GpuFun x z = GpuFun { unGpuFun :: RepGpu x -> RepGpu z }

type instance PrimalOf Gpu = Gpu
type instance DualOf Gpu = DummyDualTarget
type instance PlainOf Gpu = Gpu
type instance ShareOf Gpu = Gpu
type instance HFunOf Gpu x z = GpuFun x z
type instance BoolOf Gpu = Gpu (TKScalar Bool)

-- | What an index function is applied to.  Outside gather/scatter/build an
-- @IntOf Gpu@ is an ordinary rank-0 value ('GpuIxVal'); inside, the position
-- variables and everything computed from them are lane-batched scalars
-- ('GpuIxLane', the C side's @hh_ix@): the closure runs once for all positions.
data GpuIx = GpuIxVal ValPtr | GpuIxLane IxPtr

-- | sshape / rshape / xshape (OpsConcrete.hs:99-106): host metadata, no sync.
gpuShape :: ValPtr -> [Int]
gpuShape v = unsafePerformIO $ withForeignPtr v $ \p -> do
  r <- fromIntegral <$> c_hh_val_rank p
  allocaArray (max 1 r) $ \buf -> do
    _ <- c_hh_val_shape p buf
    map (fromIntegral :: Int64 -> Int) <$> peekArray r buf
