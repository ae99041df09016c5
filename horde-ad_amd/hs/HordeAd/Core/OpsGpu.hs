{-# LANGUAGE AllowAmbiguousTypes, DataKinds, TypeFamilies #-}
{-# OPTIONS_GHC -Wno-orphans #-}
-- | @instance BaseTensor Gpu@ — the drop-in beside
-- @instance BaseTensor Concrete@ (src/HordeAd/Core/OpsConcrete.hs:97-775).
-- Every method is one call through the C ABI; purity is kept with
-- 'unsafePerformIO' + NOINLINE: device buffers are immutable and the context
-- enqueues in call order on one stream, so forcing results in data-dependency
-- order is sufficient.
--
-- The shaped methods are spelled out; the ranked (@tr*@) and mixed (@tx*@)
-- methods are the same calls with shapes taken from 'gpuShape' at run time and
-- are omitted from this excerpt.  Not compiled in this repository's build
-- environment (no GHC there).
module HordeAd.Core.OpsGpu (revInterpretArtifactGpu, recordArtifactGpu) where

import Data.Int (Int64)
import Foreign
import Foreign.C
import System.IO.Unsafe (unsafePerformIO)

import HordeAd.Core.Ast
import HordeAd.Core.AstEnv
import HordeAd.Core.AstInterpret
import HordeAd.Core.CarriersGpu
import HordeAd.Core.Ops
import HordeAd.Core.TensorKind
import HordeAd.Core.Types
import HordeAd.Gpu.Foreign

-- * Calling conventions

{-# NOINLINE out1 #-}
out1 :: (Ptr Ctx -> Ptr (Ptr Val) -> IO CInt) -> ValPtr
out1 f = unsafePerformIO $ do
  ctx <- theCtx
  p <- alloca $ \o -> f ctx o >>= check ctx >> peek o
  newForeignPtr p_hh_free p

un1 :: (Ptr Ctx -> Ptr Val -> Ptr (Ptr Val) -> IO CInt) -> ValPtr -> ValPtr
un1 f a = out1 $ \ctx o -> withForeignPtr a $ \pa -> f ctx pa o

bin :: (Ptr Ctx -> Ptr Val -> Ptr Val -> Ptr (Ptr Val) -> IO CInt) -> ValPtr -> ValPtr -> ValPtr
bin f a b = out1 $ \ctx o -> withForeignPtr a $ \pa -> withForeignPtr b $ \pb -> f ctx pa pb o

withShape :: [Int] -> (CInt -> Ptr Int64 -> IO a) -> IO a
withShape sh k = withArrayLen (map fromIntegral sh) $ \n p -> k (fromIntegral n) p

-- opcodes of include/hordead_gpu.h
opNeg, opAbs, opSignum, opRecip, opExp, opLog, opSqrt, opSin, opCos, opTanh :: CInt
opNeg = 0; opAbs = 1; opSignum = 2; opRecip = 3; opExp = 4; opLog = 5; opSqrt = 6
opSin = 7; opCos = 8; opTanh = 15
opAdd, opMul, opSub, opDiv, opPow, opLogBase, opAtan2, opQuot, opRem :: CInt
opAdd = 0; opMul = 1; opSub = 2; opDiv = 3; opPow = 4; opLogBase = 5; opAtan2 = 6
opQuot = 7; opRem = 8

-- * Numeric classes (the superclass context of BaseTensor, Ops.hs:274-296)

instance Num (Gpu (TKS sh r)) where
  Gpu a + Gpu b = Gpu (bin (\c -> c_hh_ewise2 c opAdd) a b)
  Gpu a * Gpu b = Gpu (bin (\c -> c_hh_ewise2 c opMul) a b)
  Gpu a - Gpu b = Gpu (bin (\c -> c_hh_ewise2 c opSub) a b)
  negate (Gpu a) = Gpu (un1 (\c -> c_hh_ewise1 c opNeg) a)
  abs (Gpu a) = Gpu (un1 (\c -> c_hh_ewise1 c opAbs) a)
  signum (Gpu a) = Gpu (un1 (\c -> c_hh_ewise1 c opSignum) a)
  fromInteger = error "fromInteger: shape unknown (as for Concrete arrays)"

instance Fractional (Gpu (TKS sh r)) where
  Gpu a / Gpu b = Gpu (bin (\c -> c_hh_ewise2 c opDiv) a b)
  recip (Gpu a) = Gpu (un1 (\c -> c_hh_ewise1 c opRecip) a)
  fromRational = error "fromRational: shape unknown (as for Concrete arrays)"

instance Floating (Gpu (TKS sh r)) where
  pi = error "pi is not defined for tensors"
  exp (Gpu a) = Gpu (un1 (\c -> c_hh_ewise1 c opExp) a)
  log (Gpu a) = Gpu (un1 (\c -> c_hh_ewise1 c opLog) a)
  sqrt (Gpu a) = Gpu (un1 (\c -> c_hh_ewise1 c opSqrt) a)
  sin (Gpu a) = Gpu (un1 (\c -> c_hh_ewise1 c opSin) a)
  cos (Gpu a) = Gpu (un1 (\c -> c_hh_ewise1 c opCos) a)
  tanh (Gpu a) = Gpu (un1 (\c -> c_hh_ewise1 c opTanh) a)
  Gpu a ** Gpu b = Gpu (bin (\c -> c_hh_ewise2 c opPow) a b)
  logBase (Gpu a) (Gpu b) = Gpu (bin (\c -> c_hh_ewise2 c opLogBase) a b)
  -- tan, asin, ..., atanh: opcodes 9..18, same shape

instance RealFloatH (Gpu (TKS sh r)) where
  atan2H (Gpu a) (Gpu b) = Gpu (bin (\c -> c_hh_ewise2 c opAtan2) a b)

instance IntegralH (Gpu (TKS sh r)) where
  quotH (Gpu a) (Gpu b) = Gpu (bin (\c -> c_hh_ewise2 c opQuot) a b)
  remH (Gpu a) (Gpu b) = Gpu (bin (\c -> c_hh_ewise2 c opRem) a b)

-- * The tensor class

instance BaseTensor Gpu where
  isConcreteInstance = False
  sshape (Gpu v) = shsFromListUnsafe (gpuShape v)            -- OpsConcrete.hs:101
  tpair (Gpu a) (Gpu b) = Gpu (a, b)                          -- :107
  tproject1 (Gpu (a, _)) = Gpu a
  tproject2 (Gpu (_, b)) = Gpu b
  tsconcrete a = Gpu $ out1 $ \ctx o ->                       -- :120-124: an upload
    withShape (shapeOfNested a) $ \n sh -> withNestedData a $ \dt p ->
      c_hh_upload ctx dt n sh p 0 o
  tssum (Gpu t) = Gpu (un1 (\c p -> c_hh_tssumN c p 1) t)     -- :215
  tssumN @shm (Gpu t) = Gpu (un1 (\c p -> c_hh_tssumN c p (rankOf @shm)) t)   -- :222
  tssum0 (Gpu t) = Gpu (un1 c_hh_tssum0 t)                    -- :229
  tsdot0 (Gpu a) (Gpu b) = Gpu (bin c_hh_tsdot0 a b)          -- :231
  tsdot1In _ (Gpu a) (Gpu b) = Gpu (bin c_hh_tsdot1In a b)    -- :233
  tsmatvecmul (Gpu m) (Gpu v) = Gpu (bin c_hh_tsmatvecmul m v)  -- :236
  tsmatmul2 (Gpu a) (Gpu b) = Gpu (bin c_hh_tsmatmul2 a b)    -- :237
  tsreplicateN shm (Gpu t) = Gpu $ out1 $ \ctx o ->           -- :243
    withForeignPtr t $ \p -> withShape (shsToList shm) $ \n sh -> c_hh_tsreplicateN ctx p n sh o
  tsreplicate0N sh (Gpu t) = Gpu $ out1 $ \ctx o ->           -- :245
    withForeignPtr t $ \p -> withShape (shsToList sh) $ \n s -> c_hh_tsreplicateN ctx p n s o
  tsappend (Gpu a) (Gpu b) = Gpu (bin c_hh_tsappend a b)      -- :638
  tsslice i n _ (Gpu t) = Gpu (un1 (\c p -> c_hh_tsslice c p (fromSNat' i) (fromSNat' n)) t)  -- :641
  tsreverse (Gpu t) = Gpu (un1 c_hh_tsreverse t)              -- :644
  tstranspose perm (Gpu t) = Gpu $ out1 $ \ctx o ->           -- :647
    withForeignPtr t $ \p -> withArrayLen (map fromIntegral (permToList perm)) $ \n pp ->
      c_hh_tstranspose ctx p (fromIntegral n) pp o
  tsreshape sh (Gpu t) = Gpu $ out1 $ \ctx o ->               -- :650
    withForeignPtr t $ \p -> withShape (shsToList sh) $ \n s -> c_hh_tsreshape ctx p n s o
  tsargMin (Gpu t) = Gpu (un1 (\c p -> c_hh_tsargminmax c p 0) t)   -- :533
  tsargMax (Gpu t) = Gpu (un1 (\c p -> c_hh_tsargminmax c p 1) t)   -- :534
  tsiota @n = Gpu $ out1 $ \ctx o -> c_hh_tsiota ctx (valueOf @n) 2 o   -- :535
  -- tsgather (OpsConcrete.hs:1621-1665): the closure is applied ONCE, to the
  -- symbolic position variables; its result is handed over as hh_ix handles.
  tsgather @shm (Gpu t) f = Gpu $ out1 $ \ctx o ->
    let shm = shsToList (knownShS @shm)
    in withShape shm $ \n sh -> do
         vars <- mapM (laneVar ctx n sh) [0 .. length shm - 1]
         ixs <- mapM (forceLane ctx n sh) (ixsToList (f (ixsFromList vars)))
         withForeignPtr t $ \p -> withIxArray ixs $ \k pix -> c_hh_tsgather ctx p n sh k pix o
  -- tsscatter (OpsConcrete.hs:1581-1619)
  tsscatter @shm @shn @shp (Gpu t) f = Gpu $ out1 $ \ctx o ->
    let shm = shsToList (knownShS @shm)
        shp = shsToList (knownShS @shp)
    in withShape shm $ \n sh -> withShape shp $ \np shpP -> do
         vars <- mapM (laneVar ctx n sh) [0 .. length shm - 1]
         ixs <- mapM (forceLane ctx n sh) (ixsToList (f (ixsFromList vars)))
         withForeignPtr t $ \p -> withIxArray ixs $ \_ pix -> c_hh_tsscatter ctx p n np shpP pix o
  -- kcond / scond on a host Bool stay host conditionals (OpsConcrete.hs:113-119);
  -- inside an index function kcond is c_hh_ix_select on lanes.
  -- tmapAccumLDer (OpsConcrete.hs:990-1019) is the same host loop over
  -- tsindex'ed steps; each step dispatches the methods above.
  -- ... remaining methods: see the header for the entry point of each.

-- | revInterpretArtifact at the Gpu carrier: the 10-line sibling of
-- src/HordeAd/ADEngine.hs:266-288 (that one is hard-typed to Concrete).
revInterpretArtifactGpu
  :: AstArtifactRev x z -> Gpu x -> Maybe (Gpu (ADTensorKind z)) -> (Gpu (ADTensorKind x), Gpu z)
revInterpretArtifactGpu AstArtifactRev{..} parameters mdt =
  let azftk = adFTK (ftkAst artPrimalRev)
      env = extendEnv artVarDomainRev parameters emptyEnv
      envDt = case mdt of
        Nothing -> extendEnv artVarDtRev (treplTarget 1 azftk) env
        Just dt -> extendEnv artVarDtRev dt env
  in (interpretAstFull envDt artDerivativeRev, interpretAstFull env artPrimalRev)


-- | The same artifact recorded once as a device graph: returns an action that
-- re-runs the whole gradient in one submission, refreshing (in place) the
-- arrays behind the returned values.  Call 'revInterpretArtifactGpu' once
-- beforehand so that constants and generated kernels exist; feed new inputs
-- with @hh_overwrite@ on the arrays of @parameters@.
recordArtifactGpu
  :: AstArtifactRev x z -> Gpu x -> Maybe (Gpu (ADTensorKind z))
  -> IO ((Gpu (ADTensorKind x), Gpu z), IO ())
recordArtifactGpu art parameters mdt = do
  ctx <- theCtx
  c_hh_capture_begin ctx >>= check ctx
  let r@(g, v) = revInterpretArtifactGpu art parameters mdt
  forceGpu ctx g >> forceGpu ctx v          -- hh_force on every array of the results
  gr <- alloca $ \o -> c_hh_capture_end ctx o >>= check ctx >> peek o
  pure (r, c_hh_graph_launch ctx gr >>= check ctx)
