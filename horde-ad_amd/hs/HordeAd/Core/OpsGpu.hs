{-# LANGUAGE AllowAmbiguousTypes, DataKinds, GADTs, LambdaCase, RankNTypes,
             RecordWildCards, ScopedTypeVariables, TypeApplications, TypeFamilies,
             TypeOperators #-}
{-# OPTIONS_GHC -Wno-orphans -fplugin GHC.TypeLits.KnownNat.Solver #-}
-- | The tensor classes at the GPU carrier -- the drop-in beside
-- @instance BaseTensor Concrete@ (src/HordeAd/Core/OpsConcrete.hs:97-775) and
-- its @LetTensor@ / @ShareTensor@ / @ConvertTensor@ instances (:84-96, 777-904).
--
-- Every method is one call (or a host loop of calls, where the reference has
-- a host loop) through the C ABI of include/hordead_host.h.  The ranked,
-- shaped and mixed methods of one operation are the same call: the shape
-- lives with the device value, and what differs is how the static part of
-- the result's shape is put together for the type.
--
-- Not compiled in this repository's build environment (no GHC there); written
-- against horde-ad's own modules as they are in the reference checkout.
module HordeAd.Core.OpsGpu
  ( revInterpretArtifactGpu, recordArtifactGpu
  ) where

import Prelude

import Data.Foldable qualified as Foldable
import Data.Int (Int64)
import Data.List (foldl')
import Data.List.NonEmpty qualified as NonEmpty
import Data.Proxy (Proxy (Proxy))
import Data.Type.Equality (gcastWith, testEquality, (:~:) (Refl))
import Data.Vector qualified as V
import Data.Vector.Storable qualified as VS
import Foreign
import Foreign.C
import GHC.Exts qualified
import GHC.TypeLits (KnownNat, type (+))
import System.IO.Unsafe (unsafePerformIO)
import Type.Reflection (typeRep)

import Data.Array.Nested (type (++))
import Data.Array.Nested qualified as Nested
import Data.Array.Nested.Convert (shxFromShR, shxFromShS, withShsFromShR)
import Data.Array.Nested.Mixed.Shape
import Data.Array.Nested.Permutation qualified as Permutation
import Data.Array.Nested.Ranked.Shape
import Data.Array.Nested.Shaped.Shape
import Data.Array.Nested.Types (unsafeCoerceRefl)

import HordeAd.Core.Ast
import HordeAd.Core.AstEnv
import HordeAd.Core.AstInterpret
import HordeAd.Core.CarriersConcrete
import HordeAd.Core.CarriersGpu
import HordeAd.Core.Conversion
import HordeAd.Core.ConvertTensor
import HordeAd.Core.Ops
import HordeAd.Core.OpsADVal
import HordeAd.Core.TensorKind
import HordeAd.Core.Types
import HordeAd.Core.UnwindNum
import HordeAd.Gpu.Foreign

-- * Shapes: from the device value's run-time dims to the typed shapes

dims :: RepGpu y ~ ValPtr => Gpu y -> [Int]
dims (Gpu v) = gpuShape v

-- | rshape (OpsConcrete.hs:99): the rank in the type is the rank of the value.
shrOf :: forall n. [Int] -> IShR n
shrOf l = withSNat (length l) $ \(m :: SNat m) ->
  gcastWith (unsafeCoerceRefl :: m :~: n) $ shrFromList m l

-- | sshape (OpsConcrete.hs:101): the dims in the type are the dims of the value.
shsOf :: forall sh. [Int] -> ShS sh
shsOf l = withShsFromShR (shrOf @(Rank sh) l) $ \(sh' :: ShS sh') ->
  gcastWith (unsafeCoerceRefl :: sh' :~: sh) sh'

-- | xshape (OpsConcrete.hs:103): the static skeleton filled in with the value's dims.
shxOf :: StaticShX sh -> [Int] -> IShX sh
shxOf ZKX _ = ZSX
shxOf (SKnown n :!% rest) (_ : ds) = SKnown n :$% shxOf rest ds
shxOf (SUnknown () :!% rest) (d : ds) = SUnknown d :$% shxOf rest ds
shxOf _ [] = error "shxOf: the value has fewer dims than its type"

ixList :: Foldable f => f (Gpu (TKScalar Int)) -> [GpuIx]
ixList = map unGpu . Foldable.toList

-- * Helpers shared by the ranked, shaped and mixed methods (all on 'ValPtr')

sumPrefix :: Int -> ValPtr -> ValPtr                  -- trsumN / tssumN / txsumN
sumPrefix k = un1 (\c p -> c_hh_tssumN c p (fromIntegral k))

replicatePrefix :: [Int] -> ValPtr -> ValPtr          -- t?replicateN, t?replicate0N
replicatePrefix shm t = out1 $ \ctx o ->
  withForeignPtr t $ \p -> withShape shm $ \n sh -> c_hh_tsreplicateN ctx p n sh o

reshapeTo :: [Int] -> ValPtr -> ValPtr
reshapeTo sh t = out1 $ \ctx o ->
  withForeignPtr t $ \p -> withShape sh $ \n s -> c_hh_tsreshape ctx p n s o

transposeBy :: [Int] -> ValPtr -> ValPtr
transposeBy perm t = out1 $ \ctx o ->
  withForeignPtr t $ \p -> withArrayLen (map fromIntegral perm) $ \n pp ->
    c_hh_tstranspose ctx p (fromIntegral n) pp o

sliceOuter :: Int -> Int -> ValPtr -> ValPtr
sliceOuter i n = un1 (\c p -> c_hh_tsslice c p (fromIntegral i) (fromIntegral n))

argExtremum :: Bool -> ValPtr -> ValPtr               -- over the last dim, the first extremum
argExtremum wantMax = un1 (\c p -> c_hh_tsargminmax c p (if wantMax then 1 else 0))

convertArr :: CInt -> CInt -> ValPtr -> ValPtr        -- mode 1 = floor, 0 = cast
convertArr dt mode = un1 (\c p -> c_hh_convert c p dt mode)

iotaArr :: CInt -> Int -> ValPtr
iotaArr dt n = out1 $ \ctx o -> c_hh_tsiota ctx (fromIntegral n) dt o

-- | Upload of a host array (tsconcrete and friends, OpsConcrete.hs:120-124):
-- the array's elements in row-major order, as ox-arrays hands them out.
uploadArr :: forall r. GoodScalar r => [Int] -> VS.Vector r -> ValPtr
uploadArr sh xs = out1 $ \ctx o -> withShape sh $ \n s -> VS.unsafeWith xs $ \p ->
  c_hh_upload ctx (dtypeOf @r) n s (castPtr p) 0 o

-- | t !$ ix with the index known on the host; with an index that is a device
-- scalar it is the gather over the empty position space.
indexPrefix :: [GpuIx] -> ValPtr -> ValPtr
indexPrefix ix t
  | Just lits <- mapM (\case GpuIxLit x -> Just (round x :: Int); _ -> Nothing) ix =
      out1 $ \ctx o -> withForeignPtr t $ \p -> withShape lits $ \n s -> c_hh_tsindex ctx p n s o
  | otherwise = gatherBy [] t (const ix)

-- | tgatherZS / tscatterZS (OpsConcrete.hs:1581-1665): the closure is applied
-- once, to the lane variables of the position space @shm@.
laneVars :: [Int] -> [GpuIx]
laneVars shm =
  [ GpuIxLane shm (outIx $ \ctx o -> withShape shm $ \n sh -> c_hh_ix_var ctx n sh (fromIntegral d) o)
  | d <- [0 .. length shm - 1] ]

gatherBy :: [Int] -> ValPtr -> ([GpuIx] -> [GpuIx]) -> ValPtr
gatherBy shm t f = out1 $ \ctx o ->
  let ixs = map (laneOf 2 shm) (f (laneVars shm))
  in withForeignPtr t $ \p -> withShape shm $ \n sh -> withIxArray ixs $ \k pix ->
       c_hh_tsgather ctx p n sh k pix o

scatterBy :: [Int] -> [Int] -> ValPtr -> ([GpuIx] -> [GpuIx]) -> ValPtr
scatterBy shm shp t f = out1 $ \ctx o ->
  let ixs = map (laneOf 2 shm) (f (laneVars shm))
  in withForeignPtr t $ \p -> withShape shp $ \np sp -> withIxArray ixs $ \_ pix ->
       c_hh_tsscatter ctx p (fromIntegral (length shm)) np sp pix o

-- | tsfromVectorN and friends: the pieces are stacked along a new outer dim by
-- appending their [1, ..] reshapes, then the outer dim is reshaped to @shm@.
stackVals :: [Int] -> [Int] -> [ValPtr] -> ValPtr
stackVals shm shn [] = out1 $ \ctx o -> withShape (shm ++ shn) $ \n s -> c_hh_constant ctx 0 0 n s o
stackVals shm shn vs =
  reshapeTo (shm ++ shn) $ foldl1 (bin c_hh_tsappend) (map (reshapeTo (1 : shn)) vs)

-- * LetTensor, ShareTensor: device values are immutable handles, already shared
-- (OpsConcrete.hs:84-96)

instance LetTensor Gpu where
  ttlet = (&)
  ttletPrimal = (&)
  ttletPlain = (&)
  toShare = id
  tunshare = id

(&) :: a -> (a -> b) -> b
x & f = f x

instance ShareTensor Gpu where
  tshare = id
  tunpair (Gpu (a, b)) = (Gpu a, Gpu b)

-- * The tensor class

instance BaseTensor Gpu where
  isConcreteInstance = False

  rshape = shrOf . dims
  sshape = shsOf . dims
  xshape @sh (Gpu v) = shxOf (mixedSkeleton @sh v) (gpuShape v)
  tftk stk (Gpu v) = case stk of             -- CarriersConcrete.hs:164 (tftkG)
    STKScalar -> FTKScalar
    STKR _ x -> FTKR (shrOf (gpuShape v)) (scalarsOnly x)
    STKS sh x -> FTKS sh (scalarsOnly x)
    STKX ssx x -> FTKX (shxOf ssx (gpuShape v)) (scalarsOnly x)
    STKProduct s1 s2 -> FTKProduct (tftk s1 (Gpu (fst v))) (tftk s2 (Gpu (snd v)))

  tpair (Gpu a) (Gpu b) = Gpu (a, b)                              -- :107
  tproject1 (Gpu (a, _)) = Gpu a
  tproject2 (Gpu (_, b)) = Gpu b

  -- :113-119.  A condition known on the host selects on the host; a device
  -- condition selects elementwise over the broadcast Bool.
  kcond @r (Gpu b) (Gpu u) (Gpu v) = Gpu (scSelect (dtypeOf @r) b u v)
  scond (Gpu b) u v = condArr b u v
  tcond stk (Gpu b) u v = case stk of
    STKScalar -> kcond (Gpu b) u v
    STKR{} -> condArr b u v
    STKS{} -> condArr b u v
    STKX{} -> condArr b u v
    STKProduct s1 s2 -> tpair (tcond s1 (Gpu b) (tproject1 u) (tproject1 v))
                              (tcond s2 (Gpu b) (tproject2 u) (tproject2 v))

  tkconcrete = Gpu . literal'                                      -- :120-124
  trconcrete a = Gpu (uploadArr (Foldable.toList (Nested.rshape a)) (Nested.rtoVector a))
  tsconcrete a = Gpu (uploadArr (shsToList (Nested.sshape a)) (Nested.stoVector a))
  txconcrete a = Gpu (uploadArr (shxToList' (Nested.mshape a)) (Nested.mtoVector a))
  tconcrete ftk (Concrete a) = case ftk of
    FTKScalar -> tkconcrete a
    FTKR _ FTKScalar -> trconcrete a
    FTKS _ FTKScalar -> tsconcrete a
    FTKX _ FTKScalar -> txconcrete a
    FTKProduct f1 f2 -> tpair (tconcrete f1 (Concrete (fst a))) (tconcrete f2 (Concrete (snd a)))
    _ -> nestedArrays "tconcrete"

  -- :125-214
  trfromVectorN shm v = stackOf (Foldable.toList shm) (V.toList v)
  trfromVectorLinear @_ @r shm v = Gpu (stackVals (Foldable.toList shm) [] (map (scalarVal (dtypeOf @r) . unGpu) (V.toList v)))
  tsfromVectorN shm v = stackOf (shsToList shm) (V.toList v)
  tsfromVectorLinear @_ @r shm v = Gpu (stackVals (shsToList shm) [] (map (scalarVal (dtypeOf @r) . unGpu) (V.toList v)))
  txfromVectorN shm v = stackOf (shxToList' shm) (V.toList v)
  txfromVectorLinear @_ @r shm v = Gpu (stackVals (shxToList' shm) [] (map (scalarVal (dtypeOf @r) . unGpu) (V.toList v)))

  trsumN @m (Gpu t) = Gpu (sumPrefix (valueOf @m) t)                                 -- :215-230
  trsum0 (Gpu t) = Gpu (valScalar (un1 c_hh_tssum0 t))
  trdot0 (Gpu a) (Gpu b) = Gpu (valScalar (bin c_hh_tsdot0 a b))
  trdot1In (Gpu a) (Gpu b) = Gpu (bin c_hh_tsdot1In a b)
  trmatvecmul (Gpu m) (Gpu v) = Gpu (bin c_hh_tsmatvecmul m v)
  trmatmul2 (Gpu a) (Gpu b) = Gpu (bin c_hh_tsmatmul2 a b)
  trreplicateN shm (Gpu t) = Gpu (replicatePrefix (Foldable.toList shm) t)
  trreplicate0N @_ @r shm (Gpu s) = Gpu (replicatePrefix (Foldable.toList shm) (scalarVal (dtypeOf @r) s))

  tssumN @shm (Gpu t) = Gpu (sumPrefix (shsLength (knownShS @shm)) t)
  tssum0 (Gpu t) = Gpu (valScalar (un1 c_hh_tssum0 t))
  tsdot0 (Gpu a) (Gpu b) = Gpu (valScalar (bin c_hh_tsdot0 a b))                     -- :231
  tsdot1In _ (Gpu a) (Gpu b) = Gpu (bin c_hh_tsdot1In a b)                           -- :233
  tsmatvecmul (Gpu m) (Gpu v) = Gpu (bin c_hh_tsmatvecmul m v)                       -- :236
  tsmatmul2 (Gpu a) (Gpu b) = Gpu (bin c_hh_tsmatmul2 a b)                           -- :237
  tsreplicateN shm (Gpu t) = Gpu (replicatePrefix (shsToList shm) t)                 -- :243
  tsreplicate0N @_ @r shm (Gpu s) = Gpu (replicatePrefix (shsToList shm) (scalarVal (dtypeOf @r) s))

  txsumN @shm (Gpu t) = Gpu (sumPrefix (ssxLength (knownShX @shm)) t)
  txsum0 (Gpu t) = Gpu (valScalar (un1 c_hh_tssum0 t))
  txdot0 (Gpu a) (Gpu b) = Gpu (valScalar (bin c_hh_tsdot0 a b))
  txdot1In _ (Gpu a) (Gpu b) = Gpu (bin c_hh_tsdot1In a b)
  txmatvecmul _ _ (Gpu m) (Gpu v) = Gpu (bin c_hh_tsmatvecmul m v)
  txmatmul2 (Gpu a) (Gpu b) = Gpu (bin c_hh_tsmatmul2 a b)
  txreplicateN shm (Gpu t) = Gpu (replicatePrefix (shxToList' shm) t)
  txreplicate0N @_ @r shm (Gpu s) = Gpu (replicatePrefix (shxToList' shm) (scalarVal (dtypeOf @r) s))

  -- :246-360: indexing, gather, scatter
  trindex (Gpu t) ix = Gpu (indexPrefix (ixList ix) t)
  trindex0 (Gpu t) ix = Gpu (valScalar (indexPrefix (ixList ix) t))
  trscatter @m shp (Gpu t) f =
    Gpu (scatterBy (take (valueOf @m) (gpuShape t)) (Foldable.toList shp) t (viaIxR f))
  trgather shm (Gpu t) f = Gpu (gatherBy (Foldable.toList shm) t (viaIxR f))
  tsindex (Gpu t) ix = Gpu (indexPrefix (ixList ix) t)
  tsindex0 (Gpu t) ix = Gpu (valScalar (indexPrefix (ixList ix) t))
  tsscatter @shm @_ @shp (Gpu t) f =
    Gpu (scatterBy (shsToList (knownShS @shm)) (shsToList (knownShS @shp)) t (viaIxS f))
  tsgather @shm (Gpu t) f = Gpu (gatherBy (shsToList (knownShS @shm)) t (viaIxS f))
  txindex (Gpu t) ix = Gpu (indexPrefix (ixList ix) t)
  txindex0 (Gpu t) ix = Gpu (valScalar (indexPrefix (ixList ix) t))
  txscatter @shm shp (Gpu t) f =
    Gpu (scatterBy (take (ssxLength (knownShX @shm)) (gpuShape t)) (shxToList' shp) t (viaIxX f))
  txgather shm (Gpu t) f = Gpu (gatherBy (shxToList' shm) t (viaIxX f))

  -- :361-560: conversions of the element type, arg-extrema, iota
  tkfloor @_ @r2 (Gpu a) = Gpu (scConvert (dtypeOf @r2) 1 a)
  tkfromIntegral @_ @r2 (Gpu a) = Gpu (scConvert (dtypeOf @r2) 0 a)
  tkcast @_ @r2 (Gpu a) = Gpu (scConvert (dtypeOf @r2) 0 a)
  tkargMin (Gpu t) = Gpu (valScalar (argExtremum False t))
  tkargMax (Gpu t) = Gpu (valScalar (argExtremum True t))
  trfloor @_ @r2 (Gpu a) = Gpu (convertArr (dtypeOf @r2) 1 a)
  trfromIntegral @_ @r2 (Gpu a) = Gpu (convertArr (dtypeOf @r2) 0 a)
  trcast @_ @r2 (Gpu a) = Gpu (convertArr (dtypeOf @r2) 0 a)
  trargMin (Gpu t) = Gpu (argExtremum False t)
  trargMax (Gpu t) = Gpu (argExtremum True t)
  triota @r n = Gpu (iotaArr (dtypeOf @r) n)
  tsfloor @_ @r2 (Gpu a) = Gpu (convertArr (dtypeOf @r2) 1 a)
  tsfromIntegral @_ @r2 (Gpu a) = Gpu (convertArr (dtypeOf @r2) 0 a)
  tscast @_ @r2 (Gpu a) = Gpu (convertArr (dtypeOf @r2) 0 a)
  tsargMin (Gpu t) = Gpu (argExtremum False t)                                       -- :533
  tsargMax (Gpu t) = Gpu (argExtremum True t)                                        -- :534
  tsiota @n @r = Gpu (iotaArr (dtypeOf @r) (valueOf @n))                             -- :535
  txfloor @_ @r2 (Gpu a) = Gpu (convertArr (dtypeOf @r2) 1 a)
  txfromIntegral @_ @r2 (Gpu a) = Gpu (convertArr (dtypeOf @r2) 0 a)
  txcast @_ @r2 (Gpu a) = Gpu (convertArr (dtypeOf @r2) 0 a)
  txargMin (Gpu t) = Gpu (argExtremum False t)
  txargMax (Gpu t) = Gpu (argExtremum True t)
  txiota @n @r = Gpu (iotaArr (dtypeOf @r) (valueOf @n))

  -- :561-660: the views
  trappend (Gpu a) (Gpu b) = Gpu (bin c_hh_tsappend a b)
  trslice i n (Gpu t) = Gpu (sliceOuter i n t)
  trreverse (Gpu t) = Gpu (un1 c_hh_tsreverse t)
  trtranspose perm (Gpu t) = Gpu (transposeBy perm t)
  trreshape sh (Gpu t) = Gpu (reshapeTo (Foldable.toList sh) t)
  tsappend (Gpu a) (Gpu b) = Gpu (bin c_hh_tsappend a b)                             -- :638
  tsslice i n _ (Gpu t) = Gpu (sliceOuter (fromSNat' i) (fromSNat' n) t)            -- :641
  tsreverse (Gpu t) = Gpu (un1 c_hh_tsreverse t)                                     -- :644
  tstranspose perm (Gpu t) = Gpu (transposeBy (Permutation.permToList' perm) t)      -- :647
  tsreshape sh (Gpu t) = Gpu (reshapeTo (shsToList sh) t)                            -- :650
  txappend (Gpu a) (Gpu b) = Gpu (bin c_hh_tsappend a b)
  txslice i n _ (Gpu t) = Gpu (sliceOuter (fromSMayNat' i) (fromSMayNat' n) t)
  txreverse (Gpu t) = Gpu (un1 c_hh_tsreverse t)
  txtranspose perm (Gpu t) = Gpu (transposeBy (Permutation.permToList' perm) t)
  txreshape sh (Gpu t) = Gpu (reshapeTo (shxToList' sh) t)

  -- :661-740: build is the reference's host loop (tbuild1S, :1075-1100); the
  -- closure may do anything a tensor program does, so it runs once per index
  tkbuild1 @k @r f = Gpu (stackVals [valueOf @k] [] [scalarVal (dtypeOf @r) (unGpu (f (Gpu (literal i)))) | i <- [0 .. valueOf @k - 1 :: Int]])
  trbuild1 k f = stackOfUnknown [k] [f (Gpu (literal i)) | i <- [0 .. k - 1]]
  tsbuild1 @k f = stackOfUnknown [valueOf @k] [f (Gpu (literal i)) | i <- [0 .. valueOf @k - 1 :: Int]]
  txbuild1 @k f = stackOfUnknown [valueOf @k] [f (Gpu (literal i)) | i <- [0 .. valueOf @k - 1 :: Int]]

  -- :736-760
  tmapAccumLDer _ k _ bftk eftk (GpuFun f) _df _rf acc0 es = mapAccumLGpu k bftk eftk f acc0 es
  tmapAccumRDer p k aftk bftk eftk f df rf acc0 es =
    let r = tmapAccumLDer p k aftk bftk eftk f df rf acc0 (treverse k (ftkToSTK eftk) es)
    in tpair (tproject1 r) (treverse k (ftkToSTK bftk) (tproject2 r))
  tapply (GpuFun f) = Gpu . f . unGpu
  tlambda _ f = GpuFun $ unGpu . unHFun f . Gpu
  tgrad @_ @r xftk h | Dict0 <- lemTKScalarAllNumAD (Proxy @r) =
    GpuFun $ unGpu . snd . crevOnParams Nothing (unHFun h) xftk . Gpu
  tvjp xftk h = GpuFun $ \db_a ->
    unGpu $ snd $ crevOnParamsDt (Gpu $ fst db_a) (unHFun h) xftk (Gpu $ snd db_a)
  tjvp xftk h = GpuFun $ \da_a ->
    unGpu $ snd $ cfwdOnParams xftk (Gpu $ snd da_a) (unHFun h) (Gpu $ fst da_a)

  tprimalPart = id                                                                   -- :761-775
  tdualPart stk t = DummyDualTarget (tftk stk t)
  tplainPart = id
  tfromPrimal _ t = t
  tfromDual (DummyDualTarget ftk) = tdefTarget ftk
  tfromPlain _ t = t
  tScale _ _ t = t
  taddTarget = addTarget
  tmultTarget = multTarget
  tsum0Target = sum0Target
  tdot0Target = dot0Target

-- Pieces of the instance

literal' :: forall r. GoodScalar r => r -> GpuIx
literal' x
  | Just Refl <- testEquality (typeRep @r) (typeRep @Double) = GpuIxLit x
  | Just Refl <- testEquality (typeRep @r) (typeRep @Float) = GpuIxLit (realToFrac x)
  | Just Refl <- testEquality (typeRep @r) (typeRep @Int) = GpuIxLit (fromIntegral x)
  | Just Refl <- testEquality (typeRep @r) (typeRep @Int64) = GpuIxLit (fromIntegral x)
  | Just Refl <- testEquality (typeRep @r) (typeRep @Bool) = GpuIxLit (if x then 1 else 0)
  | otherwise = GpuIxVal (uploadArr @r [] (VS.singleton x))

-- | The mixed skeleton of a value whose type is all we have.  xshape's signature
-- offers no singleton for @sh@, and the device value knows its dims but not
-- which of them the type leaves open, so every dim is reported as a known one
-- (@SKnown@).  That is exact for the mixed types horde-ad's own conversions
-- produce from shaped arrays (@MapJust sh@); a mixed type with a @Nothing@ dim
-- needs the shape kept beside the handle, as ox-arrays keeps it, before code
-- that matches on @SUnknown@ may look at the result of 'xshape'.  'tftk', which
-- does get the singleton, fills the skeleton in properly ('shxOf').
mixedSkeleton :: forall sh. ValPtr -> StaticShX sh
mixedSkeleton v = withShsFromShR (shrOf @(Rank sh) (gpuShape v)) $ \(sh' :: ShS sh') ->
  gcastWith (unsafeCoerceRefl :: MapJust sh' :~: sh) $ ssxFromShX (shxFromShS sh')

scalarsOnly :: SingletonTK x -> FullShapeTK x
scalarsOnly = \case
  STKScalar -> FTKScalar
  _ -> nestedArrays "tftk"

nestedArrays :: String -> a
nestedArrays what = error (what ++ ": arrays of arrays and arrays of products are not represented on this carrier")

shxToList' :: IShX sh -> [Int]
shxToList' = Foldable.toList

condArr :: RepGpu y ~ ValPtr => GpuIx -> Gpu y -> Gpu y -> Gpu y
condArr (GpuIxLit c) u v = if c /= 0 then u else v
condArr b (Gpu u) (Gpu v) = Gpu $ out1 $ \ctx o ->
  let cond = replicatePrefix (gpuShape u) (scalarVal 6 b)
  in withForeignPtr cond $ \pc -> withForeignPtr u $ \pu -> withForeignPtr v $ \pv -> c_hh_select ctx pc pu pv o

stackOf :: (RepGpu y ~ ValPtr, RepGpu z ~ ValPtr) => [Int] -> [Gpu y] -> Gpu z
stackOf shm vs = case vs of
  [] -> error "fromVector: an empty vector carries no element shape"
  Gpu v0 : _ -> Gpu (stackVals shm (gpuShape v0) (map unGpu vs))

stackOfUnknown :: (RepGpu y ~ ValPtr, RepGpu z ~ ValPtr) => [Int] -> [Gpu y] -> Gpu z
stackOfUnknown = stackOf

viaIxR :: (IxROf Gpu m -> IxROf Gpu p) -> [GpuIx] -> [GpuIx]
viaIxR f vars = ixList (f (fromList' vars))
viaIxS :: (IxSOf Gpu shm -> IxSOf Gpu shp) -> [GpuIx] -> [GpuIx]
viaIxS f vars = ixList (f (fromList' vars))
viaIxX :: (IxXOf Gpu shm -> IxXOf Gpu shp) -> [GpuIx] -> [GpuIx]
viaIxX f vars = ixList (f (fromList' vars))

-- | The sized index lists are instances of IsList (OverloadedLists, Types.hs:264-289).
fromList' :: (GHC.Exts.IsList l, GHC.Exts.Item l ~ Gpu (TKScalar Int)) => [GpuIx] -> l
fromList' = GHC.Exts.fromList . map Gpu

-- | tmapAccumLC (OpsConcrete.hs:990-1019): a strict left fold on the host over
-- the unravelled inputs; each step dispatches the methods above.
mapAccumLGpu
  :: forall k accy by ey.
     SNat k -> FullShapeTK by -> FullShapeTK ey
  -> (RepGpu (TKProduct accy ey) -> RepGpu (TKProduct accy by))
  -> Gpu accy -> Gpu (BuildTensorKind k ey)
  -> Gpu (TKProduct accy (BuildTensorKind k by))
mapAccumLGpu k bftk eftk f acc0 es =
  let step (acc, outs) e = let (acc', b) = f (unGpu acc, unGpu e) in (Gpu acc', Gpu b : outs)
      (xout, louts) = foldl' step (acc0, []) (tunravelToListShare k (ftkToSTK eftk) es)
  in case NonEmpty.nonEmpty (reverse louts) of
       Just nl -> tpair xout (fromListGpu k (ftkToSTK bftk) (NonEmpty.toList nl))
       Nothing -> tpair xout (tdefTarget (buildFTK k bftk))

-- | tfromList (OpsConcrete.hs:960-988): k values stacked along a new outer dim,
-- componentwise through products.
fromListGpu :: forall y k. SNat k -> SingletonTK y -> [Gpu y] -> Gpu (BuildTensorKind k y)
fromListGpu snat@SNat stk l = case stk of
  STKScalar @r -> Gpu (stackVals [fromSNat' snat] [] (map (scalarVal (dtypeOf @r) . unGpu) l))
  STKR{} -> stackOf [fromSNat' snat] l
  STKS{} -> stackOf [fromSNat' snat] l
  STKX{} -> stackOf [fromSNat' snat] l
  STKProduct s1 s2 ->
    tpair (fromListGpu snat s1 (map tproject1 l)) (fromListGpu snat s2 (map tproject2 l))

-- * ConvertTensor (ConvertTensor.hs:25-236, OpsConcrete.hs:777-904): arrays hold
-- their shape at run time, so a conversion between array kinds is the identity
-- on the device value, checked against the shape the target type names; a
-- scalar and a rank-0 array are the two forms of 'GpuIx'.

instance ConvertTensor Gpu where
  tconvert c astk a = convertGpu c astk a

  kfromR (Gpu v) = Gpu (valScalar v)
  kfromS (Gpu v) = Gpu (valScalar v)
  kfromX (Gpu v) = Gpu (valScalar v)
  rfromK @r (Gpu s) = Gpu (scalarVal (dtypeOf @r) s)
  rfromS (Gpu v) = Gpu v
  rfromX (Gpu v) = Gpu v
  sfromK @r (Gpu s) = Gpu (scalarVal (dtypeOf @r) s)
  sfromR @sh (Gpu v) = Gpu (checkedShape (shsToList (knownShS @sh)) v)
  sfromX @sh (Gpu v) = Gpu (checkedShape (shsToList (knownShS @sh)) v)
  xfromK @r (Gpu s) = Gpu (scalarVal (dtypeOf @r) s)
  xfromR (Gpu v) = Gpu v
  xfromS (Gpu v) = Gpu v

  rzip _ = nestedArrays "rzip"
  runzip _ = nestedArrays "runzip"
  szip _ = nestedArrays "szip"
  sunzip _ = nestedArrays "sunzip"
  xzip _ = nestedArrays "xzip"
  xunzip _ = nestedArrays "xunzip"
  xnestR _ _ = nestedArrays "xnestR"
  xnestS _ _ = nestedArrays "xnestS"
  xnest _ _ = nestedArrays "xnest"
  xunNestR _ = nestedArrays "xunNestR"
  xunNestS _ = nestedArrays "xunNestS"
  xunNest _ = nestedArrays "xunNest"

  tpairConv = tpair
  tunpairConv = tunpair

checkedShape :: [Int] -> ValPtr -> ValPtr
checkedShape want v
  | gpuShape v == want = v
  | otherwise = error ("the array has shape " ++ show (gpuShape v) ++ ", the shaped type names " ++ show want)

-- | The universal conversion, by recursion on the recipe (Conversion.hs:37-73).
convertGpu :: TKConversion a b -> SingletonTK a -> Gpu a -> Gpu b
convertGpu c0 astk a = case c0 of
  ConvId -> a
  ConvCmp c2 c1 -> convertGpu c2 (convertSTK c1 astk) (convertGpu c1 astk a)
  ConvRX -> Gpu (unGpu a)
  ConvSX -> Gpu (unGpu a)
  ConvXR _ -> Gpu (unGpu a)
  ConvXS -> Gpu (unGpu a)
  ConvXS' (FTKS sh _) -> Gpu (checkedShape (shsToList sh) (unGpu a))
  ConvXX' (FTKX sh _) -> Gpu (checkedShape (shxToList' sh) (unGpu a))
  ConvRR c | Just Refl <- isIdentity c -> a
  ConvSS c | Just Refl <- isIdentity c -> a
  ConvXX c | Just Refl <- isIdentity c -> a
  ConvT2 c1 c2 | STKProduct s1 s2 <- astk ->
    tpair (convertGpu c1 s1 (tproject1 a)) (convertGpu c2 s2 (tproject2 a))
  Conv0X STKScalar | STKScalar @r <- astk -> Gpu (scalarVal (dtypeOf @r) (unGpu a))
  ConvX0 | STKX _ STKScalar <- astk -> Gpu (valScalar (unGpu a))
  _ -> nestedArrays "tconvert"
 where
  isIdentity :: TKConversion x y -> Maybe (x :~: y)
  isIdentity ConvId = Just Refl
  isIdentity _ = Nothing

-- * Interpreting a gradient artifact at the carrier

-- | revInterpretArtifact (src/HordeAd/ADEngine.hs:266-288) with @Gpu@ for
-- @Concrete@: the same environment, the same check of the incoming cotangent's
-- shape, the same order of the results (primal first).
revInterpretArtifactGpu
  :: forall x z. TKAllNum (ADTensorKind z)
  => AstArtifactRev x z
  -> Gpu x
  -> Maybe (Gpu (ADTensorKind z))
  -> (Gpu z, Gpu (ADTensorKind x))
revInterpretArtifactGpu AstArtifactRev{..} parameters mdt =
  let azftk = varNameToFTK artVarDtRev
      env = extendEnv artVarDomainRev parameters emptyEnv
      envDt = case mdt of
        Nothing -> extendEnv artVarDtRev (treplTarget 1 azftk) env
        Just dt ->
          if tftk (ftkToSTK azftk) dt == azftk
          then extendEnv artVarDtRev dt env
          else error $ "revInterpretArtifactGpu: reverse derivative incoming cotangent must have the same shape as the codomain of the objective function: "
                       ++ show (tftk (ftkToSTK azftk) dt, azftk)
      gradient = interpretAstFull envDt artDerivativeRev
      primal = interpretAstFull env artPrimalRev
  in (primal, gradient)

-- | The same artifact recorded once as a device graph: returns the results and
-- an action that re-runs the whole gradient in one submission, refreshing (in
-- place) the arrays behind them.  Call 'revInterpretArtifactGpu' once
-- beforehand so that constants and generated kernels exist; feed new inputs
-- with @hh_overwrite@ on the arrays of @parameters@, which the caller keeps
-- alive as long as the action is used.
recordArtifactGpu
  :: forall x z. TKAllNum (ADTensorKind z)
  => SingletonTK x -> SingletonTK z
  -> AstArtifactRev x z -> Gpu x -> Maybe (Gpu (ADTensorKind z))
  -> IO ((Gpu z, Gpu (ADTensorKind x)), IO ())
recordArtifactGpu xstk zstk art parameters mdt = do
  ctx <- theCtx
  c_hh_capture_begin ctx >>= check ctx
  let r@(v, g) = revInterpretArtifactGpu art parameters mdt
  mapM_ (forceVal ctx) (arraysOf zstk v ++ arraysOf (adSTK xstk) g)
  gr <- alloca $ \o -> c_hh_capture_end ctx o >>= check ctx >> peek o
  pure (r, c_hh_graph_launch ctx gr >>= check ctx)
 where
  forceVal ctx v = withForeignPtr v $ \p -> c_hh_force ctx p >>= check ctx

-- | Every device array of a value, scalars included when they are device values.
arraysOf :: SingletonTK y -> Gpu y -> [ValPtr]
arraysOf stk (Gpu v) = case stk of
  STKScalar -> case v of
    GpuIxVal p -> [p]
    _ -> []
  STKR{} -> [v]
  STKS{} -> [v]
  STKX{} -> [v]
  STKProduct s1 s2 -> arraysOf s1 (Gpu (fst v)) ++ arraysOf s2 (Gpu (snd v))
