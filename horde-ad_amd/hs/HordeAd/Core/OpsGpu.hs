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
-- the result's shape is put together for the type.  Methods that are
-- polymorphic in the element kind @x@ (indexing, gather, scatter, the views,
-- replicate, sum, stacking) make that call once per device array of the value
-- ('arrMap': an array of pairs is a pair of arrays, an array of arrays one
-- array with the inner dims behind the outer ones).
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

-- | The outer dims of an array value of any element kind: the first @n@ dims of its first device array.
outerDims :: SingletonTK x -> Int -> ArrGpu x -> [Int]
outerDims stk n a = take n (gpuShape (head (arrLeaves stk a)))

-- | Reshape of the outer dims (the first @nOld@ of them) with whatever inner dims there are kept behind.
reshapeOuter :: Int -> [Int] -> ValPtr -> ValPtr
reshapeOuter nOld new v = reshapeTo (new ++ drop nOld (gpuShape v)) v

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

  rshape @n @x (Gpu v) = shrOf (outerDims (knownSTK @x) (valueOf @n) v)
  sshape @sh @x (Gpu v) = shsOf (outerDims (knownSTK @x) (shsLength (knownShS @sh)) v)
  xshape @sh @x (Gpu v) =
    let v0 = head (arrLeaves (knownSTK @x) v)
        n = ssxLength (mixedSkeleton @sh v0)
    in shxOf (mixedSkeleton @sh v0) (take n (gpuShape v0))
  tftk stk (Gpu v) = case stk of             -- CarriersConcrete.hs:164 (tftkG)
    STKScalar -> FTKScalar
    STKR n x -> FTKR (shrOf (outerDims x (fromSNat' n) v)) (elemFTK x (fromSNat' n) v)
    STKS sh x -> FTKS sh (elemFTK x (shsLength sh) v)
    STKX ssx x -> FTKX (shxOf ssx (outerDims x (ssxLength ssx) v)) (elemFTK x (ssxLength ssx) v)
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
    -- arrays of arrays and of pairs: unzipped and unnested on the host (both free in ox-arrays), then uploaded leaf by leaf
    FTKR sh x -> Gpu (uploadNested (ftkToSTK x) (Foldable.toList sh) (Nested.rtoMixed a))
    FTKS sh x -> Gpu (uploadNested (ftkToSTK x) (shsToList sh) (Nested.stoMixed a))
    FTKX sh x -> Gpu (uploadNested (ftkToSTK x) (shxToList' sh) a)

  -- :125-214
  trfromVectorN @_ @x shm v = stackOf (knownSTK @x) (Foldable.toList shm) (V.toList v)
  trfromVectorLinear @_ @r shm v = Gpu (stackVals (Foldable.toList shm) [] (map (scalarVal (dtypeOf @r) . unGpu) (V.toList v)))
  tsfromVectorN @_ @_ @x shm v = stackOf (knownSTK @x) (shsToList shm) (V.toList v)
  tsfromVectorLinear @_ @r shm v = Gpu (stackVals (shsToList shm) [] (map (scalarVal (dtypeOf @r) . unGpu) (V.toList v)))
  txfromVectorN @_ @_ @x shm v = stackOf (knownSTK @x) (shxToList' shm) (V.toList v)
  txfromVectorLinear @_ @r shm v = Gpu (stackVals (shxToList' shm) [] (map (scalarVal (dtypeOf @r) . unGpu) (V.toList v)))

  trsumN @m @_ @x (Gpu t) = Gpu (arrMap (knownSTK @x) (sumPrefix (valueOf @m)) t)      -- :215-230
  trsum0 (Gpu t) = Gpu (valScalar (un1 c_hh_tssum0 t))
  trdot0 (Gpu a) (Gpu b) = Gpu (valScalar (bin c_hh_tsdot0 a b))
  trdot1In (Gpu a) (Gpu b) = Gpu (bin c_hh_tsdot1In a b)
  trmatvecmul (Gpu m) (Gpu v) = Gpu (bin c_hh_tsmatvecmul m v)
  trmatmul2 (Gpu a) (Gpu b) = Gpu (bin c_hh_tsmatmul2 a b)
  trreplicateN @_ @_ @x shm (Gpu t) = Gpu (arrMap (knownSTK @x) (replicatePrefix (Foldable.toList shm)) t)
  trreplicate0N @_ @r shm (Gpu s) = Gpu (replicatePrefix (Foldable.toList shm) (scalarVal (dtypeOf @r) s))

  tssumN @shm @_ @x (Gpu t) = Gpu (arrMap (knownSTK @x) (sumPrefix (shsLength (knownShS @shm))) t)
  tssum0 (Gpu t) = Gpu (valScalar (un1 c_hh_tssum0 t))
  tsdot0 (Gpu a) (Gpu b) = Gpu (valScalar (bin c_hh_tsdot0 a b))                     -- :231
  tsdot1In _ (Gpu a) (Gpu b) = Gpu (bin c_hh_tsdot1In a b)                           -- :233
  tsmatvecmul (Gpu m) (Gpu v) = Gpu (bin c_hh_tsmatvecmul m v)                       -- :236
  tsmatmul2 (Gpu a) (Gpu b) = Gpu (bin c_hh_tsmatmul2 a b)                           -- :237
  tsreplicateN @_ @_ @x shm (Gpu t) = Gpu (arrMap (knownSTK @x) (replicatePrefix (shsToList shm)) t)   -- :243
  tsreplicate0N @_ @r shm (Gpu s) = Gpu (replicatePrefix (shsToList shm) (scalarVal (dtypeOf @r) s))

  txsumN @shm @_ @x (Gpu t) = Gpu (arrMap (knownSTK @x) (sumPrefix (ssxLength (knownShX @shm))) t)
  txsum0 (Gpu t) = Gpu (valScalar (un1 c_hh_tssum0 t))
  txdot0 (Gpu a) (Gpu b) = Gpu (valScalar (bin c_hh_tsdot0 a b))
  txdot1In _ (Gpu a) (Gpu b) = Gpu (bin c_hh_tsdot1In a b)
  txmatvecmul _ _ (Gpu m) (Gpu v) = Gpu (bin c_hh_tsmatvecmul m v)
  txmatmul2 (Gpu a) (Gpu b) = Gpu (bin c_hh_tsmatmul2 a b)
  txreplicateN @_ @_ @x shm (Gpu t) = Gpu (arrMap (knownSTK @x) (replicatePrefix (shxToList' shm)) t)
  txreplicate0N @_ @r shm (Gpu s) = Gpu (replicatePrefix (shxToList' shm) (scalarVal (dtypeOf @r) s))

  -- :246-360: indexing, gather, scatter
  -- (the index function is applied once per device array of the value: it is pure, and the host layer
  -- recognises equal index lanes)
  trindex @_ @_ @x (Gpu t) ix = Gpu (arrMap (knownSTK @x) (indexPrefix (ixList ix)) t)
  trindex0 (Gpu t) ix = Gpu (valScalar (indexPrefix (ixList ix) t))
  trscatter @m @_ @_ @x shp (Gpu t) f =
    Gpu (arrMap (knownSTK @x) (\v -> scatterBy (take (valueOf @m) (gpuShape v)) (Foldable.toList shp) v (viaIxR f)) t)
  trgather @_ @_ @_ @x shm (Gpu t) f = Gpu (arrMap (knownSTK @x) (\v -> gatherBy (Foldable.toList shm) v (viaIxR f)) t)
  tsindex @_ @_ @x (Gpu t) ix = Gpu (arrMap (knownSTK @x) (indexPrefix (ixList ix)) t)
  tsindex0 (Gpu t) ix = Gpu (valScalar (indexPrefix (ixList ix) t))
  tsscatter @shm @_ @shp @x (Gpu t) f =
    Gpu (arrMap (knownSTK @x) (\v -> scatterBy (shsToList (knownShS @shm)) (shsToList (knownShS @shp)) v (viaIxS f)) t)
  tsgather @shm @_ @_ @x (Gpu t) f = Gpu (arrMap (knownSTK @x) (\v -> gatherBy (shsToList (knownShS @shm)) v (viaIxS f)) t)
  txindex @_ @_ @x (Gpu t) ix = Gpu (arrMap (knownSTK @x) (indexPrefix (ixList ix)) t)
  txindex0 (Gpu t) ix = Gpu (valScalar (indexPrefix (ixList ix) t))
  txscatter @shm @_ @_ @x shp (Gpu t) f =
    Gpu (arrMap (knownSTK @x) (\v -> scatterBy (take (ssxLength (knownShX @shm)) (gpuShape v)) (shxToList' shp) v (viaIxX f)) t)
  txgather @_ @_ @_ @x shm (Gpu t) f = Gpu (arrMap (knownSTK @x) (\v -> gatherBy (shxToList' shm) v (viaIxX f)) t)

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
  trappend @_ @x (Gpu a) (Gpu b) = Gpu (arrZip (knownSTK @x) (bin c_hh_tsappend) a b)
  trslice @_ @x i n (Gpu t) = Gpu (arrMap (knownSTK @x) (sliceOuter i n) t)
  trreverse @_ @x (Gpu t) = Gpu (arrMap (knownSTK @x) (un1 c_hh_tsreverse) t)
  trtranspose @_ @x perm (Gpu t) = Gpu (arrMap (knownSTK @x) (transposeBy perm) t)
  trreshape @n @_ @x sh (Gpu t) = Gpu (arrMap (knownSTK @x) (reshapeOuter (valueOf @n) (Foldable.toList sh)) t)
  tsappend @_ @_ @_ @x (Gpu a) (Gpu b) = Gpu (arrZip (knownSTK @x) (bin c_hh_tsappend) a b)                      -- :638
  tsslice @_ @_ @_ @_ @x i n _ (Gpu t) = Gpu (arrMap (knownSTK @x) (sliceOuter (fromSNat' i) (fromSNat' n)) t)   -- :641
  tsreverse @_ @_ @x (Gpu t) = Gpu (arrMap (knownSTK @x) (un1 c_hh_tsreverse) t)                                  -- :644
  tstranspose @_ @_ @x perm (Gpu t) = Gpu (arrMap (knownSTK @x) (transposeBy (Permutation.permToList' perm)) t)   -- :647
  tsreshape @sh @_ @x sh2 (Gpu t) = Gpu (arrMap (knownSTK @x) (reshapeOuter (shsLength (knownShS @sh)) (shsToList sh2)) t)   -- :650
  txappend @_ @_ @_ @x (Gpu a) (Gpu b) = Gpu (arrZip (knownSTK @x) (bin c_hh_tsappend) a b)
  txslice @_ @_ @_ @_ @x i n _ (Gpu t) = Gpu (arrMap (knownSTK @x) (sliceOuter (fromSMayNat' i) (fromSMayNat' n)) t)
  txreverse @_ @_ @x (Gpu t) = Gpu (arrMap (knownSTK @x) (un1 c_hh_tsreverse) t)
  txtranspose @_ @_ @x perm (Gpu t) = Gpu (arrMap (knownSTK @x) (transposeBy (Permutation.permToList' perm)) t)
  txreshape @sh @_ @x sh2 (Gpu t) = Gpu (arrMap (knownSTK @x) (reshapeOuter (ssxLength (knownShX @sh)) (shxToList' sh2)) t)

  -- :661-740.  A build or a map whose closure yields SCALARS runs the closure once,
  -- on lanes (the position variables of the index space, or the array's own
  -- elements: hh_ix_from_val), and writes the resulting lane out as an array
  -- (hh_ix_to_val): one fused pass on the device, where Concrete runs one vector
  -- generate / map (tbuildK :1081-1087, tmap0NS / tzipWith0NS :1748-1759).
  tkbuild1 @k @r f = Gpu (laneToArr (dtypeOf @r) [valueOf @k] (unGpu (f (Gpu (head (laneVars [valueOf @k]))))))
  tkbuild @sh @r f =
    let shm = shsToList (knownShS @sh)
    in Gpu (laneToArr (dtypeOf @r) shm (unGpu (f (fromList' (laneVars shm)))))
  trmap0N @_ @_ @r f (Gpu v) = Gpu (laneToArr (dtypeOf @r) (gpuShape v) (unGpu (f (Gpu (arrToLane v)))))
  trzipWith0N @_ @r f (Gpu u) (Gpu v) = Gpu (laneToArr (dtypeOf @r) (gpuShape u) (unGpu (f (Gpu (arrToLane u)) (Gpu (arrToLane v)))))
  tsmap0N @_ @_ @r f (Gpu v) = Gpu (laneToArr (dtypeOf @r) (gpuShape v) (unGpu (f (Gpu (arrToLane v)))))      -- :708
  tszipWith0N @_ @r f (Gpu u) (Gpu v) = Gpu (laneToArr (dtypeOf @r) (gpuShape u) (unGpu (f (Gpu (arrToLane u)) (Gpu (arrToLane v)))))   -- :710-714
  -- A build whose closure yields ARRAYS is the reference's host loop (tbuild1S,
  -- :1761-1774): the closure may do anything a tensor program does, so it runs
  -- once per index, and the results are stacked.
  trbuild1 @_ @x k f = stackOf (knownSTK @x) [k] [f (Gpu (literal i)) | i <- [0 .. k - 1]]
  tsbuild1 @k @_ @x f = stackOf (knownSTK @x) [valueOf @k] [f (Gpu (literal i)) | i <- [0 .. valueOf @k - 1 :: Int]]
  txbuild1 @k @_ @x f = stackOf (knownSTK @x) [valueOf @k] [f (Gpu (literal i)) | i <- [0 .. valueOf @k - 1 :: Int]]

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
  | Just Refl <- testEquality (typeRep @r) (typeRep @Int), abs x < 2 ^ (53 :: Int) = GpuIxLit (fromIntegral x)      -- exact as a Double
  | Just Refl <- testEquality (typeRep @r) (typeRep @Int64), abs x < 2 ^ (53 :: Int) = GpuIxLit (fromIntegral x)
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

-- | The shape of the elements of an array value: what lies behind the first @n@ (outer) dims of its device arrays.
elemFTK :: SingletonTK x -> Int -> ArrGpu x -> FullShapeTK x
elemFTK stk n a = case stk of
  STKScalar -> FTKScalar
  STKR m x -> FTKR (shrOf (take (fromSNat' m) (drop n (gpuShape (head (arrLeaves x a)))))) (elemFTK x (n + fromSNat' m) a)
  STKS sh x -> FTKS sh (elemFTK x (n + shsLength sh) a)
  STKX ssx x -> FTKX (shxOf ssx (take (ssxLength ssx) (drop n (gpuShape (head (arrLeaves x a)))))) (elemFTK x (n + ssxLength ssx) a)
  STKProduct s1 s2 -> FTKProduct (elemFTK s1 n (fst a)) (elemFTK s2 n (snd a))

-- | A host array of any element kind onto the device: pairs are unzipped, inner arrays unnested
-- (their dims join the outer ones), scalars uploaded with the dims collected on the way.
uploadNested :: SingletonTK x -> [Int] -> Nested.Mixed sh (RepConcrete x) -> ArrGpu x
uploadNested stk outer a = case stk of
  STKScalar -> uploadArr (outer ++ drop (length outer) (shxToList' (Nested.mshape a))) (Nested.mtoVector a)
  STKProduct s1 s2 | Dict <- eltDictRep s1, Dict <- eltDictRep s2 ->
    let (a1, a2) = Nested.munzip a in (uploadNested s1 outer a1, uploadNested s2 outer a2)
  STKR _ x | Dict <- eltDictRep x ->
    let flat = Nested.munNest (Nested.convert (Nested.ConvXX Nested.ConvRX) a)
    in uploadNested x (shxToList' (Nested.mshape flat)) flat
  STKS _ x | Dict <- eltDictRep x ->
    let flat = Nested.munNest (Nested.convert (Nested.ConvXX Nested.ConvSX) a)
    in uploadNested x (shxToList' (Nested.mshape flat)) flat
  STKX _ x | Dict <- eltDictRep x ->
    let flat = Nested.munNest a
    in uploadNested x (shxToList' (Nested.mshape flat)) flat

shxToList' :: IShX sh -> [Int]
shxToList' = Foldable.toList

condArr :: RepGpu y ~ ValPtr => GpuIx -> Gpu y -> Gpu y -> Gpu y
condArr (GpuIxLit c) u v = if c /= 0 then u else v
condArr b (Gpu u) (Gpu v) = Gpu $ out1 $ \ctx o ->
  let cond = replicatePrefix (gpuShape u) (scalarVal 6 b)
  in withForeignPtr cond $ \pc -> withForeignPtr u $ \pu -> withForeignPtr v $ \pv -> c_hh_select ctx pc pu pv o

-- | Array values of one element kind stacked along new outer dims @shm@, device array by device array.
stackOf :: (RepGpu y ~ ArrGpu x, RepGpu z ~ ArrGpu x) => SingletonTK x -> [Int] -> [Gpu y] -> Gpu z
stackOf stk shm vs = case vs of
  [] -> error "fromVector: an empty vector carries no element shape"
  _ -> Gpu (arrZipN stk (\leaves -> stackVals shm (gpuShape (head leaves)) leaves) (map unGpu vs))

-- | A lane written out as an array of shape @shm@ (a literal or a rank-0 value is replicated).
laneToArr :: CInt -> [Int] -> GpuIx -> ValPtr
laneToArr dt shm s = out1 $ \ctx o -> withForeignPtr (laneOf dt shm s) $ \p -> c_hh_ix_to_val ctx p o

-- | The elements of an array as a lane over the array's own index space.
arrToLane :: ValPtr -> GpuIx
arrToLane v = GpuIxLane (gpuShape v) (outIx $ \ctx o -> withForeignPtr v $ \p -> c_hh_ix_from_val ctx p o)

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
  STKR _ x -> stackOf x [fromSNat' snat] l
  STKS _ x -> stackOf x [fromSNat' snat] l
  STKX _ x -> stackOf x [fromSNat' snat] l
  STKProduct s1 s2 ->
    tpair (fromListGpu snat s1 (map tproject1 l)) (fromListGpu snat s2 (map tproject2 l))

-- * ConvertTensor (ConvertTensor.hs:25-236, OpsConcrete.hs:777-904): arrays hold
-- their shape at run time, so a conversion between array kinds is the identity
-- on the device value, checked against the shape the target type names; a
-- scalar and a rank-0 array are the two forms of 'GpuIx'; zip / unzip / nest /
-- unnest relate two types of one representation ('ArrGpu').

instance ConvertTensor Gpu where
  tconvert c astk a = convertGpu c astk a

  kfromR (Gpu v) = Gpu (valScalar v)
  kfromS (Gpu v) = Gpu (valScalar v)
  kfromX (Gpu v) = Gpu (valScalar v)
  rfromK @r (Gpu s) = Gpu (scalarVal (dtypeOf @r) s)
  rfromS (Gpu v) = Gpu v
  rfromX (Gpu v) = Gpu v
  sfromK @r (Gpu s) = Gpu (scalarVal (dtypeOf @r) s)
  sfromR @sh @x (Gpu v) = Gpu (arrMap (knownSTK @x) (checkedOuter (shsToList (knownShS @sh))) v)
  sfromX @sh @_ @x (Gpu v) = Gpu (arrMap (knownSTK @x) (checkedOuter (shsToList (knownShS @sh))) v)
  xfromK @r (Gpu s) = Gpu (scalarVal (dtypeOf @r) s)
  xfromR (Gpu v) = Gpu v
  xfromS (Gpu v) = Gpu v

  -- :821-876.  An array of pairs IS the pair of arrays, an array of arrays IS the flat array
  -- ('ArrGpu'): the two sides of each of these have one representation, and no data moves.
  rzip (Gpu p) = Gpu p
  runzip (Gpu p) = Gpu p
  szip (Gpu p) = Gpu p
  sunzip (Gpu p) = Gpu p
  xzip (Gpu p) = Gpu p
  xunzip (Gpu p) = Gpu p
  xnestR _ (Gpu a) = Gpu a
  xnestS _ (Gpu a) = Gpu a
  xnest _ (Gpu a) = Gpu a
  xunNestR (Gpu a) = Gpu a
  xunNestS (Gpu a) = Gpu a
  xunNest (Gpu a) = Gpu a

  tpairConv = tpair
  tunpairConv = tunpair

checkedShape :: [Int] -> ValPtr -> ValPtr
checkedShape want v
  | gpuShape v == want = v
  | otherwise = error ("the array has shape " ++ show (gpuShape v) ++ ", the shaped type names " ++ show want)

-- | The same check on the outer dims of a device array that may carry inner dims behind them.
checkedOuter :: [Int] -> ValPtr -> ValPtr
checkedOuter want v
  | take (length want) (gpuShape v) == want = v
  | otherwise = error ("the array has outer shape " ++ show (take (length want) (gpuShape v)) ++ ", the shaped type names " ++ show want)

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
  -- a conversion of the elements: arrays of arrays and of pairs share their elements' representation,
  -- so only the shape checks inside the recipe are left of it
  ConvRR c | STKR _ x <- astk -> convertElems c x a
  ConvSS c | STKS _ x <- astk -> convertElems c x a
  ConvXX c | STKX _ x <- astk -> convertElems c x a
  ConvNest _ -> Gpu (unGpu a)
  ConvUnnest -> Gpu (unGpu a)
  ConvZip _ _ -> Gpu (unGpu a)
  ConvUnzip _ _ -> Gpu (unGpu a)
  ConvT2 c1 c2 | STKProduct s1 s2 <- astk ->
    tpair (convertGpu c1 s1 (tproject1 a)) (convertGpu c2 s2 (tproject2 a))
  Conv0X STKScalar | STKScalar @r <- astk -> Gpu (scalarVal (dtypeOf @r) (unGpu a))
  ConvX0 | STKX _ STKScalar <- astk -> Gpu (valScalar (unGpu a))
 where
  -- the element conversions that change the representation are the two between a scalar and a
  -- rank-0 array (Conv0X / ConvX0): inside an array both are a device array already
  convertElems :: forall x y f g. (RepGpu (f x) ~ ArrGpu x, RepGpu (g y) ~ ArrGpu y)
               => TKConversion x y -> SingletonTK x -> Gpu (f x) -> Gpu (g y)
  convertElems c x (Gpu v) = Gpu (elemsAs c x v)
  elemsAs :: TKConversion x y -> SingletonTK x -> ArrGpu x -> ArrGpu y
  elemsAs c x v = case c of
    ConvId -> v
    ConvCmp c2 c1 -> elemsAs c2 (convertSTK c1 x) (elemsAs c1 x v)
    ConvRX -> v
    ConvSX -> v
    ConvXR _ -> v
    ConvXS -> v
    ConvXS' _ -> v
    ConvXX' _ -> v
    ConvRR c' | STKR _ x' <- x -> elemsAs c' x' v
    ConvSS c' | STKS _ x' <- x -> elemsAs c' x' v
    ConvXX c' | STKX _ x' <- x -> elemsAs c' x' v
    ConvT2 c1 c2 | STKProduct s1 s2 <- x -> (elemsAs c1 s1 (fst v), elemsAs c2 s2 (snd v))
    Conv0X _ -> v
    ConvX0 -> v
    ConvNest _ -> v
    ConvUnnest -> v
    ConvZip _ _ -> v
    ConvUnzip _ _ -> v

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
