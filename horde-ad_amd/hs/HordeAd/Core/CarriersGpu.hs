{-# LANGUAGE AllowAmbiguousTypes, DataKinds, RoleAnnotations, ScopedTypeVariables,
             StandaloneDeriving, TypeApplications, TypeFamilies, TypeOperators,
             UndecidableInstances #-}
-- | The GPU carrier: the counterpart of @Concrete@
-- (src/HordeAd/Core/CarriersConcrete.hs:150-155, 293-343).
--
-- * Every array kind (@TKR@, @TKS@, @TKX@ of scalars) is a handle to a device
--   value of the host layer (include/hordead_host.h); the shape lives with the
--   value, so the three kinds share one representation and differ in what the
--   types promise.  An array of pairs is a pair of arrays, and an array of
--   arrays is one device array with the inner dims behind the outer ones
--   ('ArrGpu') -- the layout ox-arrays gives them on the CPU -- so zip, unzip,
--   nest and unnest (OpsConcrete.hs:821-876) move no data.
-- * A scalar (@TKScalar r@) is a 'GpuIx': a literal known on the host, a
--   rank-0 device value, or -- inside the closure of a gather, scatter or
--   build -- a /lane/: one scalar per position of the index space, all
--   positions at once (the C side's @hh_ix@).  The closure is therefore
--   applied ONCE, to lane variables, where the Concrete backend applies it
--   once per position (OpsConcrete.hs:1581-1665).
-- * Products are Haskell pairs, as in @RepConcrete@.
--
-- Not compiled in this repository's build environment (no GHC there): it is
-- written against horde-ad's modules as they are in the reference checkout.
module HordeAd.Core.CarriersGpu
  ( -- * The carrier
    Gpu (..), RepGpu, ArrGpu, GpuFun (..), GpuIx (..)
  , arrMap, arrZip, arrZipN, arrLeaves
    -- * Calling the host layer
  , out1, un1, bin, withShape, withIxArray, outIx
  , gpuShape, dtypeOf, scalarVal, valScalar, laneOf, literal
    -- * Opcodes of include/hordead_gpu.h
  , Op1 (..), Op2 (..), Cmp (..), op1Code, op2Code, cmpCode
  , arr1, arr2, arrCmp, sc1, sc2, scCmp, scSelect, scConvert
  ) where

import Prelude

import Control.DeepSeq (NFData (..))
import Data.Boolean (Boolean (..))
import Data.Int (Int16, Int32, Int64, Int8)
import Data.Kind (Type)
import Data.Type.Equality (testEquality, (:~:) (Refl))
import Foreign
import Foreign.C
import System.IO.Unsafe (unsafePerformIO)
import Type.Reflection (Typeable, typeRep)

import HordeAd.Core.TensorKind
import HordeAd.Core.Types
import HordeAd.Gpu.Foreign

-- * The carrier

type family RepGpu (y :: TK) :: Type where
  RepGpu (TKScalar r) = GpuIx
  RepGpu (TKR2 n x) = ArrGpu x
  RepGpu (TKS2 sh x) = ArrGpu x
  RepGpu (TKX2 sh x) = ArrGpu x
  RepGpu (TKProduct x z) = (RepGpu x, RepGpu z)

-- | An array (of any shape) whose elements have kind @x@.  Scalars: one device
-- array.  Pairs: a pair of arrays of one outer shape (struct of arrays, which is
-- how @Nested.Mixed sh (a, b)@ is laid out too).  Arrays: the element's array
-- with the inner dims trailing the outer ones, so that every operation on the
-- outer dims (index, gather, transpose of a prefix, append, sum over the
-- outermost dim) is the same call on the one flat array.
type family ArrGpu (x :: TK) :: Type where
  ArrGpu (TKScalar r) = ValPtr
  ArrGpu (TKR2 n x) = ArrGpu x
  ArrGpu (TKS2 sh x) = ArrGpu x
  ArrGpu (TKX2 sh x) = ArrGpu x
  ArrGpu (TKProduct x z) = (ArrGpu x, ArrGpu z)

-- | One call per device array of an array value.
arrMap :: SingletonTK x -> (ValPtr -> ValPtr) -> ArrGpu x -> ArrGpu x
arrMap stk f a = case stk of
  STKScalar -> f a
  STKR _ x -> arrMap x f a
  STKS _ x -> arrMap x f a
  STKX _ x -> arrMap x f a
  STKProduct s1 s2 -> (arrMap s1 f (fst a), arrMap s2 f (snd a))

-- | The same for two array values of one element kind (append, select, addition of cotangents).
arrZip :: SingletonTK x -> (ValPtr -> ValPtr -> ValPtr) -> ArrGpu x -> ArrGpu x -> ArrGpu x
arrZip stk f a b = case stk of
  STKScalar -> f a b
  STKR _ x -> arrZip x f a b
  STKS _ x -> arrZip x f a b
  STKX _ x -> arrZip x f a b
  STKProduct s1 s2 -> (arrZip s1 f (fst a) (fst b), arrZip s2 f (snd a) (snd b))

-- | ... for a list of them (stacking).
arrZipN :: SingletonTK x -> ([ValPtr] -> ValPtr) -> [ArrGpu x] -> ArrGpu x
arrZipN stk f as = case stk of
  STKScalar -> f as
  STKR _ x -> arrZipN x f as
  STKS _ x -> arrZipN x f as
  STKX _ x -> arrZipN x f as
  STKProduct s1 s2 -> (arrZipN s1 f (map fst as), arrZipN s2 f (map snd as))

-- | Every device array of an array value, leftmost first (all share the outer dims).
arrLeaves :: SingletonTK x -> ArrGpu x -> [ValPtr]
arrLeaves stk a = case stk of
  STKScalar -> [a]
  STKR _ x -> arrLeaves x a
  STKS _ x -> arrLeaves x a
  STKX _ x -> arrLeaves x a
  STKProduct s1 s2 -> arrLeaves s1 (fst a) ++ arrLeaves s2 (snd a)

type role Gpu nominal
newtype Gpu y = Gpu {unGpu :: RepGpu y}

-- | As for @Concrete@ (CarriersConcrete.hs:295-298): 'AllTargetShow' asks for it
-- (Ops.hs:1297-1313).  A device array shows as its element type, shape and elements
-- (downloaded: showing is for tests and error messages).
instance KnownSTK y => Show (Gpu y) where
  showsPrec d (Gpu t) = showsRep (knownSTK @y) d t

showsRep :: SingletonTK y -> Int -> RepGpu y -> ShowS
showsRep stk d t = case stk of
  STKScalar -> showsPrec d t
  STKR _ x -> showsArr x t
  STKS _ x -> showsArr x t
  STKX _ x -> showsArr x t
  STKProduct s1 s2 -> showParen (d > 10) $ showString "(" . showsRep s1 0 (fst t) . showString ", " . showsRep s2 0 (snd t) . showString ")"
 where
  showsArr :: SingletonTK x -> ArrGpu x -> ShowS
  showsArr x a = showString "gpu" . showList (map showVal (arrLeaves x a))

instance Show GpuIx where
  showsPrec d (GpuIxLit x) = showsPrec d x
  showsPrec _ (GpuIxVal v) = showString (showVal v)
  showsPrec _ (GpuIxLane shm _) = showString "<lane over " . shows shm . showString ">"

-- | dtype, shape and the elements of a device value as doubles (a synchronous read-back).
showVal :: ValPtr -> String
showVal v = unsafePerformIO $ do
  ctx <- theCtx
  let sh = gpuShape v
      n = product sh
  xs <- withForeignPtr (arr1AsDouble v) $ \p -> allocaArray (max 1 n) $ \buf -> do
    c_hh_download ctx p (castPtr buf) >>= check ctx
    peekArray n (buf :: Ptr Double)
  pure (show sh ++ " " ++ show xs)
 where
  arr1AsDouble = un1 (\c p -> c_hh_convert c p 0 0)       -- tscast to Double (dtype code 0), the identity on Double arrays

-- | Device values are evaluated when they are made: the calls are strict, the
-- kernels run in stream order.  Forcing the handles is all @rnf@ has to do
-- (CarriersConcrete.hs:297-298 forces the host arrays).
instance KnownSTK y => NFData (Gpu y) where
  rnf (Gpu t) = rnfRep (knownSTK @y) t

rnfRep :: SingletonTK y -> RepGpu y -> ()
rnfRep stk t = case stk of
  STKScalar -> case t of
    GpuIxLit x -> x `seq` ()
    GpuIxVal v -> v `seq` ()
    GpuIxLane _ x -> x `seq` ()
  STKR _ x -> foldr seq () (arrLeaves x t)
  STKS _ x -> foldr seq () (arrLeaves x t)
  STKX _ x -> foldr seq () (arrLeaves x t)
  STKProduct s1 s2 -> rnfRep s1 (fst t) `seq` rnfRep s2 (snd t)

type role GpuFun nominal nominal
newtype GpuFun x z = GpuFun (RepGpu x -> RepGpu z)
type instance HFunOf Gpu = GpuFun          -- CarriersConcrete.hs:304-305

type instance PrimalOf Gpu = Gpu            -- CarriersConcrete.hs:307-310
type instance DualOf Gpu = DummyDualTarget
type instance PlainOf Gpu = Gpu
type instance ShareOf Gpu = Gpu
-- BoolOf Gpu = PlainOf Gpu (TKScalar Bool) = Gpu (TKScalar Bool) and
-- IntOf Gpu = Gpu (TKScalar Int) are synonyms (Types.hs:242-244): both are 'GpuIx'.

-- | A scalar of the carrier.
data GpuIx
  = GpuIxLit Double          -- ^ a literal (@fromInteger@, @fromRational@, a host constant).  Integers are exact for
                             --   |n| < 2^53 -- every index is -- so @tkconcrete \@Int64@ of a larger value takes the
                             --   other road ('GpuIxVal', an uploaded rank-0 array: see @literal'@ in OpsGpu)
  | GpuIxVal ValPtr          -- ^ a rank-0 device value
  | GpuIxLane [Int] IxPtr    -- ^ one scalar per position of the space @shm@ (inside an index function)

-- * Calling the host layer

{-# NOINLINE out1 #-}
-- | Runs an entry point that makes one device value.  Device arrays are
-- immutable and the context enqueues in call order on one stream, so forcing
-- results in data-dependency order is all the ordering that is needed.
out1 :: (Ptr Ctx -> Ptr (Ptr Val) -> IO CInt) -> ValPtr
out1 f = unsafePerformIO $ do
  ctx <- theCtx
  p <- alloca $ \o -> f ctx o >>= check ctx >> peek o
  newForeignPtr p_hh_free p

{-# NOINLINE outIx #-}
outIx :: (Ptr Ctx -> Ptr (Ptr Ix) -> IO CInt) -> IxPtr
outIx f = unsafePerformIO $ do
  ctx <- theCtx
  p <- alloca $ \o -> f ctx o >>= check ctx >> peek o
  newForeignPtr p_hh_ix_free p

un1 :: (Ptr Ctx -> Ptr Val -> Ptr (Ptr Val) -> IO CInt) -> ValPtr -> ValPtr
un1 f a = out1 $ \ctx o -> withForeignPtr a $ \pa -> f ctx pa o

bin :: (Ptr Ctx -> Ptr Val -> Ptr Val -> Ptr (Ptr Val) -> IO CInt) -> ValPtr -> ValPtr -> ValPtr
bin f a b = out1 $ \ctx o -> withForeignPtr a $ \pa -> withForeignPtr b $ \pb -> f ctx pa pb o

withShape :: [Int] -> (CInt -> Ptr Int64 -> IO a) -> IO a
withShape sh k = withArrayLen (map fromIntegral sh) $ \n p -> k (fromIntegral n) p

-- | The lanes of an index function's result as the array of handles the C side takes.
withIxArray :: [IxPtr] -> (CInt -> Ptr (Ptr Ix) -> IO a) -> IO a
withIxArray ixs k = go ixs []
 where
  go [] acc = withArrayLen (reverse acc) $ \n p -> k (fromIntegral n) p
  go (x : xs) acc = withForeignPtr x $ \p -> go xs (p : acc)

-- | sshape / rshape / xshape (OpsConcrete.hs:99-106): host metadata, no sync.
gpuShape :: ValPtr -> [Int]
gpuShape v = unsafePerformIO $ withForeignPtr v $ \p -> do
  r <- fromIntegral <$> c_hh_val_rank p
  allocaArray (max 1 r) $ \buf -> do
    _ <- c_hh_val_shape p buf
    map (fromIntegral :: Int64 -> Int) <$> peekArray r buf

-- | The element type code of include/hordead_gpu.h (F64 .. BOOL) for the
-- reference's scalar whitelist (Types.hs:300-330).
dtypeOf :: forall r. Typeable r => CInt
dtypeOf
  | Just Refl <- testEquality (typeRep @r) (typeRep @Double) = 0
  | Just Refl <- testEquality (typeRep @r) (typeRep @Float) = 1
  | Just Refl <- testEquality (typeRep @r) (typeRep @Int64) = 2
  | Just Refl <- testEquality (typeRep @r) (typeRep @Int) = 2
  | Just Refl <- testEquality (typeRep @r) (typeRep @Int32) = 3
  | Just Refl <- testEquality (typeRep @r) (typeRep @CInt) = 3
  | Just Refl <- testEquality (typeRep @r) (typeRep @Int16) = 4
  | Just Refl <- testEquality (typeRep @r) (typeRep @Int8) = 5
  | Just Refl <- testEquality (typeRep @r) (typeRep @Bool) = 6
  | otherwise = error "dtypeOf: a scalar type outside the whitelist"

literal :: Real a => a -> GpuIx
literal = GpuIxLit . realToFrac

-- | A scalar as a rank-0 device value of element type @dt@.
scalarVal :: CInt -> GpuIx -> ValPtr
scalarVal dt (GpuIxLit x) = out1 $ \ctx o -> c_hh_constant ctx dt (realToFrac x) 0 nullPtr o
scalarVal _ (GpuIxVal v) = v
scalarVal _ (GpuIxLane _ _) =
  error "a scalar that depends on the position of an index function was used outside of it"

valScalar :: ValPtr -> GpuIx
valScalar = GpuIxVal

-- | A scalar as a lane of the position space @shm@.
laneOf :: CInt -> [Int] -> GpuIx -> IxPtr
laneOf dt shm (GpuIxLit x) = outIx $ \ctx o -> withShape shm $ \n sh -> c_hh_ix_const ctx n sh dt (realToFrac x) o
laneOf _ shm (GpuIxVal v) = outIx $ \ctx o -> withShape shm $ \n sh -> withForeignPtr v $ \p -> c_hh_ix_lift ctx n sh p o
laneOf _ shm (GpuIxLane shm' x)
  | shm == shm' = x
  | otherwise = error "index values of two different position spaces were combined"

-- * Opcodes (enum hgpu_op1 / hgpu_op2 / hgpu_cmp of include/hordead_gpu.h)

data Op1 = Neg | Abs | Signum | Recip | Exp | Log | Sqrt | Sin | Cos | Tan | Asin | Acos | Atan
         | Sinh | Cosh | Tanh | Asinh | Acosh | Atanh | Not
  deriving (Enum)
data Op2 = Add | Mul | Sub | Div | Pow | LogBase | Atan2 | Quot | Rem | RemScalar | Min | Max | And
  deriving (Enum)
data Cmp = Leq | Eq | Lt
  deriving (Enum)

op1Code :: Op1 -> CInt
op1Code = fromIntegral . fromEnum
op2Code :: Op2 -> CInt
op2Code = fromIntegral . fromEnum
cmpCode :: Cmp -> CInt
cmpCode = fromIntegral . fromEnum

-- arrays
arr1 :: Op1 -> ValPtr -> ValPtr
arr1 op = un1 (\c -> c_hh_ewise1 c (op1Code op))
arr2 :: Op2 -> ValPtr -> ValPtr -> ValPtr
arr2 op = bin (\c -> c_hh_ewise2 c (op2Code op))
arrCmp :: Cmp -> ValPtr -> ValPtr -> ValPtr
arrCmp op = bin (\c -> c_hh_compare c (cmpCode op))

-- scalars: two literals fold on the host, a lane on either side makes a lane,
-- otherwise rank-0 device values
sc1 :: CInt -> Op1 -> (Double -> Double) -> GpuIx -> GpuIx
sc1 _ _ f (GpuIxLit x) = GpuIxLit (f x)
sc1 _ op _ (GpuIxVal v) = GpuIxVal (arr1 op v)
sc1 _ op _ (GpuIxLane shm x) =
  GpuIxLane shm $ outIx $ \ctx o -> withForeignPtr x $ \p -> c_hh_ix_op1 ctx (op1Code op) p o

sc2 :: CInt -> Op2 -> (Double -> Double -> Double) -> GpuIx -> GpuIx -> GpuIx
sc2 _ _ f (GpuIxLit x) (GpuIxLit y) = GpuIxLit (f x y)
sc2 dt op _ a b = case (spaceOf a, spaceOf b) of
  (Nothing, Nothing) -> GpuIxVal (arr2 op (scalarVal dt a) (scalarVal dt b))
  (sa, sb) ->
    let shm = maybe (maybe [] id sb) id sa
    in GpuIxLane shm $ outIx $ \ctx o ->
         withForeignPtr (laneOf dt shm a) $ \pa -> withForeignPtr (laneOf dt shm b) $ \pb ->
           c_hh_ix_op2 ctx (op2Code op) pa pb o

scCmp :: CInt -> Cmp -> (Double -> Double -> Bool) -> GpuIx -> GpuIx -> GpuIx
scCmp _ _ f (GpuIxLit x) (GpuIxLit y) = GpuIxLit (if f x y then 1 else 0)
scCmp dt op _ a b = case (spaceOf a, spaceOf b) of
  (Nothing, Nothing) -> GpuIxVal (arrCmp op (scalarVal dt a) (scalarVal dt b))
  (sa, sb) ->
    let shm = maybe (maybe [] id sb) id sa
    in GpuIxLane shm $ outIx $ \ctx o ->
         withForeignPtr (laneOf dt shm a) $ \pa -> withForeignPtr (laneOf dt shm b) $ \pb ->
           c_hh_ix_compare ctx (cmpCode op) pa pb o

-- | kcond / ifH on scalars (OpsConcrete.hs:113-119; inside an index function AstCondK).
scSelect :: CInt -> GpuIx -> GpuIx -> GpuIx -> GpuIx
scSelect _ (GpuIxLit c) a b = if c /= 0 then a else b
scSelect dt c a b = case (spaceOf c, spaceOf a, spaceOf b) of
  (Nothing, Nothing, Nothing) ->
    GpuIxVal $ out1 $ \ctx o ->
      withForeignPtr (scalarVal 6 c) $ \pc -> withForeignPtr (scalarVal dt a) $ \pa ->
        withForeignPtr (scalarVal dt b) $ \pb -> c_hh_select ctx pc pa pb o
  (sc, sa, sb) ->
    let shm = head [s | Just s <- [sc, sa, sb]]
    in GpuIxLane shm $ outIx $ \ctx o ->
         withForeignPtr (laneOf 6 shm c) $ \pc -> withForeignPtr (laneOf dt shm a) $ \pa ->
           withForeignPtr (laneOf dt shm b) $ \pb -> c_hh_ix_select ctx pc pa pb o

-- | tkfloor / tkfromIntegral / tkcast (mode 1 = floor, 0 = cast).
scConvert :: CInt -> CInt -> GpuIx -> GpuIx
scConvert _ mode (GpuIxLit x) = GpuIxLit (if mode == 1 then fromIntegral (floor x :: Int64) else x)
scConvert dt mode (GpuIxVal v) = GpuIxVal $ un1 (\c p -> c_hh_convert c p dt mode) v
scConvert dt mode (GpuIxLane shm x) =
  GpuIxLane shm $ outIx $ \ctx o -> withForeignPtr x $ \p -> c_hh_ix_convert ctx p dt mode o

spaceOf :: GpuIx -> Maybe [Int]
spaceOf (GpuIxLane shm _) = Just shm
spaceOf _ = Nothing

-- * Numeric classes of scalars (CarriersConcrete.hs:334-343 derives them from the
-- representation; here they dispatch on the three forms of a scalar)

instance GoodScalar r => Num (Gpu (TKScalar r)) where
  Gpu a + Gpu b = Gpu (sc2 (dtypeOf @r) Add (+) a b)
  Gpu a * Gpu b = Gpu (sc2 (dtypeOf @r) Mul (*) a b)
  Gpu a - Gpu b = Gpu (sc2 (dtypeOf @r) Sub (-) a b)
  negate (Gpu a) = Gpu (sc1 (dtypeOf @r) Neg negate a)
  abs (Gpu a) = Gpu (sc1 (dtypeOf @r) Abs abs a)
  signum (Gpu a) = Gpu (sc1 (dtypeOf @r) Signum signum a)
  fromInteger = Gpu . GpuIxLit . fromInteger

instance (GoodScalar r, IntegralH r) => IntegralH (Gpu (TKScalar r)) where
  -- quotH a 0 = a, remH a 0 = a: the rule of scalars (Types.hs:395-419), opcode RemScalar
  quotH (Gpu a) (Gpu b) = Gpu (sc2 (dtypeOf @r) Quot (\x y -> if y == 0 then x else fromIntegral (quot (truncate x :: Int64) (truncate y))) a b)
  remH (Gpu a) (Gpu b) = Gpu (sc2 (dtypeOf @r) RemScalar (\x y -> if y == 0 then x else fromIntegral (rem (truncate x :: Int64) (truncate y))) a b)

instance (GoodScalar r, Fractional r) => Fractional (Gpu (TKScalar r)) where
  Gpu a / Gpu b = Gpu (sc2 (dtypeOf @r) Div (/) a b)
  recip (Gpu a) = Gpu (sc1 (dtypeOf @r) Recip recip a)
  fromRational = Gpu . GpuIxLit . fromRational

instance (GoodScalar r, Floating r) => Floating (Gpu (TKScalar r)) where
  pi = Gpu (GpuIxLit pi)
  exp (Gpu a) = Gpu (sc1 (dtypeOf @r) Exp exp a)
  log (Gpu a) = Gpu (sc1 (dtypeOf @r) Log log a)
  sqrt (Gpu a) = Gpu (sc1 (dtypeOf @r) Sqrt sqrt a)
  sin (Gpu a) = Gpu (sc1 (dtypeOf @r) Sin sin a)
  cos (Gpu a) = Gpu (sc1 (dtypeOf @r) Cos cos a)
  tan (Gpu a) = Gpu (sc1 (dtypeOf @r) Tan tan a)
  asin (Gpu a) = Gpu (sc1 (dtypeOf @r) Asin asin a)
  acos (Gpu a) = Gpu (sc1 (dtypeOf @r) Acos acos a)
  atan (Gpu a) = Gpu (sc1 (dtypeOf @r) Atan atan a)
  sinh (Gpu a) = Gpu (sc1 (dtypeOf @r) Sinh sinh a)
  cosh (Gpu a) = Gpu (sc1 (dtypeOf @r) Cosh cosh a)
  tanh (Gpu a) = Gpu (sc1 (dtypeOf @r) Tanh tanh a)
  asinh (Gpu a) = Gpu (sc1 (dtypeOf @r) Asinh asinh a)
  acosh (Gpu a) = Gpu (sc1 (dtypeOf @r) Acosh acosh a)
  atanh (Gpu a) = Gpu (sc1 (dtypeOf @r) Atanh atanh a)
  Gpu a ** Gpu b = Gpu (sc2 (dtypeOf @r) Pow (**) a b)
  logBase (Gpu a) (Gpu b) = Gpu (sc2 (dtypeOf @r) LogBase logBase a b)

instance (GoodScalar r, Floating r) => RealFloatH (Gpu (TKScalar r)) where
  atan2H (Gpu a) (Gpu b) = Gpu (sc2 (dtypeOf @r) Atan2 atan2 a b)

-- | Data.Boolean, as @deriving instance Boolean (Concrete (TKScalar Bool))@
-- (CarriersConcrete.hs:333).
instance Boolean (Gpu (TKScalar Bool)) where
  true = Gpu (GpuIxLit 1)
  false = Gpu (GpuIxLit 0)
  notB (Gpu a) = Gpu (sc1 6 Not (\x -> if x /= 0 then 0 else 1) a)
  Gpu a &&* Gpu b = Gpu (sc2 6 And (\x y -> if x /= 0 && y /= 0 then 1 else 0) a b)
  Gpu a ||* Gpu b = notB (notB (Gpu a) &&* notB (Gpu b))

instance GoodScalar r => EqH Gpu (TKScalar r) where       -- CarriersConcrete.hs:312-313
  Gpu u ==. Gpu v = Gpu (scCmp (dtypeOf @r) Eq (==) u v)
instance GoodScalar r => OrdH Gpu (TKScalar r) where      -- CarriersConcrete.hs:314-315
  Gpu u <=. Gpu v = Gpu (scCmp (dtypeOf @r) Leq (<=) u v)
  Gpu u <. Gpu v = Gpu (scCmp (dtypeOf @r) Lt (<) u v)

-- * Numeric classes of arrays.  @==.@ and @<=.@ on whole arrays are the
-- reference's: one Bool for the lexicographic comparison of the two arrays'
-- elements (hh_compare_all), as @rtoPrimitive u <= rtoPrimitive v@ is.

{-# NOINLINE compareAll #-}
compareAll :: Cmp -> ValPtr -> ValPtr -> GpuIx
compareAll op a b = unsafePerformIO $ do
  ctx <- theCtx
  withForeignPtr a $ \pa -> withForeignPtr b $ \pb -> alloca $ \out -> do
    c_hh_compare_all ctx (cmpCode op) pa pb out >>= check ctx
    r <- peek out
    pure (GpuIxLit (if r /= 0 then 1 else 0))

shapeless :: String -> a
shapeless what = error (what ++ ": the shape of the array is not known here (as for Concrete's ranked arrays)")

instance GoodScalar r => EqH Gpu (TKR n r) where
  Gpu u ==. Gpu v = Gpu (compareAll Eq u v)
instance GoodScalar r => OrdH Gpu (TKR n r) where
  Gpu u <=. Gpu v = Gpu (compareAll Leq u v)
instance GoodScalar r => EqH Gpu (TKS sh r) where
  Gpu u ==. Gpu v = Gpu (compareAll Eq u v)
instance GoodScalar r => OrdH Gpu (TKS sh r) where
  Gpu u <=. Gpu v = Gpu (compareAll Leq u v)
instance GoodScalar r => EqH Gpu (TKX sh r) where
  Gpu u ==. Gpu v = Gpu (compareAll Eq u v)
instance GoodScalar r => OrdH Gpu (TKX sh r) where
  Gpu u <=. Gpu v = Gpu (compareAll Leq u v)

instance GoodScalar r => Num (Gpu (TKR n r)) where
  Gpu a + Gpu b = Gpu (arr2 Add a b)
  Gpu a * Gpu b = Gpu (arr2 Mul a b)
  Gpu a - Gpu b = Gpu (arr2 Sub a b)
  negate (Gpu a) = Gpu (arr1 Neg a)
  abs (Gpu a) = Gpu (arr1 Abs a)
  signum (Gpu a) = Gpu (arr1 Signum a)
  fromInteger _ = shapeless "fromInteger"
instance GoodScalar r => Num (Gpu (TKS sh r)) where
  Gpu a + Gpu b = Gpu (arr2 Add a b)
  Gpu a * Gpu b = Gpu (arr2 Mul a b)
  Gpu a - Gpu b = Gpu (arr2 Sub a b)
  negate (Gpu a) = Gpu (arr1 Neg a)
  abs (Gpu a) = Gpu (arr1 Abs a)
  signum (Gpu a) = Gpu (arr1 Signum a)
  fromInteger _ = shapeless "fromInteger"
instance GoodScalar r => Num (Gpu (TKX sh r)) where
  Gpu a + Gpu b = Gpu (arr2 Add a b)
  Gpu a * Gpu b = Gpu (arr2 Mul a b)
  Gpu a - Gpu b = Gpu (arr2 Sub a b)
  negate (Gpu a) = Gpu (arr1 Neg a)
  abs (Gpu a) = Gpu (arr1 Abs a)
  signum (Gpu a) = Gpu (arr1 Signum a)
  fromInteger _ = shapeless "fromInteger"

-- quotH / remH on arrays: a zero divisor yields 0 (the array rule of ox-arrays, opcode Rem)
instance (GoodScalar r, IntegralH r) => IntegralH (Gpu (TKR n r)) where
  quotH (Gpu a) (Gpu b) = Gpu (arr2 Quot a b)
  remH (Gpu a) (Gpu b) = Gpu (arr2 Rem a b)
instance (GoodScalar r, IntegralH r) => IntegralH (Gpu (TKS sh r)) where
  quotH (Gpu a) (Gpu b) = Gpu (arr2 Quot a b)
  remH (Gpu a) (Gpu b) = Gpu (arr2 Rem a b)
instance (GoodScalar r, IntegralH r) => IntegralH (Gpu (TKX sh r)) where
  quotH (Gpu a) (Gpu b) = Gpu (arr2 Quot a b)
  remH (Gpu a) (Gpu b) = Gpu (arr2 Rem a b)

instance (GoodScalar r, Fractional r) => Fractional (Gpu (TKR n r)) where
  Gpu a / Gpu b = Gpu (arr2 Div a b)
  recip (Gpu a) = Gpu (arr1 Recip a)
  fromRational _ = shapeless "fromRational"
instance (GoodScalar r, Fractional r) => Fractional (Gpu (TKS sh r)) where
  Gpu a / Gpu b = Gpu (arr2 Div a b)
  recip (Gpu a) = Gpu (arr1 Recip a)
  fromRational _ = shapeless "fromRational"
instance (GoodScalar r, Fractional r) => Fractional (Gpu (TKX sh r)) where
  Gpu a / Gpu b = Gpu (arr2 Div a b)
  recip (Gpu a) = Gpu (arr1 Recip a)
  fromRational _ = shapeless "fromRational"

floatingArr :: RepGpu y ~ ValPtr => Op1 -> Gpu y -> Gpu y
floatingArr op (Gpu a) = Gpu (arr1 op a)

instance (GoodScalar r, Floating r) => Floating (Gpu (TKR n r)) where
  pi = shapeless "pi"
  exp = floatingArr Exp; log = floatingArr Log; sqrt = floatingArr Sqrt
  sin = floatingArr Sin; cos = floatingArr Cos; tan = floatingArr Tan
  asin = floatingArr Asin; acos = floatingArr Acos; atan = floatingArr Atan
  sinh = floatingArr Sinh; cosh = floatingArr Cosh; tanh = floatingArr Tanh
  asinh = floatingArr Asinh; acosh = floatingArr Acosh; atanh = floatingArr Atanh
  Gpu a ** Gpu b = Gpu (arr2 Pow a b)
  logBase (Gpu a) (Gpu b) = Gpu (arr2 LogBase a b)
instance (GoodScalar r, Floating r) => Floating (Gpu (TKS sh r)) where
  pi = shapeless "pi"
  exp = floatingArr Exp; log = floatingArr Log; sqrt = floatingArr Sqrt
  sin = floatingArr Sin; cos = floatingArr Cos; tan = floatingArr Tan
  asin = floatingArr Asin; acos = floatingArr Acos; atan = floatingArr Atan
  sinh = floatingArr Sinh; cosh = floatingArr Cosh; tanh = floatingArr Tanh
  asinh = floatingArr Asinh; acosh = floatingArr Acosh; atanh = floatingArr Atanh
  Gpu a ** Gpu b = Gpu (arr2 Pow a b)
  logBase (Gpu a) (Gpu b) = Gpu (arr2 LogBase a b)
instance (GoodScalar r, Floating r) => Floating (Gpu (TKX sh r)) where
  pi = shapeless "pi"
  exp = floatingArr Exp; log = floatingArr Log; sqrt = floatingArr Sqrt
  sin = floatingArr Sin; cos = floatingArr Cos; tan = floatingArr Tan
  asin = floatingArr Asin; acos = floatingArr Acos; atan = floatingArr Atan
  sinh = floatingArr Sinh; cosh = floatingArr Cosh; tanh = floatingArr Tanh
  asinh = floatingArr Asinh; acosh = floatingArr Acosh; atanh = floatingArr Atanh
  Gpu a ** Gpu b = Gpu (arr2 Pow a b)
  logBase (Gpu a) (Gpu b) = Gpu (arr2 LogBase a b)

instance (GoodScalar r, Floating r) => RealFloatH (Gpu (TKR n r)) where
  atan2H (Gpu a) (Gpu b) = Gpu (arr2 Atan2 a b)
instance (GoodScalar r, Floating r) => RealFloatH (Gpu (TKS sh r)) where
  atan2H (Gpu a) (Gpu b) = Gpu (arr2 Atan2 a b)
instance (GoodScalar r, Floating r) => RealFloatH (Gpu (TKX sh r)) where
  atan2H (Gpu a) (Gpu b) = Gpu (arr2 Atan2 a b)
