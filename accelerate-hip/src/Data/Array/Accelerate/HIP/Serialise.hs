{-# LANGUAGE GADTs               #-}
{-# LANGUAGE LambdaCase          #-}
{-# LANGUAGE RankNTypes          #-}
{-# LANGUAGE ScopedTypeVariables #-}
{-# LANGUAGE TypeApplications    #-}
{-# LANGUAGE TypeOperators       #-}
-- |
-- Module      : Data.Array.Accelerate.HIP.Serialise
--
-- The fused, delayed array program as the text libacchip reads (docs/WIRE.md, version 1): one
-- S-expression per constructor of 'PreOpenAcc', 'OpenExp' and 'PrimFun', de Bruijn indices
-- kept as they are.  Host arrays embedded by 'Use' do not travel in the text: they are
-- numbered in order of appearance and handed to @acchip_execute@ beside the arguments.
--
-- NOT COMPILED: no GHC was available where this was written.  It follows accelerate-1.4.0.0
-- (src/Data/Array/Accelerate/AST.hs:230-753); the texts under tests/golden/terms/ are what
-- 'serialiseAfun' must produce for the five benchmark programs.
--
module Data.Array.Accelerate.HIP.Serialise (

  UsedArray(..), serialiseAfun, serialiseAcc, typeText, wireVersion,

) where

import Data.Array.Accelerate.AST
import Data.Array.Accelerate.AST.Idx
import Data.Array.Accelerate.AST.LeftHandSide
import Data.Array.Accelerate.AST.Var
import Data.Array.Accelerate.Representation.Array
import Data.Array.Accelerate.Representation.Shape
import Data.Array.Accelerate.Representation.Slice
import Data.Array.Accelerate.Representation.Stencil
import Data.Array.Accelerate.Representation.Type
import Data.Array.Accelerate.Representation.Vec
import Data.Array.Accelerate.Sugar.Foreign                ( strForeign )
import Data.Array.Accelerate.Trafo.Delayed
import Data.Array.Accelerate.Type
import Data.Primitive.Vec                                 ( listOfVec )

import Control.Monad.State.Strict
import Data.Bits
import Data.Char                                          ( intToDigit, ord )
import Data.List                                          ( intersperse )
import qualified Data.ByteString                          as B
import qualified Data.Text                                as T
import qualified Data.Text.Encoding                       as T


-- | A host array a 'Use' node embeds; its position in the list is its slot number.
data UsedArray where
  UsedArray :: ArrayR (Array sh e) -> Array sh e -> UsedArray

wireVersion :: Int
wireVersion = 1

type S = State [UsedArray]          -- used arrays, latest first

-- | @(acchip-ir 1 AFUN)@ and the arrays of its 'Use' nodes, slot 0 first.
serialiseAfun :: DelayedOpenAfun aenv f -> (String, [UsedArray])
serialiseAfun f =
  let (body, used) = runState (openAfun f) []
  in  (header body "", reverse used)

serialiseAcc :: DelayedOpenAcc aenv a -> (String, [UsedArray])
serialiseAcc a =
  let (body, used) = runState (openAcc a) []
  in  (header body "", reverse used)

header :: ShowS -> ShowS
header body = list [ atom "acchip-ir", shows wireVersion, body ]


-- Building blocks
-- ---------------

atom :: String -> ShowS
atom = showString

list :: [ShowS] -> ShowS
list xs = showChar '(' . foldr (.) id (intersperse (showChar ' ') xs) . showChar ')'

node :: String -> [S ShowS] -> S ShowS
node h xs = (\ys -> list (atom h : ys)) <$> sequence xs

-- the UTF-8 bytes of a text as hexadecimal digits, "-" for the empty text
hex :: T.Text -> ShowS
hex t
  | T.null t  = atom "-"
  | otherwise = atom (concatMap byte (B.unpack (T.encodeUtf8 t)))
  where byte w = [ intToDigit (fromIntegral (w `shiftR` 4)), intToDigit (fromIntegral (w .&. 15)) ]


-- Types
-- -----

integralType :: IntegralType t -> ShowS
integralType = atom . \case
  TypeInt    -> "i64"     -- Int and Word are 64 bits wide on every platform this backend runs on
  TypeInt8   -> "i8"
  TypeInt16  -> "i16"
  TypeInt32  -> "i32"
  TypeInt64  -> "i64"
  TypeWord   -> "u64"
  TypeWord8  -> "u8"
  TypeWord16 -> "u16"
  TypeWord32 -> "u32"
  TypeWord64 -> "u64"

floatingType :: FloatingType t -> ShowS
floatingType = atom . \case
  TypeHalf   -> "f16"
  TypeFloat  -> "f32"
  TypeDouble -> "f64"

numType :: NumType t -> ShowS
numType (IntegralNumType t) = integralType t
numType (FloatingNumType t) = floatingType t

singleType :: SingleType t -> ShowS
singleType (NumSingleType t) = numType t

scalarType :: ScalarType t -> ShowS
scalarType (SingleScalarType t)                = singleType t
scalarType (VectorScalarType (VectorType n t)) = showChar 'v' . shows n . singleType t

typeR :: TypeR t -> ShowS
typeR TupRunit       = atom "unit"
typeR (TupRsingle t) = scalarType t
typeR (TupRpair a b) = list [ atom "pair", typeR a, typeR b ]

-- | An element type as the library spells it (the @elt_type@ argument of @acchip_array_wrap@).
typeText :: TypeR t -> String
typeText t = typeR t ""

arrayR :: ArrayR a -> ShowS
arrayR (ArrayR shr tr) = list [ atom "array", shows (rank shr), typeR tr ]

arraysR :: ArraysR a -> ShowS
arraysR TupRunit       = atom "unit"
arraysR (TupRsingle a) = arrayR a
arraysR (TupRpair a b) = list [ atom "pair", arraysR a, arraysR b ]

elhs :: ELeftHandSide t env env' -> ShowS
elhs (LeftHandSideSingle t)   = list [ atom "single", scalarType t ]
elhs (LeftHandSideWildcard t) = list [ atom "wild", typeR t ]
elhs (LeftHandSidePair a b)   = list [ atom "pair", elhs a, elhs b ]

alhs :: ALeftHandSide t aenv aenv' -> ShowS
alhs (LeftHandSideSingle a)   = list [ atom "single", arrayR a ]
alhs (LeftHandSideWildcard a) = list [ atom "wild", arraysR a ]
alhs (LeftHandSidePair a b)   = list [ atom "pair", alhs a, alhs b ]

sliceIndex :: SliceIndex slix sl co sh -> ShowS
sliceIndex = list . go
  where
    go :: SliceIndex slix sl co sh -> [ShowS]
    go SliceNil       = []
    go (SliceAll r)   = atom "all"   : go r       -- innermost dimension first
    go (SliceFixed r) = atom "fixed" : go r

stencilR :: StencilR sh e pat -> ShowS
stencilR = \case
  StencilRunit3 t -> list [ atom "unit3", typeR t ]
  StencilRunit5 t -> list [ atom "unit5", typeR t ]
  StencilRunit7 t -> list [ atom "unit7", typeR t ]
  StencilRunit9 t -> list [ atom "unit9", typeR t ]
  StencilRtup3 a b c             -> list [ atom "tup3", stencilR a, stencilR b, stencilR c ]
  StencilRtup5 a b c d e         -> list [ atom "tup5", stencilR a, stencilR b, stencilR c, stencilR d, stencilR e ]
  StencilRtup7 a b c d e f g     -> list [ atom "tup7", stencilR a, stencilR b, stencilR c, stencilR d, stencilR e, stencilR f, stencilR g ]
  StencilRtup9 a b c d e f g h i -> list [ atom "tup9", stencilR a, stencilR b, stencilR c, stencilR d, stencilR e, stencilR f, stencilR g, stencilR h, stencilR i ]


-- Literals
-- --------

-- integers in decimal; floating point in C99 hexadecimal notation with 13 hexadecimal digits,
-- the spelling of Python's float.hex: 0x1.8000000000000p+1, 0x0.0p+0, -0x0.0p+0, inf, -inf, nan
hexFloat :: Double -> String
hexFloat x
  | isNaN x          = "nan"
  | isInfinite x     = if x > 0 then "inf" else "-inf"
  | isNegativeZero x = "-0x0.0p+0"
  | x == 0           = "0x0.0p+0"
  | x < 0            = '-' : hexFloat (negate x)
  | otherwise        =
      let (m, e)       = decodeFloat x                    -- x = m * 2^e with 2^52 <= m < 2^53, also for subnormals
          subnormal    = e < -1074
          (lead, frac, ex)
            | subnormal = (0 :: Integer, m `shiftR` negate (e + 1074), -1022 :: Int)
            | otherwise = (1, m - bit 52, e + 52)
          digits       = [ intToDigit (fromIntegral ((frac `shiftR` (4 * k)) .&. 15)) | k <- [12, 11 .. 0] ]
      in  "0x" ++ show lead ++ "." ++ digits ++ "p" ++ (if ex >= 0 then "+" else "-") ++ show (abs ex)

literal :: ScalarType t -> t -> ShowS
literal (SingleScalarType t) x = single t x
literal (VectorScalarType (VectorType _ t)) v
  | SingleDict <- singleDict t  -- (brings Prim into scope through its superclasses in Type.hs)
  = list (map (single t) (listOfVec v))

single :: SingleType t -> t -> ShowS
single (NumSingleType (IntegralNumType t)) x | IntegralDict <- integralDict t = shows (toInteger x)
single (NumSingleType (FloatingNumType t)) x | FloatingDict <- floatingDict t = atom (hexFloat (realToFrac x))

-- a constant of a tuple type, as nested pairs of constants
constant :: TypeR t -> t -> ShowS
constant TupRunit         ()     = atom "nil"
constant (TupRsingle t)   x      = list [ atom "const", scalarType t, literal t x ]
constant (TupRpair ta tb) (a, b) = list [ atom "pair", constant ta a, constant tb b ]


-- Scalar expressions
-- ------------------

openFun :: OpenFun env aenv t -> S ShowS
openFun (Body e)    = openExp e
openFun (Lam lhs f) = node "lam" [ pure (elhs lhs), openFun f ]

avarIx :: ArrayVar aenv a -> S ShowS
avarIx (Var _ ix) = pure (shows (idxToInt ix))

openExp :: forall env aenv t. OpenExp env aenv t -> S ShowS
openExp = \case
  Let lhs bnd body      -> node "let" [ pure (elhs lhs), openExp bnd, openExp body ]
  Evar (Var _ ix)       -> node "var" [ pure (shows (idxToInt ix)) ]
  Foreign _ _ f x       -> node "foreign" [ openFun f, openExp x ]
  Pair a b              -> node "pair" [ openExp a, openExp b ]
  Nil                   -> pure (atom "nil")
  VecPack vecr e
    | VectorType n s <- vecRvector vecr
                        -> node "vecpack"   [ pure (shows n), pure (singleType s), openExp e ]
  VecUnpack vecr e
    | VectorType n s <- vecRvector vecr
                        -> node "vecunpack" [ pure (shows n), pure (singleType s), openExp e ]
  IndexSlice slice slix sh
                        -> node "indexslice" [ pure (sliceIndex slice), openExp slix, openExp sh ]
  IndexFull slice slix sl
                        -> node "indexfull"  [ pure (sliceIndex slice), openExp slix, openExp sl ]
  ToIndex shr sh ix     -> node "toindex"   [ pure (shows (rank shr)), openExp sh, openExp ix ]
  FromIndex shr sh i    -> node "fromindex" [ pure (shows (rank shr)), openExp sh, openExp i ]
  Case e rhs def        -> node "case" [ openExp e
                                       , list <$> mapM (\(tag, r) -> (\r' -> list [ shows tag, r' ]) <$> openExp r) rhs
                                       , maybe (pure (atom "none")) openExp def ]
  Cond p t e            -> node "cond" [ openExp p, openExp t, openExp e ]
  While p f x           -> node "while" [ openFun p, openFun f, openExp x ]
  Const t c             -> pure (list [ atom "const", scalarType t, literal t c ])
  PrimConst c           -> pure (primConst c)
  PrimApp f x           -> let (name, tys) = primFun f
                           in  node "prim" (pure (atom name) : map pure tys ++ [ openExp x ])
  Index v ix            -> node "index"       [ avarIx v, openExp ix ]
  LinearIndex v i       -> node "linearindex" [ avarIx v, openExp i ]
  Shape v               -> node "shape"       [ avarIx v ]
  ShapeSize shr sh      -> node "shapesize"   [ pure (shows (rank shr)), openExp sh ]
  Undef t               -> pure (list [ atom "undef", scalarType t ])
  Coerce t1 t2 e        -> node "coerce" [ pure (scalarType t1), pure (scalarType t2), openExp e ]

primConst :: PrimConst t -> ShowS
primConst (PrimMinBound (IntegralBoundedType t)) = list [ atom "minbound", integralType t ]
primConst (PrimMaxBound (IntegralBoundedType t)) = list [ atom "maxbound", integralType t ]
primConst (PrimPi t)                             = list [ atom "pi", floatingType t ]

-- name and type arguments of a primitive, in the order of the constructor's fields
primFun :: PrimFun f -> (String, [ShowS])
primFun = \case
  PrimAdd t                -> ("add",      [numType t])
  PrimSub t                -> ("sub",      [numType t])
  PrimMul t                -> ("mul",      [numType t])
  PrimNeg t                -> ("neg",      [numType t])
  PrimAbs t                -> ("abs",      [numType t])
  PrimSig t                -> ("sig",      [numType t])
  PrimQuot t               -> ("quot",     [integralType t])
  PrimRem t                -> ("rem",      [integralType t])
  PrimQuotRem t            -> ("quotrem",  [integralType t])
  PrimIDiv t               -> ("idiv",     [integralType t])
  PrimMod t                -> ("mod",      [integralType t])
  PrimDivMod t             -> ("divmod",   [integralType t])
  PrimBAnd t               -> ("band",     [integralType t])
  PrimBOr t                -> ("bor",      [integralType t])
  PrimBXor t               -> ("bxor",     [integralType t])
  PrimBNot t               -> ("bnot",     [integralType t])
  PrimBShiftL t            -> ("shl",      [integralType t])
  PrimBShiftR t            -> ("shr",      [integralType t])
  PrimBRotateL t           -> ("rotl",     [integralType t])
  PrimBRotateR t           -> ("rotr",     [integralType t])
  PrimPopCount t           -> ("popcount", [integralType t])
  PrimCountLeadingZeros t  -> ("clz",      [integralType t])
  PrimCountTrailingZeros t -> ("ctz",      [integralType t])
  PrimFDiv t               -> ("fdiv",     [floatingType t])
  PrimRecip t              -> ("recip",    [floatingType t])
  PrimSin t                -> ("sin",      [floatingType t])
  PrimCos t                -> ("cos",      [floatingType t])
  PrimTan t                -> ("tan",      [floatingType t])
  PrimAsin t               -> ("asin",     [floatingType t])
  PrimAcos t               -> ("acos",     [floatingType t])
  PrimAtan t               -> ("atan",     [floatingType t])
  PrimSinh t               -> ("sinh",     [floatingType t])
  PrimCosh t               -> ("cosh",     [floatingType t])
  PrimTanh t               -> ("tanh",     [floatingType t])
  PrimAsinh t              -> ("asinh",    [floatingType t])
  PrimAcosh t              -> ("acosh",    [floatingType t])
  PrimAtanh t              -> ("atanh",    [floatingType t])
  PrimExpFloating t        -> ("exp",      [floatingType t])
  PrimSqrt t               -> ("sqrt",     [floatingType t])
  PrimLog t                -> ("log",      [floatingType t])
  PrimFPow t               -> ("fpow",     [floatingType t])
  PrimLogBase t            -> ("logbase",  [floatingType t])
  PrimAtan2 t              -> ("atan2",    [floatingType t])
  PrimTruncate a b         -> ("truncate", [floatingType a, integralType b])
  PrimRound a b            -> ("round",    [floatingType a, integralType b])
  PrimFloor a b            -> ("floor",    [floatingType a, integralType b])
  PrimCeiling a b          -> ("ceiling",  [floatingType a, integralType b])
  PrimIsNaN t              -> ("isnan",    [floatingType t])
  PrimIsInfinite t         -> ("isinf",    [floatingType t])
  PrimLt t                 -> ("lt",       [singleType t])
  PrimGt t                 -> ("gt",       [singleType t])
  PrimLtEq t               -> ("lte",      [singleType t])
  PrimGtEq t               -> ("gte",      [singleType t])
  PrimEq t                 -> ("eq",       [singleType t])
  PrimNEq t                -> ("neq",      [singleType t])
  PrimMax t                -> ("max",      [singleType t])
  PrimMin t                -> ("min",      [singleType t])
  PrimLAnd                 -> ("land",     [])
  PrimLOr                  -> ("lor",      [])
  PrimLNot                 -> ("lnot",     [])
  PrimFromIntegral a b     -> ("fromintegral", [integralType a, numType b])
  PrimToFloating a b       -> ("tofloating",   [numType a, floatingType b])


-- Array computations
-- ------------------

openAfun :: PreOpenAfun DelayedOpenAcc aenv f -> S ShowS
openAfun (Abody b)    = openAcc b
openAfun (Alam lhs f) = node "alam" [ pure (alhs lhs), openAfun f ]

openAcc :: DelayedOpenAcc aenv a -> S ShowS
openAcc (Manifest pacc)        = preOpenAcc pacc
openAcc (Delayed repr sh f lf) = node "delayed" [ pure (arrayR repr), openExp sh, openFun f, openFun lf ]

seed :: Maybe (OpenExp env aenv e) -> S ShowS
seed Nothing  = pure (atom "nothing")
seed (Just z) = node "just" [ openExp z ]

direction :: Direction -> ShowS
direction LeftToRight = atom "l"
direction RightToLeft = atom "r"

boundary :: TypeR e -> Boundary aenv (Array sh e) -> S ShowS
boundary _  Clamp        = pure (atom "clamp")
boundary _  Mirror       = pure (atom "mirror")
boundary _  Wrap         = pure (atom "wrap")
boundary tp (Constant v) = pure (list [ atom "constant", constant tp v ])
boundary _  (Function f) = node "function" [ openFun f ]

preOpenAcc :: forall aenv a. PreOpenAcc DelayedOpenAcc aenv a -> S ShowS
preOpenAcc = \case
  Alet lhs bnd body         -> node "alet" [ pure (alhs lhs), openAcc bnd, openAcc body ]
  Avar (Var _ ix)           -> node "avar" [ pure (shows (idxToInt ix)) ]
  Apair a b                 -> node "apair" [ openAcc a, openAcc b ]
  Anil                      -> pure (atom "anil")
  Apply _ f a               -> node "apply" [ openAfun f, openAcc a ]
  -- the foreign function is named, its pure fallback (a closed function) travels
  Aforeign _ asm f a        -> node "aforeign" [ pure (hex (T.pack (strForeign asm))), openAfun f, openAcc a ]
  Acond p t e               -> node "acond" [ openExp p, openAcc t, openAcc e ]
  Awhile p f a              -> node "awhile" [ openAfun p, openAfun f, openAcc a ]
  Atrace (Message _ _ msg) a b
                            -> node "atrace" [ pure (hex msg), openAcc a, openAcc b ]
  Use repr arr              -> do
    slot <- gets length
    modify (UsedArray repr arr :)
    return (list [ atom "use", arrayR repr, shows slot ])
  Unit tp e                 -> node "unit" [ pure (typeR tp), openExp e ]
  Reshape shr sh a          -> node "reshape" [ pure (shows (rank shr)), openExp sh, openAcc a ]
  Generate repr sh f        -> node "generate" [ pure (arrayR repr), openExp sh, openFun f ]
  Transform repr sh p f a   -> node "transform" [ pure (arrayR repr), openExp sh, openFun p, openFun f, openAcc a ]
  Replicate slice slix a    -> node "replicate" [ pure (sliceIndex slice), openExp slix, openAcc a ]
  Slice slice a slix        -> node "slice" [ pure (sliceIndex slice), openAcc a, openExp slix ]
  Map tp f a                -> node "map" [ pure (typeR tp), openFun f, openAcc a ]
  ZipWith tp f a b          -> node "zipwith" [ pure (typeR tp), openFun f, openAcc a, openAcc b ]
  Fold f z a                -> node "fold" [ openFun f, seed z, openAcc a ]
  FoldSeg it f z a s        -> node "foldseg" [ pure (integralType it), openFun f, seed z, openAcc a, openAcc s ]
  Scan d f z a              -> node "scan" [ pure (direction d), openFun f, seed z, openAcc a ]
  Scan' d f z a             -> node "scan'" [ pure (direction d), openFun f, openExp z, openAcc a ]
  Permute f d p a           -> node "permute" [ openFun f, openAcc d, openFun p, openAcc a ]
  Backpermute shr sh p a    -> node "backpermute" [ pure (shows (rank shr)), openExp sh, openFun p, openAcc a ]
  Stencil sr tp f b a       -> node "stencil" [ pure (stencilR sr), pure (typeR tp), openFun f
                                              , boundary (stencilEltR sr) b, openAcc a ]
  Stencil2 sr1 sr2 tp f b1 a1 b2 a2
                            -> node "stencil2" [ pure (stencilR sr1), pure (stencilR sr2), pure (typeR tp), openFun f
                                               , boundary (stencilEltR sr1) b1, openAcc a1
                                               , boundary (stencilEltR sr2) b2, openAcc a2 ]
