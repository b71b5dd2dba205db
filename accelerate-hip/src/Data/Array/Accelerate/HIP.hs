{-# LANGUAGE BangPatterns        #-}
{-# LANGUAGE GADTs               #-}
{-# LANGUAGE RankNTypes          #-}
{-# LANGUAGE ScopedTypeVariables #-}
{-# LANGUAGE TypeApplications    #-}
-- |
-- Module      : Data.Array.Accelerate.HIP
--
-- A backend for AMD Instinct MI355X (gfx950) GPUs: the same three entry points as the reference
-- interpreter ('Data.Array.Accelerate.Interpreter', Interpreter.hs:31-42), over libacchip.
--
-- 'runN' does everything that can be done without the arguments when it is partially applied:
-- sharing recovery and fusion ('convertAfun'), printing the fused term, code generation and
-- compilation for gfx950 in the library (@acchip_compile@).  Use it as
--
-- > let !go = runN f in ... go xs ys ...
--
-- NOT COMPILED: no GHC was available where this was written; it follows accelerate-1.4.0.0.
--
module Data.Array.Accelerate.HIP (

  Smart.Acc, Sugar.Arrays,
  Afunction, AfunctionR,

  run, run1, runN,

) where

import Data.Array.Accelerate.AST                                    ( PreOpenAfun(..) )
import Data.Array.Accelerate.Array.Data
import Data.Array.Accelerate.Array.Unique
import Data.Array.Accelerate.Representation.Array
import Data.Array.Accelerate.Representation.Shape
import Data.Array.Accelerate.Representation.Type
import Data.Array.Accelerate.Trafo                                  ( convertAcc, convertAfun )
import Data.Array.Accelerate.Trafo.Delayed
import Data.Array.Accelerate.Trafo.Sharing                          ( Afunction(..), AfunctionR, AfunctionRepr(..), ArraysFunctionR, afunctionRepr )
import Data.Array.Accelerate.Type
import qualified Data.Array.Accelerate.Smart                        as Smart
import qualified Data.Array.Accelerate.Sugar.Array                  as Sugar

import Data.Array.Accelerate.HIP.Array.Remote
import Data.Array.Accelerate.HIP.FFI
import Data.Array.Accelerate.HIP.Serialise

import Control.Exception
import Control.Monad
import Foreign.C.String
import Foreign.ForeignPtr
import Foreign.Marshal.Alloc
import Foreign.Marshal.Array
import Foreign.Ptr
import Foreign.Storable
import System.IO.Unsafe


-- | Run a complete embedded array program (Interpreter.hs:93-101).
run :: forall a. Sugar.Arrays a => Smart.Acc a -> a
run a = unsafePerformIO $ do
  let (text, used) = serialiseAcc (convertAcc a)
  prog <- compile text
  Sugar.toArr <$> execute prog used [] (Sugar.arraysR @a)

-- | 'runN' for functions of one argument (Interpreter.hs:105-106).
run1 :: (Sugar.Arrays a, Sugar.Arrays b) => (Smart.Acc a -> Smart.Acc b) -> a -> b
run1 = runN

-- | Prepare an array function; the result is applied to arrays (Interpreter.hs:110-126).
runN :: forall f. Afunction f => f -> AfunctionR f
runN f = go
  where
    !afun         = convertAfun f
    (text, !used) = serialiseAfun afun
    !prog         = unsafePerformIO (compile text)       -- once, at partial application
    !go           = eval (afunctionRepr @f) afun []
    --
    -- peel the arguments off as the interpreter does, collecting them as (representation, arrays)
    eval :: AfunctionRepr g (AfunctionR g) (ArraysFunctionR g)
         -> DelayedOpenAfun aenv (ArraysFunctionR g)
         -> [Argument]
         -> AfunctionR g
    eval (AfunctionReprLam reprF) (Alam lhs g) args = \a -> eval reprF g (Argument (lhsToTupR lhs) (Sugar.fromArr a) : args)
    eval AfunctionReprBody        (Abody b)    args = unsafePerformIO $
      Sugar.toArr <$> execute prog used (reverse args) (arraysR b)
    eval _                        _            _    = error "runN: function and its representation disagree"


-- Compilation
-- -----------

-- | A prepared program; released when the garbage collector finds it dead.
type Program = ForeignPtr Prog

compile :: String -> IO Program
compile text = withContext $ \ctx -> withCStringLen text $ \(p, n) -> alloca $ \out -> do
  check "acchip_compile" =<< c_compile ctx p (fromIntegral n) out
  newForeignPtr p_program_release =<< peek out


-- Execution
-- ---------

data Argument where
  Argument :: ArraysR a -> a -> Argument

-- | Apply a prepared program: arguments and 'Use'd arrays are brought to the device through the
-- array table (uploaded on first use only), results are copied back and their device buffers kept
-- in the table under the new host arrays, so that a result fed to the next call is not uploaded.
execute :: Program -> [UsedArray] -> [Argument] -> ArraysR r -> IO r
execute prog used args reprR = withContext $ \ctx -> withForeignPtr prog $ \p ->
  withArguments args $ \argHandles ->
  withUsed used $ \useHandles ->
  withArray argHandles $ \pargs ->
  withArray useHandles $ \puses ->
  alloca $ \out -> do
    check "acchip_execute" =<< c_execute ctx p pargs (fromIntegral (length argHandles)) puses (fromIntegral (length useHandles)) out
    res <- peek out
    r   <- download reprR res            -- waits for the stream; errors only a kernel can see surface here
    c_array_release res
    return r

withArguments :: [Argument] -> ([Ptr Arr] -> IO b) -> IO b
withArguments []                  k = k []
withArguments (Argument r a : as) k = withArrays r a $ \h -> withArguments as (k . (h :))

withUsed :: [UsedArray] -> ([Ptr Arr] -> IO b) -> IO b
withUsed []                     k = k []
withUsed (UsedArray r a : rest) k = withArrayHandle r a $ \h -> withUsed rest (k . (h :))

-- a tuple of arrays as one handle (acchip_array_pair / acchip_array_unit)
withArrays :: ArraysR a -> a -> (Ptr Arr -> IO b) -> IO b
withArrays TupRunit         ()       k = alloca $ \out -> do
  check "acchip_array_unit" =<< c_array_unit out
  h <- peek out
  k h `finally` c_array_release h
withArrays (TupRsingle r)   a        k = withArrayHandle r a k
withArrays (TupRpair ra rb) (a, b)   k =
  withArrays ra a $ \ha ->
  withArrays rb b $ \hb -> alloca $ \out -> do
    check "acchip_array_pair" =<< c_array_pair ha hb out
    h <- peek out
    k h `finally` c_array_release h

-- one array: its buffers through the table, described to the library without giving them away
withArrayHandle :: ArrayR (Array sh e) -> Array sh e -> (Ptr Arr -> IO b) -> IO b
withArrayHandle (ArrayR shr tp) (Array sh adata) k =
  withArrayData tp adata (size shr sh) $ \bufs ->
  withArray (map fromIntegral (reverse (shapeToList shr sh))) $ \pshape ->   -- outermost extent first
  withArray bufs $ \pbufs ->
  withCString (typeText tp) $ \ptype ->
  alloca $ \out -> do
    withContext $ \ctx ->
      check "acchip_array_wrap" =<< c_array_wrap ctx (fromIntegral (rank shr)) pshape ptype pbufs (fromIntegral (length bufs)) out
    h <- peek out
    k h `finally` c_array_release h

-- results: allocate the host arrays, copy back, keep the device buffers in the table
download :: ArraysR r -> Ptr Arr -> IO r
download TupRunit         _ = return ()
download (TupRpair ra rb) h = do
  ha <- alloca $ \o -> check "acchip_array_fst" =<< c_array_fst h o >> peek o
  hb <- alloca $ \o -> check "acchip_array_snd" =<< c_array_snd h o >> peek o
  a  <- download ra ha `finally` c_array_release ha
  b  <- download rb hb `finally` c_array_release hb
  return (a, b)
download (TupRsingle repr@(ArrayR shr tp)) h = do
  dims <- allocaArray (rank shr) $ \p -> do
    check "acchip_array_shape" =<< c_array_shape h p
    peekArray (rank shr) p
  let sh = listToShape shr (reverse (map fromIntegral dims))   -- shapeToList / listToShape go innermost first
  arr@(Array _ adata) <- allocateArray repr sh
  _ <- leaves tp adata (size shr sh) 0
  return arr
  where
    leaves :: TypeR e -> ArrayData e -> Int -> Int -> IO Int
    leaves TupRunit         ()     _ i = return i
    leaves (TupRpair ta tb) (a, b) n i = leaves ta a n i >>= leaves tb b n
    leaves (TupRsingle t)   ad     n i
      | ScalarArrayDict w s <- scalarArrayDict t
      , SingleArrayDict     <- singleArrayDict s
      , SingleDict          <- singleDict s
      = do dev   <- c_array_buffer h (fromIntegral i)
           bytes <- c_array_buffer_bytes h (fromIntegral i)
           withContext $ \ctx -> withUniqueArrayPtr ad $ \host ->
             check "acchip_peek" =<< c_peek ctx (castPtr host) dev bytes
           adoptLeaf ad (n * w) h i
           return (i + 1)
