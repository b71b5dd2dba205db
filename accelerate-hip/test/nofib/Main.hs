-- |
-- The reference's backend-parametric test-suite (Data.Array.Accelerate.Test.NoFib, built with
-- cabal flag `nofib` of the accelerate package) instantiated with this backend's runN, exactly as
-- test/nofib/Main.hs:19-24 instantiates it with the interpreter's.
--
-- NOT COMPILED: no GHC was available where this was written.
--
module Main where

import Data.Array.Accelerate.Test.NoFib
import Data.Array.Accelerate.HIP

import System.Environment
import Test.Tasty

main :: IO ()
main = do
  setEnv "TASTY_HEDGEHOG_TESTS" "50"
  nofib runN (testGroup "runQ" [])
