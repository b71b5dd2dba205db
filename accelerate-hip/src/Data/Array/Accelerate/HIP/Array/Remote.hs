{-# LANGUAGE GADTs                      #-}
{-# LANGUAGE GeneralizedNewtypeDeriving #-}
{-# LANGUAGE RankNTypes                 #-}
{-# LANGUAGE ScopedTypeVariables #-}
{-# LANGUAGE TypeFamilies        #-}
-- |
-- Module      : Data.Array.Accelerate.HIP.Array.Remote
--
-- Device memory for host arrays.  The reference's 'Data.Array.Accelerate.Array.Remote.LRU' keeps
-- its table in Haskell; here the table is the native one of libacchip (@acchip_table_*@), keyed
-- by the 'Unique' of each 'UniqueArray', so that eviction, copy-back and the allocation ladder
-- run below the C boundary.  What stays in Haskell: taking the pinned host pointer, attaching
-- the finaliser that tells the table an array has died, and 'performGC' as the table's clean
-- hook (Table.clean, Array/Remote/Table.hs:313-339).
--
-- For code written against 'RemoteMemory' (Array/Remote/Class.hs:47-73) the instance is given
-- as well, over a reader of the context.
--
-- NOT COMPILED: no GHC was available where this was written.
--
module Data.Array.Accelerate.HIP.Array.Remote (

  Context(..), theContext, withContext, check,
  withLeaf, withArrayData, adoptLeaf, HIP(..), StreamEvent(..), mirrorCounters,

) where

import Data.Array.Accelerate.Array.Data
import Data.Array.Accelerate.Array.Remote.Class
import Data.Array.Accelerate.Array.Remote.LRU                      ( Task(..) )
import Data.Array.Accelerate.Array.Unique
import Data.Array.Accelerate.Error
import Data.Array.Accelerate.Lifetime
import Data.Array.Accelerate.Representation.Type
import Data.Array.Accelerate.Type

import Data.Array.Accelerate.HIP.FFI

import Control.Monad
import Control.Monad.Reader
import Data.Hashable                                               ( hash )
import Data.Int                                                    ( Int64 )
import Data.Word
import Foreign.C.String
import Foreign.C.Types
import Foreign.Marshal.Alloc
import Foreign.Ptr
import Foreign.Storable
import System.IO.Unsafe
import System.Mem                                                  ( performGC )


-- | One device, one stream, one memory pool, one kernel cache.
newtype Context = Context { ctxPtr :: Ptr Ctx }

-- | The process-wide context on device 0 (or $ACCELERATE_HIP_DEVICE), created on first use.  The clean
-- hook is the garbage collector: dead host arrays give their blocks back before anything is evicted.
{-# NOINLINE theContext #-}
theContext :: Context
theContext = unsafePerformIO $ alloca $ \out -> do
  check "acchip_init" =<< c_init 0 out
  ctx  <- peek out
  hook <- mkCleanHook (\_ -> performGC)
  check "acchip_set_clean_hook" =<< c_set_clean_hook ctx hook nullPtr
  -- -fno-inplace, -ffast-math, -fno-fast-permute-const, -fforce-recomp, -ddump-cc / -exec / -gc reach
  -- the library as the reference's own bit layout (cbits/flags.h:19-49)
  check "acchip_set_flags" =<< c_set_flags ctx =<< peek cmdLineFlags
  return (Context ctx)

withContext :: (Ptr Ctx -> IO a) -> IO a
withContext k = k (ctxPtr theContext)

-- | A non-zero status becomes 'internalError' with the library's message (Error.hs:33-62).
check :: HasCallStack => String -> CInt -> IO ()
check _    0 = return ()
check what _ = do
  msg <- peekCString =<< c_last_error
  internalError (what ++ ": " ++ msg)

-- | The reference's monitoring counters (cbits/monitoring.c:26-32, read by its @-ddump-gc@ report and
-- by the Tracy plots): the library keeps the same quantities per context, and they are copied
-- over after every program and collection, so that tools written against the reference's
-- counters see this backend's remote memory.  This backend is the only user of the remote
-- counters in a process, hence totals are stored, not added.
foreign import ccall "&__total_bytes_allocated_remote"    total_bytes_allocated_remote    :: Ptr Int64
foreign import ccall "&__total_bytes_copied_to_remote"    total_bytes_copied_to_remote    :: Ptr Int64
foreign import ccall "&__total_bytes_copied_from_remote"  total_bytes_copied_from_remote  :: Ptr Int64
foreign import ccall "&__total_bytes_evicted_from_remote" total_bytes_evicted_from_remote :: Ptr Int64
foreign import ccall "&__num_evictions"                   num_evictions                   :: Ptr Int64

mirrorCounters :: IO ()
mirrorCounters = withContext $ \ctx -> do
  let copy name dst = withCString name $ \n -> poke dst . fromIntegral =<< c_stat ctx n
  copy "bytes_allocated_remote"    total_bytes_allocated_remote
  copy "bytes_copied_to_remote"    total_bytes_copied_to_remote
  copy "bytes_copied_from_remote"  total_bytes_copied_from_remote
  copy "bytes_evicted_from_remote" total_bytes_evicted_from_remote
  copy "arrays_evicted"            num_evictions

-- the table's name for a host buffer
ident :: UniqueArray e -> Word64
ident = fromIntegral . hash . uniqueArrayId

-- | Run an action with the device copy of one host buffer (LRU.withRemote, LRU.hs:140-207).  The
-- first use allocates the block, uploads the host data and attaches the finaliser; a buffer that
-- was evicted since is uploaded again by the table.  The block stays pinned for the duration of
-- the action and, through the table's task, until the work queued in it has finished.
withLeaf :: forall e b. Storable e => UniqueArray e -> Int -> (Ptr e -> IO b) -> IO b
withLeaf ua n k = withContext $ \ctx -> withUniqueArrayPtr ua $ \host -> do
  let bytes = fromIntegral (n * sizeOf (undefined :: e))
      key   = ident ua
  fresh <- alloca $ \p -> do
    check "acchip_table_malloc" =<< c_table_malloc ctx key host bytes 1 p
    peek p
  when (fresh /= 0) $
    addFinalizer (uniqueArrayData ua) (c_table_free ctx key)
  dev <- alloca $ \p -> do
    check "acchip_table_use" =<< c_table_use ctx key p
    peek p
  when (fresh /= 0) $
    check "acchip_poke" =<< c_poke ctx dev host bytes
  r <- k dev
  check "acchip_table_release" =<< c_table_release ctx key
  mirrorCounters
  return r

-- | The same for all buffers of an array's payload, left to right (the struct-of-arrays order of
-- Array/Data.hs:95-119, which is also the order @acchip_array_wrap@ expects).
withArrayData :: TypeR e -> ArrayData e -> Int -> ([Ptr ()] -> IO b) -> IO b
withArrayData TupRunit         ()       _ k = k []
withArrayData (TupRpair ta tb) (a, b)   n k =
  withArrayData ta a n $ \pa ->
  withArrayData tb b n $ \pb -> k (pa ++ pb)
withArrayData (TupRsingle t)   ad       n k
  | ScalarArrayDict w s <- scalarArrayDict t
  , SingleArrayDict     <- singleArrayDict s
  , SingleDict          <- singleDict s
  = withLeaf ad (n * w) (k . (: []) . castPtr)

-- | A buffer of a program's result becomes the device copy of the host buffer it was just copied
-- to (Clean): feeding the result to the next program then needs no upload.
adoptLeaf :: forall e. Storable e => UniqueArray e -> Int -> Ptr Arr -> Int -> IO ()
adoptLeaf ua n arr leaf = withContext $ \ctx -> withUniqueArrayPtr ua $ \host -> do
  let bytes = fromIntegral (n * sizeOf (undefined :: e))
      key   = ident ua
  rc <- c_table_adopt ctx key host bytes arr (fromIntegral leaf) 1
  when (rc == 0) $ addFinalizer (uniqueArrayData ua) (c_table_free ctx key)
  -- (a buffer the handle does not own cannot be adopted: the copy on the host is all there is)


-- The classes of the reference's remote-memory layer
-- --------------------------------------------------

-- | Computations that talk to the device of a context.
newtype HIP a = HIP { runHIP :: ReaderT Context IO a }
  deriving (Functor, Applicative, Monad, MonadIO, MonadReader Context)

instance RemoteMemory HIP where
  type RemotePtr HIP = Ptr
  mallocRemote n
    | n <= 0    = return (Just nullPtr)
    | otherwise = do
        Context ctx <- ask
        p <- liftIO $ c_malloc ctx (fromIntegral n)
        return $ if p == nullPtr then Nothing else Just p        -- never throws (Class.hs:52-54)
  pokeRemote t n dst ad
    | SingleArrayDict <- singleArrayDict t
    , SingleDict      <- singleDict t
    = do Context ctx <- ask
         liftIO $ withUniqueArrayPtr ad $ \src ->
           check "acchip_poke" =<< c_poke ctx dst src (fromIntegral (n * sizeOf (undefined `asPtrOf` src)))
  peekRemote t n src ad
    | SingleArrayDict <- singleArrayDict t
    , SingleDict      <- singleDict t
    = do Context ctx <- ask
         liftIO $ withUniqueArrayPtr ad $ \dst ->
           check "acchip_peek" =<< c_peek ctx dst src (fromIntegral (n * sizeOf (undefined `asPtrOf` dst)))
  castRemotePtr        = castPtr
  totalRemoteMem       = memInfo fst
  availableRemoteMem   = memInfo snd
  remoteAllocationSize = return 1024                              -- the pool's size classes

asPtrOf :: a -> Ptr a -> a
asPtrOf x _ = x

memInfo :: ((Int64, Int64) -> Int64) -> HIP Int64
memInfo sel = do
  Context ctx <- ask
  liftIO $ alloca $ \pt -> alloca $ \pa -> do
    check "acchip_mem_info" =<< c_mem_info ctx pt pa
    t <- peek pt
    a <- peek pa
    return (sel (fromIntegral t, fromIntegral a))

-- | A point in the context's stream: 'completed' when everything queued before it has run.
newtype StreamEvent = StreamEvent (Ptr Event)

instance Task StreamEvent where
  completed (StreamEvent ev) = alloca $ \p -> do
    check "acchip_event_query" =<< c_event_query ev p
    (/= 0) <$> peek p
