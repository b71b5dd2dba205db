{-# LANGUAGE ForeignFunctionInterface #-}
-- |
-- Module      : Data.Array.Accelerate.HIP.FFI
--
-- Imports of libacchip (include/acchip.h).  Calls that may block (compilation, synchronisation,
-- transfers, anything that may run the allocation ladder) are @safe@; the rest are @unsafe@.
--
-- NOT COMPILED: no GHC was available where this was written.
--
module Data.Array.Accelerate.HIP.FFI where

import Data.Int
import Data.Word
import Foreign.C.String
import Foreign.C.Types
import Foreign.Ptr

data Ctx
data Prog
data Arr
data Event

foreign import ccall unsafe "acchip_last_error"        c_last_error        :: IO CString
foreign import ccall safe   "acchip_init"              c_init              :: CInt -> Ptr (Ptr Ctx) -> IO CInt
foreign import ccall safe   "acchip_shutdown"          c_shutdown          :: Ptr Ctx -> IO ()
foreign import ccall unsafe "acchip_mem_info"          c_mem_info          :: Ptr Ctx -> Ptr CSize -> Ptr CSize -> IO CInt
foreign import ccall safe   "acchip_malloc"            c_malloc            :: Ptr Ctx -> CSize -> IO (Ptr a)
foreign import ccall unsafe "acchip_free"              c_free              :: Ptr Ctx -> Ptr a -> IO ()
foreign import ccall safe   "acchip_purge"             c_purge             :: Ptr Ctx -> IO ()
foreign import ccall safe   "acchip_poke"              c_poke              :: Ptr Ctx -> Ptr a -> Ptr a -> CSize -> IO CInt
foreign import ccall safe   "acchip_peek"              c_peek              :: Ptr Ctx -> Ptr a -> Ptr a -> CSize -> IO CInt
foreign import ccall unsafe "acchip_stat"              c_stat              :: Ptr Ctx -> CString -> IO CLLong

foreign import ccall safe   "acchip_table_malloc"      c_table_malloc      :: Ptr Ctx -> Word64 -> Ptr a -> CSize -> CInt -> Ptr CInt -> IO CInt
foreign import ccall safe   "acchip_table_use"         c_table_use         :: Ptr Ctx -> Word64 -> Ptr (Ptr a) -> IO CInt
foreign import ccall unsafe "acchip_table_release"     c_table_release     :: Ptr Ctx -> Word64 -> IO CInt
foreign import ccall unsafe "acchip_table_free"        c_table_free        :: Ptr Ctx -> Word64 -> IO ()
foreign import ccall unsafe "acchip_table_insert_unmanaged"
                                                       c_table_insert_unmanaged :: Ptr Ctx -> Word64 -> Ptr a -> IO CInt
foreign import ccall unsafe "acchip_table_adopt"       c_table_adopt       :: Ptr Ctx -> Word64 -> Ptr a -> CSize -> Ptr Arr -> CInt -> CInt -> IO CInt
foreign import ccall safe   "acchip_table_reclaim"     c_table_reclaim     :: Ptr Ctx -> IO ()
foreign import ccall unsafe "acchip_table_status"      c_table_status      :: Ptr Ctx -> Word64 -> IO CInt
foreign import ccall safe   "acchip_set_clean_hook"    c_set_clean_hook    :: Ptr Ctx -> FunPtr (Ptr () -> IO ()) -> Ptr () -> IO CInt
foreign import ccall "wrapper"                         mkCleanHook         :: (Ptr () -> IO ()) -> IO (FunPtr (Ptr () -> IO ()))

foreign import ccall unsafe "acchip_set_flags"         c_set_flags         :: Ptr Ctx -> Word32 -> IO CInt
foreign import ccall unsafe "acchip_get_flags"         c_get_flags         :: Ptr Ctx -> IO Word32
-- the option word that accelerate's own cbits parse from the command line and $ACCELERATE_FLAGS (cbits/flags.c:44)
foreign import ccall        "&__cmd_line_flags"        cmdLineFlags        :: Ptr Word32
foreign import ccall unsafe "acchip_set_knob"          c_set_knob          :: Ptr Ctx -> CString -> CLLong -> IO CInt
foreign import ccall unsafe "acchip_get_knob"          c_get_knob          :: Ptr Ctx -> CString -> Ptr CLLong -> IO CInt

foreign import ccall unsafe "acchip_event_record"      c_event_record      :: Ptr Ctx -> Ptr (Ptr Event) -> IO CInt
foreign import ccall unsafe "acchip_event_query"       c_event_query       :: Ptr Event -> Ptr CInt -> IO CInt
foreign import ccall safe   "acchip_event_sync"        c_event_sync        :: Ptr Event -> IO CInt
foreign import ccall unsafe "acchip_event_destroy"     c_event_destroy     :: Ptr Event -> IO ()
foreign import ccall safe   "acchip_sync"              c_sync              :: Ptr Ctx -> IO CInt

foreign import ccall unsafe "acchip_array_wrap"        c_array_wrap        :: Ptr Ctx -> CInt -> Ptr Int64 -> CString -> Ptr (Ptr ()) -> CInt -> Ptr (Ptr Arr) -> IO CInt
foreign import ccall unsafe "acchip_array_pair"        c_array_pair        :: Ptr Arr -> Ptr Arr -> Ptr (Ptr Arr) -> IO CInt
foreign import ccall unsafe "acchip_array_unit"        c_array_unit        :: Ptr (Ptr Arr) -> IO CInt
foreign import ccall unsafe "acchip_array_kind"        c_array_kind        :: Ptr Arr -> IO CInt
foreign import ccall unsafe "acchip_array_fst"         c_array_fst         :: Ptr Arr -> Ptr (Ptr Arr) -> IO CInt
foreign import ccall unsafe "acchip_array_snd"         c_array_snd         :: Ptr Arr -> Ptr (Ptr Arr) -> IO CInt
foreign import ccall unsafe "acchip_array_rank"        c_array_rank        :: Ptr Arr -> IO CInt
foreign import ccall unsafe "acchip_array_shape"       c_array_shape       :: Ptr Arr -> Ptr Int64 -> IO CInt
foreign import ccall unsafe "acchip_array_buffer"      c_array_buffer      :: Ptr Arr -> CInt -> IO (Ptr ())
foreign import ccall unsafe "acchip_array_buffer_bytes" c_array_buffer_bytes :: Ptr Arr -> CInt -> IO CSize
foreign import ccall unsafe "acchip_array_release"     c_array_release     :: Ptr Arr -> IO ()

foreign import ccall safe   "acchip_compile"           c_compile           :: Ptr Ctx -> CString -> CSize -> Ptr (Ptr Prog) -> IO CInt
foreign import ccall unsafe "&acchip_program_release"  p_program_release   :: FunPtr (Ptr Prog -> IO ())
foreign import ccall unsafe "acchip_program_arity"     c_program_arity     :: Ptr Prog -> IO CInt
foreign import ccall safe   "acchip_execute"           c_execute           :: Ptr Ctx -> Ptr Prog -> Ptr (Ptr Arr) -> CInt -> Ptr (Ptr Arr) -> CInt -> Ptr (Ptr Arr) -> IO CInt
foreign import ccall safe   "acchip_execute_into"      c_execute_into      :: Ptr Ctx -> Ptr Prog -> Ptr (Ptr Arr) -> CInt -> Ptr (Ptr Arr) -> CInt -> Ptr Arr -> IO CInt

foreign import ccall safe   "acchip_set_trace"         c_set_trace         :: Ptr Ctx -> FunPtr (Ptr () -> CString -> Ptr Arr -> IO ()) -> Ptr () -> IO CInt
foreign import ccall "wrapper"                         mkTrace             :: (Ptr () -> CString -> Ptr Arr -> IO ()) -> IO (FunPtr (Ptr () -> CString -> Ptr Arr -> IO ()))
