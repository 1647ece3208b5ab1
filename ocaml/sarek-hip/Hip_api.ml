(* Device / Memory / Stream / Event / Kernel over the stubs of Hip_bindings: the typed layer the
   plugin modules are written against (the CUDA plugin's is sarek-cuda/Cuda_api.ml:27-512). *)
open Ctypes

let ( !! ) = Lazy.force

let null_voidp = from_voidp void null

let sz = Unsigned.Size_t.of_int

(* Status -> exception.  The library keeps the text of the last failure per thread. *)
let failure_text rc = Printf.sprintf "%s: %s" (!!Hip_bindings.status_name rc) (!!Hip_bindings.last_error ())

let check (operation : string) (rc : int) : unit =
  if rc <> 0 then Hip_error.raise_error (Hip_error.context_error operation (failure_text rc))

(* The ABI the library was built to and the struct layout this file declares must agree before
   the first call that fills a struct. *)
let expected_abi_version = 3

let verified =
  lazy
    (let v = !!Hip_bindings.abi_version () in
     if v <> expected_abi_version then
       Hip_error.raise_error
         (Hip_error.initialization_failed
            (Printf.sprintf "libsarek_hip.so has ABI version %d, this plugin was written for %d" v expected_abi_version)) ;
     let n = !!Hip_bindings.device_info_size () in
     if n <> sizeof Hip_bindings.device_info then
       Hip_error.raise_error
         (Hip_error.initialization_failed
            (Printf.sprintf "sarek_hip_device_info is %d bytes in the library, %d here" n (sizeof Hip_bindings.device_info))))

module Device = struct
  type t = {
    id : int;
    name : string;
    arch : string;
    total_mem : int64;
    compute_capability : int * int;
    max_threads_per_block : int;
    max_block_dims : int * int * int;
    max_grid_dims : int * int * int;
    shared_mem_per_block : int;
    warp_size : int;
    multiprocessor_count : int;
    clock_rate_khz : int;
    max_registers_per_block : int;
  }

  let initialised = ref false

  let cache : (int, t) Hashtbl.t = Hashtbl.create 4

  let init () =
    if not !initialised then begin
      Lazy.force verified ;
      check "init" (!!Hip_bindings.init ()) ;
      initialised := true
    end

  let count () =
    init () ;
    let n = allocate int 0 in
    check "device_count" (!!Hip_bindings.device_count n) ;
    !@n

  let c_string (a : char CArray.t) =
    let b = Buffer.create 32 in
    (try
       for i = 0 to CArray.length a - 1 do
         let c = CArray.get a i in
         if c = '\000' then raise Exit else Buffer.add_char b c
       done
     with Exit -> ()) ;
    Buffer.contents b

  let triple (a : int CArray.t) = (CArray.get a 0, CArray.get a 1, CArray.get a 2)

  let query idx =
    let n = count () in
    if idx < 0 || idx >= n then Hip_error.raise_error (Hip_error.device_not_found idx n) ;
    let info = make Hip_bindings.device_info in
    check "device_get_info" (!!Hip_bindings.device_get_info idx (addr info)) ;
    let g f = getf info f in
    {
      id = idx;
      name = c_string (g Hip_bindings.di_name);
      arch = c_string (g Hip_bindings.di_arch);
      total_mem = Unsigned.UInt64.to_int64 (g Hip_bindings.di_mem);
      compute_capability = (g Hip_bindings.di_major, g Hip_bindings.di_minor);
      max_threads_per_block = g Hip_bindings.di_threads;
      max_block_dims = triple (g Hip_bindings.di_bdim);
      max_grid_dims = triple (g Hip_bindings.di_gdim);
      shared_mem_per_block = g Hip_bindings.di_lds;
      warp_size = g Hip_bindings.di_warp;
      multiprocessor_count = g Hip_bindings.di_cus;
      clock_rate_khz = g Hip_bindings.di_clock;
      max_registers_per_block = g Hip_bindings.di_regs;
    }

  let get idx =
    match Hashtbl.find_opt cache idx with
    | Some d -> d
    | None ->
        let d = query idx in
        Hashtbl.replace cache idx d ;
        d

  let set_current d = check "device_set_current" (!!Hip_bindings.device_set_current d.id)

  let synchronize d =
    set_current d ;
    let rc = !!Hip_bindings.device_synchronize () in
    if rc <> 0 then Hip_error.raise_error (Hip_error.synchronization_failed (failure_text rc))
end

module Memory = struct
  (* size is in ELEMENTS (Framework_sig.ml Memory.alloc).  `freed` makes free safe to call twice
     from this side: the library's own idempotence is by address, and an address can be issued
     again by a later allocation before a late finaliser runs. *)
  type 'a buffer = {
    ptr : unit ptr;
    size : int;
    elem_size : int;
    device : Device.t;
    zero_copy : bool;
    mutable freed : bool;
  }

  let alloc_bytes device ~size ~elem_size =
    Device.set_current device ;
    let p = allocate (ptr void) null_voidp in
    let bytes = size * elem_size in
    let rc = !!Hip_bindings.mem_alloc p (sz bytes) in
    if rc <> 0 then
      Hip_error.raise_error (Hip_error.memory_allocation_failed (Int64.of_int bytes) (failure_text rc)) ;
    {ptr = !@p; size; elem_size; device; zero_copy = false; freed = false}

  let alloc device size kind = alloc_bytes device ~size ~elem_size:(Bigarray.kind_size_in_bytes kind)

  let alloc_custom device ~size ~elem_size = alloc_bytes device ~size ~elem_size

  (* Some only when the Bigarray lies in a block from host_alloc (pinned_bigarray below): the
     device then reads and writes the host block itself.  For any other Bigarray the library
     answers "not supported" and Transfer falls back to alloc + copy. *)
  let alloc_zero_copy device ba _kind =
    Device.set_current device ;
    let host = to_voidp (bigarray_start array1 ba) in
    let bytes = Bigarray.Array1.size_in_bytes ba in
    let p = allocate (ptr void) null_voidp and ok = allocate int 0 in
    check "alloc_zero_copy" (!!Hip_bindings.mem_alloc_zero_copy host (sz bytes) p ok) ;
    if !@ok = 0 then None
    else
      let n = Bigarray.Array1.dim ba in
      Some {ptr = !@p; size = n; elem_size = bytes / max 1 n; device; zero_copy = true; freed = false}

  let is_zero_copy b = b.zero_copy

  let free b =
    if not b.freed then begin
      b.freed <- true ;
      if not b.zero_copy then ignore (!!Hip_bindings.mem_free b.ptr)
    end

  let copy_failed direction bytes rc =
    Hip_error.raise_error (Hip_error.memory_copy_failed direction bytes (failure_text rc))

  let host_ptr_to_device ~src_ptr ~byte_size ~dst =
    let rc = !!Hip_bindings.memcpy_htod dst.ptr src_ptr (sz byte_size) in
    if rc <> 0 then copy_failed "host to device" byte_size rc

  let device_to_host_ptr ~src ~dst_ptr ~byte_size =
    let rc = !!Hip_bindings.memcpy_dtoh dst_ptr src.ptr (sz byte_size) in
    if rc <> 0 then copy_failed "device to host" byte_size rc

  let host_to_device ~src ~dst =
    host_ptr_to_device
      ~src_ptr:(to_voidp (bigarray_start array1 src))
      ~byte_size:(Bigarray.Array1.size_in_bytes src)
      ~dst

  let device_to_host ~src ~dst =
    device_to_host_ptr ~src
      ~dst_ptr:(to_voidp (bigarray_start array1 dst))
      ~byte_size:(Bigarray.Array1.size_in_bytes dst)

  let device_to_device ~src ~dst =
    let bytes = min (src.size * src.elem_size) (dst.size * dst.elem_size) in
    let rc = !!Hip_bindings.memcpy_dtod dst.ptr src.ptr (sz bytes) in
    if rc <> 0 then copy_failed "device to device" bytes rc

  let memset b value =
    check "memset" (!!Hip_bindings.memset_d8 b.ptr (Unsigned.UChar.of_int value) (sz (b.size * b.elem_size)))

  let size b = b.size

  let device_ptr b = raw_address_of_ptr b.ptr

  (* A Bigarray over a pinned host block.  Copies from and to it run at the PCIe rate without the
     library's staging step, and alloc_zero_copy accepts it.  To be called where the vector's host
     storage is created (sarek/core/Vector_storage.ml:22) when the HIP backend is in use. *)
  let pinned_bigarray kind n =
    let bytes = n * Bigarray.kind_size_in_bytes kind in
    let p = allocate (ptr void) null_voidp in
    check "host_alloc" (!!Hip_bindings.host_alloc p (sz bytes)) ;
    let block = !@p in
    let ba = bigarray_of_ptr array1 n kind (from_voidp (typ_of_bigarray_kind kind) block) in
    Gc.finalise (fun _ -> ignore (!!Hip_bindings.host_free block)) ba ;
    ba
end

module Stream = struct
  type t = {handle : unit ptr; device : Device.t}

  let create device =
    Device.set_current device ;
    let p = allocate (ptr void) null_voidp in
    check "stream_create" (!!Hip_bindings.stream_create p) ;
    {handle = !@p; device}

  let destroy s = if not (is_null s.handle) then check "stream_destroy" (!!Hip_bindings.stream_destroy s.handle)

  let synchronize s =
    let rc = !!Hip_bindings.stream_synchronize s.handle in
    if rc <> 0 then Hip_error.raise_error (Hip_error.synchronization_failed (failure_text rc))

  (* NULL is the device's default stream *)
  let default device = {handle = null_voidp; device}
end

module Event = struct
  type t = {handle : unit ptr}

  let create () =
    let p = allocate (ptr void) null_voidp in
    check "event_create" (!!Hip_bindings.event_create p) ;
    {handle = !@p}

  let destroy e = check "event_destroy" (!!Hip_bindings.event_destroy e.handle)

  let record e (s : Stream.t) = check "event_record" (!!Hip_bindings.event_record e.handle s.Stream.handle)

  let synchronize e = check "event_synchronize" (!!Hip_bindings.event_synchronize e.handle)

  (* milliseconds, as cuEventElapsedTime gives the CUDA plugin (Cuda_api.ml:289-293) *)
  let elapsed ~start ~stop =
    let ms = allocate float 0.0 in
    check "event_elapsed" (!!Hip_bindings.event_elapsed_ms start.handle stop.handle ms) ;
    !@ms
end

module Kernel = struct
  type t = {handle : unit ptr; name : string}

  (* Arguments are kept by position: Framework_sig's setters carry the index, and run_source lets
     a buffer's binder write its slot (Cuda_plugin.ml:189-199). *)
  type arg =
    | Buffer of unit ptr
    | Int32 of int32
    | Int64 of int64
    | Float32 of float
    | Float64 of float
    | Ptr of nativeint

  type args = {mutable slots : arg option array}

  let log_bytes = 16384

  let compile_with stub (device : Device.t) ~name ~source =
    Device.set_current device ;
    let out = allocate (ptr void) null_voidp in
    let log = allocate_n char ~count:log_bytes in
    let rc = !!stub source name out log (sz log_bytes) in
    if rc <> 0 then begin
      let text = coerce (ptr char) string log in
      let text = if text = "" then failure_text rc else text in
      Hip_error.raise_error (Hip_error.compilation_failed source text)
    end ;
    {handle = !@out; name}

  (* compile: a handle of the caller's own, to be released with destroy.  compile_cached: the
     library keeps one handle per (source, name) and device, in memory and as a code object on
     disk; those handles are released by clear_cache only. *)
  let compile device ~name ~source = compile_with Hip_bindings.kernel_compile device ~name ~source

  let compile_cached device ~name ~source = compile_with Hip_bindings.kernel_compile_cached device ~name ~source

  let destroy k = check "kernel_destroy" (!!Hip_bindings.kernel_destroy k.handle)

  let clear_cache () = check "kernel_clear_cache" (!!Hip_bindings.kernel_clear_cache ())

  let create_args () = {slots = [||]}

  let set args idx a =
    let n = Array.length args.slots in
    if idx >= n then args.slots <- Array.append args.slots (Array.make (idx + 1 - n) None) ;
    args.slots.(idx) <- Some a

  let set_arg_buffer args idx (b : _ Memory.buffer) = set args idx (Buffer b.Memory.ptr)

  let set_arg_int32 args idx v = set args idx (Int32 v)

  let set_arg_int64 args idx v = set args idx (Int64 v)

  let set_arg_float32 args idx v = set args idx (Float32 v)

  let set_arg_float64 args idx v = set args idx (Float64 v)

  let set_arg_ptr args idx v = set args idx (Ptr v)

  let to_list args =
    Array.to_list
      (Array.mapi
         (fun i -> function
           | Some a -> a
           | None -> Hip_error.raise_error (Hip_error.kernel_launch_failed "?" (Printf.sprintf "argument %d was never set" i)))
         args.slots)

  (* hipModuleLaunchKernel reads each argument through a pointer to a cell of the argument's own C
     type.  The cells must outlive the call: `keep` holds them. *)
  let launch k ~args ~grid:(gx, gy, gz) ~block:(bx, by, bz) ~shared_mem ~(stream : Stream.t option) =
    let cells =
      List.map
        (function
          | Buffer p -> to_voidp (allocate (ptr void) p)
          | Ptr n -> to_voidp (allocate (ptr void) (ptr_of_raw_address n))
          | Int32 v -> to_voidp (allocate int32_t v)
          | Int64 v -> to_voidp (allocate int64_t v)
          | Float32 v -> to_voidp (allocate float v)
          | Float64 v -> to_voidp (allocate double v))
        (to_list args)
    in
    let params = CArray.of_list (ptr void) cells in
    let dims a b c = CArray.of_list uint (List.map Unsigned.UInt.of_int [a; b; c]) in
    let g = dims gx gy gz and b = dims bx by bz in
    let s = match stream with Some s -> s.Stream.handle | None -> null_voidp in
    let rc =
      !!Hip_bindings.kernel_launch k.handle (CArray.start g) (CArray.start b) (Unsigned.UInt.of_int shared_mem) s
        (CArray.start params) (CArray.length params)
    in
    ignore (Sys.opaque_identity (cells, params, g, b)) ;
    if rc <> 0 then Hip_error.raise_error (Hip_error.kernel_launch_failed k.name (failure_text rc))
end

let is_available () =
  Hip_bindings.is_available ()
  && (try !!Hip_bindings.available () = 1 with _ -> false)

let driver_version () =
  let v = allocate int 0 in
  check "driver_version" (!!Hip_bindings.driver_version v) ;
  !@v

(* (free, total) bytes of the current device *)
let memory_info (device : Device.t) =
  Device.set_current device ;
  let free = allocate size_t Unsigned.Size_t.zero and total = allocate size_t Unsigned.Size_t.zero in
  check "mem_get_info" (!!Hip_bindings.mem_get_info free total) ;
  (Unsigned.Size_t.to_int64 !@free, Unsigned.Size_t.to_int64 !@total)

(* A text the library hands out in the "ask for the size, then fetch" style. *)
let fetch_text operation (call : char ptr -> Unsigned.size_t -> Unsigned.size_t ptr -> int) =
  let need = allocate size_t Unsigned.Size_t.zero in
  ignore (call (from_voidp char null) Unsigned.Size_t.zero need) ;
  let n = Unsigned.Size_t.to_int !@need in
  let buf = allocate_n char ~count:(max n 1) in
  check operation (call buf (sz (max n 1)) need) ;
  coerce (ptr char) string buf

(* The text tools/device_info.ml prints (tools/device_info.ml:45-93) and the device count. *)
let device_report () =
  let count = allocate int 0 in
  let text = fetch_text "device_report" (fun buf cap need -> !!Hip_bindings.device_report buf cap need count) in
  (text, !@count)

(* Names of the library kernels, and the (source, kernel_name) pair to hand to Execute.run_source:
   "gemm_bf16", "gemm_f16", "gemm_f16_bias_relu_rowsum", "triad_sum_f32". *)
let library_kernel_names () =
  String.split_on_char ' ' (fetch_text "library_kernel_list" (fun buf cap need -> !!Hip_bindings.library_kernel_list buf cap need))

let library_kernel name =
  let entry = allocate_n char ~count:128 in
  let source =
    fetch_text "library_kernel_source" (fun buf cap need ->
        !!Hip_bindings.library_kernel_source name buf cap need entry (sz 128))
  in
  (source, coerce (ptr char) string entry)

let set_tunable name value = check "set_tunable" (!!Hip_bindings.set_tunable name (Int64.of_int value))

let set_specialisation on = check "set_specialisation" (!!Hip_bindings.set_specialisation (if on then 1 else 0))

let last_run_path () = !!Hip_bindings.last_run_path ()
