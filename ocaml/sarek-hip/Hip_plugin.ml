(* The HIP backend: Framework_sig.BACKEND for AMD Instinct GPUs, registered when this module is
   linked (the CUDA plugin's is sarek-cuda/Cuda_plugin.ml:146-256).

   generate_source prints the IR (Sarek_ir_hip) and has the library lower it to HIP text.  When
   the kernel is one the library has a hand-written kernel for, the text starts with a
   "// sarek-hip-specialise: <tag>" line; run_source hands the text back unchanged and the library
   serves the launch with that kernel when block, grid and the arguments fit, otherwise it
   compiles the text with hiprtc and launches it as written. *)
open Spoc_framework
open Spoc_framework_registry

module Hip_base = struct
  include Hip_plugin_base.Hip
end

type Framework_sig.kargs += Hip_kargs of Hip_base.Kernel.args

type hip_intrinsic = {
  intr_name : string;
  intr_codegen : string;
  intr_convergence : Framework_sig.convergence;
}

(* The registry lives in the library, because the lowering that consults it does: thread indices,
   barriers and fences are preloaded there in HIP spelling (sarek-cuda/Cuda_plugin.ml:47-143 holds
   the CUDA plugin's thirteen). *)
module Hip_intrinsics : Framework_sig.INTRINSIC_REGISTRY with type intrinsic_impl = hip_intrinsic = struct
  type intrinsic_impl = hip_intrinsic

  let convergence_tag = function Framework_sig.Uniform -> 0 | Divergent -> 1 | Sync -> 2

  let convergence_of_tag = function 0 -> Framework_sig.Uniform | 2 -> Framework_sig.Sync | _ -> Framework_sig.Divergent

  let register name impl =
    Hip_api.check "intrinsic_register"
      (Lazy.force Hip_bindings.intrinsic_register name impl.intr_codegen (convergence_tag impl.intr_convergence))

  let find name =
    let open Ctypes in
    let cap = 1024 in
    let buf = allocate_n char ~count:cap and conv = allocate int 0 and found = allocate int 0 in
    Hip_api.check "intrinsic_find"
      (Lazy.force Hip_bindings.intrinsic_find name buf (Unsigned.Size_t.of_int cap) conv found) ;
    if !@found = 0 then None
    else
      Some
        {
          intr_name = name;
          intr_codegen = coerce (ptr char) string buf;
          intr_convergence = convergence_of_tag !@conv;
        }

  let list_all () =
    Hip_api.fetch_text "intrinsic_list" (fun buf cap need -> Lazy.force Hip_bindings.intrinsic_list buf cap need)
    |> String.split_on_char '\n'
    |> List.filter (fun s -> s <> "")
end

(* Framework_sig.source_lang -> the library's language tags (the SAREK_HIP_LANG_ constants).  CUDA_Source text
   is taken as HIP text: the dialects agree on everything the generators and the benchmarks'
   external kernels use.  Tag 5 is HIP_Source, for when Framework_sig.source_lang has it. *)
let lang_tag = function
  | Framework_sig.CUDA_Source -> 0
  | Framework_sig.OpenCL_Source -> 1
  | Framework_sig.PTX -> 2
  | Framework_sig.SPIR_V -> 3
  | Framework_sig.GLSL_Source -> 4

let lang_name = function
  | Framework_sig.CUDA_Source -> "CUDA_Source"
  | Framework_sig.OpenCL_Source -> "OpenCL_Source"
  | Framework_sig.PTX -> "PTX"
  | Framework_sig.SPIR_V -> "SPIR_V"
  | Framework_sig.GLSL_Source -> "GLSL_Source"

(* run_source_arg list -> sarek_hip_arg[].  A buffer's binder writes its device pointer into the
   slot it is given (Memory.bind_to_kargs -> Kernel.set_arg_buffer, sarek/core/Memory.ml:78-81);
   the vector length travels beside it, the hand-written kernels check their launch against it. *)
let marshal_args (args : Framework_sig.run_source_arg list) =
  let open Ctypes in
  let n = List.length args in
  let arr = CArray.make Hip_bindings.arg n in
  List.iteri
    (fun i a ->
      let s = CArray.get arr i in
      let kind k = setf s Hip_bindings.a_kind k in
      match a with
      | Framework_sig.RSA_Buffer {binder; length} -> (
          let ka = Hip_base.Kernel.create_args () in
          binder (Hip_kargs ka) 0 ;
          match Hip_api.Kernel.to_list ka with
          | [Hip_api.Kernel.Buffer p] ->
              kind 0 ;
              setf s Hip_bindings.a_buffer p ;
              setf s Hip_bindings.a_length (Int64.of_int length)
          | [Hip_api.Kernel.Ptr p] ->
              kind 0 ;
              setf s Hip_bindings.a_buffer (ptr_of_raw_address p) ;
              setf s Hip_bindings.a_length (Int64.of_int length)
          | _ ->
              Hip_error.raise_error
                (Hip_error.kernel_launch_failed "run_source" (Printf.sprintf "argument %d: the binder bound no buffer" i)))
      | Framework_sig.RSA_Int32 v -> kind 1 ; setf s Hip_bindings.a_i32 v
      | Framework_sig.RSA_Int64 v -> kind 2 ; setf s Hip_bindings.a_i64 v
      | Framework_sig.RSA_Float32 v -> kind 3 ; setf s Hip_bindings.a_f32 v
      | Framework_sig.RSA_Float64 v -> kind 4 ; setf s Hip_bindings.a_f64 v)
    args ;
  arr

let dims_array (d : Framework_sig.dims) = Ctypes.(CArray.of_list int [d.x; d.y; d.z])

module Backend : Framework_sig.BACKEND = struct
  include Hip_base

  let execution_model = Framework_sig.JIT

  (* IR -> HIP text, lowered by the library.  ?block matters here (the CUDA plugin ignores it,
     Cuda_plugin.ml:153-157): the size of a shared array written in terms of the block dimensions
     becomes the constant a __shared__ declaration needs. *)
  let generate_source ?block (ir : Sarek_ir_types.kernel) : string option =
    try
      let open Ctypes in
      let text = Sarek_ir_hip.kernel ir in
      let blk = Option.map dims_array block in
      let blk_ptr = match blk with Some a -> CArray.start a | None -> from_voidp int null in
      let source =
        Hip_api.fetch_text "generate_source" (fun buf cap need ->
            Lazy.force Hip_bindings.generate_source text blk_ptr buf cap need)
      in
      ignore (Sys.opaque_identity blk) ;
      Some source
    with e ->
      Spoc_core.Log.debug Spoc_core.Log.Kernel ("Hip_plugin.generate_source: " ^ Printexc.to_string e) ;
      None

  let execute_direct ~native_fn:_ ~ir:_ ~block:_ ~grid:_ _args =
    Hip_error.raise_error (Hip_error.unsupported_source_lang "direct execution")

  module Intrinsics = Hip_intrinsics

  let supported_source_langs = [Framework_sig.CUDA_Source]

  let run_source ~source ~lang ~kernel_name ~block ~grid ~shared_mem args =
    match lang with
    | Framework_sig.CUDA_Source ->
        (match Hip_base.Device.get_current_device () with
        | Some d -> Hip_api.Device.set_current d
        | None -> Hip_error.raise_error (Hip_error.no_device_selected "run_source")) ;
        let arr = marshal_args args in
        let b = dims_array block and g = dims_array grid in
        let rc =
          Lazy.force Hip_bindings.run_source source (lang_tag lang) kernel_name (Ctypes.CArray.start b)
            (Ctypes.CArray.start g) shared_mem (Ctypes.CArray.start arr) (Ctypes.CArray.length arr)
        in
        ignore (Sys.opaque_identity (arr, b, g)) ;
        if rc = -3 (* SAREK_HIP_E_COMPILE *) then
          Hip_error.raise_error (Hip_error.compilation_failed source (Lazy.force Hip_bindings.last_error ()))
        else if rc <> 0 then
          Hip_error.raise_error (Hip_error.kernel_launch_failed kernel_name (Hip_api.failure_text rc))
    | other -> Hip_error.raise_error (Hip_error.unsupported_source_lang (lang_name other))

  let wrap_kargs a = Hip_kargs a

  let unwrap_kargs = function Hip_kargs a -> Some a | _ -> None
end

(* Several run_source calls handed to the library at once, in order, so that neighbouring kernels
   can share a launch (today: the stream triad followed by the block-256 sum of the vector it
   wrote runs as one pass over the data; the results are those of the separate launches).
   Every entry: (source, kernel_name, block, grid, shared_mem, arguments). *)
let run_sources
    (launches :
      (string * string * Framework_sig.dims * Framework_sig.dims * int * Framework_sig.run_source_arg list) list) =
  let open Ctypes in
  let arr = CArray.make Hip_bindings.launch (List.length launches) in
  let c_string s = CArray.of_string s in
  let keep =
    List.mapi
      (fun i (source, name, block, grid, shared_mem, args) ->
        let st = CArray.get arr i in
        let src = c_string source and nm = c_string name and a = marshal_args args in
        setf st Hip_bindings.l_source (CArray.start src) ;
        setf st Hip_bindings.l_lang (lang_tag Framework_sig.CUDA_Source) ;
        setf st Hip_bindings.l_name (CArray.start nm) ;
        let put field (d : Framework_sig.dims) =
          let c = getf st field in
          CArray.set c 0 d.x ; CArray.set c 1 d.y ; CArray.set c 2 d.z
        in
        put Hip_bindings.l_block block ;
        put Hip_bindings.l_grid grid ;
        setf st Hip_bindings.l_shmem shared_mem ;
        setf st Hip_bindings.l_args (CArray.start a) ;
        setf st Hip_bindings.l_nargs (CArray.length a) ;
        (src, nm, a))
      launches
  in
  let rc =
    Lazy.force Hip_bindings.run_sources (CArray.start arr) (CArray.length arr) (from_voidp int null)
      (from_voidp int null)
  in
  ignore (Sys.opaque_identity keep) ;
  Hip_api.check "run_sources" rc

let is_disabled () =
  Sys.getenv_opt "SPOC_DISABLE_GPU" = Some "1" || Sys.getenv_opt "SPOC_DISABLE_HIP" = Some "1"

(* Registered above CUDA's priority 100 (Cuda_plugin.ml:243-245): on a machine that has both
   libraries the devices of this backend come first in Device.best. *)
let registered_backend =
  lazy
    (if Backend.is_available () then begin
       Spoc_core.Log.debug Spoc_core.Log.Device "Hip_plugin: libsarek_hip.so and a device found, registering" ;
       Framework_registry.register_backend ~priority:110 (module Backend : Framework_sig.BACKEND)
     end
     else Spoc_core.Log.debug Spoc_core.Log.Device "Hip_plugin: HIP not available")

let () = if not (is_disabled ()) then Lazy.force registered_backend

let init () = if not (is_disabled ()) then Lazy.force registered_backend

(* extras beside the BACKEND signature *)
let register_intrinsic = Hip_intrinsics.register

let find_intrinsic = Hip_intrinsics.find

let library_kernel = Hip_api.library_kernel

let library_kernel_names = Hip_api.library_kernel_names

let device_report = Hip_api.device_report

let last_run_path = Hip_api.last_run_path
