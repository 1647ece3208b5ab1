(* Unit tests of Hip_error: the shared Backend_error functor under the name "HIP"
   (counterpart of sarek-cuda/test/test_cuda_error.ml for this plugin).  What matters for a
   backend is that every error the veneer raises (Hip_api.ml) carries the backend's name, the
   operation and the library's own failure text, and that the generic helpers see it. *)
open Sarek_hip

let has ~sub s =
  let n = String.length sub and m = String.length s in
  let rec at i = i + n <= m && (String.sub s i n = sub || at (i + 1)) in
  at 0

let shows what err subs () =
  let text = Hip_error.to_string err in
  List.iter (fun sub -> Alcotest.(check bool) (what ^ ": " ^ sub) true (has ~sub text)) ("HIP" :: subs)

(* the constructors Hip_api.ml raises, with arguments of the kind it passes *)
let raised_by_the_veneer =
  [ ("a failing call", Hip_error.context_error "sarek_hip_mem_get_info" "hipErrorInvalidDevice (101)",
     ["sarek_hip_mem_get_info"; "hipErrorInvalidDevice"]);
    ("library too old", Hip_error.initialization_failed "libsarek_hip.so has ABI version 2, this plugin expects 3", ["ABI version 2"]);
    ("device ordinal", Hip_error.device_not_found 5 1, ["5"]);
    ("synchronize", Hip_error.synchronization_failed "hipErrorLaunchFailure (719)", ["hipErrorLaunchFailure"]);
    ("allocation", Hip_error.memory_allocation_failed 1073741824L "hipErrorOutOfMemory (2)", ["1073741824"; "hipErrorOutOfMemory"]);
    ("copy", Hip_error.memory_copy_failed "host to device" 4096 "hipErrorInvalidValue (1)", ["host to device"; "4096"]);
    ("hiprtc log", Hip_error.compilation_failed "extern \"C\" __global__ void k() { oops }" "error: use of undeclared identifier 'oops'",
     ["undeclared identifier 'oops'"]);
    ("launch", Hip_error.kernel_launch_failed "sarek_kern" "argument 2 was never set", ["sarek_kern"; "argument 2"]) ]

let raised_by_the_plugin =
  [ ("a language this backend does not take", Hip_error.unsupported_source_lang "GLSL", ["GLSL"]);
    ("library not on the path", Hip_error.library_not_found "libsarek_hip.so" ["/usr/lib"; "/opt/rocm/lib"],
     ["libsarek_hip.so"; "/opt/rocm/lib"]);
    ("direct execution", Hip_error.feature_not_supported "execute_direct", ["execute_direct"]);
    ("generator refusal", Hip_error.unsupported_construct "SNative" "no HIP text in this node", ["SNative"]) ]

let test_helpers () =
  let err = Hip_error.no_device_selected "launch" in
  Alcotest.(check int) "with_default falls back" 7
    (Hip_error.with_default ~default:7 (fun () -> raise (Hip_error.Hip_error err))) ;
  Alcotest.(check int) "with_default passes a value through" 3 (Hip_error.with_default ~default:7 (fun () -> 3)) ;
  (match Hip_error.to_result (fun () -> Hip_error.raise_error err) with
   | Ok () -> Alcotest.fail "to_result lost the error"
   | Error e -> Alcotest.(check bool) "to_result keeps the error" true (e = err)) ;
  (* Hip_error.Hip_error IS the framework's exception: a handler written against either name catches both *)
  (try raise (Hip_error.Hip_error err) with
   | Spoc_framework.Backend_error.Backend_error e -> Alcotest.(check bool) "same exception" true (e = err)) ;
  Alcotest.(check bool) "equal arguments, equal errors" true
    (Hip_error.device_not_found 1 1 = Hip_error.device_not_found 1 1) ;
  Alcotest.(check bool) "different arguments, different errors" false
    (Hip_error.unsupported_source_lang "PTX" = Hip_error.unsupported_source_lang "SPIR-V")

let cases table = List.map (fun (what, err, subs) -> Alcotest.test_case what `Quick (shows what err subs)) table

let () =
  Alcotest.run "Hip_error"
    [ ("raised by Hip_api", cases raised_by_the_veneer);
      ("raised by Hip_plugin", cases raised_by_the_plugin);
      ("helpers", [Alcotest.test_case "with_default, to_result, the exception's identity" `Quick test_helpers]) ]
