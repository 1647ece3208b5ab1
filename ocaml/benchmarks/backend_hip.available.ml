(* Goes to benchmarks/, sarek/tests/e2e/ and tools/ beside backend_cuda.available.ml (:7-10), with a
   select stanza in each dune file:
     (select backend_hip.ml from (sarek_hip -> backend_hip.available.ml) (-> backend_hip.unavailable.ml))
   and `Backend_hip.init ()` added to backend_loader.ml:9-17. *)
let init () =
  let no_gpu = Sys.getenv_opt "SPOC_DISABLE_GPU" = Some "1" in
  let no_hip = Sys.getenv_opt "SPOC_DISABLE_HIP" = Some "1" in
  if not (no_gpu || no_hip) then Sarek_hip.Hip_plugin.init ()
