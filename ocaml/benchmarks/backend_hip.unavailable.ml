(* The HIP plugin is not part of this build: nothing to initialise. *)
let init () = ()
