(* Structured errors of the HIP backend: the shared Backend_error functor under this backend's
   name (the CUDA plugin does the same, sarek-cuda/Cuda_error.ml:14-22). *)
include Spoc_framework.Backend_error.Make (struct
  let name = "HIP"
end)

exception Hip_error = Spoc_framework.Backend_error.Backend_error
