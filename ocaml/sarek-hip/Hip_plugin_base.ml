(* Framework_sig.BACKEND without the code-generation half: Device / Memory / Stream / Event /
   Kernel in the framework's types, over Hip_api (the CUDA plugin's is
   sarek-cuda/Cuda_plugin_base.ml:146-303). *)
open Spoc_framework

module Hip = struct
  let name = "HIP"

  let version =
    try
      let major = Ctypes.allocate Ctypes.int 0
      and minor = Ctypes.allocate Ctypes.int 0
      and patch = Ctypes.allocate Ctypes.int 0 in
      ignore (Lazy.force Hip_bindings.backend_version major minor patch) ;
      Ctypes.(!@major, !@minor, !@patch)
    with _ -> (1, 0, 0)

  (* the device run_source compiles for and launches on; Execute sets it before every run *)
  let current_device : Hip_api.Device.t option ref = ref None

  module Device = struct
    type t = Hip_api.Device.t

    type id = int

    let init = Hip_api.Device.init

    let count = Hip_api.Device.count

    let get = Hip_api.Device.get

    let id (d : t) = d.Hip_api.Device.id

    let name (d : t) = d.Hip_api.Device.name

    let set_current (d : t) =
      Hip_api.Device.set_current d ;
      current_device := Some d

    let get_current_device () = !current_device

    let synchronize = Hip_api.Device.synchronize

    (* every member comes from the device query; the CUDA plugin has constants for the register
       file and the clock (Cuda_plugin_base.ml:190-193) *)
    let capabilities (d : t) : Framework_sig.capabilities =
      let open Hip_api.Device in
      {
        Framework_sig.max_threads_per_block = d.max_threads_per_block;
        max_block_dims = d.max_block_dims;
        max_grid_dims = d.max_grid_dims;
        shared_mem_per_block = d.shared_mem_per_block;
        total_global_mem = d.total_mem;
        compute_capability = d.compute_capability;
        supports_fp64 = true;
        supports_atomics = true;
        warp_size = d.warp_size;  (* 64: a wavefront *)
        max_registers_per_block = d.max_registers_per_block;
        clock_rate_khz = d.clock_rate_khz;
        multiprocessor_count = d.multiprocessor_count;  (* compute units *)
        is_cpu = false;
      }
  end

  module Memory = struct
    type 'a buffer = 'a Hip_api.Memory.buffer

    let alloc = Hip_api.Memory.alloc

    let alloc_custom = Hip_api.Memory.alloc_custom

    let alloc_zero_copy = Hip_api.Memory.alloc_zero_copy

    let is_zero_copy = Hip_api.Memory.is_zero_copy

    let free = Hip_api.Memory.free

    let host_to_device = Hip_api.Memory.host_to_device

    let device_to_host = Hip_api.Memory.device_to_host

    let host_ptr_to_device = Hip_api.Memory.host_ptr_to_device

    let device_to_host_ptr = Hip_api.Memory.device_to_host_ptr

    let device_to_device = Hip_api.Memory.device_to_device

    let size = Hip_api.Memory.size

    let device_ptr = Hip_api.Memory.device_ptr
  end

  module Stream = struct
    type t = Hip_api.Stream.t

    let create = Hip_api.Stream.create

    let destroy = Hip_api.Stream.destroy

    let synchronize = Hip_api.Stream.synchronize

    let default = Hip_api.Stream.default
  end

  module Event = struct
    type t = Hip_api.Event.t

    let create = Hip_api.Event.create

    let destroy = Hip_api.Event.destroy

    let record = Hip_api.Event.record

    let synchronize = Hip_api.Event.synchronize

    let elapsed = Hip_api.Event.elapsed
  end

  module Kernel = struct
    type t = Hip_api.Kernel.t

    type args = Hip_api.Kernel.args

    let compile = Hip_api.Kernel.compile

    let compile_cached = Hip_api.Kernel.compile_cached

    let clear_cache = Hip_api.Kernel.clear_cache

    let create_args = Hip_api.Kernel.create_args

    let set_arg_buffer = Hip_api.Kernel.set_arg_buffer

    let set_arg_int32 = Hip_api.Kernel.set_arg_int32

    let set_arg_int64 = Hip_api.Kernel.set_arg_int64

    let set_arg_float32 = Hip_api.Kernel.set_arg_float32

    let set_arg_float64 = Hip_api.Kernel.set_arg_float64

    let set_arg_ptr = Hip_api.Kernel.set_arg_ptr

    let launch kernel ~args ~grid ~block ~shared_mem ~stream =
      let open Framework_sig in
      Hip_api.Kernel.launch kernel ~args
        ~grid:(grid.x, grid.y, grid.z)
        ~block:(block.x, block.y, block.z)
        ~shared_mem ~stream
  end

  let enable_profiling () = ignore (Lazy.force Hip_bindings.profiler_start ())

  let disable_profiling () = ignore (Lazy.force Hip_bindings.profiler_stop ())

  let is_available = Hip_api.is_available
end
