(* Selected by dune when the optional library [hip_backend] can be built (libocannl_hip.so and ctypes
   are present): the real backend.  The twin of arrayjit/lib/cuda_backend_impl.cudajit.ml. *)
include Hip_backend
