(* Selected by dune when the optional library [hip_backend] is absent: every entry point fails with
   "Backend hip missing -- install the corresponding library".  The twin of
   arrayjit/lib/cuda_backend_impl.missing.ml. *)
module Fresh () = struct
  include Lowered_backend_missing.Missing (struct
    let name = "hip"
  end)
end
