(** The MI355X (gfx950) backend: [Backend_impl.Lowered_backend] (arrayjit/lib/backend_impl.ml:334-367)
    over the C ABI of [libocannl_hip.so] (include/ocannl_hip.h). The counterpart of
    arrayjit/lib/cuda_backend.ml; where that file calls [cudajit], this one calls the library, which
    owns the HIP runtime, hiprtc, the planner and the kernels.

    Division of labour: this module serialises [Low_level.optimized] ({!Hip_wire}), keeps the opaque
    handles alive for as long as OCaml values refer to them, translates status codes into the
    exceptions the CUDA backend raises, and maps the shared layer's [(device_id, pool_id)] keys onto
    pool ids of the library (which keys pools by physical device only). *)

open Base
open Ir
module Tn = Tnode
module Lazy = Utils.Lazy
open Backend_intf
open Ctypes
open Foreign

let _get_local_debug_runtime = Utils.get_local_debug_runtime

(* {1 The C ABI} *)

let lib = Dl.dlopen ~filename:"libocannl_hip.so" ~flags:[ Dl.RTLD_NOW; Dl.RTLD_GLOBAL ]
let f name typ = foreign ~from:lib ("ocannl_hip_" ^ name) typ
let last_error = f "last_error" (void @-> returning string)

(* status -> exception, as the CUDA backend raises them: User_error for user mistakes
   (cuda_backend.ml:668-689,1017-1029), Invalid_argument for misuse (:304,1031-1035), Failure for
   a failing driver. *)
let check (rc : int) : unit =
  if rc < 0 then
    let msg = last_error () in
    match rc with
    | -1 -> raise (Utils.User_error msg)
    | -2 -> invalid_arg msg
    | _ -> failwith msg

type handle = unit ptr

let h : handle typ = ptr void
let out_h = ptr (ptr void)

type node_loc

let node_loc : node_loc structure typ = structure "ocannl_hip_node_loc"
let nl_node = field node_loc "node_id" int32_t
let nl_pool = field node_loc "pool_id" int32_t
let nl_offset = field node_loc "offset" uint64_t
let () = seal node_loc
let init_ = f "init" (void @-> returning int)
let num_devices_ = f "num_devices" (ptr int @-> returning int)
let get_device_ = f "get_device" (int @-> out_h @-> returning int)
let static_properties_ = f "static_properties" (ptr char @-> size_t @-> returning int)
let get_used_memory_ = f "get_used_memory" (h @-> ptr uint64_t @-> returning int)
let get_debug_info_ = f "get_debug_info" (h @-> ptr char @-> size_t @-> returning int)
let get_global_debug_info_ = f "get_global_debug_info" (ptr char @-> size_t @-> returning int)
let await_ = f "await" (h @-> returning int)
let is_idle_ = f "is_idle" (h @-> ptr int @-> returning int)
let all_work_ = f "all_work" (h @-> out_h @-> returning int)
let sync_ = f "sync" (h @-> returning int)
let is_done_ = f "is_done" (h @-> ptr int @-> returning int)
let will_wait_for_ = f "will_wait_for" (h @-> h @-> returning int)
let event_free_ = f "event_free" (h @-> returning void)
let alloc_pool_ = f "alloc_pool" (h @-> int @-> uint64_t @-> uint64_t @-> returning int)
let free_pool_ = f "free_pool" (h @-> int @-> returning int)
let memset_zero_ = f "memset_zero" (h @-> int @-> uint64_t @-> uint64_t @-> returning int)
let from_host_ = f "from_host" (h @-> int @-> uint64_t @-> ptr void @-> uint64_t @-> returning int)
let to_host_ = f "to_host" (h @-> int @-> uint64_t @-> ptr void @-> uint64_t @-> returning int)

let device_to_device_ =
  f "device_to_device"
    (h @-> int @-> uint64_t @-> h @-> int @-> uint64_t @-> uint64_t @-> returning int)

let compile_opts_ = f "compile_opts" (string @-> size_t @-> string @-> out_h @-> returning int)
let code_free_ = f "code_free" (h @-> returning void)
let code_source_ = f "code_source" (h @-> ptr char @-> size_t @-> ptr size_t @-> returning int)

let code_object_ =
  f "code_object" (h @-> int @-> ptr char @-> size_t @-> ptr size_t @-> returning int)

let link_ = f "link" (h @-> h @-> int @-> ptr node_loc @-> int @-> out_h @-> returning int)
let routine_free_ = f "routine_free" (h @-> returning void)
let routine_set_static_ = f "routine_set_static" (h @-> int @-> int64_t @-> returning int)
let routine_run_ = f "routine_run" (h @-> returning int)
let routine_log_id_ = f "routine_log_id" (h @-> ptr int @-> returning int)
let u64 (n : int) = Unsigned.UInt64.of_int n

let get_handle (call : handle ptr -> int) : handle =
  let out = allocate (ptr void) null in
  check (call out);
  !@out

(* A text result of unknown length: the library truncates to [cap] and NUL-terminates. *)
let get_text ?(cap = 1 lsl 16) (call : char ptr -> Unsigned.size_t -> int) : string =
  let buf = CArray.make char cap in
  check (call (CArray.start buf) (Unsigned.Size_t.of_int cap));
  string_from_ptr (CArray.start buf)
    ~length:(Option.value ~default:cap (List.findi (CArray.to_list buf) ~f:(fun _ c -> Char.(c = '\000')) |> Option.map ~f:fst))

let sexp_of_text text = try Sexp.of_string text with _ -> Sexp.Atom text

(* {1 Types of the backend} *)

module Backend_buffer = struct
  (* The library resolves (pool, offset) itself, so the "pointer" of the implementation-facing layer
     is the library's id of the pool. *)
  type buffer_ptr = int [@@deriving sexp_of]

  include Backend_impl.Buffer_types (struct
    type nonrec buffer_ptr = buffer_ptr [@@deriving sexp_of]
  end)
end

module Device_config = struct
  include Backend_buffer

  type dev = { handle : (handle[@sexp.opaque]); ordinal : int } [@@deriving sexp_of]

  (* One non-blocking HIP stream per device lives inside the library's device object. *)
  type runner = unit [@@deriving sexp_of]

  (* [ocannl_hip_event*]; freed by a finaliser. *)
  type event = { ev : (handle[@sexp.opaque]) } [@@deriving sexp_of]

  let name = "hip"
end

module Device_stream = Backend_impl.Device_types_ll (Device_config)
open Device_config

(* The slab allocator (Backend_intf.Slab_alloc; cuda_backend.ml:60-94). The shared layer's pool ids
   are unique per device *instance* ([device_id]); instances of several [Fresh ()] backends may stand
   for the same GPU, for which the library keeps one pool table. So every [(device_id, pool_id)] gets
   a pool id of the library's that is unique in the process -- except the merge buffer, which is the
   library's pool 0 of the device (it grows that pool itself, see [device_to_device]). *)
module Slab = struct
  type device = Device_stream.device
  type buffer_ptr = int

  let pools : (int * int, int) Hashtbl.Poly.t = Hashtbl.Poly.create ()
  let next_lib_pool = ref 1

  let lib_pool (device : device) ~pool_id : int =
    if pool_id = merge_buffer_pool_id then 0
    else
      Hashtbl.find_or_add pools (device.device_id, pool_id) ~default:(fun () ->
          let id = !next_lib_pool in
          Int.incr next_lib_pool;
          id)

  let alloc_pool ?mode:_ (device : device) ~pool_id ~size_in_bytes ~alignment =
    (* allocating an id that exists frees the old slab first (only the merge pool regrows,
       cuda_backend.ml:71-76): the library does the same *)
    check
      (alloc_pool_ device.dev.handle (lib_pool device ~pool_id)
         (u64 (max 1 size_in_bytes))
         (u64 (max 1 alignment)))

  let free_pool =
    Some
      (fun (device : device) ~pool_id ->
        match
          if pool_id = merge_buffer_pool_id then Some 0
          else Hashtbl.find pools (device.device_id, pool_id)
        with
        | None -> ()
        | Some id ->
            check (free_pool_ device.dev.handle id);
            Hashtbl.remove pools (device.device_id, pool_id))

  let resolve_pool (device : device) ({ pool_id; offset = _ } : buffer_loc) : buffer_ptr =
    lib_pool device ~pool_id

  let memset_zero (device : device) ~pool_id ~offset ~size_in_bytes =
    if size_in_bytes > 0 then
      check
        (memset_zero_ device.dev.handle (lib_pool device ~pool_id) (u64 offset) (u64 size_in_bytes))
end

let initialized = ref false

module Fresh () : Ir.Backend_impl.Lowered_backend = struct
  include Backend_impl.Device (Device_stream) (Slab)
  include Backend_buffer

  let () =
    if not !initialized then (
      check (init_ ());
      initialized := true)

  let num_devices () =
    let n = allocate int 0 in
    check (num_devices_ n);
    !@n

  let devices = ref @@ Array.create ~len:(num_devices ()) None

  (* {2 Events (backend_intf.ml:221-251; cuda_backend.ml:108-111)} *)

  let all_work (device : device) : event =
    let ev = get_handle (all_work_ device.dev.handle) in
    let result = { ev } in
    Stdlib.Gc.finalise (fun (e : event) -> event_free_ e.ev) result;
    result

  let sync (event : event) = check (sync_ event.ev)

  let is_done (event : event) =
    let done_ = allocate int 0 in
    check (is_done_ event.ev done_);
    !@done_ <> 0

  let will_wait_for (context : context) (event : event) =
    check (will_wait_for_ context.device.dev.handle event.ev)

  (* {2 Devices (backend_intf.ml:206-266; cuda_backend.ml:113-260)} *)

  let get_used_memory (device : device) =
    let bytes = allocate uint64_t Unsigned.UInt64.zero in
    check (get_used_memory_ device.dev.handle bytes);
    Unsigned.UInt64.to_int !@bytes

  let finalize_device (device : device) =
    (* constants are bump-packed: free each distinct pool once (cuda_backend.ml:136-147) *)
    check (await_ device.dev.handle);
    Hashtbl.data device.constant_buffer_cache
    |> List.map ~f:(fun (loc : buffer_loc) -> loc.pool_id)
    |> List.dedup_and_sort ~compare:Int.compare
    |> List.iter ~f:(fun pool_id -> Option.iter Slab.free_pool ~f:(fun free -> free device ~pool_id))

  let get_device ~(ordinal : int) : device =
    if num_devices () <= ordinal then
      invalid_arg [%string "Hip_backend.get_device %{ordinal#Int}: not enough devices"];
    (if Array.length !devices <= ordinal then
       let old, len = (!devices, Array.length !devices) in
       devices := Array.init (ordinal + 1) ~f:(fun i -> if i < len then old.(i) else None));
    let default () =
      let handle = get_handle (get_device_ ordinal) in
      let result = make_device { handle; ordinal } () ~ordinal in
      Stdlib.Gc.finalise finalize_device result;
      !devices.(ordinal) <- Some result;
      result
    in
    Option.value_or_thunk !devices.(ordinal) ~default

  let new_stream (device : device) : device = device
  let await (device : device) : unit = check (await_ device.dev.handle)

  let is_idle (device : device) =
    let idle = allocate int 0 in
    check (is_idle_ device.dev.handle idle);
    !@idle <> 0

  let static_properties = sexp_of_text (get_text static_properties_)
  let get_debug_info (device : device) = sexp_of_text (get_text (get_debug_info_ device.dev.handle))

  (* live devices, events, compiled codes, linked routines and pool bytes of the whole process
     (backend_intf.ml:242; the CUDA backend reports its live streams, cuda_backend.ml:1088-1090) *)
  let get_global_debug_info () = sexp_of_text (get_text get_global_debug_info_)

  (* {2 Copies (backend_impl.ml:292-314; cuda_backend.ml:267-314)} *)

  (* The host array is the caller's and has to stay valid until the caller's [await]; the copy is
     asynchronous on the device's stream. *)
  let from_host ~(dst : context) ~(dst_loc : buffer_loc) hosted =
    check
      (from_host_ dst.device.dev.handle
         (Slab.lib_pool dst.device ~pool_id:dst_loc.pool_id)
         (u64 dst_loc.offset)
         (Ndarray.get_voidptr_not_managed hosted)
         (u64 (Ndarray.size_in_bytes hosted)))

  let to_host ~(src : context) ~(src_loc : buffer_loc) hosted =
    check
      (to_host_ src.device.dev.handle
         (Slab.lib_pool src.device ~pool_id:src_loc.pool_id)
         (u64 src_loc.offset)
         (Ndarray.get_voidptr_not_managed hosted)
         (u64 (Ndarray.size_in_bytes hosted)))

  let device_to_device (tn : Tn.t) ~into_merge_buffer ~(dst_loc : buffer_loc option) ~(dst : context)
      ~(src_loc : buffer_loc) ~(src : context) =
    let size_in_bytes = Lazy.force tn.Tn.size_in_bytes in
    let copy ~dst_pool ~dst_offset =
      check
        (device_to_device_ dst.device.dev.handle dst_pool (u64 dst_offset) src.device.dev.handle
           (Slab.lib_pool src.device ~pool_id:src_loc.pool_id)
           (u64 src_loc.offset) (u64 size_in_bytes))
    in
    match (into_merge_buffer, dst_loc) with
    | No, None -> invalid_arg "Hip_backend.device_to_device: missing dst_loc"
    | No, Some dst_loc ->
        copy ~dst_pool:(Slab.lib_pool dst.device ~pool_id:dst_loc.pool_id) ~dst_offset:dst_loc.offset
    | Copy, _ ->
        (* a destination pool of -1 asks the library for the device's merge buffer: its pool 0, which
           it regrows when the node does not fit (cuda_backend.ml:130-134) *)
        copy ~dst_pool:(-1) ~dst_offset:0;
        if dst.device.merge_buffer_capacity < size_in_bytes then
          dst.device.merge_buffer_capacity <- size_in_bytes;
        dst.device.merge_buffer := Some { pool_id = merge_buffer_pool_id; offset = 0 }

  (* {2 Compilation (backend_impl.ml:347-353; cuda_backend.ml:898-974)} *)

  type code_handle = { handle : (handle[@sexp.opaque]) } [@@deriving sexp_of]

  type code = {
    compiled : code_handle;
    index : int;  (** position of the routine inside the compiled blob *)
    name : string;
    bindings : Indexing.unit_bindings;
  }
  [@@deriving sexp_of]

  type code_batch = {
    compiled : code_handle;
    indices : int option array;  (** per position of the batch; [None] where it has no routine *)
    names : string option array;
    bindings : Indexing.unit_bindings;
  }
  [@@deriving sexp_of]

  let options () =
    String.concat ~sep:";"
    @@ List.filter_opt
         [
           Option.some_if Utils.settings.large_models "large_models=1";
           Option.some_if (Utils.debug_log_from_routines ()) "debug_log=1";
           (* anything else a user wants to try: [hip_options] in ocannl_config, e.g. "mfma=0;coop=0" for
              the summation order of the serial C code *)
           (match Utils.get_global_arg ~arg_name:"hip_options" ~default:"" with
           | "" -> None
           | s -> Some s);
         ]

  (* [output_debug_files_in_build_directory] (cuda_backend.ml:151-154,193-202): the generated source as
     [<name>.hip], and per routine the gfx950 code object as [<name>.hsaco] (what the CUDA backend
     writes as [.cu] and [.ptx]; `llvm-objdump -d` shows its ISA). *)
  let dump_debug_files ~name (compiled : code_handle) ~(n_routines : int) =
    let needed = allocate size_t Unsigned.Size_t.zero in
    let fetch call =
      check (call (from_voidp char null) Unsigned.Size_t.zero needed);
      let cap = Unsigned.Size_t.to_int !@needed in
      let buf = CArray.make char (max 1 cap) in
      check (call (CArray.start buf) (Unsigned.Size_t.of_int cap) needed);
      string_from_ptr (CArray.start buf) ~length:(min cap (Unsigned.Size_t.to_int !@needed))
    in
    let write ~extension contents =
      let build_file = Utils.open_build_file ~base_name:name ~extension in
      Stdio.Out_channel.output_string build_file.oc contents;
      build_file.finalize ()
    in
    write ~extension:".hip" (fetch (code_source_ compiled.handle));
    for index = 0 to n_routines - 1 do
      let suffix = if n_routines = 1 then "" else "-" ^ Int.to_string index in
      write ~extension:(suffix ^ ".hsaco") (fetch (code_object_ compiled.handle index))
    done

  let compile_batch ~(names : string option array) bindings (lowereds : Low_level.optimized option array)
      : code_batch =
    let debug = Utils.debug_log_from_routines () in
    let blob, indices = Hip_wire.to_wire ~debug ~names bindings lowereds in
    let compiled : code_handle =
      if String.is_empty blob then { handle = null }
      else
        {
          handle =
            get_handle (compile_opts_ blob (Unsigned.Size_t.of_int (String.length blob)) (options ()));
        }
    in
    (* drops this reference only: a linked routine keeps what it needs of the code alive *)
    Stdlib.Gc.finalise
      (fun (c : code_handle) -> if not (is_null c.handle) then code_free_ c.handle)
      compiled;
    (if Utils.settings.output_debug_files_in_build_directory && not (is_null compiled.handle) then
       let name =
         String.(
           strip ~drop:(equal_char '_')
           @@ common_prefix (Array.to_list names |> List.concat_map ~f:Option.to_list))
       in
       dump_debug_files ~name compiled ~n_routines:(Array.count indices ~f:Option.is_some));
    { compiled; indices; names; bindings }

  let compile ~name bindings (lowered : Low_level.optimized) : code =
    let batch = compile_batch ~names:[| Some name |] bindings [| Some lowered |] in
    { compiled = batch.compiled; index = 0; name; bindings }

  (* {2 Linking and running (backend_impl.ml:355-367; cuda_backend.ml:983-1086)} *)

  type routine_handle = { routine : (handle[@sexp.opaque]); keeps : (code_handle[@sexp.opaque]) }

  let link_proc ~(prior_context : context) ~(compiled : code_handle) ~index ~name
      ~(ctx_buffers : ctx_buffers) (lowered_bindings : Indexing.lowered_bindings) : Task.t =
    let device = prior_context.device in
    let stream_name = get_name device in
    (* ctx_buffers: Tnode -> { pool_id; offset }  =>  array of { node_id; pool id of the library; offset };
       the library picks out the nodes the routine takes as parameters and raises User_error when one
       is missing (as cc_backend.ml:411-415 does) *)
    let locs = CArray.make node_loc (Map.length ctx_buffers) in
    List.iteri (Map.to_alist ctx_buffers) ~f:(fun i ((tn : Tn.t), (loc : buffer_loc)) ->
        let entry = CArray.get locs i in
        setf entry nl_node (Int32.of_int_exn tn.id);
        setf entry nl_pool (Int32.of_int_exn (Slab.lib_pool device ~pool_id:loc.pool_id));
        setf entry nl_offset (u64 loc.offset));
    let handle =
      {
        routine =
          get_handle
            (link_ device.dev.handle compiled.handle index (CArray.start locs) (CArray.length locs));
        keeps = compiled;
      }
    in
    Stdlib.Gc.finalise (fun (r : routine_handle) -> routine_free_ r.routine) handle;
    let work () : unit =
      (* Static indices are read from their refs when the task runs (cuda_backend.ml:1015-1030); the
         library range-checks them and raises User_error before anything is enqueued.  The merge
         buffer, for a routine that reads one, is the device's pool 0 as it is now (:1009-1011). *)
      List.iter lowered_bindings ~f:(fun ((s : Indexing.static_symbol), (i : int ref)) ->
          check
            (routine_set_static_ handle.routine (Hip_wire.symbol_id s.static_symbol) (Int64.of_int !i)));
      check (routine_run_ handle.routine);
      if Utils.debug_log_from_routines () then (
        (* the kernels print `<log id>: ...$` lines to the process's standard output when the device
           is next synchronised; the reference's own reader picks them out by prefix
           (cuda_backend.ml:1040-1042, utils.ml:920,1047) *)
        let id = allocate int 0 in
        check (routine_log_id_ handle.routine id);
        Utils.add_log_processor ~prefix:(Int.to_string !@id ^ ": ") @@ fun log_contents ->
        Utils.log_debug_routine_logs ~log_contents ~stream_name)
    in
    Task.Task
      {
        context_lifetime = handle;
        description = "launches " ^ name ^ " on " ^ stream_name;
        work;
      }

  let fresh_bindings bindings : Indexing.lowered_bindings =
    List.map (Indexing.bound_symbols bindings) ~f:(fun s -> (s, ref 0))

  let link (prior_context : context) (code : code) ctx_buffers =
    let lowered_bindings = fresh_bindings code.bindings in
    let task =
      link_proc ~prior_context ~compiled:code.compiled ~index:code.index ~name:code.name ~ctx_buffers
        lowered_bindings
    in
    (lowered_bindings, task)

  let link_batch (prior_context : context) (code_batch : code_batch)
      (ctx_buffers : ctx_buffers option array) =
    let lowered_bindings = fresh_bindings code_batch.bindings in
    let procs =
      Array.mapi code_batch.indices ~f:(fun i index ->
          match (index, code_batch.names.(i), ctx_buffers.(i)) with
          | Some index, Some name, Some ctx_buffers ->
              Some
                (link_proc ~prior_context ~compiled:code_batch.compiled ~index ~name ~ctx_buffers
                   lowered_bindings)
          | _ -> None)
    in
    (lowered_bindings, procs)
end
