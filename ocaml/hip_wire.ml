(** Serialises [Low_level.optimized] for [libocannl_hip.so]: one S-expression per routine, the form
    that [ocannl_hip_compile_opts] reads (reader: ocannl_amd/csrc/llir.cpp; executable twin of this
    file: ocannl_amd/llir.py, [to_wire]).

    {v
    (routine NAME
      (static (SYM RANGE|-1) ...)          Indexing.static_symbol, arrayjit/lib/indexing.ml:32-36
      (merge NODE_ID|-1)                   optimized.merge_node, low_level.mli:160-166
      (nodes (ID "IDENT" PREC MODE ZERO_INIT READ_ONLY (DIM ...)) ...)
      (body STMT ...))
    v}

    Statements and scalars map one to one onto the constructors of [Low_level.t] / [scalar_t]
    (arrayjit/lib/low_level.mli:22-68), indices onto [Indexing.axis_index] (indexing.ml:104-120).
    [Noop] and [Seq] flatten into statement lists. [Staged_compilation] holds a closure that prints
    backend-specific source and cannot cross a serialised boundary: [Utils.User_error]. *)

open Base
open Ir
module Tn = Tnode
module Ll = Low_level

let symbol_id (Indexing.Symbol s) = s

(* A double-quoted atom: backslash and double quote escaped, nothing else (the reader undoes exactly
   these two). *)
let quote s =
  let b = Buffer.create (String.length s + 2) in
  Buffer.add_char b '"';
  String.iter s ~f:(fun c ->
      if Char.equal c '\\' || Char.equal c '"' then Buffer.add_char b '\\';
      Buffer.add_char b c);
  Buffer.add_char b '"';
  Buffer.contents b

(* C99 hexadecimal floating literal of a double, digit for digit what Python's [float.hex] prints:
   exact, and the text is then the same whichever side serialised the routine. *)
let hex_float (x : float) : string =
  if Float.is_nan x then "nan"
  else if Float.is_inf x then if Float.(x > 0.) then "inf" else "-inf"
  else
    let bits = Int64.bits_of_float x in
    let sign = if Int64.(bits < 0L) then "-" else "" in
    let exponent = Int64.(to_int_exn ((bits lsr 52) land 0x7FFL)) in
    let mantissa = Int64.(bits land 0xFFFFFFFFFFFFFL) in
    if exponent = 0 && Int64.(mantissa = 0L) then sign ^ "0x0.0p+0"
    else
      let lead, e = if exponent = 0 then (0, -1022) else (1, exponent - 1023) in
      Printf.sprintf "%s0x%d.%013Lxp%+d" sign lead mantissa e

let prec_atom (p : Ops.prec) = Ops.prec_string p

let binop_atom : Ops.binop -> string = function
  | Arg1 -> "arg1"
  | Arg2 -> "arg2"
  | Add -> "add"
  | Sub -> "sub"
  | Mul -> "mul"
  | Div -> "div"
  | ToPowOf -> "pow"
  | Relu_gate -> "relu_gate"
  | Satur01_gate -> "sat01_gate"
  | Max -> "max"
  | Min -> "min"
  | Mod -> "mod"
  | Cmplt -> "lt"
  | Cmpeq -> "eq"
  | Cmpne -> "ne"
  | Or -> "or"
  | And -> "and"
  | Threefry4x32_crypto -> "threefry4x32_crypto"
  | Threefry4x32_light -> "threefry4x32_light"

let unop_atom : Ops.unop -> string = function
  | Identity -> "id"
  | Relu -> "relu"
  | Satur01 -> "sat01"
  | Exp -> "exp"
  | Log -> "log"
  | Exp2 -> "exp2"
  | Log2 -> "log2"
  | Sin -> "sin"
  | Cos -> "cos"
  | Sqrt -> "sqrt"
  | Recip -> "recip"
  | Recip_sqrt -> "recip_sqrt"
  | Neg -> "neg"
  | Trunc -> "trunc"
  | Tanh_approx -> "tanh"
  | Not -> "not"
  | Uint4x32_to_prec_uniform1 -> "uint4x32_to_prec_uniform1"

let ternop_atom : Ops.ternop -> string = function Where -> "where" | FMA -> "fma" | Mul3 -> "mul3"

let vec_unop_atom : Ops.vec_unop -> string = function
  | Uint4x32_to_prec_uniform -> "uint4x32_to_prec_uniform"

let add = Buffer.add_string

let wire_idx b : Indexing.axis_index -> unit = function
  | Fixed_idx i -> add b (Printf.sprintf "(fixed %d)" i)
  | Iterator s -> add b (Printf.sprintf "(it %d)" (symbol_id s))
  | Sub_axis -> add b "(sub)"
  | Affine { symbols; offset } ->
      add b "(affine (";
      List.iteri symbols ~f:(fun i (coeff, s) ->
          if i > 0 then add b " ";
          add b (Printf.sprintf "(%d %d)" coeff (symbol_id s)));
      add b (Printf.sprintf ") %d)" offset)
  | Concat _ ->
      (* eliminated during lowering (indexing.ml:117-119) *)
      raise @@ Utils.User_error "hip backend: a Concat index reached the backend"

let wire_idcs b (idcs : Indexing.axis_index array) =
  add b "(";
  Array.iteri idcs ~f:(fun i idx ->
      if i > 0 then add b " ";
      wire_idx b idx);
  add b ")"

(* [debug]: every [Set] carries its [debug] field, the statement as [Low_level] prints it, which
   in-routine logging prints ahead of the values (c_syntax.ml:493-535). *)
let rec wire_stmts ~debug b (c : Ll.t) : unit =
  (* one statement per line inside the enclosing parentheses, [Noop] / [Seq] flattened *)
  let first = ref true in
  let rec go (c : Ll.t) =
    match c with
    | Noop -> ()
    | Seq (c1, c2) ->
        go c1;
        go c2
    | c ->
        if not !first then add b "\n";
        first := false;
        wire_stmt ~debug b c
  in
  add b "(";
  go c;
  add b ")"

and wire_stmt ~debug b (c : Ll.t) : unit =
  match c with
  | Noop | Seq _ -> assert false
  | Comment text -> add b (Printf.sprintf "(comment %s)" (quote text))
  | Staged_compilation _ ->
      raise
      @@ Utils.User_error
           "hip backend: Staged_compilation (backend-specific source text) cannot be serialised"
  | For_loop { index; from_; to_; body; trace_it = _ } ->
      add b (Printf.sprintf "(for %d %d %d " (symbol_id index) from_ to_);
      wire_stmts ~debug b body;
      add b ")"
  | Zero_out tn -> add b (Printf.sprintf "(zero_out %d)" tn.Tn.id)
  | Set { tn; idcs; llsc; debug = text } ->
      add b (Printf.sprintf "(set %d " tn.Tn.id);
      wire_idcs b idcs;
      add b " ";
      wire_scalar ~debug b llsc;
      if debug then add b (" " ^ quote text);
      add b ")"
  | Set_from_vec { tn; idcs; length; vec_unop; arg = arg, arg_prec; debug = _ } ->
      add b (Printf.sprintf "(set_vec %d " tn.Tn.id);
      wire_idcs b idcs;
      add b (Printf.sprintf " %d %s %s " length (vec_unop_atom vec_unop) (prec_atom arg_prec));
      wire_scalar ~debug b arg;
      add b ")"
  | Set_local ({ tn; scope_id }, llsc) ->
      add b (Printf.sprintf "(set_local %d %d " tn.Tn.id scope_id);
      wire_scalar ~debug b llsc;
      add b ")"
  | Declare_local { id = { tn; scope_id }; needs_init } ->
      add b (Printf.sprintf "(declare_local %d %d %d)" tn.Tn.id scope_id (Bool.to_int needs_init))

and wire_scalar ~debug b (s : Ll.scalar_t) : unit =
  match s with
  | Get (tn, idcs) ->
      add b (Printf.sprintf "(get %d " tn.Tn.id);
      wire_idcs b idcs;
      add b ")"
  | Get_merge_buffer (tn, idcs) ->
      add b (Printf.sprintf "(get_merge %d " tn.Tn.id);
      wire_idcs b idcs;
      add b ")"
  | Get_dynamic { tn; idcs; dyn_axis; dyn_value = value, value_prec } ->
      add b (Printf.sprintf "(get_dyn %d " tn.Tn.id);
      wire_idcs b idcs;
      add b (Printf.sprintf " %d %s " dyn_axis (prec_atom value_prec));
      wire_scalar ~debug b value;
      add b ")"
  | Get_local { tn; scope_id } -> add b (Printf.sprintf "(get_local %d %d)" tn.Tn.id scope_id)
  | Local_scope { id = { tn; scope_id }; body; orig_indices = _ } ->
      add b (Printf.sprintf "(local_scope %d %d " tn.Tn.id scope_id);
      wire_stmts ~debug b body;
      add b ")"
  | Constant c -> add b (Printf.sprintf "(const %s)" (hex_float c))
  | Constant_bits i -> add b (Printf.sprintf "(bits %Ld)" i)
  | Embed_index idx ->
      add b "(index ";
      wire_idx b idx;
      add b ")"
  | Unop (op, (arg, arg_prec)) ->
      add b (Printf.sprintf "(unop %s %s " (unop_atom op) (prec_atom arg_prec));
      wire_scalar ~debug b arg;
      add b ")"
  | Binop (op, (a1, _), (a2, _)) ->
      (* homogeneous-precision operation: the arguments' own precisions are overridden by the
         destination's (low_level.mli:66-68), so they do not travel *)
      add b (Printf.sprintf "(binop %s " (binop_atom op));
      wire_scalar ~debug b a1;
      add b " ";
      wire_scalar ~debug b a2;
      add b ")"
  | Ternop (op, (a1, a1_prec), (a2, _), (a3, _)) ->
      (* [Where] keeps the precision of its condition (ops.ml:798-829): the first argument's travels *)
      add b (Printf.sprintf "(ternop %s %s " (ternop_atom op) (prec_atom a1_prec));
      wire_scalar ~debug b a1;
      add b " ";
      wire_scalar ~debug b a2;
      add b " ";
      wire_scalar ~debug b a3;
      add b ")"

(* Memory mode of a node as the C printer classifies it for a routine (c_syntax.ml:1028-1045,
   1179-1196): [ctx] a kernel pointer parameter resolved through ctx_buffers at link time, [local] an
   array private to the routine, [virtual] never stored. *)
let mode_atom (tn : Tn.t) =
  if Tn.is_virtual_force tn 3341 then "virtual"
  else if Tn.is_in_context_force tn 3342 || Tn.is_materialized_force tn 3343 then "ctx"
  else "local"

(* A routine name has to be a C identifier (it names the generated kernels). *)
let c_identifier name =
  let s = String.map name ~f:(fun c -> if Char.is_alphanum c || Char.equal c '_' then c else '_') in
  if String.is_empty s || Char.is_digit s.[0] then "r_" ^ s else s

let wire_routine ~debug b ~(name : string) (statics : Indexing.static_symbol list)
    (lowered : Ll.optimized) : unit =
  let get_ident = Ll.get_ident_within_code ~no_dots:true [| lowered.llc |] in
  add b (Printf.sprintf "(routine %s\n(static " (quote (c_identifier name)));
  List.iteri statics ~f:(fun i (s : Indexing.static_symbol) ->
      if i > 0 then add b " ";
      add b
        (Printf.sprintf "(%d %d)" (symbol_id s.static_symbol) (Option.value s.static_range ~default:(-1))));
  add b
    (Printf.sprintf ")\n(merge %d)\n(nodes"
       (Option.value_map lowered.merge_node ~default:(-1) ~f:(fun tn -> tn.Tn.id)));
  (* every node the code mentions is in the traced store (low_level.mli:104-142); sorted by id so that
     the text does not depend on the hash table's iteration order *)
  let nodes =
    Hashtbl.to_alist lowered.traced_store
    |> List.sort ~compare:(fun (tn1, _) (tn2, _) -> Int.compare tn1.Tn.id tn2.Tn.id)
  in
  List.iter nodes ~f:(fun ((tn : Tn.t), (traced : Ll.traced_array)) ->
      add b
        (Printf.sprintf "\n(%d %s %s %s %d %d (" tn.id
           (quote (get_ident tn))
           (prec_atom (Lazy.force tn.prec))
           (mode_atom tn)
           (Bool.to_int traced.zero_initialized_by_code)
           (Bool.to_int traced.read_only));
      Array.iteri (Lazy.force tn.dims) ~f:(fun i d ->
          if i > 0 then add b " ";
          add b (Int.to_string d));
      add b "))");
  add b ")\n(body\n";
  (* the body's statements without the enclosing parentheses of a statement list *)
  let body = Buffer.create 4096 in
  wire_stmts ~debug body lowered.llc;
  let text = Buffer.contents body in
  add b (String.sub text ~pos:1 ~len:(String.length text - 2));
  add b "))\n"

(** The blob for a batch: one [(routine ...)] per [Some] entry, in order. Returns the blob and, per
    position of the batch, the index of its routine inside the blob ([None] entries have none): what
    [ocannl_hip_link] takes as [index]. *)
let to_wire ~debug ~(names : string option array) (bindings : Indexing.unit_bindings)
    (lowereds : Ll.optimized option array) : string * int option array =
  let statics = Indexing.bound_symbols bindings in
  let b = Buffer.create 65536 in
  let next = ref 0 in
  let indices =
    Array.map2_exn names lowereds ~f:(fun name lowered ->
        match (name, lowered) with
        | Some name, Some lowered ->
            wire_routine ~debug b ~name statics lowered;
            let i = !next in
            Int.incr next;
            Some i
        | None, None -> None
        | _ -> invalid_arg "Hip_wire.to_wire: names and routines disagree on which entries exist")
  in
  (Buffer.contents b, indices)
