(* nx_backend.ml for nx_hip — the OCaml half of the binding over libnxhip.

   Mirrors packages/nx/lib/backend_c/nx_backend.ml: compute ops allocate a fresh
   C-contiguous output and hand the strided operands to one C stub; movement
   ops are View metadata only. Not compiled in this repository's image (no
   OCaml toolchain); raven_amd/nx_backend.py is its executable twin and is what
   the parity tests drive.

   Every member of Backend_intf.S except the fft and linalg families is wired to
   the GPU. Those two must exist for the module to satisfy the signature; until
   they have device kernels they are answered by copying to the host, calling
   the C backend's routine and copying back, and are omitted from this excerpt. *)

open Nx_core

type context
type dev (* device allocation; finalised through the allocator of its context *)

external create_context : unit -> context = "caml_nx_hip_create_context"
external dev_alloc : context -> int -> dev = "caml_nx_hip_alloc"
external dev_bytes : dev -> int = "caml_nx_hip_bytes"

(* FIELD ORDER IS ABI (nx_hip_stubs.c reads slots 0-4). *)
type ('a, 'b) t = {
  buffer : dev;
  shape : int array;
  strides : int array;
  offset : int;
  tag : int; (* Dtype.Packed.tag *)
  dtype : ('a, 'b) Dtype.t;
  context : context;
}

let view t = View.create ~offset:t.offset ~strides:t.strides t.shape
let dtype t = t.dtype
let context t = t.context
let numel shape = Array.fold_left ( * ) 1 shape

let nbytes (type a b) (dt : (a, b) Dtype.t) n =
  match Dtype.Packed.tag (Dtype.Packed.P dt) with
  | 6 | 7 -> (n + 1) / 2
  | _ -> n * Dtype.itemsize dt

let create_tensor ctx dtype shape =
  let buffer = dev_alloc ctx (nbytes dtype (numel shape)) in
  { buffer; shape; strides = Shape.c_contiguous_strides shape; offset = 0;
    tag = Dtype.Packed.tag (Dtype.Packed.P dtype); dtype; context = ctx }

let buffer ctx dtype shape = create_tensor ctx dtype shape

external caml_from_host : dev -> ('a, 'b) Nx_buffer.t -> unit = "caml_nx_hip_from_host"
external caml_to_host : ('a, 'b) Nx_buffer.t -> dev -> unit = "caml_nx_hip_to_host"
external caml_fill : ('a, 'b) t -> ('a, 'b) Nx_buffer.t -> unit = "caml_nx_hip_fill"

let from_host ctx buf =
  let dtype = Nx_buffer.kind buf in
  let t = create_tensor ctx dtype [| Nx_buffer.length buf |] in
  caml_from_host t.buffer buf;
  t

(* The whole backing storage, to be read through the view (backend_intf.ml:108-116). *)
let to_host t =
  let bytes = dev_bytes t.buffer in
  let storage_len = (* elements the allocation holds *)
    if t.tag = 6 || t.tag = 7 then bytes * 2 else bytes / Dtype.itemsize t.dtype in
  let host = Nx_buffer.create t.dtype storage_len in
  caml_to_host host t.buffer;
  host

let full ctx dtype shape value =
  let t = create_tensor ctx dtype shape in
  let one = Nx_buffer.create dtype 1 in
  Nx_buffer.fill one value; (* the buffer layer owns the f16/bf16/fp8 encoding *)
  caml_fill t one;
  t

let of_view t v =
  { t with shape = View.shape v; strides = View.strides v; offset = View.offset v }

let expand t shape = of_view t (View.expand (view t) shape)
let reshape t shape = of_view t (View.reshape (view t) shape)
let permute t axes = of_view t (View.permute (view t) axes)
let shrink t bounds = of_view t (View.shrink (view t) bounds)
let flip t axes = of_view t (View.flip (view t) axes)
let is_c_contiguous t = View.is_c_contiguous (view t) && t.offset = 0

external caml_add : ('a, 'b) t -> ('a, 'b) t -> ('a, 'b) t -> unit = "caml_nx_hip_add"
external caml_mul : ('a, 'b) t -> ('a, 'b) t -> ('a, 'b) t -> unit = "caml_nx_hip_mul"
external caml_sin : ('a, 'b) t -> ('a, 'b) t -> unit = "caml_nx_hip_sin"
external caml_cmplt : (bool, Dtype.bool_elt) t -> ('a, 'b) t -> ('a, 'b) t -> unit = "caml_nx_hip_cmplt"
external caml_where : ('a, 'b) t -> (bool, Dtype.bool_elt) t -> ('a, 'b) t -> ('a, 'b) t -> unit = "caml_nx_hip_where"
external caml_cast : ('c, 'd) t -> ('a, 'b) t -> unit = "caml_nx_hip_cast"
external caml_copy : ('a, 'b) t -> ('a, 'b) t -> unit = "caml_nx_hip_copy"
external caml_reduce : int -> ('a, 'b) t -> ('a, 'b) t -> int array -> unit = "caml_nx_hip_reduce"
external caml_argreduce : bool -> (int32, Dtype.int32_elt) t -> ('a, 'b) t -> int -> unit = "caml_nx_hip_argreduce"
external caml_matmul : ('a, 'b) t -> ('a, 'b) t -> ('a, 'b) t -> unit = "caml_nx_hip_matmul"
external caml_gather : ('a, 'b) t -> ('a, 'b) t -> (int32, Dtype.int32_elt) t -> int -> unit = "caml_nx_hip_gather"
external caml_scatter : ('a, 'b) t -> (int32, Dtype.int32_elt) t -> ('a, 'b) t -> int -> int -> unit = "caml_nx_hip_scatter"
external caml_pad : ('a, 'b) t -> ('a, 'b) t -> ('a, 'b) Nx_buffer.t -> int array -> unit = "caml_nx_hip_pad"
external caml_cat : ('a, 'b) t -> ('a, 'b) t array -> int -> unit = "caml_nx_hip_cat"
external caml_scan : int -> ('a, 'b) t -> ('a, 'b) t -> int -> unit = "caml_nx_hip_scan"
external caml_threefry :
  (int32, Dtype.int32_elt) t -> (int32, Dtype.int32_elt) t -> (int32, Dtype.int32_elt) t -> unit = "caml_nx_hip_threefry"
external caml_sort : ('a, 'b) t -> ('a, 'b) t -> int -> bool -> unit = "caml_nx_hip_sort"
external caml_argsort : (int32, Dtype.int32_elt) t -> ('a, 'b) t -> int -> bool -> unit = "caml_nx_hip_argsort"
external caml_unfold : ('a, 'b) t -> ('a, 'b) t -> int array -> int array -> int array -> int array -> unit
  = "caml_nx_hip_unfold_bc" "caml_nx_hip_unfold"
external caml_fold_window :
  ('a, 'b) t -> ('a, 'b) t -> int array -> int array -> int array -> int array -> int array -> unit
  = "caml_nx_hip_fold_bc" "caml_nx_hip_fold"
(* ... one external per remaining unary / binary / compare stub, same shapes ... *)

let unary op x = let out = create_tensor x.context x.dtype x.shape in op out x; out
let binary op x y = let out = create_tensor x.context x.dtype x.shape in op out x y; out
let comparison op x y = let out = create_tensor x.context Dtype.Bool x.shape in op out x y; out

let add x y = binary caml_add x y
let mul x y = binary caml_mul x y
let sin x = unary caml_sin x
let cmplt x y = comparison caml_cmplt x y

let where cond a b =
  let out = create_tensor a.context a.dtype a.shape in
  caml_where out cond a b; out

let cast ~dtype x = let out = create_tensor x.context dtype x.shape in caml_cast out x; out
let copy x = let out = create_tensor x.context x.dtype x.shape in caml_copy out x; out
let contiguous x = if is_c_contiguous x then x else copy x
let assign dst src = caml_copy dst src

let reduce ~op ~axes x =
  let code, extreme =
    match op with
    | `Sum -> (0, None) | `Prod -> (1, None)
    | `Max -> (2, Some "reduce_max") | `Min -> (3, Some "reduce_min")
  in
  let axes = let a = Array.copy axes in Array.sort compare a; a in
  (match extreme with
   | Some name ->
     Array.iter (fun ax -> if x.shape.(ax) = 0 then
                    invalid_arg (name ^ ": reduction over an empty axis has no identity")) axes
   | None -> ());
  let out = create_tensor x.context x.dtype (Shape.reduce_output_shape x.shape axes false) in
  caml_reduce code out x axes; out

let argreduce name is_min ~axis ~keepdims x =
  if x.shape.(axis) = 0 then invalid_arg (name ^ ": argument reduction over an empty axis");
  let out = create_tensor x.context Dtype.Int32 (Shape.reduce_output_shape x.shape [| axis |] keepdims) in
  caml_argreduce is_min out x axis; out

let argmax ~axis ~keepdims x = argreduce "argmax" false ~axis ~keepdims x
let argmin ~axis ~keepdims x = argreduce "argmin" true ~axis ~keepdims x

let gather data indices ~axis =
  let out = create_tensor data.context data.dtype indices.shape in
  caml_gather out data indices axis; out

let matmul x y =
  let xs = x.shape and ys = y.shape in
  let xnd = Array.length xs and ynd = Array.length ys in
  let nd = Int.max xnd ynd in
  let batch = Array.init (nd - 2) (fun i ->
      let ai = i - (nd - xnd) and bi = i - (nd - ynd) in
      Int.max (if ai >= 0 then xs.(ai) else 1) (if bi >= 0 then ys.(bi) else 1)) in
  let out = create_tensor x.context x.dtype (Array.append batch [| xs.(xnd - 2); ys.(ynd - 1) |]) in
  caml_matmul out x y; out

(* nx_backend.ml:309-319 of the C backend *)
let associative_scan ~axis ~op x =
  let code = match op with `Sum -> 0 | `Prod -> 1 | `Max -> 2 | `Min -> 3 in
  let out = create_tensor x.context x.dtype x.shape in
  caml_scan code out x axis; out

(* nx_backend.ml:362-373: the fill value is stored into a 1-element host buffer
   with the typed Nx_buffer setter (so narrow floats use the buffer layer's
   converters) and handed to the stub as bytes *)
let pad x padding fill_value =
  let out_shape = Array.mapi (fun i d -> let b, a = padding.(i) in d + b + a) x.shape in
  let out = create_tensor x.context x.dtype out_shape in
  let fill = Nx_buffer.create x.dtype 1 in
  Nx_buffer.set fill 0 fill_value;
  caml_pad out x fill (Array.map fst padding); out

(* nx_backend.ml:379-393 *)
let cat tensors ~axis =
  match tensors with
  | [] -> invalid_arg "cat: empty tensor list"
  | first :: _ ->
    let ndim = Array.length first.shape in
    let axis = if axis < 0 then axis + ndim else axis in
    let total = List.fold_left (fun acc t -> acc + t.shape.(axis)) 0 tensors in
    let out = create_tensor first.context first.dtype
        (Array.mapi (fun i d -> if i = axis then total else d) first.shape) in
    caml_cat out (Array.of_list tensors) axis; out

(* nx_backend.ml:412-416 *)
let scatter ~mode ~unique_indices:_ template ~indices ~updates ~axis =
  let out = copy template in
  caml_scatter out indices updates axis (match mode with `Set -> 0 | `Add -> 1); out

(* nx_backend.ml:474-477 *)
let threefry key counter =
  let out = create_tensor counter.context Dtype.Int32 counter.shape in
  caml_threefry out key counter; out

(* nx_backend.ml:330-338 *)
let sort ~axis ~descending x =
  let out = create_tensor x.context x.dtype x.shape in
  caml_sort out x axis descending; out

let argsort ~axis ~descending x =
  let out = create_tensor x.context Dtype.Int32 x.shape in
  caml_argsort out x axis descending; out

(* nx_backend.ml:427-464 *)
let flatten_pairs p = Array.concat (Array.to_list (Array.map (fun (a, b) -> [| a; b |]) p))

let unfold x ~kernel_size ~stride ~dilation ~padding =
  let k = Array.length kernel_size in
  let leading_ndim = Array.length x.shape - k in
  let windows = ref 1 in
  for i = 0 to k - 1 do
    let before, after = padding.(i) in
    let padded = x.shape.(leading_ndim + i) + before + after in
    let extent = (dilation.(i) * (kernel_size.(i) - 1)) + 1 in
    windows := !windows * (((padded - extent) / stride.(i)) + 1)
  done;
  let taps = Array.fold_left ( * ) 1 kernel_size in
  let out = create_tensor x.context x.dtype
      (Array.append (Array.sub x.shape 0 leading_ndim) [| taps; !windows |]) in
  caml_unfold out x kernel_size stride dilation (flatten_pairs padding); out

let fold x ~output_size ~kernel_size ~stride ~dilation ~padding =
  let leading = Array.sub x.shape 0 (Array.length x.shape - 2) in
  let out = create_tensor x.context x.dtype (Array.append leading output_size) in
  caml_fold_window out x output_size kernel_size stride dilation (flatten_pairs padding); out
