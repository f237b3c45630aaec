(* nx_backend.ml for nx_hip — the OCaml half of the binding over libnxhip.

   Mirrors packages/nx/lib/backend_c/nx_backend.ml: compute ops allocate a fresh
   C-contiguous output and hand the strided operands to one C stub; movement
   ops are View metadata only. Not compiled in this repository's image (no
   OCaml toolchain); raven_amd/nx_backend.py is its executable twin and is what
   the parity tests drive.

   Every member of Backend_intf.S is wired to the GPU, the fft and linalg
   families included. *)

open Nx_core

type context
type dev (* device allocation; finalised through the allocator of its context *)

external create_context : unit -> context = "caml_nx_hip_create_context"
external dev_alloc : context -> int -> dev = "caml_nx_hip_alloc"
external dev_bytes : dev -> int = "caml_nx_hip_bytes"
external dtype_bytes : int -> int -> int = "caml_nx_hip_dtype_bytes" (* tag, count: the library's own count *)

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
external caml_sub : ('a, 'b) t -> ('a, 'b) t -> ('a, 'b) t -> unit = "caml_nx_hip_sub"
external caml_fdiv : ('a, 'b) t -> ('a, 'b) t -> ('a, 'b) t -> unit = "caml_nx_hip_fdiv"
external caml_idiv : ('a, 'b) t -> ('a, 'b) t -> ('a, 'b) t -> unit = "caml_nx_hip_idiv"
external caml_mod : ('a, 'b) t -> ('a, 'b) t -> ('a, 'b) t -> unit = "caml_nx_hip_mod"
external caml_pow : ('a, 'b) t -> ('a, 'b) t -> ('a, 'b) t -> unit = "caml_nx_hip_pow"
external caml_atan2 : ('a, 'b) t -> ('a, 'b) t -> ('a, 'b) t -> unit = "caml_nx_hip_atan2"
external caml_max : ('a, 'b) t -> ('a, 'b) t -> ('a, 'b) t -> unit = "caml_nx_hip_max"
external caml_min : ('a, 'b) t -> ('a, 'b) t -> ('a, 'b) t -> unit = "caml_nx_hip_min"
external caml_xor : ('a, 'b) t -> ('a, 'b) t -> ('a, 'b) t -> unit = "caml_nx_hip_xor"
external caml_or : ('a, 'b) t -> ('a, 'b) t -> ('a, 'b) t -> unit = "caml_nx_hip_or"
external caml_and : ('a, 'b) t -> ('a, 'b) t -> ('a, 'b) t -> unit = "caml_nx_hip_and"
external caml_neg : ('a, 'b) t -> ('a, 'b) t -> unit = "caml_nx_hip_neg"
external caml_recip : ('a, 'b) t -> ('a, 'b) t -> unit = "caml_nx_hip_recip"
external caml_abs : ('a, 'b) t -> ('a, 'b) t -> unit = "caml_nx_hip_abs"
external caml_sqrt : ('a, 'b) t -> ('a, 'b) t -> unit = "caml_nx_hip_sqrt"
external caml_sign : ('a, 'b) t -> ('a, 'b) t -> unit = "caml_nx_hip_sign"
external caml_exp : ('a, 'b) t -> ('a, 'b) t -> unit = "caml_nx_hip_exp"
external caml_log : ('a, 'b) t -> ('a, 'b) t -> unit = "caml_nx_hip_log"
external caml_cos : ('a, 'b) t -> ('a, 'b) t -> unit = "caml_nx_hip_cos"
external caml_tan : ('a, 'b) t -> ('a, 'b) t -> unit = "caml_nx_hip_tan"
external caml_asin : ('a, 'b) t -> ('a, 'b) t -> unit = "caml_nx_hip_asin"
external caml_acos : ('a, 'b) t -> ('a, 'b) t -> unit = "caml_nx_hip_acos"
external caml_atan : ('a, 'b) t -> ('a, 'b) t -> unit = "caml_nx_hip_atan"
external caml_sinh : ('a, 'b) t -> ('a, 'b) t -> unit = "caml_nx_hip_sinh"
external caml_cosh : ('a, 'b) t -> ('a, 'b) t -> unit = "caml_nx_hip_cosh"
external caml_tanh : ('a, 'b) t -> ('a, 'b) t -> unit = "caml_nx_hip_tanh"
external caml_trunc : ('a, 'b) t -> ('a, 'b) t -> unit = "caml_nx_hip_trunc"
external caml_ceil : ('a, 'b) t -> ('a, 'b) t -> unit = "caml_nx_hip_ceil"
external caml_floor : ('a, 'b) t -> ('a, 'b) t -> unit = "caml_nx_hip_floor"
external caml_round : ('a, 'b) t -> ('a, 'b) t -> unit = "caml_nx_hip_round"
external caml_erf : ('a, 'b) t -> ('a, 'b) t -> unit = "caml_nx_hip_erf"
external caml_cmpeq : (bool, Dtype.bool_elt) t -> ('a, 'b) t -> ('a, 'b) t -> unit = "caml_nx_hip_cmpeq"
external caml_cmpne : (bool, Dtype.bool_elt) t -> ('a, 'b) t -> ('a, 'b) t -> unit = "caml_nx_hip_cmpne"
external caml_cmple : (bool, Dtype.bool_elt) t -> ('a, 'b) t -> ('a, 'b) t -> unit = "caml_nx_hip_cmple"

let unary op x = let out = create_tensor x.context x.dtype x.shape in op out x; out
let binary op x y = let out = create_tensor x.context x.dtype x.shape in op out x y; out
let comparison op x y = let out = create_tensor x.context Dtype.Bool x.shape in op out x y; out

let add x y = binary caml_add x y
let mul x y = binary caml_mul x y
let sin x = unary caml_sin x
let cmplt x y = comparison caml_cmplt x y
let sub x y = binary caml_sub x y
let fdiv x y = binary caml_fdiv x y
let idiv x y = binary caml_idiv x y
let mod_ x y = binary caml_mod x y
let pow x y = binary caml_pow x y
let atan2 x y = binary caml_atan2 x y
let max x y = binary caml_max x y
let min x y = binary caml_min x y
let xor x y = binary caml_xor x y
let or_ x y = binary caml_or x y
let and_ x y = binary caml_and x y
let neg x = unary caml_neg x
let recip x = unary caml_recip x
let abs x = unary caml_abs x
let sqrt x = unary caml_sqrt x
let sign x = unary caml_sign x
let exp x = unary caml_exp x
let log x = unary caml_log x
let cos x = unary caml_cos x
let tan x = unary caml_tan x
let asin x = unary caml_asin x
let acos x = unary caml_acos x
let atan x = unary caml_atan x
let sinh x = unary caml_sinh x
let cosh x = unary caml_cosh x
let tanh x = unary caml_tanh x
let trunc x = unary caml_trunc x
let ceil x = unary caml_ceil x
let floor x = unary caml_floor x
let round x = unary caml_round x
let erf x = unary caml_erf x
let cmpeq x y = comparison caml_cmpeq x y
let cmpne x y = comparison caml_cmpne x y
let cmple x y = comparison caml_cmple x y

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
  let shape = Array.append batch [| xs.(xnd - 2); ys.(ynd - 1) |] in
  (* A long row that is no whole number of 128-byte lines (GPT-2's 50257 logits per token) gets a
     row pitch rounded up to whole lines; the result is the [..; n] view of that block, so every
     row of the GEMM's output starts on a line. The C backend allocates C-contiguous
     (nx_backend.ml:485-500 there). *)
  let n = shape.(nd - 1) in
  let line = 128 / Int.max 1 (nbytes x.dtype 1) in
  let out =
    if n < 4096 || n mod line = 0 || Array.exists (fun d -> d = 0) shape then create_tensor x.context x.dtype shape
    else begin
      let padded = Array.copy shape in
      padded.(nd - 1) <- (n + line - 1) / line * line;
      shrink (create_tensor x.context x.dtype padded) (Array.map (fun d -> (0, d)) shape)
    end in
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

(* Fourier transforms, nx_backend.ml:502-548: unnormalised; the binding owns shape and dtype *)
external caml_fft : (Complex.t, 'b) t -> (Complex.t, 'b) t -> int array -> unit = "caml_nx_hip_fft"
external caml_ifft : (Complex.t, 'b) t -> (Complex.t, 'b) t -> int array -> unit = "caml_nx_hip_ifft"
external caml_rfft : (Complex.t, 'b) t -> (float, 'a) t -> int array -> unit = "caml_nx_hip_rfft"
external caml_irfft : (float, 'b) t -> (Complex.t, 'a) t -> int array -> int array -> unit = "caml_nx_hip_irfft"

let fft x ~axes =
  let out = create_tensor x.context x.dtype x.shape in
  caml_fft out x axes; out

let ifft x ~axes =
  let out = create_tensor x.context x.dtype x.shape in
  caml_ifft out x axes; out

let rfft x ~dtype ~axes =
  let last = axes.(Array.length axes - 1) in
  let shape = Array.copy x.shape in
  shape.(last) <- (x.shape.(last) / 2) + 1;
  let out = create_tensor x.context dtype shape in
  caml_rfft out x axes; out

let irfft ?s x ~dtype ~axes =
  let li = Array.length axes - 1 in
  let last = axes.(li) in
  let size = match s with Some sizes -> sizes.(li) | None -> (x.shape.(last) - 1) * 2 in
  let shape = Array.copy x.shape in
  shape.(last) <- size;
  let out = create_tensor x.context dtype shape in
  caml_irfft out x axes (match s with Some sizes -> sizes | None -> [||]); out

(* linear algebra, nx_backend.ml:550-707. Numeric failures arrive as Failure with the
   reference's status text as suffix and are lifted to Linalg_error the same way. *)
external caml_cholesky : ('a, 'b) t -> ('a, 'b) t -> bool -> unit = "caml_nx_hip_cholesky"
external caml_triangular_solve : ('a, 'b) t -> ('a, 'b) t -> ('a, 'b) t -> int -> unit = "caml_nx_hip_triangular_solve"
external caml_qr : ('a, 'b) t -> ('a, 'b) t -> ('a, 'b) t -> bool -> unit = "caml_nx_hip_qr"
external caml_eigh : (float, Dtype.float64_elt) t -> ('a, 'b) t -> ('a, 'b) t -> bool -> unit = "caml_nx_hip_eigh"
external caml_svd : ('a, 'b) t -> (float, Dtype.float64_elt) t -> ('a, 'b) t -> ('a, 'b) t -> unit = "caml_nx_hip_svd"
external caml_eig :
  (Complex.t, Dtype.complex64_elt) t -> (Complex.t, Dtype.complex64_elt) t -> ('a, 'b) t -> bool -> unit
  = "caml_nx_hip_eig"

let reraise_linalg ~op f =
  try f ()
  with Failure msg as e ->
    let ends suffix = String.ends_with ~suffix msg in
    if ends "matrix is not positive definite" then raise (Backend_intf.Linalg_error { op; kind = `Not_positive_definite })
    else if ends "triangular matrix is singular" then raise (Backend_intf.Linalg_error { op; kind = `Singular })
    else if ends "eigenvalue iteration did not converge" then raise (Backend_intf.Linalg_error { op; kind = `No_convergence })
    else raise e

let cholesky ~upper x =
  let out = create_tensor x.context x.dtype x.shape in
  reraise_linalg ~op:"cholesky" (fun () -> caml_cholesky out x upper); out

let triangular_solve ~upper ~transpose ~unit_diag a b =
  let vector_rhs = Array.length b.shape = Array.length a.shape - 1 in
  let bm = if vector_rhs then reshape b (Array.append b.shape [| 1 |]) else b in
  let out = create_tensor b.context b.dtype bm.shape in
  let flags = (if upper then 1 else 0) lor (if transpose then 2 else 0) lor (if unit_diag then 4 else 0) in
  reraise_linalg ~op:"triangular_solve" (fun () -> caml_triangular_solve out a bm flags);
  if vector_rhs then reshape out b.shape else out

let matrix_dims x =
  let nd = Array.length x.shape in
  (Array.sub x.shape 0 (nd - 2), x.shape.(nd - 2), x.shape.(nd - 1))

let qr ~reduced x =
  let batch, m, n = matrix_dims x in
  let k = Int.min m n in
  let q = create_tensor x.context x.dtype (Array.append batch [| m; (if reduced then k else m) |]) in
  let r = create_tensor x.context x.dtype (Array.append batch [| (if reduced then k else m); n |]) in
  reraise_linalg ~op:"qr" (fun () -> caml_qr q r x reduced); (q, r)

let eigh_values x =
  let batch, _, n = matrix_dims x in
  create_tensor x.context Dtype.Float64 (Array.append batch [| n |])

let eigvalsh x =
  let w = eigh_values x in
  reraise_linalg ~op:"eigvalsh" (fun () -> caml_eigh w x x false); w

let eigh x =
  let w = eigh_values x in
  let v = create_tensor x.context x.dtype x.shape in
  reraise_linalg ~op:"eigh" (fun () -> caml_eigh w v x true); (w, v)

let svd ~full_matrices x =
  let batch, m, n = matrix_dims x in
  let k = Int.min m n in
  let u = create_tensor x.context x.dtype (Array.append batch (if full_matrices then [| m; m |] else [| m; k |])) in
  let s = create_tensor x.context Dtype.Float64 (Array.append batch [| k |]) in
  let vt = create_tensor x.context x.dtype (Array.append batch (if full_matrices then [| n; n |] else [| k; n |])) in
  reraise_linalg ~op:"svd" (fun () -> caml_svd u s vt x); (u, s, vt)

let eig_values x =
  let batch, _, n = matrix_dims x in
  create_tensor x.context Dtype.Complex128 (Array.append batch [| n |])

let eigvals x =
  let w = eig_values x in
  reraise_linalg ~op:"eigvals" (fun () -> caml_eig w w x false); w

let eig x =
  let w = eig_values x in
  let v = create_tensor x.context Dtype.Complex128 x.shape in
  reraise_linalg ~op:"eig" (fun () -> caml_eig w v x true); (w, v)

(* ── beyond Backend_intf.S ────────────────────────────────────────────────────
   Nothing below has a counterpart in the C backend. The frontend needs none of
   it to reach the fused kernels: [set_deferred ctx true] makes the primitive
   stubs above record their calls, and the library replaces the runs that spell
   softmax (frontend.ml:4242-4252), layer norm (kaun/lib/layer_norm.ml:43-68),
   GELU (fn.ml:31-38), the attention core (attention.ml:67-110) and linear +
   residual (linear.ml:50-52) by one kernel each when the next host read,
   [synchronize] or non-recordable operation executes the record. Intermediates
   are dropped from the record when their buffers are finalised before that, so
   a caller that wants the fusion to happen regardless of the collector's timing
   calls the operation by name through [Fused]. *)

external synchronize : context -> unit = "caml_nx_hip_synchronize"
external trim : context -> unit = "caml_nx_hip_trim"
external device_info : context -> int * string * int = "caml_nx_hip_device_info"
external memory_stats : context -> int array = "caml_nx_hip_memory_stats"
external last_path : context -> string = "caml_nx_hip_last_path"
external timer_start : context -> unit = "caml_nx_hip_timer_start"
external timer_stop : context -> float = "caml_nx_hip_timer_stop"
external set_deferred : context -> bool -> unit = "caml_nx_hip_set_deferred"

(* recorded, issued as recorded, flushes, fallbacks, then the runs replaced by
   softmax_rows, layer_norm_rows, gelu_tanh, attention and linear *)
external deferred_stats : context -> int array = "caml_nx_hip_deferred_stats"

(* bit 0 allows streaming loads, bit 1 streaming stores, of blocks whose history
   says they are not touched again while the memory-side cache still holds them *)
external set_cache_policy : context -> int -> unit = "caml_nx_hip_set_cache_policy"
external cache_policy_stats : context -> int * int = "caml_nx_hip_cache_policy_stats"

(* nx_effect.ml:376 returns its argument: the reference has one memory. Here a
   tensor of another context of the same GPU is copied by the target context's
   stream once the source stream has drained, and the target is drained before
   the source may be released. *)
let to_device ctx t =
  if t.context == ctx then t
  else begin
    synchronize t.context;
    let out = create_tensor ctx t.dtype t.shape in
    caml_copy out t;
    synchronize ctx;
    out
  end

(* reduce for callers that may not allocate: the split partials live in a static
   device array, the output is the caller's *)
external caml_reduce_noalloc : int -> ('a, 'b) t -> ('a, 'b) t -> int array -> unit = "caml_nx_hip_reduce_noalloc"

let reduce_into ~op ~axes ~out x =
  let code = match op with `Sum -> 0 | `Prod -> 1 | `Max -> 2 | `Min -> 3 in
  let axes = let a = Array.copy axes in Array.sort compare a; a in
  caml_reduce_noalloc code out x axes

module Fused = struct
  external caml_softmax_rows :
    ('c, 'd) t -> ('a, 'b) t -> ('a, 'b) Nx_buffer.t option -> (bool, Dtype.bool_elt) t option ->
    ('a, 'b) Nx_buffer.t option -> unit = "caml_nx_hip_softmax_rows"
  external caml_layer_norm_rows :
    ('a, 'b) t -> ('a, 'b) t -> ('a, 'b) t option -> ('a, 'b) t option -> float -> unit = "caml_nx_hip_layer_norm_rows"
  external caml_gelu_tanh : ('a, 'b) t -> ('a, 'b) t -> ('a, 'b) Nx_buffer.t -> unit = "caml_nx_hip_gelu_tanh"
  external caml_attention :
    ('a, 'b) t -> ('a, 'b) t -> ('a, 'b) t -> ('a, 'b) t -> (float, Dtype.float32_elt) Nx_buffer.t option ->
    (bool, Dtype.bool_elt) t option -> (float, Dtype.float32_elt) Nx_buffer.t option -> bool -> unit
    = "caml_nx_hip_attention_bc" "caml_nx_hip_attention"
  external caml_linear :
    ('a, 'b) t -> ('a, 'b) t -> ('a, 'b) t -> ('a, 'b) t option -> ('a, 'b) t option -> unit = "caml_nx_hip_linear"

  external caml_linear_gelu_tanh :
    ('a, 'b) t -> ('a, 'b) t -> ('a, 'b) t -> ('a, 'b) t option -> ('a, 'b) Nx_buffer.t -> unit
    = "caml_nx_hip_linear_gelu_tanh"

  let host_scalar dtype v =
    let b = Nx_buffer.create dtype 1 in
    Nx_buffer.set b 0 v; b

  (* softmax over the last axis of [x * scale], masked positions replaced by [fill] first *)
  let softmax ?scale ?mask x =
    let out = create_tensor x.context x.dtype x.shape in
    let mask, fill = match mask with
      | Some (m, fill) -> (Some (expand m x.shape), Some (host_scalar x.dtype fill))
      | None -> (None, None) in
    caml_softmax_rows out x (Option.map (host_scalar x.dtype) scale) mask fill; out

  let layer_norm ?gamma ?beta ~eps x =
    let out = create_tensor x.context x.dtype x.shape in
    caml_layer_norm_rows out x gamma beta eps; out

  let gelu_approx x =
    let out = create_tensor x.context x.dtype x.shape in
    let c = Nx_buffer.create x.dtype 4 in
    List.iteri (Nx_buffer.set c) [ 0.044715; Float.sqrt (2. /. Float.pi); 1.0; 0.5 ];
    caml_gelu_tanh out (contiguous x) c; out

  let gelu_constants dtype =
    let c = Nx_buffer.create dtype 4 in
    List.iteri (Nx_buffer.set c) [ 0.044715; Float.sqrt (2. /. Float.pi); 1.0; 0.5 ];
    c

  (* gelu_approx (linear x w + bias) in the GEMM's epilogue; Failure for shapes it does not take *)
  let linear_gelu ?bias x w =
    let nd = Array.length x.shape in
    let shape = Array.copy x.shape in
    shape.(nd - 1) <- w.shape.(Array.length w.shape - 1);
    let out = create_tensor x.context x.dtype shape in
    caml_linear_gelu_tanh out x w bias (gelu_constants x.dtype); out

  (* attention.ml:67-110 for float16 / bfloat16 operands of [batch..., seq, head_dim] *)
  let attention ?mask ?(causal = false) ~scale q k v =
    let out = create_tensor q.context q.dtype q.shape in
    let masked = if causal || mask <> None then Some (host_scalar Dtype.Float32 Float.neg_infinity) else None in
    let mask = Option.map (fun m ->
        let nd = Array.length q.shape in
        let target = Array.copy q.shape in
        target.(nd - 1) <- k.shape.(nd - 2);
        expand m target) mask in
    caml_attention out q k v (Some (host_scalar Dtype.Float32 scale)) mask masked causal; out

  (* linear.ml:50-52 and the residual add of gpt2.ml:165-176 in the GEMM's epilogue *)
  let linear ?bias ?residual x w =
    let nd = Array.length x.shape in
    let shape = Array.copy x.shape in
    shape.(nd - 1) <- w.shape.(Array.length w.shape - 1);
    let out = create_tensor x.context x.dtype shape in
    caml_linear out x w bias residual; out
end

(* Recorded sequences: every operation between [capture_begin] and [capture_end]
   is recorded instead of run; [Graph.launch] replays the whole sequence with
   one call, reading the inputs' current contents and writing the same outputs.
   Host reads, [synchronize], [trim] and the timer fail during a capture. *)
module Graph = struct
  type graph

  external capture_begin : context -> unit = "caml_nx_hip_capture_begin"
  external capture_end : context -> graph = "caml_nx_hip_capture_end"
  external launch : graph -> unit = "caml_nx_hip_graph_launch"
  external destroy : graph -> unit = "caml_nx_hip_graph_destroy"

  let record ctx f =
    capture_begin ctx;
    match f () with
    | result -> (capture_end ctx, result)
    | exception e -> (try destroy (capture_end ctx) with _ -> ()); raise e
end
