## `HipTensor`: storage backend for AMD Instinct MI355X (gfx950), enabled with `-d:hip`.
##
## Occupies the slot of `CudaTensor` (src/arraymancer/tensor/data_structure.nim:29-67 and the
## `*_cuda.nim` operator files), for T in {float32, float64, int32, int64}, row-major by default,
## arbitrary strides everywhere. All device work goes through hip_abi.nim; there is no inline
## device code and no C++ backend requirement (`nim c` is enough).
##
## Hook-up inside Arraymancer:
##   tensor.nim:77-79      add  `when defined(hip): import ./tensor/tensor_hip; export tensor_hip`
##
## NOT COMPILED in the environment this repository is built in (no Nim toolchain there). The
## Python twin arraymancer_amd/tensor_hip.py issues exactly the same ABI calls and is what the
## parity tests drive.

import ./hip_abi
import arraymancer/laser/dynamic_stack_arrays      # Metadata
import arraymancer/laser/tensor/datatypes          # Tensor[T], KnownSupportsCopyMem
import arraymancer/tensor/data_structure            # shape_to_strides, is_C_contiguous, get_offset_ptr
import arraymancer/tensor/init_cpu                  # newTensorUninit
import arraymancer/tensor/shapeshifting             # asContiguous (host side, upload only)
import arraymancer/io/io_npy                        # read_npy / write_npy on host tensors
import arraymancer/tensor/private/p_display         # prettyImpl
import std/typetraits                               # type names for `pretty`
import std/math                                     # scalar sqrt for `std`

type
  HipScalar* = float32 | float64 | int32 | int64
  HipUnsigned* = uint32 | uint64
    ## ride the kernels of their signed twins for + - * and products (see the last section of this file)
  HipElem* = HipScalar | HipUnsigned | bool | uint8
    ## what a HipTensor can hold: the four arithmetic types, the two unsigned ones for ring operations, plus bool
    ## (one byte, the result of the comparison family) and uint8 (FloatClass ordinals of `classify`) as
    ## result-only element types

  HipRefTrackerObj*[T: HipElem] = object
    value*: ptr UncheckedArray[T]
  HipRefTracker*[T] = ref HipRefTrackerObj[T]

  HipStorage*[T: HipElem] = object
    Flen*: int
    Fdata*: ptr UncheckedArray[T]
    Fref_tracking*: HipRefTracker[T]

  HipTensor*[T: HipElem] = object
    ## Same fields as Tensor / CudaTensor: views share `storage`; shape, strides, offset in elements.
    shape*: Metadata
    strides*: Metadata
    offset*: int
    storage*: HipStorage[T]

proc `=destroy`*[T](p: HipRefTrackerObj[T]) =
  if not p.value.isNil:
    discard am_hip_free(p.value)

# ---------------------------------------------------------------- allocation / metadata
proc newHipStorage[T: HipElem](length: int): HipStorage[T] =
  result.Flen = length
  new result.Fref_tracking
  var p: pointer
  check am_hip_malloc(csize_t(length * sizeof(T)), p.addr)
  result.Fdata = cast[ptr UncheckedArray[T]](p)
  result.Fref_tracking.value = result.Fdata

proc size*(t: HipTensor): int {.inline.} = t.shape.product
proc rank*(t: HipTensor): int {.inline.} = t.shape.len

proc newHipTensor*[T: HipElem](shape: varargs[int] | Metadata): HipTensor[T] =
  ## Row-major, uninitialised.
  result.shape.copyFrom(shape)
  shape_to_strides(result.shape, rowMajor, result.strides)
  result.offset = 0
  result.storage = newHipStorage[T](result.shape.product)

proc get_offset_ptr*[T](t: HipTensor[T]): ptr T {.inline.} =
  t.storage.Fdata[t.offset].unsafeAddr

proc is_C_contiguous*(t: HipTensor): bool =
  var cur = 1
  for i in countdown(t.rank - 1, 0):
    if t.shape[i] != 1 and t.strides[i] != cur: return false
    cur *= t.shape[i]
  true

template i64s(m: Metadata): array[LASER_MAXRANK, int64] =
  var r: array[LASER_MAXRANK, int64]
  for i in 0 ..< m.len: r[i] = int64(m[i])
  r

# ---------------------------------------------------------------- transfers
proc toHip*[T: HipScalar | HipUnsigned](t: Tensor[T]): HipTensor[T] =
  ## Host -> device (the `cuda` proc, init_cuda.nim:23-41). Row-major on the device.
  let contig = t.asContiguous(rowMajor, force = true)
  result = newHipTensor[T](t.shape)
  if result.size > 0:
    check am_hip_memcpy_h2d(result.storage.Fdata, contig.get_offset_ptr, csize_t(result.size * sizeof(T)))

proc toCpu*[T: HipScalar | HipUnsigned](t: HipTensor[T]): Tensor[T] =
  ## Device -> host, blocking (the `cpu` proc, init_cuda.nim:43-59): the whole storage is copied
  ## and shape / strides / offset are kept.
  result = newTensorUninit[T](t.storage.Flen)
  if t.storage.Flen > 0:
    check am_hip_memcpy_d2h(result.get_offset_ptr, t.storage.Fdata, csize_t(t.storage.Flen * sizeof(T)))
  result.shape = t.shape
  result.strides = t.strides
  result.offset = t.offset

# ---------------------------------------------------------------- views (metadata only)
proc transpose*(t: HipTensor): HipTensor =
  t.shape.reversed(result.shape)
  t.strides.reversed(result.strides)
  result.offset = t.offset
  result.storage = t.storage

proc slice*[T](t: HipTensor[T], axis, first, last: int, step = 1): HipTensor[T] =
  ## `t[.., first..last|step, ..]` on one axis (inclusive ends), the arithmetic of slicerImpl
  ## (private/p_accessors_macros_read.nim:39-58).
  result = t
  result.offset += first * t.strides[axis]
  result.strides[axis] *= step
  result.shape[axis] = abs((last - first) div step) + 1

proc broadcast*[T](t: HipTensor[T], shape: varargs[int]): HipTensor[T] =
  ## broadcastImpl, private/p_shapeshifting.nim:76-94
  result = t
  doAssert t.rank == shape.len
  for i in 0 ..< t.rank:
    if t.shape[i] == 1:
      if shape[i] != 1:
        result.shape[i] = shape[i]
        result.strides[i] = 0
    elif t.shape[i] != shape[i]:
      raise newException(ValueError, "The broadcasted size of the tensor must match existing size for non-singleton dimension")

proc broadcast*[T: HipScalar | HipUnsigned](val: T, shape: varargs[int]): HipTensor[T] =
  ## Broadcast a number (shapeshifting.nim:136-176): one element of storage, every stride 0. Like the reference's,
  ## the result must not be written through (all positions share the element).
  result.shape.copyFrom(shape)
  result.strides = default(Metadata)
  result.strides.len = shape.len
  result.offset = 0
  result.storage = newHipStorage[T](1)
  var v = val
  check am_hip_memcpy_h2d(result.storage.Fdata, v.addr, csize_t(sizeof(T)))

template bc*[T: HipScalar | HipUnsigned](val: T, shape: varargs[int]): untyped = broadcast(val, shape)

proc broadcast2*[T](a, b: HipTensor[T]): tuple[a, b: HipTensor[T]] =
  ## broadcast2Impl, private/p_shapeshifting.nim:96-134
  if a.rank != b.rank:
    raise newException(ValueError, "Broadcasting error: ranks differ")
  result.a = a
  result.b = b
  for i in 0 ..< a.rank:
    if a.shape[i] == b.shape[i]: continue
    if a.shape[i] == 1:
      result.a.shape[i] = b.shape[i]; result.a.strides[i] = 0
    elif b.shape[i] == 1:
      result.b.shape[i] = a.shape[i]; result.b.strides[i] = 0
    else:
      raise newException(ValueError, "Broadcasting error: non-singleton dimensions must be the same in both tensors. Tensors' shapes were: " &
        $a.shape & " and " & $b.shape)

# ---------------------------------------------------------------- element-wise plumbing
template ewBinary(T: typedesc, op: AmBinaryOp, dst, a, b: untyped) =
  var sh = i64s(dst.shape)
  var sd = i64s(dst.strides)
  var sa = i64s(a.strides)
  var sb = i64s(b.strides)
  when T is float32:
    check am_hip_ew_binary_f32(cint(op), cint(dst.rank), sh[0].addr, dst.get_offset_ptr, sd[0].addr, a.get_offset_ptr, sa[0].addr, b.get_offset_ptr, sb[0].addr)
  elif T is float64:
    check am_hip_ew_binary_f64(cint(op), cint(dst.rank), sh[0].addr, dst.get_offset_ptr, sd[0].addr, a.get_offset_ptr, sa[0].addr, b.get_offset_ptr, sb[0].addr)
  elif T is int32:
    check am_hip_ew_binary_i32(cint(op), cint(dst.rank), sh[0].addr, dst.get_offset_ptr, sd[0].addr, a.get_offset_ptr, sa[0].addr, b.get_offset_ptr, sb[0].addr)
  else:
    check am_hip_ew_binary_i64(cint(op), cint(dst.rank), sh[0].addr, dst.get_offset_ptr, sd[0].addr, a.get_offset_ptr, sa[0].addr, b.get_offset_ptr, sb[0].addr)

template ewScalar(T: typedesc, op: AmBinaryOp, left: bool, dst, a: untyped, s: untyped) =
  var sh = i64s(dst.shape)
  var sd = i64s(dst.strides)
  var sa = i64s(a.strides)
  when T is float32:
    check am_hip_ew_scalar_f32(cint(op), cint(left), cint(dst.rank), sh[0].addr, dst.get_offset_ptr, sd[0].addr, a.get_offset_ptr, sa[0].addr, s)
  elif T is float64:
    check am_hip_ew_scalar_f64(cint(op), cint(left), cint(dst.rank), sh[0].addr, dst.get_offset_ptr, sd[0].addr, a.get_offset_ptr, sa[0].addr, s)
  elif T is int32:
    check am_hip_ew_scalar_i32(cint(op), cint(left), cint(dst.rank), sh[0].addr, dst.get_offset_ptr, sd[0].addr, a.get_offset_ptr, sa[0].addr, s)
  else:
    check am_hip_ew_scalar_i64(cint(op), cint(left), cint(dst.rank), sh[0].addr, dst.get_offset_ptr, sd[0].addr, a.get_offset_ptr, sa[0].addr, s)

template ewUnary(T: typedesc, op: AmUnaryOp, dst, a: untyped) =
  var sh = i64s(dst.shape)
  var sd = i64s(dst.strides)
  var sa = i64s(a.strides)
  when T is float32:
    check am_hip_ew_unary_f32(cint(op), cint(dst.rank), sh[0].addr, dst.get_offset_ptr, sd[0].addr, a.get_offset_ptr, sa[0].addr)
  elif T is float64:
    check am_hip_ew_unary_f64(cint(op), cint(dst.rank), sh[0].addr, dst.get_offset_ptr, sd[0].addr, a.get_offset_ptr, sa[0].addr)
  elif T is int32:
    check am_hip_ew_unary_i32(cint(op), cint(dst.rank), sh[0].addr, dst.get_offset_ptr, sd[0].addr, a.get_offset_ptr, sa[0].addr)
  else:
    check am_hip_ew_unary_i64(cint(op), cint(dst.rank), sh[0].addr, dst.get_offset_ptr, sd[0].addr, a.get_offset_ptr, sa[0].addr)

proc check_elementwise(a, b: HipTensor) =
  if a.shape != b.shape:
    raise newException(ValueError, "Both Tensors should have the same shape. Left-hand side has shape " &
      $a.shape & " while right-hand side has shape " & $b.shape)

proc map2*[T](a: HipTensor[T], op: AmBinaryOp, b: HipTensor[T]): HipTensor[T] =
  ## map2_inline with an enumerated body (a C ABI cannot carry a Nim expression).
  check_elementwise(a, b)
  result = newHipTensor[T](a.shape)
  if result.size > 0: ewBinary(T, op, result, a, b)

proc apply2Into[T](dst: var HipTensor[T], a: HipTensor[T], op: AmBinaryOp, b: HipTensor[T]) =
  ## dst[i] = op(a[i], b[i]) into an existing tensor of the operands' shape
  if dst.size > 0: ewBinary(T, op, dst, a, b)

proc apply2*[T](dest: var HipTensor[T], op: AmBinaryOp, src: HipTensor[T]) =
  check_elementwise(dest, src)
  if dest.size > 0: ewBinary(T, op, dest, dest, src)

proc clone*[T](t: HipTensor[T]): HipTensor[T] =
  result = newHipTensor[T](t.shape)
  if result.size > 0: ewUnary(T, uopCopy, result, t)

# ---------------------------------------------------------------- map bodies with another result type
# map_inline / map2_inline infer the result type from the body (higher_order_applymap.nim:69-120); over a C ABI
# the bodies are enumerated: the comparison family -> Tensor[bool], sgn -> Tensor[int], classify -> FloatClass.
template ewCompare(T: typedesc, op: AmCompareOp, dst, a, b: untyped) =
  var sh = i64s(dst.shape)
  var sd = i64s(dst.strides)
  var sa = i64s(a.strides)
  var sb = i64s(b.strides)
  let d = cast[ptr uint8](dst.get_offset_ptr)
  when T is float32:
    check am_hip_ew_compare_f32(cint(op), cint(dst.rank), sh[0].addr, d, sd[0].addr, a.get_offset_ptr, sa[0].addr, b.get_offset_ptr, sb[0].addr)
  elif T is float64:
    check am_hip_ew_compare_f64(cint(op), cint(dst.rank), sh[0].addr, d, sd[0].addr, a.get_offset_ptr, sa[0].addr, b.get_offset_ptr, sb[0].addr)
  elif T is int32:
    check am_hip_ew_compare_i32(cint(op), cint(dst.rank), sh[0].addr, d, sd[0].addr, a.get_offset_ptr, sa[0].addr, b.get_offset_ptr, sb[0].addr)
  else:
    check am_hip_ew_compare_i64(cint(op), cint(dst.rank), sh[0].addr, d, sd[0].addr, a.get_offset_ptr, sa[0].addr, b.get_offset_ptr, sb[0].addr)

template ewCompareScalar(T: typedesc, op: AmCompareOp, dst, a: untyped, s: untyped) =
  var sh = i64s(dst.shape)
  var sd = i64s(dst.strides)
  var sa = i64s(a.strides)
  let d = cast[ptr uint8](dst.get_offset_ptr)
  when T is float32:
    check am_hip_ew_compare_scalar_f32(cint(op), cint(dst.rank), sh[0].addr, d, sd[0].addr, a.get_offset_ptr, sa[0].addr, s)
  elif T is float64:
    check am_hip_ew_compare_scalar_f64(cint(op), cint(dst.rank), sh[0].addr, d, sd[0].addr, a.get_offset_ptr, sa[0].addr, s)
  elif T is int32:
    check am_hip_ew_compare_scalar_i32(cint(op), cint(dst.rank), sh[0].addr, d, sd[0].addr, a.get_offset_ptr, sa[0].addr, s)
  else:
    check am_hip_ew_compare_scalar_i64(cint(op), cint(dst.rank), sh[0].addr, d, sd[0].addr, a.get_offset_ptr, sa[0].addr, s)

proc map2*[T: HipScalar](a: HipTensor[T], op: AmCompareOp, b: HipTensor[T]): HipTensor[bool] =
  ## map2_inline with a bool-valued body, e.g. `map2(a, cmpModIsZero, b)` for `x mod y == 0`
  ## (tests/tensor/test_higherorder.nim:103-112).
  check_elementwise(a, b)
  result = newHipTensor[bool](a.shape)
  if result.size > 0: ewCompare(T, op, result, a, b)

proc compareScalar[T: HipScalar](t: HipTensor[T], op: AmCompareOp, value: T): HipTensor[bool] =
  result = newHipTensor[bool](t.shape)          # returnEmptyIfEmpty: an empty tensor comes back empty
  if result.size > 0: ewCompareScalar(T, op, result, t, value)

template genComparison(opName: untyped, code, mirrored: AmCompareOp) =
  ## operators_comparison.nim:41-94 (tensor, tensor: broadcast2 then map2_inline), :111-146 (tensor, scalar),
  ## :150-185 (scalar, tensor: the mirrored comparison of the tensor)
  proc opName*[T: HipScalar](a, b: HipTensor[T]): HipTensor[bool] =
    let (x, y) = broadcast2(a, b)
    map2(x, code, y)
  proc opName*[T: HipScalar](t: HipTensor[T], value: T): HipTensor[bool] = compareScalar(t, code, value)
  proc opName*[T: HipScalar](value: T, t: HipTensor[T]): HipTensor[bool] = compareScalar(t, mirrored, value)

genComparison(`==.`, cmpEq, cmpEq)
genComparison(`!=.`, cmpNe, cmpNe)
genComparison(`<.`, cmpLt, cmpGt)
genComparison(`<=.`, cmpLe, cmpGe)
genComparison(`>.`, cmpGt, cmpLt)
genComparison(`>=.`, cmpGe, cmpLe)

proc predicate[T: float32 | float64; D: bool | uint8](t: HipTensor[T], op: AmPredicate): HipTensor[D] =
  result = newHipTensor[D](t.shape)
  if result.size > 0:
    var sh = i64s(t.shape)
    var sd = i64s(result.strides)
    var sa = i64s(t.strides)
    let d = cast[ptr uint8](result.get_offset_ptr)
    when T is float32:
      check am_hip_ew_predicate_f32(cint(op), cint(t.rank), sh[0].addr, d, sd[0].addr, t.get_offset_ptr, sa[0].addr)
    else:
      check am_hip_ew_predicate_f64(cint(op), cint(t.rank), sh[0].addr, d, sd[0].addr, t.get_offset_ptr, sa[0].addr)

proc isNaN*[T: float32 | float64](t: HipTensor[T]): HipTensor[bool] = predicate[T, bool](t, predIsNaN)        ## operators_comparison.nim:192-198
proc isNotNaN*[T: float32 | float64](t: HipTensor[T]): HipTensor[bool] = predicate[T, bool](t, predIsNotNaN)  ## :200-206
proc classify*[T: float32 | float64](t: HipTensor[T]): HipTensor[uint8] = predicate[T, uint8](t, predClassify)
  ## ord(FloatClass) per element (math_functions.nim:264-276); `FloatClass(v)` converts a copied-back value

proc sgn*[T: HipScalar](t: HipTensor[T]): HipTensor[int64] =
  ## math_functions.nim:110-117: -1 / 0 / 1, zeros of either sign and NaN give 0
  result = newHipTensor[int64](t.shape)
  if result.size > 0:
    var sh = i64s(t.shape)
    var sd = i64s(result.strides)
    var sa = i64s(t.strides)
    when T is float32: check am_hip_ew_sgn_f32(cint(t.rank), sh[0].addr, result.get_offset_ptr, sd[0].addr, t.get_offset_ptr, sa[0].addr)
    elif T is float64: check am_hip_ew_sgn_f64(cint(t.rank), sh[0].addr, result.get_offset_ptr, sd[0].addr, t.get_offset_ptr, sa[0].addr)
    elif T is int32: check am_hip_ew_sgn_i32(cint(t.rank), sh[0].addr, result.get_offset_ptr, sd[0].addr, t.get_offset_ptr, sa[0].addr)
    else: check am_hip_ew_sgn_i64(cint(t.rank), sh[0].addr, result.get_offset_ptr, sd[0].addr, t.get_offset_ptr, sa[0].addr)

template ewClamp(T: typedesc, dst, a: untyped, lo, hi: untyped) =
  var sh = i64s(dst.shape)
  var sd = i64s(dst.strides)
  var sa = i64s(a.strides)
  when T is float32: check am_hip_ew_clamp_f32(cint(dst.rank), sh[0].addr, dst.get_offset_ptr, sd[0].addr, a.get_offset_ptr, sa[0].addr, lo, hi)
  elif T is float64: check am_hip_ew_clamp_f64(cint(dst.rank), sh[0].addr, dst.get_offset_ptr, sd[0].addr, a.get_offset_ptr, sa[0].addr, lo, hi)
  elif T is int32: check am_hip_ew_clamp_i32(cint(dst.rank), sh[0].addr, dst.get_offset_ptr, sd[0].addr, a.get_offset_ptr, sa[0].addr, lo, hi)
  else: check am_hip_ew_clamp_i64(cint(dst.rank), sh[0].addr, dst.get_offset_ptr, sd[0].addr, a.get_offset_ptr, sa[0].addr, lo, hi)

proc clamp*[T: HipScalar](t: HipTensor[T], min, max: T): HipTensor[T] =
  ## math_functions.nim:146-148; both bounds travel by value, one pass
  result = newHipTensor[T](t.shape)
  if result.size > 0: ewClamp(T, result, t, min, max)

proc mclamp*[T: HipScalar](t: var HipTensor[T], min, max: T) =
  ## math_functions.nim:150-152
  if t.size > 0: ewClamp(T, t, t, min, max)

proc floorMod*[T: HipScalar](t1, t2: HipTensor[T]): HipTensor[T] = map2(t1, opFloorMod, t2)      ## math_functions.nim:134-136
proc floorMod*[T: HipScalar](t: HipTensor[T], val: T): HipTensor[T] =                              ## :138-140
  result = newHipTensor[T](t.shape)
  if result.size > 0: ewScalar(T, opFloorMod, false, result, t, val)
proc floorMod*[T: HipScalar](val: T, t: HipTensor[T]): HipTensor[T] =                              ## :142-144
  result = newHipTensor[T](t.shape)
  if result.size > 0: ewScalar(T, opFloorMod, true, result, t, val)
proc copySign*[T: float32 | float64](t1, t2: HipTensor[T]): HipTensor[T] = map2(t1, opCopySign, t2)   ## :119-125
proc mcopySign*[T: float32 | float64](t1: var HipTensor[T], t2: HipTensor[T]) = apply2(t1, opCopySign, t2)   ## :127-132

# ---------------------------------------------------------------- BLAS L1-like operators
proc `+`*[T](a, b: HipTensor[T]): HipTensor[T] = map2(a, opAdd, b)
proc `-`*[T](a, b: HipTensor[T]): HipTensor[T] = map2(a, opSub, b)
proc `+=`*[T](a: var HipTensor[T], b: HipTensor[T]) = apply2(a, opAdd, b)
proc `-=`*[T](a: var HipTensor[T], b: HipTensor[T]) = apply2(a, opSub, b)

proc `*`*[T](s: T, t: HipTensor[T]): HipTensor[T] =
  result = newHipTensor[T](t.shape)
  if result.size > 0: ewScalar(T, opMul, true, result, t, s)
proc `*`*[T](t: HipTensor[T], s: T): HipTensor[T] = s * t
proc `/`*[T](t: HipTensor[T], s: T): HipTensor[T] =
  result = newHipTensor[T](t.shape)
  if result.size > 0: ewScalar(T, opDiv, false, result, t, s)
proc `*=`*[T](t: var HipTensor[T], s: T) =
  if t.size > 0: ewScalar(T, opMul, false, t, t, s)
proc `/=`*[T](t: var HipTensor[T], s: T) =
  if t.size > 0: ewScalar(T, opDiv, false, t, t, s)

# ---------------------------------------------------------------- broadcasting operators
proc `+.`*[T](a, b: HipTensor[T]): HipTensor[T] =
  let (ta, tb) = broadcast2(a, b)
  ta + tb
proc `-.`*[T](a, b: HipTensor[T]): HipTensor[T] =
  let (ta, tb) = broadcast2(a, b)
  ta - tb
proc `*.`*[T](a, b: HipTensor[T]): HipTensor[T] =
  let (ta, tb) = broadcast2(a, b)
  map2(ta, opMul, tb)
proc `/.`*[T](a, b: HipTensor[T]): HipTensor[T] =
  let (ta, tb) = broadcast2(a, b)
  map2(ta, opDiv, tb)       # integers: truncating `div`
proc `mod`*[T: HipScalar](a, b: HipTensor[T]): HipTensor[T] =
  let (ta, tb) = broadcast2(a, b)
  map2(ta, opMod, tb)       # integers: sign of the dividend; floats: C fmod, like std/math `mod`

proc `+.=`*[T](a: var HipTensor[T], b: HipTensor[T]) = apply2(a, opAdd, b.broadcast(a.shape.toSeq))
proc `-.=`*[T](a: var HipTensor[T], b: HipTensor[T]) = apply2(a, opSub, b.broadcast(a.shape.toSeq))
proc `*.=`*[T](a: var HipTensor[T], b: HipTensor[T]) = apply2(a, opMul, b.broadcast(a.shape.toSeq))
proc `/.=`*[T](a: var HipTensor[T], b: HipTensor[T]) = apply2(a, opDiv, b.broadcast(a.shape.toSeq))

proc `+.`*[T](t: HipTensor[T], s: T): HipTensor[T] =
  result = newHipTensor[T](t.shape)
  if result.size > 0: ewScalar(T, opAdd, false, result, t, s)
proc `+.`*[T](s: T, t: HipTensor[T]): HipTensor[T] = t +. s
proc `-.`*[T](t: HipTensor[T], s: T): HipTensor[T] =
  result = newHipTensor[T](t.shape)
  if result.size > 0: ewScalar(T, opSub, false, result, t, s)
proc `-.`*[T](s: T, t: HipTensor[T]): HipTensor[T] =
  result = newHipTensor[T](t.shape)
  if result.size > 0: ewScalar(T, opSub, true, result, t, s)
proc `*.`*[T](t: HipTensor[T], s: T): HipTensor[T] = s * t
proc `*.`*[T](s: T, t: HipTensor[T]): HipTensor[T] = s * t
proc `/.`*[T](t: HipTensor[T], s: T): HipTensor[T] = t / s
proc `/.`*[T](s: T, t: HipTensor[T]): HipTensor[T] =
  result = newHipTensor[T](t.shape)
  if result.size > 0: ewScalar(T, opDiv, true, result, t, s)

proc `^.`*[T: float32 | float64](t: HipTensor[T], exponent: T): HipTensor[T] =
  ## operators_broadcasted.nim:153-156
  result = newHipTensor[T](t.shape)
  if result.size > 0: ewScalar(T, opPow, false, result, t, exponent)
proc `^.`*[T: float32 | float64](base: T, t: HipTensor[T]): HipTensor[T] =
  ## operators_broadcasted.nim:158-161
  result = newHipTensor[T](t.shape)
  if result.size > 0: ewScalar(T, opPow, true, result, t, base)
proc `^.=`*[T: float32 | float64](t: var HipTensor[T], exponent: T) =
  ## operators_broadcasted.nim:178-182
  if t.size > 0: ewScalar(T, opPow, false, t, t, exponent)

template makeHipUniversal(name: untyped, code: AmUnaryOp) =
  ## The device twin of makeUniversal (ufunc.nim:56-68): `name` applied element-wise.
  proc name*[T: float32 | float64](t: HipTensor[T]): HipTensor[T] =
    result = newHipTensor[T](t.shape)
    if result.size > 0: ewUnary(T, code, result, t)

makeHipUniversal(ln, uopLn)
makeHipUniversal(log10, uopLog10)
makeHipUniversal(log2, uopLog2)
makeHipUniversal(exp, uopExp)
makeHipUniversal(sin, uopSin)
makeHipUniversal(cos, uopCos)
makeHipUniversal(tan, uopTan)
makeHipUniversal(sinh, uopSinh)
makeHipUniversal(cosh, uopCosh)
makeHipUniversal(tanh, uopTanh)
makeHipUniversal(arcsin, uopArcsin)
makeHipUniversal(arccos, uopArccos)
makeHipUniversal(arctan, uopArctan)
makeHipUniversal(arcsinh, uopArcsinh)
makeHipUniversal(arccosh, uopArccosh)
makeHipUniversal(arctanh, uopArctanh)
makeHipUniversal(cbrt, uopCbrt)
makeHipUniversal(erf, uopErf)
makeHipUniversal(erfc, uopErfc)
makeHipUniversal(gamma, uopGamma)
makeHipUniversal(lgamma, uopLgamma)
makeHipUniversal(floor, uopFloor)
makeHipUniversal(ceil, uopCeil)
makeHipUniversal(trunc, uopTrunc)
makeHipUniversal(round, uopRound)
makeHipUniversal(reciprocal, uopReciprocal)   # math_functions.nim:52-54
makeHipUniversal(degToRad, uopDegToRad)       # ufunc.nim:129
makeHipUniversal(radToDeg, uopRadToDeg)       # ufunc.nim:130
proc fac*[T: int32 | int64](t: HipTensor[T]): HipTensor[T] =
  ## ufunc.nim:84-85: Nim's `fac` over every element; it asserts 0 <= n <= 20, checked here with two reductions first.
  if t.size > 0: doAssert t.min >= T(0) and t.max <= T(20), "fac: every element must lie in 0 .. 20"
  result = newHipTensor[T](t.shape)
  if result.size > 0: ewUnary(T, uopFac, result, t)

proc mreciprocal*[T: float32 | float64](t: var HipTensor[T]) =
  ## math_functions.nim:56-58
  if t.size > 0: ewUnary(T, uopReciprocal, t, t)

proc relu*[T: float32 | float64](t: HipTensor[T]): HipTensor[T] =
  result = newHipTensor[T](t.shape)
  if result.size > 0: ewUnary(T, uopRelu, result, t)

proc biasRelu*[T: float32 | float64](x, b: HipTensor[T]): HipTensor[T] =
  ## map2_inline(x, b.broadcast(x.shape), max(0.T, x + y)) in one pass.
  map2(x, opAddRelu, b.broadcast(x.shape.toSeq))

proc relu_backward*[T: HipScalar](gradient, cached_tensor: HipTensor[T]): HipTensor[T] =
  ## nnp_activation.nim:65-70
  map2(cached_tensor, opReluBwd, gradient)
proc sigmoid_backward*[T: HipScalar](gradient, cached_tensor: HipTensor[T]): HipTensor[T] =
  ## x * (1 - x) * y, nnp_activation.nim:61-63
  map2(cached_tensor, opSigmoidBwd, gradient)
proc tanh_backward*[T: HipScalar](gradient, cached_tensor: HipTensor[T]): HipTensor[T] =
  ## y * (1 - x * x), nnp_activation.nim:72-74
  map2(cached_tensor, opTanhBwd, gradient)

# ---------------------------------------------------------------- GEMM
proc gemm*[T: HipScalar](alpha: T, A, B: HipTensor[T], beta: T, C: var HipTensor[T]) =
  ## C <- alpha A B + beta C (operators_blas_l2l3.nim:58-81). Any strides; no host copy.
  if A.rank != 2 or B.rank != 2 or C.rank != 2:
    raise newException(ValueError, "gemm: A, B and C must be matrices")
  when compileOption("boundChecks"):
    if A.shape[1] != B.shape[0]:
      raise newException(IndexDefect, "Number of columns in the first matrix: " & $A.shape[1] &
        ", must be the same as the number of rows in the second matrix: " & $B.shape[0])
  let (M, N, K) = (int64 A.shape[0], int64 B.shape[1], int64 A.shape[1])
  template call(f: untyped) =
    check f(M, N, K, alpha, A.get_offset_ptr, int64 A.strides[0], int64 A.strides[1],
            B.get_offset_ptr, int64 B.strides[0], int64 B.strides[1], beta,
            C.get_offset_ptr, int64 C.strides[0], int64 C.strides[1])
  when T is float32: call am_hip_gemm_f32
  elif T is float64: call am_hip_gemm_f64
  elif T is int32: call am_hip_gemm_i32
  else: call am_hip_gemm_i64

# Digit planes of an integer matrix split once for products that reuse it (a weight matrix): no counterpart in the
# reference, whose gemm_strided packs both operands in every call (gemm_packing.nim:24-99).
type
  HipDigitPlanesObj* = object
    handle*: pointer
  HipDigitPlanes* = ref HipDigitPlanesObj

proc `=destroy`*(p: HipDigitPlanesObj) =
  if not p.handle.isNil: discard am_hip_digits_release(p.handle)

proc digitsPrepare*[T: int32 | int64](t: HipTensor[T], rightOperand = true): HipDigitPlanes =
  ## Planes of `t` as the right ([K x N]) or left ([M x K]) operand of later products. A snapshot: prepare again
  ## after `t` changes. Blocking.
  new result
  when T is int32:
    check am_hip_digits_prepare_i32(cint(ord(rightOperand)), int64 t.shape[0], int64 t.shape[1], t.get_offset_ptr,
                                    int64 t.strides[0], int64 t.strides[1], result.handle.addr)
  else:
    check am_hip_digits_prepare_i64(cint(ord(rightOperand)), int64 t.shape[0], int64 t.shape[1], t.get_offset_ptr,
                                    int64 t.strides[0], int64 t.strides[1], result.handle.addr)

proc gemm*[T: int32 | int64](alpha: T, A, B: HipTensor[T], beta: T, C: var HipTensor[T], aDigits, bDigits: HipDigitPlanes) =
  ## `gemm` with the digit planes of A and / or B split ahead of time (nil: split that operand in the call).
  if A.rank != 2 or B.rank != 2 or C.rank != 2:
    raise newException(ValueError, "gemm: A, B and C must be matrices")
  let (M, N, K) = (int64 A.shape[0], int64 B.shape[1], int64 A.shape[1])
  let ha = if aDigits.isNil: nil else: aDigits.handle
  let hb = if bDigits.isNil: nil else: bDigits.handle
  template call(f: untyped) =
    check f(M, N, K, alpha, A.get_offset_ptr, int64 A.strides[0], int64 A.strides[1], ha,
            B.get_offset_ptr, int64 B.strides[0], int64 B.strides[1], hb, beta,
            C.get_offset_ptr, int64 C.strides[0], int64 C.strides[1])
  when T is int32: call am_hip_gemm_prepared_i32
  else: call am_hip_gemm_prepared_i64

proc gemv*[T: HipScalar](alpha: T, A, x: HipTensor[T], beta: T, y: var HipTensor[T]) =
  ## y <- alpha A x + beta y (operators_blas_l2l3.nim:24-56)
  template call(f: untyped) =
    check f(int64 A.shape[0], int64 A.shape[1], alpha, A.get_offset_ptr, int64 A.strides[0], int64 A.strides[1],
            x.get_offset_ptr, int64 x.strides[0], beta, y.get_offset_ptr, int64 y.strides[0])
  when T is float32: call am_hip_gemv_f32
  elif T is float64: call am_hip_gemv_f64
  elif T is int32: call am_hip_gemv_i32
  else: call am_hip_gemv_i64

proc dot*[T: HipScalar](a, b: HipTensor[T]): T =
  ## operators_blas_l1.nim:27-38
  when T is float32: check am_hip_dot_f32(int64 a.shape[0], a.get_offset_ptr, int64 a.strides[0], b.get_offset_ptr, int64 b.strides[0], result.addr)
  elif T is float64: check am_hip_dot_f64(int64 a.shape[0], a.get_offset_ptr, int64 a.strides[0], b.get_offset_ptr, int64 b.strides[0], result.addr)
  elif T is int32: check am_hip_dot_i32(int64 a.shape[0], a.get_offset_ptr, int64 a.strides[0], b.get_offset_ptr, int64 b.strides[0], result.addr)
  else: check am_hip_dot_i64(int64 a.shape[0], a.get_offset_ptr, int64 a.strides[0], b.get_offset_ptr, int64 b.strides[0], result.addr)

proc `*`*[T: HipScalar](a, b: HipTensor[T]): HipTensor[T] =
  ## Matrix-matrix product (operators_blas_l2l3.nim:88-100); matrix-vector goes to gemv.
  if a.rank == 2 and b.rank == 2:
    result = newHipTensor[T]([a.shape[0], b.shape[1]])
    gemm(T(1), a, b, T(0), result)
  elif a.rank == 2 and b.rank == 1:
    result = newHipTensor[T]([a.shape[0]])
    gemv(T(1), a, b, T(0), result)
  else:
    raise newException(ValueError, "Matrix-Matrix or Matrix-Vector multiplication valid only if first Tensor is a Matrix and second is a Matrix or Vector")

proc linear*[T: float32 | float64](x, weight, bias: HipTensor[T], relu = false): HipTensor[T] =
  ## out = x * weight.transpose +. bias (then relu): nnp_linear.nim:20-29 + nnp_activation.nim:35-36
  ## as ONE kernel (fused GEMM epilogue).
  result = newHipTensor[T]([x.shape[0], weight.shape[0]])
  let wt = weight.transpose
  let bb = bias.broadcast(result.shape.toSeq)
  let epi = if relu: AM_EPI_BIAS_RELU else: AM_EPI_BIAS
  when T is float32:
    check am_hip_gemm_ex_f32(int64 x.shape[0], int64 wt.shape[1], int64 x.shape[1], 1'f32,
      x.get_offset_ptr, int64 x.strides[0], int64 x.strides[1],
      wt.get_offset_ptr, int64 wt.strides[0], int64 wt.strides[1], 0'f32,
      result.get_offset_ptr, int64 result.strides[0], int64 result.strides[1],
      epi, bb.get_offset_ptr, int64 bb.strides[0], int64 bb.strides[1])
  else:
    check am_hip_gemm_ex_f64(int64 x.shape[0], int64 wt.shape[1], int64 x.shape[1], 1'f64,
      x.get_offset_ptr, int64 x.strides[0], int64 x.strides[1],
      wt.get_offset_ptr, int64 wt.strides[0], int64 wt.strides[1], 0'f64,
      result.get_offset_ptr, int64 result.strides[0], int64 result.strides[1],
      epi, bb.get_offset_ptr, int64 bb.strides[0], int64 bb.strides[1])

proc gru_cell_inference*[T: float32 | float64](input, W3, U3, bW3, bU3: HipTensor[T], hidden: var HipTensor[T]) =
  ## nn_primitives/nnp_gru.nim:40-88: h(t) -> h'(t) in place. The two dense layers carry their bias in the GEMM
  ## epilogue; steps 2-4 (the three apply2 / apply3 passes over column slices) are one launch.
  let H = hidden.shape[1]
  let W3x = linear(input, W3, bW3)
  let U3h = linear(hidden, U3, bU3)
  assert hidden.strides[1] == 1
  template call(f: untyped) =
    check f(int64 hidden.shape[0], int64 H, W3x.get_offset_ptr, int64 W3x.strides[0], U3h.get_offset_ptr, int64 U3h.strides[0],
            hidden.get_offset_ptr, int64 hidden.strides[0], nil, nil, nil, nil, 0'i64)
  when T is float32: call am_hip_gru_gates_f32
  else: call am_hip_gru_gates_f64

proc gru_cell_forward*[T: float32 | float64](input, W3, U3, bW3, bU3: HipTensor[T], r, z, n, Uh, hidden: var HipTensor[T]) =
  ## nn_primitives/nnp_gru.nim:90-146: the same cell, keeping r, z, n and the candidate's U3h slice for the backward pass.
  let H = hidden.shape[1]
  let W3x = linear(input, W3, bW3)
  let U3h = linear(hidden, U3, bU3)
  r = newHipTensor[T]([hidden.shape[0], H]); z = newHipTensor[T]([hidden.shape[0], H])
  n = newHipTensor[T]([hidden.shape[0], H]); Uh = newHipTensor[T]([hidden.shape[0], H])
  assert hidden.strides[1] == 1
  template call(f: untyped) =
    check f(int64 hidden.shape[0], int64 H, W3x.get_offset_ptr, int64 W3x.strides[0], U3h.get_offset_ptr, int64 U3h.strides[0],
            hidden.get_offset_ptr, int64 hidden.strides[0], r.get_offset_ptr, z.get_offset_ptr, n.get_offset_ptr, Uh.get_offset_ptr, int64 H)
  when T is float32: call am_hip_gru_gates_f32
  else: call am_hip_gru_gates_f64

# ---------------------------------------------------------------- reductions, softmax, pooling
proc reduce_axis[T: HipScalar](op: cint, t: HipTensor[T], axis: int): HipTensor[T] =
  ## reduce_axis_inline (higher_order_foldreduce.nim:46-61): the result keeps `axis` with extent 1.
  if axis < 0 or axis >= t.rank:
    raise newException(IndexDefect, "Input tensor rank (" & $t.rank & ") must be greater than reduction axis (" & $axis & ")")
  if t.size == 0: return newHipTensor[T](t.shape.toSeq)     # returnEmptyIfEmpty
  var oshape = t.shape.toSeq
  oshape[axis] = 1
  result = newHipTensor[T](oshape)
  var sh = i64s(t.shape)
  var sd = i64s(result.strides)
  var sa = i64s(t.strides)
  when T is float32: check am_hip_reduce_axis_f32(op, cint t.rank, sh[0].addr, cint axis, result.get_offset_ptr, sd[0].addr, t.get_offset_ptr, sa[0].addr)
  elif T is float64: check am_hip_reduce_axis_f64(op, cint t.rank, sh[0].addr, cint axis, result.get_offset_ptr, sd[0].addr, t.get_offset_ptr, sa[0].addr)
  elif T is int32: check am_hip_reduce_axis_i32(op, cint t.rank, sh[0].addr, cint axis, result.get_offset_ptr, sd[0].addr, t.get_offset_ptr, sa[0].addr)
  else: check am_hip_reduce_axis_i64(op, cint t.rank, sh[0].addr, cint axis, result.get_offset_ptr, sd[0].addr, t.get_offset_ptr, sa[0].addr)

proc argreduce[T: HipScalar](op: cint, t: HipTensor[T], axis: int): tuple[indices: HipTensor[int64], values: HipTensor[T]] =
  ## argmax_max / argmin_min (aggregate.nim:159-193, 216-250); the indices are the reference's Tensor[int].
  if axis < 0 or axis >= t.rank:
    raise newException(IndexDefect, "Input tensor rank (" & $t.rank & ") must be greater than reduction axis (" & $axis & ")")
  var oshape = t.shape.toSeq
  if t.size != 0: oshape[axis] = 1
  result.indices = newHipTensor[int64](oshape)
  result.values = newHipTensor[T](oshape)
  if t.size == 0: return
  var sh = i64s(t.shape)
  var si = i64s(result.indices.strides)
  var sv = i64s(result.values.strides)
  var sa = i64s(t.strides)
  when T is float32: check am_hip_argreduce_f32(op, cint t.rank, sh[0].addr, cint axis, result.indices.get_offset_ptr, si[0].addr, result.values.get_offset_ptr, sv[0].addr, t.get_offset_ptr, sa[0].addr)
  elif T is float64: check am_hip_argreduce_f64(op, cint t.rank, sh[0].addr, cint axis, result.indices.get_offset_ptr, si[0].addr, result.values.get_offset_ptr, sv[0].addr, t.get_offset_ptr, sa[0].addr)
  elif T is int32: check am_hip_argreduce_i32(op, cint t.rank, sh[0].addr, cint axis, result.indices.get_offset_ptr, si[0].addr, result.values.get_offset_ptr, sv[0].addr, t.get_offset_ptr, sa[0].addr)
  else: check am_hip_argreduce_i64(op, cint t.rank, sh[0].addr, cint axis, result.indices.get_offset_ptr, si[0].addr, result.values.get_offset_ptr, sv[0].addr, t.get_offset_ptr, sa[0].addr)

proc argmax_max*[T: HipScalar](t: HipTensor[T], axis: int): tuple[indices: HipTensor[int64], maxes: HipTensor[T]] =
  let r = argreduce(AM_RED_MAX, t, axis)
  (indices: r.indices, maxes: r.values)
proc argmax*[T: HipScalar](t: HipTensor[T], axis: int): HipTensor[int64] = argreduce(AM_RED_MAX, t, axis).indices   ## aggregate.nim:195-214
proc argmin_min*[T: HipScalar](t: HipTensor[T], axis: int): tuple[indices: HipTensor[int64], mins: HipTensor[T]] =
  let r = argreduce(AM_RED_MIN, t, axis)
  (indices: r.indices, mins: r.values)
proc argmin*[T: HipScalar](t: HipTensor[T], axis: int): HipTensor[int64] = argreduce(AM_RED_MIN, t, axis).indices   ## aggregate.nim:252-271

proc reduce_all[T: HipScalar](op: cint, t: HipTensor[T]): T =
  ## reduce_inline (higher_order_foldreduce.nim:22-31), value returned to the host.
  var sh = i64s(t.shape)
  var sa = i64s(t.strides)
  when T is float32: check am_hip_reduce_all_f32(op, cint t.rank, sh[0].addr, t.get_offset_ptr, sa[0].addr, result.addr)
  elif T is float64: check am_hip_reduce_all_f64(op, cint t.rank, sh[0].addr, t.get_offset_ptr, sa[0].addr, result.addr)
  elif T is int32: check am_hip_reduce_all_i32(op, cint t.rank, sh[0].addr, t.get_offset_ptr, sa[0].addr, result.addr)
  else: check am_hip_reduce_all_i64(op, cint t.rank, sh[0].addr, t.get_offset_ptr, sa[0].addr, result.addr)

# aggregate.nim:33-113
proc sum*[T: HipScalar](t: HipTensor[T]): T = reduce_all(AM_RED_SUM, t)
proc sum*[T: HipScalar](t: HipTensor[T], axis: int): HipTensor[T] = reduce_axis(AM_RED_SUM, t, axis)

proc linear_backward*[T: HipScalar](input, weight, gradOutput: HipTensor[T],
                                    gradInput, gradWeight, gradBias: var HipTensor[T]) =
  ## nnp_linear.nim:39-55; the transposed view reaches the GEMM as strides.
  gradInput = gradOutput * weight
  gradWeight = gradOutput.transpose * input
  gradBias = sum(gradOutput, axis = 0)

proc linear_backward*[T: HipScalar](input, weight, gradOutput: HipTensor[T],
                                    gradInput, gradWeight: var HipTensor[T]) =
  ## nnp_linear.nim:57-66
  gradInput = gradOutput * weight
  gradWeight = gradOutput.transpose * input
proc product*[T: HipScalar](t: HipTensor[T]): T = reduce_all(AM_RED_PROD, t)
proc product*[T: HipScalar](t: HipTensor[T], axis: int): HipTensor[T] = reduce_axis(AM_RED_PROD, t, axis)
proc min*[T: HipScalar](t: HipTensor[T]): T = reduce_all(AM_RED_MIN, t)
proc min*[T: HipScalar](t: HipTensor[T], axis: int): HipTensor[T] = reduce_axis(AM_RED_MIN, t, axis)
proc max*[T: HipScalar](t: HipTensor[T]): T = reduce_all(AM_RED_MAX, t)
proc max*[T: HipScalar](t: HipTensor[T], axis: int): HipTensor[T] = reduce_axis(AM_RED_MAX, t, axis)
proc mean*[T: int32 | int64](t: HipTensor[T]): T = t.sum div T(t.size)
proc mean*[T: float32 | float64](t: HipTensor[T]): T = t.sum / T(t.size)
proc mean*[T: int32 | int64](t: HipTensor[T], axis: int): HipTensor[T] = t.sum(axis) / T(t.shape[axis])   # opDiv truncates like `div` on integers
proc mean*[T: float32 | float64](t: HipTensor[T], axis: int): HipTensor[T] = t.sum(axis) / T(t.shape[axis])

proc sqrt*[T: float32 | float64](t: HipTensor[T]): HipTensor[T] =
  ## ufunc.nim:91
  result = newHipTensor[T](t.shape)
  if result.size > 0: ewUnary(T, uopSqrt, result, t)
proc square*[T: HipScalar](t: HipTensor[T]): HipTensor[T] =
  ## math_functions.nim:218-222
  result = newHipTensor[T](t.shape)
  if result.size > 0: ewUnary(T, uopSquare, result, t)

proc variance*[T: float32 | float64](t: HipTensor[T]): T =
  ## aggregate.nim:115-129: the mean, then the sum of square(y - mean), over n - 1
  square(t -. t.mean).sum / T(t.size - 1)
proc variance*[T: float32 | float64](t: HipTensor[T], axis: int): HipTensor[T] =
  ## aggregate.nim:131-146
  if t.size == 0: return t
  let m = t.mean(axis)
  map2(t, opSqDiff, m.broadcast(t.shape.toSeq)).sum(axis) / T(t.shape[axis] - 1)
proc std*[T: float32 | float64](t: HipTensor[T]): T = math.sqrt(t.variance)                        ## aggregate.nim:148-151
proc std*[T: float32 | float64](t: HipTensor[T], axis: int): HipTensor[T] =                   ## aggregate.nim:153-158
  if t.size == 0: return t
  sqrt(t.variance(axis))

proc softmax*[T: float32 | float64](input: HipTensor[T]): HipTensor[T] =
  ## nn_primitives/nnp_softmax.nim:18-38 on a [batch_size, number_of_classes] matrix.
  result = newHipTensor[T](input.shape.toSeq)
  when T is float32:
    check am_hip_softmax_rows_f32(int64 input.shape[0], int64 input.shape[1], result.get_offset_ptr, int64 result.strides[0], int64 result.strides[1],
      input.get_offset_ptr, int64 input.strides[0], int64 input.strides[1])
  else:
    check am_hip_softmax_rows_f64(int64 input.shape[0], int64 input.shape[1], result.get_offset_ptr, int64 result.strides[0], int64 result.strides[1],
      input.get_offset_ptr, int64 input.strides[0], int64 input.strides[1])

proc softmax_cross_entropy*[T: float32 | float64](input, target: HipTensor[T]): T =
  ## nn_primitives/nnp_softmax_cross_entropy.nim:17-86: softmax and cross-entropy in one pass, averaged over the batch.
  assert input.rank == 2 and input.shape == target.shape
  template call(f: untyped) =
    check f(int64 input.shape[0], int64 input.shape[1], input.get_offset_ptr, int64 input.strides[0], int64 input.strides[1],
            target.get_offset_ptr, int64 target.strides[0], int64 target.strides[1], result.addr)
  when T is float32: call am_hip_softmax_cross_entropy_f32
  else: call am_hip_softmax_cross_entropy_f64

proc sparse_softmax_cross_entropy*[T: float32 | float64](input: HipTensor[T], target: HipTensor[int64]): T =
  ## nnp_softmax_cross_entropy.nim:88-177: one class index per row.
  assert input.rank == 2 and target.rank == 1 and target.shape[0] == input.shape[0]
  template call(f: untyped) =
    check f(int64 input.shape[0], int64 input.shape[1], input.get_offset_ptr, int64 input.strides[0], int64 input.strides[1],
            target.get_offset_ptr, int64 target.strides[0], result.addr)
  when T is float32: call am_hip_sparse_softmax_cross_entropy_f32
  else: call am_hip_sparse_softmax_cross_entropy_f64

proc softmax_cross_entropy_backward*[T: float32 | float64](gradient: T, cached_tensor, target: HipTensor[T]): HipTensor[T] =
  ## nnp_softmax_cross_entropy.nim:186-214: gradient * (softmax(cached_tensor) - target) / batch_size, one launch.
  assert cached_tensor.rank == 2 and cached_tensor.shape == target.shape
  result = newHipTensor[T](cached_tensor.shape)
  template call(f: untyped) =
    check f(int64 cached_tensor.shape[0], int64 cached_tensor.shape[1], gradient, cached_tensor.get_offset_ptr,
            int64 cached_tensor.strides[0], int64 cached_tensor.strides[1], target.get_offset_ptr, int64 target.strides[0],
            int64 target.strides[1], result.get_offset_ptr, int64 result.strides[0], int64 result.strides[1])
  when T is float32: call am_hip_softmax_cross_entropy_backward_f32
  else: call am_hip_softmax_cross_entropy_backward_f64

proc sparse_softmax_cross_entropy_backward*[T: float32 | float64](gradient: T, cached_tensor: HipTensor[T],
                                                                  target: HipTensor[int64]): HipTensor[T] =
  ## nnp_softmax_cross_entropy.nim:217-256: gradient * (softmax(cached_tensor) - onehot(target)) / batch_size, one launch.
  assert cached_tensor.rank == 2 and target.rank == 1 and target.shape[0] == cached_tensor.shape[0]
  result = newHipTensor[T](cached_tensor.shape)
  template call(f: untyped) =
    check f(int64 cached_tensor.shape[0], int64 cached_tensor.shape[1], gradient, cached_tensor.get_offset_ptr,
            int64 cached_tensor.strides[0], int64 cached_tensor.strides[1], target.get_offset_ptr, int64 target.strides[0],
            result.get_offset_ptr, int64 result.strides[0], int64 result.strides[1])
  when T is float32: call am_hip_sparse_softmax_cross_entropy_backward_f32
  else: call am_hip_sparse_softmax_cross_entropy_backward_f64

proc sigmoid_cross_entropy*[T: float32 | float64](input, target: HipTensor[T]): T =
  ## nn_primitives/nnp_sigmoid_cross_entropy.nim:23-45: the map2 body and its sum in one pass, averaged over the batch.
  assert input.rank == 2 and input.shape == target.shape
  template call(f: untyped) =
    check f(int64 input.shape[0], int64 input.shape[1], input.get_offset_ptr, int64 input.strides[0], int64 input.strides[1],
            target.get_offset_ptr, int64 target.strides[0], int64 target.strides[1], result.addr)
  when T is float32: call am_hip_sigmoid_cross_entropy_f32
  else: call am_hip_sigmoid_cross_entropy_f64

proc sigmoid_cross_entropy_backward*[T: float32 | float64](gradient: T, cached_tensor, target: HipTensor[T]): HipTensor[T] =
  ## nnp_sigmoid_cross_entropy.nim:47-62: gradient * (sigmoid(cached_tensor) - target) / batch_size.
  assert cached_tensor.rank == 2 and cached_tensor.shape == target.shape
  result = newHipTensor[T](cached_tensor.shape)
  template call(f: untyped) =
    check f(int64 cached_tensor.shape[0], int64 cached_tensor.shape[1], gradient, cached_tensor.get_offset_ptr,
            int64 cached_tensor.strides[0], int64 cached_tensor.strides[1], target.get_offset_ptr, int64 target.strides[0],
            int64 target.strides[1], result.get_offset_ptr, int64 result.strides[0], int64 result.strides[1])
  when T is float32: call am_hip_sigmoid_cross_entropy_backward_f32
  else: call am_hip_sigmoid_cross_entropy_backward_f64

proc sgd_update*[T: float32 | float64](values: var openArray[HipTensor[T]], gradients: openArray[HipTensor[T]], learning_rate: T) =
  ## nn/optimizers/optimizers.nim:35-51 (one apply2_inline per parameter: x - lr * y) for every parameter in ONE launch.
  assert values.len == gradients.len
  var v, g = newSeq[ptr T](values.len)
  var n = newSeq[int64](values.len)
  for i in 0 ..< values.len:
    assert values[i].shape == gradients[i].shape and values[i].is_C_contiguous and gradients[i].is_C_contiguous
    v[i] = values[i].get_offset_ptr; g[i] = gradients[i].get_offset_ptr; n[i] = int64 values[i].size
  if values.len > 0:
    when T is float32: check am_hip_sgd_update_f32(cint values.len, v[0].addr, g[0].addr, n[0].addr, learning_rate)
    else: check am_hip_sgd_update_f64(cint values.len, v[0].addr, g[0].addr, n[0].addr, learning_rate)

proc conv2d*[T: SomeFloat](input, kernel, bias: HipTensor[T], padding = (0, 0), stride = (1, 1), relu = false): HipTensor[T] =
  ## im2colgemm_conv2d (nn_primitives/fallback/conv.nim:81-106), optionally followed by relu, in one launch: the GEMM's
  ## B loader gathers the column matrix from the images. input [N, C, H, W], kernel [C_out, C, kH, kW] (C-contiguous),
  ## bias [C_out, 1, 1].
  assert input.rank == 4 and kernel.rank == 4 and kernel.shape[1] == input.shape[1]
  let kc = if kernel.is_C_contiguous: kernel else: kernel.clone()
  let (N, C, H, W) = (input.shape[0], input.shape[1], input.shape[2], input.shape[3])
  let (co, kH, kW) = (kernel.shape[0], kernel.shape[2], kernel.shape[3])
  let outH = (H + 2 * padding[0] - kH) div stride[0] + 1
  let outW = (W + 2 * padding[1] - kW) div stride[1] + 1
  result = newHipTensor[T]([N, co, outH, outW])
  let epilogue = cint(if relu: AM_EPI_BIAS_RELU else: AM_EPI_BIAS)
  template call(f: untyped) =
    check f(int64 N, cint C, cint H, cint W, cint co, cint kH, cint kW, cint padding[0], cint padding[1], cint stride[0], cint stride[1],
            input.get_offset_ptr, int64 input.strides[0], int64 input.strides[1], int64 input.strides[2], int64 input.strides[3],
            kc.get_offset_ptr, int64(C * kH * kW), epilogue, bias.get_offset_ptr, int64 bias.strides[0], result.get_offset_ptr)
  when T is float32: call am_hip_conv2d_f32
  else: call am_hip_conv2d_f64

proc conv2d_backward*[T: HipScalar](input, weight, bias: HipTensor[T], padding, stride: tuple[height, width: int],
                                    grad_output: HipTensor[T], grad_input, grad_weight, grad_bias: var HipTensor[T]) =
  ## conv2d_backward (nn_primitives/nnp_convolution.nim:65-107) over im2colgemm_conv2d_gradient
  ## (fallback/conv.nim:107-145). The reference loops over the images; here the batch is folded into the columns:
  ## g [C_out, N*P] is grad_output with its first two axes swapped, col [C*kH*kW, N*P] the column matrices side by
  ## side, and the pass is grad_bias = row sums of g, grad_weight = g * col^T, grad_input = col2im(kernel_col^T * g).
  assert input.rank == 4 and weight.rank == 4 and weight.shape[1] == input.shape[1]
  assert bias.rank == 3 or bias.rank == 0
  let (N, C, H, W) = (input.shape[0], input.shape[1], input.shape[2], input.shape[3])
  let (co, kH, kW) = (weight.shape[0], weight.shape[2], weight.shape[3])
  let outH = (H + 2 * padding.height - kH) div stride.height + 1
  let outW = (W + 2 * padding.width - kW) div stride.width + 1
  let P = outH * outW
  assert grad_output.shape[0] == N and grad_output.shape[1] == co and grad_output.shape[2] == outH and grad_output.shape[3] == outW
  let go = if grad_output.is_C_contiguous: grad_output else: grad_output.clone()
  # g[co, n, p] = grad_output[n, co, p]: a strided view of the same memory, packed by one copy pass
  var gview: HipTensor[T]
  gview.shape.copyFrom([co, N, P]); gview.strides.copyFrom([P, co * P, 1])
  gview.offset = go.offset; gview.storage = go.storage
  var g = gview.clone()
  g.shape.copyFrom([co, N * P]); g.strides.copyFrom([N * P, 1])
  if bias.rank > 0:
    grad_bias = sum(g, axis = 1)
    grad_bias.shape.copyFrom([co, 1, 1]); grad_bias.strides.copyFrom([1, 1, 1])
  let wc = if weight.is_C_contiguous: weight else: weight.clone()
  var kcol = wc
  kcol.shape.copyFrom([co, C * kH * kW]); kcol.strides.copyFrom([C * kH * kW, 1])
  # one launch where the library's loader can gather col^T from the images in 16-byte pieces: col is never written
  var gathered = false
  when T is float32 or T is float64:
    const vk = 16 div sizeof(T)
    if stride.width == 1 and input.strides[3] == 1 and outW mod vk == 0 and W >= vk and N >= 1 and P >= 1 and
       N * P < (1 shl 31) and C * kH * kW * kH * kW < (1 shl 32) and co * C * kH * kW < 1_000_000:   # (larger gradients: the plain product's larger tiles win)
      grad_weight = newHipTensor[T]([co, C, kH, kW])
      template gather(f: untyped) =
        check f(int64 N, cint C, cint H, cint W, cint co, cint kH, cint kW, cint padding.height, cint padding.width,
                cint stride.height, cint stride.width, input.get_offset_ptr, int64 input.strides[0], int64 input.strides[1],
                int64 input.strides[2], int64 input.strides[3], g.get_offset_ptr, int64 g.strides[0], grad_weight.get_offset_ptr)
      when T is float32: gather am_hip_conv2d_grad_weight_f32
      else: gather am_hip_conv2d_grad_weight_f64
      gathered = true
  if not gathered:
    var col = newHipTensor[T]([C * kH * kW, N * P])
    template unroll(f: untyped) =
      check f(int64 N, cint C, cint H, cint W, cint kH, cint kW, cint padding.height, cint padding.width, cint stride.height, cint stride.width,
              input.get_offset_ptr, int64 input.strides[0], int64 input.strides[1], int64 input.strides[2], int64 input.strides[3],
              col.get_offset_ptr, int64 P, int64(N * P))
    when T is float32: unroll am_hip_im2col_strided_f32
    elif T is float64: unroll am_hip_im2col_strided_f64
    elif T is int32: unroll am_hip_im2col_strided_i32
    else: unroll am_hip_im2col_strided_i64
    grad_weight = g * col.transpose
    grad_weight.shape.copyFrom([co, C, kH, kW]); grad_weight.strides.copyFrom([C * kH * kW, kH * kW, kW, 1])
  let gcol = kcol.transpose * g
  grad_input = newHipTensor[T]([N, C, H, W])
  template fold(f: untyped) =
    check f(int64 N, cint C, cint H, cint W, cint kH, cint kW, cint padding.height, cint padding.width, cint stride.height, cint stride.width,
            gcol.get_offset_ptr, int64 P, int64(N * P), grad_input.get_offset_ptr,
            int64 grad_input.strides[0], int64 grad_input.strides[1], int64 grad_input.strides[2], int64 grad_input.strides[3])
  when T is float32: fold am_hip_col2im_f32
  elif T is float64: fold am_hip_col2im_f64
  elif T is int32: fold am_hip_col2im_i32
  else: fold am_hip_col2im_i64

proc maxpool2d*[T: HipScalar](input: HipTensor[T], kernel: tuple[height, width: int], padding = (0, 0), stride = (1, 1)):
    tuple[max_indices: HipTensor[int64], maxpooled: HipTensor[T]] =
  ## nn_primitives/nnp_maxpooling.nim:19-66 (the reference asserts a C-contiguous rank-4 input too).
  assert input.rank == 4 and input.is_C_contiguous
  let (N, C, H, W) = (input.shape[0], input.shape[1], input.shape[2], input.shape[3])
  let outH = (H + 2 * padding[0] - kernel.height) div stride[0] + 1
  let outW = (W + 2 * padding[1] - kernel.width) div stride[1] + 1
  result.max_indices = newHipTensor[int64]([N * C * outH * outW])
  result.maxpooled = newHipTensor[T]([N, C, outH, outW])
  template call(f: untyped) =
    check f(int64 N, cint C, cint H, cint W, cint kernel.height, cint kernel.width, cint padding[0], cint padding[1],
            cint stride[0], cint stride[1], input.get_offset_ptr, result.maxpooled.get_offset_ptr, result.max_indices.get_offset_ptr)
  when T is float32: call am_hip_maxpool2d_f32
  elif T is float64: call am_hip_maxpool2d_f64
  elif T is int32: call am_hip_maxpool2d_i32
  else: call am_hip_maxpool2d_i64

proc maxpool2d_backward*[T: HipScalar](cached_input_shape: openArray[int], cached_max_indices: HipTensor[int64],
                                       gradOutput: HipTensor[T], kernel: tuple[height, width: int],
                                       padding = (0, 0), stride = (1, 1)): HipTensor[T] =
  ## nn_primitives/nnp_maxpooling.nim:68-83. The device runs the scatter as a gather over the pooling
  ## windows, so kernel, padding and stride of the forward pass are passed again.
  assert cached_input_shape.len == 4 and gradOutput.size == cached_max_indices.size
  assert gradOutput.is_C_contiguous and cached_max_indices.is_C_contiguous
  let (N, C, H, W) = (cached_input_shape[0], cached_input_shape[1], cached_input_shape[2], cached_input_shape[3])
  result = newHipTensor[T]([N, C, H, W])
  template call(f: untyped) =
    check f(int64 N, cint C, cint H, cint W, cint kernel.height, cint kernel.width, cint padding[0], cint padding[1],
            cint stride[0], cint stride[1], cached_max_indices.get_offset_ptr, gradOutput.get_offset_ptr, result.get_offset_ptr)
  when T is float32: call am_hip_maxpool2d_backward_f32
  elif T is float64: call am_hip_maxpool2d_backward_f64
  elif T is int32: call am_hip_maxpool2d_backward_i32
  else: call am_hip_maxpool2d_backward_i64

# ---------------------------------------------------------------- HIP graphs
type HipGraph* = object
  ## A recorded sequence of device operations, replayed with one launch (no counterpart in the reference).
  exec: pointer

proc `=destroy`*(g: HipGraph) =
  if not g.exec.isNil: discard am_hip_graph_destroy(g.exec)

proc `=copy`*(dst: var HipGraph, src: HipGraph) {.error: "a HipGraph owns its executable graph".}

template recordGraph*(body: untyped): HipGraph =
  ## Runs `body` twice: once as a rehearsal with the allocator holding back every block that is freed (its cache then
  ## has one block per allocation of `body`, the library workspace its final size), then under capture, where
  ## allocation is served from that cache. `body` must only issue device work on tensors that outlive the graph.
  block:
    var g: HipGraph
    check am_hip_alloc_hold(1)
    try:
      body
    finally:
      check am_hip_alloc_hold(0)
    check am_hip_graph_begin()
    try:
      body
    finally:
      check am_hip_graph_end(g.exec.addr)
    g

proc launch*(g: HipGraph) = check am_hip_graph_launch(g.exec)

# ---------------------------------------------------------------- unsigned element types
# The reference's GEMM takes uint32 | uint64 | uint | int by casting the pointers onto its int32 / int64 kernels
# (laser/primitives/matrix_multiplication/gemm.nim:275-307). In the rings Z/2^32 and Z/2^64 the bits of + - * (hence of
# matrix products, dot, sums and products of elements) do not depend on how the operands are read, so those run on
# the signed kernels here too. Whatever reads the sign (div, mod, comparisons, min / max, clamp, sgn) has no overload
# for these types and does not compile.
template signedTwin(T: typedesc): typedesc =
  when sizeof(T) == 4: int32 else: int64

proc signedView[T: HipUnsigned](t: HipTensor[T]): HipTensor[signedTwin(T)] =
  ## The same device memory read as the signed twin. Non-owning (no ref tracker): valid while `t` is alive, i.e.
  ## inside the proc that made it.
  result.shape = t.shape
  result.strides = t.strides
  result.offset = t.offset
  result.storage.Flen = t.storage.Flen
  result.storage.Fdata = cast[ptr UncheckedArray[signedTwin(T)]](t.storage.Fdata)

proc gemm*[T: HipUnsigned](alpha: T, A, B: HipTensor[T], beta: T, C: var HipTensor[T]) =
  var c = C.signedView
  gemm(cast[signedTwin(T)](alpha), A.signedView, B.signedView, cast[signedTwin(T)](beta), c)

proc gemv*[T: HipUnsigned](alpha: T, A, x: HipTensor[T], beta: T, y: var HipTensor[T]) =
  var v = y.signedView
  gemv(cast[signedTwin(T)](alpha), A.signedView, x.signedView, cast[signedTwin(T)](beta), v)

proc dot*[T: HipUnsigned](a, b: HipTensor[T]): T = cast[T](dot(a.signedView, b.signedView))

proc `*`*[T: HipUnsigned](a, b: HipTensor[T]): HipTensor[T] =
  if a.rank == 2 and b.rank == 2:
    result = newHipTensor[T]([a.shape[0], b.shape[1]])
    gemm(T(1), a, b, T(0), result)
  elif a.rank == 2 and b.rank == 1:
    result = newHipTensor[T]([a.shape[0]])
    gemv(T(1), a, b, T(0), result)
  else:
    raise newException(ValueError, "Matrix-Matrix or Matrix-Vector multiplication valid only if first Tensor is a Matrix and second is a Matrix or Vector")

proc ringMap2[T: HipUnsigned](a: HipTensor[T], op: AmBinaryOp, b: HipTensor[T]): HipTensor[T] =
  check_elementwise(a, b)
  result = newHipTensor[T](a.shape)
  if result.size > 0:
    var r = result.signedView
    apply2Into(r, a.signedView, op, b.signedView)

proc `+`*[T: HipUnsigned](a, b: HipTensor[T]): HipTensor[T] = ringMap2(a, opAdd, b)
proc `-`*[T: HipUnsigned](a, b: HipTensor[T]): HipTensor[T] = ringMap2(a, opSub, b)
proc `+.`*[T: HipUnsigned](a, b: HipTensor[T]): HipTensor[T] =
  let (x, y) = broadcast2(a, b)
  ringMap2(x, opAdd, y)
proc `-.`*[T: HipUnsigned](a, b: HipTensor[T]): HipTensor[T] =
  let (x, y) = broadcast2(a, b)
  ringMap2(x, opSub, y)
proc `*.`*[T: HipUnsigned](a, b: HipTensor[T]): HipTensor[T] =
  let (x, y) = broadcast2(a, b)
  ringMap2(x, opMul, y)
proc `*`*[T: HipUnsigned](s: T, t: HipTensor[T]): HipTensor[T] =
  result = newHipTensor[T](t.shape)
  if result.size > 0:
    var r = result.signedView
    let tv = t.signedView
    ewScalar(signedTwin(T), opMul, true, r, tv, cast[signedTwin(T)](s))
proc `*`*[T: HipUnsigned](t: HipTensor[T], s: T): HipTensor[T] = s * t
proc sum*[T: HipUnsigned](t: HipTensor[T]): T = cast[T](sum(t.signedView))
proc product*[T: HipUnsigned](t: HipTensor[T]): T = cast[T](product(t.signedView))
proc clone*[T: HipUnsigned](t: HipTensor[T]): HipTensor[T] =
  result = newHipTensor[T](t.shape)
  if result.size > 0:
    var r = result.signedView
    let tv = t.signedView
    ewUnary(signedTwin(T), uopCopy, r, tv)

# ---------------------------------------------------------------- .npy files and display
# The file parsing and the pretty printer are the reference's own host code (io/io_npy.nim:64-183,
# tensor/private/p_display.nim); the device tensor goes through a host copy, exactly as
# display_cuda.nim:19-36 does for CudaTensor.
proc read_npy_hip*[T: HipScalar](npyPath: string): HipTensor[T] =
  read_npy[T](npyPath).toHip

proc write_npy*[T: HipScalar](t: HipTensor[T], npyPath: string) =
  t.toCpu.write_npy(npyPath)

proc pretty*[T](t: HipTensor[T], precision = -1): string =
  var desc = t.type.name & " of shape \"" & $t.shape & "\" on backend \"" & "Hip" & "\""
  if t.storage.isNil: return "Uninitialized " & $desc
  let cpu_t = t.toCpu
  if cpu_t.size() == 0: return desc & "\n    [] (empty)"
  elif cpu_t.rank == 1: return desc & "\n    " & cpu_t.prettyImpl(precision = precision)
  else: return desc & "\n" & cpu_t.prettyImpl(precision = precision)

proc `$`*[T](t: HipTensor[T]): string = t.pretty()

