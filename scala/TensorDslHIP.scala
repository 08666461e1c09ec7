// BackendHIP: Lantern's operator trait on liblantern_hip (MI355X).  Reference-side source, to be dropped into
// src/main/scala/lantern/ of the Lantern tree next to TensorDslCublas.scala / TensorDslCudnn.scala.
//
// NOT COMPILED in this repository: the Lantern tree needs a JVM, sbt and its un-vendored LMS snapshot.  It is kept a thin
// one-to-one mapping so that it can be checked by reading: every trait method of `Backend`
// (TensorDifferentiation.scala:137-379) is overridden below, keeps the staging-time checks of the cuBLAS/cuDNN backend it
// replaces (cited per method as CUB:line = TensorDslCublas.scala, CDN:line = TensorDslCudnn.scala) and emits its library
// calls through ONE helper, `hip("lh_name", args...)`, so that names and argument counts can be compared mechanically
// with include/lantern_hip.h.
//
// What the generated program looks like: plain host C++ (no kernels, no cuBLAS/cuDNN handles, no descriptors):
//     #include "lantern_hip.h"
//     void Snippet(char* a) { lh_setup(HEAP_SIZE_HIP); ... lh_conv2d_fwd(x3, x7, (float*)0, x9, 64, 3, 224, ...); ... lh_cleanup(); }
package lantern

import scala.util.continuations._
import scala.virtualization.lms._
import scala.virtualization.lms.common._

// ---- code generation for the GPU array nodes (replaces CudaGenGPUOps, common/GPUOps.scala:60-102) ----------------------
trait HipGenGPUOps extends CGenBase {
  val IR: GPUOpsExp
  import IR._

  override def emitNode(sym: Sym[Any], rhs: Def[Any]) = rhs match {
    case a@GPUArrayNew(n) =>                                    // arena memory reads zero, as Tensor.zeros expects (TD:1075-1076); large blocks are cleared only if something reads them before writing
      val dataType = remap(a.m)
      emitValDef(sym, "(" + dataType + "*)lh_malloc((size_t)" + quote(n) + " * sizeof(" + dataType + "))")
    case a@GPUArrayFromSeq(xs) =>
      val dataType = remap(a.m)
      stream.println(dataType + " " + quote(sym) + "_host[] = {" + xs.map(quote).mkString(", ") + "};")
      emitValDef(sym, "(" + dataType + "*)lh_malloc_uninit(" + xs.length + " * sizeof(" + dataType + "))")
      stream.println("lh_h2d(" + quote(sym) + ", " + quote(sym) + "_host, " + xs.length + " * sizeof(" + dataType + "));")
    case a@GPUArrayCopy(src, dest, len, direction) =>
      val bytes = "(size_t)" + quote(len) + " * sizeof(" + remap(a.m) + ")"
      val call = direction match {
        case CopyDirection.HostToDevice => "lh_h2d"
        case CopyDirection.DeviceToHost => "lh_d2h"
        case CopyDirection.DeviceToDevice => "lh_d2d"
      }
      stream.println(call + "(" + quote(dest) + ", " + quote(src) + ", " + bytes + ");")
    case _ => super.emitNode(sym, rhs)
  }
}

// ---- file prelude (replaces DslGenCublas / DslGenCudnn, DslAPI.scala:433-881, 884-900) -----------------------------------
// No kernel source text and no error macros: the kernels live in the library, which prints file:line and exits on error
// exactly as CUDA_CALL does (DslAPI.scala:435-451).
trait DslGenHIP extends DslGenBase with HipGenGPUOps {
  val IR: DslExp
  override def templateHeaders: Seq[String] = super.templateHeaders ++ Seq("\"lantern_hip.h\"")
  override def templateRawCode: String = super.templateRawCode +
    """
      |// device arena: the reference's 8 GiB constant (DslAPI.scala:385) is a parameter of lh_setup here
      |#ifndef HEAP_SIZE_HIP
      |#define HEAP_SIZE_HIP ((size_t)16 << 30)
      |#endif
      |enum { LH_HOST_TRUE = 1, LH_HOST_FALSE = 0 };
    """.stripMargin
}

abstract class DslDriverHIP[A: Manifest, B: Manifest] extends DslDriverBase[A, B] with DslGPUExp { self =>
  override val codegen = new DslGenHIP { val IR: self.type = self }
  // The emitted file is host code only, so any C++ compiler does: hipcc is not needed.
  def compilerArguments: Seq[String] = Seq("-std=c++11", "-O1", "-I", sys.env.getOrElse("LANTERN_HIP_INCLUDE", "include"),
                                           "-L", sys.env.getOrElse("LANTERN_HIP_LIB", "lantern_amd/csrc"), "-llantern_hip", "-lstdc++")
  override def eval(a: A) {
    val cppFileName = "/tmp/lantern-snippet-hip.cpp"
    val binaryFileName = "/tmp/lantern-snippet-hip"
    val out = new java.io.PrintWriter(cppFileName)
    out.println(code)
    out.close()
    new java.io.File(binaryFileName).delete
    import scala.sys.process._
    System.out.println("Compile C++ (HIP backend) code")
    (s"g++ $cppFileName -o $binaryFileName ${compilerArguments.mkString(" ")}": ProcessBuilder).lines.foreach(System.out.println)
    System.out.println("Run C++ (HIP backend) code")
    (s"$binaryFileName $a": ProcessBuilder).lines.foreach(System.out.println)
  }
}

trait TensorDslHIP extends TensorDslCPU with GPUOps {

  // ---- arena mark / rewind (CUB:18-25: getCudaMallocAddr / resetCudaMallocAddr = memset of the used span + reset) ----------
  def getHipMallocAddr(): Rep[Long] = unchecked[Long]("(long)lh_mark()")
  def resetHipMallocAddr(addr: Rep[Long]) = hip("lh_rewind", cast("size_t", addr))
  // the applications call the CUDA-named pair; both names work
  def getCudaMallocAddr(): Rep[Long] = getHipMallocAddr()
  def resetCudaMallocAddr(addr: Rep[Long]) = resetHipMallocAddr(addr)

  // ---- the one way a library call is emitted: name(arg, arg, ...) ------------------------------------------------------
  case class CText(text: Seq[Any])                       // a C expression assembled from literals and staged values
  def cast(ty: String, v: Any): CText = CText(Seq("(" + ty + ")", v))
  def cfloat(v: Float): CText = CText(Seq(v.toString + "f"))
  def nullFloats: CText = CText(Seq("(float*)0"))
  def nullInts: CText = CText(Seq("(int*)0"))
  def hip(name: String, args: Any*): Rep[Unit] = {
    val pieces = scala.collection.mutable.ArrayBuffer[Any](name + "(")
    args.zipWithIndex.foreach { case (a, i) =>
      if (i > 0) pieces += ", "
      a match {
        case CText(t) => pieces ++= t
        case f: Float => pieces += (f.toString + "f")
        case b: Boolean => pieces += (if (b) "1" else "0")
        case other => pieces += other
      }
    }
    pieces += ")"
    unchecked[Unit](pieces: _*)
  }
  // shape and permutation arguments are host int arrays that the library reads during the call
  def hostInts(vals: Seq[Rep[Int]]): Rep[Array[Int]] = {
    val a = NewArray[Int](vals.length max 1)
    vals.zipWithIndex.foreach { case (v, i) => a(i) = v }
    a
  }
  def hostPointers(ptrs: Seq[Rep[Array[Float]]]): Rep[Array[Array[Float]]] = {
    val a = NewArray[Array[Float]](ptrs.length max 1)
    ptrs.zipWithIndex.foreach { case (p, i) => a(i) = p }
    a
  }

  // operator codes of include/lantern_hip.h
  val (lhAdd, lhSub, lhMul, lhDiv) = ("LH_ADD", "LH_SUB", "LH_MUL", "LH_DIV")
  val (lhRelu, lhTanh, lhSigmoid, lhExp, lhLog, lhSqrt, lhSquare, lhHardTanh) =
    ("LH_RELU", "LH_TANH", "LH_SIGMOID", "LH_EXP", "LH_LOG", "LH_SQRT", "LH_SQUARE", "LH_HARDTANH")

  // ---- transfers (CUB:37-107, unchanged in shape: the copy nodes now emit lh_h2d / lh_d2h / lh_d2d) --------------------------
  class ArrayTransferOps[T: Manifest](array: Rep[Array[T]]) {
    def toCPU(length: Rep[Int]): Rep[Array[T]] = { val res = BackendCPU().mallocArray[T](length); gpu_array_copy_device_to_host(array, res, length); res }
    def toGPU(length: Rep[Int]): Rep[Array[T]] = { val res = BackendGPU.mallocArray[T](length); gpu_array_copy_host_to_device(array, res, length); res }
    def moveToCPU(length: Rep[Int]): Unit = { val res = BackendCPU().mallocArray[T](length); gpu_array_copy_device_to_host(array, res, length); unchecked[Unit](array, " = ", res) }
    def moveToGPU(length: Rep[Int]): Unit = { val res = BackendGPU.mallocArray[T](length); gpu_array_copy_host_to_device(array, res, length); unchecked[Unit](array, " = ", res) }
  }
  implicit def arrayToTransferOps[T: Manifest](array: Rep[Array[T]]) = new ArrayTransferOps(array)
  class TensorTransferOps(t: Tensor) {
    def toCPU(): Tensor = { generateRawComment("Tensor 'toCPU' invocation."); new Tensor(t.data.toCPU(t.scalarCount), t.shape) }
    def toGPU(): Tensor = { generateRawComment("Tensor 'toGPU' invocation."); new Tensor(t.data.toGPU(t.scalarCount), t.shape) }
    def moveToCPU(): Unit = { generateRawComment("Tensor 'moveToCPU' invocation."); t.data.moveToCPU(t.scalarCount) }
    def moveToGPU(): Unit = { generateRawComment("Tensor 'moveToGPU' invocation."); t.data.moveToGPU(t.scalarCount) }
  }
  implicit def tensorToTransferOps(t: Tensor) = new TensorTransferOps(t)
  class TensorRTransferOps(t: TensorR) {
    def toCPU(): TensorR = new TensorR(t.x.toCPU(), t.d.toCPU())
    def toGPU(): TensorR = { val temp = new TensorR(t.x.toGPU(), t.d.toGPU()); temp.isInput = t.isInput; temp }
    def moveToCPU(): Unit = { t.x.moveToCPU(); t.d.moveToCPU() }
    def moveToGPU(): Unit = { t.x.moveToGPU(); t.d.moveToGPU() }
  }
  implicit def tensorRToTransferOps(t: TensorR) = new TensorRTransferOps(t)

  // cuDNN's mode objects, kept so that NNModule's RNNBase compiles unchanged (CDN:112-131)
  sealed trait RnnMode { def id: Int; def numGates: Int }
  case object RnnReluMode extends RnnMode { val id = 0; val numGates = 1 }
  case object RnnTanhMode extends RnnMode { val id = 1; val numGates = 1 }
  case object LstmMode extends RnnMode { val id = 2; val numGates = 4 }
  case object GruMode extends RnnMode { val id = 3; val numGates = 3 }

  class BackendHIP protected() extends Backend {
    // ---- lifetime (CUB:113-126; CDN:143-151) ---------------------------------------------------------------------------
    override def setup(): Unit = hip("lh_setup", CText(Seq("HEAP_SIZE_HIP")))
    // launch-bound programs (TreeLSTM): follow with hip("lh_cmdlist_begin"); small operator calls are then recorded and run
    // from the library's command list, in program order with everything else; nothing else in the generated code changes
    override def cleanup(): Unit = hip("lh_cleanup")
    override def mallocArray[T: Manifest](length: Rep[Int]): Rep[Array[T]] = NewGPUArray[T](length)            // CUB:126
    override def copyFloatArray(dest: Rep[Array[Float]], src: Rep[Array[Float]], length: Rep[Int]): Unit =
      gpu_array_copy_device_to_device(src, dest, length)                                                          // CUB:128-129
    // TD:154-158 (concrete in the trait; restated so the size check sits beside the device copy it guards)
    override def copyTensorData(dest: Tensor, src: Tensor): Unit = {
      assertC(dest.scalarCount == src.scalarCount, "Tensors do not have same scalar count: %d, %d", dest.scalarCount, src.scalarCount)
      copyFloatArray(dest.data, src.data, dest.scalarCount)
    }
    override def arrayToTensor(array: Rep[Array[Float]], dims: Rep[Int]*): Tensor = new Tensor(array, dims)       // CUB:131
    override def makeTensor(dims: Seq[Rep[Int]], scalars: Float*): Tensor = BackendCPU().makeTensor(dims, scalars: _*).toGPU()   // CUB:133-134

    // ---- fills (CUB:136-161) ----------------------------------------------------------------------------------------------
    override def fill(dims: Seq[Rep[Int]], value: Rep[Float]): Tensor = {
      val size: Rep[Int] = dims.foldLeft(unit(1)) { case (a, b) => a * b }
      val res = Tensor(mallocArray[Float](size), dims: _*)
      hip("lh_fill", res.data, value, cast("int64_t", size))
      res
    }
    override def fillWithBias(dims: Seq[Rep[Int]], bias: Tensor, dim: Int): Tensor = {
      assert(dim >= 0 && dim < dims.size, s"Target dimension $dim is out of range $dims")
      assert(bias.rank == 1, s"Bias should be 1D, got ${bias.shape}")
      val outer: Rep[Int] = dims.take(dim).foldLeft(unit(1)) { case (a, b) => a * b }
      val inner: Rep[Int] = dims.drop(dim + 1).foldLeft(unit(1)) { case (a, b) => a * b }
      val res = Tensor(mallocArray[Float](outer * dims(dim) * inner), dims: _*)
      hip("lh_fill_with_bias", res.data, bias.data, cast("int64_t", outer), cast("int64_t", dims(dim)), cast("int64_t", inner))
      res
    }
    override def fillInPlace(x: Tensor, value: Rep[Float]): Unit = hip("lh_fill", x.data, value, cast("int64_t", x.scalarCount))
    override def randinit(dims: Seq[Int], scale: Float = 1.0f, seed: Option[Int] = None): Tensor =
      BackendCPU().randinit(dims, scale, seed).toGPU()                                                            // host rand(), then H2D (CUB:154-155)
    override def clipAt(x: Tensor, bound: Float) = hip("lh_clip", x.data, bound, cast("int64_t", x.scalarCount))   // CUB:157-161

    // host lambdas cannot run on the device: `???` in the reference's GPU backends too (CUB:164-168)
    override def mutate(x: Tensor, delta: Rep[Int] => Rep[Float]): Unit = ???
    override def mapInPlace(x: Tensor, op: Rep[Float] => Rep[Float]): Unit = ???
    override def changeTo(x: Tensor, gen: Rep[Int] => Rep[Float]): Unit = ???
    override def map(x: Tensor, op: Rep[Float] => Rep[Float]): Tensor = ???
    override def fold(init: Rep[Float])(x: Tensor, op: (Rep[Float], Rep[Float]) => Rep[Float]): Rep[Float] = ???

    // ---- dot family (CUB:173-282).  Row-major entry points: no operand swapping as with column-major cuBLAS ------------------
    override def vectorVectorDot(x: Tensor, y: Tensor): Tensor = {
      val res = mallocArray[Float](1)                                                  // the result stays on the device (CUB:181-184 goes through the host)
      hip("lh_dot_vv", x.data, y.data, res, x.scalarCount)
      Tensor(res, 1)
    }
    override def matrixVectorDot(x: Tensor, y: Tensor): Tensor = {
      val m = x.shape(0); val n = x.shape(1)
      val res = mallocArray[Float](m)
      hip("lh_sgemv", 0, m, n, 1.0f, x.data, n, y.data, 0.0f, res)
      Tensor(res, m)
    }
    override def matrixMatrixDot(x: Tensor, y: Tensor): Tensor = {
      val m = x.shape(0); val n = y.shape(1); val k = y.shape(0)
      val res = mallocArray[Float](m * n)
      hip("lh_sgemm", 0, 0, m, n, k, 1.0f, x.data, k, y.data, n, 0.0f, res, n)
      Tensor(res, m, n)
    }
    override def dot_grad(x: TensorR, y: TensorR, output: TensorR): Unit = (x.x.rank, y.x.rank) match {          // CUB:222-247
      case (1, 1) =>
        val dim = x.x.shape(0)
        // x.d += output.d(0) * y.x with the scalar read on the device (CUB:226 copies it to the host first)
        if (!x.isInput) hip("lh_axpy_dev", x.d.data, output.d.data, y.x.data, cast("int64_t", dim))
        if (!y.isInput) hip("lh_axpy_dev", y.d.data, output.d.data, x.x.data, cast("int64_t", dim))
      case (2, 1) =>
        if (!x.isInput) add_cartesian(x.d, y.x, output.d)
        if (!y.isInput) add_composition(y.d, x.x, output.d)
      case (2, 2) =>
        generateRawComment("backprop of matrix-matrix-dot")
        if (!x.isInput) add_dotTrans2(x.d, output.d, y.x)
        if (!y.isInput) add_dotTrans1(y.d, x.x, output.d)
    }
    // x[d1,d2] += output[d1] (x) y[d2]
    override def add_cartesian(x: Tensor, y: Tensor, output: Tensor): Unit = hip("lh_ger", x.shape(0), x.shape(1), output.data, y.data, x.data)
    // x[d2] += y[d1,d2]^T output[d1]
    override def add_composition(x: Tensor, y: Tensor, output: Tensor): Unit =
      hip("lh_sgemv", 1, y.shape(0), y.shape(1), 1.0f, y.data, y.shape(1), output.data, 1.0f, x.data)
    // x[d2,d3] += y[d1,d2]^T output[d1,d3]
    override def add_dotTrans1(x: Tensor, y: Tensor, output: Tensor): Unit = {
      val dim1 = y.shape(0); val dim2 = y.shape(1); val dim3 = output.shape(1)
      hip("lh_sgemm", 1, 0, dim2, dim3, dim1, 1.0f, y.data, dim2, output.data, dim3, 1.0f, x.data, dim3)
    }
    // x[d1,d2] += y[d1,d3] output[d2,d3]^T
    override def add_dotTrans2(x: Tensor, y: Tensor, output: Tensor): Unit = {
      val dim1 = x.shape(0); val dim2 = x.shape(1); val dim3 = output.shape(1)
      hip("lh_sgemm", 0, 1, dim1, dim2, dim3, 1.0f, y.data, dim3, output.data, dim3, 1.0f, x.data, dim2)
    }

    // ---- element-wise arithmetic with broadcasting (CDN:153-375).  One library kernel per rank instead of generated text,
    //      and without the generated kernels' indexing bug (CDN:166-171) --------------------------------------------------------
    def scalarOp(op: String, x: Tensor, y: Rep[Float], inPlace: Boolean): Tensor = {
      val res = if (inPlace) x else Tensor(mallocArray[Float](x.scalarCount), x.shape: _*)
      hip("lh_scalar_op", CText(Seq(op)), x.data, res.data, y, cast("int64_t", x.scalarCount))
      res
    }
    def broadcastOp(op: String, x: Tensor, y: Tensor): (Tensor, Dimensions, Dimensions) = {
      Tensor.dimBroadcast(x.shape, y.shape) match {
        case None => throw new IllegalArgumentException(s"dimensions of tensors do not match for broadcasting! ${x.shape.seq} != ${y.shape.seq}")
        case Some((xShape, yShape, resShape)) =>
          val res = Tensor(mallocArray[Float](resShape.scalarCount), resShape: _*)
          hip("lh_bcast_op", CText(Seq(op)), x.data, hostInts(xShape.dims), y.data, hostInts(yShape.dims), res.data, hostInts(resShape.dims), resShape.dims.size)
          (res, xShape, yShape)
      }
    }
    // the gradient of both operands in one call: the library reduces over the broadcast axes of whichever operand was stretched
    def broadcastGrad(op: String, x: TensorR, y: TensorR, output: TensorR, xShape: Dimensions, yShape: Dimensions): Unit = {
      val xd: Any = if (x.isInput) nullFloats else x.d.data
      val yd: Any = if (y.isInput) nullFloats else y.d.data
      hip("lh_bcast_op_grad", CText(Seq(op)), x.x.data, xd, hostInts(xShape.dims), x.isInput, y.x.data, yd, hostInts(yShape.dims), y.isInput,
          output.d.data, hostInts(output.x.shape.dims), output.x.rank)
    }
    def broadcastUpdate(op: String, x: Tensor, y: Tensor): Unit = {
      Tensor.dimBroadcast(x.shape, y.shape) match {
        case None => throw new IllegalArgumentException(s"dimensions of tensors do not match for broadcasting! ${x.shape.seq} != ${y.shape.seq}")
        case Some((xShape, yShape, resShape)) =>
          assert(xShape.dims == resShape.dims || yShape.dims == resShape.dims, "an in-place update broadcasts or reduces its right operand only")
          hip("lh_bcast_update", CText(Seq(op)), x.data, hostInts(xShape.dims), y.data, hostInts(yShape.dims), xShape.dims.size)
      }
    }
    override def +(x: Tensor, y: Rep[Float]): Tensor = scalarOp(lhAdd, x, y, false)
    override def +(x: Tensor, y: Tensor): (Tensor, Dimensions, Dimensions) = broadcastOp(lhAdd, x, y)
    override def add_grad(x: TensorR, y: TensorR, output: TensorR, xShape: Dimensions, yShape: Dimensions): Unit = broadcastGrad(lhAdd, x, y, output, xShape, yShape)
    override def +=(x: Tensor, y: Rep[Float]): Unit = { scalarOp(lhAdd, x, y, true); () }
    override def +=(x: Tensor, y: Tensor): Unit = broadcastUpdate(lhAdd, x, y)
    override def -(x: Tensor, y: Rep[Float]): Tensor = scalarOp(lhSub, x, y, false)
    override def -(x: Tensor, y: Tensor): (Tensor, Dimensions, Dimensions) = broadcastOp(lhSub, x, y)
    // (the reference's non-broadcast branch writes y's gradient into x.d, CDN:322: not reproduced)
    override def minus_grad(x: TensorR, y: TensorR, output: TensorR, xShape: Dimensions, yShape: Dimensions): Unit = broadcastGrad(lhSub, x, y, output, xShape, yShape)
    override def -=(x: Tensor, y: Rep[Float]): Unit = { scalarOp(lhSub, x, y, true); () }
    override def -=(x: Tensor, y: Tensor): Unit = broadcastUpdate(lhSub, x, y)
    override def *(x: Tensor, y: Rep[Float]): Tensor = scalarOp(lhMul, x, y, false)
    override def *(x: Tensor, y: Tensor): (Tensor, Dimensions, Dimensions) = broadcastOp(lhMul, x, y)
    override def mul_grad(x: TensorR, y: TensorR, output: TensorR, xShape: Dimensions, yShape: Dimensions): Unit = broadcastGrad(lhMul, x, y, output, xShape, yShape)
    override def *=(x: Tensor, y: Rep[Float]): Unit = { scalarOp(lhMul, x, y, true); () }
    override def *=(x: Tensor, y: Tensor): Unit = broadcastUpdate(lhMul, x, y)                                    // `???` in the reference (CDN:351)
    override def /(x: Tensor, y: Rep[Float]): Tensor = scalarOp(lhDiv, x, y, false)
    override def /(x: Tensor, y: Tensor): (Tensor, Dimensions, Dimensions) = broadcastOp(lhDiv, x, y)
    override def div_grad(x: TensorR, y: TensorR, output: TensorR, xShape: Dimensions, yShape: Dimensions): Unit = broadcastGrad(lhDiv, x, y, output, xShape, yShape)
    override def /=(x: Tensor, y: Rep[Float]): Unit = { scalarOp(lhDiv, x, y, true); () }
    override def /=(x: Tensor, y: Tensor): Unit = broadcastUpdate(lhDiv, x, y)                                    // `???` in the reference (CDN:376)

    // ---- plusBias / plusEqual (CDN:626-649: cudnnAddTensor in place; the gradient of `main` is shared, the bias gets the reduction) ----
    override def plusBias(main: Tensor, bias: Tensor): Tensor = { broadcastUpdate(lhAdd, main, bias); main }
    override def plusBias_grad(main: TensorR, bias: TensorR): Unit = if (!bias.isInput) {
      // bias.d += main.d summed over the axes along which the bias was broadcast: the same in-place update with the small operand on the left
      Tensor.dimBroadcast(main.x.shape, bias.x.shape) match {
        case None => throw new IllegalArgumentException("plusBias_grad: shapes do not broadcast")
        case Some((mShape, bShape, _)) => hip("lh_bcast_update", CText(Seq(lhAdd)), bias.d.data, hostInts(bShape.dims), main.d.data, hostInts(mShape.dims), mShape.dims.size)
      }
    }
    override def plusEqual(base: Tensor, adder: Tensor): Tensor = {
      assert(base.shape.dims == adder.shape.dims, s"plusEqual needs equal shapes, got ${base.shape.seq} and ${adder.shape.seq}")
      hip("lh_geam", base.data, 1.0f, adder.data, 1.0f, base.data, cast("int64_t", base.scalarCount)); base
    }
    override def plusEqual_grad(base: TensorR, adder: TensorR): Unit =
      if (!adder.isInput) hip("lh_geam", adder.d.data, 1.0f, base.d.data, 1.0f, adder.d.data, cast("int64_t", base.x.scalarCount))

    // ---- geam / trans / permute (CUB:318-587) ------------------------------------------------------------------------------
    override def geam(x: Tensor, transX: Boolean, alpha: Rep[Float], y: Tensor, transY: Boolean, beta: Rep[Float], output: Tensor): Unit = {
      assert(!transX && !transY, "lh_geam adds without transposing (the SGD step and gradient sums: NN:279-285); transposes go through trans()")
      assert(x.shape.dims == y.shape.dims && x.shape.dims == output.shape.dims, "geam: shapes must agree")
      hip("lh_geam", x.data, alpha, y.data, beta, output.data, cast("int64_t", x.scalarCount))
    }
    override def trans(x: Tensor): Tensor = {
      assert(x.rank == 2, "trans only supported for 2D matrix")
      val res = Tensor(mallocArray[Float](x.scalarCount), x.shape.reverse: _*)
      hip("lh_trans", x.data, res.data, x.shape(0), x.shape(1)); res
    }
    override def trans_grad(x: TensorR, y: TensorR): Unit = hip("lh_trans_grad", x.d.data, y.d.data, x.x.shape(0), x.x.shape(1))    // x.d += y.d^T (CUB:369-374)
    override def permute(x: Tensor, dims: Int*): Tensor = {
      assert(dims.sorted == (0 until x.rank), s"permutation dimensions should be within ranks, got rank: ${x.rank}, dims: ${dims}")
      assert(x.rank <= 4, s"TODO, only handle tensor with rank at most 4D for now")
      val res = Tensor(mallocArray[Float](x.scalarCount), dims.map(i => x.shape(i)): _*)
      hip("lh_permute", x.data, res.data, hostInts(x.shape.dims), hostInts(dims.map(unit(_))), x.rank); res
    }
    override def permute_grad(x: TensorR, y: TensorR, dims: Int*): Unit =                                         // accumulates, as CUB:584-587
      hip("lh_permute_grad", x.d.data, y.d.data, hostInts(x.x.shape.dims), hostInts(dims.map(unit(_))), x.x.rank)

    // ---- gemm (CUB:589-688) -----------------------------------------------------------------------------------------------
    override def gemm(x: Tensor, transX: Boolean, y: Tensor, transY: Boolean, alpha: Float): Tensor = {
      val m = if (transX) x.shape(1) else x.shape(0); val k = if (transX) x.shape(0) else x.shape(1)
      val n = if (transY) y.shape(0) else y.shape(1)
      val res = Tensor(mallocArray[Float](m * n), m, n)
      hip("lh_sgemm", transX, transY, m, n, k, alpha, x.data, x.shape(1), y.data, y.shape(1), 0.0f, res.data, n); res
    }
    override def gemm_grad(x: TensorR, transX: Boolean, y: TensorR, transY: Boolean, alpha: Float, output: TensorR): Unit = {
      val d1 = output.x.shape(0); val d3 = output.x.shape(1)
      val d2 = if (transX) x.x.shape(0) else x.x.shape(1)
      val od = output.d.data
      (transX, transY) match {                                   // the four cases of CUB:642-688, every product accumulating (beta 1)
        case (false, false) =>
          if (!x.isInput) hip("lh_sgemm", 0, 1, d1, d2, d3, alpha, od, d3, y.x.data, d3, 1.0f, x.d.data, d2)
          if (!y.isInput) hip("lh_sgemm", 1, 0, d2, d3, d1, alpha, x.x.data, d2, od, d3, 1.0f, y.d.data, d3)
        case (false, true) =>
          if (!x.isInput) hip("lh_sgemm", 0, 0, d1, d2, d3, alpha, od, d3, y.x.data, d2, 1.0f, x.d.data, d2)
          if (!y.isInput) hip("lh_sgemm", 1, 0, d3, d2, d1, alpha, od, d3, x.x.data, d2, 1.0f, y.d.data, d2)
        case (true, false) =>
          if (!x.isInput) hip("lh_sgemm", 0, 1, d2, d1, d3, alpha, y.x.data, d3, od, d3, 1.0f, x.d.data, d1)
          if (!y.isInput) hip("lh_sgemm", 0, 0, d2, d3, d1, alpha, x.x.data, d1, od, d3, 1.0f, y.d.data, d3)
        case (true, true) =>
          if (!x.isInput) hip("lh_sgemm", 1, 1, d2, d1, d3, alpha, y.x.data, d2, od, d3, 1.0f, x.d.data, d1)
          if (!y.isInput) hip("lh_sgemm", 1, 1, d3, d2, d1, alpha, od, d3, x.x.data, d1, 1.0f, y.d.data, d2)
      }
    }

    // ---- convolution (CDN:833-880).  No descriptors, no per-site algorithm search in the emitted text: the library measures its
    //      launch plans on first use ------------------------------------------------------------------------------------------
    var convsOpen = 0                                             // forward convolutions staged whose gradient call is still to come
    override def conv2D_batch(input: Tensor, kernel: Tensor, bias: Option[Tensor], strides: Seq[Int], pads: Seq[Int]): (Tensor, Option[Tensor], Int) = {
      assert(input.rank == 4, s"Convolution input must have rank 4, but got ${input.rank}")
      assert(kernel.rank == 4, s"Convolution kernel must have rank 4, but got ${kernel.rank}")
      assert(strides.size == 2, "Strides should have length 2: [strideRow, strideColumn]")
      assert(pads.size == 1 || pads.size == 2 || pads.size == 4, "pads should have length 1, 2, or 4")
      assert(input.shape(1) == kernel.shape(1), s"In-channel count mismatch: input.shape[1] ${input.shape(1)} should match kernel.shape[1] ${kernel.shape(1)}")
      bias.foreach(b => assert(b.rank == 1 && b.shape(0) == kernel.shape(0), "Convolution bias must have rank 1 and the kernel's output channels"))
      val (padH, padW) = if (pads.size == 1) (pads(0), pads(0)) else if (pads.size == 2) (pads(0), pads(1)) else (pads(0), pads(2))
      val (sH, sW) = (strides(0), strides(1))
      val resShape = Seq(input.shape(0), kernel.shape(0), convSize(input.shape(2) + 2 * padH, kernel.shape(2), sH), convSize(input.shape(3) + 2 * padW, kernel.shape(3), sW))
      val res = Tensor(mallocArray[Float](resShape.product1), resShape: _*)
      convsOpen += 1
      hip("lh_conv2d_fwd", input.data, kernel.data, bias.map(_.data: Any).getOrElse(nullFloats), res.data,
          input.shape(0), input.shape(1), input.shape(2), input.shape(3), kernel.shape(0), kernel.shape(2), kernel.shape(3), sH, sW, padH, padW)
      (res, None, 0)                                              // no im2col buffer, no algorithm counter (CDN:859-866 returns a counter)
    }
    override def conv2D_batch_grad(input: TensorR, finput: Option[TensorR], filter: TensorR, res: TensorR, bias: Option[TensorR] = None,
                                   padding: (Int, Int), strides: (Int, Int), dilations: (Int, Int), counter: Int): Unit = {
      assert(dilations == ((1, 1)), "dilated convolutions are not supported")
      val (n, c, h, w) = (input.x.shape(0), input.x.shape(1), input.x.shape(2), input.x.shape(3))
      val (k, r, s) = (filter.x.shape(0), filter.x.shape(2), filter.x.shape(3))
      // Only the optimizer reads filter.d: the filter gradient runs on the library's side stream beside the rest of the backward
      // pass, unless fewer than two convolution gradients are still to come (with nothing left to run beside it the hand-over
      // between the streams only delays the optimizer; the optimizer entry points join).  Gradient calls are staged in the reverse
      // order of the forward calls, so the count of forward convolutions not yet matched is known here at staging time.
      convsOpen -= 1
      val fork = !input.isInput && convsOpen >= 2
      def filterGradient(): Unit = {
        if (fork) hip("lh_side_begin")
        hip("lh_conv2d_bwd_filter", input.x.data, res.d.data, filter.d.data, bias.map(_.d.data: Any).getOrElse(nullFloats), 1.0f,
            n, c, h, w, k, r, s, strides._1, strides._2, padding._1, padding._2)
        if (fork) hip("lh_side_end")
      }
      // With a bias the filter gradient is issued first: its bias sums are the first reader of res.d, and a relu_grad(inPlace)
      // issued just before (conv -> relu networks) is applied in that pass instead of in one of its own.
      if (bias.isDefined) filterGradient()
      if (!input.isInput)                                         // CDN:873
        hip("lh_conv2d_bwd_data", res.d.data, filter.x.data, input.d.data, 1.0f, n, c, h, w, k, r, s, strides._1, strides._2, padding._1, padding._2)
      if (!bias.isDefined) filterGradient()
    }

    // ---- pooling (CDN:882-982).  Max-pool keeps its argmax (global flat input index, first maximum wins: CPU:848-948), which the
    //      cuDNN backend does not (sidx = None, CDN:968) -------------------------------------------------------------------------
    override def maxPool2D_batch(input: Tensor, kernel: Seq[Int], strides: Seq[Int], pads: Option[Seq[Int]]): (Tensor, Option[Rep[Array[Int]]]) = {
      assert(input.rank == 4, "Currently, maxpool2D only supports inputs of rank 4")
      assert(kernel.size == 2 && strides.size == 2, "kernel and strides should have length 2")
      val pad = pads match { case None => 0; case Some(p) => assert(p.forall(_ == p(0)), "one padding for all four sides"); p(0) }
      val resShape = Seq(input.shape(0), input.shape(1), convSize(input.shape(2) + 2 * pad, kernel(0), strides(0)), convSize(input.shape(3) + 2 * pad, kernel(1), strides(1)))
      val res = Tensor(mallocArray[Float](resShape.product1), resShape: _*)
      val idx = mallocArray[Int](resShape.product1)
      hip("lh_maxpool_fwd", input.data, res.data, idx, input.shape(0), input.shape(1), input.shape(2), input.shape(3), kernel(0), kernel(1), strides(0), strides(1), pad)
      (res, Some(idx))
    }
    override def maxPool2D_batch_grad(input: TensorR, output: TensorR, sidx: Option[Rep[Array[Int]]], kernel: Seq[Int], strides: Seq[Int], pads: Seq[Int]): Unit =
      // dense gather: every input pixel sums the windows whose argmax it is; accumulates (CPU:950-959; cuDNN overwrites, CDN:966-967)
      hip("lh_maxpool_bwd_dense", output.d.data, sidx.get, input.d.data, 1.0f, input.x.shape(0), input.x.shape(1), input.x.shape(2), input.x.shape(3),
          kernel(0), kernel(1), strides(0), strides(1), pads(0))
    override def averagePool2D_batch(input: Tensor, kernel: Seq[Int], strides: Seq[Int], pads: Seq[Int]): Tensor = {
      assert(input.rank == 4, "Current, averagePool2D_batch only supports inputs of rank 4")
      val (pH, pW) = (pads(0), pads(2))
      val resShape = Seq(input.shape(0), input.shape(1), convSize(input.shape(2) + 2 * pH, kernel(0), strides(0)), convSize(input.shape(3) + 2 * pW, kernel(1), strides(1)))
      val res = Tensor(mallocArray[Float](resShape.product1), resShape: _*)
      // the divisor counts the elements inside the image (CUDNN_POOLING_AVERAGE_COUNT_EXCLUDE_PADDING, CDN:975-982)
      hip("lh_avgpool_pad_fwd", input.data, res.data, input.shape(0), input.shape(1), input.shape(2), input.shape(3), kernel(0), kernel(1), strides(0), strides(1), pH, pW)
      res
    }
    override def averagePool2D_batch_grad(input: TensorR, output: TensorR, kernel: Seq[Int], strides: Seq[Int], pads: Seq[Int]): Unit =
      hip("lh_avgpool_pad_bwd", output.d.data, input.d.data, input.x.shape(0), input.x.shape(1), input.x.shape(2), input.x.shape(3),
          kernel(0), kernel(1), strides(0), strides(1), pads(0), pads(2))

    // ---- batch norm (CDN:984-1266): SPATIAL for rank 4, PER_ACTIVATION for rank 2; eps 1e-5, running-average factor 0.1 ----------
    def bnDims(x: Tensor): (Rep[Int], Rep[Int], Rep[Int]) =
      if (x.rank == 4) (x.shape(0), x.shape(1), x.shape(2) * x.shape(3)) else { assert(x.rank == 2, "batch norm takes rank 4 or rank 2"); (x.shape(0), x.shape(1), unit(1)) }
    def bnInference(x: Tensor, scale: Tensor, bias: Tensor, runningMean: Tensor, runningVar: Tensor): Tensor = {
      val (n, c, hw) = bnDims(x)
      val res = Tensor(mallocArray[Float](x.scalarCount), x.shape: _*)
      hip("lh_bn_infer", x.data, scale.data, bias.data, runningMean.data, runningVar.data, res.data, n, c, hw, 1e-5f); res
    }
    def bnTraining(x: Tensor, scale: Tensor, bias: Tensor, runningMean: Tensor, runningVar: Tensor): (Tensor, Option[Tensor], Option[Tensor], Int) = {
      val (n, c, hw) = bnDims(x)
      val res = Tensor(mallocArray[Float](x.scalarCount), x.shape: _*)
      val saveMean = Tensor(mallocArray[Float](c), c); val saveInvStd = Tensor(mallocArray[Float](c), c)
      hip("lh_bn_train_fwd", x.data, scale.data, bias.data, runningMean.data, runningVar.data, res.data, saveMean.data, saveInvStd.data, n, c, hw, 1e-5f, 0.1f)
      (res, Some(saveMean), Some(saveInvStd), 0)
    }
    def bnGrad(input: TensorR, res: TensorR, scale: TensorR, bias: TensorR, saveMean: Option[Tensor], saveInvVariance: Option[Tensor]): Unit = {
      val (n, c, hw) = bnDims(input.x)
      // accumulates into input.d, scale.d and bias.d (alpha = beta = 1, CDN:1101-1108)
      hip("lh_bn_bwd", input.x.data, res.d.data, scale.x.data, saveMean.get.data, saveInvVariance.get.data, input.d.data, 1.0f, scale.d.data, bias.d.data, n, c, hw)
    }
    override def batchNormInference(x: Tensor, scale: Tensor, bias: Tensor, runningMean: Tensor, runningVar: Tensor): Tensor = { assert(x.rank == 4); bnInference(x, scale, bias, runningMean, runningVar) }
    override def batchNormTraining(x: Tensor, scale: Tensor, bias: Tensor, runningMean: Tensor, runningVar: Tensor) = { assert(x.rank == 4); bnTraining(x, scale, bias, runningMean, runningVar) }
    override def batchNorm_grad(input: TensorR, res: TensorR, scale: TensorR, bias: TensorR, saveMean: Option[Tensor], saveInvVariance: Option[Tensor], counterId: Int): Unit =
      bnGrad(input, res, scale, bias, saveMean, saveInvVariance)
    override def batchNorm1DInference(x: Tensor, scale: Tensor, bias: Tensor, runningMean: Tensor, runningVar: Tensor): Tensor = { assert(x.rank == 2); bnInference(x, scale, bias, runningMean, runningVar) }
    override def batchNorm1DTraining(x: Tensor, scale: Tensor, bias: Tensor, runningMean: Tensor, runningVar: Tensor) = { assert(x.rank == 2); bnTraining(x, scale, bias, runningMean, runningVar) }
    override def batchNorm1D_grad(input: TensorR, res: TensorR, scale: TensorR, bias: TensorR, saveMean: Option[Tensor], saveInvVariance: Option[Tensor], counterId: Int): Unit =
      bnGrad(input, res, scale, bias, saveMean, saveInvVariance)

    // ---- dropout (CDN:1268-1347).  A counter-based generator keyed by (seed, position) instead of cuDNN's states seeded with
    //      time(NULL) (CDN:1301): reproducible, and the mask is the multiplier the backward pass needs ----------------------------
    var dropoutOffset: Rep[Long] = unit(0L)
    val dropoutSeed: Long = 42L
    override def dropout(input: Tensor, prob: Float = 0.5f): (Tensor, Rep[Array[Float]], Rep[Int]) = {
      assert(0.0f <= prob && prob < 1.0f, s"dropout rate should be [0.0, 1), got $prob")
      val res = Tensor(mallocArray[Float](input.scalarCount), input.shape: _*)
      val mask = mallocArray[Float](input.scalarCount)
      hip("lh_dropout_fwd", input.data, res.data, mask, cast("int64_t", input.scalarCount), prob, CText(Seq(dropoutSeed.toString + "ull")), cast("uint64_t", dropoutOffset))
      dropoutOffset = dropoutOffset + input.scalarCount.toLong
      (res, mask, input.scalarCount)
    }
    override def dropout_grad(input: TensorR, output: TensorR, prob: Float, helper: Rep[Array[Float]], size: Rep[Int]): Unit =
      hip("lh_dropout_bwd", output.d.data, helper, input.d.data, cast("int64_t", size))
    override def mask4D(input: Tensor, lengths: Rep[Array[Int]]): Tensor = {                                      // CUB:710-719
      assert(input.rank == 4, s"mask4D only deals with inputs of 4D, got ${input.rank}")
      hip("lh_mask4d", input.data, lengths, input.shape(0), input.shape(1), input.shape(2), input.shape(3)); input
    }

    // ---- activations (CDN:1349-1429; CUB:733-800) ------------------------------------------------------------------------------
    def unary(op: String, x: Tensor, inPlace: Boolean, lo: Float = 0.0f, hi: Float = 0.0f): Tensor = {
      val res = if (inPlace) x else Tensor(mallocArray[Float](x.scalarCount), x.shape: _*)
      hip("lh_unary", CText(Seq(op)), x.data, res.data, cast("int64_t", x.scalarCount), lo, hi); res
    }
    // input.d += f'(.) * res.d; in place (the value was overwritten by the forward pass): input.d is masked / scaled instead
    def unaryGrad(op: String, input: TensorR, res: TensorR, inPlace: Boolean, lo: Float = 0.0f, hi: Float = 0.0f): Unit =
      hip("lh_unary_grad", CText(Seq(op)), input.x.data, res.x.data, res.d.data, input.d.data, cast("int64_t", input.x.scalarCount), inPlace, lo, hi)
    override def relu(x: Tensor, inPlace: Boolean = false): Tensor = unary(lhRelu, x, inPlace)
    override def tanh(x: Tensor): Tensor = unary(lhTanh, x, false)
    override def sigmoid(x: Tensor): Tensor = unary(lhSigmoid, x, false)
    override def hardTanh(x: Tensor, min_val: Float = -1.0f, max_val: Float = 1.0f, inPlace: Boolean = false): Tensor = unary(lhHardTanh, x, inPlace, min_val, max_val)
    override def exp(x: Tensor): Tensor = unary(lhExp, x, false)
    override def log(x: Tensor): Tensor = unary(lhLog, x, false)
    override def sqrt(x: Tensor): Tensor = unary(lhSqrt, x, false)
    override def square(x: Tensor): Tensor = unary(lhSquare, x, false)
    override def relu_grad(input: TensorR, res: TensorR, inPlace: Boolean = false): Unit = unaryGrad(lhRelu, input, res, inPlace)     // mask y > 0 (CDN:1404-1405)
    override def tanh_grad(input: TensorR, res: TensorR): Unit = unaryGrad(lhTanh, input, res, false)
    override def sigmoid_grad(input: TensorR, res: TensorR): Unit = unaryGrad(lhSigmoid, input, res, false)
    override def hardTanh_grad(input: TensorR, res: TensorR, min_val: Float = -1.0f, max_val: Float = 1.0f, inPlace: Boolean = false): Unit =
      unaryGrad(lhHardTanh, input, res, inPlace, min_val, max_val)
    override def exp_grad(input: TensorR, res: TensorR): Unit = unaryGrad(lhExp, input, res, false)
    override def log_grad(input: TensorR, res: TensorR): Unit = unaryGrad(lhLog, input, res, false)
    override def sqrt_grad(input: TensorR, res: TensorR): Unit = unaryGrad(lhSqrt, input, res, false)
    override def square_grad(input: TensorR, res: TensorR): Unit = unaryGrad(lhSquare, input, res, false)

    // ---- softmax over axis `dim` of an [outer, c, inner] view (CDN:1431-1504) -----------------------------------------------------
    def softmaxView(x: Tensor, dim: Int): (Rep[Int], Rep[Int], Rep[Int]) = {
      assert(dim >= 0 && dim < x.rank, s"softmax dimension $dim out of range for rank ${x.rank}")
      (x.shape.take(dim).foldLeft(unit(1)) { case (a, b) => a * b }, x.shape(dim), x.shape.drop(dim + 1).foldLeft(unit(1)) { case (a, b) => a * b })
    }
    def softmaxHelper(x: Tensor, dim: Int, isLog: Boolean): Tensor = {
      val (outer, c, inner) = softmaxView(x, dim)
      val res = Tensor(mallocArray[Float](x.scalarCount), x.shape: _*)
      hip("lh_softmax", isLog, x.data, res.data, outer, c, inner); res
    }
    def softmaxBackwardHelper(input: TensorR, res: TensorR, dim: Int, isLog: Boolean): Unit = {
      val (outer, c, inner) = softmaxView(input.x, dim)
      hip("lh_softmax_grad", isLog, res.x.data, res.d.data, input.d.data, outer, c, inner)                        // accumulates (beta 1, CDN:1476-1486)
    }
    override def softmax(x: Tensor, dim: Int = 1): Tensor = softmaxHelper(x, dim, false)
    override def logSoftmax(x: Tensor, dim: Int = 1): Tensor = softmaxHelper(x, dim, true)
    override def softmax_grad(input: TensorR, res: TensorR, dim: Int = 1): Unit = softmaxBackwardHelper(input, res, dim, false)
    override def logSoftmax_grad(input: TensorR, res: TensorR, dim: Int = 1): Unit = softmaxBackwardHelper(input, res, dim, true)

    // ---- losses (CUB:802-813; CDN:1895-1938) -------------------------------------------------------------------------------------
    override def nllLoss(x: Tensor, target: Rep[Array[Int]]): Tensor = {
      assert(x.rank == 2, "Input must be a 2-D tensor")
      val res = Tensor(mallocArray[Float](x.shape(0)), x.shape(0))
      hip("lh_nll", x.data, target, res.data, x.shape(0), x.shape(1)); res
    }
    override def nllLoss_grad(input: TensorR, res: TensorR, target: Rep[Array[Int]]): Unit =
      hip("lh_nll_grad", input.d.data, target, res.d.data, input.d.shape(0), input.d.shape(1))
    override def ctcLoss(prob: TensorR, inputLengths: Rep[Array[Int]], labels: Rep[Array[Int]], labelLengths: Rep[Array[Int]]): Tensor = {
      assert(prob.x.rank == 3, "Probability tensor should have rank 3: [inputLength, batchSize, alphabetSize]")
      assert(prob.x.shape(1) <= 256, "'cudnnCTCLoss' requires batch size less than 256")                          // kept so that programs behave alike (CDN:1901)
      val costs = Tensor(mallocArray[Float](prob.x.shape(1)), prob.x.shape(1))
      // the length and label arrays stay HOST arrays; the gradient with respect to the softmax input is accumulated into prob.d
      hip("lh_ctc_loss", prob.x.data, prob.d.data, labels, labelLengths, inputLengths, costs.data, prob.x.shape(0), prob.x.shape(1), prob.x.shape(2))
      mean(costs)                                                 // CDN:1937: the reported loss is the batch average
    }

    // ---- reductions (CDN:1506-1636) -----------------------------------------------------------------------------------------------
    override def sum(x: Tensor): Tensor = { val res = Tensor(mallocArray[Float](1), 1); hip("lh_sum_all", x.data, res.data, cast("int64_t", x.scalarCount)); res }
    override def sum_grad(input: TensorR, res: TensorR): Unit = hip("lh_add_scalar_from", input.d.data, res.d.data, 1.0f, cast("int64_t", input.d.scalarCount))
    override def mean(x: Tensor): Tensor = { val res = Tensor(mallocArray[Float](1), 1); hip("lh_mean_all", x.data, res.data, cast("int64_t", x.scalarCount)); res }
    override def mean_grad(input: TensorR, res: TensorR): Unit =
      hip("lh_add_scalar_from", input.d.data, res.d.data, CText(Seq("1.0f / (float)", input.x.scalarCount)), cast("int64_t", input.d.scalarCount))
    override def sum(x: Tensor, dim: Int): Tensor = {
      assert(dim >= 0 && dim < x.rank, s"dim should be in range, got ${dim} from ${x.rank}")
      val resShape = x.shape.take(dim) ++ x.shape.drop(dim + 1)
      val res = Tensor(mallocArray[Float](resShape.foldLeft(unit(1)) { case (a, b) => a * b }), resShape: _*)
      hip("lh_sum_dim", x.data, res.data, x.shape.take(dim).foldLeft(unit(1)) { case (a, b) => a * b }, x.shape(dim), x.shape.drop(dim + 1).foldLeft(unit(1)) { case (a, b) => a * b })
      res
    }
    override def sum_grad(input: TensorR, output: TensorR, dim: Int): Unit =
      hip("lh_sum_dim_grad", input.d.data, output.d.data, input.x.shape.take(dim).foldLeft(unit(1)) { case (a, b) => a * b }, input.x.shape(dim),
          input.x.shape.drop(dim + 1).foldLeft(unit(1)) { case (a, b) => a * b })

    // ---- concat over any axis and any number of inputs (CUB:825-879 handles two 4-D inputs on axis 1) -------------------------------
    override def concat(dim: Int, tensors: Seq[Tensor]): Tensor = {
      assert(tensors.size >= 2, "need at least two tensors for concat")
      assert(tensors.forall(_.rank == tensors.head.rank), "all tensors of a concat must have the same rank")
      val head = tensors.head
      val outer = head.shape.take(dim).foldLeft(unit(1)) { case (a, b) => a * b }
      val inner = head.shape.drop(dim + 1).foldLeft(unit(1)) { case (a, b) => a * b }
      val total = tensors.map(_.shape(dim)).reduce(_ + _)
      val resShape = head.shape.take(dim) ++ Seq(total) ++ head.shape.drop(dim + 1)
      val res = Tensor(mallocArray[Float](outer * total * inner), resShape: _*)
      hip("lh_concat", tensors.size, hostPointers(tensors.map(_.data)), hostInts(tensors.map(_.shape(dim))), res.data, outer, inner); res
    }
    override def concat_grad(dim: Int, tensorRs: Seq[TensorR], output: TensorR): Unit = {
      val head = tensorRs.head.x
      hip("lh_concat_grad", tensorRs.size, hostPointers(tensorRs.map(_.d.data)), hostInts(tensorRs.map(_.x.shape(dim))), output.d.data,
          head.shape.take(dim).foldLeft(unit(1)) { case (a, b) => a * b }, head.shape.drop(dim + 1).foldLeft(unit(1)) { case (a, b) => a * b })
    }

    // ---- repeat0: the sliding window of the look-ahead layer (CDN:378-398) ---------------------------------------------------------
    override def repeat0(in: Tensor, context: Int): Tensor = {
      assert(in.rank <= 3, s"only support input with no more than 3D, got ${in.rank}")
      val resShape = Seq(in.shape(0) - context, unit(context + 1)) ++ in.shape.drop(1)
      val res = Tensor(mallocArray[Float](resShape.foldLeft(unit(1)) { case (a, b) => a * b }), resShape: _*)
      hip("lh_repeat0", in.data, res.data, in.shape(0), context, cast("int64_t", in.shape.strides(0))); res
    }
    override def repeat0_grad(in: TensorR, out: TensorR, context: Int): Unit =
      hip("lh_repeat0_grad", in.d.data, out.d.data, in.x.shape(0), context, cast("int64_t", in.x.shape.strides(0)))

    // ---- optimizers (CUB:884-896): clip, update, clear the gradient, in one kernel ---------------------------------------------------
    override def adagrad_update(tr: TensorR, t: Tensor, learning_rate: Float, gradClip: Float, descent: Boolean): Unit = {
      assert(descent, s"TODO: only handle gradient descent (not ascent) so far")
      assert(tr.x.shape == t.shape, s"tensor and momentum should have the same shape, got ${tr.x.shape} and ${t.shape}")
      hip("lh_adagrad", tr.x.data, tr.d.data, t.data, learning_rate, gradClip, cast("int64_t", t.scalarCount))
    }
    override def momentum_update(tr: TensorR, t: Tensor, learning_rate: Float, momentum: Float, gradClip: Float, nesterov: Boolean, descent: Boolean) = {
      assert(descent, s"TODO: only handle gradient descent (not ascent) so far")
      assert(tr.x.shape == t.shape, s"tensor and momentum should have the same shape, got ${tr.x.shape} and ${t.shape}")
      hip("lh_momentum", tr.x.data, tr.d.data, t.data, learning_rate, momentum, gradClip, nesterov, cast("int64_t", t.scalarCount))
    }

    // ---- recurrent layers (CDN:1638-1893; called by RNNBase, NNModule.scala:392-416).  One layer, zero initial states, no dropout;
    //      RNNBase stacks layers itself when numLayers > 1.  The weight buffer has cuDNN's layout (NNModule.scala:378-390) -----------
    // One library call per layer (the library's layer = cuDNN's with numLayers = 1); a stack is a loop at staging time over the
    // packed parameter buffer (per layer: forward direction W_ih, W_hh, b_ih, b_hh, then the reverse direction; NN:378-390),
    // with the backend's dropout between layers (cuDNN applies its own to every layer's output but the last) and the initial
    // states cut per layer ([numLayers * numDirections, batch, hidden], CDN:1823).  What the backward pass needs of the
    // layers in between is kept here at staging time under the call's counter.
    case class RnnLayerRecord(input: TensorR, output: TensorR, reserve: Rep[Array[Float]], mask: Option[Rep[Array[Float]]], wOffset: Int)
    val rnnRecords = scala.collection.mutable.HashMap[Int, Seq[RnnLayerRecord]]()
    var rnnCounter = 0
    def rnnForwardTraining(mode: RnnMode, x: Tensor, hx: Option[Tensor] = None, cx: Option[Tensor] = None, w: Tensor, numLayers: Int, hiddenSize: Int,
                           dropout: Float = 0f, bidirectional: Boolean = false): (Tensor, Option[Tensor], Rep[Array[Float]], Rep[Int], Int) = {
      assert(x.rank == 3, "RNN input should have rank 3: [seqLength x batchSize x inputSize]")
      assert(cx.isEmpty || mode == LstmMode, "only the LSTM has a cell state")
      val (t, b) = (x.shape(0), x.shape(1)); val d = if (bidirectional) 2 else 1
      val gated = mode == LstmMode || mode == GruMode
      val gateSize = mode.numGates * hiddenSize
      val records = scala.collection.mutable.ArrayBuffer[RnnLayerRecord]()
      var layerIn = new TensorR(x, x)                             // the first layer's gradient target is the caller's (rnnBackward)
      var wOffset = 0
      for (layer <- 0 until numLayers) {
        val i = layerIn.x.shape(2)
        val res = Tensor(mallocArray[Float](t * b * d * hiddenSize), t, b, d * hiddenSize)
        val stateOffset = layer * d * b * hiddenSize
        val h0: Any = hx.map(h => slice(h.data, stateOffset): Any).getOrElse(nullFloats)
        val c0: Any = cx.map(c => slice(c.data, stateOffset): Any).getOrElse(nullFloats)
        val wl = slice(w.data, wOffset)
        val reserve = if (gated) mallocArray[Float](t * b * (mode.numGates + 1) * hiddenSize * d) else unchecked[Array[Float]]("(float*)0")
        if (gated) hip("lh_rnn_gated_fwd_init", mode.id, layerIn.x.data, h0, c0, wl, res.data, reserve, t, b, i, hiddenSize, bidirectional)
        else hip("lh_rnn_fwd_init", mode.id, layerIn.x.data, h0, wl, res.data, t, b, i, hiddenSize, bidirectional)
        val out = TensorR(res)
        val last = layer == numLayers - 1
        val (next, mask) = if (dropout > 0f && !last) { val (y, m, _) = this.dropout(res, dropout); (TensorR(y), Some(m)) } else (out, None)
        records += RnnLayerRecord(layerIn, out, reserve, mask, wOffset)
        if (mask.isDefined) records += RnnLayerRecord(out, next, reserve, mask, -1)          // the dropout between two layers
        wOffset += d * (gateSize * i + gateSize * hiddenSize + 2 * gateSize)
        layerIn = next
      }
      rnnCounter += 1
      rnnRecords(rnnCounter) = records.toSeq
      (layerIn.x, None, records.last.reserve, unit(0), rnnCounter)
    }
    def rnnBackward(mode: RnnMode, input: TensorR, hx: Option[Tensor], cx: Option[Tensor], w: TensorR, output: TensorR, numLayers: Int, hiddenSize: Int,
                    dropout: Float = 0f, bidirectional: Boolean = false, reserve: Rep[Array[Float]], reserveSize: Rep[Int], counter: Int): Unit = {
      val (t, b) = (input.x.shape(0), input.x.shape(1)); val d = if (bidirectional) 2 else 1
      val gated = mode == LstmMode || mode == GruMode
      val records = rnnRecords(counter)
      var layer = numLayers
      records.zipWithIndex.reverse.foreach { case (r, idx) =>
        val outR = if (idx == records.size - 1) output else r.output       // the caller's TensorR carries the gradient of the last layer
        if (r.wOffset < 0) dropout_grad(r.input, outR, dropout, r.mask.get, r.input.x.scalarCount)
        else {
          layer -= 1
          val inR = if (idx == 0) input else r.input
          val i = inR.x.shape(2)
          val stateOffset = layer * d * b * hiddenSize
          val h0: Any = hx.map(h => slice(h.data, stateOffset): Any).getOrElse(nullFloats)
          val c0: Any = cx.map(c => slice(c.data, stateOffset): Any).getOrElse(nullFloats)
          val dx: Any = if (inR.isInput) nullFloats else inR.d.data       // cudnnRNNBackwardData is skipped for inputs (CDN:1889-1890)
          val (wl, dwl) = (slice(w.x.data, r.wOffset), slice(w.d.data, r.wOffset))
          if (gated) hip("lh_rnn_gated_bwd_init", mode.id, inR.x.data, h0, c0, outR.x.data, outR.d.data, wl, r.reserve, dx, 1.0f, dwl, t, b, i, hiddenSize, bidirectional)
          else hip("lh_rnn_bwd_init", mode.id, inR.x.data, h0, outR.x.data, outR.d.data, wl, dx, 1.0f, dwl, t, b, i, hiddenSize, bidirectional)
        }
      }
      rnnRecords -= counter
    }
    // the names RNNBase calls (NNModule.scala:407-416)
    def cudnnRNNForwardTraining(mode: RnnMode, x: Tensor, hx: Option[Tensor] = None, cx: Option[Tensor] = None, w: Tensor, numLayers: Int, hiddenSize: Int,
                                dropout: Float = 0f, bidirectional: Boolean = false) = rnnForwardTraining(mode, x, hx, cx, w, numLayers, hiddenSize, dropout, bidirectional)
    def cudnnRNNBackward(mode: RnnMode, input: TensorR, hx: Option[Tensor], cx: Option[Tensor], w: TensorR, output: TensorR, numLayers: Int, hiddenSize: Int,
                         dropout: Float = 0f, bidirectional: Boolean = false, reserve: Rep[Array[Float]], reserveSize: Rep[Int], counter: Int): Unit =
      rnnBackward(mode, input, hx, cx, w, output, numLayers, hiddenSize, dropout, bidirectional, reserve, reserveSize, counter)

    // ---- no fused forms here.  The trait's one-call-per-method sequence is what this backend emits; the library recognises the
    //      chains it can run as one kernel (conv -> batchNorm -> [+ shortcut] -> relu in place, their gradients in reverse, a run
    //      of momentum_update / sgd_update calls) and overwrites gradient buffers nobody has touched since `mallocArray`
    //      instead of clearing them and adding (lantern_hip.h, "Fusion of adjacent calls") -------------------------------------------
    // plain SGD in one pass (x -= lr*d; d = 0) instead of geam + clear_grad (NN:279-285); gradients are not clipped there either
    def sgd_update(tr: TensorR, learning_rate: Float, descent: Boolean): Unit =
      hip("lh_sgd", tr.x.data, tr.d.data, if (descent) learning_rate else -learning_rate, cast("int64_t", tr.x.scalarCount))
  }
  object BackendHIP { def apply() = new BackendHIP }
  def BackendGPU: Backend = BackendHIP()                                                                           // as CUB:903-904
  backend = BackendGPU
}

// ---- modules that need the backend by name (NNModule.scala:305-330) ------------------------------------------------------------
trait NNModuleHIP extends NNModule with TensorDslHIP {
  backend = BackendHIP()
  def RNNRelu(inputSize: Int, hiddenSize: Int, numLayers: Int = 1, dropout: Float = 0f, bidirectional: Boolean = false, name: String = "rnn_relu") =
    RNNBase(RnnReluMode, inputSize, hiddenSize, numLayers, dropout, bidirectional, name)
  def RNNTanh(inputSize: Int, hiddenSize: Int, numLayers: Int = 1, dropout: Float = 0f, bidirectional: Boolean = false, name: String = "rnn_tanh") =
    RNNBase(RnnTanhMode, inputSize, hiddenSize, numLayers, dropout, bidirectional, name)
  def LSTM(inputSize: Int, hiddenSize: Int, numLayers: Int = 1, dropout: Float = 0f, bidirectional: Boolean = false, name: String = "lstm") =
    RNNBase(LstmMode, inputSize, hiddenSize, numLayers, dropout, bidirectional, name)
  def GRU(inputSize: Int, hiddenSize: Int, numLayers: Int = 1, dropout: Float = 0f, bidirectional: Boolean = false, name: String = "gru") =
    RNNBase(GruMode, inputSize, hiddenSize, numLayers, dropout, bidirectional, name)
  // NN:265-287 with the update and the gradient reset in one launch per tensor
  case class SGD(override val module: Module, learning_rate: Float, gradClip: Float = 1.0f, descent: Boolean = true) extends Optim {
    def step_func = { case (tr, _) => backend.asInstanceOf[BackendHIP].sgd_update(tr, learning_rate, descent) }
  }
  // RNNBase itself (NNModule.scala:332-417) is reused with `BackendCudnn()` read as `BackendHIP()`: same calls
  // (cudnnRNNForwardTraining / cudnnRNNBackward above, initial states and dropout included).  One difference: layers after the
  // first of a bidirectional stack read 2 * hiddenSize features, which getParameterSize (NN:357) leaves out ("// * numDirections");
  // the buffer must be gateSize * inputSize + (numLayers - 1) * gateSize * hiddenSize * numDirections long per direction.
}

// ---- the driver the applications extend (DslAPI.scala:1064-1077) -------------------------------------------------------------------
abstract class LanternDriverHIP[A: Manifest, B: Manifest] extends DslDriverHIP[A, B] with LanternDriver[A, B] with TensorDslHIP with NNModuleHIP with Dataset { self =>
  override def manifestA: Manifest[A] = manifest[A]
  override def manifestB: Manifest[B] = manifest[B]
  override val codegen = new DslGenHIP { val IR: self.type = self }                      // nothing to append: no generated kernels
}
