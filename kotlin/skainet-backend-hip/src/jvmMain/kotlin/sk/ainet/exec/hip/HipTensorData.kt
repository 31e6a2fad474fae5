package sk.ainet.exec.hip

import java.lang.foreign.Arena
import java.lang.foreign.MemorySegment
import java.lang.foreign.ValueLayout
import sk.ainet.lang.tensor.Shape
import sk.ainet.lang.tensor.data.FloatArrayTensorData
import sk.ainet.lang.types.DType

/**
 * Dense FP32 tensor data whose bytes live in the GPU's memory: what [HipOps] returns, so that a chain of its ops hands
 * device addresses from kernel to kernel and nothing crosses PCIe until somebody reads a value.
 *
 * The same contract as the browser tier's resident data
 * (skainet-backends/skainet-backend-wasm-simd/src/wasmJsMain/kotlin/sk/ainet/exec/wasm/WasmLinearStorage.kt:130-195):
 * [buffer] (and with it `heapFloats`, `view`, `get`, `copyToFloatArray`) is a heap mirror, downloaded once on first
 * use after a device-wide wait, so every op that does not know about the device still computes the right numbers from
 * it; [HipOps] asks [pointer] first and never touches the mirror. A `set` writes through to the device.
 */
public class HipTensorData<T : DType>(
    initialShape: Shape,
    public val storage: HipDeviceStorage,
) : FloatArrayTensorData<T> {

    override val shape: Shape = Shape(initialShape.dimensions.copyOf())

    private val pitch: IntArray = IntArray(shape.rank).also { p ->
        var run = 1
        for (d in shape.rank - 1 downTo 0) {
            p[d] = run
            run *= shape.dimensions[d]
        }
    }
    private var mirror: FloatArray? = null

    init {
        val need = shape.volume.toLong() * Float.SIZE_BYTES
        require(storage.sizeBytes >= need) { "storage of ${storage.sizeBytes} bytes is too small for $shape ($need bytes)" }
    }

    /** `true` while the device bytes are alive (their scope has not been reset or closed). */
    public val isResident: Boolean get() = storage.isAlive

    /** `true` once the heap mirror exists (tests use it to show that a chain of device ops downloaded nothing). */
    public val isMirrored: Boolean get() = mirror != null

    /** Device address of element 0; throws when the storage is closed. */
    public fun pointer(): MemorySegment = storage.pointer()

    override val buffer: FloatArray
        get() {
            mirror?.let { return it }
            val n = shape.volume
            val host = FloatArray(n)
            if (n > 0) {
                // kernels that wrote these bytes may still be in flight on this thread's stream
                check((HipLibrary.sync!!.invoke() as Int) == 0) { "HipTensorData: ${HipLibrary.error()}" }
                Arena.ofConfined().use { arena ->
                    val seg = arena.allocate(n.toLong() * Float.SIZE_BYTES, 16)
                    val rc = HipLibrary.d2h!!.invoke(seg, storage.pointer(), n.toLong() * Float.SIZE_BYTES) as Int
                    check(rc == 0) { "HipTensorData: ${HipLibrary.error()}" }
                    MemorySegment.copy(seg, ValueLayout.JAVA_FLOAT, 0L, host, 0, n)
                }
            }
            mirror = host
            return host
        }

    private fun flat(indices: IntArray): Int {
        require(indices.size == shape.rank) { "${indices.size} indices for a tensor of rank ${shape.rank}" }
        var at = 0
        for (d in indices.indices) {
            val i = indices[d]
            require(i >= 0 && i < shape.dimensions[d]) { "index $i outside dimension $d of size ${shape.dimensions[d]}" }
            at += i * pitch[d]
        }
        return at
    }

    override fun get(vararg indices: Int): Float = buffer[flat(indices)]

    override fun set(vararg indices: Int, value: Float) {
        require(storage.isMutable) { "storage ${storage.id} is not mutable" }
        val at = flat(indices)
        mirror?.let { it[at] = value }
        Arena.ofConfined().use { arena ->
            val one = arena.allocate(Float.SIZE_BYTES.toLong(), 4)
            one.set(ValueLayout.JAVA_FLOAT, 0L, value)
            val dst = MemorySegment.ofAddress(storage.pointer().address() + at.toLong() * Float.SIZE_BYTES)
            val rc = HipLibrary.h2d!!.invoke(dst, one, Float.SIZE_BYTES.toLong()) as Int
            check(rc == 0) { "HipTensorData.set: ${HipLibrary.error()}" }
        }
    }

    override fun copyToFloatArray(): FloatArray = buffer.copyOf()
}

/**
 * A slab of device memory handed out in bump order and rewound once per forward pass: the device-side twin of the
 * forward scope's heap slab (skainet-lang/skainet-lang-core/src/commonMain/kotlin/sk/ainet/lang/memory/Scope.kt:100-230).
 * `Scope` is sealed in the language module, so this is not one; [HipOps] takes it beside the scope and the caller
 * resets both at the same point of its step. A pass that always asks for the same sizes in the same order gets the
 * same addresses every time, which is what a recorded graph of that pass needs.
 */
public class HipActivationSlab(public val capacityBytes: Long) : AutoCloseable {
    private val slab: HipDeviceStorage = HipDeviceStorage.allocate(capacityBytes)
    private val handedOut = ArrayList<HipDeviceStorage>()
    private var offset = 0L

    /** Bytes handed out since the last [reset]. */
    public val usedBytes: Long get() = offset

    /** High-water mark across passes, for sizing the slab. */
    public var peakBytes: Long = 0L
        private set

    /** [bytes] from the slab (256-byte aligned), or `null` when the slab is full: the caller then allocates on its own. */
    public fun allocate(bytes: Long): HipDeviceStorage? {
        val at = (offset + ALIGN - 1) / ALIGN * ALIGN
        if (at + bytes > capacityBytes) return null
        offset = at + bytes
        if (offset > peakBytes) peakBytes = offset
        return slab.slice(at, bytes).also { handedOut += it }
    }

    /** End of a pass: every storage handed out is closed (a later use throws), the next pass starts at offset 0. */
    public fun reset() {
        handedOut.forEach { it.close() }
        handedOut.clear()
        offset = 0L
    }

    override fun close() {
        reset()
        slab.close()
    }

    private companion object {
        const val ALIGN = 256L
    }
}
