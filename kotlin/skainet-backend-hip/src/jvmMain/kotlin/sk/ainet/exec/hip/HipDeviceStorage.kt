package sk.ainet.exec.hip

import java.lang.foreign.Arena
import java.lang.foreign.MemorySegment
import java.lang.foreign.ValueLayout
import sk.ainet.lang.memory.Owner
import sk.ainet.lang.memory.ScopeKind
import sk.ainet.lang.memory.Storage
import sk.ainet.lang.memory.StorageId
import sk.ainet.lang.memory.trace.NoopTraceSink
import sk.ainet.lang.memory.trace.TraceEvent
import sk.ainet.lang.memory.trace.TraceSink
import sk.ainet.lang.tensor.TensorId

/**
 * Bytes in the GPU's memory (`skainet_hip_malloc`): the home of resident activations and KV caches, so that the
 * device entries (`skainet_hip_matmul_fused_dev`, `skainet_hip_attn_out_proj_dev`, `skainet_hip_f32_sdpa_cache_dev`, ...)
 * run a decoder step without a round trip through the heap. `copyInto` / `copyFrom` are synchronous copies over PCIe.
 */
public class HipDeviceStorage private constructor(
    override val id: StorageId,
    private val base: MemorySegment,
    override val sizeBytes: Long,
    override val owner: Owner,
    override val debugOrigin: TensorId?,
    override val sink: TraceSink,
    private val mutable: Boolean,
) : Storage.Device() {
    override val isMutable: Boolean get() = (owner as? Owner.Alias)?.parent?.isMutable ?: mutable

    /** The device address, for the `*_dev` entries. */
    public fun pointer(): MemorySegment {
        checkAlive()
        return base
    }

    override fun slice(offsetBytes: Long, lengthBytes: Long): HipDeviceStorage {
        checkAlive()
        require(offsetBytes >= 0 && lengthBytes >= 0 && offsetBytes + lengthBytes <= sizeBytes) {
            "slice [$offsetBytes, ${offsetBytes + lengthBytes}) outside $sizeBytes bytes"
        }
        val at = MemorySegment.ofAddress(base.address() + offsetBytes)
        return HipDeviceStorage(StorageId.next(), at, lengthBytes, Owner.Alias(this), debugOrigin, sink, mutable)
    }

    override fun copyInto(dest: ByteArray, destOffset: Int, offset: Long, length: Int) {
        checkAlive()
        require(offset >= 0 && length >= 0 && offset + length <= sizeBytes) { "copyInto [$offset, ${offset + length}) outside $sizeBytes bytes" }
        if (length == 0) return
        Arena.ofConfined().use { arena ->
            val host = arena.allocate(length.toLong(), 16)
            val rc = HipLibrary.d2h!!.invoke(host, MemorySegment.ofAddress(base.address() + offset), length.toLong()) as Int
            check(rc == 0) { "HipDeviceStorage.copyInto: ${HipLibrary.error()}" }
            MemorySegment.copy(host, ValueLayout.JAVA_BYTE, 0L, dest, destOffset, length)
        }
    }

    override fun copyFrom(src: ByteArray, srcOffset: Int, offset: Long, length: Int) {
        checkAlive()
        require(isMutable) { "storage $id is not mutable" }
        require(offset >= 0 && length >= 0 && offset + length <= sizeBytes) { "copyFrom [$offset, ${offset + length}) outside $sizeBytes bytes" }
        if (length == 0) return
        Arena.ofConfined().use { arena ->
            val host = arena.allocate(length.toLong(), 16)
            MemorySegment.copy(src, srcOffset, host, ValueLayout.JAVA_BYTE, 0L, length)
            val rc = HipLibrary.h2d!!.invoke(MemorySegment.ofAddress(base.address() + offset), host, length.toLong()) as Int
            check(rc == 0) { "HipDeviceStorage.copyFrom: ${HipLibrary.error()}" }
        }
    }

    override fun onClose() {
        if (owner is Owner.Owned) HipLibrary.free?.invoke(base)
    }

    override fun toString(): String =
        "HipDevice($id, $sizeBytes B @0x${base.address().toString(16)}, $owner${debugOrigin?.let { ", $it" } ?: ""}${if (isAlive) "" else ", closed"})"

    public companion object {
        /** [bytes] of device memory owned by [scope]; throws IllegalStateException when the device cannot provide them. */
        public fun allocate(bytes: Long, scope: ScopeKind = ScopeKind.AMBIENT, origin: TensorId? = null, sink: TraceSink = NoopTraceSink): HipDeviceStorage {
            require(bytes >= 0) { "negative size $bytes" }
            check(HipLibrary.usable) { "no usable gfx950 device: ${HipLibrary.error()}" }
            val ptr = HipLibrary.malloc!!.invoke(maxOf(bytes, 1L)) as MemorySegment
            check(ptr != MemorySegment.NULL) { "skainet_hip_malloc($bytes): ${HipLibrary.error()}" }
            val s = HipDeviceStorage(StorageId.next(), ptr, bytes, Owner.Owned(scope), origin, sink, true)
            if (sink.isEnabled) sink.emit(TraceEvent.Allocation(s.id.value, scope, bytes, origin))
            return s
        }
    }
}
