package sk.ainet.exec.hip

import java.lang.foreign.Arena
import java.lang.foreign.MemorySegment
import java.lang.foreign.ValueLayout

/** Heap array <-> native segment copies shared by the host-entry wrappers (one confined arena per call). */
internal object HipStaging {
    fun floats(arena: Arena, src: FloatArray, offset: Int, count: Long, what: String): MemorySegment {
        require(offset >= 0 && offset + count <= src.size) { "$what needs $count floats from $offset, array has ${src.size}" }
        if (count == 0L) return MemorySegment.NULL
        val seg = arena.allocate(count * Float.SIZE_BYTES, 16)
        MemorySegment.copy(src, offset, seg, ValueLayout.JAVA_FLOAT, 0L, count.toInt())
        return seg
    }

    fun bytes(arena: Arena, src: ByteArray, offset: Int, count: Long, what: String): MemorySegment {
        require(offset >= 0 && offset + count <= src.size) { "$what needs $count bytes from $offset, array has ${src.size}" }
        if (count == 0L) return MemorySegment.NULL
        val seg = arena.allocate(count, 16)
        MemorySegment.copy(src, offset, seg, ValueLayout.JAVA_BYTE, 0L, count.toInt())
        return seg
    }

    fun ints(arena: Arena, src: IntArray): MemorySegment {
        if (src.isEmpty()) return MemorySegment.NULL
        val seg = arena.allocate(src.size.toLong() * Int.SIZE_BYTES, 16)
        MemorySegment.copy(src, 0, seg, ValueLayout.JAVA_INT, 0L, src.size)
        return seg
    }

    fun output(arena: Arena, count: Long): MemorySegment = arena.allocate(maxOf(count, 1L) * Float.SIZE_BYTES, 16)

    fun read(seg: MemorySegment, dst: FloatArray, offset: Int, count: Long, what: String) {
        require(offset >= 0 && offset + count <= dst.size) { "$what needs $count floats from $offset, array has ${dst.size}" }
        if (count > 0) MemorySegment.copy(seg, ValueLayout.JAVA_FLOAT, 0L, dst, offset, count.toInt())
    }
}
