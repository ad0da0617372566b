// Cache classes over libkvhip handles.  Each mirrors one reference class
// (Libraries/MLXLMCommon/KVCache.swift: KVCacheSimple :391, RotatingKVCache :541,
// QuantizedKVCache :923) member for member; bookkeeping answers come straight from
// the handle, arrays stay on the device.
import CKVHIP
import Foundation

/// Device memory the caller owns: pointer + shape + dtype.  Stands in for MLXArray on
/// a ROCm host (MLX has no HIP backend).
public protocol HIPArray {
    var devicePointer: UnsafeMutableRawPointer { get }
    var shape: [Int] { get }
    var kvhipDType: Int32 { get }
    static func empty(_ shape: [Int], dtype: Int32) -> Self
}

public struct KVHIPError: Error, CustomStringConvertible {
    public let status: Int32
    public let description: String
}

@inline(__always) func check(_ status: Int32) throws {
    if status < 0 {
        throw KVHIPError(status: status, description: String(cString: kvhip_last_error_message()))
    }
}

/// Programmer errors the reference answers with `fatalError` (KVCache.swift:1107, :784, :1141).
@inline(__always) func must(_ status: Int32) {
    if status < 0 { fatalError(String(cString: kvhip_last_error_message())) }
}

public enum HIPMask {
    case none, causal
    case array(any HIPArray, isBool: Bool)
    case window(offset: Int, window: Int)
}

public class HIPKVCache {
    var handle: OpaquePointer?
    var stream: UnsafeMutableRawPointer? = nil  // hipStream_t of the owning generation loop

    init(kind: kvhip_kind, step: Int = 0, maxSize: Int = 0, keep: Int = 0, groupSize: Int = 0, bits: Int = 0) {
        var cfg = kvhip_config(kind: Int32(kind.rawValue), step: Int32(step), max_size: Int32(maxSize),
                               keep: Int32(keep), group_size: Int32(groupSize), bits: Int32(bits))
        must(kvhip_cache_create(&cfg, &handle))
    }
    init(adopting handle: OpaquePointer?) { self.handle = handle }
    deinit { kvhip_cache_free(handle) }

    // KVCache protocol surface (KVCache.swift:46-104)
    public var offset: Int {
        get { Int(kvhip_cache_offset(handle)) }
        set { must(kvhip_cache_set_offset(handle, Int64(newValue))) }
    }
    public var maxSize: Int? { let m = kvhip_cache_max_size(handle); return m < 0 ? nil : Int(m) }
    public var isTrimmable: Bool { kvhip_cache_is_trimmable(handle, 0) != 0 }
    public func isTrimmable(after positions: Int) -> Bool { kvhip_cache_is_trimmable(handle, Int64(positions)) != 0 }
    @discardableResult public func trim(_ n: Int) -> Int { Int(kvhip_cache_trim(handle, Int64(n))) }
    /// `ropeOffset` (KVCache.swift:190): `.scalar(offset)`, read before the write.
    public var ropeOffset: Int { offset }
    /// `prepare(lengths:)` / `finalize()` keep the protocol's empty defaults (KVCache.swift:114-118).
    public func prepare(lengths: [Int]?) {}
    public func finalize() {}
    /// `eval(cache)` (LLMModel.swift:52-58): the rows are device-resident already; wait for the stream.
    public func eval() { must(kvhip_sync(stream)) }

    public var metaState: [String] {
        get {
            (0 ..< kvhip_cache_meta_count(handle)).map { i in
                var buf = [CChar](repeating: 0, count: 64)
                _ = kvhip_cache_meta_get(handle, i, &buf, 64)
                return String(cString: buf)
            }
        }
        set {
            let cstrs = newValue.map { strdup($0) }
            defer { cstrs.forEach { free($0) } }
            var ptrs = cstrs.map { UnsafePointer<CChar>($0) }
            must(kvhip_cache_meta_set(handle, Int32(ptrs.count), &ptrs))
        }
    }

    /// `state` getter: arrays sliced to `offset` in the reference's layouts.
    public func state<A: HIPArray>(_: A.Type) -> [A] {
        (0 ..< kvhip_cache_state_count(handle)).map { i in
            var shape = [Int64](repeating: 0, count: 4)
            var dt: Int32 = 0
            must(kvhip_cache_state_desc(handle, i, &shape, &dt))
            let a = A.empty(shape.map(Int.init), dtype: dt)
            must(kvhip_cache_state_export(handle, i, a.devicePointer, stream))
            return a
        }
    }

    /// `state` setter (restore order: state, then metaState; KVCache.swift:2067-2072).
    public func setState(_ arrays: [any HIPArray]) {
        var ptrs = arrays.map { UnsafeRawPointer($0.devicePointer) as UnsafeRawPointer? }
        let shapes = arrays.flatMap { $0.shape.map(Int64.init) }
        let dts = arrays.map { $0.kvhipDType }
        must(kvhip_cache_state_import(handle, Int32(arrays.count), &ptrs, shapes, dts, stream))
    }

    public func makeMask(n: Int, windowSize: Int?, returnArray: Bool) -> kvhip_mask_plan_t {
        var plan = kvhip_mask_plan_t()
        must(kvhip_cache_mask_plan(handle, Int32(n), Int32(windowSize ?? 0), returnArray ? 1 : 0, &plan))
        return plan  // .none / .causal, or the parameters kvhip_mask_materialize turns into an array
    }

    func cMask(_ mask: HIPMask) -> kvhip_mask {
        var m = kvhip_mask()
        switch mask {
        case .none: m.mode = Int32(KVHIP_MASK_NONE.rawValue)
        case .causal: m.mode = Int32(KVHIP_MASK_CAUSAL.rawValue)
        case .window(let offset, let window):
            m.mode = Int32(KVHIP_MASK_WINDOW.rawValue); m.offset = Int32(offset); m.window = Int32(window)
        case .array(let a, let isBool):
            m.mode = Int32(KVHIP_MASK_ARRAY.rawValue)
            m.dtype = isBool ? Int32(KVHIP_BOOL.rawValue) : a.kvhipDType
            m.data = UnsafeRawPointer(a.devicePointer)
            let s = a.shape  // [B or 1, H or 1, L, T]
            m.key_len = Int32(s[3]); m.stride_l = Int64(s[3])
            m.stride_h = s[1] == 1 ? 0 : Int64(s[2] * s[3])
            m.stride_b = s[0] == 1 ? 0 : Int64(s[1] * s[2] * s[3])
        }
        return m
    }

    /// `attentionWithCacheUpdate` for this cache (AttentionUtils.swift:37-95): one fused call.
    public func attend<A: HIPArray>(queries: A, keys: A, values: A, scale: Float, mask: HIPMask) -> A {
        let q = queries.shape, k = keys.shape, v = values.shape
        let out = A.empty([q[0], q[1], q[2], v[3]], dtype: queries.kvhipDType)
        var m = cMask(mask)
        must(kvhip_cache_update_attend(handle, queries.devicePointer, keys.devicePointer, values.devicePointer,
                                       Int32(q[0]), Int32(q[1]), Int32(k[1]), Int32(q[2]), Int32(k[3]), Int32(v[3]),
                                       keys.kvhipDType, scale, &m, out.devicePointer, stream))
        return out
    }

    /// An attention layer's `applyRotaryPosition(rope, to: keys, offset: cache.ropeOffset)` followed by
    /// the cache write (Llama.swift:58-62), with the rotation inside the append kernel.  `rope` carries
    /// the layer's `dimensions`, `traditional`, `base`, `scale` and optional `freqs`.
    public func updateRotating<A: HIPArray>(rope: kvhip_rope, keys: A, values: A, batchOffsets: UnsafePointer<Int32>? = nil) {
        var r = rope
        let k = keys.shape, v = values.shape
        must(kvhip_cache_update_rope(handle, &r, batchOffsets, keys.devicePointer, values.devicePointer, Int32(k[0]),
                                     Int32(k[1]), Int32(k[2]), Int32(k[3]), Int32(v[3]), keys.kvhipDType, stream))
    }

    /// `applyRotaryPosition(rope, to: queries, offset:)` (RoPEApplication.swift:62-74) on the device.
    public func rotate<A: HIPArray>(rope: kvhip_rope, _ x: A, offset: Int) -> A {
        var r = rope
        let s = x.shape
        let out = A.empty(s, dtype: x.kvhipDType)
        must(kvhip_rope_apply(&r, x.devicePointer, out.devicePointer, Int32(s[0]), Int32(s[1]), Int32(s[2]),
                              Int32(s[3]), x.kvhipDType, Int64(offset), nil, stream))
        return out
    }

    func appendOnly<A: HIPArray>(keys: A, values: A) {
        let k = keys.shape, v = values.shape
        must(kvhip_cache_update(handle, keys.devicePointer, values.devicePointer, Int32(k[0]), Int32(k[1]),
                                Int32(k[2]), Int32(k[3]), Int32(v[3]), keys.kvhipDType, stream))
    }
}

public final class HIPKVCacheSimple: HIPKVCache {
    public init(step: Int = 256) { super.init(kind: KVHIP_KIND_SIMPLE, step: step) }
    override init(adopting handle: OpaquePointer?) { super.init(adopting: handle) }

    /// `update(keys:values:)`: everything cached, in presentation order (an export).
    public func update<A: HIPArray>(keys: A, values: A) -> (A, A) {
        appendOnly(keys: keys, values: values)
        let n = Int(kvhip_cache_presented_length(handle)), k = keys.shape, v = values.shape
        let ok = A.empty([k[0], k[1], n, k[3]], dtype: keys.kvhipDType)
        let ov = A.empty([v[0], v[1], n, v[3]], dtype: values.kvhipDType)
        must(kvhip_cache_fetch(handle, ok.devicePointer, ov.devicePointer, stream))
        return (ok, ov)
    }

    /// `toQuantized(groupSize:bits:)` throws like the reference (KVCache.swift:486-523).
    public func toQuantized(groupSize: Int = 64, bits: Int = 4) throws -> HIPQuantizedKVCache {
        var out: OpaquePointer?
        try check(kvhip_cache_to_quantized(handle, Int32(groupSize), Int32(bits), stream, &out))
        return HIPQuantizedKVCache(adopting: out)
    }

    public func copy() -> HIPKVCacheSimple {
        var out: OpaquePointer?
        must(kvhip_cache_copy(handle, stream, &out))
        return HIPKVCacheSimple(adopting: out)
    }
}

public final class HIPRotatingKVCache: HIPKVCache {
    public init(maxSize: Int, keep: Int = 0, step: Int = 256) {
        super.init(kind: KVHIP_KIND_ROTATING, step: step, maxSize: maxSize, keep: keep)
    }
    override init(adopting handle: OpaquePointer?) { super.init(adopting: handle) }

    public func update<A: HIPArray>(keys: A, values: A) -> (A, A) {
        appendOnly(keys: keys, values: values)
        let n = Int(kvhip_cache_presented_length(handle)), k = keys.shape, v = values.shape
        let ok = A.empty([k[0], k[1], n, k[3]], dtype: keys.kvhipDType)
        let ov = A.empty([v[0], v[1], n, v[3]], dtype: values.kvhipDType)
        must(kvhip_cache_fetch(handle, ok.devicePointer, ov.devicePointer, stream))
        return (ok, ov)
    }

    /// `logicalView(tail:)` (KVCache.swift:631-658); nil before the first write.
    public func logicalView<A: HIPArray>(tail: Int, like: A) -> (A, A)? {
        var rows: Int64 = 0
        guard kvhip_cache_logical_view(handle, Int64(tail), &rows, nil, nil, stream) == KVHIP_OK else { return nil }
        let s = like.shape
        let k = A.empty([s[0], s[1], Int(rows), s[3]], dtype: like.kvhipDType)
        let v = A.empty([s[0], s[1], Int(rows), s[3]], dtype: like.kvhipDType)
        must(kvhip_cache_logical_view(handle, Int64(tail), &rows, k.devicePointer, v.devicePointer, stream))
        return (k, v)
    }

    public func toQuantized(groupSize: Int = 64, bits: Int = 4) throws -> HIPQuantizedKVCache {
        var out: OpaquePointer?
        try check(kvhip_cache_to_quantized(handle, Int32(groupSize), Int32(bits), stream, &out))  // always throws
        return HIPQuantizedKVCache(adopting: out)
    }
}

/// A `HIPRotatingKVCache` presented with uncommitted rows appended: the counterpart of
/// `RotatingStagedKVCache` (RotatingStagedKVCache.swift:12-132) and what
/// `RotatingRoundStrategy.presented` (KVCacheRound.swift:128-161) hands the model.  It shares
/// the live ring's handle: staged rows sit in spare slots of the ring's page store, attention
/// reads window ++ staged in place, and the ring does not move until `commit(retaining:)`.
public final class HIPRotatingStagedKVCache {
    public let live: HIPRotatingKVCache
    private var open = true

    public init(live: HIPRotatingKVCache) {
        self.live = live
        must(kvhip_cache_stage_begin(live.handle))
    }

    public var stagedCount: Int { open ? Int(kvhip_cache_stage_count(live.handle)) : 0 }
    public var offset: Int { live.offset + stagedCount }
    public var maxSize: Int? { live.maxSize }

    /// Stages the rows and returns the trailing window of the ring followed by everything staged.
    public func update<A: HIPArray>(keys: A, values: A) -> (A, A) { live.update(keys: keys, values: values) }

    /// The fused form: stage, then attend over window ++ staged without exporting it.
    public func attend<A: HIPArray>(queries: A, keys: A, values: A, scale: Float, mask: HIPMask) -> A {
        live.attend(queries: queries, keys: keys, values: values, scale: scale, mask: mask)
    }

    /// The live cache's own mask (RotatingStagedKVCache.swift:49-58).
    public func makeMask(n: Int, windowSize: Int?, returnArray: Bool) -> kvhip_mask_plan_t {
        live.makeMask(n: n, windowSize: windowSize, returnArray: returnArray)
    }

    /// `stagedArrays` (RotatingStagedKVCache.swift:27-30), for a restore point's replay.
    public func stagedArrays<A: HIPArray>(like: A) -> (A, A)? {
        let n = stagedCount
        guard n > 0 else { return nil }
        let s = like.shape
        let k = A.empty([s[0], s[1], n, s[3]], dtype: like.kvhipDType)
        let v = A.empty([s[0], s[1], n, s[3]], dtype: like.kvhipDType)
        must(kvhip_cache_stage_fetch(live.handle, k.devicePointer, v.devicePointer, live.stream))
        return (k, v)
    }

    /// `commit(retaining:)` (RotatingStagedKVCache.swift:62-76); retaining 0 is a rollback.
    public func commit(retaining: Int) {
        guard open else { return }
        open = false
        must(kvhip_cache_stage_commit(live.handle, Int64(retaining), live.stream))
    }

    // round-scoped: not trimmable, not copyable, not restorable (RotatingStagedKVCache.swift:93-125)
    public var isTrimmable: Bool { false }
    @discardableResult public func trim(_ n: Int) -> Int { 0 }
}

public final class HIPQuantizedKVCache: HIPKVCache {
    public init(groupSize: Int = 64, bits: Int = 8) {
        super.init(kind: KVHIP_KIND_QUANTIZED, groupSize: groupSize, bits: bits)
    }
    override init(adopting handle: OpaquePointer?) { super.init(adopting: handle) }

    public var groupSize: Int { Int(kvhip_cache_group_size(handle)) }
    public var bits: Int { Int(kvhip_cache_bits(handle)) }

    /// `updateQuantized(keys:values:)`: ((wq, scales, biases), (wq, scales, biases)) sliced to offset.
    public func updateQuantized<A: HIPArray>(keys: A, values: A) -> ((A, A, A), (A, A, A)) {
        appendOnly(keys: keys, values: values)
        let s = state(A.self)
        return ((s[0], s[1], s[2]), (s[3], s[4], s[5]))
    }

    /// `update` is a programmer error on this class (KVCache.swift:1106-1110).
    public func update<A: HIPArray>(keys: A, values: A) -> (A, A) {
        fatalError("`update` was called on `QuantizedKVCache`. Use `updateQuantized` instead.")
    }

    public func toUnquantized() -> HIPKVCacheSimple {
        var out: OpaquePointer?
        must(kvhip_cache_to_unquantized(handle, stream, &out))
        return HIPKVCacheSimple(adopting: out)
    }
}

/// `trimPromptCache` (KVCache.swift:2302-2306)
@discardableResult public func trimPromptCache(_ cache: [HIPKVCache], numTokens: Int) -> Int {
    guard !cache.isEmpty, cache.allSatisfy({ $0.isTrimmable }) else { return 0 }
    cache.dropFirst().forEach { $0.trim(numTokens) }
    return cache.first?.trim(numTokens) ?? 0
}
