package com.lastbot.llama2j;

import java.lang.foreign.Arena;
import java.lang.foreign.FunctionDescriptor;
import java.lang.foreign.Linker;
import java.lang.foreign.MemorySegment;
import java.lang.foreign.SymbolLookup;
import java.lang.invoke.MethodHandle;
import java.nio.ByteBuffer;

import static java.lang.foreign.ValueLayout.ADDRESS;
import static java.lang.foreign.ValueLayout.JAVA_FLOAT;
import static java.lang.foreign.ValueLayout.JAVA_INT;
import static java.lang.foreign.ValueLayout.JAVA_LONG;

/**
 * Execution context of Mode.HIP: binds libllama2j_hip.so (include/llama2j_hip.h) through the Foreign
 * Function and Memory API (Java 22+).  It plays the part ContextCUDA plays for Mode.CUDA, but the whole
 * forward pass is one downcall: the library owns every device buffer and replays the token as a graph.
 *
 * SOURCE ONLY: the build image of this repository has no JDK, so this file has never been compiled.
 */
public final class ContextHIP implements AutoCloseable {
    public static final int TOK_EMB = 0, RMS_ATT = 1, WQ = 2, WK = 3, WV = 4, WO = 5, RMS_FFN = 6,
            W1 = 7, W2 = 8, W3 = 9, RMS_FINAL = 10, WCLS = 11;

    private static final Linker LINKER = Linker.nativeLinker();
    private final SymbolLookup lib;
    private final Arena arena = Arena.ofShared();
    private final MemorySegment ctx;
    private final MethodHandle lastError, destroy, uploadQuant, uploadF32, finalizeH, forward, forwardArgmax, samplerSeed, sample;

    private MethodHandle handle(String name, FunctionDescriptor fd) {
        return LINKER.downcallHandle(lib.find(name).orElseThrow(), fd);
    }

    public ContextHIP(String libraryPath, Config p, boolean sharedWeights, int device) {
        lib = SymbolLookup.libraryLookup(libraryPath, arena);
        lastError = handle("l2j_last_error", FunctionDescriptor.of(ADDRESS));
        destroy = handle("l2j_destroy", FunctionDescriptor.ofVoid(ADDRESS));
        uploadQuant = handle("l2j_upload_quant", FunctionDescriptor.of(JAVA_INT, ADDRESS, JAVA_INT, ADDRESS, JAVA_LONG));
        uploadF32 = handle("l2j_upload_f32", FunctionDescriptor.of(JAVA_INT, ADDRESS, JAVA_INT, ADDRESS, JAVA_LONG));
        finalizeH = handle("l2j_finalize", FunctionDescriptor.of(JAVA_INT, ADDRESS));
        forward = handle("l2j_forward", FunctionDescriptor.of(JAVA_INT, ADDRESS, JAVA_INT, JAVA_INT, ADDRESS));
        forwardArgmax = handle("l2j_forward_argmax", FunctionDescriptor.of(JAVA_INT, ADDRESS, JAVA_INT, JAVA_INT, ADDRESS));
        samplerSeed = handle("l2j_sampler_seed", FunctionDescriptor.of(JAVA_INT, ADDRESS, JAVA_LONG));
        sample = handle("l2j_sample", FunctionDescriptor.of(JAVA_INT, ADDRESS, ADDRESS, JAVA_FLOAT, JAVA_FLOAT, JAVA_FLOAT, ADDRESS));
        MethodHandle create = handle("l2j_create", FunctionDescriptor.of(JAVA_INT, ADDRESS, ADDRESS));

        // l2j_config: twelve 32-bit fields
        MemorySegment cfg = arena.allocate(48, 4);
        int[] f = {p.dim, p.hidden_dim, p.n_layers, p.n_heads, p.n_kv_heads, p.vocab_size, p.seq_len,
                sharedWeights ? 1 : 0, Run.QUANT_GROUP_SIZE, Run.QUANT_BITS, device, 0};
        for (int i = 0; i < f.length; i++) cfg.setAtIndex(JAVA_INT, i, f[i]);
        MemorySegment out = arena.allocate(ADDRESS);
        check(invokeInt(create, cfg, out));
        ctx = out.get(ADDRESS, 0);
    }

    private static int invokeInt(MethodHandle h, Object... args) {
        try {
            return (int) h.invokeWithArguments(args);
        } catch (Throwable t) {
            throw new RuntimeException(t);
        }
    }

    /** Same convention as ContextCUDA.isError: a failed device call becomes a RuntimeException. */
    private void check(int rc) {
        if (rc < 0) {
            try {
                MemorySegment msg = ((MemorySegment) lastError.invoke()).reinterpret(4096);
                throw new RuntimeException("llama2j_hip error " + rc + ": " + msg.getString(0));
            } catch (RuntimeException e) {
                throw e;
            } catch (Throwable t) {
                throw new RuntimeException(t);
            }
        }
    }

    /** Replaces ContextCUDA.allocateQuantAndCopyToDevice: the exact .quant payload of one tensor. */
    public void uploadQuant(int tensor, ByteBuffer encoded) {
        int n = encoded.remaining();
        MemorySegment seg;
        if (encoded.isDirect()) {
            seg = MemorySegment.ofBuffer(encoded);            // cache reads are direct buffers
        } else {
            try (Arena a = Arena.ofConfined()) {              // Quant.encode returns a heap buffer: copy once
                seg = a.allocate(n, 16);
                seg.copyFrom(MemorySegment.ofBuffer(encoded));
                check(invokeInt(uploadQuant, ctx, tensor, seg, (long) n));
                return;
            }
        }
        check(invokeInt(uploadQuant, ctx, tensor, seg, (long) n));
    }

    /** Replaces ContextCUDA.allocateAndCopyToDevice for token_embedding_table and wcls. */
    public void uploadF32(int tensor, float[] values) {
        try (Arena a = Arena.ofConfined()) {
            MemorySegment seg = a.allocate((long) values.length * Float.BYTES, 16);
            seg.copyFrom(MemorySegment.ofArray(values));
            check(invokeInt(uploadF32, ctx, tensor, seg, (long) values.length));
        }
    }

    public void finalizeWeights() {
        check(invokeInt(finalizeH, ctx));
    }

    /** Replaces Run.transformerCUDA plus the logits copy in the token loop. */
    public void forward(int token, int pos, float[] logits) {
        try (Arena a = Arena.ofConfined()) {
            MemorySegment seg = a.allocate((long) logits.length * Float.BYTES, 16);
            check(invokeInt(forward, ctx, token, pos, seg));
            MemorySegment.ofArray(logits).copyFrom(seg);
        }
    }

    /** Greedy step with the argmax done on the device: only four bytes come back. */
    public int forwardArgmax(int token, int pos) {
        try (Arena a = Arena.ofConfined()) {
            MemorySegment next = a.allocate(JAVA_INT);
            check(invokeInt(forwardArgmax, ctx, token, pos, next));
            return next.get(JAVA_INT, 0);
        }
    }

    /** = new Sampler(rngSeed, vocab_size), kept on the device. */
    public void samplerSeed(long rngSeed) {
        check(invokeInt(samplerSeed, ctx, rngSeed));
    }

    /**
     * The sampling branch of Run.main (temperature, softmax, sample / sample_topp) on the logits of the last forward,
     * without reading them back.  coin: Random.nextFloat() of the caller's own generator, or a negative value to let
     * the device's java.util.Random (seeded by samplerSeed) draw.
     */
    public int sample(float temperature, float topp, float coin) {
        try (Arena a = Arena.ofConfined()) {
            MemorySegment next = a.allocate(JAVA_INT);
            check(invokeInt(sample, ctx, MemorySegment.NULL, temperature, topp, coin, next));
            return next.get(JAVA_INT, 0);
        }
    }

    @Override
    public void close() {
        try {
            destroy.invoke(ctx);
        } catch (Throwable t) {
            throw new RuntimeException(t);
        }
        arena.close();
    }
}
