package com.lastbot.llama2j;

import java.lang.foreign.Arena;
import java.lang.foreign.FunctionDescriptor;
import java.lang.foreign.Linker;
import java.lang.foreign.MemorySegment;
import java.lang.foreign.SymbolLookup;
import java.lang.invoke.MethodHandle;
import java.nio.ByteBuffer;

import static java.lang.foreign.ValueLayout.ADDRESS;
import static java.lang.foreign.ValueLayout.JAVA_DOUBLE;
import static java.lang.foreign.ValueLayout.JAVA_FLOAT;
import static java.lang.foreign.ValueLayout.JAVA_INT;
import static java.lang.foreign.ValueLayout.JAVA_LONG;

/**
 * Execution context of Mode.HIP: binds libllama2j_hip.so (include/llama2j_hip.h) through the Foreign
 * Function and Memory API (Java 22+).  It plays the part ContextCUDA plays for Mode.CUDA, but the whole
 * forward pass is one downcall: the library owns every device buffer and replays the token as a graph.
 *
 * Threads: uploadQuant / uploadF32 may be called from many threads at once, virtual threads included
 * (TransformerWeights uploads from ten of them); every other method belongs to the one thread that runs
 * the token loop.  A failed call is reported with the context's own error text (l2j_ctx_last_error), which is
 * right whatever carrier thread the second downcall runs on.
 *
 * SOURCE ONLY: the build image of this repository has no JDK, so this file has never been compiled.
 */
public final class ContextHIP implements AutoCloseable {
    public static final int TOK_EMB = 0, RMS_ATT = 1, WQ = 2, WK = 3, WV = 4, WO = 5, RMS_FFN = 6,
            W1 = 7, W2 = 8, W3 = 9, RMS_FINAL = 10, WCLS = 11;

    private static final Linker LINKER = Linker.nativeLinker();
    private static final int ERROR_TEXT_BYTES = 1024;

    private final SymbolLookup lib;
    private final Arena arena = Arena.ofShared();
    private final MemorySegment ctx;
    private final int vocabSize, seqLen;
    // buffers of the token loop's thread, allocated once (no allocation per token)
    private final MemorySegment logitsSeg, intSeg, tokensSeg, promptSeg, countSeg, secondsSeg;
    private final MethodHandle lastError, ctxLastError, destroy, setOption, uploadQuant, uploadF32, finalizeH, reset, forward,
            forwardArgmax, decodeGreedy, decodeGreedyBatch, decodeSampleBatch, releaseBatch, decodeSample, samplerSeed, sample, prefill;

    private MethodHandle handle(String name, FunctionDescriptor fd) {
        return LINKER.downcallHandle(lib.find(name).orElseThrow(), fd);
    }

    private ContextHIP(String libraryPath, Config p, boolean sharedWeights, int device, String checkpointPath, boolean writeCaches) {
        lib = SymbolLookup.libraryLookup(libraryPath, arena);
        lastError = handle("l2j_last_error", FunctionDescriptor.of(ADDRESS));
        ctxLastError = handle("l2j_ctx_last_error", FunctionDescriptor.of(JAVA_INT, ADDRESS, ADDRESS, JAVA_INT));
        destroy = handle("l2j_destroy", FunctionDescriptor.ofVoid(ADDRESS));
        setOption = handle("l2j_set_option", FunctionDescriptor.of(JAVA_INT, ADDRESS, ADDRESS, JAVA_INT));
        uploadQuant = handle("l2j_upload_quant", FunctionDescriptor.of(JAVA_INT, ADDRESS, JAVA_INT, ADDRESS, JAVA_LONG));
        uploadF32 = handle("l2j_upload_f32", FunctionDescriptor.of(JAVA_INT, ADDRESS, JAVA_INT, ADDRESS, JAVA_LONG));
        finalizeH = handle("l2j_finalize", FunctionDescriptor.of(JAVA_INT, ADDRESS));
        reset = handle("l2j_reset", FunctionDescriptor.of(JAVA_INT, ADDRESS));
        forward = handle("l2j_forward", FunctionDescriptor.of(JAVA_INT, ADDRESS, JAVA_INT, JAVA_INT, ADDRESS));
        forwardArgmax = handle("l2j_forward_argmax", FunctionDescriptor.of(JAVA_INT, ADDRESS, JAVA_INT, JAVA_INT, ADDRESS));
        decodeGreedy = handle("l2j_decode_greedy",
                FunctionDescriptor.of(JAVA_INT, ADDRESS, ADDRESS, JAVA_INT, JAVA_INT, ADDRESS, ADDRESS, ADDRESS));
        decodeGreedyBatch = handle("l2j_decode_greedy_batch",
                FunctionDescriptor.of(JAVA_INT, ADDRESS, ADDRESS, ADDRESS, JAVA_INT, JAVA_INT, JAVA_INT, ADDRESS, ADDRESS));
        decodeSampleBatch = handle("l2j_decode_sample_batch", FunctionDescriptor.of(JAVA_INT, ADDRESS, ADDRESS, ADDRESS, JAVA_INT, JAVA_INT,
                JAVA_INT, JAVA_FLOAT, JAVA_FLOAT, ADDRESS, ADDRESS, ADDRESS, ADDRESS));
        releaseBatch = handle("l2j_release_batch", FunctionDescriptor.of(JAVA_INT, ADDRESS));
        decodeSample = handle("l2j_decode_sample", FunctionDescriptor.of(JAVA_INT, ADDRESS, ADDRESS, JAVA_INT, JAVA_INT,
                JAVA_FLOAT, JAVA_FLOAT, JAVA_LONG, ADDRESS, ADDRESS, ADDRESS));
        samplerSeed = handle("l2j_sampler_seed", FunctionDescriptor.of(JAVA_INT, ADDRESS, JAVA_LONG));
        sample = handle("l2j_sample", FunctionDescriptor.of(JAVA_INT, ADDRESS, ADDRESS, JAVA_FLOAT, JAVA_FLOAT, JAVA_FLOAT, ADDRESS));
        prefill = handle("l2j_prefill", FunctionDescriptor.of(JAVA_INT, ADDRESS, ADDRESS, JAVA_INT, JAVA_INT, ADDRESS, ADDRESS));

        MemorySegment out = arena.allocate(ADDRESS);
        MemorySegment cfg = arena.allocate(48, 4);   // l2j_config: twelve 32-bit fields
        int rc;
        try {
            if (checkpointPath == null) {
                MethodHandle create = handle("l2j_create", FunctionDescriptor.of(JAVA_INT, ADDRESS, ADDRESS));
                int[] f = {p.dim, p.hidden_dim, p.n_layers, p.n_heads, p.n_kv_heads, p.vocab_size, p.seq_len,
                        sharedWeights ? 1 : 0, Run.QUANT_GROUP_SIZE, Run.QUANT_BITS, device, 0};
                for (int i = 0; i < f.length; i++) cfg.setAtIndex(JAVA_INT, i, f[i]);
                rc = (int) create.invoke(cfg, out);
            } else {
                // the library reads the .bin, takes or writes the .quant caches and finalizes (l2j_load_checkpoint)
                MethodHandle load = handle("l2j_load_checkpoint",
                        FunctionDescriptor.of(JAVA_INT, ADDRESS, JAVA_INT, JAVA_INT, JAVA_INT, ADDRESS));
                rc = (int) load.invoke(arena.allocateFrom(checkpointPath), device, 0, writeCaches ? 1 : 0, out);
            }
        } catch (Throwable t) {
            throw new RuntimeException(t);
        }
        if (rc < 0) {   // no context yet: the text is the calling thread's (the same platform thread made both calls)
            String msg = threadErrorText();
            arena.close();
            throw new RuntimeException("llama2j_hip error " + rc + ": " + msg);
        }
        ctx = out.get(ADDRESS, 0);
        if (checkpointPath != null) {
            MethodHandle getConfig = handle("l2j_get_config", FunctionDescriptor.of(JAVA_INT, ADDRESS, ADDRESS));
            try {
                check((int) getConfig.invoke(ctx, cfg));
            } catch (RuntimeException e) {
                throw e;
            } catch (Throwable t) {
                throw new RuntimeException(t);
            }
        }
        vocabSize = cfg.getAtIndex(JAVA_INT, 5);
        seqLen = cfg.getAtIndex(JAVA_INT, 6);
        logitsSeg = arena.allocate((long) vocabSize * Float.BYTES, 16);
        intSeg = arena.allocate(JAVA_INT);
        tokensSeg = arena.allocate((long) seqLen * Integer.BYTES, 16);
        promptSeg = arena.allocate((long) seqLen * Integer.BYTES, 16);
        countSeg = arena.allocate(JAVA_INT);
        secondsSeg = arena.allocate(JAVA_DOUBLE);
    }

    /** An empty context of the given shape: upload the tensors, then finalizeWeights(). */
    public ContextHIP(String libraryPath, Config p, boolean sharedWeights, int device) {
        this(libraryPath, p, sharedWeights, device, null, false);
    }

    /** = new TransformerWeights(...) + new RunState(...) done by the library from the checkpoint file. */
    public static ContextHIP fromCheckpoint(String libraryPath, String checkpointPath, int device, boolean writeCaches) {
        return new ContextHIP(libraryPath, null, false, device, checkpointPath, writeCaches);
    }

    private String threadErrorText() {
        try {
            return ((MemorySegment) lastError.invoke()).reinterpret(4096).getString(0);
        } catch (Throwable t) {
            return "(no error text: " + t + ")";
        }
    }

    /** Same convention as ContextCUDA.isError: a failed device call becomes a RuntimeException. */
    private void check(int rc) {
        if (rc >= 0) return;
        String msg;
        try (Arena a = Arena.ofConfined()) {
            MemorySegment buf = a.allocate(ERROR_TEXT_BYTES);
            int n = (int) ctxLastError.invoke(ctx, buf, ERROR_TEXT_BYTES);
            msg = n >= 0 ? buf.getString(0) : threadErrorText();
        } catch (Throwable t) {
            throw new RuntimeException(t);
        }
        throw new RuntimeException("llama2j_hip error " + rc + ": " + msg);
    }

    private int call(MethodHandle h, Object... args) {
        try {
            return (int) h.invokeWithArguments(args);
        } catch (Throwable t) {
            throw new RuntimeException(t);
        }
    }

    /** A launch shape or algorithm switch of this context (l2j_set_option), e.g. ("graph", 0) under a profiler. */
    public void setOption(String name, int value) {
        try (Arena a = Arena.ofConfined()) {
            check(call(setOption, ctx, a.allocateFrom(name), value));
        }
    }

    /** Replaces ContextCUDA.allocateQuantAndCopyToDevice: the exact .quant payload of one tensor.  Thread safe. */
    public void uploadQuant(int tensor, ByteBuffer encoded) {
        int n = encoded.remaining();
        if (encoded.isDirect()) {                              // cache reads are direct buffers: no copy
            check(call(uploadQuant, ctx, tensor, MemorySegment.ofBuffer(encoded), (long) n));
            return;
        }
        try (Arena a = Arena.ofConfined()) {                   // Quant.encode returns a heap buffer: copy once
            MemorySegment seg = a.allocate(n, 16);
            seg.copyFrom(MemorySegment.ofBuffer(encoded));
            check(call(uploadQuant, ctx, tensor, seg, (long) n));
        }
    }

    /** Replaces ContextCUDA.allocateAndCopyToDevice for token_embedding_table and wcls.  Thread safe. */
    public void uploadF32(int tensor, float[] values) {
        try (Arena a = Arena.ofConfined()) {
            MemorySegment seg = a.allocate((long) values.length * Float.BYTES, 16);
            seg.copyFrom(MemorySegment.ofArray(values));
            check(call(uploadF32, ctx, tensor, seg, (long) values.length));
        }
    }

    public void finalizeWeights() {
        check(call(finalizeH, ctx));
    }

    /** A fresh RunState: the KV cache zeroed. */
    public void reset() {
        check(call(reset, ctx));
    }

    /** Replaces Run.transformerCUDA plus the logits copy in the token loop; logits == null: no copy. */
    public void forward(int token, int pos, float[] logits) {
        check(call(forward, ctx, token, pos, logits == null ? MemorySegment.NULL : logitsSeg));
        if (logits != null) MemorySegment.ofArray(logits).copyFrom(logitsSeg.asSlice(0, (long) logits.length * Float.BYTES));
    }

    /** Greedy step with the argmax done on the device: only four bytes come back. */
    public int forwardArgmax(int token, int pos) {
        check(call(forwardArgmax, ctx, token, pos, intSeg));
        return intSeg.get(JAVA_INT, 0);
    }

    /** Result of a whole token loop run by the library. */
    public record Generation(int[] tokens, double secondsAfterFirst) {
    }

    private MemorySegment stagePrompt(int[] prompt) {
        if (prompt.length > seqLen) throw new IllegalArgumentException("prompt longer than seq_len");
        MemorySegment.copy(prompt, 0, promptSeg, JAVA_INT, 0, prompt.length);
        return promptSeg;
    }

    private Generation generation() {
        int n = countSeg.get(JAVA_INT, 0);
        int[] tokens = new int[n];
        MemorySegment.copy(tokensSeg, JAVA_INT, 0, tokens, 0, n);
        return new Generation(tokens, secondsSeg.get(JAVA_DOUBLE, 0));
    }

    /**
     * The token loop of Run.main at temperature 0 in one downcall: BOS first, the prompt ids forced, first-maximum
     * argmax afterwards, stop after token 1.  tokens[i] is `next` of iteration i; the seconds run from the end of the
     * first iteration, as Run's own tok/s does.  steps &lt;= 0: seq_len.
     */
    public Generation decodeGreedy(int[] prompt, int steps) {
        check(call(decodeGreedy, ctx, stagePrompt(prompt), prompt.length, steps, tokensSeg, countSeg, secondsSeg));
        return generation();
    }

    /**
     * Sixteen or thirty-two greedy token loops at once (l2j_decode_greedy_batch): every weight is read once per step for
     * all of them.  prompts: at most 32 id arrays (16 sequences run for up to sixteen prompts, else 32; missing ones run
     * without a prompt); result[b] holds `steps` tokens of sequence b, which runs on after token 1: cut it there.  No
     * counterpart in the reference.
     */
    public int[][] decodeGreedyBatch(int[][] prompts, int steps) {
        return decodeSampleBatch(prompts, steps, 0.0f, 0.0f, null);
    }

    /**
     * decodeGreedyBatch with a Sampler(rngSeeds[b], vocab_size) per sequence on the device (l2j_decode_sample_batch):
     * the unforced tokens of sequence b are sampled as decodeSample samples them.  Temperature 0 (rngSeeds may then be
     * null): the greedy loops.
     */
    public int[][] decodeSampleBatch(int[][] prompts, int steps, float temperature, float topp, long[] rngSeeds) {
        if (prompts.length > 32) throw new IllegalArgumentException("at most 32 sequences");
        final int batch = prompts.length <= 16 ? 16 : 32;
        int stride = 1;
        for (int[] p : prompts) stride = Math.max(stride, p.length);
        try (Arena a = Arena.ofConfined()) {
            MemorySegment ids = a.allocate((long) batch * stride * Integer.BYTES, 16);
            MemorySegment counts = a.allocate((long) batch * Integer.BYTES, 16);
            MemorySegment out = a.allocate((long) batch * steps * Integer.BYTES, 16);
            for (int b = 0; b < prompts.length; b++) {
                MemorySegment.copy(prompts[b], 0, ids, JAVA_INT, (long) b * stride * Integer.BYTES, prompts[b].length);
                counts.setAtIndex(JAVA_INT, b, prompts[b].length);
            }
            if (temperature == 0.0f) {
                check(call(decodeGreedyBatch, ctx, ids, counts, batch, stride, steps, out, secondsSeg));
            } else {
                MemorySegment seeds = a.allocate((long) batch * Long.BYTES, 16);
                for (int b = 0; b < batch; b++) seeds.setAtIndex(JAVA_LONG, b, b < rngSeeds.length ? rngSeeds[b] : 0L);
                check(call(decodeSampleBatch, ctx, ids, counts, batch, stride, steps, temperature, topp, seeds, out, secondsSeg,
                        MemorySegment.NULL));
            }
            int[][] tokens = new int[batch][steps];
            for (int b = 0; b < batch; b++) MemorySegment.copy(out, JAVA_INT, (long) b * steps * Integer.BYTES, tokens[b], 0, steps);
            return tokens;
        }
    }

    /** Frees what decodeGreedyBatch / decodeSampleBatch / prefill keep on the device (l2j_release_batch); they make it again. */
    public void releaseBatch() {
        check(call(releaseBatch, ctx));
    }

    /**
     * Run.transformer(tokens[i], pos0 + i, ...) for every i (the prompt positions of Run.main's loop), 32 positions per
     * step on the matrix cores (l2j_prefill); logits (may be null) receives those of the last position.  The token loop
     * then goes on at position pos0 + tokens.length with forwardArgmax / forward.
     */
    public void prefill(int[] tokens, int pos0, float[] logits) {
        try (Arena a = Arena.ofConfined()) {
            MemorySegment ids = a.allocate((long) tokens.length * Integer.BYTES, 16);
            MemorySegment.copy(tokens, 0, ids, JAVA_INT, 0, tokens.length);
            check(call(prefill, ctx, ids, tokens.length, pos0, logits == null ? MemorySegment.NULL : logitsSeg, secondsSeg));
        }
        if (logits != null) MemorySegment.ofArray(logits).copyFrom(logitsSeg.asSlice(0, (long) logits.length * Float.BYTES));
    }

    /** The token loop of Run.main with Sampler(rngSeed) on the device (temperature, top-p as in CommandLine). */
    public Generation decodeSample(int[] prompt, int steps, float temperature, float topp, long rngSeed) {
        check(call(decodeSample, ctx, stagePrompt(prompt), prompt.length, steps, temperature, topp, rngSeed, tokensSeg, countSeg,
                secondsSeg));
        return generation();
    }

    /** = new Sampler(rngSeed, vocab_size), kept on the device. */
    public void samplerSeed(long rngSeed) {
        check(call(samplerSeed, ctx, rngSeed));
    }

    /**
     * The sampling branch of Run.main (temperature, softmax, sample / sample_topp) on the logits of the last forward,
     * without reading them back.  coin: Random.nextFloat() of the caller's own generator, or a negative value to let
     * the device's java.util.Random (seeded by samplerSeed) draw.
     */
    public int sample(float temperature, float topp, float coin) {
        check(call(sample, ctx, MemorySegment.NULL, temperature, topp, coin, intSeg));
        return intSeg.get(JAVA_INT, 0);
    }

    /** Releases graph, buffers and stream (l2j_destroy) before the library is unloaded with the arena. */
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
