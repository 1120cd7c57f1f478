"""Shapes that steer the GEMM dispatcher into every kernel variant, shared by the CPU coverage test and the GPU
parity tests, plus the full-size shapes of the benchmark configurations.

A *variant* is one compiled code path: the kernel, its token-tile height, whether it writes split-K partial sums,
for the decode kernel how many 128-channel groups a workgroup walks, for the wave-split decode kernel how many waves
share a workgroup's K, whether a wave's share takes one turn of its four-slot register ring ("one_round") or several and
whether the workgroup owns one 16-channel tile or two, for the large-M kernels whether K ends on a
128-byte block.  `variant_of` maps a plan (sglang_amd._lib.gemm_plan) to such a key.
"""

# ---- FP8 (M, N, K); K % 16 != 0 means unaligned rows (byte-granular loader)
FP8_ROUTE_SHAPES = [
    # decode kernel (M <= 16, K % 128 == 0, N % 128 == 0): whole-K and split, 1 / 2 / 3+ channel groups per workgroup,
    # an uneven last workgroup (16640 = 130 groups), short last K ranges (4480 = 35 blocks, 2176 = 17 blocks)
    (1, 128, 128), (3, 256, 512), (16, 2048, 7168), (13, 18432, 7168), (13, 66560, 1152), (16, 16640, 4480), (15, 33280, 2176),
    (5, 66048, 512), (2, 133120, 384),
    # wave-split decode kernel (few tokens or a small weight, K of at least 8 blocks; N % 16 == 0 is enough): 8 waves with one
    # round (K = 4096) and two (K = 7168, 4480 = 35 blocks: a ragged second round), 4 waves with many rounds (K = 18432) and
    # with one (N % 128 != 0 at short K), ragged N (576, 1088), every token count class
    (1, 512, 4096), (4, 1536, 7168), (2, 7168, 2048), (2, 36864, 7168), (1, 512, 18432), (12, 48, 1152), (1, 512, 7168), (1, 16640, 4480),
    # ... and two channel tiles per workgroup (N / 32 >= 200 and three tokens or more, or K beyond 64 blocks): both wave counts,
    # one round and several, an uneven split of the K blocks over the waves (2176 = 17 blocks), N % 32 == 0 but N % 128 != 0
    (16, 7168, 2048), (9, 33280, 2176), (7, 16640, 4096), (7, 33280, 4096), (3, 36864, 7168), (6, 16640, 4480), (1, 7168, 18432), (16, 7168, 18432),
    (5, 6432, 1280),
    (5, 48, 128), (16, 16, 256),  # a single K block (three of the four waves have nothing to add), a single workgroup
    # three-stage mid-M kernel: 64 / 128 token tiles x 256 / 192 / 128 channel tiles, whole-K and split, ragged M, K blocks per
    # range = 1, 2, 0 mod 3
    (48, 16384, 2048), (33, 16384, 2176), (40, 65536, 512), (200, 16384, 2048), (100, 32768, 640), (130, 8192, 7168),
    (250, 8192, 7296), (100, 16384, 3584), (500, 4096, 14336),
    # the same kernel with 256-channel tiles and a K split (long K, many channels), and with 128-channel tiles
    (65, 7168, 18432), (24, 36864, 14336), (100, 36864, 640), (40, 4096, 7168), (300, 4096, 7168), (1000, 4096, 2048),
    (400, 4096, 16384), (100, 65536, 512), (130, 4096, 7168),
    # decode sizes on the mid-M kernel (4 .. 16 tokens, one round of unsplit tiles): instead of the wave-split kernel with
    # 192-channel tiles, instead of the split streaming kernel with 128- and 256-channel tiles
    (4, 36864, 7168), (13, 36864, 7168), (16, 24576, 1536), (14, 32768, 2048), (16, 49152, 2048),
    # K blocks left over after whole trips over the stages that no shape above has: 64 x 192 (four stages) 3; 128 x 128 (four) 2 and
    # 3; 128 x 192 and 128 x 256 (three; loader waves) 0
    (20, 36864, 896), (100, 32768, 768), (100, 32768, 896), (100, 36864, 768), (300, 16384, 768),
    # small tiles with more workgroups than CUs: 64 x 192 and 128 x 128
    (135, 49152, 1024), (198, 36864, 1024),
    # 192-channel tiles (a wave's three channel tiles are 64 channels apart): whole-K and split, a ragged last tile
    (100, 36864, 512), (20, 36864, 1024), (130, 3072, 7168), (300, 3072, 14336), (130, 1000, 896),
    # 256 x 256 two-phase and 256 x 128 pipelined kernels, K a multiple of 128 and not
    # (the pipelined kernel takes whole-K shapes only where N % 4 != 0 rules the mid-M kernel's split reduce out)
    (4096, 4352, 512), (4000, 4300, 400), (4096, 2178, 256), (4000, 2100, 272), (4096, 2176, 256),
    # generic kernel: every token-tile height, aligned and byte-granular loads, whole-K and split
    (7, 1088, 512), (16, 576, 7168), (7, 1096, 512), (16, 584, 7168), (1, 1088, 3884), (17, 384, 2304), (20, 256, 264), (33, 512, 512), (64, 128, 3884),
    (50, 300, 520), (127, 128, 4096), (130, 640, 896), (1500, 640, 1000), (130, 200, 300), (2048, 4224, 264),
    # between 17 and 1024 tokens only K % 128 != 0 (or unaligned rows) leaves the mid-M kernel to the generic one
    (20, 256, 2064), (33, 256, 272), (100, 256, 400), (100, 640, 2064),
    # 128-channel tiles with a ragged last channel tile; a handful of channels; a single K block
    (50, 3000, 4224), (40, 8, 1024), (100, 16, 4096), (1000, 8, 128),
]

FP8_REQUIRED_VARIANTS = {
    ("decode", "whole", "gpw1"), ("decode", "whole", "gpw2"), ("decode", "whole", "gpw3+"),
    ("decode", "split", "gpw1"), ("decode", "split", "gpw2"), ("decode", "split", "gpw3+"),
    ("decode_wavesplit", "w4", "one_round"), ("decode_wavesplit", "w4", "rounds"), ("decode_wavesplit", "w8", "one_round"),
    ("decode_wavesplit", "w8", "rounds"),
    ("decode_wavesplit", "w4", "one_round", "two_tiles"), ("decode_wavesplit", "w4", "rounds", "two_tiles"),
    ("decode_wavesplit", "w8", "one_round", "two_tiles"), ("decode_wavesplit", "w8", "rounds", "two_tiles"),
    ("dma3", 64, "whole"), ("dma3", 64, "split"), ("dma3", 128, "whole"), ("dma3", 128, "split"),
    # "deep" = more than three LDS stages: always for 64 x 192 and 128 x 128 tiles; for 64 x 128 tiles where the launch has at
    # most one workgroup per CU, which is the only place the plan puts them
    ("dma3", 64, "whole", "bn128", "deep"), ("dma3", 64, "split", "bn128", "deep"),
    ("dma3", 128, "whole", "bn128", "deep"), ("dma3", 128, "split", "bn128", "deep"),
    ("dma3", 64, "whole", "bn192", "deep"), ("dma3", 64, "split", "bn192", "deep"),
    ("dma3", 128, "whole", "bn192"), ("dma3", 128, "split", "bn192"),
    ("pingpong", "kfull"), ("pingpong", "ktail"), ("pipelined", "kfull"), ("pipelined", "ktail"),
    ("generic", 16, "aligned", "whole"), ("generic", 16, "aligned", "split"), ("generic", 16, "bytes", "split"),
    ("generic", 32, "aligned", "split"), ("generic", 32, "bytes", "whole"),
    ("generic", 64, "aligned", "whole"), ("generic", 64, "bytes", "whole"), ("generic", 64, "bytes", "split"),
    ("generic", 128, "aligned", "whole"), ("generic", 128, "aligned", "split"), ("generic", 128, "bytes", "whole"),
    ("generic", 128, "bytes", "split"), ("generic", 256, "bytes", "whole"),
}

# ---- INT8 (M, N, K): the operator requires K % 16 == 0 and N % 8 == 0
INT8_ROUTE_SHAPES = [
    (16, 128, 512), (1, 6144, 4096), (1, 16640, 4480), (9, 33280, 2176), (16, 7168, 18432), (7, 33280, 4096),
    (5, 66048, 512), (2, 133120, 384),
    # a dozen tokens or more on the mid-M kernel where one round of unsplit 64-token tiles fills the chip (128- and 256-channel tiles)
    (16, 28672, 512), (13, 36864, 1024), (12, 24576, 2304), (8, 24576, 5760),  # (eight tokens where K has more than 44 blocks)
    (400, 6144, 896),  # 128 x 128 tiles (four stages) with three K blocks left after whole trips
    (20, 8192, 4096), (40, 65536, 512), (200, 16384, 2048), (200, 32768, 1024), (300, 4096, 14336), (130, 8192, 7168),
    (100, 16384, 3584), (500, 4096, 14336),
    # the mid-M kernel's 128-channel tiles (and 128 x 256 with a K split): ragged M, a ragged last channel tile
    (700, 6144, 14336), (100, 6144, 7168), (100, 28672, 512), (40, 6144, 14336), (20, 2048, 4096), (20, 4096, 1024),
    (33, 12288, 14336),  # 64 x 256 tiles with a K split
    # the 128 x 256 tile is the two-phase 128-token kernel: whole K and split, ragged M (200, 300, 700), K steps 0, 1, 2 mod 3
    (130, 8192, 1024), (250, 16384, 1152), (256, 28672, 4096),
    (50, 3000, 4224), (40, 8, 1024), (100, 16, 4096), (1000, 8, 128),
    (4096, 4096, 512), (4000, 4088, 1024),
    (1, 16, 512), (1, 24, 512), (3, 48, 1152), (5, 48, 128), (16, 16, 256), (17, 136, 1024), (64, 1024, 512), (100, 4096, 1024), (128, 16384, 512), (2048, 4224, 272),
    # between 17 and 1024 tokens only K % 128 != 0 leaves the mid-M kernel to the generic one
    (20, 256, 2064), (33, 256, 272), (100, 256, 400), (100, 640, 2064),
]

# (INT8 decode with a K split does not exist: from 8 K blocks on every INT8 decode shape takes the wave-split kernel)
INT8_REQUIRED_VARIANTS = {
    ("decode", "whole", "gpw1"), ("decode", "whole", "gpw2"), ("decode", "whole", "gpw3+"),
    ("decode_wavesplit", "w4", "one_round"), ("decode_wavesplit", "w4", "rounds"), ("decode_wavesplit", "w8", "one_round"),
    ("decode_wavesplit", "w8", "rounds"),
    ("dma3", 64, "whole"), ("dma3", 64, "split"), ("pingpong128", "whole"), ("pingpong128", "split"),
    # (the 128-channel tiles always run more than three stages: 128 x 128 four, 64 x 128 six - the plan puts 64 x 128 tiles only
    # where the launch has at most one workgroup per CU)
    ("dma3", 64, "whole", "bn128", "deep"), ("dma3", 64, "split", "bn128", "deep"), ("dma3", 128, "whole", "bn128", "deep"), ("dma3", 128, "split", "bn128", "deep"),
    ("pingpong", "kfull"),
    ("generic", 16, "aligned", "whole"), ("generic", 32, "aligned", "split"), ("generic", 64, "aligned", "whole"),
    ("generic", 128, "aligned", "whole"), ("generic", 128, "aligned", "split"), ("generic", 256, "aligned", "whole"),
}

# ---- the benchmark configurations at full size: name -> (K, N)
DSV3_MLP = {"gate_up": (7168, 36864), "down": (18432, 7168)}
DSV3_MLA = {"q_a": (7168, 1536), "kv_a": (7168, 576), "q_b": (1536, 24576), "kv_b": (512, 32768)}
LLAMA3_8B = {"qkv": (4096, 6144), "gate_up": (4096, 28672), "down": (14336, 4096)}

FP8_DECODE_CONFIG = [(M, N, K) for M in (1, 8, 32, 128) for (K, N) in DSV3_MLP.values()]
FP8_PREFILL_CONFIG = [(4096, N, K) for (K, N) in list(DSV3_MLP.values()) + list(DSV3_MLA.values())]
INT8_CONFIG = [(M, N, K) for M in (1, 256, 4096) for (K, N) in LLAMA3_8B.values()]


def variant_of(plan: dict, K: int):
    k = plan["kernel"]
    sp = "split" if plan["splits"] > 1 else "whole"
    if k == "decode":
        g = plan["groups_per_wg"]
        return (k, sp, f"gpw{g}" if g < 3 else "gpw3+")
    if k == "decode_wavesplit":  # waves per workgroup; one turn of the wave's four-slot ring or several
        waves = plan["groups_per_wg"]
        key = (k, f"w{waves}", "rounds" if -(-K // 128) > 4 * waves else "one_round")
        return key + ("two_tiles",) if plan["bn"] == 32 else key  # 32 channels per workgroup (FP8) or 16
    if k == "pingpong128":
        return (k, sp)
    if k == "dma3":  # "deep": more than three LDS stages (small tiles when every workgroup has a CU to itself, FP8)
        key = (k, plan["bm"], sp) if plan["bn"] == 256 else (k, plan["bm"], sp, f"bn{plan['bn']}")
        return key + ("deep",) if plan["stages"] > 3 else key
    if k in ("pingpong", "pipelined"):
        return (k, "kfull" if K % 128 == 0 else "ktail")
    return (k, plan["bm"], "aligned" if plan["aligned"] else "bytes", sp)


def plan_for(kind: str, M: int, N: int, K: int) -> dict:
    from sglang_amd import _lib

    return _lib.gemm_plan(kind, M, N, K, aligned=(K % 16 == 0))
