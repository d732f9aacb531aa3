"""What the attention kernels launch by: a step planner (`engine.batch`) that an attention mixer brings with it.

The plan travels with the step's integers and reaches the kernels as `ctx.plan[...]`:
`decode_runs`     the runs of one token (each attends with one query), those with the most keys first
`longest_decode`  the most keys one of them reads
`tile_run`, `tile_start`  for every tile of QUERY_TILE queries of the longer runs its run and its first query,
                  those that see the most keys first (a kernel that takes them in this order starts its longest
                  blocks first)
and on the host, `ctx.plan_host[...]`: `longest_decode`, and `decode_shape` = (blocks of 256 keys that the longest
decoding request fills, up to 8; whether the requests are about as long as it: their mean at least 0.8 of it,
which is when cutting every request into that many blocks pays).
"""
import numpy as np

QUERY_TILE = 128    # queries of one run that one block of the prompt attention kernel takes


def attention_plan(run_lens: np.ndarray, cached: np.ndarray, page_size: int):
    single = run_lens == 1
    decode_runs = np.nonzero(single)[0]
    decode_runs = decode_runs[np.argsort(-cached[decode_runs], kind="stable")].astype(np.int32)
    longest = int((cached[single] + 1).max()) if single.any() else 0
    tiles = []
    for i in np.nonzero(run_lens > 1)[0]:
        for q0 in range(0, int(run_lens[i]), QUERY_TILE):
            tiles.append((-(int(cached[i]) + min(q0 + QUERY_TILE, int(run_lens[i]))), int(i), q0))
    tiles.sort()
    arrays = {"decode_runs": decode_runs, "tile_run": np.array([t[1] for t in tiles], dtype=np.int32),
              "tile_start": np.array([t[2] for t in tiles], dtype=np.int32),
              "longest_decode": np.array([longest], dtype=np.int32)}
    mean = float((cached[single] + 1).mean()) if single.any() else 0.0
    alike = bool(mean >= 0.8 * longest)
    return arrays, {"longest_decode": longest, "decode_shape": (min(8, -(-longest // 256)), alike)}
