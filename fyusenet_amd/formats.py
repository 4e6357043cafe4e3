"""Host-side helpers for the buffer formats at the upload/download boundary."""


def deep_tiling(channels):
    """Tile grid of a GPU_DEEP buffer (CPUBufferShape::computeDeepTiling,
    fyusenet/cpu/cpubuffershape.cpp:430-448): minimise |tx-ty| + unused tiles, first minimum in
    y-outer / x-inner ascending order with x >= y."""
    tiles = (channels + 3) // 4
    best, bx, by = None, tiles, 1
    for y in range(1, tiles + 1):
        for x in range(y, tiles + 1):
            if x * y >= tiles:
                cost = (x - y) + (x * y - tiles)
                if best is None or cost < best:
                    best, bx, by = cost, x, y
    return bx, by
