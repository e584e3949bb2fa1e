from triton_helpers_amd.layers.fully_fused_mlp.__main__ import main

if __name__ == "__main__":
    main()
