from triton_helpers_amd.layers.hash_encoding.__main__ import main

if __name__ == "__main__":
    main()
