from pylon_amd.main import main

if __name__ == "__main__":
    main()
